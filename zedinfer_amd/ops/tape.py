"""The step tape: the library calls of one step, recorded while it runs and made again with one call.

    with Recording() as rec:
        ...            # a step: every launch is a call into the kernel library
    tape = rec.tape()  # None when nothing was called
    tape.run()         # the same calls, with the same arguments, from native code

A tape holds the addresses its calls were made with.  The recorder keeps what they point to alive and at
its place (``Recording`` counts the device allocations made while it records, so that a step which
allocates, and whose memory would be someone else's at the next run, is noticed: ``allocations``), and
runs the tape on the device and stream it was recorded on.  Work that does not go through the kernel
library (a torch operator) is not on the tape: a step is recorded only when all its parts say that their
device work is the library's (``Part.tape_safe``)."""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _lib


class Tape:
    def __init__(self, calls):
        lib = _lib.load()
        self._lib = lib
        self._handle = ctypes.c_void_p(lib.zi_tape_new())
        if not self._handle:
            raise _lib.KernelLibraryError("no memory for a tape")
        words, counts = [], []
        for name, args in calls:
            w = _lib.argument_words(name, args)
            words += w
            counts.append(len(w))
        names = b"".join(name.encode() + b"\0" for name, _ in calls)
        _lib.call("zi_tape_record_many", self._handle, names, (ctypes.c_int * len(counts))(*counts),
                  (ctypes.c_int64 * len(words))(*words), len(calls))
        self.length = len(calls)

    def run(self) -> None:
        done = ctypes.c_int(0)
        rc = self._lib.zi_tape_run(self._handle, ctypes.cast(ctypes.byref(done), ctypes.c_void_p))
        if rc != 0:
            raise _lib.KernelLibraryError(f"call {done.value} of a tape of {self.length}: "
                                          + self._lib.zi_last_error().decode("utf-8", "replace"))

    def __del__(self):
        handle, self._handle = getattr(self, "_handle", None), None
        if handle:
            self._lib.zi_tape_free(handle)


class Recording:
    """Collects the library calls made inside the ``with`` block (recordings do not nest)."""

    def __init__(self, device: Optional[torch.device] = None):
        self.device = device
        self.calls: list = []
        self.allocations = 0

    def _allocated(self) -> int:
        if self.device is None or self.device.type != "cuda":
            return 0
        return int(torch.cuda.memory_stats(self.device).get("allocation.all.allocated", 0))

    def __enter__(self) -> "Recording":
        if _lib._recorded is not None:
            raise RuntimeError("a tape is being recorded already")
        self._before = self._allocated()
        _lib._recorded = self.calls
        return self

    def __exit__(self, *exc) -> None:
        _lib._recorded = None
        self.allocations = self._allocated() - self._before

    def tape(self) -> Optional[Tape]:
        return Tape(self.calls) if self.calls else None
