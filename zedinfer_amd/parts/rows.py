"""Numbers of rows that the parts with matrix products want steps to be run with (``Part.step_rows``).

The engine pads steps so that their kinds are few and recur (a recorded graph or tape serves a kind).  Which
numbers of rows are good ones is a matter of the kernels: the few-rows products work on tiles of 16 rows, the
library's products are measured size by size when an engine is made, the prompt attention cuts portions into
tiles of queries.  The parts that own those kernels say so with the functions here; the engine only asks the
model (``DecoderModel.step_rows``)."""
from __future__ import annotations

PORTION_ROWS = 64      # portions of prompts are run as multiples of this many tokens (a tile of queries)


def _pow2_at_least(n: int, floor: int = 1) -> int:
    v = max(int(floor), 1)
    while v < n:
        v *= 2
    return v


def few_rows_entries(entries: int) -> int:
    """Entries a step of ``entries`` decoding requests is run with: a power of two up to 16 (one tile of rows of
    the few-rows kernels), then a multiple of 16 up to 128 (what those kernels take) and of 32 beyond."""
    entries = max(int(entries), 1)
    if entries <= 16:
        return _pow2_at_least(entries)
    step = 16 if entries <= 128 else 32
    return -(-entries // step) * step


def _many_rows_spacing(rows: int, step: int) -> int:
    top, s = 64 * step, step
    while rows > top:
        top, s = 2 * top, 2 * s
    return s


def sizes_between(step_rows, kind: str, least: int, most: int) -> list:
    """Every number of rows from ``least`` on that ``step_rows(rows, kind)`` accepts, up to the one a step of
    ``most`` rows is run with; largest first (workspaces sized for them get their final sizes at once)."""
    top, n, sizes = int(step_rows(most, kind)), max(int(least), 1), []
    while True:
        s = int(step_rows(n, kind))
        if s > top:
            break
        sizes.append(s)
        n = s + 1
    return sizes[::-1]


class ProductRows:
    """``step_rows`` of a part whose work is matrix products over the step's rows: few-rows kernels on tiles of 16
    rows for decode steps, the library's products (measured size by size) for steps with portions, which are
    themselves run as multiples of PORTION_ROWS."""

    @staticmethod
    def step_rows(rows: int, kind: str) -> int:
        if kind == "decode":
            return few_rows_entries(rows)
        if kind in ("portion", "beside"):
            return -(-max(int(rows), 1) // PORTION_ROWS) * PORTION_ROWS
        return many_rows(rows)


def many_rows(rows: int, step: int = PORTION_ROWS) -> int:
    """Rows a step of ``rows`` rows with portions of prompts is run with: the next multiple of ``step`` up to
    4,096 rows, of 2 x ``step`` up to 8,192, of 4 x ``step`` up to 16,384 and so on (32 sizes an octave: measuring
    the library's products at every size when an engine is made stays affordable, and a step gets at most a 32nd
    more rows)."""
    rows = max(int(rows), 1)
    s = _many_rows_spacing(rows, step)
    return -(-rows // s) * s
