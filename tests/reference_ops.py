"""The plain C++ references of the operators (zedinfer_amd/csrc/host/reference_ops.cpp), compiled with the host
compiler into a temporary folder and called through ctypes with torch CPU tensors."""
import ctypes
import os
import shutil
import subprocess
import tempfile

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE = os.path.join(ROOT, "zedinfer_amd", "csrc", "host", "reference_ops.cpp")
_built = None


def _f(t):
    assert t.dtype == torch.float32 and t.is_contiguous() and t.device.type == "cpu"
    return ctypes.c_void_p(t.data_ptr())


def _i(t):
    if t is None:
        return ctypes.c_void_p(0)
    assert t.dtype == torch.int32 and t.is_contiguous() and t.device.type == "cpu"
    return ctypes.c_void_p(t.data_ptr())


def f32(t):
    return t.detach().to("cpu", torch.float32).contiguous()


def i32(t):
    return torch.as_tensor(t).detach().to("cpu", torch.int32).contiguous()


class ReferenceOps:
    def __init__(self, lib):
        self.lib = lib
        lib.ref_last_error.restype = ctypes.c_char_p

    def _call(self, name, *args):
        if getattr(self.lib, name)(*args) != 0:
            raise RuntimeError(self.lib.ref_last_error().decode())

    def embedding(self, table, ids):
        table, ids = f32(table), i32(ids)
        out = torch.empty(ids.numel(), table.shape[1])
        self._call("ref_embedding", _f(out), _f(table), _i(ids), ids.numel(), table.shape[0], table.shape[1])
        return out

    def rms_norm(self, x, w, eps, add_one=False):
        x, w = f32(x), f32(w)
        out = torch.empty_like(x)
        self._call("ref_rms_norm", _f(out), _f(x), _f(w), x.shape[0], x.shape[1], ctypes.c_float(eps), int(add_one))
        return out

    def add_rms_norm(self, resid, delta, w, eps, add_one=False):
        """(the new residual stream, its norm)"""
        resid, delta, w = f32(resid).clone(), f32(delta), f32(w)
        out = torch.empty_like(resid)
        self._call("ref_add_rms_norm", _f(resid), _f(delta), _f(out), _f(w), resid.shape[0], resid.shape[1],
                   ctypes.c_float(eps), int(add_one))
        return resid, out

    def linear(self, x, w, bias=None):
        x, w = f32(x), f32(w)
        b = f32(bias) if bias is not None else None
        out = torch.empty(x.shape[0], w.shape[0])
        self._call("ref_linear", _f(out), _f(x), _f(w), _f(b) if b is not None else ctypes.c_void_p(0), x.shape[0],
                   w.shape[0], x.shape[1])
        return out

    def rope_neox(self, x, pos, theta, rotary_dim=None):
        """x [n, heads, d]"""
        x, pos = f32(x).clone(), i32(pos)
        n, heads, d = x.shape
        self._call("ref_rope_neox", _f(x), _i(pos), n, heads, d, d if rotary_dim is None else rotary_dim,
                   ctypes.c_double(theta))
        return x

    def empty_cache(self, num_pages, nkv, d, ps):
        """(keys [page][kv_head][slot][dim], values [page][kv_head][dim][slot]), filled with NaN: a slot that was
        never stored must not be read."""
        return (torch.full((num_pages, nkv, ps, d), float("nan")), torch.full((num_pages, nkv, d, ps), float("nan")))

    def kv_store(self, kcache, vcache, k, v, slots):
        """k, v [n, nkv, d] into the caches, in place."""
        k, v, slots = f32(k), f32(v), i32(slots)
        num_pages, nkv, ps, d = kcache.shape
        self._call("ref_kv_store", _f(kcache), _f(vcache), _f(k), _f(v), _i(slots), k.shape[0], nkv, d, ps, num_pages)

    def paged_attention(self, q, kcache, vcache, block_tables, tok_seq, tok_pos, scale, window=0):
        """q [n, nh, d]"""
        q, block_tables, tok_seq, tok_pos = f32(q), i32(block_tables), i32(tok_seq), i32(tok_pos)
        n, nh, d = q.shape
        num_pages, nkv, ps, _ = kcache.shape
        out = torch.empty_like(q)
        self._call("ref_paged_attention", _f(out), _f(q), _f(kcache), _f(vcache), _i(block_tables), block_tables.shape[1],
                   _i(tok_seq), _i(tok_pos), n, nh, nkv, d, ps, num_pages, int(window or 0), ctypes.c_float(scale))
        return out

    def swiglu(self, gate, up):
        gate, up = f32(gate), f32(up)
        out = torch.empty_like(gate)
        self._call("ref_swiglu", _f(out), _f(gate), _f(up), ctypes.c_int64(gate.numel()))
        return out

    def argmax(self, logits):
        logits = f32(logits)
        out = torch.empty(logits.shape[0], dtype=torch.int32)
        self._call("ref_argmax", _i(out), _f(logits), logits.shape[0], logits.shape[1])
        return out

    def sample(self, logits, temperature, top_k, top_p, penalty, uniform, recent=None, recent_len=None):
        logits = f32(logits)
        R = logits.shape[0]
        out = torch.empty(R, dtype=torch.int32)
        t, k, p, pen, u = f32(temperature), i32(top_k), f32(top_p), f32(penalty), f32(uniform)
        rec = i32(recent) if recent is not None else None
        rlen = i32(recent_len) if recent_len is not None else None
        self._call("ref_sample", _i(out), _f(logits), R, logits.shape[1], _f(t), _i(k), _f(p), _f(pen), _f(u), _i(rec),
                   _i(rlen), rec.shape[1] if rec is not None else 0)
        return out


def load():
    """The compiled references, built once a process; None without a host C++ compiler."""
    global _built
    if _built is None:
        cxx = shutil.which("g++") or shutil.which("c++")
        if cxx is None:
            return None
        folder = tempfile.mkdtemp(prefix="zi_reference_ops_")
        lib = os.path.join(folder, "reference_ops.so")
        subprocess.run([cxx, "-O2", "-std=c++17", "-shared", "-fPIC", "-Wall", "-Werror", "-o", lib, SOURCE], check=True)
        _built = ReferenceOps(ctypes.CDLL(lib))
    return _built
