"""The entry point of the kernel library that allocates nothing (zi_argmax_static), called through
ctypes as a caller outside this package would: its results against zi_argmax with a workspace, on two
calls in a row of which the second is smaller (the library's array keeps the first call's parts), and
its refusal of sizes beyond the array."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def library():
    from zedinfer_amd import ops
    ops.load()
    lib = ctypes.CDLL(ops.library_path())
    P, I, L = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
    lib.zi_argmax_static.argtypes = [P, P, P, I, I, I, L, P]
    lib.zi_argmax_static.restype = I
    lib.zi_argmax.argtypes = [P, P, P, I, I, I, L, P, L, P]
    lib.zi_argmax.restype = I
    lib.zi_argmax_workspace.argtypes = [I, I]
    lib.zi_argmax_workspace.restype = L
    lib.zi_argmax_static_max_parts.argtypes = []
    lib.zi_argmax_static_max_parts.restype = I
    lib.zi_last_error.argtypes = []
    lib.zi_last_error.restype = ctypes.c_char_p
    return lib


def both(lib, logits, code):
    """(index, value) of zi_argmax_static and of zi_argmax with a workspace, for one logits tensor."""
    R, V = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    need = lib.zi_argmax_workspace(R, V)
    assert need > 0                      # rows long enough to be cut: the path that needs memory
    ws = torch.empty((need,), dtype=torch.float32, device="cuda")
    for name in ("static", "workspace"):
        idx = torch.full((R,), -7, dtype=torch.int32, device="cuda")
        val = torch.full((R,), float("nan"), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        if name == "static":
            rc = lib.zi_argmax_static(idx.data_ptr(), val.data_ptr(), logits.data_ptr(), code, R, V, logits.stride(0),
                                      stream)
        else:
            rc = lib.zi_argmax(idx.data_ptr(), val.data_ptr(), logits.data_ptr(), code, R, V, logits.stride(0),
                               ws.data_ptr(), need, stream)
        assert rc == 0, lib.zi_last_error()
        torch.cuda.synchronize()
        out[name] = (idx.cpu(), val.cpu())
    return out


@pytest.mark.parametrize("dtype,code", [(torch.float32, 0), (torch.bfloat16, 1)])
def test_argmax_static_equals_argmax_on_two_calls_in_a_row(dtype, code):
    lib = library()
    g = torch.Generator().manual_seed(5)
    # the first call fills the library's array with 7 rows x 19 parts, the second uses less of it
    for R, V in ((7, 151936), (3, 20011)):
        logits = torch.randn(R, V, generator=g).to(dtype).cuda()
        logits[0, V - 1] = 50.0                       # the last value of the last part
        logits[1, 8192] = logits[1, 3] = 60.0         # equal values in two parts: the lower index wins
        got = both(lib, logits, code)
        assert torch.equal(got["static"][0], got["workspace"][0])
        assert torch.equal(got["static"][1], got["workspace"][1])
        want = torch.argmax(logits.float(), dim=1).cpu()
        assert got["static"][0][0] == V - 1 and got["static"][0][1] == 3
        assert torch.equal(got["static"][0][2:].long(), want[2:])
        assert torch.equal(got["static"][1], logits.float().max(dim=1).values.cpu())


def test_argmax_static_refuses_what_its_array_cannot_hold():
    lib = library()
    limit = lib.zi_argmax_static_max_parts()
    V = 3 * 8192 + 1                                  # four parts a row
    R = limit // 4 + 1
    logits = torch.zeros((R, V), dtype=torch.bfloat16, device="cuda")
    idx = torch.full((R,), -7, dtype=torch.int32, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.zi_argmax_static(idx.data_ptr(), None, logits.data_ptr(), 1, R, V, V, stream)
    assert rc != 0 and b"parts" in lib.zi_last_error()
    torch.cuda.synchronize()
    assert int(idx.min()) == -7 and int(idx.max()) == -7        # nothing ran
    rc = lib.zi_argmax_static(idx.data_ptr(), None, logits.data_ptr(), 1, R - 1, V, V, stream)
    assert rc == 0, lib.zi_last_error()
    torch.cuda.synchronize()
    assert int(idx[:R - 1].max()) == 0 and int(idx[R - 1]) == -7
