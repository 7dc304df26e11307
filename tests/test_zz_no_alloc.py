"""The argmax entry point that allocates nothing (`picolm_argmax_static`), called through ctypes
as a C caller would: its tokens equal `picolm_argmax`'s on two calls in a row that share the
library's scratch array, the second with a smaller input; sizes beyond the array are refused."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _library():
    from picolm_amd.csrc import build
    lib = build.load()
    lib.picolm_last_error.restype = ctypes.c_char_p
    for name in ("picolm_argmax", "picolm_argmax_static", "picolm_argmax_static_max_floats",
                 "picolm_argmax_scratch_floats"):
        getattr(lib, name).restype = ctypes.c_int
    return lib


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, logits):
    n, V = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    want = torch.full((n,), -1, dtype=torch.int32, device=DEV)
    scratch = torch.empty(lib.picolm_argmax_scratch_floats(n, V), dtype=torch.float32, device=DEV)
    rc = lib.picolm_argmax(_ptr(logits), _ptr(want), n, V, ctypes.c_int64(V), _ptr(scratch), stream)
    assert rc == 0, lib.picolm_last_error()
    got = torch.full((n,), -1, dtype=torch.int32, device=DEV)
    rc = lib.picolm_argmax_static(_ptr(logits), _ptr(got), n, V, ctypes.c_int64(V), stream)
    assert rc == 0, lib.picolm_last_error()
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_argmax_static_equals_argmax_on_two_calls_in_a_row():
    lib = _library()
    g = torch.Generator().manual_seed(11)
    # a large call fills much of the array; the smaller one that follows finds its leftovers there
    first = torch.randn(48, 128256, generator=g).to(DEV)
    first[5, 77] = first[5, 100000] = 50.0            # two equal maxima: the first one wins
    got, want = _both(lib, first)
    assert torch.equal(got, want)
    assert got[5] == 77
    others = [i for i in range(48) if i != 5]
    assert torch.equal(got.long()[others], first.cpu().argmax(dim=1)[others])
    second = torch.randn(3, 5000, generator=g).to(DEV)
    second[1, 4999] = 60.0                            # the last column of a slice that is not full
    got, want = _both(lib, second)
    assert torch.equal(got, want)
    assert got[1] == 4999
    assert torch.equal(got.long(), second.cpu().argmax(dim=1))


def test_argmax_static_refuses_what_its_array_cannot_hold():
    lib = _library()
    limit = lib.picolm_argmax_static_max_floats()
    V = 128256
    slices = (V + 4095) // 4096
    rows = limit // (2 * slices) + 1
    logits = torch.zeros(1, device=DEV)               # never read: the call is refused on the host
    out = torch.zeros(1, dtype=torch.int32, device=DEV)
    rc = lib.picolm_argmax_static(_ptr(logits), _ptr(out), rows, V, ctypes.c_int64(V), ctypes.c_void_p(0))
    assert rc != 0
    assert b"scratch" in lib.picolm_last_error()
