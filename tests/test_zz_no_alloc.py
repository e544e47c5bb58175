"""The entry point that allocates nothing (liyab_argmax_static, csrc/no_alloc.h), called
through ctypes as a caller without torch would, against the existing liyab_argmax: two calls
in a row, the second with a smaller input, so that what the first left in the library's own
scratch array is still there when the second runs."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

MAX_ROWS = 1024  # LIYAB_ARGMAX_STATIC_MAX_ROWS


def _library():
    from liyab_amd.csrc import build

    path = build.find_library()
    assert path is not None, "the kernel library is not built (python -m liyab_amd.csrc.build)"
    lib = ctypes.CDLL(path)
    P = ctypes.c_void_p
    lib.liyab_last_error.restype = ctypes.c_char_p
    lib.liyab_argmax_static_init.restype = ctypes.c_int
    lib.liyab_argmax_static_init.argtypes = []
    lib.liyab_argmax_static.restype = ctypes.c_int
    lib.liyab_argmax_static.argtypes = [P, P, ctypes.c_int64, ctypes.c_int, ctypes.c_int, P, P, P]
    lib.liyab_argmax.restype = ctypes.c_int
    lib.liyab_argmax.argtypes = [P, P, ctypes.c_int64, ctypes.c_int, ctypes.c_int, P, P, P, P, P]
    return lib


def _both(lib, logits, scatter=None):
    """(the static entry point's tokens, the existing one's) for float32 logits [rows, V]."""
    rows, V = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    out_static = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)
    out_ref = torch.full((rows,), -9, dtype=torch.int32, device=logits.device)
    sv = torch.empty(rows * 64, dtype=torch.float32, device=logits.device)
    si = torch.empty(rows * 64, dtype=torch.int32, device=logits.device)
    idx = tgt = tgt_ref = None
    if scatter is not None:
        idx = scatter
        tgt = torch.full((int(idx.max()) + 1,), -1, dtype=torch.int32, device=logits.device)
        tgt_ref = tgt.clone()
    ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
    rc = lib.liyab_argmax(out_ref.data_ptr(), logits.data_ptr(), logits.stride(0), rows, V, sv.data_ptr(), si.data_ptr(),
                          ptr(idx), ptr(tgt_ref), stream)
    assert rc == 0, lib.liyab_last_error().decode()
    rc = lib.liyab_argmax_static(out_static.data_ptr(), logits.data_ptr(), logits.stride(0), rows, V, ptr(idx), ptr(tgt),
                                 stream)
    assert rc == 0, lib.liyab_last_error().decode()
    torch.cuda.synchronize()
    if scatter is not None:
        assert torch.equal(tgt, tgt_ref)
    return out_static.cpu(), out_ref.cpu()


def test_static_argmax_equals_the_workspace_one_twice_in_a_row():
    lib = _library()
    assert lib.liyab_argmax_static_init() == 0, lib.liyab_last_error().decode()
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(77)
    # first call: many rows of a vocabulary that is no multiple of anything, with ties in some rows
    big = torch.randn(300, 50257, generator=g).to(dev)
    big[5, 40000] = big[5, 123] = 9.0  # a tie: the lowest id wins
    big[17] = 0.25  # a whole row of ties
    a, b = _both(lib, big)
    assert torch.equal(a, b)
    plain_rows = [r for r in range(300) if r not in (5, 17)]  # rows without ties: the library's argmax agrees
    assert torch.equal(a.long()[plain_rows], torch.argmax(big, dim=1).cpu()[plain_rows])
    assert int(a[5]) == 123 and int(a[17]) == 0
    # second call, smaller in both sizes, rows of a wider buffer: the array still holds the first call's pairs
    wide = torch.randn(7, 1200, generator=g).to(dev)
    small = wide[:, :777]
    small[3, 776] = 50.0  # the last entry of the row
    idx = torch.tensor([4, 0, 9, 2, 6, 1, 3], dtype=torch.int32, device=dev)
    a, b = _both(lib, small, scatter=idx)
    assert torch.equal(a, b)
    assert torch.equal(a.long(), torch.argmax(small, dim=1).cpu())
    assert int(a[3]) == 776
    # a third, of one row, and the limit
    one = torch.randn(1, 33, generator=g).to(dev)
    a, b = _both(lib, one)
    assert torch.equal(a, b) and int(a[0]) == int(torch.argmax(one))
    full = torch.randn(MAX_ROWS, 130, generator=g).to(dev)
    a, b = _both(lib, full)
    assert torch.equal(a, b) and torch.equal(a.long(), torch.argmax(full, dim=1).cpu())


def test_static_argmax_refuses_what_its_array_cannot_hold():
    lib = _library()
    dev = torch.device("cuda:0")
    logits = torch.zeros(MAX_ROWS + 1, 8, device=dev)
    out = torch.zeros(MAX_ROWS + 1, dtype=torch.int32, device=dev)
    rc = lib.liyab_argmax_static(out.data_ptr(), logits.data_ptr(), 8, MAX_ROWS + 1, 8, None, None,
                                 torch.cuda.current_stream().cuda_stream)
    assert rc != 0 and b"1024" in lib.liyab_last_error()
    rc = lib.liyab_argmax_static(None, logits.data_ptr(), 8, 4, 8, None, None, torch.cuda.current_stream().cuda_stream)
    assert rc != 0
    rc = lib.liyab_argmax_static(out.data_ptr(), logits.data_ptr(), 4, 4, 8, None, None, torch.cuda.current_stream().cuda_stream)
    assert rc != 0  # rows shorter than the vocabulary
