"""The argmax entry point that allocates nothing (its scratch is a static device array), called through ctypes as a
caller outside the package would: its output against the existing entry point's, on two calls in a row, the second
with a smaller input, so that what the first call left in the shared scratch must not matter."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from inferflux_amd.kernels.library import find_library, load_module
    path = find_library("sampling") or load_module("sampling").path
    lib = ctypes.CDLL(path)
    P, I = ctypes.c_void_p, ctypes.c_int
    lib.ifx_argmax_static.argtypes, lib.ifx_argmax_static.restype = [P, I, I, P, P], I
    lib.ifx_argmax.argtypes, lib.ifx_argmax.restype = [P, I, I, P, P, P, P], I
    lib.ifx_last_error.restype = ctypes.c_char_p
    return lib


def _both(lib, logits):
    R, V = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    got = torch.full((R,), -7, dtype=torch.int32, device="cuda")
    want = torch.full((R,), -9, dtype=torch.int32, device="cuda")
    pv = torch.empty((R, 32), dtype=torch.float32, device="cuda")
    pi = torch.empty((R, 32), dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    assert lib.ifx_argmax_static(logits.data_ptr(), R, V, got.data_ptr(), stream) == 0, lib.ifx_last_error()
    assert lib.ifx_argmax(logits.data_ptr(), R, V, want.data_ptr(), pv.data_ptr(), pi.data_ptr(), stream) == 0, lib.ifx_last_error()
    torch.cuda.synchronize()
    return got.cpu(), want.cpu()


def test_static_scratch_argmax_matches_the_workspace_one_on_two_calls_in_a_row():
    lib = _lib()
    g = torch.Generator(device="cuda").manual_seed(5)
    big = torch.randn((64, 152064), generator=g, device="cuda")
    big[3, 777] = big[3, 140000] = 50.0                        # a tie: the lowest index wins in both
    big[9] = -float("inf")                                     # a row without a finite value
    small = torch.randn((5, 40001), generator=g, device="cuda")
    for logits in (big, small):                                # the second call is smaller: stale slots of the first must not be read
        got, want = _both(lib, logits)
        assert torch.equal(got, want)
        assert torch.equal(got.long(), torch.argmax(logits, dim=1).cpu()) or logits is big   # (torch's tie rule may differ)
    assert int(_both(lib, big)[0][3]) == 777
    # a narrow row takes the one-kernel path, which needs no scratch at all
    narrow = torch.randn((7, 1000), generator=g, device="cuda")
    got, want = _both(lib, narrow)
    assert torch.equal(got, want) and torch.equal(got.long(), torch.argmax(narrow, dim=1).cpu())


def test_static_scratch_argmax_refuses_more_rows_than_it_holds():
    lib = _lib()
    logits = torch.zeros((1025, 16384), device="cuda")
    out = torch.zeros(1025, dtype=torch.int32, device="cuda")
    rc = lib.ifx_argmax_static(logits.data_ptr(), 1025, 16384, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == -1 and b"at most 1024" in lib.ifx_last_error()
    assert lib.ifx_argmax_static(logits.data_ptr(), 1024, 16384, out.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    assert int(out[:1024].abs().max()) == 0                    # all zeros: index 0 is the lowest maximum


def test_static_scratch_argmax_allocates_nothing():
    lib = _lib()
    logits = torch.randn((8, 152064), device="cuda")
    out = torch.zeros(8, dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.ifx_argmax_static(logits.data_ptr(), 8, 152064, out.data_ptr(), stream) == 0     # (the first call looks the symbol up)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    reserved_before = torch.cuda.memory_reserved()
    for _ in range(20):
        assert lib.ifx_argmax_static(logits.data_ptr(), 8, 152064, out.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == reserved_before
    assert torch.equal(out.cpu().long(), torch.argmax(logits, dim=1).cpu())
