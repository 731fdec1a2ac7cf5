"""The entry point that allocates nothing: mpsa_seq_mean_static against mpsa_seq_mean through the C ABI.

Two calls in a row on the same GPU, the second on a smaller input, so that stale partial sums of the first call
sit in the library's built-in array behind the second call's; the results must equal the workspace entry point's
bit for bit (same kernels, same summation order)."""
import ctypes

import pytest
import torch

from ours import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _mean_workspace(x):
    B, H, N, D = x.shape
    L = _lib.lib()
    ws = torch.empty(max(L.mpsa_seq_mean_workspace(B, H, N, D), 4), dtype=torch.uint8, device=x.device)
    out = torch.empty((B, H, D), dtype=x.dtype, device=x.device)
    _lib.check(L.mpsa_seq_mean(_lib.ptr(x), _lib.dtype_id(x.dtype), B, H, N, D, _lib.strides4(x), _lib.ptr(ws),
                               _lib.ptr(out), _lib.stream_ptr(x.device)))
    return out


def _mean_static(x, out):
    B, H, N, D = x.shape
    return _lib.lib().mpsa_seq_mean_static(_lib.ptr(x), _lib.dtype_id(x.dtype), B, H, N, D, _lib.strides4(x),
                                           _lib.ptr(out), _lib.stream_ptr(x.device))


def test_static_scratch_mean_equals_workspace_mean_twice_in_a_row():
    g = torch.Generator().manual_seed(11)
    big = (torch.randn(1, 8, 8192 + 77, 128, generator=g) + 0.25).to(torch.bfloat16).to(DEV)
    small = (torch.randn(2, 3, 300, 64, generator=g) * 3 - 1).to(torch.float16).to(DEV)
    want_big, want_small = _mean_workspace(big), _mean_workspace(small)
    # outputs are allocated before the calls under test; those calls themselves allocate nothing
    got_big = torch.empty_like(want_big)
    got_small = torch.empty_like(want_small)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    _lib.check(_mean_static(big, got_big))
    _lib.check(_mean_static(small, got_small))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(got_big.view(torch.int16), want_big.view(torch.int16))
    assert torch.equal(got_small.view(torch.int16), want_small.view(torch.int16))
    # and the mean is the mean: against a float64 reduction, within one 16-bit rounding
    ref = big.double().mean(dim=-2)
    assert (got_big.double() - ref).abs().max().item() <= 2.0 ** -8 * max(ref.abs().max().item(), 1.0)


def test_static_scratch_mean_rejects_what_does_not_fit():
    L = _lib.lib()
    limit = 4194304
    one = ctypes.c_void_p(16)
    st = (ctypes.c_int64 * 4)(128, 128, 128, 1)
    # 64 heads x 1024 chunks x 128 channels x 4 bytes = 32 MiB of partial sums
    assert L.mpsa_seq_mean_workspace(1, 64, 262144, 128) > limit
    assert L.mpsa_seq_mean_static(one, 0, 1, 64, 262144, 128, st, one, None) == -3
    assert b"exceed" in L.mpsa_last_error()
    # exactly at the limit is accepted by the size check (the null input is what fails then)
    assert L.mpsa_seq_mean_workspace(1, 8, 262144, 128) == limit
    assert L.mpsa_seq_mean_static(None, 0, 1, 8, 262144, 128, st, one, None) == -1
