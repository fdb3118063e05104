"""sae_col_sum_static: the allocation-free column sum (partial sums in a fixed device array inside the library)
against sae_col_sum with a caller workspace, through the C ABI.  Bit-exact: both run the same kernels in the same
order of additions.  Two calls in a row, the second on a smaller input, so that what the first call left in the
shared array would show if the second read any of it."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _with_workspace(lib, pkg, src, accumulate=False, out=None):
    B, n = src.shape
    out = torch.empty(n, dtype=torch.float32, device=src.device) if out is None else out
    nbytes = lib.sae_col_sum_workspace_bytes(B, n)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=src.device)
    stream = torch.cuda.current_stream(src.device).cuda_stream
    pkg._lib.check(lib.sae_col_sum(src.data_ptr(), out.data_ptr(), B, n, int(accumulate), ws.data_ptr(), nbytes, stream))
    return out


def _static(lib, pkg, src, out, accumulate=False):
    B, n = src.shape
    stream = torch.cuda.current_stream(src.device).cuda_stream
    pkg._lib.check(lib.sae_col_sum_static(src.data_ptr(), out.data_ptr(), B, n, int(accumulate), stream))
    return out


def test_static_col_sum_matches_workspace_col_sum_on_two_calls(pkg, dev):
    lib = pkg._lib.load()
    g = torch.Generator().manual_seed(11)
    big = torch.randn(4096, 4096, generator=g).to(dev)
    small = torch.randn(37, 1000, generator=g).to(dev)          # fewer chunks, fewer columns, ragged tail
    out_big = torch.empty(4096, dtype=torch.float32, device=dev)
    out_small = torch.full((1000,), 3.0, dtype=torch.float32, device=dev)
    want_big = _with_workspace(lib, pkg, big)
    want_small = _with_workspace(lib, pkg, small, accumulate=True, out=torch.full((1000,), 3.0, device=dev))
    _static(lib, pkg, big, out_big)
    _static(lib, pkg, small, out_small, accumulate=True)         # second call, smaller input, adds to out
    torch.cuda.synchronize()
    assert torch.equal(out_big, want_big)
    assert torch.equal(out_small, want_small)
    # and against exact arithmetic: fp64 column sums
    ref = big.double().sum(0)
    assert ((out_big.double() - ref).abs().max() / ref.abs().max()).item() < 1e-5


def test_static_col_sum_rejects_what_does_not_fit(pkg, dev):
    lib = pkg._lib.load()
    src = torch.zeros(2, 16385, device=dev)
    out = torch.zeros(16385, device=dev)
    rc = lib.sae_col_sum_static(src.data_ptr(), out.data_ptr(), 2, 16385, 0, None)
    assert rc == -2 and b"16384" in lib.sae_last_error()
    assert lib.sae_col_sum_static(None, out.data_ptr(), 2, 8, 0, None) == -1
