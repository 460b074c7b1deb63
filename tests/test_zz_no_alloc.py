"""The one entry point that allocates nothing (lffn_layer_norm_bwd_noalloc_f32: partial sums in a static
device array held by the library) against the existing entry points it is a variant of
(lffn_layer_norm_bwd_f32 + lffn_sum_partials_f32 with caller-provided partial buffers), through the C ABI:
bit-identical results, on two calls in a row, the second with a smaller input, so that whatever the
first call left in the shared buffer must not show in the second."""
import numpy as np
import pytest
import torch

from lookupffn_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(x, w, eps, g_y):
    """-> (g_x, g_w, g_b) from the no-alloc entry point and from the existing pair of calls."""
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    R, B, H = g_y.shape
    xd, gd = torch.from_numpy(x).to(DEV), torch.from_numpy(g_y).to(DEV)
    wd = None if w is None else torch.from_numpy(w).to(DEV)
    p = lambda t: None if t is None else t.data_ptr()
    # the existing entry points, partial sums in a caller-provided buffer
    n = max(1, min(512, (B + 3) // 4))
    gx_ref = torch.full((B, H), float("nan"), device=DEV)
    part = torch.full((2, n, H), float("nan"), device=DEV)
    gw_ref = torch.full((H,), float("nan"), device=DEV)
    gb_ref = torch.full((H,), float("nan"), device=DEV)
    assert lib.lffn_layer_norm_bwd_f32(p(xd), p(wd), eps, p(gd), p(gx_ref), p(part[0]), p(part[1]), B, H, R, n, stream) == 0
    assert lib.lffn_sum_partials_f32(p(part[0]), p(gw_ref), H, p(part[1]), p(gb_ref), H, n, 1, stream) == 0
    # the entry point that allocates nothing: inputs and outputs only
    gx = torch.full((B, H), float("nan"), device=DEV)
    gw = torch.full((H,), float("nan"), device=DEV)
    gb = torch.full((H,), float("nan"), device=DEV)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.lffn_layer_norm_bwd_noalloc_f32(p(xd), p(wd), eps, p(gd), p(gx), p(gw), p(gb), B, H, R, stream)
    assert rc == 0, lib.lffn_error_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return [t.cpu().numpy() for t in (gx, gw, gb)], [t.cpu().numpy() for t in (gx_ref, gw_ref, gb_ref)]


def test_layer_norm_bwd_noalloc_matches_the_existing_entry_points_on_two_calls_in_a_row():
    rng = np.random.RandomState(7)
    # first call: every one of the 512 partial rows at the widest row the buffer holds
    # second call: fewer rows and narrower ones, so the buffer still holds the first call's sums
    # beside and behind the part this call uses; then a third, larger again, with two repeats
    for B, H, R, affine in ((5000, 1024, 1, True), (333, 260, 1, True), (2100, 768, 2, False)):
        x = rng.randn(B, H).astype(np.float32)
        w = (1 + 0.1 * rng.randn(H)).astype(np.float32) if affine else None
        g_y = rng.randn(R, B, H).astype(np.float32)
        got, want = _both(x, w, 1e-5, g_y)
        for a, b, name in zip(got, want, ("g_x", "g_weight", "g_bias")):
            assert not np.isnan(a).any(), (B, H, name)
            assert np.array_equal(a, b), (B, H, name)
        # and against the closed form in float64
        g = g_y.astype(np.float64).sum(0)
        x64 = x.astype(np.float64)
        mu = x64.mean(1, keepdims=True)
        xh = (x64 - mu) / np.sqrt(x64.var(1, keepdims=True) + 1e-5)
        assert np.abs(got[1] - (g * xh).sum(0)).max() <= 1e-4 * np.abs((g * xh).sum(0)).max()
        assert np.abs(got[2] - g.sum(0)).max() <= 1e-4 * np.abs(g.sum(0)).max()


def test_layer_norm_bwd_noalloc_rejects_what_the_buffer_cannot_hold():
    lib = _lib.load()
    t = torch.zeros(8, 2048, device=DEV)
    o = torch.zeros(2048, device=DEV)
    rc = lib.lffn_layer_norm_bwd_noalloc_f32(t.data_ptr(), None, 1e-5, t.data_ptr(), t.data_ptr(), o.data_ptr(), o.data_ptr(),
                                             2048, 2048, 1, None)
    assert rc == _lib.LFFN_ERR_SCRATCH
    assert b"scratch" in lib.lffn_error_string(rc)
    # ... also with so few rows that their partial sums alone would fit
    rc = lib.lffn_layer_norm_bwd_noalloc_f32(t.data_ptr(), None, 1e-5, t.data_ptr(), t.data_ptr(), o.data_ptr(), o.data_ptr(),
                                             8, 2048, 1, None)
    assert rc == _lib.LFFN_ERR_SCRATCH
    # an empty batch: zeros for the parameter gradients
    gw = torch.full((64,), float("nan"), device=DEV)
    gb = torch.full((64,), float("nan"), device=DEV)
    rc = lib.lffn_layer_norm_bwd_noalloc_f32(None, None, 1e-5, None, None, gw.data_ptr(), gb.data_ptr(), 0, 64, 1,
                                             torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert gw.abs().max().item() == 0 and gb.abs().max().item() == 0
