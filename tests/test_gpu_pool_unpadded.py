"""Pooling over row tiles that carry no halo (adh_pool2d_unpadded_{fwd,bwd}_tiles): tile t of the result must be
the rows of the pooling of the UNSPLIT, zero-padded tensor that belong to it - what pad -> exchange -> pool
(forward) and pool backward -> reduce -> unpad (backward) compute in the reference's graph.  Checked against
the CPU oracle's pooling of the unsplit padded tensor.  Max forward moves values: bit-exact.  Average forward
and both backward passes add a handful of fp32 terms: rel-err max|a-b| / max|b| <= 1e-5 in fp32, <= 2^-8 in
bf16.  Every call goes through the C ABI."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu
TOL32, TOL16 = 1e-5, 2.0 ** -8

CASES = [  # K, N, C, Ht, W, wh, ww, sh, sw, pad_h, pad_w
    (4, 2, 5, 8, 30, 3, 3, 2, 2, 1, 1),     # the stem's pooling: 3x3 stride 2 pad 1
    (2, 1, 3, 2, 9, 3, 3, 2, 2, 1, 1),      # two rows per tile: one output row, its window half in the neighbour
    (3, 2, 2, 6, 17, 3, 3, 1, 1, 1, 1),     # stride 1: rows from both neighbours
    (1, 2, 3, 8, 12, 3, 3, 2, 2, 1, 1),     # one tile: pooling with zero padding
    (2, 1, 2, 6, 10, 2, 2, 2, 2, 0, 0),     # 2x2 stride 2 without padding: no neighbour is read
    (4, 8, 64, 16, 200, 3, 3, 2, 2, 1, 1),  # several bands per plane
    (2, 2, 4, 6, 11, 5, 3, 1, 2, 2, 0),     # 5 rows (two from each neighbour), different per axis
    (5, 1, 2, 4, 8, 3, 3, 2, 1, 1, 1),
]


def unsplit_reference(oracle, mode, x, dy, geo, pad_h, pad_w):
    wh, ww, sh, sw = geo
    N, C, H, W = x.shape
    xp = np.zeros((N, C, H + 2 * pad_h, W + 2 * pad_w), np.float32)
    xp[:, :, pad_h:pad_h + H, pad_w:pad_w + W] = x
    y = np.empty(dy.shape, np.float32)
    oracle.pool_slab_fwd(mode, xp, wh, ww, sh, sw, y)
    gp = np.empty(xp.shape, np.float32)
    oracle.pool_slab_bwd(mode, xp, dy, wh, ww, sh, sw, gp)
    return y, gp[:, :, pad_h:pad_h + H, pad_w:pad_w + W]


@pytest.mark.parametrize("mode", [capi.ADH_POOL_AVG, capi.ADH_POOL_MAX])
@pytest.mark.parametrize("K,N,C,Ht,W,wh,ww,sh,sw,pad_h,pad_w", CASES)
def test_pool_unpadded_f32_vs_unsplit_oracle(oracle, mode, K, N, C, Ht, W, wh, ww, sh, sw, pad_h, pad_w):
    rng = np.random.default_rng(77 + W + K)
    geo = (wh, ww, sh, sw)
    H, OHt, OW = K * Ht, Ht // sh, (W + 2 * pad_w - ww) // sw + 1
    x = rng.uniform(-1, 1, size=(N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, C, K * OHt, OW)).astype(np.float32)
    y_want, g_want = unsplit_reference(oracle, mode, x, dy, geo, pad_h, pad_w)
    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * OHt:(r + 1) * OHt, :].copy()) for r in range(K)]
    g0 = [rng.standard_normal((N, C, Ht, W)).astype(np.float32) for _ in range(K)]
    ys = [torch.full((N, C, OHt, OW), float("nan"), device="cuda") for _ in range(K)]
    capi.check(capi.pool_unpadded_fwd_tiles(mode, xs, ys, N, C, Ht, W, *geo, pad_h, pad_w), "fwd")
    gs = [torch.full((N, C, Ht, W), float("nan"), device="cuda") for _ in range(K)]
    capi.check(capi.pool_unpadded_bwd_tiles(mode, xs, ys, dys, gs, N, C, Ht, W, *geo, pad_h, pad_w), "bwd")
    acc = [dev(a) for a in g0]
    capi.check(capi.pool_unpadded_bwd_tiles(mode, xs, None, dys, acc, N, C, Ht, W, *geo, pad_h, pad_w, beta=1.0), "bwd beta 1")
    for r in range(K):
        want_y = y_want[:, :, r * OHt:(r + 1) * OHt, :]
        if mode == capi.ADH_POOL_MAX:
            assert np.array_equal(host(ys[r]), want_y)
        else:
            assert rel_err(host(ys[r]), want_y) <= TOL32
        want_g = g_want[:, :, r * Ht:(r + 1) * Ht, :]
        assert rel_err(host(gs[r]), want_g) <= TOL32
        assert rel_err(host(acc[r]), want_g + g0[r]) <= TOL32


@pytest.mark.parametrize("mode", [capi.ADH_POOL_AVG, capi.ADH_POOL_MAX])
def test_pool_unpadded_bf16_vs_unsplit_oracle(oracle, mode):
    K, N, C, Ht, W, geo, pad = 4, 2, 6, 8, 30, (3, 3, 2, 2), 1
    rng = np.random.default_rng(78)
    bf = lambda a: oracle.f32_to_bf16(a.astype(np.float32))
    H, OHt, OW = K * Ht, Ht // 2, (W + 2 - 3) // 2 + 1
    x = bf(rng.uniform(-1, 1, size=(N, C, H, W)))
    dy = bf(rng.standard_normal((N, C, K * OHt, OW)))
    y_want, g_want = unsplit_reference(oracle, mode, oracle.bf16_to_f32(x), oracle.bf16_to_f32(dy), geo, pad, pad)
    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * OHt:(r + 1) * OHt, :].copy()) for r in range(K)]
    ys = [torch.empty((N, C, OHt, OW), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    gs = [torch.empty((N, C, Ht, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.pool_unpadded_fwd_tiles(mode, xs, ys, N, C, Ht, W, *geo, pad, pad))
    capi.check(capi.pool_unpadded_bwd_tiles(mode, xs, ys, dys, gs, N, C, Ht, W, *geo, pad, pad))
    for r in range(K):
        want_y = y_want[:, :, r * OHt:(r + 1) * OHt, :]
        if mode == capi.ADH_POOL_MAX:
            assert np.array_equal(host(ys[r]), oracle.f32_to_bf16(want_y))  # a max of bf16 values (or the padding's zero) is one of them
        else:
            assert rel_err(oracle.bf16_to_f32(host(ys[r])), want_y) <= TOL16
        assert rel_err(oracle.bf16_to_f32(host(gs[r])), g_want[:, :, r * Ht:(r + 1) * Ht, :]) <= TOL16


def test_pool_unpadded_negative_border_and_ties(oracle):
    """All values negative: at the tensor's border the padding's zero is the maximum and its gradient belongs to no
    pixel; equal values inside a window: the first in row-major order takes the gradient, across a tile border too."""
    K, N, C, Ht, W = 2, 1, 2, 4, 6
    x = np.full((N, C, K * Ht, W), -1.0, np.float32)
    x[:, :, 3:5, 2:4] = -0.5  # a tie that straddles the border between the tiles
    dy = np.arange(N * C * (K * Ht // 2) * 3, dtype=np.float32).reshape(N, C, K * Ht // 2, 3) + 1.0
    y_want, g_want = unsplit_reference(oracle, capi.ADH_POOL_MAX, x, dy, (3, 3, 2, 2), 1, 1)
    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * 2:(r + 1) * 2, :].copy()) for r in range(K)]
    ys = [torch.empty((N, C, 2, 3), device="cuda") for _ in range(K)]
    gs = [torch.empty((N, C, Ht, W), device="cuda") for _ in range(K)]
    capi.check(capi.pool_unpadded_fwd_tiles(capi.ADH_POOL_MAX, xs, ys, N, C, Ht, W, 3, 3, 2, 2, 1, 1))
    capi.check(capi.pool_unpadded_bwd_tiles(capi.ADH_POOL_MAX, xs, ys, dys, gs, N, C, Ht, W, 3, 3, 2, 2, 1, 1))
    for r in range(K):
        assert np.array_equal(host(ys[r]), y_want[:, :, r * 2:(r + 1) * 2, :])
        assert np.array_equal(host(gs[r]), g_want[:, :, r * Ht:(r + 1) * Ht, :])
    assert y_want[0, 0, 0, 0] == 0.0  # the border window's maximum is the padding


def test_pool_unpadded_limits():
    x = [torch.zeros((1, 1, 5, 8), device="cuda") for _ in range(2)]
    y = [torch.zeros((1, 1, 5, 8), device="cuda") for _ in range(2)]
    f = lambda Ht, wh, sh, pad: capi.pool_unpadded_fwd_tiles(capi.ADH_POOL_MAX, x, y, 1, 1, Ht, 8, wh, 3, sh, 1, pad, 1)
    assert f(5, 3, 2, 1) == capi.ADH_EINVAL   # five rows at stride 2: the tiles' outputs do not stitch
    assert f(4, 3, 1, 0) == capi.ADH_EINVAL   # no padding: the unsplit pooling has fewer rows than the tiles
    assert f(4, 3, 1, 2) == capi.ADH_EINVAL   # too much padding
    assert f(4, 3, 1, 1) == capi.ADH_OK
