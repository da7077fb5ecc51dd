"""Pins the pooling half of the CPU oracle.

The pooling arithmetic of the reference lives in cuDNN (closed source, absent), so the
oracle restates the published definition (window max / window mean, pad 0 over the
halo-padded tile).  It is pinned here against
  * torch.nn.functional.max_pool2d / avg_pool2d and torch autograd on the CPU;
  * closed forms: a 1x1 window with stride 1 is the identity, the average backward of
    all-ones dy counts the windows over each pixel, the gradients of one plane sum to
    the sum of dy (every window hands out exactly its dy);
  * the split/unsplit identity: pooling the packed halo tiles and stacking the outputs
    == pooling the zero-padded unsplit tensor.
Which element receives the max gradient when several window elements are equal is
cuDNN's choice: parity unpinned; the oracle takes the first in row-major window order,
which is also what torch's CPU kernel does (checked below on a constant input).
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

CASES = [(2, 3, 8, 9, 3, 3, 2, 2), (1, 2, 7, 7, 2, 2, 2, 2), (1, 1, 6, 10, 3, 3, 1, 1), (2, 2, 9, 8, 3, 2, 2, 1),
         (1, 1, 5, 5, 5, 5, 1, 1), (1, 2, 4, 6, 1, 1, 1, 1), (1, 1, 10, 12, 2, 2, 3, 3)]


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("N,C,HP,WP,wh,ww,sh,sw", CASES)
def test_pool_fwd_bwd_vs_torch(oracle, mode, N, C, HP, WP, wh, ww, sh, sw):
    rng = np.random.default_rng(5 + HP * WP)
    x = rng.uniform(-1, 1, size=(N, C, HP, WP)).astype(np.float32)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    ty = (F.max_pool2d if mode else F.avg_pool2d)(tx, (wh, ww), (sh, sw))
    dy = rng.standard_normal(tuple(ty.shape)).astype(np.float32)
    ty.backward(torch.tensor(dy, dtype=torch.float64))
    y = np.full(tuple(ty.shape), np.nan, np.float32)
    oracle.pool_slab_fwd(mode, x, wh, ww, sh, sw, y)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=0, atol=0 if mode else 1e-7)
    dx = np.full_like(x, np.nan)
    oracle.pool_slab_bwd(mode, x, dy, wh, ww, sh, sw, dx)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=0, atol=1e-6)
    # every window hands out exactly its dy
    np.testing.assert_allclose(dx.astype(np.float64).sum(axis=(2, 3)), dy.astype(np.float64).sum(axis=(2, 3)), atol=1e-5)
    # beta = 1 accumulates
    dx2 = dx.copy()
    oracle.pool_slab_bwd(mode, x, dy, wh, ww, sh, sw, dx2, beta=1.0)
    np.testing.assert_allclose(dx2, 2 * dx, rtol=1e-6, atol=1e-6)


def test_pool_closed_forms(oracle):
    rng = np.random.default_rng(6)
    x = rng.uniform(-1, 1, size=(1, 2, 5, 7)).astype(np.float32)
    for mode in (0, 1):
        y = np.empty_like(x)
        oracle.pool_slab_fwd(mode, x, 1, 1, 1, 1, y)
        assert np.array_equal(y, x)
    # average backward of ones: (number of windows over the pixel) / area
    HP, WP, w, s = 7, 9, 3, 2
    OH, OW = (HP - w) // s + 1, (WP - w) // s + 1
    cnt = np.zeros((HP, WP))
    for oh in range(OH):
        for ow in range(OW):
            cnt[oh * s:oh * s + w, ow * s:ow * s + w] += 1
    dx = np.empty((1, 1, HP, WP), np.float32)
    oracle.pool_slab_bwd(0, np.zeros((1, 1, HP, WP), np.float32), np.ones((1, 1, OH, OW), np.float32), w, w, s, s, dx)
    np.testing.assert_allclose(dx[0, 0], cnt / 9.0, rtol=1e-6)


def test_pool_max_ties_first_in_window_order(oracle):
    # constant input: every element of every window is a maximum
    HP, WP, w, s = 6, 8, 3, 2
    OH, OW = (HP - w) // s + 1, (WP - w) // s + 1
    x = np.full((1, 1, HP, WP), 0.5, np.float32)
    dy = np.arange(1, OH * OW + 1, dtype=np.float32).reshape(1, 1, OH, OW)
    dx = np.empty_like(x)
    oracle.pool_slab_bwd(1, x, dy, w, w, s, s, dx)
    want = np.zeros((HP, WP), np.float32)
    want[0:OH * s:s, 0:OW * s:s] = dy[0, 0]
    assert np.array_equal(dx[0, 0], want)
    tx = torch.tensor(x, requires_grad=True)
    F.max_pool2d(tx, w, s).backward(torch.tensor(dy))
    assert np.array_equal(tx.grad.numpy(), dx)


@pytest.mark.parametrize("mode", [0, 1])
def test_pool_split_equals_unsplit(oracle, mode):
    # 3x3 stride-2 pooling with pad 1 over an image cut into K row-tiles with halo 1
    rng = np.random.default_rng(8)
    K, N, C, H, W = 3, 2, 3, 4, 10
    xu = rng.uniform(0, 1, size=(N, C, K * H, W)).astype(np.float32)
    tiles = [np.empty((N, C, H + 2, W + 2), np.float32) for _ in range(K)]
    assert oracle.tiles_pack(K, 1, W, K * H, C, N, xu, tiles) == 0
    want = (F.max_pool2d if mode else F.avg_pool2d)(F.pad(torch.tensor(xu), (1, 1, 1, 1)), 3, 2).numpy()
    OH, OW = (H + 2 - 3) // 2 + 1, (W + 2 - 3) // 2 + 1
    got = []
    for t in tiles:
        y = np.empty((N, C, OH, OW), np.float32)
        oracle.pool_slab_fwd(mode, t, 3, 3, 2, 2, y)
        got.append(y)
    got = np.concatenate(got, axis=2)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=0, atol=0 if mode else 2e-7)  # torch averages in fp32
