"""Pins the convolution and softmax halves of the CPU oracle.

The conv arithmetic of the reference lives in cuDNN (closed source, absent), so the
oracle restates the published definition.  It is pinned here against
  * torch.nn.functional.conv2d and torch autograd on the CPU (library routine);
  * closed forms: delta kernel = identity, all-ones kernel = box sum, one hot pixel in
    dy reads the filter back in bwd-data;
  * the split/unsplit identity the whole path exists for: stitched K-tile conv over
    packed tiles == unsplit conv with zero padding.
Softmax/NLL are pinned against scipy.special.log_softmax and closed forms.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F
from scipy.special import log_softmax


def rnd(rng, *shape):
    return rng.uniform(-1, 1, size=shape).astype(np.float32)


@pytest.mark.parametrize("N,Cin,Cout,H,W,k", [(2, 3, 4, 5, 6, 3), (1, 5, 2, 4, 4, 3), (2, 2, 3, 6, 5, 5), (1, 1, 1, 3, 3, 1)])
def test_conv_fwd_bwd_vs_torch(oracle, N, Cin, Cout, H, W, k):
    rng = np.random.default_rng(10)
    xp = rnd(rng, N, Cin, H + k - 1, W + k - 1)
    wt = rnd(rng, Cout, Cin, k, k)
    dy = rng.standard_normal((N, Cout, H, W)).astype(np.float32)
    tx = torch.tensor(xp, dtype=torch.float64, requires_grad=True)
    tw = torch.tensor(wt, dtype=torch.float64, requires_grad=True)
    ty = F.conv2d(tx, tw)  # pad 0 over the padded slab, cross-correlation
    ty.backward(torch.tensor(dy, dtype=torch.float64))
    y = np.empty((N, Cout, H, W), np.float32)
    oracle.conv_slab_fwd(xp, wt, y)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=0, atol=2e-6)
    dx = np.full_like(xp, np.nan)
    oracle.conv_slab_bwd_data(wt, dy, dx)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=0, atol=4e-6)
    dw = np.full_like(wt, np.nan)
    oracle.conv_slab_bwd_filter(xp, dy, dw)
    np.testing.assert_allclose(dw, tw.grad.numpy(), rtol=1e-6, atol=1e-5)
    # beta = 1 accumulates
    y2 = y.copy()
    oracle.conv_slab_fwd(xp, wt, y2, beta=1.0)
    np.testing.assert_allclose(y2, 2 * y, rtol=1e-6, atol=1e-6)
    dw2 = dw.copy()
    oracle.conv_slab_bwd_filter(xp, dy, dw2, beta=1.0)
    np.testing.assert_allclose(dw2, 2 * dw, rtol=1e-6, atol=1e-6)
    dx2 = dx.copy()
    oracle.conv_slab_bwd_data(wt, dy, dx2, beta=1.0)
    np.testing.assert_allclose(dx2, 2 * dx, rtol=1e-6, atol=1e-6)
    yf = np.empty_like(y)
    oracle.conv_slab_fwd_f32(xp, wt, yf)
    np.testing.assert_allclose(yf, y, rtol=0, atol=1e-5)


def test_conv_closed_forms(oracle):
    rng = np.random.default_rng(11)
    N, C, H, W = 1, 3, 4, 5
    xp = rnd(rng, N, C, H + 2, W + 2)
    # delta kernel: y == interior of x (channel-wise identity)
    wt = np.zeros((C, C, 3, 3), np.float32)
    for c in range(C):
        wt[c, c, 1, 1] = 1
    y = np.empty((N, C, H, W), np.float32)
    oracle.conv_slab_fwd(xp, wt, y)
    np.testing.assert_array_equal(y, xp[:, :, 1:-1, 1:-1])
    # an off-centre delta shifts: tap (kh,kw)=(0,2) reads x[h+0, w+2]  (no filter flip)
    wt[:] = 0
    wt[0, 1, 0, 2] = 1
    oracle.conv_slab_fwd(xp, wt, y)
    np.testing.assert_array_equal(y[:, 0], xp[:, 1, 0:H, 2:2 + W])
    assert np.all(y[:, 1:] == 0)
    # all-ones kernel on integer data: box sum over channels, exact
    xi = rng.integers(-4, 5, size=xp.shape).astype(np.float32)
    wt[:] = 1
    oracle.conv_slab_fwd(xi, wt, y)
    box = sum(xi[:, :, a:a + H, b:b + W] for a in range(3) for b in range(3)).sum(axis=1)
    np.testing.assert_array_equal(y[:, 0], box)
    # one hot pixel in dy: bwd-data lays the filter down un-flipped at that position
    w2 = rnd(rng, 2, C, 3, 3)
    dy = np.zeros((N, 2, H, W), np.float32)
    dy[0, 1, 2, 3] = 1
    dx = np.empty_like(xp)
    oracle.conv_slab_bwd_data(w2, dy, dx)
    want = np.zeros_like(xp)
    want[0, :, 2:5, 3:6] = w2[1]
    np.testing.assert_array_equal(dx, want)
    # one hot pixel in dy: bwd-filter reads the 3x3 input patch under it
    dw = np.empty_like(w2)
    oracle.conv_slab_bwd_filter(xp, dy, dw)
    np.testing.assert_array_equal(dw[1], xp[0, :, 2:5, 3:6])
    assert np.all(dw[0] == 0)


def test_split_conv_equals_unsplit(oracle):
    """The claim of the whole path: pack -> per-tile slab conv -> gather == unsplit conv;
    per-tile bwd-data -> halo reduce -> unpad -> gather == unsplit bwd-data; sum of per-tile
    bwd-filter == unsplit bwd-filter."""
    rng = np.random.default_rng(12)
    K, p, N, C, Co, H, W = 4, 1, 2, 3, 4, 8, 5
    Ht = H // K
    X = rnd(rng, N, C, H, W)
    wt = rnd(rng, Co, C, 3, 3)
    dY = rng.standard_normal((N, Co, H, W)).astype(np.float32)
    tX = torch.tensor(X, dtype=torch.float64, requires_grad=True)
    tw = torch.tensor(wt, dtype=torch.float64, requires_grad=True)
    tY = F.conv2d(tX, tw, padding=1)
    tY.backward(torch.tensor(dY, dtype=torch.float64))

    tiles = [np.empty((N, C, Ht + 2, W + 2), np.float32) for _ in range(K)]
    oracle.tiles_pack(K, p, W, H, C, N, X, tiles)
    Y = np.empty((N, Co, H, W), np.float32)
    dW = np.zeros_like(wt)
    gt = []
    for r in range(K):
        y = np.empty((N, Co, Ht, W), np.float32)
        oracle.conv_slab_fwd(tiles[r], wt, y)
        Y[:, :, r * Ht:(r + 1) * Ht] = y
        dy = np.ascontiguousarray(dY[:, :, r * Ht:(r + 1) * Ht])
        g = np.zeros_like(tiles[r])
        oracle.conv_slab_bwd_data(wt, dy, g, beta=1.0)
        gt.append(g)
        oracle.conv_slab_bwd_filter(tiles[r], dy, dW, beta=1.0)
    np.testing.assert_allclose(Y, tY.detach().numpy(), rtol=0, atol=2e-6)
    oracle.halo_op(oracle.REDUCE, 1, K, p, W, Ht, C, N, gt)
    dX = np.empty_like(X)
    oracle.tiles_unpack(K, p, W, H, C, N, gt, dX)
    np.testing.assert_allclose(dX, tX.grad.numpy(), rtol=0, atol=4e-6)
    np.testing.assert_allclose(dW, tw.grad.numpy(), rtol=1e-6, atol=1e-5)


def test_softmax_vs_scipy_and_closed_forms(oracle):
    rng = np.random.default_rng(13)
    N, C = 16, 1000
    x = (2.0 * rng.standard_normal((N, C))).astype(np.float32)
    y = np.empty_like(x)
    oracle.softmax_fwd(x, y)
    want = np.exp(log_softmax(x.astype(np.float64), axis=1))
    np.testing.assert_allclose(y, want, rtol=2e-7, atol=0)
    np.testing.assert_allclose(y.astype(np.float64).sum(axis=1), 1.0, atol=1e-6)
    # shift invariance, including a shift that would overflow a naive exp
    y2 = np.empty_like(x)
    oracle.softmax_fwd((x + np.float32(64.0)), y2)
    np.testing.assert_allclose(y2, y, rtol=2e-5)
    big = np.full((1, 8), 1000.0, np.float32)
    yb = np.empty_like(big)
    oracle.softmax_fwd(big, yb)
    np.testing.assert_array_equal(yb, np.full((1, 8), 0.125, np.float32))
    # nll: -log y[label]
    label = rng.integers(0, C, size=N).astype(np.uint32)
    loss = np.empty(N, np.float32)
    oracle.softmax_nll_loss_fwd(y, label, loss)
    want_loss = -log_softmax(x.astype(np.float64), axis=1)[np.arange(N), label]
    np.testing.assert_allclose(loss, want_loss, rtol=1e-6)
    # uniform logits: loss = log C
    u = np.zeros((2, C), np.float32)
    yu = np.empty_like(u)
    oracle.softmax_fwd(u, yu)
    lu = np.empty(2, np.float32)
    oracle.softmax_nll_loss_fwd(yu, np.array([3, 999], np.uint32), lu)
    np.testing.assert_allclose(lu, np.log(C), rtol=1e-6)
    # bwd: dx += dloss * (y - onehot); rows of a zero-initialised dx sum to ~0
    dloss = np.full(N, 1.0 / N, np.float32)
    dx = np.zeros_like(x)
    oracle.softmax_nll_loss_bwd(y, label, dloss, dx)
    onehot = np.zeros_like(x)
    onehot[np.arange(N), label] = 1
    np.testing.assert_allclose(dx, (y - onehot) / N, rtol=1e-6, atol=1e-9)
    assert np.all(np.abs(dx.astype(np.float64).sum(axis=1)) < 1e-7)
    dx3 = dx.copy()
    oracle.softmax_nll_loss_bwd(y, label, dloss, dx3)  # accumulates
    np.testing.assert_allclose(dx3, 2 * dx, rtol=1e-6)
    # autograd cross-check of the composite
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tl = F.cross_entropy(tx, torch.tensor(label.astype(np.int64)), reduction="mean")
    tl.backward()
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-5, atol=1e-9)


GENERAL = [  # N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw
    (2, 3, 4, 13, 15, 7, 7, 2, 2, 1, 1), (1, 4, 3, 9, 10, 3, 3, 2, 2, 1, 1), (1, 2, 2, 11, 12, 3, 3, 1, 1, 3, 3),
    (2, 5, 3, 6, 7, 1, 1, 2, 2, 1, 1), (1, 2, 3, 10, 9, 3, 2, 2, 1, 2, 1), (1, 1, 1, 8, 8, 2, 2, 3, 3, 1, 1),
    (1, 3, 2, 7, 9, 3, 3, 1, 1, 1, 1)]


@pytest.mark.parametrize("N,Cin,Cout,HP,WP,kh,kw,sh,sw,dh,dw", GENERAL)
def test_general_conv_vs_torch(oracle, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw):
    rng = np.random.default_rng(20 + HP)
    xp = rnd(rng, N, Cin, HP, WP)
    wt = rnd(rng, Cout, Cin, kh, kw)
    tx = torch.tensor(xp, dtype=torch.float64, requires_grad=True)
    tw = torch.tensor(wt, dtype=torch.float64, requires_grad=True)
    ty = F.conv2d(tx, tw, stride=(sh, sw), dilation=(dh, dw))
    assert tuple(ty.shape[2:]) == oracle.conv2d_out_dims(HP, WP, kh, kw, sh, sw, dh, dw)
    dy = rng.standard_normal(tuple(ty.shape)).astype(np.float32)
    ty.backward(torch.tensor(dy, dtype=torch.float64))
    y = np.full(tuple(ty.shape), np.nan, np.float32)
    oracle.conv2d_slab_fwd(xp, wt, sh, sw, dh, dw, y)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=0, atol=4e-6)
    dx = np.full_like(xp, np.nan)
    oracle.conv2d_slab_bwd_data(wt, dy, sh, sw, dh, dw, dx)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=0, atol=8e-6)
    dwt = np.full_like(wt, np.nan)
    oracle.conv2d_slab_bwd_filter(xp, dy, sh, sw, dh, dw, dwt)
    np.testing.assert_allclose(dwt, tw.grad.numpy(), rtol=1e-6, atol=2e-5)
    # beta = 1 accumulates
    for fn, out, args in ((oracle.conv2d_slab_fwd, y, (xp, wt)), (oracle.conv2d_slab_bwd_data, dx, (wt, dy)),
                          (oracle.conv2d_slab_bwd_filter, dwt, (xp, dy))):
        twice = out.copy()
        fn(*args, sh, sw, dh, dw, twice, beta=1.0)
        np.testing.assert_allclose(twice, 2 * out, rtol=1e-6, atol=1e-6)
    if (kh, kw, sh, sw, dh, dw) == (3, 3, 1, 1, 1, 1):  # the 3x3 stride-1 functions are the same map
        y3 = np.empty_like(y)
        oracle.conv_slab_fwd(xp, wt, y3)
        assert np.array_equal(y3, y)
        dx3 = np.empty_like(dx)
        oracle.conv_slab_bwd_data(wt, dy, dx3)
        np.testing.assert_allclose(dx3, dx, rtol=0, atol=1e-6)


@pytest.mark.parametrize("N,Cin,Cout,H,W,k", [(2, 3, 4, 5, 6, 3), (3, 2, 5, 4, 7, 1), (1, 3, 64, 6, 6, 7)])
def test_conv_bias_vs_torch(oracle, N, Cin, Cout, H, W, k):
    """cudnnAddTensor(bias) after the conv and cudnnConvolutionBackwardBias (src/op.cc:1602-1610,
    1632-1648) against torch's conv2d with a bias and its autograd, and against numpy's
    broadcasting / axis sums (neither reuses the oracle's loops)."""
    rng = np.random.default_rng(12)
    xp = rnd(rng, N, Cin, H + k - 1, W + k - 1)
    wt = rnd(rng, Cout, Cin, k, k)
    b = rnd(rng, Cout)
    dy = rng.standard_normal((N, Cout, H, W)).astype(np.float32)
    tb = torch.tensor(b, dtype=torch.float64, requires_grad=True)
    ty = F.conv2d(torch.tensor(xp, dtype=torch.float64), torch.tensor(wt, dtype=torch.float64), bias=tb)
    ty.backward(torch.tensor(dy, dtype=torch.float64))
    y = np.empty((N, Cout, H, W), np.float32)
    oracle.conv_slab_fwd(xp, wt, y)
    y0 = y.copy()
    oracle.conv_bias_add(b, y)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=0, atol=3e-6)
    assert np.array_equal(y, y0 + b[None, :, None, None])  # one rounding per element
    db = np.full(Cout, np.nan, np.float32)
    oracle.conv_bwd_bias(dy, db)
    np.testing.assert_allclose(db, tb.grad.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(db, dy.astype(np.float64).sum(axis=(0, 2, 3)), rtol=1e-6, atol=1e-6)
    db2 = db.copy()
    oracle.conv_bwd_bias(dy, db2, beta=1.0)
    np.testing.assert_allclose(db2, 2 * db, rtol=1e-6, atol=1e-6)
    # a transposed (c, n) index or a dropped plane would change these closed forms
    ones = np.ones((N, Cout, H, W), np.float32)
    oracle.conv_bwd_bias(ones, db)
    assert np.array_equal(db, np.full(Cout, N * H * W, np.float32))
    hot = np.zeros((N, Cout, H, W), np.float32)
    hot[N - 1, 1, H - 1, W - 1] = 3.0
    oracle.conv_bwd_bias(hot, db)
    want = np.zeros(Cout, np.float32)
    want[1] = 3.0
    assert np.array_equal(db, want)
