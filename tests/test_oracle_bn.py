"""Pins the batch-norm / rectifier / residual-sum part of the CPU oracle.

The arithmetic of the reference lives in cuDNN (closed source, absent); the oracle restates the
published definition of spatial batch normalisation.  Pinned here against
  * torch.nn.functional.batch_norm (training with momentum 1 = cuDNN's factor 1, and evaluation),
    relu, constant padding and autograd on the CPU in float64;
  * closed forms: the normalised output of every channel has mean 0 and variance 1 / (1 + eps/var),
    the input gradient of every channel sums to zero and is orthogonal to x, the shift gradient is
    the sum of dy.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

CASES = [(3, 4, 5, 6, 0, 0), (2, 3, 4, 7, 1, 0), (2, 5, 6, 5, 1, 1), (1, 2, 9, 4, 0, 3), (4, 1, 3, 3, 1, 2)]


@pytest.mark.parametrize("N,C,H,W,relu,p", CASES)
def test_batchnorm_train_fwd_bwd_vs_torch(oracle, N, C, H, W, relu, p):
    rng = np.random.default_rng(60 + H)
    eps = 1e-5
    x = (rng.standard_normal((N, C, H, W)) * 2 + 3).astype(np.float32)
    scale = rng.uniform(0.5, 1.5, C).astype(np.float32)
    shift = rng.uniform(-0.5, 0.5, C).astype(np.float32)
    dy = rng.standard_normal((N, C, H + 2 * p, W + 2 * p)).astype(np.float32)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    ts = torch.tensor(scale, dtype=torch.float64, requires_grad=True)
    tb = torch.tensor(shift, dtype=torch.float64, requires_grad=True)
    rm, rv = torch.zeros(C, dtype=torch.float64), torch.ones(C, dtype=torch.float64)
    ty = F.batch_norm(tx, rm, rv, ts, tb, training=True, momentum=1.0, eps=eps)
    if relu:
        ty = F.relu(ty)
    ty = F.pad(ty, (p, p, p, p))
    ty.backward(torch.tensor(dy, dtype=torch.float64))
    y = np.full((N, C, H + 2 * p, W + 2 * p), np.nan, np.float32)
    run_mean, run_var, save_mean, save_invstd = (np.full(C, np.nan, np.float32) for _ in range(4))
    oracle.batchnorm2d_fwd_train(x, scale, shift, eps, relu, p, y, run_mean, run_var, save_mean, save_invstd)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=0, atol=2e-6)
    np.testing.assert_allclose(run_mean, rm.numpy(), rtol=1e-6)
    np.testing.assert_allclose(run_var, rv.numpy(), rtol=1e-6)
    np.testing.assert_allclose(save_mean, x.astype(np.float64).mean(axis=(0, 2, 3)), rtol=1e-6)
    np.testing.assert_allclose(save_invstd, 1 / np.sqrt(x.astype(np.float64).var(axis=(0, 2, 3)) + eps), rtol=1e-6)
    dx = np.full_like(x, np.nan)
    dscale, dshift = np.full(C, np.nan, np.float32), np.full(C, np.nan, np.float32)
    oracle.batchnorm2d_bwd(x, dy, scale, shift, save_mean, save_invstd, relu, p, dx, dscale, dshift)
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=0, atol=5e-6)
    np.testing.assert_allclose(dscale, ts.grad.numpy(), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(dshift, tb.grad.numpy(), rtol=1e-5, atol=1e-5)
    # closed forms
    if not relu:
        inner = y[:, :, p:p + H, p:p + W].astype(np.float64)
        xhat = (inner - shift[None, :, None, None]) / scale[None, :, None, None]
        np.testing.assert_allclose(xhat.mean(axis=(0, 2, 3)), 0, atol=1e-6)
        var = x.astype(np.float64).var(axis=(0, 2, 3))
        np.testing.assert_allclose(xhat.var(axis=(0, 2, 3)), var / (var + eps), rtol=1e-5)
    np.testing.assert_allclose(dx.astype(np.float64).sum(axis=(0, 2, 3)), 0, atol=1e-4)
    xc = x.astype(np.float64) - x.astype(np.float64).mean(axis=(0, 2, 3), keepdims=True)
    np.testing.assert_allclose((dx * xc).sum(axis=(0, 2, 3)), 0, atol=2e-3)
    # beta = 1 accumulates data and parameter gradients
    dx2, ds2, db2 = dx.copy(), dscale.copy(), dshift.copy()
    oracle.batchnorm2d_bwd(x, dy, scale, shift, save_mean, save_invstd, relu, p, dx2, ds2, db2, beta_data=1.0, beta_param=1.0)
    np.testing.assert_allclose(dx2, 2 * dx, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(ds2, 2 * dscale, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(db2, 2 * dshift, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("relu,p", [(0, 0), (1, 1)])
def test_batchnorm_inference_vs_torch(oracle, relu, p):
    rng = np.random.default_rng(61)
    N, C, H, W, eps = 2, 3, 4, 5, 1e-5
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    scale, shift = rng.uniform(0.5, 1.5, C).astype(np.float32), rng.uniform(-1, 1, C).astype(np.float32)
    mean, var = rng.standard_normal(C).astype(np.float32), rng.uniform(0.5, 2, C).astype(np.float32)
    want = F.batch_norm(torch.tensor(x, dtype=torch.float64), torch.tensor(mean, dtype=torch.float64),
                        torch.tensor(var, dtype=torch.float64), torch.tensor(scale, dtype=torch.float64),
                        torch.tensor(shift, dtype=torch.float64), training=False, eps=eps)
    if relu:
        want = F.relu(want)
    want = F.pad(want, (p, p, p, p)).numpy()
    y = np.full((N, C, H + 2 * p, W + 2 * p), np.nan, np.float32)
    oracle.batchnorm2d_fwd_infer(x, scale, shift, mean, var, eps, relu, p, y)
    np.testing.assert_allclose(y, want, rtol=0, atol=1e-6)


def test_relu_and_sum(oracle):
    rng = np.random.default_rng(62)
    x = rng.standard_normal(1000).astype(np.float32)
    y = np.empty_like(x)
    oracle.relu_fwd(x, y)
    assert np.array_equal(y, np.maximum(x, 0))
    dy = rng.standard_normal(1000).astype(np.float32)
    dx0 = rng.standard_normal(1000).astype(np.float32)
    dx = dx0.copy()
    oracle.relu_bwd(y, dy, dx, beta=1.0)
    assert np.array_equal(dx, np.where(x > 0, dy, 0).astype(np.float32) + dx0)
    xs = [rng.standard_normal(1000).astype(np.float32) for _ in range(3)]
    s = np.empty(1000, np.float32)
    oracle.sum_fwd(xs, s)
    assert np.array_equal(s, (xs[0] + xs[1]) + xs[2])
