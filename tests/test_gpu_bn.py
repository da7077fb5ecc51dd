"""GPU parity of the shard-local ops (batch norm with tile-local statistics, rectifier, residual
sum) against the CPU oracle, through the C ABI.  fp32: rel-err max|a-b| / max|b| <= 1e-5; bf16
tensors (fp32 arithmetic, one rounding): <= 2^-8.  Rectifier and sum are bit-exact.  Elements whose
pre-activation is within 1e-4 of zero are left out of the fused-rectifier gradient comparison: there
the fp32 mask and the oracle's float64 mask may disagree."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5

CASES = [(1, 3, 4, 5, 6, 0, 0), (2, 2, 3, 4, 7, 1, 0), (3, 2, 5, 6, 5, 1, 1), (1, 1, 2, 9, 4, 0, 3), (4, 8, 64, 14, 56, 1, 1),
         (1, 40, 3, 20, 33, 1, 1), (2, 1, 1, 1, 1, 0, 0), (1, 2, 70, 7, 7, 0, 0)]


def vecs(rng, K, C, lo, hi):
    return [rng.uniform(lo, hi, C).astype(np.float32) for _ in range(K)]


@pytest.mark.parametrize("K,N,C,H,W,relu,p", CASES)
def test_batchnorm_f32_vs_oracle(oracle, K, N, C, H, W, relu, p):
    rng = np.random.default_rng(70 + W)
    eps = 1e-5
    xs = [(rng.standard_normal((N, C, H, W)) * 2 + 3).astype(np.float32) for _ in range(K)]
    scales, shifts = vecs(rng, K, C, 0.5, 1.5), vecs(rng, K, C, -0.5, 0.5)
    dys = [rng.standard_normal((N, C, H + 2 * p, W + 2 * p)).astype(np.float32) for _ in range(K)]
    dx0 = [rng.standard_normal((N, C, H, W)).astype(np.float32) for _ in range(K)]
    dp0 = vecs(rng, K, C, -1, 1)
    ws = torch.empty(capi.batchnorm_workspace_bytes(K, N, C) // 4, device="cuda")
    d_xs, d_sc, d_sh, d_dys = ([dev(a) for a in l] for l in (xs, scales, shifts, dys))
    ys = [torch.full((N, C, H + 2 * p, W + 2 * p), float("nan"), device="cuda") for _ in range(K)]
    stats = [[torch.full((C,), float("nan"), device="cuda") for _ in range(K)] for _ in range(4)]
    capi.check(capi.batchnorm_fwd_tiles(d_xs, d_sc, d_sh, ys, N, C, H, W, eps=eps, relu=relu, out_halo=p, run_means=stats[0],
                                        run_vars=stats[1], save_means=stats[2], save_invstds=stats[3], ws=ws))
    dxs = [torch.full((N, C, H, W), float("nan"), device="cuda") for _ in range(K)]
    dsc = [torch.full((C,), float("nan"), device="cuda") for _ in range(K)]
    dsh = [torch.full((C,), float("nan"), device="cuda") for _ in range(K)]
    capi.check(capi.batchnorm_bwd_tiles(d_xs, d_dys, d_sc, d_sh, stats[2], stats[3], dxs, dsc, dsh, N, C, H, W, relu=relu,
                                        dy_halo=p, ws=ws))
    acc = [dev(a) for a in dx0]
    asc, ash = [dev(a) for a in dp0], [dev(a) for a in dp0]
    capi.check(capi.batchnorm_bwd_tiles(d_xs, d_dys, d_sc, d_sh, stats[2], stats[3], acc, asc, ash, N, C, H, W, relu=relu,
                                        dy_halo=p, beta_data=1.0, beta_param=1.0, ws=ws))
    for r in range(K):
        y = np.empty((N, C, H + 2 * p, W + 2 * p), np.float32)
        want = [np.empty(C, np.float32) for _ in range(4)]
        oracle.batchnorm2d_fwd_train(xs[r], scales[r], shifts[r], eps, relu, p, y, *want)
        assert rel_err(host(ys[r]), y) <= TOL
        for got, w in zip(stats, want):
            np.testing.assert_allclose(host(got[r]), w, rtol=2e-5, atol=1e-6)
        dx, ds, db = np.empty((N, C, H, W), np.float32), np.empty(C, np.float32), np.empty(C, np.float32)
        oracle.batchnorm2d_bwd(xs[r], dys[r], scales[r], shifts[r], want[2], want[3], relu, p, dx, ds, db)
        keep = np.ones((N, C, H, W), bool)
        if relu:
            pre = (scales[r][None, :, None, None] * (xs[r].astype(np.float64) - want[2][None, :, None, None]) *
                   want[3][None, :, None, None] + shifts[r][None, :, None, None])
            keep = np.abs(pre) > 1e-4
        assert rel_err(np.where(keep, host(dxs[r]), 0), np.where(keep, dx, 0)) <= 2e-5
        np.testing.assert_allclose(host(dsc[r]), ds, rtol=1e-4, atol=1e-4 * max(1.0, np.abs(ds).max()))
        np.testing.assert_allclose(host(dsh[r]), db, rtol=1e-4, atol=1e-4 * max(1.0, np.abs(db).max()))
        assert rel_err(np.where(keep, host(acc[r]), 0), np.where(keep, dx + dx0[r], 0)) <= 2e-5
        np.testing.assert_allclose(host(asc[r]), ds + dp0[r], rtol=1e-4, atol=1e-4 * max(1.0, np.abs(ds).max()))
        np.testing.assert_allclose(host(ash[r]), db + dp0[r], rtol=1e-4, atol=1e-4 * max(1.0, np.abs(db).max()))
    # evaluation mode with fixed statistics
    means, vars_ = vecs(rng, K, C, -1, 1), vecs(rng, K, C, 0.5, 2)
    yi = [torch.full((N, C, H + 2 * p, W + 2 * p), float("nan"), device="cuda") for _ in range(K)]
    capi.check(capi.batchnorm_fwd_tiles(d_xs, d_sc, d_sh, yi, N, C, H, W, eps=eps, relu=relu, out_halo=p, training=False,
                                        fixed_means=[dev(a) for a in means], fixed_vars=[dev(a) for a in vars_], ws=ws))
    for r in range(K):
        y = np.empty((N, C, H + 2 * p, W + 2 * p), np.float32)
        oracle.batchnorm2d_fwd_infer(xs[r], scales[r], shifts[r], means[r], vars_[r], eps, relu, p, y)
        assert rel_err(host(yi[r]), y) <= TOL


def test_batchnorm_bf16_vs_oracle(oracle):
    rng = np.random.default_rng(71)
    K, N, C, H, W, relu, p, eps = 2, 4, 16, 10, 24, 1, 1, 1e-5
    bf = lambda a: oracle.f32_to_bf16(a.astype(np.float32))
    xs = [bf(rng.standard_normal((N, C, H, W)) + 0.5) for _ in range(K)]
    scales, shifts = vecs(rng, K, C, 0.5, 1.5), vecs(rng, K, C, -0.5, 0.5)
    dys = [bf(rng.standard_normal((N, C, H + 2, W + 2))) for _ in range(K)]
    ws = torch.empty(capi.batchnorm_workspace_bytes(K, N, C) // 4, device="cuda")
    d_xs, d_sc, d_sh, d_dys = ([dev(a) for a in l] for l in (xs, scales, shifts, dys))
    ys = [torch.empty((N, C, H + 2, W + 2), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    sm = [torch.empty(C, device="cuda") for _ in range(K)]
    si = [torch.empty(C, device="cuda") for _ in range(K)]
    capi.check(capi.batchnorm_fwd_tiles(d_xs, d_sc, d_sh, ys, N, C, H, W, eps=eps, relu=relu, out_halo=p, save_means=sm,
                                        save_invstds=si, ws=ws))
    dxs = [torch.empty((N, C, H, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    dsc, dsh = [torch.empty(C, device="cuda") for _ in range(K)], [torch.empty(C, device="cuda") for _ in range(K)]
    capi.check(capi.batchnorm_bwd_tiles(d_xs, d_dys, d_sc, d_sh, sm, si, dxs, dsc, dsh, N, C, H, W, relu=relu, dy_halo=p, ws=ws))
    for r in range(K):
        xf, dyf = oracle.bf16_to_f32(xs[r]), oracle.bf16_to_f32(dys[r])
        y = np.empty((N, C, H + 2, W + 2), np.float32)
        m, i = np.empty(C, np.float32), np.empty(C, np.float32)
        oracle.batchnorm2d_fwd_train(xf, scales[r], shifts[r], eps, relu, p, y, None, None, m, i)
        assert rel_err(oracle.bf16_to_f32(host(ys[r])), y) <= 2.0 ** -8
        dx, ds, db = np.empty((N, C, H, W), np.float32), np.empty(C, np.float32), np.empty(C, np.float32)
        oracle.batchnorm2d_bwd(xf, dyf, scales[r], shifts[r], m, i, relu, p, dx, ds, db)
        pre = scales[r][None, :, None, None] * (xf - m[None, :, None, None]) * i[None, :, None, None] + shifts[r][None, :, None, None]
        keep = np.abs(pre) > 1e-4
        assert rel_err(np.where(keep, oracle.bf16_to_f32(host(dxs[r])), 0), np.where(keep, dx, 0)) <= 2.0 ** -7
        np.testing.assert_allclose(host(dsc[r]), ds, rtol=1e-3, atol=1e-3)


def test_batchnorm_large_offset_statistics(oracle):
    # mean 1000 times the standard deviation: the shifted sums keep the variance
    rng = np.random.default_rng(72)
    N, C, H, W = 8, 4, 16, 16
    x = (rng.standard_normal((N, C, H, W)) * 0.1 + 100.0).astype(np.float32)
    scale, shift = np.ones(C, np.float32), np.zeros(C, np.float32)
    ws = torch.empty(capi.batchnorm_workspace_bytes(1, N, C) // 4, device="cuda")
    y = torch.empty((N, C, H, W), device="cuda")
    rv = torch.empty(C, device="cuda")
    capi.check(capi.batchnorm_fwd_tiles([dev(x)], [dev(scale)], [dev(shift)], [y], N, C, H, W, run_vars=[rv], ws=ws))
    want = np.empty_like(x)
    wv = np.empty(C, np.float32)
    oracle.batchnorm2d_fwd_train(x, scale, shift, 1e-5, 0, 0, want, None, wv, None, None)
    np.testing.assert_allclose(host(rv), wv, rtol=1e-4)
    assert rel_err(host(y), want) <= 2e-5


def test_relu_and_sum_bit_exact(oracle):
    rng = np.random.default_rng(73)
    n = 100003
    x = rng.standard_normal(n).astype(np.float32)
    dy = rng.standard_normal(n).astype(np.float32)
    dx0 = rng.standard_normal(n).astype(np.float32)
    y = torch.empty(n, device="cuda")
    capi.check(capi.relu_fwd(dev(x), y))
    assert np.array_equal(host(y), np.maximum(x, 0))
    g = dev(dx0)
    capi.check(capi.relu_bwd(y, dev(dy), g, beta=1.0))
    want = dx0.copy()
    oracle.relu_bwd(np.maximum(x, 0), dy, want, beta=1.0)
    assert np.array_equal(host(g), want)
    inplace = dev(x)
    capi.check(capi.relu_fwd(inplace, inplace))
    assert np.array_equal(host(inplace), np.maximum(x, 0))
    xs = [rng.standard_normal(n).astype(np.float32) for _ in range(3)]
    s = torch.empty(n, device="cuda")
    capi.check(capi.sum_fwd([dev(a) for a in xs], s))
    assert np.array_equal(host(s), (xs[0] + xs[1]) + xs[2])
    xb = oracle.f32_to_bf16(x)
    yb = torch.empty(n, device="cuda", dtype=torch.bfloat16)
    capi.check(capi.relu_fwd(dev(xb), yb))
    assert np.array_equal(oracle.bf16_to_f32(host(yb)), np.maximum(oracle.bf16_to_f32(xb), 0))


def test_bn_error_codes():
    x = torch.zeros((1, 2, 3, 3), device="cuda")
    v = torch.ones(2, device="cuda")
    ws = torch.empty(capi.batchnorm_workspace_bytes(1, 1, 2) // 4, device="cuda")
    assert capi.batchnorm_fwd_tiles([x], [v], [v], [x.clone()], 1, 2, 3, 3, ws=ws) == capi.ADH_OK
    assert capi.batchnorm_fwd_tiles([x], [v], [v], [x.clone()], 1, 2, 3, 3) == capi.ADH_ENULL
    assert capi.batchnorm_fwd_tiles([x], [v], [v], [x.clone()], 1, 2, 3, 3, ws=torch.empty(2, device="cuda")) == capi.ADH_EWORKSPACE
    assert capi.batchnorm_fwd_tiles([x], [v], [v], [x.clone()], 1, 2, 3, 3, training=False, ws=ws) == capi.ADH_ENULL
    assert capi.batchnorm_bwd_tiles([x], [x], [v], [v], [v], [v], [x.clone()], [v.clone()], [v.clone()], 1, 2, 3, 3,
                                    beta_data=0.5, ws=ws) == capi.ADH_EINVAL
    assert capi.lib().adh_relu_fwd(capi.ADH_F32, 4, None, x.data_ptr(), None) == capi.ADH_ENULL
    assert capi.lib().adh_sum_fwd(capi.ADH_F32, 0, 4, None, x.data_ptr(), None) == capi.ADH_EINVAL
    torch.cuda.synchronize()
