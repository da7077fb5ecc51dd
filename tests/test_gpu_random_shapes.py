"""Seeded sweeps over small random shapes: general slab conv (forward, backward-data, backward-filter),
pooling (max / average, forward, backward) and batch norm against the CPU oracle through the C ABI.
They exist to hit tilings the hand-picked cases miss (block edges, residue classes with no taps,
bands, channel counts off every step).  Tolerances as in the per-kernel tests."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu


def _conv_cases(seed, count, max_n=3, max_cin=20, max_cout=40):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        sh, sw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        dh, dw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        eh, ew = (kh - 1) * dh + 1, (kw - 1) * dw + 1
        HP, WP = eh + int(rng.integers(0, 12)), ew + int(rng.integers(0, 40))
        out.append((int(rng.integers(1, 3)), int(rng.integers(1, max_n + 1)), int(rng.integers(1, max_cin + 1)),
                    int(rng.integers(1, max_cout + 1)),
                    HP, WP, kh, kw, sh, sw, dh, dw))
    return out


@pytest.mark.parametrize("K,N,Cin,Cout,HP,WP,kh,kw,sh,sw,dh,dw", _conv_cases(2024, 24))
def test_general_conv_random(oracle, K, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw):
    rng = np.random.default_rng(HP * 131 + WP)
    geo = (kh, kw, sh, sw, dh, dw)
    OH, OW = oracle.conv2d_out_dims(HP, WP, *geo)
    xs = [rng.uniform(-1, 1, size=(N, Cin, HP, WP)).astype(np.float32) for _ in range(K)]
    w = rng.standard_normal((Cout, Cin, kh, kw)).astype(np.float32)
    dys = [rng.standard_normal((N, Cout, OH, OW)).astype(np.float32) for _ in range(K)]
    d_xs, d_dys, d_w = [dev(x) for x in xs], [dev(d) for d in dys], dev(w)
    ws = torch.empty(max(capi.conv2d_workspace_bytes(wh, capi.ADH_F32, K, N, Cin, Cout, HP, WP, *geo) for wh in (0, 1, 2)) // 4,
                     device="cuda")
    ys = [torch.full((N, Cout, OH, OW), float("nan"), device="cuda") for _ in range(K)]
    gs = [torch.full((N, Cin, HP, WP), float("nan"), device="cuda") for _ in range(K)]
    gw = torch.full((Cout, Cin, kh, kw), float("nan"), device="cuda")
    capi.check(capi.conv2d_fwd_tiles(d_xs, d_w, ys, N, Cin, Cout, HP, WP, *geo, ws=ws))
    capi.check(capi.conv2d_bwd_data_tiles(d_w, d_dys, gs, N, Cin, Cout, HP, WP, *geo, ws=ws))
    capi.check(capi.conv2d_bwd_filter_tiles(d_xs, d_dys, gw, N, Cin, Cout, HP, WP, *geo, ws=ws))
    want_w = np.zeros_like(w)
    for r in range(K):
        y = np.empty((N, Cout, OH, OW), np.float32)
        oracle.conv2d_slab_fwd(xs[r], w, sh, sw, dh, dw, y)
        assert rel_err(host(ys[r]), y) <= 1e-5
        g = np.empty((N, Cin, HP, WP), np.float32)
        oracle.conv2d_slab_bwd_data(w, dys[r], sh, sw, dh, dw, g)
        assert rel_err(host(gs[r]), g) <= 1e-5
        oracle.conv2d_slab_bwd_filter(xs[r], dys[r], sh, sw, dh, dw, want_w, beta=1.0)
    assert rel_err(host(gw), want_w) <= 1e-5


def _pool_cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        wh, ww = int(rng.integers(1, 5)), int(rng.integers(1, 5))
        out.append((int(rng.integers(1, 3)), int(rng.integers(1, 4)), int(rng.integers(1, 9)), wh + int(rng.integers(0, 20)),
                    ww + int(rng.integers(0, 150)), wh, ww, int(rng.integers(1, 4)), int(rng.integers(1, 4)), int(rng.integers(0, 2))))
    return out


# more images and channels: several images per block / per backward-filter unit, 16- and 32-channel chunks (some padded)
@pytest.mark.parametrize("K,N,Cin,Cout,HP,WP,kh,kw,sh,sw,dh,dw", _conv_cases(7, 48, max_n=9, max_cin=70, max_cout=70))
def test_general_conv_random_wide(oracle, K, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw):
    test_general_conv_random(oracle, K, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw)


@pytest.mark.parametrize("K,N,C,HP,WP,wh,ww,sh,sw,mode", _pool_cases(2025, 20))
def test_pool_random(oracle, K, N, C, HP, WP, wh, ww, sh, sw, mode):
    rng = np.random.default_rng(HP * 977 + WP)
    OH, OW = (HP - wh) // sh + 1, (WP - ww) // sw + 1
    xs = [rng.uniform(-1, 1, size=(N, C, HP, WP)).astype(np.float32) for _ in range(K)]
    dys = [rng.standard_normal((N, C, OH, OW)).astype(np.float32) for _ in range(K)]
    d_xs, d_dys = [dev(x) for x in xs], [dev(d) for d in dys]
    ys = [torch.full((N, C, OH, OW), float("nan"), device="cuda") for _ in range(K)]
    gs = [torch.full((N, C, HP, WP), float("nan"), device="cuda") for _ in range(K)]
    capi.check(capi.pool_fwd_tiles(mode, d_xs, ys, N, C, HP, WP, wh, ww, sh, sw))
    capi.check(capi.pool_bwd_tiles(mode, d_xs, ys, d_dys, gs, N, C, HP, WP, wh, ww, sh, sw))
    for r in range(K):
        y = np.empty((N, C, OH, OW), np.float32)
        oracle.pool_slab_fwd(mode, xs[r], wh, ww, sh, sw, y)
        assert rel_err(host(ys[r]), y) <= 1e-5
        g = np.empty((N, C, HP, WP), np.float32)
        oracle.pool_slab_bwd(mode, xs[r], dys[r], wh, ww, sh, sw, g)
        assert rel_err(host(gs[r]), g) <= 1e-5


def _bn_cases(seed, count):
    rng = np.random.default_rng(seed)
    return [(int(rng.integers(1, 4)), int(rng.integers(1, 6)), int(rng.integers(1, 12)), int(rng.integers(1, 12)),
             int(rng.integers(1, 40)), int(rng.integers(0, 2)), int(rng.integers(0, 3))) for _ in range(count)]


@pytest.mark.parametrize("K,N,C,H,W,relu,p", _bn_cases(2026, 16))
def test_batchnorm_random(oracle, K, N, C, H, W, relu, p):
    rng = np.random.default_rng(H * 59 + W)
    xs = [(rng.standard_normal((N, C, H, W)) + 1).astype(np.float32) for _ in range(K)]
    sc = [rng.uniform(0.5, 1.5, C).astype(np.float32) for _ in range(K)]
    sh = [rng.uniform(-0.5, 0.5, C).astype(np.float32) for _ in range(K)]
    dys = [rng.standard_normal((N, C, H + 2 * p, W + 2 * p)).astype(np.float32) for _ in range(K)]
    ws = torch.empty(capi.batchnorm_workspace_bytes(K, N, C) // 4, device="cuda")
    d_xs, d_sc, d_sh, d_dys = ([dev(a) for a in l] for l in (xs, sc, sh, dys))
    ys = [torch.full((N, C, H + 2 * p, W + 2 * p), float("nan"), device="cuda") for _ in range(K)]
    sm = [torch.empty(C, device="cuda") for _ in range(K)]
    si = [torch.empty(C, device="cuda") for _ in range(K)]
    capi.check(capi.batchnorm_fwd_tiles(d_xs, d_sc, d_sh, ys, N, C, H, W, relu=relu, out_halo=p, save_means=sm, save_invstds=si,
                                        ws=ws))
    dxs = [torch.full((N, C, H, W), float("nan"), device="cuda") for _ in range(K)]
    dsc, dsh = [torch.empty(C, device="cuda") for _ in range(K)], [torch.empty(C, device="cuda") for _ in range(K)]
    capi.check(capi.batchnorm_bwd_tiles(d_xs, d_dys, d_sc, d_sh, sm, si, dxs, dsc, dsh, N, C, H, W, relu=relu, dy_halo=p, ws=ws))
    for r in range(K):
        y = np.empty((N, C, H + 2 * p, W + 2 * p), np.float32)
        m, i = np.empty(C, np.float32), np.empty(C, np.float32)
        oracle.batchnorm2d_fwd_train(xs[r], sc[r], sh[r], 1e-5, relu, p, y, None, None, m, i)
        # a single value per channel has variance 0 and 1/sqrt(eps) ~ 316: its output is the shift, errors scale with it
        assert rel_err(host(ys[r]), y) <= 2e-5
        dx, ds, db = np.empty((N, C, H, W), np.float32), np.empty(C, np.float32), np.empty(C, np.float32)
        oracle.batchnorm2d_bwd(xs[r], dys[r], sc[r], sh[r], m, i, relu, p, dx, ds, db)
        pre = sc[r][None, :, None, None] * (xs[r].astype(np.float64) - m[None, :, None, None]) * i[None, :, None, None] + \
            sh[r][None, :, None, None]
        keep = (np.abs(pre) > 1e-4) if relu else np.ones_like(pre, bool)
        if N * H * W > 1:
            scale = max(float(np.abs(dx).max()), 1e-3)
            assert np.max(np.abs(np.where(keep, host(dxs[r]) - dx, 0))) <= 5e-5 * max(scale, 1.0) * max(1.0, float(i.max()) / 10)
        np.testing.assert_allclose(host(dsh[r]), db, rtol=1e-4, atol=1e-4 * max(1.0, float(np.abs(db).max())))


def _row_tile_cases(seed, count, max_c):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        out.append((int(rng.integers(1, 6)), int(rng.integers(1, 4)), int(rng.integers(1, max_c + 1)),
                    int(rng.integers(1, max_c + 1)), int(rng.integers(1, 12)), int(rng.integers(1, 90))))
    return out


@pytest.mark.parametrize("K,N,Cin,Cout,Ht,W", _row_tile_cases(2027, 20, 40))
def test_conv_over_row_tiles_without_halo_kernels_random(oracle, K, N, Cin, Cout, Ht, W):
    """Forward over unexchanged tiles, the filter gradient over them and the input gradient with the reduce folded
    in, against the UNSPLIT convolution of the stitched tensors (fp32, rel-err <= 1e-5)."""
    rng = np.random.default_rng(K * 1000 + W)
    H = K * Ht
    x = rng.uniform(-1, 1, size=(N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9))).astype(np.float32)
    dy = rng.standard_normal((N, Cout, H, W)).astype(np.float32)
    xp = np.zeros((N, Cin, H + 2, W + 2), np.float32)
    xp[:, :, 1:-1, 1:-1] = x
    y = np.empty((N, Cout, H, W), np.float32)
    oracle.conv_slab_fwd(xp, w, y)
    gx = np.empty_like(xp)
    oracle.conv_slab_bwd_data(w, dy, gx)
    gw = np.zeros_like(w)
    oracle.conv_slab_bwd_filter(xp, dy, gw)
    # tiles as after HaloPad2DOp: zero halo, nothing exchanged
    xs = []
    for r in range(K):
        t = np.zeros((N, Cin, Ht + 2, W + 2), np.float32)
        t[:, :, 1:-1, 1:-1] = x[:, :, r * Ht:(r + 1) * Ht, :]
        xs.append(dev(t))
    dys = [dev(dy[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    ys = [torch.full((N, Cout, Ht, W), float("nan"), device="cuda") for _ in range(K)]
    gs = [torch.full((N, Cin, Ht + 2, W + 2), float("nan"), device="cuda") for _ in range(K)]
    d_gw = torch.full((Cout, Cin, 3, 3), float("nan"), device="cuda")
    nbytes = capi.conv_workspace_bytes(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, K, N, Cin, Cout, Ht, W)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")
    capi.check(capi.conv_fwd_tiles(xs, dev(w), ys, N, Cin, Cout, Ht, W, unexchanged=True))
    capi.check(capi.conv_bwd_data_tiles(dev(w), dys, gs, N, Cin, Cout, Ht, W, reduced=True))
    capi.check(capi.conv_bwd_filter_tiles(xs, dys, d_gw, N, Cin, Cout, Ht, W, ws=ws, unexchanged=True))
    for r in range(K):
        assert rel_err(host(ys[r]), y[:, :, r * Ht:(r + 1) * Ht, :]) <= 1e-5
        assert rel_err(host(gs[r])[:, :, 1:-1, 1:-1], gx[:, :, 1 + r * Ht:1 + (r + 1) * Ht, 1:-1]) <= 1e-5
    assert rel_err(host(d_gw), gw) <= 1e-5


def _bf16_wide_cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        out.append((int(rng.integers(1, 4)), int(rng.integers(1, 3)), int(rng.integers(1, 200)), int(rng.integers(1, 200)),
                    int(rng.integers(1, 11)), 8 * int(rng.integers(1, 12))))
    return out


# channel counts the 128-channel kernel takes in one launch (both sides above 64), in launches of 128 with fp32 sums
# between them (192 = 128 + 64 by the 64-channel kernel, 256 = 128 + 128, 320 = 128 + 128 + 64, 200 = 128 + 72), with
# output-channel remainders (130, 136, 200), strips off the 32-column step and several row segments
_BF16_WIDE_FIXED = [(2, 1, 128, 128, 9, 72), (1, 2, 192, 136, 6, 40), (2, 1, 256, 256, 5, 64), (1, 1, 320, 130, 4, 24),
                    (3, 1, 200, 200, 3, 8), (1, 1, 128, 256, 23, 104), (2, 2, 256, 128, 12, 32)]


# more than 64 reduction channels at widths the eight-wave kernels do not take (odd; even but no multiple of 8 for
# backward-data): one launch of the four-wave kernel per 64 channels with fp32 sums between them; the last tiles of a
# ResNet (7 x 7 at 512 channels), one column, channel remainders on both sides
_BF16_WIDE_ANY_WIDTH = [(2, 1, 128, 128, 9, 7), (1, 2, 192, 136, 6, 13), (2, 1, 100, 70, 5, 66), (1, 1, 320, 130, 4, 27),
                        (3, 1, 65, 65, 3, 1), (1, 1, 512, 512, 7, 7), (2, 2, 130, 40, 12, 33), (1, 1, 72, 200, 10, 70),
                        (1, 2, 96, 96, 17, 131)]


@pytest.mark.parametrize("K,N,Cin,Cout,H,W", _bf16_wide_cases(2028, 16) + _BF16_WIDE_FIXED + _BF16_WIDE_ANY_WIDTH)
def test_bf16_conv_random_channel_counts(oracle, K, N, Cin, Cout, H, W):
    """bf16 forward and backward-data (beta 0 and 1 each) and filter gradient on the matrix cores for channel counts
    on both sides of 64 and 128 (launches of 64 or 128 reduction channels, 64 x 64 pairs for the filter gradient).
    Tolerances as in test_gpu_conv_bf16.py."""
    rng = np.random.default_rng(Cin * 211 + Cout)
    bf = lambda a: oracle.f32_to_bf16(a.astype(np.float32))
    xs = [bf(rng.uniform(-1, 1, size=(N, Cin, H + 2, W + 2))) for _ in range(K)]
    w = bf(rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9)))
    dys = [bf(rng.standard_normal((N, Cout, H, W))) for _ in range(K)]
    g0 = [bf(rng.standard_normal((N, Cin, H + 2, W + 2))) for _ in range(K)]
    y0 = [bf(rng.standard_normal((N, Cout, H, W))) for _ in range(K)]
    wf = oracle.bf16_to_f32(w)

    def ws_for(which):
        return torch.empty(capi.conv_workspace_bytes(which, capi.ADH_BF16, K, N, Cin, Cout, H, W) // 4 + 64, device="cuda")

    d_xs, d_dys, d_w = [dev(a) for a in xs], [dev(a) for a in dys], dev(w)
    ys = [torch.empty((N, Cout, H, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    gs = [torch.empty((N, Cin, H + 2, W + 2), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    ga = [dev(a) for a in g0]
    ya = [dev(a) for a in y0]
    dw = torch.full((Cout, Cin, 3, 3), float("nan"), device="cuda")
    capi.check(capi.conv_fwd_tiles(d_xs, d_w, ys, N, Cin, Cout, H, W, ws=ws_for(capi.ADH_CONV_FWD)))
    capi.check(capi.conv_fwd_tiles(d_xs, d_w, ya, N, Cin, Cout, H, W, beta=1.0, ws=ws_for(capi.ADH_CONV_FWD)))
    capi.check(capi.conv_bwd_data_tiles(d_w, d_dys, gs, N, Cin, Cout, H, W, ws=ws_for(capi.ADH_CONV_BWD_DATA)))
    capi.check(capi.conv_bwd_data_tiles(d_w, d_dys, ga, N, Cin, Cout, H, W, beta=1.0, ws=ws_for(capi.ADH_CONV_BWD_DATA)))
    capi.check(capi.conv_bwd_filter_tiles(d_xs, d_dys, dw, N, Cin, Cout, H, W, ws=ws_for(capi.ADH_CONV_BWD_FILTER)))
    dw_want = np.zeros((Cout, Cin, 3, 3), np.float32)
    for r in range(K):
        xf, dyf = oracle.bf16_to_f32(xs[r]), oracle.bf16_to_f32(dys[r])
        y = np.empty((N, Cout, H, W), np.float32)
        oracle.conv_slab_fwd(xf, wf, y)
        assert rel_err(oracle.bf16_to_f32(host(ys[r])), y) <= 5e-3
        assert rel_err(oracle.bf16_to_f32(host(ya[r])), y + oracle.bf16_to_f32(y0[r])) <= 5e-3
        g = np.empty((N, Cin, H + 2, W + 2), np.float32)
        oracle.conv_slab_bwd_data(wf, dyf, g)
        assert rel_err(oracle.bf16_to_f32(host(gs[r])), g) <= 5e-3
        assert rel_err(oracle.bf16_to_f32(host(ga[r])), g + oracle.bf16_to_f32(g0[r])) <= 5e-3
        oracle.conv_slab_bwd_filter(xf, dyf, dw_want, beta=1.0)
    assert rel_err(host(dw), dw_want) <= 1e-4


@pytest.mark.parametrize("K,N,Cin,Cout,Ht,W", _bf16_wide_cases(2029, 16) + _BF16_WIDE_FIXED)
def test_bf16_conv_over_tiles_without_halo_random(oracle, K, N, Cin, Cout, Ht, W):
    """adh_conv3x3_unpadded_{fwd,bwd_data,bwd_filter}_tiles against the UNSPLIT convolution with zero padding."""
    rng = np.random.default_rng(Cin * 311 + Cout + K)
    bf = lambda a: oracle.f32_to_bf16(a.astype(np.float32))
    H = K * Ht
    x = bf(rng.uniform(-1, 1, size=(N, Cin, H, W)))
    w = bf(rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9)))
    dy = bf(rng.standard_normal((N, Cout, H, W)))
    xf, wf, dyf = oracle.bf16_to_f32(x), oracle.bf16_to_f32(w), oracle.bf16_to_f32(dy)
    xp = np.zeros((N, Cin, H + 2, W + 2), np.float32)
    xp[:, :, 1:-1, 1:-1] = xf
    y_want = np.empty((N, Cout, H, W), np.float32)
    oracle.conv_slab_fwd(xp, wf, y_want)
    gx_want = np.empty((N, Cin, H + 2, W + 2), np.float32)
    oracle.conv_slab_bwd_data(wf, dyf, gx_want)
    dw_want = np.zeros((Cout, Cin, 3, 3), np.float32)
    oracle.conv_slab_bwd_filter(xp, dyf, dw_want)

    def ws_for(which):
        return torch.empty(capi.conv_workspace_bytes(which, capi.ADH_BF16, K, N, Cin, Cout, Ht, W) // 4 + 64, device="cuda")

    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    ys = [torch.empty((N, Cout, Ht, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    gs = [torch.empty((N, Cin, Ht, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    dw = torch.full((Cout, Cin, 3, 3), float("nan"), device="cuda")
    capi.check(capi.conv_unpadded_fwd_tiles(xs, dev(w), ys, N, Cin, Cout, Ht, W, ws=ws_for(capi.ADH_CONV_FWD)))
    capi.check(capi.conv_unpadded_bwd_data_tiles(dev(w), dys, gs, N, Cin, Cout, Ht, W, ws=ws_for(capi.ADH_CONV_BWD_DATA)))
    capi.check(capi.conv_unpadded_bwd_filter_tiles(xs, dys, dw, N, Cin, Cout, Ht, W, ws=ws_for(capi.ADH_CONV_BWD_FILTER)))
    # accumulating forms: prior contents are added to (beta 1)
    y0 = bf(rng.standard_normal((N, Cout, H, W)))
    g0 = bf(rng.standard_normal((N, Cin, H, W)))
    ya = [dev(y0[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    ga = [dev(g0[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    capi.check(capi.conv_unpadded_fwd_tiles(xs, dev(w), ya, N, Cin, Cout, Ht, W, beta=1.0, ws=ws_for(capi.ADH_CONV_FWD)))
    capi.check(capi.conv_unpadded_bwd_data_tiles(dev(w), dys, ga, N, Cin, Cout, Ht, W, beta=1.0, ws=ws_for(capi.ADH_CONV_BWD_DATA)))
    for r in range(K):
        rows = slice(r * Ht, (r + 1) * Ht)
        assert rel_err(oracle.bf16_to_f32(host(ys[r])), y_want[:, :, rows, :]) <= 5e-3
        assert rel_err(oracle.bf16_to_f32(host(gs[r])), gx_want[:, :, 1 + r * Ht:1 + (r + 1) * Ht, 1:-1]) <= 5e-3
        assert rel_err(oracle.bf16_to_f32(host(ya[r])), y_want[:, :, rows, :] + oracle.bf16_to_f32(y0[:, :, rows, :])) <= 5e-3
        assert rel_err(oracle.bf16_to_f32(host(ga[r])),
                       gx_want[:, :, 1 + r * Ht:1 + (r + 1) * Ht, 1:-1] + oracle.bf16_to_f32(g0[:, :, rows, :])) <= 5e-3
    assert rel_err(host(dw), dw_want) <= 1e-4


def _unpadded_geometries(seed, count, max_k):
    """(K, Ht, W, k_h, k_w, s_h, s_w, d_h, d_w, pad_h, pad_w) whose row split stitches: Ht a multiple of s_h,
    0 < (k_h - 1) d_h + 1 - 2 pad_h <= s_h, a window that reaches the adjacent tiles only."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        kh, kw = int(rng.integers(1, max_k + 1)), int(rng.integers(1, max_k + 1))
        sh, sw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        dh, dw = int(rng.integers(1, 3)), int(rng.integers(1, 3))
        eh, ew = (kh - 1) * dh + 1, (kw - 1) * dw + 1
        pads = [p for p in range(0, eh) if 0 < eh - 2 * p <= sh]
        if not pads:
            continue
        pad_h = int(rng.choice(pads))
        pad_w = int(rng.integers(0, ew))
        Ht = sh * int(rng.integers(1, 6))
        if pad_h > Ht or eh - 1 - pad_h > Ht:
            continue
        W = max(1, ew - 2 * pad_w) + int(rng.integers(0, 30))
        out.append((int(rng.integers(1, 5)), Ht, W, kh, kw, sh, sw, dh, dw, pad_h, pad_w))
    return out


@pytest.mark.parametrize("K,Ht,W,kh,kw,sh,sw,dh,dw,pad_h,pad_w", _unpadded_geometries(2030, 32, 5))
def test_general_conv_over_tiles_without_halo_random(oracle, K, Ht, W, kh, kw, sh, sw, dh, dw, pad_h, pad_w):
    """adh_conv2d_unpadded_*_tiles against the oracle's convolution of the unsplit zero-padded tensor (rel-err 1e-5)."""
    rng = np.random.default_rng(Ht * 977 + W * 13 + kh)
    N, Cin, Cout = int(rng.integers(1, 4)), int(rng.integers(1, 40)), int(rng.integers(1, 40))
    geo = (kh, kw, sh, sw, dh, dw)
    H, OHt = K * Ht, Ht // sh
    OW = (W + 2 * pad_w - ((kw - 1) * dw + 1)) // sw + 1
    x = rng.uniform(-1, 1, size=(N, Cin, H, W)).astype(np.float32)
    w = rng.standard_normal((Cout, Cin, kh, kw)).astype(np.float32)
    dy = rng.standard_normal((N, Cout, K * OHt, OW)).astype(np.float32)
    xp = np.zeros((N, Cin, H + 2 * pad_h, W + 2 * pad_w), np.float32)
    xp[:, :, pad_h:pad_h + H, pad_w:pad_w + W] = x
    y_want = np.empty(dy.shape, np.float32)
    oracle.conv2d_slab_fwd(xp, w, sh, sw, dh, dw, y_want)
    gp = np.empty(xp.shape, np.float32)
    oracle.conv2d_slab_bwd_data(w, dy, sh, sw, dh, dw, gp)
    g_want = gp[:, :, pad_h:pad_h + H, pad_w:pad_w + W]
    gw_want = np.zeros(w.shape, np.float32)
    oracle.conv2d_slab_bwd_filter(xp, dy, sh, sw, dh, dw, gw_want)
    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * OHt:(r + 1) * OHt, :].copy()) for r in range(K)]
    d_w = dev(w)
    ws = torch.empty(max(capi.conv2d_unpadded_workspace_bytes(wh, capi.ADH_F32, K, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w)
                         for wh in (0, 1, 2)) // 4, device="cuda")
    ys = [torch.full((N, Cout, OHt, OW), float("nan"), device="cuda") for _ in range(K)]
    gs = [torch.full((N, Cin, Ht, W), float("nan"), device="cuda") for _ in range(K)]
    gw = torch.full(w.shape, float("nan"), device="cuda")
    capi.check(capi.conv2d_unpadded_fwd_tiles(xs, d_w, ys, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w, ws=ws), "fwd")
    capi.check(capi.conv2d_unpadded_bwd_data_tiles(d_w, dys, gs, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w, ws=ws), "bwd-data")
    capi.check(capi.conv2d_unpadded_bwd_filter_tiles(xs, dys, gw, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w, ws=ws), "bwd-filter")
    assert rel_err(host(gw), gw_want) <= 1e-5
    for r in range(K):
        assert rel_err(host(ys[r]), y_want[:, :, r * OHt:(r + 1) * OHt, :]) <= 1e-5
        assert rel_err(host(gs[r]), g_want[:, :, r * Ht:(r + 1) * Ht, :]) <= 1e-5


def _own_kernel_cases(seed, count):
    """(K, N, Cin, Cout, Ht, W, k, s, pad) that the 1x1 kernels (output rows of a multiple of 4 pixels, tile sides a
    multiple of the stride) and the stride-2 3x3 kernels (output rows of 8 or a multiple of 16 pixels, input channels a
    multiple of 4; the forward one from 256 input channels on) take instead of the general kernel."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        k = int(rng.choice([1, 3]))
        if k == 1:
            s = int(rng.integers(1, 3))
            OW, OH = 4 * int(rng.integers(1, 9)), int(rng.integers(1, 7))
            Cin, Cout = int(rng.integers(1, 150)), int(rng.integers(1, 150))
        else:
            s = 2
            OW, OH = int(rng.choice([8, 16, 32, 48])), int(rng.choice([1, 2, 3, 4, 6, 8]))
            Cin = 4 * int(rng.integers(1, 20)) if rng.integers(0, 3) else 256 + 4 * int(rng.integers(0, 5))
            Cout = int(rng.integers(1, 90 if Cin < 256 else 20))
        K, N = int(rng.integers(1, 5)), int(rng.integers(1, 7))
        if K * N * Cin * Cout * k * k * OH * OW > 6e7:  # keeps the scalar oracle to a second or two
            continue
        out.append((K, N, Cin, Cout, s * OH, s * OW, k, s, k // 2))
    return out


@pytest.mark.parametrize("K,N,Cin,Cout,Ht,W,k,s,pad", _own_kernel_cases(2033, 40))
def test_pointwise_and_strided_3x3_kernels_random(oracle, K, N, Cin, Cout, Ht, W, k, s, pad):
    """The three passes (backward-data with beta 0 and 1, the filter gradient with beta 0 and 1) of the shapes that have
    kernels of their own behind adh_conv2d_unpadded_*_tiles, against the oracle's convolution of the unsplit
    zero-padded tensor (fp32, rel-err <= 1e-5)."""
    rng = np.random.default_rng(Cin * 131 + Cout * 7 + W)
    geo = (k, k, s, s, 1, 1)
    H, OHt, OW = K * Ht, Ht // s, W // s
    x = rng.uniform(-1, 1, size=(N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, k, k)) * np.sqrt(2.0 / (Cin * k * k))).astype(np.float32)
    dy = rng.standard_normal((N, Cout, K * OHt, OW)).astype(np.float32)
    g0 = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    gw0 = rng.standard_normal(w.shape).astype(np.float32)
    xp = np.zeros((N, Cin, H + 2 * pad, W + 2 * pad), np.float32)
    xp[:, :, pad:pad + H, pad:pad + W] = x
    y_want = np.empty(dy.shape, np.float32)
    oracle.conv2d_slab_fwd(xp, w, s, s, 1, 1, y_want)
    gp = np.empty(xp.shape, np.float32)
    oracle.conv2d_slab_bwd_data(w, dy, s, s, 1, 1, gp)
    g_want = gp[:, :, pad:pad + H, pad:pad + W]
    gw_want = np.zeros(w.shape, np.float32)
    oracle.conv2d_slab_bwd_filter(xp, dy, s, s, 1, 1, gw_want)
    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * OHt:(r + 1) * OHt, :].copy()) for r in range(K)]
    d_w = dev(w)
    ws = torch.empty(max(capi.conv2d_unpadded_workspace_bytes(wh, capi.ADH_F32, K, N, Cin, Cout, Ht, W, *geo, pad, pad)
                         for wh in (0, 1, 2)) // 4, device="cuda")
    ys = [torch.full((N, Cout, OHt, OW), float("nan"), device="cuda") for _ in range(K)]
    gs = [torch.full((N, Cin, Ht, W), float("nan"), device="cuda") for _ in range(K)]
    ga = [dev(g0[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    gw, gwa = torch.full(w.shape, float("nan"), device="cuda"), dev(gw0)
    capi.check(capi.conv2d_unpadded_fwd_tiles(xs, d_w, ys, N, Cin, Cout, Ht, W, *geo, pad, pad, ws=ws), "fwd")
    capi.check(capi.conv2d_unpadded_bwd_data_tiles(d_w, dys, gs, N, Cin, Cout, Ht, W, *geo, pad, pad, ws=ws), "bwd-data")
    capi.check(capi.conv2d_unpadded_bwd_data_tiles(d_w, dys, ga, N, Cin, Cout, Ht, W, *geo, pad, pad, beta=1.0, ws=ws), "bwd-data +")
    capi.check(capi.conv2d_unpadded_bwd_filter_tiles(xs, dys, gw, N, Cin, Cout, Ht, W, *geo, pad, pad, ws=ws), "bwd-filter")
    capi.check(capi.conv2d_unpadded_bwd_filter_tiles(xs, dys, gwa, N, Cin, Cout, Ht, W, *geo, pad, pad, beta=1.0, ws=ws), "bwd-filter +")
    assert rel_err(host(gw), gw_want) <= 1e-5
    assert rel_err(host(gwa), gw0 + gw_want) <= 1e-5
    for r in range(K):
        assert rel_err(host(ys[r]), y_want[:, :, r * OHt:(r + 1) * OHt, :]) <= 1e-5
        assert rel_err(host(gs[r]), g_want[:, :, r * Ht:(r + 1) * Ht, :]) <= 1e-5
        assert rel_err(host(ga[r]), (g0 + g_want)[:, :, r * Ht:(r + 1) * Ht, :]) <= 1e-5


def _thin_cases(seed, count):
    """(K, N, Cin, Cout, HP, WP, kh, kw, sh, sw): at most three input channels and Cin kh kw <= 160, the shapes whose
    forward and filter gradient over halo-padded tiles take the kernels for a network's stem."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        Cin, kh, kw = int(rng.integers(1, 4)), int(rng.integers(1, 8)), int(rng.integers(1, 8))
        if (kh == 1 and kw == 1) or Cin * kh * kw > 160:
            continue
        sh, sw = int(rng.integers(1, 3)), int(rng.integers(1, 3))
        HP, WP = kh + int(rng.integers(0, 40)), kw + int(rng.integers(0, 90))
        K, N, Cout = int(rng.integers(1, 4)), int(rng.integers(1, 4)), int(rng.integers(1, 90))
        if K * N * Cin * Cout * kh * kw * ((HP - kh) // sh + 1) * ((WP - kw) // sw + 1) > 4e7:
            continue
        out.append((K, N, Cin, Cout, HP, WP, kh, kw, sh, sw))
    return out


@pytest.mark.parametrize("K,N,Cin,Cout,HP,WP,kh,kw,sh,sw", _thin_cases(2034, 32))
def test_few_input_channels_kernels_random(oracle, K, N, Cin, Cout, HP, WP, kh, kw, sh, sw):
    """Forward and filter gradient (beta 0 and 1) over halo-padded tiles with one to three input channels against the
    oracle (fp32, rel-err <= 1e-5)."""
    rng = np.random.default_rng(HP * 101 + WP * 3 + Cout)
    geo = (kh, kw, sh, sw, 1, 1)
    OH, OW = (HP - kh) // sh + 1, (WP - kw) // sw + 1
    xs = [rng.uniform(-1, 1, size=(N, Cin, HP, WP)).astype(np.float32) for _ in range(K)]
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * np.sqrt(2.0 / (Cin * kh * kw))).astype(np.float32)
    dys = [rng.standard_normal((N, Cout, OH, OW)).astype(np.float32) for _ in range(K)]
    y0 = [rng.standard_normal((N, Cout, OH, OW)).astype(np.float32) for _ in range(K)]
    gw0 = rng.standard_normal(w.shape).astype(np.float32)
    d_xs, d_dys, d_w = [dev(a) for a in xs], [dev(a) for a in dys], dev(w)
    ws = torch.empty(max(capi.conv2d_workspace_bytes(wh, capi.ADH_F32, K, N, Cin, Cout, HP, WP, *geo) for wh in (0, 2)) // 4,
                     device="cuda")
    ys = [torch.full((N, Cout, OH, OW), float("nan"), device="cuda") for _ in range(K)]
    ya = [dev(a) for a in y0]
    gw, gwa = torch.full(w.shape, float("nan"), device="cuda"), dev(gw0)
    capi.check(capi.conv2d_fwd_tiles(d_xs, d_w, ys, N, Cin, Cout, HP, WP, *geo, ws=ws), "fwd")
    capi.check(capi.conv2d_fwd_tiles(d_xs, d_w, ya, N, Cin, Cout, HP, WP, *geo, beta=1.0, ws=ws), "fwd +")
    capi.check(capi.conv2d_bwd_filter_tiles(d_xs, d_dys, gw, N, Cin, Cout, HP, WP, *geo, ws=ws), "bwd-filter")
    capi.check(capi.conv2d_bwd_filter_tiles(d_xs, d_dys, gwa, N, Cin, Cout, HP, WP, *geo, beta=1.0, ws=ws), "bwd-filter +")
    gw_want = np.zeros(w.shape, np.float32)
    for r in range(K):
        y = np.empty((N, Cout, OH, OW), np.float32)
        oracle.conv2d_slab_fwd(xs[r], w, sh, sw, 1, 1, y)
        assert rel_err(host(ys[r]), y) <= 1e-5
        assert rel_err(host(ya[r]), y0[r] + y) <= 1e-5
        oracle.conv2d_slab_bwd_filter(xs[r], dys[r], sh, sw, 1, 1, gw_want, beta=1.0)
    assert rel_err(host(gw), gw_want) <= 1e-5
    assert rel_err(host(gwa), gw0 + gw_want) <= 1e-5


@pytest.mark.parametrize("K,Ht,W,wh,ww,sh,sw,dh,dw,pad_h,pad_w", _unpadded_geometries(2031, 24, 4))
def test_pool_over_tiles_without_halo_random(oracle, K, Ht, W, wh, ww, sh, sw, dh, dw, pad_h, pad_w):
    """adh_pool2d_unpadded_*_tiles against the oracle's pooling of the unsplit zero-padded tensor (windows without
    dilation: the geometry's dilation is dropped and the row padding chosen again for the plain window)."""
    pads = [p for p in range(0, wh) if 0 < wh - 2 * p <= sh and p + (wh - 1 - p) // sh * sh <= Ht and wh - 1 - p <= Ht]
    if not pads:
        pytest.skip("no row padding stitches for this window and stride")
    pad_h = pads[0]
    pad_w = min(pad_w, ww - 1)
    rng = np.random.default_rng(Ht * 31 + W * 7 + wh)
    W = max(W, ww)
    N, C = int(rng.integers(1, 4)), int(rng.integers(1, 9))
    H, OHt, OW = K * Ht, Ht // sh, (W + 2 * pad_w - ww) // sw + 1
    x = rng.uniform(-1, 1, size=(N, C, H, W)).astype(np.float32)
    dy = rng.standard_normal((N, C, K * OHt, OW)).astype(np.float32)
    xp = np.zeros((N, C, H + 2 * pad_h, W + 2 * pad_w), np.float32)
    xp[:, :, pad_h:pad_h + H, pad_w:pad_w + W] = x
    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * OHt:(r + 1) * OHt, :].copy()) for r in range(K)]
    for mode in (capi.ADH_POOL_AVG, capi.ADH_POOL_MAX):
        y_want = np.empty(dy.shape, np.float32)
        oracle.pool_slab_fwd(mode, xp, wh, ww, sh, sw, y_want)
        gp = np.empty(xp.shape, np.float32)
        oracle.pool_slab_bwd(mode, xp, dy, wh, ww, sh, sw, gp)
        g_want = gp[:, :, pad_h:pad_h + H, pad_w:pad_w + W]
        ys = [torch.full((N, C, OHt, OW), float("nan"), device="cuda") for _ in range(K)]
        gs = [torch.full((N, C, Ht, W), float("nan"), device="cuda") for _ in range(K)]
        capi.check(capi.pool_unpadded_fwd_tiles(mode, xs, ys, N, C, Ht, W, wh, ww, sh, sw, pad_h, pad_w), "fwd")
        capi.check(capi.pool_unpadded_bwd_tiles(mode, xs, ys, dys, gs, N, C, Ht, W, wh, ww, sh, sw, pad_h, pad_w), "bwd")
        for r in range(K):
            want_y = y_want[:, :, r * OHt:(r + 1) * OHt, :]
            if mode == capi.ADH_POOL_MAX:
                assert np.array_equal(host(ys[r]), want_y)
            else:
                assert rel_err(host(ys[r]), want_y) <= 1e-5
            assert rel_err(host(gs[r]), g_want[:, :, r * Ht:(r + 1) * Ht, :]) <= 1e-5


def _residual_cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        K = int(rng.integers(1, 6))
        N = int(rng.integers(1, 5))
        Cin, Cout = int(rng.integers(1, 97)), int(rng.integers(1, 97))
        Ht, W = int(rng.integers(1, 20)), int(rng.integers(1, 70))
        if N * (Cin + 2 * Cout) * K * Ht * W <= 3_000_000:
            out.append((K, N, Cin, Cout, Ht, W))
    return out


@pytest.mark.parametrize("K,N,Cin,Cout,Ht,W", _residual_cases(2031, 24))
def test_fp32_forward_with_residual_random(oracle, K, N, Cin, Cout, Ht, W):
    """adh_conv3x3_unpadded_fwd_residual_tiles over random shapes: the unsplit convolution plus the residual (rel-err
    <= 1e-5), and the same bits as beta = 1 over a result that holds the residual."""
    rng = np.random.default_rng(Cin * 131 + Cout * 7 + K)
    H = K * Ht
    x = rng.uniform(-1, 1, size=(N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9))).astype(np.float32)
    res = rng.standard_normal((N, Cout, H, W)).astype(np.float32)
    xp = np.zeros((N, Cin, H + 2, W + 2), np.float32)
    xp[:, :, 1:-1, 1:-1] = x
    y_want = np.empty((N, Cout, H, W), np.float32)
    oracle.conv_slab_fwd(xp, w, y_want)
    y_want += res
    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    rs = [dev(res[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    ys = [torch.full_like(t, float("nan")) for t in rs]
    capi.check(capi.conv_unpadded_fwd_residual_tiles(xs, dev(w), rs, ys, N, Cin, Cout, Ht, W), "fwd + residual")
    by_beta = [t.clone() for t in rs]
    capi.check(capi.conv_unpadded_fwd_tiles(xs, dev(w), by_beta, N, Cin, Cout, Ht, W, beta=1.0), "fwd, beta 1")
    for r in range(K):
        assert rel_err(host(ys[r]), y_want[:, :, r * Ht:(r + 1) * Ht, :]) <= 1e-5
        assert torch.equal(ys[r], by_beta[r])
