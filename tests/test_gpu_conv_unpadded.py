"""Convolution over row tiles that carry no halo (adh_conv3x3_unpadded_{fwd,bwd_data,bwd_filter}_tiles): tile t of the
result must be rows [t*H, (t+1)*H) of the UNSPLIT 3x3 convolution with zero padding 1 - what pad -> exchange ->
conv (forward) and conv backward-data -> reduce -> unpad (backward) compute in the reference's graph.  Checked
against the CPU oracle's unsplit convolution and, bit for bit, against this library's own padded chain.
bf16; rel-err max|a-b| / max|b| <= 5e-3 (one rounding of the result to bf16).  Every call goes through the
C ABI."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu

SHAPES = [  # K, N, Cin, Cout, Ht, W
    (1, 2, 8, 16, 5, 8), (2, 1, 19, 7, 6, 32), (3, 2, 64, 64, 7, 56), (4, 1, 64, 64, 1, 64), (4, 2, 20, 70, 2, 72),
    (8, 1, 64, 64, 3, 136), (2, 2, 64, 64, 40, 64), (5, 1, 33, 40, 4, 200), (2, 1, 128, 64, 12, 64), (3, 1, 64, 130, 5, 24),
    (2, 3, 100, 70, 9, 72)]


def ws_for(which, K, N, Cin, Cout, H, W):
    nbytes = capi.conv_workspace_bytes(which, capi.ADH_BF16, K, N, Cin, Cout, H, W)
    return torch.empty(nbytes // 4 + 64, device="cuda")


@pytest.mark.parametrize("K,N,Cin,Cout,Ht,W", SHAPES)
def test_unpadded_tiles_vs_unsplit_oracle(oracle, K, N, Cin, Cout, Ht, W):
    rng = np.random.default_rng(5100 + K * 13 + Cin)
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
    gx_want = gx_want[:, :, 1:-1, 1:-1]
    dw_want = np.zeros((Cout, Cin, 3, 3), np.float32)
    oracle.conv_slab_bwd_filter(xp, dyf, dw_want)

    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    y0 = [dev(bf(rng.standard_normal((N, Cout, Ht, W)))) for _ in range(K)]
    g0 = [dev(bf(rng.standard_normal((N, Cin, Ht, W)))) for _ in range(K)]
    d_w = dev(w)
    dw0 = dev(rng.standard_normal((Cout, Cin, 3, 3)).astype(np.float32))
    for beta in (0.0, 1.0):
        ys = [t.clone() for t in y0]
        gs = [t.clone() for t in g0]
        capi.check(capi.conv_unpadded_fwd_tiles(xs, d_w, ys, N, Cin, Cout, Ht, W, beta=beta,
                                                ws=ws_for(capi.ADH_CONV_FWD, K, N, Cin, Cout, Ht, W)), "fwd")
        capi.check(capi.conv_unpadded_bwd_data_tiles(d_w, dys, gs, N, Cin, Cout, Ht, W, beta=beta,
                                                     ws=ws_for(capi.ADH_CONV_BWD_DATA, K, N, Cin, Cout, Ht, W)), "bwd-data")
        dw = dw0.clone()
        capi.check(capi.conv_unpadded_bwd_filter_tiles(xs, dys, dw, N, Cin, Cout, Ht, W, beta=beta,
                                                       ws=ws_for(capi.ADH_CONV_BWD_FILTER, K, N, Cin, Cout, Ht, W)), "bwd-filter")
        assert rel_err(host(dw), dw_want + beta * host(dw0)) <= 1e-4  # fp32 output, exact bf16 products
        for r in range(K):
            want_y = y_want[:, :, r * Ht:(r + 1) * Ht, :] + beta * oracle.bf16_to_f32(host(y0[r]))
            want_g = gx_want[:, :, r * Ht:(r + 1) * Ht, :] + beta * oracle.bf16_to_f32(host(g0[r]))
            assert rel_err(oracle.bf16_to_f32(host(ys[r])), want_y) <= 5e-3
            assert rel_err(oracle.bf16_to_f32(host(gs[r])), want_g) <= 5e-3


@pytest.mark.parametrize("K,N,C,Ht,W", [(4, 2, 64, 12, 128), (8, 2, 64, 128, 2048), (4, 2, 192, 12, 128), (8, 2, 128, 128, 1024)])
def test_unpadded_forward_equals_the_padded_chain_bit_for_bit(K, N, C, Ht, W):
    """pack (pad) -> halo exchange -> conv over padded tiles multiplies the same values in the same order as the
    one launch over the tiles without halo: equal bits, at the full high-resolution configuration too."""
    g = torch.Generator(device="cuda").manual_seed(77)
    H = K * Ht
    X = (torch.rand((N, C, H, W), device="cuda", generator=g) * 2 - 1).to(torch.bfloat16)
    w = (torch.randn((C, C, 3, 3), device="cuda", generator=g) * (2.0 / (C * 9)) ** 0.5).to(torch.bfloat16)
    tiles = [torch.empty((N, C, Ht + 2, W + 2), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.tiles_pack(K, 1, W, H, C, N, X, tiles), "pack")  # pads, splits and exchanges in one pass
    ws = ws_for(capi.ADH_CONV_FWD, K, N, C, C, Ht, W)
    want = [torch.empty((N, C, Ht, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.conv_fwd_tiles(tiles, w, want, N, C, C, Ht, W, ws=ws), "fwd padded")
    xs = [X[:, :, r * Ht:(r + 1) * Ht, :].contiguous() for r in range(K)]
    got = [torch.empty_like(t) for t in want]
    capi.check(capi.conv_unpadded_fwd_tiles(xs, w, got, N, C, C, Ht, W, ws=ws), "fwd unpadded")
    for r in range(K):
        assert torch.equal(got[r].view(torch.int16), want[r].view(torch.int16))


def test_unpadded_entry_limits():
    x = [torch.zeros((1, 8, 4, 12), device="cuda", dtype=torch.bfloat16)]
    y = [torch.zeros((1, 8, 4, 12), device="cuda", dtype=torch.bfloat16)]
    w = torch.zeros((8, 8, 3, 3), device="cuda", dtype=torch.bfloat16)
    ws = torch.empty(1 << 16, device="cuda")
    assert capi.conv_unpadded_fwd_tiles(x, w, y, 1, 8, 8, 4, 12, ws=ws) == capi.ADH_EUNIMPL  # width not a multiple of 8
    x16 = [torch.zeros((1, 8, 4, 16), device="cuda", dtype=torch.bfloat16)]
    assert capi.conv_unpadded_fwd_tiles(x16, w, [torch.zeros_like(x16[0])], 1, 8, 8, 4, 16, beta=0.5, ws=ws) == capi.ADH_EINVAL
    assert capi.conv_unpadded_fwd_tiles(x16, w, [torch.zeros_like(x16[0])], 1, 8, 8, 4, 16, ws=None) == capi.ADH_ENULL


@pytest.mark.parametrize("K,N,Cin,Cout,Ht,W", [(1, 2, 8, 16, 5, 9), (2, 1, 19, 7, 6, 33), (4, 2, 9, 70, 1, 13), (3, 1, 24, 40, 23, 5),
                                              (4, 32, 64, 64, 14, 56), (2, 96, 8, 16, 11, 20), (5, 1, 16, 8, 3, 150)])
def test_unpadded_tiles_fp32_vs_unsplit_oracle(oracle, K, N, Cin, Cout, Ht, W):
    """The fp32 forms (any width): forward, backward-data and filter gradient over tiles without halo against the
    unsplit convolution, rel-err <= 1e-5, beta 0 and 1."""
    rng = np.random.default_rng(5200 + K * 13 + Cin)
    H = K * Ht
    x = rng.uniform(-1, 1, size=(N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9))).astype(np.float32)
    dy = rng.standard_normal((N, Cout, H, W)).astype(np.float32)
    xp = np.zeros((N, Cin, H + 2, W + 2), np.float32)
    xp[:, :, 1:-1, 1:-1] = x
    y_want = np.empty((N, Cout, H, W), np.float32)
    oracle.conv_slab_fwd(xp, w, y_want)
    gx_want = np.empty((N, Cin, H + 2, W + 2), np.float32)
    oracle.conv_slab_bwd_data(w, dy, gx_want)
    gx_want = gx_want[:, :, 1:-1, 1:-1]
    dw_want = np.zeros((Cout, Cin, 3, 3), np.float32)
    oracle.conv_slab_bwd_filter(xp, dy, dw_want)
    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    y0 = [dev(rng.standard_normal((N, Cout, Ht, W)).astype(np.float32)) for _ in range(K)]
    g0 = [dev(rng.standard_normal((N, Cin, Ht, W)).astype(np.float32)) for _ in range(K)]
    dw0 = dev(rng.standard_normal((Cout, Cin, 3, 3)).astype(np.float32))
    nbytes = capi.conv_workspace_bytes(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, K, N, Cin, Cout, Ht, W)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")
    for beta in (0.0, 1.0):
        ys, gs, dw = [t.clone() for t in y0], [t.clone() for t in g0], dw0.clone()
        capi.check(capi.conv_unpadded_fwd_tiles(xs, dev(w), ys, N, Cin, Cout, Ht, W, beta=beta), "fwd")
        capi.check(capi.conv_unpadded_bwd_data_tiles(dev(w), dys, gs, N, Cin, Cout, Ht, W, beta=beta), "bwd-data")
        capi.check(capi.conv_unpadded_bwd_filter_tiles(xs, dys, dw, N, Cin, Cout, Ht, W, beta=beta, ws=ws), "bwd-filter")
        assert rel_err(host(dw), dw_want + beta * host(dw0)) <= 1e-5
        for r in range(K):
            assert rel_err(host(ys[r]), y_want[:, :, r * Ht:(r + 1) * Ht, :] + beta * host(y0[r])) <= 1e-5
            assert rel_err(host(gs[r]), gx_want[:, :, r * Ht:(r + 1) * Ht, :] + beta * host(g0[r])) <= 1e-5


@pytest.mark.parametrize("K,N,Cin,Cout,Ht,W", [(1, 2, 8, 16, 5, 9), (2, 1, 19, 7, 6, 33), (4, 2, 9, 70, 1, 13), (3, 1, 24, 40, 23, 5),
                                              (4, 32, 64, 64, 14, 56), (2, 8, 128, 128, 14, 28), (5, 1, 16, 8, 3, 150)])
def test_unpadded_forward_with_residual(oracle, K, N, Cin, Cout, Ht, W):
    """adh_conv3x3_unpadded_fwd_residual_tiles: y = conv(x, w) + res against the oracle's unsplit convolution plus the
    same residual (rel-err <= 1e-5), and bit for bit against adh_conv3x3_unpadded_fwd_tiles with beta = 1 over a result
    that holds the residual (the same kernel, the same order of additions) - with the residual in its own tensors and
    with the result's tensors themselves as the residual."""
    rng = np.random.default_rng(5300 + K * 13 + Cin)
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
    kept = [t.clone() for t in rs]
    ys = [torch.full_like(t, float("nan")) for t in rs]
    capi.check(capi.conv_unpadded_fwd_residual_tiles(xs, dev(w), rs, ys, N, Cin, Cout, Ht, W), "fwd + residual")
    by_beta = [t.clone() for t in rs]
    capi.check(capi.conv_unpadded_fwd_tiles(xs, dev(w), by_beta, N, Cin, Cout, Ht, W, beta=1.0), "fwd, beta 1")
    in_place = [t.clone() for t in rs]
    capi.check(capi.conv_unpadded_fwd_residual_tiles(xs, dev(w), in_place, in_place, N, Cin, Cout, Ht, W), "fwd + residual, in place")
    for r in range(K):
        assert rel_err(host(ys[r]), y_want[:, :, r * Ht:(r + 1) * Ht, :]) <= 1e-5
        assert torch.equal(ys[r], by_beta[r]) and torch.equal(ys[r], in_place[r])
        assert torch.equal(rs[r], kept[r])  # the residual is read only


def test_unpadded_forward_with_residual_rejects():
    x = [torch.zeros(1, 8, 4, 16, device="cuda")]
    y = [torch.zeros(1, 8, 4, 16, device="cuda")]
    w = torch.zeros(8, 8, 3, 3, device="cuda")
    xb, yb, wb = [t.bfloat16() for t in x], [t.bfloat16() for t in y], w.bfloat16()
    assert capi.conv_unpadded_fwd_residual_tiles(xb, wb, yb, yb, 1, 8, 8, 4, 16) == capi.ADH_EUNIMPL  # fp32 only
    from ctypes import c_void_p
    tbl = (c_void_p * 1)(x[0].data_ptr())
    nul = (c_void_p * 1)(None)
    out = (c_void_p * 1)(y[0].data_ptr())
    f = capi.lib().adh_conv3x3_unpadded_fwd_residual_tiles
    assert f(capi.ADH_F32, 1, 1, 8, 8, 4, 16, tbl, w.data_ptr(), None, out, None) == capi.ADH_ENULL
    assert f(capi.ADH_F32, 1, 1, 8, 8, 4, 16, tbl, w.data_ptr(), nul, out, None) == capi.ADH_ENULL
