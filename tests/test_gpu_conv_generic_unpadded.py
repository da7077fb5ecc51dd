"""The general convolution over row tiles that carry no halo (adh_conv2d_unpadded_{fwd,bwd_data,bwd_filter}_tiles):
tile t of the result must be the rows of the UNSPLIT convolution with zero padding that belong to it - what
pad -> exchange -> conv (forward) and conv backward-data -> reduce -> unpad (backward) compute in the
reference's graph.  Checked against the CPU oracle's convolution of the unsplit, zero-padded tensor.
fp32: rel-err max|a-b| / max|b| <= 1e-5; bf16 tensors (fp32 arithmetic, one rounding of the result) <= 5e-3.
Every call goes through the C ABI."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5

CASES = [  # K, N, Cin, Cout, Ht, W, kh, kw, sh, sw, dh, dw, pad_h, pad_w
    (4, 3, 16, 24, 4, 16, 3, 3, 1, 1, 1, 1, 1, 1),    # a late layer's tile: stride-1 3x3 on 4x16
    (4, 5, 40, 48, 2, 8, 3, 3, 1, 1, 1, 1, 1, 1),     # 2x8 tiles: both neighbours' rows in every window
    (4, 2, 16, 24, 8, 32, 3, 3, 2, 2, 1, 1, 1, 1),    # stride-2 3x3, pad 1: the row above comes from the neighbour
    (2, 2, 33, 20, 4, 16, 3, 3, 2, 2, 1, 1, 1, 1),    # the same on 4x16 tiles, channel counts off the steps
    (3, 2, 3, 16, 8, 40, 7, 7, 1, 1, 1, 1, 3, 3),     # the 7x7 stem over halo 3
    (2, 1, 3, 64, 16, 38, 7, 7, 2, 2, 1, 1, 3, 3),    # 7x7 stride 2 pad 3: 7 - 6 = 1 <= 2
    (2, 2, 32, 40, 6, 18, 1, 1, 2, 2, 1, 1, 0, 0),    # strided 1x1 projection: no neighbour is ever read
    (2, 1, 8, 8, 9, 20, 3, 3, 1, 1, 3, 3, 3, 3),      # dilation 3 over halo 3
    (1, 2, 19, 30, 6, 10, 3, 3, 1, 1, 1, 1, 1, 1),    # one tile: a convolution with zero padding
    (3, 1, 5, 7, 4, 13, 3, 2, 2, 1, 1, 1, 1, 0),      # different per axis, no column padding
    (5, 2, 64, 64, 2, 72, 3, 3, 1, 1, 1, 1, 1, 1),    # wide rows, five tiles of two rows
    (2, 1, 12, 20, 4, 12, 5, 5, 1, 1, 1, 1, 2, 2),    # 5x5: two rows from each neighbour
    (4, 32, 8, 16, 2, 8, 3, 3, 2, 2, 1, 1, 1, 1),     # 1x4 outputs per tile: many images per block
    # stride-2 3x3 whose backward-data takes the kernel of its own (fp32, output rows of 8 or a multiple of 16 pixels)
    (2, 6, 20, 24, 4, 16, 3, 3, 2, 2, 1, 1, 1, 1),    # 2x8 outputs: four images per workgroup, the second group holds two
    (3, 2, 8, 40, 16, 64, 3, 3, 2, 2, 1, 1, 1, 1),    # 8x32 outputs: two row blocks and two column blocks per image
    (2, 3, 68, 16, 4, 32, 3, 3, 2, 2, 1, 1, 1, 1),    # 2x16 outputs: two images per workgroup, a second channel group of 4
    (1, 2, 4, 4, 16, 16, 3, 3, 2, 2, 1, 1, 1, 1),     # 8x8 outputs on a single tile: zeros below
    # ... and with at least 256 input channels the forward takes its own kernel too
    (2, 5, 256, 72, 4, 16, 3, 3, 2, 2, 1, 1, 1, 1),   # 2x8 outputs, four images per workgroup (then one), 64 + 8 output channels
    (2, 2, 260, 16, 8, 32, 3, 3, 2, 2, 1, 1, 1, 1),   # 4x16 outputs, a last chunk of four input channels
    (3, 1, 256, 8, 16, 64, 3, 3, 2, 2, 1, 1, 1, 1),   # 8x32 outputs over three tiles: row -1 from the tile above
    (1, 1, 256, 8, 16, 16, 3, 3, 2, 2, 1, 1, 1, 1),   # 8x8 outputs on a single tile: zeros above
    # many channels over few, full blocks of pixels: blocks of 64 output channels, the channel chunks dealt to 4 and 8 workgroups
    (2, 16, 128, 64, 2, 8, 3, 3, 1, 1, 1, 1, 1, 1),   # 16 chunks of 8 channels in 4 parts
    (2, 16, 256, 208, 2, 8, 3, 3, 1, 1, 1, 1, 1, 1),  # 32 chunks in 8 parts, 192 + 16 output channels; backward-data: 26 chunks in 4
    (4, 4, 512, 64, 4, 16, 3, 3, 1, 1, 1, 1, 1, 1),   # 4x16 tiles, four images per block: 32 chunks of 16 channels in 8 parts
]


def out_w(W, kw, sw, dw, pad_w):
    return (W + 2 * pad_w - ((kw - 1) * dw + 1)) // sw + 1


def unsplit_reference(oracle, x, w, dy, geo, pad_h, pad_w):
    """y, dx and dw of the unsplit convolution with zero padding, from the oracle's padded-slab functions."""
    kh, kw, sh, sw, dh, dw_ = geo
    N, Cin, H, W = x.shape
    Cout = w.shape[0]
    xp = np.zeros((N, Cin, H + 2 * pad_h, W + 2 * pad_w), np.float32)
    xp[:, :, pad_h:pad_h + H, pad_w:pad_w + W] = x
    y = np.empty(dy.shape, np.float32)
    oracle.conv2d_slab_fwd(xp, w, sh, sw, dh, dw_, y)
    gp = np.empty(xp.shape, np.float32)
    oracle.conv2d_slab_bwd_data(w, dy, sh, sw, dh, dw_, gp)
    gw = np.zeros(w.shape, np.float32)
    oracle.conv2d_slab_bwd_filter(xp, dy, sh, sw, dh, dw_, gw)
    return y, gp[:, :, pad_h:pad_h + H, pad_w:pad_w + W], gw


@pytest.mark.parametrize("K,N,Cin,Cout,Ht,W,kh,kw,sh,sw,dh,dw,pad_h,pad_w", CASES)
def test_general_unpadded_f32_vs_unsplit_oracle(oracle, K, N, Cin, Cout, Ht, W, kh, kw, sh, sw, dh, dw, pad_h, pad_w):
    rng = np.random.default_rng(900 + K * 7 + W + kh)
    geo = (kh, kw, sh, sw, dh, dw)
    H, OHt, OW = K * Ht, Ht // sh, out_w(W, kw, sw, dw, pad_w)
    x = rng.uniform(-1, 1, size=(N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * np.sqrt(2.0 / (Cin * kh * kw))).astype(np.float32)
    dy = rng.standard_normal((N, Cout, K * OHt, OW)).astype(np.float32)
    y_want, gx_want, gw_want = unsplit_reference(oracle, x, w, dy, geo, pad_h, pad_w)
    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * OHt:(r + 1) * OHt, :].copy()) for r in range(K)]
    y0 = [rng.standard_normal((N, Cout, OHt, OW)).astype(np.float32) for _ in range(K)]
    g0 = [rng.standard_normal((N, Cin, Ht, W)).astype(np.float32) for _ in range(K)]
    gw0 = rng.standard_normal(w.shape).astype(np.float32)
    d_w = dev(w)
    ws = {}
    for which in (capi.ADH_CONV_FWD, capi.ADH_CONV_BWD_DATA, capi.ADH_CONV_BWD_FILTER):
        nbytes = capi.conv2d_unpadded_workspace_bytes(which, capi.ADH_F32, K, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w)
        assert nbytes > 0
        ws[which] = torch.empty(nbytes // 4, device="cuda")
    for beta in (0.0, 1.0):
        nan = float("nan")
        ys = [dev(a) if beta else torch.full(a.shape, nan, device="cuda") for a in y0]
        gs = [dev(a) if beta else torch.full(a.shape, nan, device="cuda") for a in g0]
        gw = dev(gw0) if beta else torch.full(w.shape, nan, device="cuda")
        capi.check(capi.conv2d_unpadded_fwd_tiles(xs, d_w, ys, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w, beta=beta,
                                                  ws=ws[capi.ADH_CONV_FWD]), "fwd")
        capi.check(capi.conv2d_unpadded_bwd_data_tiles(d_w, dys, gs, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w, beta=beta,
                                                       ws=ws[capi.ADH_CONV_BWD_DATA]), "bwd-data")
        capi.check(capi.conv2d_unpadded_bwd_filter_tiles(xs, dys, gw, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w, beta=beta,
                                                         ws=ws[capi.ADH_CONV_BWD_FILTER]), "bwd-filter")
        assert rel_err(host(gw), gw_want + beta * gw0) <= TOL
        for r in range(K):
            assert rel_err(host(ys[r]), y_want[:, :, r * OHt:(r + 1) * OHt, :] + beta * y0[r]) <= TOL
            assert rel_err(host(gs[r]), gx_want[:, :, r * Ht:(r + 1) * Ht, :] + beta * g0[r]) <= TOL


@pytest.mark.parametrize("K,N,Cin,Cout,Ht,W,kh,kw,sh,sw,dh,dw,pad_h,pad_w", [CASES[0], CASES[2], CASES[4], CASES[6]])
def test_general_unpadded_bf16_vs_unsplit_oracle(oracle, K, N, Cin, Cout, Ht, W, kh, kw, sh, sw, dh, dw, pad_h, pad_w):
    rng = np.random.default_rng(901 + K * 7 + W + kh)
    geo = (kh, kw, sh, sw, dh, dw)
    bf = lambda a: oracle.f32_to_bf16(a.astype(np.float32))
    H, OHt, OW = K * Ht, Ht // sh, out_w(W, kw, sw, dw, pad_w)
    x = bf(rng.uniform(-1, 1, size=(N, Cin, H, W)))
    w = bf(rng.standard_normal((Cout, Cin, kh, kw)) * np.sqrt(2.0 / (Cin * kh * kw)))
    dy = bf(rng.standard_normal((N, Cout, K * OHt, OW)))
    y_want, gx_want, gw_want = unsplit_reference(oracle, oracle.bf16_to_f32(x), oracle.bf16_to_f32(w), oracle.bf16_to_f32(dy),
                                                 geo, pad_h, pad_w)
    xs = [dev(x[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    dys = [dev(dy[:, :, r * OHt:(r + 1) * OHt, :].copy()) for r in range(K)]
    d_w = dev(w)
    ys = [torch.empty((N, Cout, OHt, OW), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    gs = [torch.empty((N, Cin, Ht, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    gw = torch.empty(w.shape, device="cuda")
    wsf = lambda which: torch.empty(capi.conv2d_unpadded_workspace_bytes(which, capi.ADH_BF16, K, N, Cin, Cout, Ht, W, *geo,
                                                                         pad_h, pad_w) // 4, device="cuda")
    capi.check(capi.conv2d_unpadded_fwd_tiles(xs, d_w, ys, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w, ws=wsf(capi.ADH_CONV_FWD)))
    capi.check(capi.conv2d_unpadded_bwd_data_tiles(d_w, dys, gs, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w,
                                                   ws=wsf(capi.ADH_CONV_BWD_DATA)))
    capi.check(capi.conv2d_unpadded_bwd_filter_tiles(xs, dys, gw, N, Cin, Cout, Ht, W, *geo, pad_h, pad_w,
                                                     ws=wsf(capi.ADH_CONV_BWD_FILTER)))
    assert rel_err(host(gw), gw_want) <= 1e-4  # fp32 output, exact bf16 products
    for r in range(K):
        assert rel_err(oracle.bf16_to_f32(host(ys[r])), y_want[:, :, r * OHt:(r + 1) * OHt, :]) <= 5e-3
        assert rel_err(oracle.bf16_to_f32(host(gs[r])), gx_want[:, :, r * Ht:(r + 1) * Ht, :]) <= 5e-3


def test_general_unpadded_limits():
    """Splits the kernels do not serve are refused, not computed wrongly."""
    K, N, C = 2, 1, 4
    xs = [torch.zeros((N, C, 5, 8), device="cuda") for _ in range(K)]
    ys = [torch.zeros((N, C, 5, 8), device="cuda") for _ in range(K)]
    w = torch.zeros((C, C, 3, 3), device="cuda")
    ws = torch.empty(1 << 16, device="cuda")
    # 5 rows per tile at stride 2: the tiles' outputs do not stitch
    assert capi.conv2d_unpadded_fwd_tiles(xs, w, ys, N, C, C, 5, 8, 3, 3, 2, 2, 1, 1, 1, 1, ws=ws) == capi.ADH_EINVAL
    # 3x3 with no padding loses rows: H / sh output rows per tile is not what the unsplit convolution has
    assert capi.conv2d_unpadded_fwd_tiles(xs, w, ys, N, C, C, 5, 8, 3, 3, 1, 1, 1, 1, 0, 1, ws=ws) == capi.ADH_EINVAL
    # padding of 2 for a 3x3 grows the output
    assert capi.conv2d_unpadded_fwd_tiles(xs, w, ys, N, C, C, 5, 8, 3, 3, 1, 1, 1, 1, 2, 1, ws=ws) == capi.ADH_EINVAL
    # a window that reaches past the adjacent tile: 13x13 (pad 6) over tiles of 5 rows
    w13 = torch.zeros((C, C, 13, 13), device="cuda")
    assert capi.conv2d_unpadded_fwd_tiles(xs, w13, ys, N, C, C, 5, 8, 13, 13, 1, 1, 1, 1, 6, 6, ws=ws) == capi.ADH_EINVAL
    assert capi.conv2d_unpadded_workspace_bytes(capi.ADH_CONV_FWD, capi.ADH_F32, K, N, C, C, 5, 8, 3, 3, 2, 2, 1, 1, 1, 1) == 0
