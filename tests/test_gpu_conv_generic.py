"""GPU parity of the general slab convolution (any window / stride / dilation) against the CPU
oracle, through the C ABI: rel-err max|a-b| / max|b| <= 1e-5 in fp32; bf16 tensors (fp32
arithmetic, one rounding of the result) <= 5e-3."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5

CASES = [  # K, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw
    (2, 2, 3, 64, 20, 38, 7, 7, 2, 2, 1, 1),   # the stem: 7x7 stride 2 over halo 3, 3 input channels
    (1, 2, 3, 16, 12, 40, 7, 7, 1, 1, 1, 1),   # the spatial stem as built: 7x7 stride 1
    (2, 2, 16, 24, 10, 30, 3, 3, 2, 2, 1, 1),  # stride-2 3x3 over halo 1
    (1, 1, 8, 8, 14, 20, 3, 3, 1, 1, 3, 3),    # dilation 3 over halo 3
    (1, 2, 19, 70, 9, 17, 1, 1, 1, 1, 1, 1),   # 1x1 projection, channel counts off the steps
    (2, 1, 32, 40, 9, 33, 1, 1, 2, 2, 1, 1),   # strided 1x1 projection
    (1, 1, 5, 7, 11, 13, 3, 2, 2, 1, 2, 1),    # everything different per axis
    (1, 1, 4, 4, 9, 9, 2, 2, 3, 3, 1, 1),      # stride larger than the window: unread pixels
    (1, 3, 64, 128, 8, 72, 3, 3, 1, 1, 1, 1),  # two groups of output channels, wide rows
    (1, 1, 130, 20, 6, 6, 3, 3, 1, 1, 1, 1),   # many channel chunks, fewer than 16 columns
    (1, 1, 2, 3, 5, 5, 5, 5, 1, 1, 1, 1),      # a single output pixel
    (1, 1, 6, 5, 12, 70, 4, 4, 4, 4, 1, 1),    # 16 residue classes in backward-data
    (1, 7, 12, 20, 10, 34, 3, 3, 2, 2, 1, 1),  # 4x16 outputs: four images per block, the last block holds three
    (2, 5, 40, 48, 6, 18, 3, 3, 2, 2, 1, 1),   # 2x8 outputs (a late layer's tile): all five images in one block
    (2, 6, 33, 20, 4, 16, 1, 1, 2, 2, 1, 1),   # strided 1x1 over a tiny tile, several images per block
    (1, 2, 62, 30, 6, 10, 3, 3, 1, 1, 1, 1),   # 32-channel chunks whose last one is padded, in both passes
    (1, 3, 31, 31, 8, 8, 1, 1, 1, 1, 1, 1),    # one padded 32-channel chunk
    (1, 64, 8, 128, 18, 66, 3, 3, 1, 1, 1, 1), # enough blocks to keep them 64 output channels wide
    (1, 32, 8, 128, 18, 66, 3, 3, 1, 1, 1, 1), # half as many: 32 output channels per block
    (1, 48, 128, 8, 10, 66, 3, 3, 1, 1, 1, 1), # backward-data with 64-channel blocks and 32-channel chunks
    # 1x1 windows with output rows of a multiple of 4 pixels take the matrix-product kernels of their own
    (4, 5, 64, 128, 8, 32, 1, 1, 2, 2, 1, 1),    # a projection shortcut: 64 pixels x 64 channels per workgroup
    (2, 3, 70, 150, 6, 24, 1, 1, 2, 2, 1, 1),    # channel counts off every step: padded chunks and channel blocks
    (4, 16, 16, 130, 64, 64, 1, 1, 2, 2, 1, 1),  # 128 x 128 blocks forward (the last channel block holds 2), 128 x 64 backward
    (4, 16, 72, 24, 32, 64, 1, 1, 1, 1, 1, 1),   # stride 1: 128 x 64 blocks forward, 128 x 128 backward
    (3, 2, 5, 3, 2, 4, 1, 1, 2, 2, 1, 1),        # a single row of four pixels per image: most of the block is idle
    # at most three input channels: the forward pass flattens (channel, tap) pairs and stages the whole filter once
    (1, 2, 3, 64, 22, 70, 7, 7, 1, 1, 1, 1),     # the stem on 16x64 outputs: two row blocks and two column blocks, 16-byte stores
    (3, 2, 3, 70, 14, 45, 7, 7, 1, 1, 1, 1),     # 39 output columns (stores element by element), 64 + 6 output channels
    (2, 3, 1, 20, 19, 71, 3, 3, 2, 2, 1, 1),     # one input channel, stride 2
    # 3x3 at dilation 3 over halo 3 on launches of at least 256 workgroups: the 3x3 kernels with their taps three apart
    (2, 16, 20, 70, 40, 70, 3, 3, 1, 1, 3, 3),   # a ragged channel chunk, 64 + 6 output channels, two column tiles
    (1, 130, 8, 64, 23, 37, 3, 3, 1, 1, 3, 3),   # one column tile narrower than the patch, a short last row tile
    (1, 300, 8, 8, 7, 7, 3, 3, 1, 1, 3, 3),      # a single output pixel per image, 300 workgroups
    (1, 140, 9, 130, 12, 20, 3, 3, 1, 1, 3, 3),  # three groups of output channels (the last holds 2), 9 input channels
]


def out_dims(HP, WP, kh, kw, sh, sw, dh, dw):
    return (HP - ((kh - 1) * dh + 1)) // sh + 1, (WP - ((kw - 1) * dw + 1)) // sw + 1


def ws_for(which, dtype, K, N, Cin, Cout, HP, WP, *geo):
    nbytes = capi.conv2d_workspace_bytes(which, dtype, K, N, Cin, Cout, HP, WP, *geo)
    assert nbytes > 0
    return torch.empty(nbytes // 4, device="cuda")


@pytest.mark.parametrize("K,N,Cin,Cout,HP,WP,kh,kw,sh,sw,dh,dw", CASES)
def test_general_conv_f32_vs_oracle(oracle, K, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw):
    rng = np.random.default_rng(41 + WP)
    geo = (kh, kw, sh, sw, dh, dw)
    OH, OW = out_dims(HP, WP, *geo)
    xs = [rng.uniform(-1, 1, size=(N, Cin, HP, WP)).astype(np.float32) for _ in range(K)]
    w = (rng.standard_normal((Cout, Cin, kh, kw)) * np.sqrt(2.0 / (Cin * kh * kw))).astype(np.float32)
    dys = [rng.standard_normal((N, Cout, OH, OW)).astype(np.float32) for _ in range(K)]
    y0 = [rng.standard_normal((N, Cout, OH, OW)).astype(np.float32) for _ in range(K)]
    g0 = [rng.standard_normal((N, Cin, HP, WP)).astype(np.float32) for _ in range(K)]
    d_xs, d_dys, d_w = [dev(x) for x in xs], [dev(d) for d in dys], dev(w)
    ys = [torch.full((N, Cout, OH, OW), float("nan"), device="cuda") for _ in range(K)]
    ws_f = ws_for(capi.ADH_CONV_FWD, capi.ADH_F32, K, N, Cin, Cout, HP, WP, *geo)
    ws_b = ws_for(capi.ADH_CONV_BWD_DATA, capi.ADH_F32, K, N, Cin, Cout, HP, WP, *geo)
    capi.check(capi.conv2d_fwd_tiles(d_xs, d_w, ys, N, Cin, Cout, HP, WP, *geo, ws=ws_f))
    ya = [dev(a) for a in y0]
    capi.check(capi.conv2d_fwd_tiles(d_xs, d_w, ya, N, Cin, Cout, HP, WP, *geo, beta=1.0, ws=ws_f))
    gs = [torch.full((N, Cin, HP, WP), float("nan"), device="cuda") for _ in range(K)]
    capi.check(capi.conv2d_bwd_data_tiles(d_w, d_dys, gs, N, Cin, Cout, HP, WP, *geo, ws=ws_b))
    ga = [dev(a) for a in g0]
    capi.check(capi.conv2d_bwd_data_tiles(d_w, d_dys, ga, N, Cin, Cout, HP, WP, *geo, beta=1.0, ws=ws_b))
    for r in range(K):
        y = np.empty((N, Cout, OH, OW), np.float32)
        oracle.conv2d_slab_fwd(xs[r], w, sh, sw, dh, dw, y)
        assert rel_err(host(ys[r]), y) <= TOL
        y1 = y0[r].copy()
        oracle.conv2d_slab_fwd(xs[r], w, sh, sw, dh, dw, y1, beta=1.0)
        assert rel_err(host(ya[r]), y1) <= TOL
        g = np.empty((N, Cin, HP, WP), np.float32)
        oracle.conv2d_slab_bwd_data(w, dys[r], sh, sw, dh, dw, g)
        assert rel_err(host(gs[r]), g) <= TOL
        g1 = g0[r].copy()
        oracle.conv2d_slab_bwd_data(w, dys[r], sh, sw, dh, dw, g1, beta=1.0)
        assert rel_err(host(ga[r]), g1) <= TOL
    # filter gradient summed over the tiles, beta = 0 then beta = 1
    ws_w = ws_for(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, K, N, Cin, Cout, HP, WP, *geo)
    gw = torch.full((Cout, Cin, kh, kw), float("nan"), device="cuda")
    capi.check(capi.conv2d_bwd_filter_tiles(d_xs, d_dys, gw, N, Cin, Cout, HP, WP, *geo, ws=ws_w))
    dw_want = np.zeros((Cout, Cin, kh, kw), np.float32)
    for r in range(K):
        oracle.conv2d_slab_bwd_filter(xs[r], dys[r], sh, sw, dh, dw, dw_want, beta=1.0)
    assert rel_err(host(gw), dw_want) <= TOL
    capi.check(capi.conv2d_bwd_filter_tiles(d_xs, d_dys, gw, N, Cin, Cout, HP, WP, *geo, beta=1.0, ws=ws_w))
    assert rel_err(host(gw), 2 * dw_want) <= TOL
    small = torch.empty(8, device="cuda")
    assert capi.conv2d_bwd_filter_tiles(d_xs, d_dys, gw, N, Cin, Cout, HP, WP, *geo, ws=small) == capi.ADH_EWORKSPACE
    assert capi.conv2d_fwd_tiles(d_xs, d_w, ys, N, Cin, Cout, HP, WP, *geo, ws=small) == capi.ADH_EWORKSPACE
    assert capi.conv2d_fwd_tiles(d_xs, d_w, ys, N, Cin, Cout, HP, WP, *geo) == capi.ADH_ENULL


@pytest.mark.parametrize("K,N,Cin,Cout,HP,WP,kh,kw,sh,sw,dh,dw", [CASES[0], CASES[2], CASES[3], CASES[4], CASES[6], CASES[13]])
def test_general_conv_bf16_vs_oracle(oracle, K, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw):
    rng = np.random.default_rng(42 + WP)
    geo = (kh, kw, sh, sw, dh, dw)
    OH, OW = out_dims(HP, WP, *geo)
    bf = lambda a: oracle.f32_to_bf16(a.astype(np.float32))
    xs = [bf(rng.uniform(-1, 1, size=(N, Cin, HP, WP))) for _ in range(K)]
    w = bf(rng.standard_normal((Cout, Cin, kh, kw)) * np.sqrt(2.0 / (Cin * kh * kw)))
    dys = [bf(rng.standard_normal((N, Cout, OH, OW))) for _ in range(K)]
    d_xs, d_dys, d_w = [dev(x) for x in xs], [dev(d) for d in dys], dev(w)
    ys = [torch.empty((N, Cout, OH, OW), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    gs = [torch.empty((N, Cin, HP, WP), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.conv2d_fwd_tiles(d_xs, d_w, ys, N, Cin, Cout, HP, WP, *geo,
                                     ws=ws_for(capi.ADH_CONV_FWD, capi.ADH_BF16, K, N, Cin, Cout, HP, WP, *geo)))
    capi.check(capi.conv2d_bwd_data_tiles(d_w, d_dys, gs, N, Cin, Cout, HP, WP, *geo,
                                          ws=ws_for(capi.ADH_CONV_BWD_DATA, capi.ADH_BF16, K, N, Cin, Cout, HP, WP, *geo)))
    wf = oracle.bf16_to_f32(w)
    for r in range(K):
        y = np.empty((N, Cout, OH, OW), np.float32)
        oracle.conv2d_slab_fwd(oracle.bf16_to_f32(xs[r]), wf, sh, sw, dh, dw, y)
        assert rel_err(oracle.bf16_to_f32(host(ys[r])), y) <= 5e-3
        g = np.empty((N, Cin, HP, WP), np.float32)
        oracle.conv2d_slab_bwd_data(wf, oracle.bf16_to_f32(dys[r]), sh, sw, dh, dw, g)
        assert rel_err(oracle.bf16_to_f32(host(gs[r])), g) <= 5e-3
    gw = torch.empty((Cout, Cin, kh, kw), device="cuda")
    capi.check(capi.conv2d_bwd_filter_tiles(d_xs, d_dys, gw, N, Cin, Cout, HP, WP, *geo,
                                            ws=ws_for(capi.ADH_CONV_BWD_FILTER, capi.ADH_BF16, K, N, Cin, Cout, HP, WP, *geo)))
    dw_want = np.zeros((Cout, Cin, kh, kw), np.float32)
    for r in range(K):
        oracle.conv2d_slab_bwd_filter(oracle.bf16_to_f32(xs[r]), oracle.bf16_to_f32(dys[r]), sh, sw, dh, dw, dw_want, beta=1.0)
    assert rel_err(host(gw), dw_want) <= 1e-4  # fp32 output, exact bf16 products


def test_general_conv_stem_stitched_vs_unsplit():
    # 7x7 stride-2 stem over 4 row-tiles with halo 3 at N=8, 3->64 channels, 224x224: the stitched
    # tile outputs against torch's convolution of the zero-padded unsplit image, forward and backward
    K, N, Cin, Cout, H, W, p = 4, 8, 3, 64, 224, 224, 3
    Ht = H // K
    g = torch.Generator(device="cuda").manual_seed(12)
    xu = torch.rand((N, Cin, H, W), device="cuda", generator=g) * 2 - 1
    w = torch.randn((Cout, Cin, 7, 7), device="cuda", generator=g) * (2.0 / (Cin * 49)) ** 0.5
    tiles = [torch.empty((N, Cin, Ht + 2 * p, W + 2 * p), device="cuda") for _ in range(K)]
    capi.check(capi.tiles_pack(K, p, W, H, Cin, N, xu, tiles))
    geo = (7, 7, 2, 2, 1, 1)
    OH, OW = out_dims(Ht + 2 * p, W + 2 * p, *geo)
    assert (OH, OW) == (Ht // 2, W // 2)
    ys = [torch.empty((N, Cout, OH, OW), device="cuda") for _ in range(K)]
    ws = torch.empty(capi.conv2d_workspace_bytes(capi.ADH_CONV_FWD, capi.ADH_F32, K, N, Cin, Cout, Ht + 2 * p, W + 2 * p,
                                                 *geo) // 4, device="cuda")
    capi.check(capi.conv2d_fwd_tiles(tiles, w, ys, N, Cin, Cout, Ht + 2 * p, W + 2 * p, *geo, ws=ws))
    xp = F.pad(xu, (p, p, p, p)).double().requires_grad_(True)
    want = F.conv2d(xp, w.double(), stride=2)
    got = torch.cat(ys, dim=2)
    assert got.shape == want.shape
    dyu = torch.randn(want.shape, device="cuda", generator=g)
    want.backward(dyu.double())
    want = want.detach()
    assert float((got - want).abs().max() / want.abs().max()) <= TOL
    dys = [dyu[:, :, r * OH:(r + 1) * OH].contiguous() for r in range(K)]
    gs = [torch.empty((N, Cin, Ht + 2 * p, W + 2 * p), device="cuda") for _ in range(K)]
    wsb = torch.empty(capi.conv2d_workspace_bytes(capi.ADH_CONV_BWD_DATA, capi.ADH_F32, K, N, Cin, Cout, Ht + 2 * p,
                                                  W + 2 * p, *geo) // 4, device="cuda")
    capi.check(capi.conv2d_bwd_data_tiles(w, dys, gs, N, Cin, Cout, Ht + 2 * p, W + 2 * p, *geo, ws=wsb))
    total = torch.zeros_like(xp)
    for r in range(K):
        total[:, :, r * Ht:r * Ht + Ht + 2 * p] += gs[r]
    assert float((total - xp.grad).abs().max() / xp.grad.abs().max()) <= TOL
    # filter gradient summed over the tiles == the unsplit one
    wsw = torch.empty(capi.conv2d_workspace_bytes(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, K, N, Cin, Cout, Ht + 2 * p,
                                                  W + 2 * p, *geo) // 4, device="cuda")
    gw = torch.empty_like(w)
    capi.check(capi.conv2d_bwd_filter_tiles(tiles, dys, gw, N, Cin, Cout, Ht + 2 * p, W + 2 * p, *geo, ws=wsw))
    wd = w.double().requires_grad_(True)
    F.conv2d(xp.detach(), wd, stride=2).backward(dyu.double())
    assert float((gw - wd.grad).abs().max() / wd.grad.abs().max()) <= TOL


def test_general_conv_error_codes():
    x = torch.zeros((1, 4, 9, 9), device="cuda")
    w = torch.zeros((4, 4, 3, 3), device="cuda")
    y = torch.zeros((1, 4, 4, 4), device="cuda")
    ws = torch.empty(1 << 16, device="cuda")
    f = lambda kh, kw, sh, sw, dh, dw: capi.conv2d_fwd_tiles([x], w, [y], 1, 4, 4, 9, 9, kh, kw, sh, sw, dh, dw, ws=ws)
    assert f(3, 3, 2, 2, 1, 1) == capi.ADH_OK
    assert f(3, 3, 0, 2, 1, 1) == capi.ADH_EINVAL
    assert f(3, 3, 2, 2, 0, 1) == capi.ADH_EINVAL
    assert f(0, 3, 2, 2, 1, 1) == capi.ADH_EINVAL
    assert f(3, 3, 1, 1, 5, 5) == capi.ADH_EINVAL   # dilated window larger than the tile
    assert f(9, 9, 1, 1, 1, 1) == capi.ADH_EUNIMPL  # more than 64 taps
    assert f(3, 3, 5, 5, 1, 1) == capi.ADH_EUNIMPL  # more than 16 residue classes
    assert capi.conv2d_fwd_tiles([x], w, [y], 1, 4, 4, 9, 9, 3, 3, 2, 2, 1, 1, beta=0.5, ws=ws) == capi.ADH_EINVAL
    torch.cuda.synchronize()


@pytest.mark.parametrize("K,N,C,H,W,k,s,d", [(4, 32, 64, 128, 512, 3, 1, 3),   # tools/microbench_spatial_conv.cc:25-32 at full size
                                             (4, 8, 64, 32, 128, 3, 2, 1)])    # a strided 3x3 over padded tiles
def test_general_conv_three_passes_agree_on_one_number(K, N, C, H, W, k, s, d):
    """<dy, conv(x, w)> = <x_pad, conv_bwd_data(w, dy)> = <w, conv_bwd_filter(x_pad, dy)> for the general entry points
    at the reference's microbenchmark shape (3x3 at dilation 3 over halo 3: the 3x3 kernels with their taps three
    apart), fp32: a size-independent check that ties the three kernels together where the oracle would take minutes.
    Each stored output carries a relative rounding error of about 2^-20; the three numbers may differ by a few of
    those times the random-walk size of the sum."""
    g = torch.Generator(device="cuda").manual_seed(41)
    p = d * (k - 1) // 2
    HP, WP = H + 2 * p, W + 2 * p
    OH, OW = (HP - ((k - 1) * d + 1)) // s + 1, (WP - ((k - 1) * d + 1)) // s + 1
    xs = [torch.rand((N, C, HP, WP), device="cuda", generator=g) * 2 - 1 for _ in range(K)]
    dys = [torch.randn((N, C, OH, OW), device="cuda", generator=g) for _ in range(K)]
    w = torch.randn((C, C, k, k), device="cuda", generator=g) * (2.0 / (C * k * k)) ** 0.5
    geo = (k, k, s, s, d, d)
    nbytes = max(capi.lib().adh_conv2d_workspace_bytes(wh, capi.ADH_F32, K, N, C, C, HP, WP, *geo) for wh in (0, 1, 2))
    ws = torch.empty(nbytes // 4 + 64, device="cuda")
    ys = [torch.full((N, C, OH, OW), float("nan"), device="cuda") for _ in range(K)]
    gs = [torch.full((N, C, HP, WP), float("nan"), device="cuda") for _ in range(K)]
    gw = torch.full((C, C, k, k), float("nan"), device="cuda")
    capi.check(capi.conv2d_fwd_tiles(xs, w, ys, N, C, C, HP, WP, *geo, ws=ws), "fwd")
    capi.check(capi.conv2d_bwd_data_tiles(w, dys, gs, N, C, C, HP, WP, *geo, ws=ws), "bwd-data")
    capi.check(capi.conv2d_bwd_filter_tiles(xs, dys, gw, N, C, C, HP, WP, *geo, ws=ws), "bwd-filter")
    dot = lambda a, b: float((a.double() * b.double()).sum())
    via_fwd = sum(dot(dy, y) for dy, y in zip(dys, ys))
    via_data = sum(dot(x, gx) for x, gx in zip(xs, gs))
    via_filter = dot(w, gw)
    walk = sum(float(((dy.double() * y.double()) ** 2).sum()) for dy, y in zip(dys, ys)) ** 0.5
    eps = 2.0 ** -20
    assert np.isfinite(via_fwd) and abs(via_fwd) < 6.0 * walk
    assert abs(via_fwd - via_data) <= 6.0 * eps * walk
    assert abs(via_fwd - via_filter) <= 6.0 * eps * walk
