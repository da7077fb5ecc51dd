"""GPU parity of the bf16 slab convolution (bf16 in HBM, fp32 accumulate): rel-err
max|a-b| / max|b| <= 2e-2 against the oracle fed with the same bf16 values, on small shapes in
full and at the full high-resolution configuration (N=2, C=64, 1024x2048, 8 row-tiles of 128
rows, halo 1) by sampling: every tile-boundary row for some channels plus >= 1e5 random outputs,
each recomputed in float64 from the UNSPLIT tensors.  Every call goes through the C ABI."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu
TOL = 2e-2


def ws_for(which, K, N, Cin, Cout, H, W):
    nbytes = capi.conv_workspace_bytes(which, capi.ADH_BF16, K, N, Cin, Cout, H, W)
    assert nbytes > 0
    return torch.empty(nbytes // 4 + 64, device="cuda")


# shapes cover: channel counts off the 8/32/64 steps, two output-channel groups, odd widths,
# widths off the 32-column strip, row counts off the 8-row step and split into row segments,
# and reductions wider than 64 channels (the widening route)
@pytest.mark.parametrize("K,N,Cin,Cout,H,W", [(1, 2, 8, 16, 5, 9), (2, 1, 19, 7, 6, 33), (3, 2, 64, 64, 7, 56),
                                              (1, 1, 20, 70, 9, 61), (2, 2, 64, 64, 40, 70), (1, 1, 64, 64, 3, 130),
                                              (1, 1, 72, 64, 6, 20), (1, 1, 64, 72, 6, 20), (1, 3, 33, 40, 17, 31),
                                              # widths that are multiples of eight: the bf16 filter-gradient kernel
                                              (1, 2, 16, 24, 5, 8), (2, 1, 64, 64, 9, 72), (1, 1, 40, 48, 3, 136),
                                              (3, 2, 7, 5, 1, 64), (1, 1, 64, 64, 2, 200),
                                              # more than 64 reduction channels on the matrix cores: one pass per
                                              # 64 with fp32 sums in between (two and three passes, a last pass of
                                              # 36 channels, edge strips, output-channel remainders, both directions)
                                              (2, 1, 128, 64, 12, 64), (1, 1, 192, 32, 9, 128), (1, 2, 100, 70, 8, 72),
                                              (1, 1, 160, 16, 5, 16), (2, 1, 64, 128, 12, 64), (1, 1, 48, 130, 6, 24),
                                              (1, 1, 256, 256, 4, 64)])
def test_bf16_conv_small_vs_oracle(oracle, K, N, Cin, Cout, H, W):
    rng = np.random.default_rng(77 + Cin)
    bf = lambda a: oracle.f32_to_bf16(a.astype(np.float32))
    xs = [bf(rng.uniform(-1, 1, size=(N, Cin, H + 2, W + 2))) for _ in range(K)]
    w = bf(rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9)))
    dys = [bf(rng.standard_normal((N, Cout, H, W))) for _ in range(K)]
    wf = oracle.bf16_to_f32(w)
    dw_want = np.zeros((Cout, Cin, 3, 3), np.float32)
    d_xs, d_dys, d_w = [dev(x) for x in xs], [dev(d) for d in dys], dev(w)
    ys = [torch.empty((N, Cout, H, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    gs = [torch.empty((N, Cin, H + 2, W + 2), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.conv_fwd_tiles(d_xs, d_w, ys, N, Cin, Cout, H, W, ws=ws_for(capi.ADH_CONV_FWD, K, N, Cin, Cout, H, W)))
    capi.check(capi.conv_bwd_data_tiles(d_w, d_dys, gs, N, Cin, Cout, H, W,
                                        ws=ws_for(capi.ADH_CONV_BWD_DATA, K, N, Cin, Cout, H, W)))
    dw = torch.zeros((Cout, Cin, 3, 3), device="cuda")
    capi.check(capi.conv_bwd_filter_tiles(d_xs, d_dys, dw, N, Cin, Cout, H, W, beta=1.0,
                                          ws=ws_for(capi.ADH_CONV_BWD_FILTER, K, N, Cin, Cout, H, W)))
    for r in range(K):
        xf, dyf = oracle.bf16_to_f32(xs[r]), oracle.bf16_to_f32(dys[r])
        y = np.empty((N, Cout, H, W), np.float32)
        oracle.conv_slab_fwd(xf, wf, y)
        assert rel_err(oracle.bf16_to_f32(host(ys[r])), y) <= TOL
        # exact products and fp32 sums: only the final rounding to bf16 (2^-9 relative) remains
        assert rel_err(oracle.bf16_to_f32(host(ys[r])), y) <= 5e-3
        g = np.empty((N, Cin, H + 2, W + 2), np.float32)
        oracle.conv_slab_bwd_data(wf, dyf, g)
        assert rel_err(oracle.bf16_to_f32(host(gs[r])), g) <= 5e-3
        oracle.conv_slab_bwd_filter(xf, dyf, dw_want, beta=1.0)
    assert rel_err(host(dw), dw_want) <= 1e-4  # fp32 output, exact bf16 products
    # beta = 1 accumulates onto a bf16 output
    y2 = [y.clone() for y in ys]
    capi.check(capi.conv_fwd_tiles(d_xs, d_w, y2, N, Cin, Cout, H, W, beta=1.0,
                                   ws=ws_for(capi.ADH_CONV_FWD, K, N, Cin, Cout, H, W)))
    assert rel_err(y2[0].float().cpu().numpy(), 2 * ys[0].float().cpu().numpy()) <= TOL
    small = torch.empty(16, device="cuda")
    assert capi.conv_fwd_tiles(d_xs, d_w, ys, N, Cin, Cout, H, W, ws=small) == capi.ADH_EWORKSPACE


def test_bf16_conv_odd_pointers_and_many_images(oracle):
    """Tile buffers that are only 2-byte aligned (views one element into an allocation), more work
    items than workgroups, a one-row image, a single channel, and more than 64 channels on both sides
    (several launches with fp32 sums between them)."""
    rng = np.random.default_rng(404)
    bf = lambda a: oracle.f32_to_bf16(a.astype(np.float32))
    for (N, Cin, Cout, H, W) in ((300, 8, 8, 1, 8), (3, 1, 1, 5, 16), (2, 64, 64, 6, 64), (2, 160, 136, 6, 64)):
        x = bf(rng.uniform(-1, 1, size=(N, Cin, H + 2, W + 2)))
        w = bf(rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9)))
        dy = bf(rng.standard_normal((N, Cout, H, W)))

        def odd(a):  # device copy whose first element sits at an odd 2-byte offset
            buf = torch.empty(a.size + 1, device="cuda", dtype=torch.bfloat16)
            v = buf[1:].view(a.shape)
            v.copy_(dev(a).view(a.shape))
            return v

        d_x, d_dy, d_w = odd(x), odd(dy), dev(w)
        y = odd(np.zeros((N, Cout, H, W), np.uint16))
        gx = odd(np.zeros((N, Cin, H + 2, W + 2), np.uint16))
        dw = torch.zeros((Cout, Cin, 3, 3), device="cuda")
        capi.check(capi.conv_fwd_tiles([d_x], d_w, [y], N, Cin, Cout, H, W, ws=ws_for(capi.ADH_CONV_FWD, 1, N, Cin, Cout, H, W)))
        capi.check(capi.conv_bwd_data_tiles(d_w, [d_dy], [gx], N, Cin, Cout, H, W,
                                            ws=ws_for(capi.ADH_CONV_BWD_DATA, 1, N, Cin, Cout, H, W)))
        capi.check(capi.conv_bwd_filter_tiles([d_x], [d_dy], dw, N, Cin, Cout, H, W,
                                              ws=ws_for(capi.ADH_CONV_BWD_FILTER, 1, N, Cin, Cout, H, W)))
        xf, dyf, wf = oracle.bf16_to_f32(x), oracle.bf16_to_f32(dy), oracle.bf16_to_f32(w)
        y_want = np.empty((N, Cout, H, W), np.float32)
        oracle.conv_slab_fwd(xf, wf, y_want)
        assert rel_err(y.float().cpu().numpy(), y_want) <= 5e-3
        g_want = np.empty((N, Cin, H + 2, W + 2), np.float32)
        oracle.conv_slab_bwd_data(wf, dyf, g_want)
        assert rel_err(gx.float().cpu().numpy(), g_want) <= 5e-3
        dw_want = np.zeros((Cout, Cin, 3, 3), np.float32)
        oracle.conv_slab_bwd_filter(xf, dyf, dw_want, beta=0.0)
        assert rel_err(host(dw), dw_want) <= 1e-4


@pytest.mark.parametrize("C,W", [(64, 2048), (128, 1024)])
def test_config5_highres_bf16_fwd_bwd_sampled(oracle, C, W):
    """bf16 N=2, C=64, 1024x2048 in 8 row-tiles of 128 rows + halo 1 (and the same flops at 128 channels, 1024 columns:
    one launch of 128 reduction channels): pack, conv fwd, bwd-data + halo reduce + unpack, bwd-filter, each checked
    against the UNSPLIT convolution on samples."""
    K, N, H, p = 8, 2, 1024, 1
    Ht = H // K
    g = torch.Generator(device="cuda").manual_seed(0x5EED)
    X = (torch.rand((N, C, H, W), device="cuda", generator=g) * 2 - 1).to(torch.bfloat16)
    wt = (torch.randn((C, C, 3, 3), device="cuda", generator=g) * (2.0 / (C * 9)) ** 0.5).to(torch.bfloat16)
    dY = torch.randn((N, C, H, W), device="cuda", generator=g).to(torch.bfloat16)
    tiles = [torch.empty((N, C, Ht + 2, W + 2), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.tiles_pack(K, p, W, H, C, N, X, tiles))
    ys = [torch.empty((N, C, Ht, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    ws = ws_for(capi.ADH_CONV_BWD_FILTER, K, N, C, C, Ht, W)
    assert ws.numel() * 4 >= capi.conv_workspace_bytes(capi.ADH_CONV_FWD, capi.ADH_BF16, K, N, C, C, Ht, W)
    capi.check(capi.conv_fwd_tiles(tiles, wt, ys, N, C, C, Ht, W, ws=ws))
    Y = torch.cat(ys, dim=2)
    dys = [dY[:, :, r * Ht:(r + 1) * Ht].contiguous() for r in range(K)]
    gs = [torch.empty((N, C, Ht + 2, W + 2), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.conv_bwd_data_tiles(wt, dys, gs, N, C, C, Ht, W, ws=ws))
    capi.check(capi.halo_reduce(gs, 1, K, p, W, Ht, C, N))
    gX = torch.empty_like(X)
    capi.check(capi.tiles_unpack(K, p, W, H, C, N, gs, gX))
    gw = torch.zeros((C, C, 3, 3), device="cuda")
    capi.check(capi.conv_bwd_filter_tiles(tiles, dys, gw, N, C, C, Ht, W, beta=1.0, ws=ws))
    torch.cuda.synchronize()
    del ws, tiles, gs

    Xh = np.pad(X.float().cpu().numpy(), ((0, 0), (0, 0), (1, 1), (1, 1)))
    dYh = np.pad(dY.float().cpu().numpy(), ((0, 0), (0, 0), (1, 1), (1, 1)))
    wh = wt.float().cpu().numpy().astype(np.float64)
    Yh = Y.float().cpu().numpy()
    gXh = gX.float().cpu().numpy()
    rng = np.random.default_rng(5)

    def sample_coords(count):
        n = rng.integers(0, N, count)
        c = rng.integers(0, C, count)
        h = rng.integers(0, H, count)
        w_ = rng.integers(0, W, count)
        # all tile-boundary rows (+-2) for two (n, c) pairs, every column
        rows = np.array([r * Ht + d for r in range(1, K) for d in (-2, -1, 0, 1)] + [0, 1, H - 2, H - 1])
        for (nn, cc) in ((0, 3), (1, C - 24)):
            hh, ww = np.meshgrid(rows, np.arange(W), indexing="ij")
            n = np.concatenate([n, np.full(hh.size, nn)])
            c = np.concatenate([c, np.full(hh.size, cc)])
            h = np.concatenate([h, hh.ravel()])
            w_ = np.concatenate([w_, ww.ravel()])
        return n, c, h, w_

    # forward: y[n,co,h,w] = sum_{ci,a,b} w[co,ci,a,b] * Xp[n,ci,h+a,w+b]
    n, co, h, w_ = sample_coords(100000)
    ref = np.zeros(n.size, np.float64)
    for a in range(3):
        for b in range(3):
            patch = Xh[n, :, h + a, w_ + b].astype(np.float64)      # (samples, C)
            ref += np.einsum("sc,sc->s", patch, wh[co, :, a, b])
    got = Yh[n, co, h, w_]
    assert np.max(np.abs(got - ref)) / np.max(np.abs(ref)) <= TOL
    # backward-data of the unsplit conv: dx[n,ci,h,w] = sum_{co,a,b} w[co,ci,a,b] * dYp[n,co,h+2-a,w+2-b]
    n, ci, h, w_ = sample_coords(100000)
    ref = np.zeros(n.size, np.float64)
    for a in range(3):
        for b in range(3):
            patch = dYh[n, :, h + 2 - a, w_ + 2 - b].astype(np.float64)
            ref += np.einsum("sc,sc->s", patch, wh[:, ci, a, b].T)
    got = gXh[n, ci, h, w_]
    assert np.max(np.abs(got - ref)) / np.max(np.abs(ref)) <= TOL
    # backward-filter on 48 (co, ci) pairs, all 9 taps, summed over every pixel
    gwh = gw.cpu().numpy()
    dYc = dYh[:, :, 1:-1, 1:-1]
    errs, mags = [], []
    for _ in range(48):
        co_, ci_ = int(rng.integers(0, C)), int(rng.integers(0, C))
        for a in range(3):
            for b in range(3):
                ref1 = float(np.sum(dYc[:, co_].astype(np.float64) * Xh[:, ci_, a:a + H, b:b + W]))
                errs.append(abs(gwh[co_, ci_, a, b] - ref1))
                mags.append(abs(ref1))
    assert max(errs) / max(mags) <= 1e-3


@pytest.mark.parametrize("dtype,K,N,C,Ht,W,eps", [(torch.bfloat16, 8, 2, 64, 128, 2048, 2.0 ** -9),
                                                  (torch.bfloat16, 4, 1, 128, 64, 512, 2.0 ** -9),
                                                  (torch.float32, 4, 32, 64, 14, 56, 2.0 ** -20)])
def test_three_passes_agree_on_one_number(dtype, K, N, C, Ht, W, eps):
    """<dy, conv(x, w)> = <x_pad, conv_bwd_data(w, dy)> = <w, conv_bwd_filter(x_pad, dy)>: the three kernels compute
    the same trilinear form, at the full high-resolution configuration too (a size-independent check that ties
    forward, backward-data and backward-filter together; a wrong tap, a transposed filter or a dropped row or
    channel in any one of them breaks an equality).  The sums run in float64 on the GPU over the stored outputs.
    The terms dy*y have random signs, so the number itself is a random-walk sum of size sqrt(sum (dy*y)^2), and each
    stored output carries an independent relative rounding error eps (bf16: 2^-9; fp32: the order of its 576 or
    1152 additions, 2^-20): the three numbers may differ by a few eps * sqrt(sum (dy*y)^2), six of which are
    allowed.  One tap, row or channel dropped in one kernel moves its number by a tenth of that root or more."""
    g = torch.Generator(device="cuda").manual_seed(31)
    xs = [(torch.rand((N, C, Ht + 2, W + 2), device="cuda", generator=g) * 2 - 1).to(dtype) for _ in range(K)]
    dys = [torch.randn((N, C, Ht, W), device="cuda", generator=g).to(dtype) for _ in range(K)]
    w = (torch.randn((C, C, 3, 3), device="cuda", generator=g) * (2.0 / (C * 9)) ** 0.5).to(dtype)
    code = capi.ADH_BF16 if dtype == torch.bfloat16 else capi.ADH_F32
    nbytes = max(capi.conv_workspace_bytes(wh, code, K, N, C, C, Ht, W)
                 for wh in (capi.ADH_CONV_FWD, capi.ADH_CONV_BWD_DATA, capi.ADH_CONV_BWD_FILTER))
    ws = torch.empty(nbytes // 4 + 64, device="cuda")
    ys = [torch.empty((N, C, Ht, W), device="cuda", dtype=dtype) for _ in range(K)]
    gs = [torch.empty((N, C, Ht + 2, W + 2), device="cuda", dtype=dtype) for _ in range(K)]
    gw = torch.empty((C, C, 3, 3), device="cuda")
    capi.check(capi.conv_fwd_tiles(xs, w, ys, N, C, C, Ht, W, ws=ws))
    capi.check(capi.conv_bwd_data_tiles(w, dys, gs, N, C, C, Ht, W, ws=ws))
    capi.check(capi.conv_bwd_filter_tiles(xs, dys, gw, N, C, C, Ht, W, ws=ws))
    dot = lambda a, b: float((a.double() * b.double()).sum())
    via_fwd = sum(dot(dy, y) for dy, y in zip(dys, ys))
    via_data = sum(dot(x, gx) for x, gx in zip(xs, gs))
    via_filter = dot(w, gw)
    walk = sum(float(((dy.double() * y.double()) ** 2).sum()) for dy, y in zip(dys, ys)) ** 0.5
    assert abs(via_fwd) < 6.0 * walk  # sanity of the scale itself
    assert abs(via_fwd - via_data) <= 6.0 * eps * walk
    assert abs(via_fwd - via_filter) <= 6.0 * eps * walk
