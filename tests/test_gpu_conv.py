"""GPU parity of the 3x3 slab convolution (fwd, bwd-data, bwd-filter) against the CPU oracle
and against the UNSPLIT convolution.  fp32 tolerance: rel-err = max|a-b| / max|b| <= 1e-5.

Every call goes through the C ABI."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


def he_normal(rng, Cout, Cin, k=3):
    return (rng.standard_normal((Cout, Cin, k, k)) * np.sqrt(2.0 / (Cin * k * k))).astype(np.float32)


def workspace(which, K, N, Cin, Cout, H, W):
    nbytes = capi.conv_workspace_bytes(which, capi.ADH_F32, K, N, Cin, Cout, H, W)
    return torch.empty(max(nbytes // 4, 1), device="cuda") if nbytes else None


SMALL = [  # K, N, Cin, Cout, H, W
    (1, 1, 8, 16, 4, 8), (1, 2, 3, 5, 5, 7), (2, 2, 16, 16, 6, 17), (1, 1, 64, 64, 14, 56), (3, 1, 9, 70, 11, 13),
    (1, 1, 130, 20, 3, 60), (2, 3, 24, 40, 23, 5), (1, 2, 4, 4, 1, 1), (1, 1, 8, 8, 5, 61), (2, 1, 16, 8, 9, 150),
    (1, 1, 4, 36, 3, 257),
    # many planes of a 16x20 / 11x20 tile: the launch is large enough for the 8-wave kernels, whose tall form
    # (tiles of up to 18 rows, 20 staged patch rows) then wins: forward 16 and 11 rows per tile, backward-data 18 and 13
    (2, 96, 8, 8, 16, 20), (2, 96, 8, 16, 11, 20)]


@pytest.mark.parametrize("K,N,Cin,Cout,H,W", SMALL)
def test_conv_fwd_vs_oracle(oracle, K, N, Cin, Cout, H, W):
    rng = np.random.default_rng(1000 + Cin)
    xs = [rng.uniform(-1, 1, size=(N, Cin, H + 2, W + 2)).astype(np.float32) for _ in range(K)]
    w = he_normal(rng, Cout, Cin)
    y0 = [rng.standard_normal((N, Cout, H, W)).astype(np.float32) for _ in range(K)]
    for beta in (0.0, 1.0):
        want = [y.copy() for y in y0]
        for r in range(K):
            oracle.conv_slab_fwd(xs[r], w, want[r], beta=beta)
        dy = [dev(y) for y in y0]
        capi.check(capi.conv_fwd_tiles([dev(x) for x in xs], dev(w), dy, N, Cin, Cout, H, W, beta=beta), "fwd")
        for r in range(K):
            assert rel_err(host(dy[r]), want[r]) <= TOL


@pytest.mark.parametrize("K,N,Cin,Cout,H,W", SMALL)
def test_conv_bwd_data_vs_oracle(oracle, K, N, Cin, Cout, H, W):
    rng = np.random.default_rng(2000 + Cin)
    dys = [rng.standard_normal((N, Cout, H, W)).astype(np.float32) for _ in range(K)]
    w = he_normal(rng, Cout, Cin)
    g0 = [rng.standard_normal((N, Cin, H + 2, W + 2)).astype(np.float32) for _ in range(K)]
    for beta in (0.0, 1.0):
        want = [g.copy() for g in g0]
        for r in range(K):
            oracle.conv_slab_bwd_data(w, dys[r], want[r], beta=beta)
        dg = [dev(g) for g in g0]
        capi.check(capi.conv_bwd_data_tiles(dev(w), [dev(d) for d in dys], dg, N, Cin, Cout, H, W, beta=beta), "bwd_data")
        for r in range(K):
            assert rel_err(host(dg[r]), want[r]) <= TOL


@pytest.mark.parametrize("K,N,Cin,Cout,H,W", SMALL)
def test_conv_bwd_filter_vs_oracle(oracle, K, N, Cin, Cout, H, W):
    rng = np.random.default_rng(3000 + Cin)
    xs = [rng.uniform(-1, 1, size=(N, Cin, H + 2, W + 2)).astype(np.float32) for _ in range(K)]
    dys = [rng.standard_normal((N, Cout, H, W)).astype(np.float32) for _ in range(K)]
    dw0 = rng.standard_normal((Cout, Cin, 3, 3)).astype(np.float32)
    ws = workspace(capi.ADH_CONV_BWD_FILTER, K, N, Cin, Cout, H, W)
    for beta in (0.0, 1.0):
        want = dw0.copy() if beta else np.zeros_like(dw0)
        for r in range(K):
            oracle.conv_slab_bwd_filter(xs[r], dys[r], want, beta=1.0)
        ddw = dev(dw0)
        capi.check(capi.conv_bwd_filter_tiles([dev(x) for x in xs], [dev(d) for d in dys], ddw, N, Cin, Cout, H, W,
                                              beta=beta, ws=ws), "bwd_filter")
        got = host(ddw)
        assert rel_err(got, want) <= TOL
        # deterministic: a second run gives the same bits
        ddw2 = dev(dw0)
        capi.check(capi.conv_bwd_filter_tiles([dev(x) for x in xs], [dev(d) for d in dys], ddw2, N, Cin, Cout, H, W,
                                              beta=beta, ws=ws))
        np.testing.assert_array_equal(host(ddw2), got)


def test_conv_closed_forms():
    # delta kernel = identity on the interior; hot pixel in dy lays the filter down in dx
    N, C, H, W = 2, 16, 6, 9
    x = torch.rand(N, C, H + 2, W + 2, device="cuda") * 2 - 1
    w = torch.zeros(C, C, 3, 3, device="cuda")
    for c in range(C):
        w[c, c, 1, 1] = 1
    y = torch.empty(N, C, H, W, device="cuda")
    capi.check(capi.conv_fwd_tiles([x], w, [y], N, C, C, H, W))
    assert torch.equal(y, x[:, :, 1:-1, 1:-1])
    w2 = torch.randn(C, C, 3, 3, device="cuda")
    dy = torch.zeros(N, C, H, W, device="cuda")
    dy[1, 3, 2, 4] = 1
    dx = torch.full((N, C, H + 2, W + 2), float("nan"), device="cuda")
    capi.check(capi.conv_bwd_data_tiles(w2, [dy], [dx], N, C, C, H, W))
    want = torch.zeros_like(dx)
    want[1, :, 2:5, 4:7] = w2[3]
    assert torch.equal(dx, want)
    ws = workspace(capi.ADH_CONV_BWD_FILTER, 1, N, C, C, H, W)
    dw = torch.full((C, C, 3, 3), float("nan"), device="cuda")
    capi.check(capi.conv_bwd_filter_tiles([x], [dy], dw, N, C, C, H, W, ws=ws))
    want = torch.zeros_like(dw)
    want[3] = x[1, :, 2:5, 4:7]
    assert torch.equal(dw, want)


def test_conv_error_codes():
    x = torch.zeros(1, 4, 5, 5, device="cuda")
    w = torch.zeros(4, 4, 3, 3, device="cuda")
    y = torch.zeros(1, 4, 3, 3, device="cuda")
    assert capi.conv_fwd_tiles([x], w, [y], 1, 4, 4, 3, 3, beta=0.5) == capi.ADH_EINVAL
    xb = x.to(torch.bfloat16)
    # bf16 needs the workspace its query asks for
    assert capi.conv_fwd_tiles([xb], w.to(torch.bfloat16), [y.to(torch.bfloat16)], 1, 4, 4, 3, 3) == capi.ADH_ENULL
    dw = torch.zeros_like(w)
    small = torch.empty(4, device="cuda")
    assert capi.conv_bwd_filter_tiles([x], [y], dw, 1, 4, 4, 3, 3, ws=small) == capi.ADH_EWORKSPACE


def assert_close_elementwise(got, ref):
    """Every element on its own: the max-norm bar alone would pass a 1 % error on an output that is a thousandth
    of the largest.  rtol 1e-4 with an absolute floor of 1e-5 of the largest reference value (sums of 576 and
    more products that cancel towards zero keep the absolute error of their terms)."""
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-5 * float(np.max(np.abs(ref))))


def _config(rng, K=4, N=32, C=64, H=56, W=56):
    X = rng.uniform(-1, 1, size=(N, C, H, W)).astype(np.float32)
    w = he_normal(rng, C, C)
    dY = rng.standard_normal((N, C, H, W)).astype(np.float32)
    return X, w, dY


def test_config2_fwd_stitched_vs_unsplit(oracle):
    """fp32 N=32, C=64, 56x56 in 4 row-tiles of 14(+2)x56(+2): stitched tiles vs the unsplit conv."""
    rng = np.random.default_rng(0x5EED)
    K, N, C, H, W, p = 4, 32, 64, 56, 56, 1
    Ht = H // K
    X, w, _ = _config(rng)
    dX, dw = dev(X), dev(w)
    tiles = [torch.empty((N, C, Ht + 2, W + 2), device="cuda") for _ in range(K)]
    capi.check(capi.tiles_pack(K, p, W, H, C, N, dX, tiles))
    ys = [torch.empty((N, C, Ht, W), device="cuda") for _ in range(K)]
    capi.check(capi.conv_fwd_tiles(tiles, dw, ys, N, C, C, Ht, W))
    Y = torch.cat(ys, dim=2)
    ref = F.conv2d(torch.from_numpy(X).double(), torch.from_numpy(w).double(), padding=1).numpy()
    assert rel_err(host(Y), ref) <= TOL
    assert_close_elementwise(host(Y), ref)
    # the oracle agrees on one full tile (scalar fp64 accumulate)
    want = np.empty((N, C, Ht, W), np.float32)
    oracle.conv_slab_fwd(host(tiles[1]), w, want)
    assert rel_err(host(ys[1]), want) <= TOL
    # the single-slab entry point gives the same bits as the batched launch
    y1 = torch.empty_like(ys[2])
    capi.check(capi.lib().adh_conv3x3_slab_fwd(0, N, C, C, Ht, W, tiles[2].data_ptr(), dw.data_ptr(), y1.data_ptr(),
                                              0.0, None, 0, None))
    assert torch.equal(y1, ys[2])


def test_config3_fwd_bwd_vs_unsplit(oracle):
    """cfg2 plus bwd-data + halo reduce + bwd-filter, compared with the unsplit backward."""
    rng = np.random.default_rng(0x5EED + 3)
    K, N, C, H, W, p = 4, 32, 64, 56, 56, 1
    Ht = H // K
    X, w, dY = _config(rng)
    tX = torch.from_numpy(X).double().requires_grad_()
    tw = torch.from_numpy(w).double().requires_grad_()
    F.conv2d(tX, tw, padding=1).backward(torch.from_numpy(dY).double())
    dX, dw = dev(X), dev(w)
    tiles = [torch.empty((N, C, Ht + 2, W + 2), device="cuda") for _ in range(K)]
    capi.check(capi.tiles_pack(K, p, W, H, C, N, dX, tiles))
    dys = [dev(np.ascontiguousarray(dY[:, :, r * Ht:(r + 1) * Ht])) for r in range(K)]
    # bwd-data onto zeroed slabs with beta = 1 (the reference's call), then reduce, then unpack
    gs = [torch.zeros((N, C, Ht + 2, W + 2), device="cuda") for _ in range(K)]
    capi.check(capi.conv_bwd_data_tiles(dw, dys, gs, N, C, C, Ht, W, beta=1.0))
    capi.check(capi.halo_reduce(gs, 1, K, p, W, Ht, C, N))
    gX = torch.empty_like(dX)
    capi.check(capi.tiles_unpack(K, p, W, H, C, N, gs, gX))
    assert rel_err(host(gX), tX.grad.numpy()) <= TOL
    assert_close_elementwise(host(gX), tX.grad.numpy())
    ws = workspace(capi.ADH_CONV_BWD_FILTER, K, N, C, C, Ht, W)
    gw = torch.zeros_like(dw)
    capi.check(capi.conv_bwd_filter_tiles(tiles, dys, gw, N, C, C, Ht, W, beta=1.0, ws=ws))
    assert rel_err(host(gw), tw.grad.numpy()) <= TOL
    assert_close_elementwise(host(gw), tw.grad.numpy())
    # oracle on one image of one tile (scalar fp64)
    want = np.zeros((1, C, Ht + 2, W + 2), np.float32)
    oracle.conv_slab_bwd_data(w, host(dys[1])[:1].copy(), want)
    g1 = torch.empty((1, C, Ht + 2, W + 2), device="cuda")
    capi.check(capi.conv_bwd_data_tiles(dw, [dys[1][:1].contiguous()], [g1], 1, C, C, Ht, W))
    assert rel_err(host(g1), want) <= TOL
