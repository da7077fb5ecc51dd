"""The exchange-free forms of the 3x3 slab convolution (the input gradient that needs no halo reduce is further
down): forward and filter gradient over row tiles whose
inner halo rows were never exchanged must equal halo exchange followed by the ordinary entry point, bit for
bit (same kernels, same order of additions, only the address of two input rows per tile differs), and the
fp32 forms must not read the inner halo rows at all (they hold NaN here).  One case is also checked against
the CPU oracle's exchange + convolution.  Every call goes through the C ABI."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu

SHAPES = [  # K, N, Cin, Cout, H, W
    (1, 2, 8, 8, 5, 9), (2, 1, 3, 5, 1, 7), (2, 2, 16, 16, 6, 17), (4, 2, 9, 70, 11, 13), (3, 1, 24, 40, 23, 5),
    (2, 1, 16, 8, 9, 150), (8, 1, 8, 8, 2, 30), (4, 32, 64, 64, 14, 56), (2, 96, 8, 16, 11, 20)]


def make_tiles(rng, K, N, C, H, W, dtype=torch.float32):
    """Padded tiles as after HaloPad2DOp (outer halo and halo columns zero) with NaN in the part of the inner
    halo rows that an exchange overwrites (the interior columns; the corners stay zero)."""
    xs = []
    for r in range(K):
        x = torch.zeros((N, C, H + 2, W + 2), device="cuda", dtype=dtype)
        x[:, :, 1:-1, 1:-1] = dev(rng.uniform(-1, 1, size=(N, C, H, W)).astype(np.float32)).to(dtype)
        if r > 0:
            x[:, :, 0, 1:-1] = float("nan")
        if r + 1 < K:
            x[:, :, -1, 1:-1] = float("nan")
        xs.append(x)
    return xs


def he_normal(rng, Cout, Cin):
    return (rng.standard_normal((Cout, Cin, 3, 3)) * np.sqrt(2.0 / (Cin * 9))).astype(np.float32)


def workspace(which, dtype, K, N, Cin, Cout, H, W):
    nbytes = capi.conv_workspace_bytes(which, dtype, K, N, Cin, Cout, H, W)
    return torch.empty(max(nbytes // 4, 1), device="cuda") if nbytes else None


@pytest.mark.parametrize("K,N,Cin,Cout,H,W", SHAPES)
def test_forward_equals_exchange_then_forward(K, N, Cin, Cout, H, W):
    rng = np.random.default_rng(4100 + K * 7 + Cin)
    xs = make_tiles(rng, K, N, Cin, H, W)
    w = dev(he_normal(rng, Cout, Cin))
    y0 = [dev(rng.standard_normal((N, Cout, H, W)).astype(np.float32)) for _ in range(K)]
    exchanged = [x.clone() for x in xs]
    capi.check(capi.halo_exchange(exchanged, 1, K, 1, W, H, Cin, N), "exchange")
    for beta in (0.0, 1.0):
        want = [y.clone() for y in y0]
        capi.check(capi.conv_fwd_tiles(exchanged, w, want, N, Cin, Cout, H, W, beta=beta), "fwd")
        got = [y.clone() for y in y0]
        before = [x.clone() for x in xs]
        capi.check(capi.conv_fwd_tiles(xs, w, got, N, Cin, Cout, H, W, beta=beta, unexchanged=True), "fwd unexchanged")
        for r in range(K):
            assert not torch.isnan(got[r]).any()
            assert torch.equal(got[r], want[r])
            # the input is left as it was, NaN rows included
            assert torch.equal(xs[r].view(torch.int32), before[r].view(torch.int32))


@pytest.mark.parametrize("K,N,Cin,Cout,H,W", SHAPES)
def test_filter_gradient_equals_exchange_then_filter_gradient(K, N, Cin, Cout, H, W):
    rng = np.random.default_rng(4200 + K * 7 + Cin)
    xs = make_tiles(rng, K, N, Cin, H, W)
    dys = [dev(rng.standard_normal((N, Cout, H, W)).astype(np.float32)) for _ in range(K)]
    dw0 = dev(rng.standard_normal((Cout, Cin, 3, 3)).astype(np.float32))
    ws = workspace(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, K, N, Cin, Cout, H, W)
    exchanged = [x.clone() for x in xs]
    capi.check(capi.halo_exchange(exchanged, 1, K, 1, W, H, Cin, N), "exchange")
    for beta in (0.0, 1.0):
        want = dw0.clone()
        capi.check(capi.conv_bwd_filter_tiles(exchanged, dys, want, N, Cin, Cout, H, W, beta=beta, ws=ws), "wgrad")
        got = dw0.clone()
        capi.check(capi.conv_bwd_filter_tiles(xs, dys, got, N, Cin, Cout, H, W, beta=beta, ws=ws, unexchanged=True),
                   "wgrad unexchanged")
        assert not torch.isnan(got).any()
        assert torch.equal(got, want)


@pytest.mark.parametrize("K,N,Cin,Cout,H,W", SHAPES)
def test_reduced_input_gradient_equals_backward_data_then_reduce(K, N, Cin, Cout, H, W):
    rng = np.random.default_rng(4500 + K * 7 + Cin)
    w = dev(he_normal(rng, Cout, Cin))
    dys = [dev(rng.standard_normal((N, Cout, H, W)).astype(np.float32)) for _ in range(K)]
    g0 = [dev(rng.standard_normal((N, Cin, H + 2, W + 2)).astype(np.float32)) for _ in range(K)]
    for beta in (0.0, 1.0):
        # the two-launch form: backward-data into a cleared buffer, halo reduce, then the accumulation
        part = [torch.zeros_like(g) for g in g0]
        capi.check(capi.conv_bwd_data_tiles(w, dys, part, N, Cin, Cout, H, W), "bwd-data")
        if H >= 2:
            capi.check(capi.halo_reduce(part, 1, K, 1, W, H, Cin, N), "reduce")
        want = [p + beta * g for p, g in zip(part, g0)]
        got = [g.clone() for g in g0]
        capi.check(capi.conv_bwd_data_tiles(w, dys, got, N, Cin, Cout, H, W, beta=beta, reduced=True), "bwd-data reduced")
        for r in range(K):
            if H >= 2:
                # same terms in another order of additions: fp32 tolerance 1e-5 of the largest value
                # (interior columns: the reduce moves the W interior columns of a halo row, the halo columns of
                # the gradient are read by nobody)
                assert rel_err(host(got[r][:, :, 1:-1, 1:-1]), host(want[r][:, :, 1:-1, 1:-1])) <= 1e-5
            # outer halo rows have no neighbour: the plain backward-data's values
            if r == 0:
                assert rel_err(host(got[r][:, :, 0, :]), host(want[r][:, :, 0, :])) <= 1e-5
            if r == K - 1:
                assert rel_err(host(got[r][:, :, -1, :]), host(want[r][:, :, -1, :])) <= 1e-5


def test_reduced_input_gradient_vs_unsplit_oracle(oracle):
    """The interiors of the K gradient tiles, stitched, are the unsplit convolution's input gradient."""
    K, N, Cin, Cout, Ht, W = 4, 2, 6, 10, 5, 12
    H = K * Ht
    rng = np.random.default_rng(4600)
    w = he_normal(rng, Cout, Cin)
    dy = rng.standard_normal((N, Cout, H, W)).astype(np.float32)
    want = np.zeros((N, Cin, H + 2, W + 2), np.float32)
    oracle.conv_slab_bwd_data(w, dy, want)
    dys = [dev(dy[:, :, r * Ht:(r + 1) * Ht, :].copy()) for r in range(K)]
    gs = [torch.empty((N, Cin, Ht + 2, W + 2), device="cuda") for _ in range(K)]
    capi.check(capi.conv_bwd_data_tiles(dev(w), dys, gs, N, Cin, Cout, Ht, W, reduced=True), "bwd-data reduced")
    for r in range(K):
        got = host(gs[r])[:, :, 1:-1, :]
        assert rel_err(got, want[:, :, 1 + r * Ht:1 + (r + 1) * Ht, :]) <= 1e-5


def test_forward_and_filter_gradient_vs_oracle(oracle):
    K, N, Cin, Cout, H, W = 4, 2, 6, 10, 5, 12
    rng = np.random.default_rng(4300)
    xs = make_tiles(rng, K, N, Cin, H, W)
    w = he_normal(rng, Cout, Cin)
    dys = [rng.standard_normal((N, Cout, H, W)).astype(np.float32) for _ in range(K)]
    # the oracle exchanges (zeros stand in for the never-written halo rows) and convolves each tile
    ref = [np.nan_to_num(host(x), nan=0.0) for x in xs]
    assert oracle.halo_op(oracle.EXCH, 1, K, 1, W, H, Cin, N, ref) == 0
    want_dw = np.zeros((Cout, Cin, 3, 3), np.float32)
    ys = [torch.empty((N, Cout, H, W), device="cuda") for _ in range(K)]
    capi.check(capi.conv_fwd_tiles(xs, dev(w), ys, N, Cin, Cout, H, W, unexchanged=True), "fwd unexchanged")
    for r in range(K):
        want = np.zeros((N, Cout, H, W), np.float32)
        oracle.conv_slab_fwd(ref[r], w, want)
        assert rel_err(host(ys[r]), want) <= 1e-5
        oracle.conv_slab_bwd_filter(ref[r], dys[r], want_dw, beta=1.0)
    dw = torch.empty((Cout, Cin, 3, 3), device="cuda")
    ws = workspace(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, K, N, Cin, Cout, H, W)
    capi.check(capi.conv_bwd_filter_tiles(xs, [dev(d) for d in dys], dw, N, Cin, Cout, H, W, ws=ws, unexchanged=True),
               "wgrad unexchanged")
    assert rel_err(host(dw), want_dw) <= 1e-5


@pytest.mark.parametrize("K,N,Cin,Cout,H,W", [(2, 1, 64, 64, 12, 64), (4, 1, 16, 32, 6, 22)])
def test_bf16_exchanges_then_convolves(K, N, Cin, Cout, H, W):
    rng = np.random.default_rng(4400 + K)
    xs = make_tiles(rng, K, N, Cin, H, W, dtype=torch.bfloat16)
    w = dev(he_normal(rng, Cout, Cin)).to(torch.bfloat16)
    ws = workspace(capi.ADH_CONV_FWD, capi.ADH_BF16, K, N, Cin, Cout, H, W)
    exchanged = [x.clone() for x in xs]
    capi.check(capi.halo_exchange(exchanged, 1, K, 1, W, H, Cin, N), "exchange")
    want = [torch.empty((N, Cout, H, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.conv_fwd_tiles(exchanged, w, want, N, Cin, Cout, H, W, ws=ws), "fwd")
    got = [torch.empty_like(y) for y in want]
    capi.check(capi.conv_fwd_tiles(xs, w, got, N, Cin, Cout, H, W, ws=ws, unexchanged=True), "fwd unexchanged")
    for r in range(K):
        assert torch.equal(got[r].view(torch.int16), want[r].view(torch.int16))
        assert torch.equal(xs[r].view(torch.int16), exchanged[r].view(torch.int16))  # halo rows were refreshed
