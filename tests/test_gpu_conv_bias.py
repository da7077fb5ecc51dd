"""GPU parity of the convolution bias (y += bias per channel after the conv; db = beta*db + sum of dy
over tiles, images and pixels) against the CPU oracle, through the C ABI.  The add is one fp32 sum per
element: bit-exact in fp32, and in bf16 equal to the oracle's sum rounded once.  The gradient is a sum
of up to millions of terms in another order than the oracle's: |a-b| <= 1e-5 * sum|dy| per channel
(fp32 and bf16 alike, the terms are widened exactly), and identical bits on a second call."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host

pytestmark = pytest.mark.gpu

# K, N, C, H, W: planes that are / are not whole 16-byte groups, one tile, the stem's tiles (64 x 256) at
# a reduced batch, more channels than workgroup splits, one pixel
CASES = [(1, 2, 3, 4, 8), (2, 3, 5, 3, 5), (4, 2, 64, 14, 56), (4, 4, 64, 64, 256), (3, 1, 1200, 2, 2), (2, 5, 7, 1, 1),
         (1, 1, 1, 1, 3)]


@pytest.mark.parametrize("K,N,C,H,W", CASES)
@pytest.mark.parametrize("bf16", [False, True])
def test_conv_bias_add_vs_oracle(oracle, K, N, C, H, W, bf16):
    rng = np.random.default_rng(300 + C + W)
    ys = [rng.uniform(-1, 1, (N, C, H, W)).astype(np.float32) for _ in range(K)]
    bs = [rng.uniform(-1, 1, C).astype(np.float32) for _ in range(K)]
    if bf16:
        ys = [oracle.bf16_to_f32(oracle.f32_to_bf16(y)) for y in ys]
    d_ys = [dev(oracle.f32_to_bf16(y)) if bf16 else dev(y) for y in ys]
    d_bs = [dev(b) for b in bs]
    capi.check(capi.conv_bias_add_tiles(d_bs, d_ys, N, C, H, W), "bias add")
    for t in range(K):
        want = ys[t].copy()
        oracle.conv_bias_add(bs[t], want)
        got = host(d_ys[t])
        if bf16:
            assert np.array_equal(got, oracle.f32_to_bf16(want))
        else:
            assert np.array_equal(got, want)
    # one shared vector for every tile (replicated parameters)
    d_ys = [dev(oracle.f32_to_bf16(y)) if bf16 else dev(y) for y in ys]
    capi.check(capi.conv_bias_add_tiles([d_bs[0]] * K, d_ys, N, C, H, W), "bias add (shared)")
    want = ys[K - 1].copy()
    oracle.conv_bias_add(bs[0], want)
    got = host(d_ys[K - 1])
    assert np.array_equal(got, oracle.f32_to_bf16(want) if bf16 else want)


@pytest.mark.parametrize("K,N,C,H,W", CASES)
@pytest.mark.parametrize("bf16", [False, True])
def test_conv_bwd_bias_vs_oracle(oracle, K, N, C, H, W, bf16):
    rng = np.random.default_rng(400 + C + W)
    dys = [rng.standard_normal((N, C, H, W)).astype(np.float32) for _ in range(K)]
    if bf16:
        dys = [oracle.bf16_to_f32(oracle.f32_to_bf16(d)) for d in dys]
    d_dys = [dev(oracle.f32_to_bf16(d)) if bf16 else dev(d) for d in dys]
    db0 = rng.standard_normal(C).astype(np.float32)
    nbytes = capi.conv_bwd_bias_workspace_bytes(K, N, C)
    ws = torch.full((nbytes // 4 + 64,), float("nan"), device="cuda")
    want = np.zeros(C, np.float32)
    for t in range(K):
        oracle.conv_bwd_bias(dys[t], want, beta=1.0 if t else 0.0)
    scale = sum(np.abs(d).astype(np.float64).sum(axis=(0, 2, 3)) for d in dys)
    db = torch.full((C,), float("nan"), device="cuda")
    capi.check(capi.conv_bwd_bias_tiles(d_dys, db, N, C, H, W, beta=0.0, ws=ws), "bwd bias")
    got = host(db)
    assert np.all(np.abs(got.astype(np.float64) - want) <= 1e-5 * scale + 1e-30)
    db2 = torch.full((C,), float("nan"), device="cuda")
    capi.check(capi.conv_bwd_bias_tiles(d_dys, db2, N, C, H, W, beta=0.0, ws=ws), "bwd bias (again)")
    assert np.array_equal(host(db2), got)
    acc = dev(db0)
    capi.check(capi.conv_bwd_bias_tiles(d_dys, acc, N, C, H, W, beta=1.0, ws=ws), "bwd bias (beta 1)")
    assert np.all(np.abs(host(acc).astype(np.float64) - (want.astype(np.float64) + db0)) <= 1e-5 * scale + 1e-6)


def test_conv_bias_argument_errors():
    y = torch.zeros((1, 2, 2, 2), device="cuda")
    b = torch.zeros(2, device="cuda")
    db = torch.zeros(2, device="cuda")
    ws = torch.zeros(1024, device="cuda")
    small = torch.zeros(1, device="cuda")
    L = capi.lib()
    yt, k1 = capi.ptr_table([y.data_ptr()])
    bt, k2 = capi.ptr_table([b.data_ptr()])
    nul, k3 = capi.ptr_table([None])
    assert L.adh_conv_bias_add_tiles(capi.ADH_F32, 1, 1, 2, 2, 2, nul, yt, None) == capi.ADH_ENULL
    assert L.adh_conv_bias_add_tiles(capi.ADH_F32, 0, 1, 2, 2, 2, bt, yt, None) == capi.ADH_EINVAL
    assert L.adh_conv_bias_add_tiles(7, 1, 1, 2, 2, 2, bt, yt, None) == capi.ADH_EINVAL
    assert L.adh_conv_bwd_bias_tiles(capi.ADH_F32, 1, 1, 2, 2, 2, yt, db.data_ptr(), 0.5, ws.data_ptr(), 4096, None) == capi.ADH_EINVAL
    assert L.adh_conv_bwd_bias_tiles(capi.ADH_F32, 1, 1, 2, 2, 2, yt, db.data_ptr(), 0.0, small.data_ptr(), 4, None) == capi.ADH_EWORKSPACE
    assert L.adh_conv_bwd_bias_tiles(capi.ADH_F32, 1, 1, 2, 2, 2, nul, db.data_ptr(), 0.0, ws.data_ptr(), 4096, None) == capi.ADH_ENULL
    torch.cuda.synchronize()


# K, N, Cin, Cout, HP, WP, kh, kw, sh, sw: the stem's shapes (at most three input channels: the bias goes into the
# convolution's stores; 16-byte and element-wise stores, a channel remainder) and one the general kernel serves
# (the add follows the convolution inside the library)
FUSED_CASES = [(2, 2, 3, 64, 22, 70, 7, 7, 1, 1), (3, 2, 3, 70, 14, 45, 7, 7, 1, 1), (2, 3, 1, 20, 19, 71, 3, 3, 2, 2),
               (2, 2, 3, 64, 20, 38, 7, 7, 2, 2), (2, 2, 16, 24, 10, 30, 3, 3, 2, 2)]


@pytest.mark.parametrize("K,N,Cin,Cout,HP,WP,kh,kw,sh,sw", FUSED_CASES)
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_conv_fwd_with_bias_equals_conv_then_bias(K, N, Cin, Cout, HP, WP, kh, kw, sh, sw, beta):
    """adh_conv2d_slab_fwd_bias_tiles has the bits of adh_conv2d_slab_fwd_tiles followed by adh_conv_bias_add_tiles
    (which the tests above and tests/test_gpu_conv_generic.py hold against the oracle)."""
    rng = np.random.default_rng(500 + Cout + WP)
    OH, OW = (HP - kh) // sh + 1, (WP - kw) // sw + 1
    xs = [dev(rng.uniform(-1, 1, (N, Cin, HP, WP)).astype(np.float32)) for _ in range(K)]
    w = dev((rng.standard_normal((Cout, Cin, kh, kw)) * 0.1).astype(np.float32))
    bs = [dev(rng.uniform(-1, 1, Cout).astype(np.float32)) for _ in range(K)]
    y0 = [rng.standard_normal((N, Cout, OH, OW)).astype(np.float32) for _ in range(K)]
    nbytes = capi.lib().adh_conv2d_workspace_bytes(capi.ADH_CONV_FWD, capi.ADH_F32, K, N, Cin, Cout, HP, WP, kh, kw, sh, sw, 1, 1)
    ws = torch.empty(nbytes // 4 + 64, device="cuda")
    want = [dev(a) for a in y0]
    capi.check(capi.conv2d_fwd_tiles(xs, w, want, N, Cin, Cout, HP, WP, kh, kw, sh, sw, 1, 1, beta=beta, ws=ws), "conv")
    capi.check(capi.conv_bias_add_tiles(bs, want, N, Cout, OH, OW), "bias")
    got = [dev(a) for a in y0]
    capi.check(capi.conv2d_fwd_bias_tiles(xs, w, bs, got, N, Cin, Cout, HP, WP, kh, kw, sh, sw, 1, 1, beta=beta, ws=ws), "conv + bias")
    for t in range(K):
        assert np.array_equal(host(got[t]), host(want[t]))
    # the bias took part: the result differs from the convolution alone wherever the bias is not zero
    plain = [dev(a) for a in y0]
    capi.check(capi.conv2d_fwd_tiles(xs, w, plain, N, Cin, Cout, HP, WP, kh, kw, sh, sw, 1, 1, beta=beta, ws=ws), "conv")
    assert not np.array_equal(host(got[0]), host(plain[0]))


def test_conv_fwd_with_bias_argument_errors():
    x = torch.zeros((1, 3, 9, 9), device="cuda")
    w = torch.zeros((4, 3, 3, 3), device="cuda")
    y = torch.zeros((1, 4, 7, 7), device="cuda")
    b = torch.zeros(4, device="cuda")
    ws = torch.zeros(1 << 16, device="cuda")
    L = capi.lib()
    xt, k1 = capi.ptr_table([x.data_ptr()])
    yt, k2 = capi.ptr_table([y.data_ptr()])
    bt, k3 = capi.ptr_table([b.data_ptr()])
    nul, k4 = capi.ptr_table([None])
    args = (capi.ADH_F32, 1, 1, 3, 4, 9, 9, 3, 3, 1, 1, 1, 1, xt, w.data_ptr())
    tail = (yt, 0.0, ws.data_ptr(), ws.numel() * 4, None)
    assert L.adh_conv2d_slab_fwd_bias_tiles(*args, None, *tail) == capi.ADH_ENULL
    assert L.adh_conv2d_slab_fwd_bias_tiles(*args, nul, *tail) == capi.ADH_ENULL
    assert L.adh_conv2d_slab_fwd_bias_tiles(*args, bt, *tail) == capi.ADH_OK
    torch.cuda.synchronize()
