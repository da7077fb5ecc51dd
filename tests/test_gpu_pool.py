"""GPU parity of pooling over the halo-padded slab against the CPU oracle, through the C ABI.

Max pooling moves values: forward is bit-exact in fp32 and bf16.  Average pooling and both
backward passes add a handful of fp32 terms: rel-err max|a-b| / max|b| <= 1e-5 in fp32 and
<= 2^-8 in bf16 (one rounding of the fp32 result to bf16)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu
TOL32, TOL16 = 1e-5, 2.0 ** -8

CASES = [(1, 2, 3, 8, 9, 3, 3, 2, 2), (2, 1, 2, 7, 7, 2, 2, 2, 2), (1, 1, 1, 6, 70, 3, 3, 1, 1), (3, 2, 2, 9, 8, 3, 2, 2, 1),
         (1, 1, 1, 5, 5, 5, 5, 1, 1), (1, 1, 2, 4, 6, 1, 1, 1, 1), (2, 1, 1, 10, 131, 2, 2, 3, 3), (4, 2, 5, 30, 114, 3, 3, 2, 2),
         # several bands of several rows per plane (enough planes that the bands stay tall)
         (1, 8, 64, 64, 200, 3, 3, 2, 2), (1, 8, 64, 61, 203, 2, 2, 2, 2), (1, 4, 64, 40, 150, 5, 3, 1, 2),
         # rows too wide to stage / windows over 256 elements: the direct kernels
         (1, 1, 1, 4, 11000, 3, 3, 1, 1), (1, 1, 2, 20, 21, 17, 17, 1, 2)]


def out_dims(HP, WP, wh, ww, sh, sw):
    return (HP - wh) // sh + 1, (WP - ww) // sw + 1


@pytest.mark.parametrize("mode", [capi.ADH_POOL_AVG, capi.ADH_POOL_MAX])
@pytest.mark.parametrize("K,N,C,HP,WP,wh,ww,sh,sw", CASES)
def test_pool_f32_vs_oracle(oracle, mode, K, N, C, HP, WP, wh, ww, sh, sw):
    rng = np.random.default_rng(31 + WP)
    OH, OW = out_dims(HP, WP, wh, ww, sh, sw)
    xs = [rng.uniform(-1, 1, size=(N, C, HP, WP)).astype(np.float32) for _ in range(K)]
    dys = [rng.standard_normal((N, C, OH, OW)).astype(np.float32) for _ in range(K)]
    dx0 = [rng.standard_normal((N, C, HP, WP)).astype(np.float32) for _ in range(K)]
    d_xs, d_dys = [dev(x) for x in xs], [dev(d) for d in dys]
    ys = [torch.full((N, C, OH, OW), float("nan"), device="cuda") for _ in range(K)]
    capi.check(capi.pool_fwd_tiles(mode, d_xs, ys, N, C, HP, WP, wh, ww, sh, sw))
    gs = [torch.full((N, C, HP, WP), float("nan"), device="cuda") for _ in range(K)]
    capi.check(capi.pool_bwd_tiles(mode, d_xs, ys, d_dys, gs, N, C, HP, WP, wh, ww, sh, sw))
    acc = [dev(a) for a in dx0]
    capi.check(capi.pool_bwd_tiles(mode, d_xs, ys, d_dys, acc, N, C, HP, WP, wh, ww, sh, sw, beta=1.0))
    for r in range(K):
        y = np.empty((N, C, OH, OW), np.float32)
        oracle.pool_slab_fwd(mode, xs[r], wh, ww, sh, sw, y)
        if mode == capi.ADH_POOL_MAX:
            assert np.array_equal(host(ys[r]), y)
        else:
            assert rel_err(host(ys[r]), y) <= TOL32
        g = np.empty((N, C, HP, WP), np.float32)
        oracle.pool_slab_bwd(mode, xs[r], dys[r], wh, ww, sh, sw, g)
        assert rel_err(host(gs[r]), g) <= TOL32
        g1 = dx0[r].copy()
        oracle.pool_slab_bwd(mode, xs[r], dys[r], wh, ww, sh, sw, g1, beta=1.0)
        assert rel_err(host(acc[r]), g1) <= TOL32


@pytest.mark.parametrize("mode", [capi.ADH_POOL_AVG, capi.ADH_POOL_MAX])
@pytest.mark.parametrize("K,N,C,HP,WP,wh,ww,sh,sw", [CASES[0], CASES[3], CASES[6], CASES[7], CASES[8], CASES[9], CASES[11],
                                                     CASES[12]])
def test_pool_bf16_vs_oracle(oracle, mode, K, N, C, HP, WP, wh, ww, sh, sw):
    rng = np.random.default_rng(32 + WP)
    OH, OW = out_dims(HP, WP, wh, ww, sh, sw)
    bf = lambda a: oracle.f32_to_bf16(a.astype(np.float32))
    xs = [bf(rng.uniform(-1, 1, size=(N, C, HP, WP))) for _ in range(K)]
    dys = [bf(rng.standard_normal((N, C, OH, OW))) for _ in range(K)]
    d_xs, d_dys = [dev(x) for x in xs], [dev(d) for d in dys]
    ys = [torch.empty((N, C, OH, OW), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.pool_fwd_tiles(mode, d_xs, ys, N, C, HP, WP, wh, ww, sh, sw))
    gs = [torch.empty((N, C, HP, WP), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.pool_bwd_tiles(mode, d_xs, ys, d_dys, gs, N, C, HP, WP, wh, ww, sh, sw))
    for r in range(K):
        xf, dyf = oracle.bf16_to_f32(xs[r]), oracle.bf16_to_f32(dys[r])
        y = np.empty((N, C, OH, OW), np.float32)
        oracle.pool_slab_fwd(mode, xf, wh, ww, sh, sw, y)
        if mode == capi.ADH_POOL_MAX:
            assert np.array_equal(host(ys[r]), oracle.f32_to_bf16(y))  # a max of bf16 values is one of them
        else:
            assert rel_err(oracle.bf16_to_f32(host(ys[r])), y) <= TOL16
        g = np.empty((N, C, HP, WP), np.float32)
        oracle.pool_slab_bwd(mode, xf, dyf, wh, ww, sh, sw, g)
        assert rel_err(oracle.bf16_to_f32(host(gs[r])), g) <= TOL16


def test_pool_max_ties(oracle):
    # few distinct values: most windows hold their maximum several times; the first one in
    # row-major window order takes the gradient (the oracle's rule)
    rng = np.random.default_rng(33)
    N, C, HP, WP = 2, 3, 12, 70
    x = rng.integers(0, 3, size=(N, C, HP, WP)).astype(np.float32)
    OH, OW = out_dims(HP, WP, 3, 3, 2, 2)
    dy = rng.standard_normal((N, C, OH, OW)).astype(np.float32)
    d_x, d_dy = dev(x), dev(dy)
    y = torch.empty((N, C, OH, OW), device="cuda")
    capi.check(capi.pool_fwd_tiles(capi.ADH_POOL_MAX, [d_x], [y], N, C, HP, WP, 3, 3, 2, 2))
    g = torch.empty((N, C, HP, WP), device="cuda")
    capi.check(capi.pool_bwd_tiles(capi.ADH_POOL_MAX, [d_x], [y], [d_dy], [g], N, C, HP, WP, 3, 3, 2, 2))
    want = np.empty_like(x)
    oracle.pool_slab_bwd(1, x, dy, 3, 3, 2, 2, want)
    assert rel_err(host(g), want) <= TOL32


@pytest.mark.parametrize("mode", [capi.ADH_POOL_AVG, capi.ADH_POOL_MAX])
def test_pool_stitched_vs_unsplit_full_size(mode):
    # the stem pooling of a residual network at full size: N=32, C=64, 112x112 in 4 row-tiles of
    # 28 rows with halo 1, 3x3 window, stride 2 -> 56x56.  Checked against torch's own pooling of
    # the zero-padded unsplit tensor (inputs >= 0, as after a rectifier, so zero padding and
    # cuDNN's -inf padding of the max agree), forward and backward.
    K, N, C, H, W = 4, 32, 64, 28, 112
    g = torch.Generator(device="cuda").manual_seed(9)
    xu = torch.rand((N, C, K * H, W), device="cuda", generator=g)
    tiles = [torch.empty((N, C, H + 2, W + 2), device="cuda") for _ in range(K)]
    capi.check(capi.tiles_pack(K, 1, W, K * H, C, N, xu, tiles))
    OH, OW = out_dims(H + 2, W + 2, 3, 3, 2, 2)
    ys = [torch.empty((N, C, OH, OW), device="cuda") for _ in range(K)]
    capi.check(capi.pool_fwd_tiles(mode, tiles, ys, N, C, H + 2, W + 2, 3, 3, 2, 2))
    xp = F.pad(xu, (1, 1, 1, 1)).requires_grad_(True)
    want = (F.max_pool2d if mode else F.avg_pool2d)(xp, 3, 2)
    got = torch.cat(ys, dim=2)
    assert got.shape == want.shape
    if mode:
        assert torch.equal(got, want.detach())
    else:
        assert float((got - want.detach()).abs().max()) <= 1e-6
    dyu = torch.randn(want.shape, device="cuda", generator=g)
    want.backward(dyu)
    dys = [dyu[:, :, r * OH:(r + 1) * OH].contiguous() for r in range(K)]
    gs = [torch.empty((N, C, H + 2, W + 2), device="cuda") for _ in range(K)]
    capi.check(capi.pool_bwd_tiles(mode, tiles, ys, dys, gs, N, C, H + 2, W + 2, 3, 3, 2, 2))
    # a tile's padded gradient: its own rows plus the halo rows, whose sum over the two
    # neighbouring tiles is what the halo reduction adds back; compare the stitched total
    total = torch.zeros_like(xp)
    for r in range(K):
        total[:, :, r * H:r * H + H + 2] += gs[r]
    assert float((total - xp.grad).abs().max()) <= 1e-5


def test_pool_error_codes():
    x = torch.zeros((1, 1, 6, 6), device="cuda")
    y = torch.zeros((1, 1, 2, 2), device="cuda")
    f = lambda mode, wh, ww, sh, sw: capi.pool_fwd_tiles(mode, [x], [y], 1, 1, 6, 6, wh, ww, sh, sw)
    assert f(capi.ADH_POOL_MAX, 3, 3, 2, 2) == capi.ADH_OK
    assert f(2, 3, 3, 2, 2) == capi.ADH_EINVAL
    assert f(capi.ADH_POOL_MAX, 0, 3, 2, 2) == capi.ADH_EINVAL
    assert f(capi.ADH_POOL_MAX, 3, 3, 0, 2) == capi.ADH_EINVAL
    assert f(capi.ADH_POOL_MAX, 7, 3, 2, 2) == capi.ADH_EINVAL
    L = capi.lib()
    assert L.adh_pool2d_slab_fwd(capi.ADH_F32, 1, 1, 1, 6, 6, 3, 3, 2, 2, None, y.data_ptr(), None) == capi.ADH_ENULL
    assert L.adh_pool2d_slab_fwd(capi.ADH_F32, 1, 1, 1, 6, 6, 3, 3, 2, 2, x.data_ptr() + 2, y.data_ptr(), None) == capi.ADH_EALIGN
    assert L.adh_pool2d_slab_fwd(7, 1, 1, 1, 6, 6, 3, 3, 2, 2, x.data_ptr(), y.data_ptr(), None) == capi.ADH_EINVAL
    assert L.adh_pool2d_slab_bwd(capi.ADH_F32, 1, 1, 1, 6, 6, 3, 3, 2, 2, x.data_ptr(), y.data_ptr(), y.data_ptr(),
                                 x.data_ptr(), 0.5, None) == capi.ADH_EINVAL
    # average backward needs neither x nor y
    dx = torch.empty_like(x)
    assert L.adh_pool2d_slab_bwd(capi.ADH_F32, 0, 1, 1, 6, 6, 3, 3, 2, 2, None, None, y.data_ptr(), dx.data_ptr(),
                                 0.0, None) == capi.ADH_OK
    torch.cuda.synchronize()
    # empty batch is a no-op
    assert L.adh_pool2d_slab_fwd(capi.ADH_F32, 1, 0, 1, 6, 6, 3, 3, 2, 2, None, None, None) == capi.ADH_OK
