"""GPU parity of the data-movement kernels against the CPU oracle: bit-exact.

Every call goes through the C ABI (arraydiff_cuda_amd.capi -> libadh.so)."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host

pytestmark = pytest.mark.gpu


def rand_tiles(rng, K, N, C, PH, PW, dtype):
    if dtype == np.float32:
        return [rng.standard_normal((N, C, PH, PW)).astype(np.float32) for _ in range(K)]
    return [rng.integers(0, 0x7F00, size=(N, C, PH, PW)).astype(np.uint16) for _ in range(K)]


SHAPES = [  # K, p, Ht, W, C, N
    (1, 1, 3, 4, 2, 1), (2, 1, 4, 5, 3, 2), (4, 1, 14, 56, 8, 3), (4, 2, 5, 7, 3, 2), (8, 1, 4, 6, 2, 2),
    (3, 3, 6, 9, 2, 1), (16, 1, 2, 3, 1, 1), (4, 1, 3, 62, 5, 2),
    # rows of 512 and more elements
    (2, 1, 3, 520, 3, 2), (3, 2, 4, 517, 2, 1), (1, 3, 5, 1030, 1, 2)]


@pytest.mark.parametrize("dtype", [np.float32, np.uint16])
@pytest.mark.parametrize("K,p,Ht,W,C,N", SHAPES)
def test_pack_unpack_vs_oracle(oracle, K, p, Ht, W, C, N, dtype):
    rng = np.random.default_rng(100 + K + p)
    H = K * Ht
    if dtype == np.float32:
        X = rng.uniform(-1, 1, size=(N, C, H, W)).astype(np.float32)
    else:
        X = oracle.f32_to_bf16(rng.uniform(-1, 1, size=(N, C, H, W)).astype(np.float32))
    want = [np.empty((N, C, Ht + 2 * p, W + 2 * p), dtype) for _ in range(K)]
    assert oracle.tiles_pack(K, p, W, H, C, N, X, want) == 0
    dX = dev(X)
    tiles = [dev(np.full((N, C, Ht + 2 * p, W + 2 * p), 0x7FC0 if dtype == np.uint16 else np.nan, dtype))
             for _ in range(K)]
    capi.check(capi.tiles_pack(K, p, W, H, C, N, dX, tiles), "pack")
    for r in range(K):
        np.testing.assert_array_equal(host(tiles[r]), want[r])
    # unpack ignores halo contents
    for t in tiles:
        t[:, :, :p] = float("nan")
        t[:, :, :, :p] = float("nan")
        t[:, :, Ht + p:] = float("nan")
        t[:, :, :, W + p:] = float("nan")
    Y = torch.empty_like(dX)
    capi.check(capi.tiles_unpack(K, p, W, H, C, N, tiles, Y), "unpack")
    np.testing.assert_array_equal(host(Y), X)


@pytest.mark.parametrize("dtype", [np.float32, np.uint16])
@pytest.mark.parametrize("K,p,Ht,W,C,N", SHAPES[1:])
@pytest.mark.parametrize("which", ["exch", "reduce"])
def test_halo_exchange_reduce_vs_oracle(oracle, K, p, Ht, W, C, N, dtype, which):
    if which == "reduce" and Ht < 2 * p:
        pytest.skip("reduce needs H >= 2p")
    rng = np.random.default_rng(200 + K)
    tiles = rand_tiles(rng, K, N, C, Ht + 2 * p, W + 2 * p, dtype)
    want = [t.copy() for t in tiles]
    code = oracle.EXCH if which == "exch" else oracle.REDUCE
    assert oracle.halo_op(code, 1, K, p, W, Ht, C, N, want) == 0
    fn = capi.halo_exchange if which == "exch" else capi.halo_reduce
    d = [dev(t) for t in tiles]
    capi.check(fn(d, 1, K, p, W, Ht, C, N), which)
    for r in range(K):
        np.testing.assert_array_equal(host(d[r]), want[r])
    # per-rank launches (the reference's call shape) compose to the same result
    d2 = [dev(t) for t in tiles]
    for r in range(K):
        capi.check(fn(d2, 1, K, p, W, Ht, C, N, rank=r), which + " rank")
    for r in range(K):
        np.testing.assert_array_equal(host(d2[r]), want[r])


# a reduce over a halo of two or more columns runs the LDS-staged kernel (planes of up to 48 KB), every other
# case the direct one: (2, 2, ...), (2, 3, ...) and (3, 2, ...) cover the former, the 200-row planes exceed 48 KB
@pytest.mark.parametrize("dtype", [np.float32, np.uint16])
@pytest.mark.parametrize("which", ["exch", "reduce"])
@pytest.mark.parametrize("Kw,p,H,Wt,C,N", [(2, 1, 5, 4, 3, 2), (2, 2, 6, 7, 2, 2), (4, 1, 3, 5, 2, 1), (2, 3, 9, 64, 4, 2),
                                           (3, 2, 33, 14, 5, 3), (2, 2, 200, 60, 2, 1)])
def test_column_halos_vs_oracle(oracle, Kw, p, H, Wt, C, N, which, dtype):
    rng = np.random.default_rng(300)
    tiles = rand_tiles(rng, Kw, N, C, H + 2 * p, Wt + 2 * p, dtype)
    want = [t.copy() for t in tiles]
    code = oracle.EXCH if which == "exch" else oracle.REDUCE
    assert oracle.halo_op(code, Kw, 1, p, Wt, H, C, N, want) == 0
    fn = capi.halo_exchange if which == "exch" else capi.halo_reduce
    d = [dev(t) for t in tiles]
    capi.check(fn(d, Kw, 1, p, Wt, H, C, N), which)
    for r in range(Kw):
        np.testing.assert_array_equal(host(d[r]), want[r])


def test_halo_error_codes(oracle):
    t = [torch.zeros(1, 1, 4, 4, device="cuda") for _ in range(4)]
    assert capi.halo_exchange(t, 2, 2, 1, 2, 2, 1, 1) == capi.ADH_EUNIMPL
    assert capi.halo_exchange(t[:1], 1, 1, 1, 2, 2, 1, 1) == capi.ADH_OK
    tb, keep = capi.ptr_table([t[0].data_ptr(), None])
    assert capi.lib().adh_halo_exchange_nchw(0, 1, 2, 1, 2, 2, 1, 1, tb, None) == capi.ADH_ENULL
    assert capi.halo_reduce(t[:2], 1, 2, 2, 2, 2, 1, 1) == capi.ADH_EINVAL  # H < 2p
    assert capi.tiles_pack(3, 1, 2, 8, 1, 1, t[0], t[:3]) == capi.ADH_EINVAL  # H % K


@pytest.mark.parametrize("dtype", [np.float32, np.uint16])
@pytest.mark.parametrize("p,W,H,C,N", [(1, 5, 4, 3, 2), (2, 56, 14, 4, 2), (3, 7, 9, 2, 1), (1, 62, 3, 2, 2)])
def test_pad_unpad_repad_vs_oracle(oracle, p, W, H, C, N, dtype):
    rng = np.random.default_rng(400)
    mk = (lambda s: rng.standard_normal(s).astype(np.float32)) if dtype == np.float32 else \
        (lambda s: oracle.f32_to_bf16(rng.standard_normal(s).astype(np.float32)))
    x = mk((N, C, H, W))
    g = mk((N, C, H + 2 * p, W + 2 * p))
    # pad
    want = np.empty_like(g)
    oracle.halo_pad(p, W, H, C, N, x, want)
    y = dev(g)
    capi.check(capi.halo_pad(p, W, H, C, N, dev(x), y))
    np.testing.assert_array_equal(host(y), want)
    # unpad
    want = np.empty_like(x)
    oracle.halo_unpad(p, W, H, C, N, g, want)
    y = dev(x)
    capi.check(capi.halo_unpad(p, W, H, C, N, dev(g), y))
    np.testing.assert_array_equal(host(y), want)
    # pad_add / unpad_add
    want = g.copy()
    oracle.halo_pad_add(p, W, H, C, N, x, want)
    y = dev(g)
    capi.check(capi.halo_pad_add(p, W, H, C, N, dev(x), y))
    np.testing.assert_array_equal(host(y), want)
    want = x.copy()
    oracle.halo_unpad_add(p, W, H, C, N, g, want)
    y = dev(x)
    capi.check(capi.halo_unpad_add(p, W, H, C, N, dev(g), y))
    np.testing.assert_array_equal(host(y), want)
    # repad p -> q
    q = 4 - p
    want = np.empty((N, C, H + 2 * q, W + 2 * q), dtype)
    oracle.halo_repad(p, q, W, H, C, N, g, want)
    y = dev(np.zeros_like(want))
    y.fill_(1.0)
    capi.check(capi.halo_repad(p, q, W, H, C, N, dev(g), y))
    np.testing.assert_array_equal(host(y), want)


@pytest.mark.parametrize("dtype", [np.float32, np.uint16])
def test_slices_vs_oracle(oracle, dtype):
    rng = np.random.default_rng(500)
    mk = (lambda s: rng.standard_normal(s).astype(np.float32)) if dtype == np.float32 else \
        (lambda s: oracle.f32_to_bf16(rng.standard_normal(s).astype(np.float32)))
    N, C, H, W = 2, 6, 9, 11
    src = mk((N, C, H, W))
    dst = mk((N, 4, 7, 13))
    for add in (False, True):
        # partial window
        want = dst.copy()
        args = ((5, 3, 3), N, src, (W, H, C), (1, 4, 2), want, (13, 7, 4), (3, 2, 1))
        assert oracle.slice_nchw(oracle.OP_ADD if add else oracle.OP_COPY, *args) == 0
        d = dev(dst)
        capi.check(capi.slice_nchw(add, (5, 3, 3), N, dev(src), (W, H, C), (1, 4, 2), d, (13, 7, 4), (3, 2, 1)))
        np.testing.assert_array_equal(host(d), want)
    # scatter of rows (the reference's use: SpatialScatter2DOp) and its gather
    K, Ht = 3, 3
    for r in range(K):
        tile = np.empty((N, C, Ht, W), dtype)
        oracle.slice_nchw(oracle.OP_COPY, (W, Ht, C), N, src, (W, H, C), (0, r * Ht, 0), tile, (W, Ht, C), (0, 0, 0))
        d = dev(np.zeros_like(tile))
        capi.check(capi.slice_nchw(False, (W, Ht, C), N, dev(src), (W, H, C), (0, r * Ht, 0), d, (W, Ht, C), (0, 0, 0)))
        np.testing.assert_array_equal(host(d), tile)
    # out-of-bounds window
    d = dev(dst)
    assert capi.slice_nchw(False, (12, 3, 3), N, dev(src), (W, H, C), (0, 0, 0), d, (13, 7, 4), (0, 0, 0)) == capi.ADH_EINVAL


def test_channel_slice_full_size(oracle):
    # channels [16,48) of N=32, C=64, 56x56 fp32, and its backward (+=)
    rng = np.random.default_rng(501)
    N, C, H, W = 32, 64, 56, 56
    x = rng.uniform(-1, 1, size=(N, C, H, W)).astype(np.float32)
    y = torch.full((N, 32, H, W), float("nan"), device="cuda")
    dx = dev(x)
    capi.check(capi.slice_nchw(False, (W, H, 32), N, dx, (W, H, C), (0, 0, 16), y, (W, H, 32), (0, 0, 0)))
    np.testing.assert_array_equal(host(y), x[:, 16:48])
    g = dev(x)
    capi.check(capi.slice_nchw(True, (W, H, 32), N, y, (W, H, 32), (0, 0, 0), g, (W, H, C), (0, 0, 16)))
    want = x.copy()
    want[:, 16:48] += x[:, 16:48]
    np.testing.assert_array_equal(host(g), want)


def test_config1_pack_full_size(oracle):
    # fp32 N=32, C=64, 56x56, 4 tiles of 14 rows, halo 1: bit-exact vs the zero-padded unsplit tensor
    rng = np.random.default_rng(0x5EED)
    N, C, H, W, K, p = 32, 64, 56, 56, 4, 1
    Ht = H // K
    X = rng.uniform(-1, 1, size=(N, C, H, W)).astype(np.float32)
    dX = dev(X)
    tiles = [torch.full((N, C, Ht + 2, W + 2), float("nan"), device="cuda") for _ in range(K)]
    capi.check(capi.tiles_pack(K, p, W, H, C, N, dX, tiles))
    Xzp = np.pad(X, ((0, 0), (0, 0), (p, p), (p, p)))
    for r in range(K):
        np.testing.assert_array_equal(host(tiles[r]), Xzp[:, :, r * Ht:r * Ht + Ht + 2 * p])
    # oracle agrees on one tile at full size
    want = [np.empty((N, C, Ht + 2, W + 2), np.float32) for _ in range(K)]
    oracle.tiles_pack(K, p, W, H, C, N, X, want)
    np.testing.assert_array_equal(host(tiles[2]), want[2])
    # pad -> exchange (the unfused sequence) gives the same tiles
    t2 = []
    for r in range(K):
        t = torch.full((N, C, Ht + 2, W + 2), float("nan"), device="cuda")
        xs = torch.empty((N, C, Ht, W), device="cuda")
        capi.check(capi.slice_nchw(False, (W, Ht, C), N, dX, (W, H, C), (0, r * Ht, 0), xs, (W, Ht, C), (0, 0, 0)))
        capi.check(capi.halo_pad(p, W, Ht, C, N, xs, t))
        t2.append(t)
    capi.check(capi.halo_exchange(t2, 1, K, p, W, Ht, C, N))
    for r in range(K):
        assert torch.equal(t2[r], tiles[r])
    Y = torch.empty_like(dX)
    capi.check(capi.tiles_unpack(K, p, W, H, C, N, tiles, Y))
    assert torch.equal(Y, dX)


def test_config5_size_round_trip_bf16():
    # bf16 N=2, C=64, 1024x2048, 8 tiles of 128 rows + halo 1: size-independent properties
    N, C, H, W, K, p = 2, 64, 1024, 2048, 8, 1
    Ht = H // K
    g = torch.Generator(device="cuda").manual_seed(5)
    X = (torch.rand((N, C, H, W), device="cuda", generator=g) * 2 - 1).to(torch.bfloat16)
    tiles = [torch.full((N, C, Ht + 2, W + 2), float("nan"), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    capi.check(capi.tiles_pack(K, p, W, H, C, N, X, tiles))
    for r in (0, 3, 7):
        t = tiles[r]
        assert torch.equal(t[:, :, p:p + Ht, p:p + W], X[:, :, r * Ht:(r + 1) * Ht])
        assert torch.count_nonzero(t[:, :, :, 0]) == 0 and torch.count_nonzero(t[:, :, :, W + 1]) == 0
        if r > 0:
            assert torch.equal(t[:, :, 0, p:p + W], X[:, :, r * Ht - 1])
        else:
            assert torch.count_nonzero(t[:, :, 0]) == 0
        if r < K - 1:
            assert torch.equal(t[:, :, Ht + 1, p:p + W], X[:, :, (r + 1) * Ht])
        else:
            assert torch.count_nonzero(t[:, :, Ht + 1]) == 0
    Y = torch.empty_like(X)
    capi.check(capi.tiles_unpack(K, p, W, H, C, N, tiles, Y))
    assert torch.equal(Y, X)
    # exchange is idempotent on packed tiles
    before = [t.clone() for t in tiles[:2]]
    capi.check(capi.halo_exchange(tiles, 1, K, p, W, Ht, C, N))
    assert torch.equal(tiles[0], before[0]) and torch.equal(tiles[1], before[1])


def test_fill_add(oracle):
    for n in (1, 5, 1024, 100003):
        x = torch.randn(n + 1, device="cuda")
        y = torch.randn(n + 1, device="cuda")
        for off in (0, 1):  # aligned and misaligned base
            xs, ys = x[off:off + n], y[off:off + n]
            want = host(xs) + host(ys)
            capi.check(capi.lib().adh_add_f32(n, xs.data_ptr(), ys.data_ptr(), None))
            np.testing.assert_array_equal(host(ys), want)
            capi.check(capi.lib().adh_fill_f32(n, 2.5, xs.data_ptr(), None))
            assert bool((xs == 2.5).all())
