"""Pins the data-movement half of the CPU oracle WITHOUT re-using its formulas.

Independent checks used here:
  * numpy slicing / np.pad on (N, C, H, W) arrays (a library routine, no index
    arithmetic of ours) for pad, unpad, slices, scatter/gather;
  * the invariant  pack(X)[r] == zero_pad(X)[rows r*Ht-p .. r*Ht+Ht+p)  which fixes
    the exchange strips (a wrong row, sign or neighbour fails it);
  * the adjoint identity  <E a, b> == <a, R b>  on small-integer floats, which fixes
    halo reduce given exchange;
  * a bijective fill (value == linear index) so that any mis-addressed element shows.
"""
import itertools

import numpy as np
import pytest


def bijective(shape, dtype=np.float32, start=1):
    n = int(np.prod(shape))
    assert n < (1 << 24)
    return (np.arange(n, dtype=np.int64) + start).astype(dtype).reshape(shape)


def np_tiles_from_unsplit(X, K, p):
    N, C, H, W = X.shape
    Ht = H // K
    Xzp = np.pad(X, ((0, 0), (0, 0), (p, p), (p, p)))
    return [np.ascontiguousarray(Xzp[:, :, r * Ht:r * Ht + Ht + 2 * p, :]) for r in range(K)]


def test_padded_index_closed_form(oracle):
    # brute force: position of element in a numpy (N,C,H+2p,W+2p) array
    p, W, H, C, N = 2, 5, 4, 3, 2
    buf = np.arange(N * C * (H + 2 * p) * (W + 2 * p)).reshape(N, C, H + 2 * p, W + 2 * p)
    for n, c, h, w in itertools.product(range(N), range(C), range(-p, H + p), range(-p, W + p)):
        assert oracle.padded_index(w, h, c, n, p, W, H, C) == buf[n, c, h + p, w + p]


def test_bf16_round_trip(oracle):
    rng = np.random.default_rng(0)
    x = rng.standard_normal(4096).astype(np.float32)
    b = oracle.f32_to_bf16(x)
    # scalar C twin agrees with the vectorised numpy one
    import ctypes
    for i in range(0, 4096, 97):
        assert oracle._lib.orc_f32_to_bf16(ctypes.c_float(float(x[i]))) == int(b[i])
    back = oracle.bf16_to_f32(b)
    assert np.all(np.abs(back - x) <= np.abs(x) * 2.0 ** -8)
    # exactly representable values are unchanged, ties go to even
    assert oracle.f32_to_bf16(np.array([1.0, -2.5, 0.0], np.float32)).tolist() == [0x3F80, 0xC020, 0]
    tie = np.array([0x3F808000, 0x3F818000], dtype=np.uint32).view(np.float32)
    assert oracle.f32_to_bf16(tie).tolist() == [0x3F80, 0x3F82]


@pytest.mark.parametrize("K,p,H,W,C,N", [
    (1, 1, 3, 4, 2, 1), (2, 1, 4, 5, 3, 2), (4, 1, 8, 5, 2, 2), (4, 2, 12, 3, 1, 2),
    (3, 1, 6, 4, 2, 1), (8, 1, 16, 6, 2, 1), (2, 3, 6, 7, 2, 2), (4, 3, 12, 4, 3, 1)])
def test_pack_equals_zero_padded_unsplit(oracle, K, p, H, W, C, N):
    X = bijective((N, C, H, W))
    Ht = H // K
    tiles = [np.full((N, C, Ht + 2 * p, W + 2 * p), np.nan, np.float32) for _ in range(K)]
    assert oracle.tiles_pack(K, p, W, H, C, N, X, tiles) == 0
    want = np_tiles_from_unsplit(X, K, p)
    for r in range(K):
        np.testing.assert_array_equal(tiles[r], want[r])


def test_pack_brute_force_all_small(oracle):
    # every (K<=4, p<=3, H<=6 per tile with H>=p, W<=5, C<=3, N<=2) combination, coarse strides
    count = 0
    for K, p, Ht, W, C, N in itertools.product((1, 2, 3, 4), (1, 2, 3), (3, 4, 6), (1, 4, 5), (1, 3), (1, 2)):
        H = K * Ht
        X = bijective((N, C, H, W))
        tiles = [np.full((N, C, Ht + 2 * p, W + 2 * p), -7.0, np.float32) for _ in range(K)]
        assert oracle.tiles_pack(K, p, W, H, C, N, X, tiles) == 0
        want = np_tiles_from_unsplit(X, K, p)
        for r in range(K):
            assert np.array_equal(tiles[r], want[r]), (K, p, Ht, W, C, N, r)
        count += 1
    assert count == 4 * 3 * 3 * 3 * 2 * 2


def test_exchange_touches_only_inner_halo_rows(oracle):
    K, p, Ht, W, C, N = 4, 2, 5, 6, 2, 2
    rng = np.random.default_rng(1)
    tiles = [rng.standard_normal((N, C, Ht + 2 * p, W + 2 * p)).astype(np.float32) for _ in range(K)]
    before = [t.copy() for t in tiles]
    assert oracle.halo_op(oracle.EXCH, 1, K, p, W, Ht, C, N, tiles) == 0
    for r in range(K):
        # interior rows, halo columns everywhere, outer halo rows of the end tiles: unchanged
        np.testing.assert_array_equal(tiles[r][:, :, p:p + Ht, :], before[r][:, :, p:p + Ht, :])
        np.testing.assert_array_equal(tiles[r][:, :, :, :p], before[r][:, :, :, :p])
        np.testing.assert_array_equal(tiles[r][:, :, :, W + p:], before[r][:, :, :, W + p:])
        if r == 0:
            np.testing.assert_array_equal(tiles[r][:, :, :p, :], before[r][:, :, :p, :])
        else:
            np.testing.assert_array_equal(tiles[r][:, :, :p, p:W + p], before[r - 1][:, :, Ht:Ht + p, p:W + p])
        if r == K - 1:
            np.testing.assert_array_equal(tiles[r][:, :, Ht + p:, :], before[r][:, :, Ht + p:, :])
        else:
            np.testing.assert_array_equal(tiles[r][:, :, Ht + p:, p:W + p], before[r + 1][:, :, p:2 * p, p:W + p])


def test_per_rank_calls_compose_to_full_exchange(oracle):
    K, p, Ht, W, C, N = 4, 1, 3, 5, 2, 1
    rng = np.random.default_rng(2)
    a = [rng.standard_normal((N, C, Ht + 2 * p, W + 2 * p)).astype(np.float32) for _ in range(K)]
    b = [t.copy() for t in a]
    oracle.halo_op(oracle.EXCH, 1, K, p, W, Ht, C, N, a)
    for r in reversed(range(K)):  # any rank order gives the same result
        assert oracle.halo_op_rank(oracle.EXCH, 1, K, r, p, W, Ht, C, N, b) == 0
    for r in range(K):
        np.testing.assert_array_equal(a[r], b[r])


@pytest.mark.parametrize("K,p,Ht,W,C,N", [(2, 1, 3, 4, 2, 2), (4, 1, 4, 5, 3, 1), (4, 2, 5, 3, 2, 2), (3, 3, 6, 4, 1, 1)])
def test_reduce_is_adjoint_of_exchange(oracle, K, p, Ht, W, C, N):
    rng = np.random.default_rng(3)
    shape = (N, C, Ht + 2 * p, W + 2 * p)

    def rand_int():
        return [rng.integers(-8, 9, size=shape).astype(np.float32) for _ in range(K)]

    A = rand_int()
    for t in A:  # all halos of A zero
        m = np.zeros(shape, bool)
        m[:, :, p:p + Ht, p:p + W] = True
        t[~m] = 0
    B = rand_int()
    EA = [t.copy() for t in A]
    oracle.halo_op(oracle.EXCH, 1, K, p, W, Ht, C, N, EA)
    RB = [t.copy() for t in B]
    oracle.halo_op(oracle.REDUCE, 1, K, p, W, Ht, C, N, RB)
    lhs = sum(float(np.sum(EA[r].astype(np.float64) * B[r])) for r in range(K))
    rhs = sum(float(np.sum(A[r][:, :, p:p + Ht, p:p + W].astype(np.float64) * RB[r][:, :, p:p + Ht, p:p + W]))
              for r in range(K))
    assert lhs == rhs
    # reduce leaves every halo as it was
    for r in range(K):
        m = np.ones(shape, bool)
        m[:, :, p:p + Ht, p:p + W] = False
        np.testing.assert_array_equal(RB[r][m], B[r][m])


@pytest.mark.parametrize("K,p,H,Wt,C,N", [(2, 1, 4, 3, 2, 2), (3, 2, 3, 5, 1, 2), (4, 1, 2, 4, 3, 1)])
def test_column_reduce_is_adjoint_of_column_exchange(oracle, K, p, H, Wt, C, N):
    """K x 1 grid (column halos): <E a, b> == <a, R b> on small-integer floats, and the closed form
    of the column reduce (right interior columns += next tile's left halo columns, left interior
    columns += previous tile's right halo columns) written with numpy slices."""
    rng = np.random.default_rng(31)
    shape = (N, C, H + 2 * p, Wt + 2 * p)

    def rand_int():
        return [rng.integers(-8, 9, size=shape).astype(np.float32) for _ in range(K)]

    A = rand_int()
    for t in A:
        m = np.zeros(shape, bool)
        m[:, :, p:p + H, p:p + Wt] = True
        t[~m] = 0
    B = rand_int()
    EA = [t.copy() for t in A]
    assert oracle.halo_op(oracle.EXCH, K, 1, p, Wt, H, C, N, EA) == 0
    RB = [t.copy() for t in B]
    assert oracle.halo_op(oracle.REDUCE, K, 1, p, Wt, H, C, N, RB) == 0
    lhs = sum(float(np.sum(EA[r].astype(np.float64) * B[r])) for r in range(K))
    rhs = sum(float(np.sum(A[r][:, :, p:p + H, p:p + Wt].astype(np.float64) * RB[r][:, :, p:p + H, p:p + Wt]))
              for r in range(K))
    assert lhs == rhs
    want = [b.copy() for b in B]
    for r in range(K):
        if r < K - 1:
            want[r][:, :, p:p + H, Wt:Wt + p] += B[r + 1][:, :, p:p + H, 0:p]
        if r > 0:
            want[r][:, :, p:p + H, p:2 * p] += B[r - 1][:, :, p:p + H, Wt + p:Wt + 2 * p]
    for r in range(K):
        np.testing.assert_array_equal(RB[r], want[r])


def test_thread_per_rank_forms_equal_the_serial_ones(oracle):
    """The one-thread-per-rank forms timed as the parallel CPU baseline give the same bits as the loops."""
    K, p, H, W, C, N = 4, 1, 8, 6, 3, 2
    Ht = H // K
    rng = np.random.default_rng(5)
    X = rng.uniform(-1, 1, size=(N, C, H, W)).astype(np.float32)
    a = [np.full((N, C, Ht + 2 * p, W + 2 * p), np.nan, np.float32) for _ in range(K)]
    b = [t.copy() for t in a]
    assert oracle.tiles_pack(K, p, W, H, C, N, X, a) == 0
    assert oracle.tiles_pack_threaded(K, p, W, H, C, N, X, b) == 0
    for r in range(K):
        np.testing.assert_array_equal(a[r], b[r])
    ya, yb = np.empty_like(X), np.empty_like(X)
    assert oracle.tiles_unpack(K, p, W, H, C, N, a, ya) == 0
    assert oracle.tiles_unpack_threaded(K, p, W, H, C, N, b, yb) == 0
    np.testing.assert_array_equal(ya, X)
    np.testing.assert_array_equal(yb, X)
    for which in (oracle.EXCH, oracle.REDUCE):
        ga = [rng.integers(-5, 6, size=a[0].shape).astype(np.float32) for _ in range(K)]
        gb = [t.copy() for t in ga]
        assert oracle.halo_op(which, 1, K, p, W, Ht, C, N, ga) == 0
        assert oracle.halo_op_threaded(which, 1, K, p, W, Ht, C, N, gb) == 0
        for r in range(K):
            np.testing.assert_array_equal(ga[r], gb[r])
    wt = rng.standard_normal((5, C, 3, 3)).astype(np.float32)
    y1 = [np.empty((N, 5, Ht, W), np.float32) for _ in range(K)]
    y2 = [np.empty((N, 5, Ht, W), np.float32) for _ in range(K)]
    for r in range(K):
        oracle.conv_slab_fwd_f32(a[r], wt, y1[r])
    assert oracle.conv_slab_fwd_f32_threaded(a, wt, y2) == 0
    for r in range(K):
        np.testing.assert_array_equal(y1[r], y2[r])
    assert oracle.hardware_threads() >= 1


def test_reduce_closed_form_rows(oracle):
    K, p, Ht, W, C, N = 4, 2, 5, 3, 2, 1
    rng = np.random.default_rng(4)
    G = [rng.integers(-9, 10, size=(N, C, Ht + 2 * p, W + 2 * p)).astype(np.float32) for _ in range(K)]
    want = [g.copy() for g in G]
    for r in range(K):
        if r < K - 1:  # bottom interior rows += next tile's top halo rows
            want[r][:, :, Ht:Ht + p, p:p + W] += G[r + 1][:, :, 0:p, p:p + W]
        if r > 0:      # top interior rows += previous tile's bottom halo rows
            want[r][:, :, p:2 * p, p:p + W] += G[r - 1][:, :, Ht + p:Ht + 2 * p, p:p + W]
    oracle.halo_op(oracle.REDUCE, 1, K, p, W, Ht, C, N, G)
    for r in range(K):
        np.testing.assert_array_equal(G[r], want[r])


def test_column_halo_exchange_kx1(oracle):
    # W-direction split: tiles side by side; check against a zero-padded unsplit tensor
    Kw, p, H, Wt, C, N = 2, 2, 4, 5, 2, 2
    X = bijective((N, C, H, Kw * Wt))
    tiles = []
    for r in range(Kw):
        t = np.zeros((N, C, H + 2 * p, Wt + 2 * p), np.float32)
        t[:, :, p:p + H, p:p + Wt] = X[:, :, :, r * Wt:(r + 1) * Wt]
        tiles.append(t)
    assert oracle.halo_op(oracle.EXCH, Kw, 1, p, Wt, H, C, N, tiles) == 0
    Xzp = np.pad(X, ((0, 0), (0, 0), (p, p), (p, p)))
    for r in range(Kw):
        want = Xzp[:, :, :, r * Wt:r * Wt + Wt + 2 * p].copy()
        want[:, :, :p, :] = 0   # halo rows are not exchanged by the column kernel
        want[:, :, H + p:, :] = 0
        np.testing.assert_array_equal(tiles[r], want)


def test_grid_dispatch_errors(oracle):
    t = [np.zeros((1, 1, 4, 4), np.float32) for _ in range(4)]
    assert oracle.halo_op(oracle.EXCH, 2, 2, 1, 2, 2, 1, 1, t) == -2      # 2x2: unimplemented
    assert oracle.halo_op(oracle.EXCH, 1, 1, 1, 2, 2, 1, 1, t[:1]) == 0    # 1x1: no-op
    assert oracle.halo_op(oracle.EXCH, 1, 2, 1, 2, 2, 1, 1, [t[0], None]) == -1  # NULL buffer


@pytest.mark.parametrize("dtype", [np.float32, np.uint16])
def test_slice_copy_matches_numpy(oracle, dtype):
    N, C, H, W = 2, 5, 7, 6
    src = bijective((N, C, H, W), np.float32)
    if dtype == np.uint16:
        src = (src.astype(np.int64) % 65521).astype(np.uint16)
    dst = np.zeros((N, 4, 5, 9), dtype)
    want = dst.copy()
    want[:, 1:4, 2:5, 3:8] = src[:, 2:5, 4:7, 1:6]
    assert oracle.slice_nchw(oracle.OP_COPY, (5, 3, 3), N, src, (W, H, C), (1, 4, 2), dst, (9, 5, 4), (3, 2, 1)) == 0
    np.testing.assert_array_equal(dst, want)
    # out-of-bounds window is rejected (slice.cu:61-64)
    assert oracle.slice_nchw(oracle.OP_COPY, (6, 3, 3), N, src, (W, H, C), (1, 4, 2), dst, (9, 5, 4), (3, 2, 1)) == -1


def test_slice_add_and_channel_slice(oracle):
    rng = np.random.default_rng(5)
    N, C, H, W = 2, 8, 4, 5
    x = rng.integers(-50, 50, size=(N, C, H, W)).astype(np.float32)
    y = rng.integers(-50, 50, size=(N, 3, H, W)).astype(np.float32)
    want = y + x[:, 2:5]
    assert oracle.slice_nchw(oracle.OP_ADD, (W, H, 3), N, x, (W, H, C), (0, 0, 2), y, (W, H, 3), (0, 0, 0)) == 0
    np.testing.assert_array_equal(y, want)


def test_bf16_add_rounds_to_nearest_even(oracle):
    rng = np.random.default_rng(6)
    a = oracle.f32_to_bf16(rng.standard_normal((1, 2, 3, 4)).astype(np.float32))
    b = oracle.f32_to_bf16(rng.standard_normal((1, 2, 3, 4)).astype(np.float32))
    want = oracle.f32_to_bf16(oracle.bf16_to_f32(a) + oracle.bf16_to_f32(b))
    y = b.copy()
    oracle.slice_nchw(oracle.OP_ADD, (4, 3, 2), 1, a, (4, 3, 2), (0, 0, 0), y, (4, 3, 2), (0, 0, 0))
    np.testing.assert_array_equal(y, want)


@pytest.mark.parametrize("p", [1, 2, 3])
def test_pad_unpad_match_numpy(oracle, p):
    N, C, H, W = 2, 3, 4, 5
    x = bijective((N, C, H, W))
    y = np.full((N, C, H + 2 * p, W + 2 * p), np.nan, np.float32)
    oracle.halo_pad(p, W, H, C, N, x, y)
    np.testing.assert_array_equal(y, np.pad(x, ((0, 0), (0, 0), (p, p), (p, p))))
    z = np.empty_like(x)
    y[:, :, :p] = np.nan  # unpad must ignore the halo
    y[:, :, :, :p] = np.nan
    oracle.halo_unpad(p, W, H, C, N, y, z)
    np.testing.assert_array_equal(z, x)
    g = bijective((N, C, H + 2 * p, W + 2 * p))
    acc = x.copy()
    oracle.halo_unpad_add(p, W, H, C, N, g, acc)
    np.testing.assert_array_equal(acc, x + g[:, :, p:p + H, p:p + W])
    acc2 = g.copy()
    oracle.halo_pad_add(p, W, H, C, N, x, acc2)
    want = g.copy()
    want[:, :, p:p + H, p:p + W] += x
    np.testing.assert_array_equal(acc2, want)
    q = 4 - p
    rp = np.full((N, C, H + 2 * q, W + 2 * q), np.nan, np.float32)
    clean = np.pad(x, ((0, 0), (0, 0), (p, p), (p, p)))
    oracle.halo_repad(p, q, W, H, C, N, clean, rp)
    np.testing.assert_array_equal(rp, np.pad(x, ((0, 0), (0, 0), (q, q), (q, q))))


def test_unpack_inverts_pack_and_ignores_halos(oracle):
    K, p, H, W, C, N = 4, 1, 8, 6, 3, 2
    rng = np.random.default_rng(7)
    X = rng.standard_normal((N, C, H, W)).astype(np.float32)
    Ht = H // K
    tiles = [np.empty((N, C, Ht + 2 * p, W + 2 * p), np.float32) for _ in range(K)]
    oracle.tiles_pack(K, p, W, H, C, N, X, tiles)
    for t in tiles:  # poison halos
        t[:, :, :p] = np.nan
        t[:, :, Ht + p:] = np.nan
        t[:, :, :, :p] = np.nan
        t[:, :, :, W + p:] = np.nan
    Y = np.empty_like(X)
    assert oracle.tiles_unpack(K, p, W, H, C, N, tiles, Y) == 0
    np.testing.assert_array_equal(Y, X)
    assert oracle.tiles_pack(3, p, W, H, C, N, X, tiles[:3]) == -1  # H % K != 0 (op.cc:2385)


def test_fill_add(oracle):
    x = np.arange(10, dtype=np.float32)
    y = np.ones(10, np.float32)
    oracle.add_f32(x, y)
    np.testing.assert_array_equal(y, x + 1)
    oracle.fill_f32(y, 3.5)
    assert np.all(y == 3.5)
