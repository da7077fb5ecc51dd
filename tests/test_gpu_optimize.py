"""GPU parity of the flat-vector copies and the fused SGD update against the CPU oracle, through the
C ABI.  Everything here is bit-exact: the copies move bytes, and the update's arithmetic is fixed to
one fused multiply-add per axpy in both the kernel and the oracle."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


@pytest.mark.parametrize("n,shift", [(1, 0), (5, 0), (1024, 0), (4099, 0), (1 << 20, 0), (777, 1), (4096, 3)])
def test_scale_add_and_online_bit_exact(oracle, n, shift):
    rng = np.random.default_rng(n + shift)
    x, y0 = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    # `shift` moves the device views off 16-byte alignment (scalar kernel path)
    bx, by = torch.zeros(n + 8, device="cuda"), torch.zeros(n + 8, device="cuda")
    dx, dy = bx[shift:shift + n], by[shift:shift + n]
    for alpha, beta in [(0.25, -1.5), (1.0, 0.9), (-0.1, 1.0)]:
        dx.copy_(dev(x)); dy.copy_(dev(y0))
        capi.check(capi.scale_add(alpha, dx, beta, dy))
        want = y0.copy()
        oracle.array_add_scaled(alpha, x, beta, want)
        np.testing.assert_array_equal(bits(host(dy)), bits(want))
    dy.copy_(dev(y0))
    capi.check(capi.add_online(0.003, dx, dy))
    want = y0.copy()
    oracle.array_add_online(0.003, x, want)
    np.testing.assert_array_equal(bits(host(dy)), bits(want))
    run, stat = dev(y0), torch.full((n,), float("nan"), device="cuda")
    capi.check(capi.stat_step(0.01, dx.contiguous(), run, stat))
    w_run, w_stat = y0.copy(), np.empty(n, np.float32)
    oracle.stat_step(0.01, x, w_run, w_stat)
    np.testing.assert_array_equal(bits(host(run)), bits(w_run))
    np.testing.assert_array_equal(bits(host(stat)), bits(w_stat))


SHAPE_SETS = [
    [(64, 3, 7, 7), (64,), (64,), (64, 64, 3, 3), (1000, 512), (1000,)],
    [(1,), (3,), (0,), (5, 2, 2), (7,), (4097,), (8192,), (16385,)],
    [(17 + 3 * i,) for i in range(120)],  # more arrays than one launch's table holds
]


@pytest.mark.parametrize("which", range(len(SHAPE_SETS)))
@pytest.mark.parametrize("offset", [0, 3])
@pytest.mark.parametrize("misalign", [False, True])
def test_flat_store_load_bit_exact(oracle, which, offset, misalign):
    rng = np.random.default_rng(10 * which + offset)
    shapes = SHAPE_SETS[which]
    arrays = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    dim = oracle.flat_store(arrays, None, 0)
    if misalign:  # device arrays that start one float off a 16-byte boundary
        backing = [torch.zeros(a.size + 4, device="cuda") for a in arrays]
        d_arrays = [b[1:1 + a.size] for a, b in zip(arrays, backing)]
        for d, a in zip(d_arrays, arrays):
            d.copy_(dev(a.ravel()))
    else:
        d_arrays = [dev(a) for a in arrays]
    flat = torch.full((dim + offset + 5,), -7.0, device="cuda")
    capi.check(capi.flat_store(d_arrays, flat, offset))
    want = np.full(dim + offset + 5, -7.0, np.float32)
    assert oracle.flat_store(arrays, want, offset) == dim + offset
    np.testing.assert_array_equal(bits(host(flat)), bits(want))
    # and back, from a different flat vector
    src = rng.standard_normal(dim + offset + 5).astype(np.float32)
    for d in d_arrays:
        d.fill_(float("nan"))
    capi.check(capi.flat_load(d_arrays, dev(src), offset))
    back = [np.empty_like(a) for a in arrays]
    oracle.flat_load(back, src, offset)
    for d, b in zip(d_arrays, back):
        np.testing.assert_array_equal(bits(host(d).reshape(b.shape)), bits(b))
    if misalign:  # nothing outside the views was touched
        for b, a in zip(backing, arrays):
            hb = host(b)
            assert hb[0] == 0 and (hb[1 + a.size:] == 0).all()


@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
@pytest.mark.parametrize("K", [1, 3, 4])
@pytest.mark.parametrize("nesterov", [False, True])
@pytest.mark.parametrize("l2", [0.0, 1e-4])
def test_sgd_step_bit_exact_over_steps(oracle, n, K, nesterov, l2):
    rng = np.random.default_rng(n + K)
    p = rng.standard_normal(n).astype(np.float32)
    m = np.zeros(n, np.float32)
    lag, sg = np.zeros(n, np.float32), np.zeros(n, np.float32)
    d_p, d_m = dev(p), dev(m)
    d_lag, d_sg = torch.full((n,), float("nan"), device="cuda"), torch.full((n,), float("nan"), device="cuda")
    steps = [0.1, 0.05, 0.025, 0.0125]
    for t in range(3):
        grads = [rng.standard_normal(n).astype(np.float32) for _ in range(K)]
        d_grads = [dev(g) for g in grads]
        capi.check(capi.sgd_step(d_grads, d_p, d_m, d_lag, d_sg, l2_reg=l2, momentum=0.9, step_size=steps[t],
                                 next_step_size=steps[t + 1], nesterov=nesterov))
        oracle.sgd_step(grads, p, m, lag, sg, l2, 0.9, steps[t], steps[t + 1], nesterov)
        for got, want in ((d_p, p), (d_m, m), (d_lag, lag), (d_sg, sg)):
            np.testing.assert_array_equal(bits(host(got)), bits(want))


def test_sgd_step_optional_outputs_aliasing_and_errors(oracle):
    rng = np.random.default_rng(5)
    n = 5001
    grads = [rng.standard_normal(n).astype(np.float32) for _ in range(2)]
    p0 = rng.standard_normal(n).astype(np.float32)
    m0 = rng.standard_normal(n).astype(np.float32)
    p, m, sg = p0.copy(), m0.copy(), np.zeros(n, np.float32)
    oracle.sgd_step(grads, p, m, None, sg, 0.0, 0.5, 0.1, 0.1, False)
    # no lagged copy, and the reduced gradient written over rank 0's vector (as the reference's
    # in-place reduce does)
    d_g = [dev(g) for g in grads]
    d_p, d_m = dev(p0), dev(m0)
    capi.check(capi.sgd_step(d_g, d_p, d_m, None, d_g[0], momentum=0.5, step_size=0.1, next_step_size=0.1))
    np.testing.assert_array_equal(bits(host(d_p)), bits(p))
    np.testing.assert_array_equal(bits(host(d_m)), bits(m))
    np.testing.assert_array_equal(bits(host(d_g[0])), bits(sg))
    np.testing.assert_array_equal(bits(host(d_g[1])), bits(grads[1]))
    # unaligned views take the scalar path, same bits
    back = [torch.zeros(n + 4, device="cuda") for _ in range(4)]
    v = [b[1:1 + n] for b in back]
    v[0].copy_(dev(grads[0])); v[1].copy_(dev(grads[1])); v[2].copy_(dev(p0)); v[3].copy_(dev(m0))
    capi.check(capi.sgd_step(v[:2], v[2], v[3], None, None, momentum=0.5, step_size=0.1, next_step_size=0.1))
    np.testing.assert_array_equal(bits(host(v[2])), bits(p))
    np.testing.assert_array_equal(bits(host(v[3])), bits(m))
    # argument errors enqueue nothing
    assert capi.sgd_step([d_p], d_p, d_m) == capi.ADH_EINVAL            # a gradient aliases the parameters
    assert capi.sgd_step([d_g[0]] * 17, d_p, d_m) == capi.ADH_EINVAL    # more vectors than ADH_MAX_TILES
    assert capi.lib().adh_sgd_step_f32(n, 0, None, 0, 0, 0, 0, 0, d_p.data_ptr(), d_m.data_ptr(), None, None, None) \
        == capi.ADH_EINVAL
    torch.cuda.synchronize()
    np.testing.assert_array_equal(bits(host(d_p)), bits(p))
