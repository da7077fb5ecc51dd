"""GPU parity of softmax / NLL against the CPU oracle.  fp32 tolerance: rel-err <= 1e-5
(max|a-b| / max|b|).  Every call goes through the C ABI."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi
from gpu_util import dev, host, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.mark.parametrize("N,C", [(256, 1000), (1, 1), (3, 7), (5, 64), (4, 1024), (2, 1025), (3, 5000), (300, 10)])
def test_softmax_nll_vs_oracle(oracle, N, C):
    rng = np.random.default_rng(C)
    x = (2.0 * rng.standard_normal((N, C))).astype(np.float32)
    label = rng.integers(0, C, size=N).astype(np.uint32)
    y = np.empty_like(x)
    oracle.softmax_fwd(x, y)
    loss = np.empty(N, np.float32)
    oracle.softmax_nll_loss_fwd(y, label, loss)
    dloss = np.full(N, 1.0 / N, np.float32)
    dx0 = rng.standard_normal((N, C)).astype(np.float32)
    dx = dx0.copy()
    oracle.softmax_nll_loss_bwd(y, label, dloss, dx)

    gx, gl = dev(x), dev(label)
    gy = torch.full((N, C), float("nan"), device="cuda")
    capi.check(capi.softmax_fwd(gx, gy))
    assert rel_err(host(gy), y) <= TOL
    np.testing.assert_allclose(host(gy).astype(np.float64).sum(axis=1), 1.0, atol=1e-5)
    gloss = torch.full((N,), float("nan"), device="cuda")
    capi.check(capi.softmax_nll_loss_fwd(gy, gl, gloss))
    assert rel_err(host(gloss), loss) <= TOL
    # fused forward gives the same y and loss bits as the two-step path
    gy2 = torch.full((N, C), float("nan"), device="cuda")
    gloss2 = torch.full((N,), float("nan"), device="cuda")
    capi.check(capi.softmax_xent_fwd(gx, gl, gy2, gloss2))
    assert torch.equal(gy2, gy) and torch.equal(gloss2, gloss)
    gdx = dev(dx0)
    capi.check(capi.softmax_nll_loss_bwd(gy, gl, dev(dloss), gdx))
    assert rel_err(host(gdx), dx) <= TOL
    # bwd on the oracle's y: the same arithmetic up to the fused multiply-add a host compiler may contract
    # `dx + dloss*(y-1)` into (one rounding instead of the kernel's two)
    gdx2 = dev(dx0)
    capi.check(capi.softmax_nll_loss_bwd(dev(y), gl, dev(dloss), gdx2))
    np.testing.assert_allclose(host(gdx2), dx, rtol=1e-6, atol=1e-7)

    # one kernel for y, loss and dx: the same bits as the separate entry points, for a per-example
    # gradient and for one number, accumulating and overwriting
    for beta in (1.0, 0.0):
        for per_example in (True, False):
            gdl = dev(dloss) if per_example else None
            want = dev(dx0)
            capi.check(capi.softmax_nll_loss_bwd_scaled(gy, gl, gdl, 1.0 / N, beta, want))
            if per_example and beta == 1.0:
                assert torch.equal(want, gdx)
            if beta == 0.0:
                ref = np.zeros_like(dx0)
                oracle.softmax_nll_loss_bwd(host(gy), label, dloss, ref)
                np.testing.assert_array_equal(host(want), ref)
            gy3 = torch.full((N, C), float("nan"), device="cuda")
            gloss3 = torch.full((N,), float("nan"), device="cuda")
            got = dev(dx0)
            capi.check(capi.softmax_xent_fwd_bwd(gx, gl, gdl, 1.0 / N, gy3, gloss3, beta, got))
            assert torch.equal(gy3, gy) and torch.equal(gloss3, gloss) and torch.equal(got, want)


def test_softmax_properties():
    N, C = 256, 1000
    g = torch.Generator(device="cuda").manual_seed(4)
    x = torch.randn(N, C, device="cuda", generator=g) * 2
    y = torch.empty_like(x)
    capi.check(capi.softmax_fwd(x, y))
    y2 = torch.empty_like(x)
    capi.check(capi.softmax_fwd(x + 100.0, y2))  # shift invariance, no overflow
    assert rel_err(host(y2), host(y)) <= 1e-4
    u = torch.zeros(4, C, device="cuda")
    yu = torch.empty_like(u)
    lab = torch.tensor([0, 1, 500, 999], dtype=torch.int32, device="cuda")
    loss = torch.empty(4, device="cuda")
    capi.check(capi.softmax_xent_fwd(u, lab, yu, loss))
    np.testing.assert_allclose(host(loss), np.log(C), rtol=1e-6)
    # zero-initialised dx rows sum to ~0
    dx = torch.zeros_like(x)
    labels = torch.randint(0, C, (N,), device="cuda", dtype=torch.int32)
    dl = torch.full((N,), 1.0 / N, device="cuda")
    capi.check(capi.softmax_nll_loss_bwd(y, labels, dl, dx))
    assert float(dx.double().sum(dim=1).abs().max()) < 1e-7


def test_fused_forward_backward_error_codes():
    x = torch.zeros(2, 8, device="cuda")
    lab = torch.zeros(2, dtype=torch.int32, device="cuda")
    y, dx, loss = torch.empty_like(x), torch.empty_like(x), torch.empty(2, device="cuda")
    assert capi.softmax_xent_fwd_bwd(x, lab, None, 1.0, y, loss, 0.5, dx) == capi.ADH_EINVAL
    assert capi.softmax_xent_fwd_bwd(x, lab, None, 1.0, y, loss, 0.0, y) == capi.ADH_EINVAL
    assert capi.softmax_nll_loss_bwd_scaled(y, lab, None, 1.0, 2.0, dx) == capi.ADH_EINVAL
    # the gradient may overwrite the logits of a short row
    capi.check(capi.softmax_xent_fwd(x, lab, y, loss))
    want = torch.empty_like(x)
    capi.check(capi.softmax_nll_loss_bwd_scaled(y, lab, None, 0.5, 0.0, want))
    xin = x.clone()
    capi.check(capi.softmax_xent_fwd_bwd(xin, lab, None, 0.5, y, loss, 0.0, xin))
    assert torch.equal(xin, want)
