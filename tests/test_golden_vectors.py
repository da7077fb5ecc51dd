"""The committed known-answer vectors of tests/golden/vectors.npz (made by tests/golden/make_vectors.py with numpy
slicing and torch's CPU convolution in float64, neither the oracle nor the library) against the oracle (CPU) and
against the HIP path through the C ABI (GPU).  Data movement bit for bit; conv and softmax within 1e-5."""
import os

import numpy as np
import pytest

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz"), allow_pickle=False)
K, P, N, C, H, W = (int(v) for v in V["geom"])
HT = H // K


def close(a, b, tol=1e-5):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.max(np.abs(a - b)) <= tol * max(np.max(np.abs(b)), 1e-30)


# ---------------------------------------------------------------- the oracle (CPU)
def test_oracle_data_movement_vs_vectors(oracle):
    tiles = [np.full((N, C, HT + 2 * P, W + 2 * P), np.nan, np.float32) for _ in range(K)]
    assert oracle.tiles_pack(K, P, W, H, C, N, V["unsplit"], tiles) == 0
    for r in range(K):
        assert np.array_equal(tiles[r], V["packed"][r])
    ex = [V["padded"][r].copy() for r in range(K)]
    assert oracle.halo_op(oracle.EXCH, 1, K, P, W, HT, C, N, ex) == 0
    for r in range(K):
        assert np.array_equal(ex[r], V["packed"][r])
    rd = [V["reduce_in"][r].copy() for r in range(K)]
    assert oracle.halo_op(oracle.REDUCE, 1, K, P, W, HT, C, N, rd) == 0
    for r in range(K):
        assert np.array_equal(rd[r][:, :, P:-P, P:-P], V["reduce_out"][r][:, :, P:-P, P:-P])
    back = np.full((N, C, H, W), np.nan, np.float32)
    assert oracle.tiles_unpack(K, P, W, H, C, N, [V["packed"][r].copy() for r in range(K)], back) == 0
    assert np.array_equal(back, V["unsplit"])


def test_oracle_conv_bias_softmax_vs_vectors(oracle):
    x, w, dy = V["conv_x_pad"], V["conv_w"], V["conv_dy"]
    y = np.empty(V["conv_y"].shape, np.float32)
    oracle.conv_slab_fwd(x, w, y)
    assert close(y, V["conv_y"])
    dx = np.empty(x.shape, np.float32)
    oracle.conv_slab_bwd_data(w, dy, dx)
    assert close(dx, V["conv_dx_pad"])
    dw = np.empty(w.shape, np.float32)
    oracle.conv_slab_bwd_filter(x, dy, dw)
    assert close(dw, V["conv_dw"])
    yb = V["conv_y"].astype(np.float32)
    oracle.conv_bias_add(V["bias"], yb)
    assert np.array_equal(yb, V["bias_y"])
    db = np.empty(V["bias"].shape, np.float32)
    oracle.conv_bwd_bias(dy, db)
    assert close(db, V["bias_db"])
    prob = np.empty(V["sm_logits"].shape, np.float32)
    oracle.softmax_fwd(V["sm_logits"], prob)
    assert close(prob, V["sm_y"])
    loss = np.empty(V["sm_loss"].shape, np.float32)
    oracle.softmax_nll_loss_fwd(prob, V["sm_label"], loss)
    assert close(loss, V["sm_loss"])
    dxs = V["sm_dx0"].copy()
    oracle.softmax_nll_loss_bwd(prob, V["sm_label"], V["sm_dloss"], dxs)
    assert close(dxs, V["sm_dx"])


# ---------------------------------------------------------------- the HIP path (GPU)
@pytest.mark.gpu
def test_hip_data_movement_vs_vectors():
    import torch
    from arraydiff_cuda_amd import capi
    from gpu_util import dev, host
    tiles = [torch.full((N, C, HT + 2 * P, W + 2 * P), float("nan"), device="cuda") for _ in range(K)]
    capi.check(capi.tiles_pack(K, P, W, H, C, N, dev(V["unsplit"]), tiles), "pack")
    for r in range(K):
        assert np.array_equal(host(tiles[r]), V["packed"][r])
    ex = [dev(V["padded"][r]) for r in range(K)]
    capi.check(capi.halo_exchange(ex, 1, K, P, W, HT, C, N), "exchange")
    for r in range(K):
        assert np.array_equal(host(ex[r]), V["packed"][r])
    rd = [dev(V["reduce_in"][r]) for r in range(K)]
    capi.check(capi.halo_reduce(rd, 1, K, P, W, HT, C, N), "reduce")
    for r in range(K):
        assert np.array_equal(host(rd[r])[:, :, P:-P, P:-P], V["reduce_out"][r][:, :, P:-P, P:-P])
    back = torch.full((N, C, H, W), float("nan"), device="cuda")
    capi.check(capi.tiles_unpack(K, P, W, H, C, N, [dev(V["packed"][r]) for r in range(K)], back), "unpack")
    assert np.array_equal(host(back), V["unsplit"])


@pytest.mark.gpu
def test_hip_conv_bias_softmax_vs_vectors():
    import torch
    from arraydiff_cuda_amd import capi
    from gpu_util import dev, host
    x, w, dy = V["conv_x_pad"], V["conv_w"], V["conv_dy"]
    n, co, h, wd = V["conv_y"].shape
    ci = x.shape[1]
    y = torch.full((n, co, h, wd), float("nan"), device="cuda")
    capi.check(capi.conv_fwd_tiles([dev(x)], dev(w), [y], n, ci, co, h, wd), "fwd")
    assert close(host(y), V["conv_y"])
    dx = torch.full(x.shape, float("nan"), device="cuda")
    capi.check(capi.conv_bwd_data_tiles(dev(w), [dev(dy)], [dx], n, ci, co, h, wd), "bwd-data")
    assert close(host(dx), V["conv_dx_pad"])
    dw = torch.full(w.shape, float("nan"), device="cuda")
    nbytes = capi.conv_workspace_bytes(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, 1, n, ci, co, h, wd)
    ws = torch.empty(max(nbytes // 4, 1), device="cuda")
    capi.check(capi.conv_bwd_filter_tiles([dev(x)], [dev(dy)], dw, n, ci, co, h, wd, ws=ws), "bwd-filter")
    assert close(host(dw), V["conv_dw"])
    yb = dev(V["conv_y"].astype(np.float32))
    capi.check(capi.conv_bias_add_tiles([dev(V["bias"])], [yb], n, co, h, wd), "bias")
    assert np.array_equal(host(yb), V["bias_y"])
    db = torch.full((co,), float("nan"), device="cuda")
    wsb = torch.empty(capi.conv_bwd_bias_workspace_bytes(1, n, co) // 4 + 64, device="cuda")
    capi.check(capi.conv_bwd_bias_tiles([dev(dy)], db, n, co, h, wd, ws=wsb), "bias gradient")
    assert close(host(db), V["bias_db"])
    prob = torch.empty(V["sm_logits"].shape, device="cuda")
    capi.check(capi.softmax_fwd(dev(V["sm_logits"]), prob), "softmax")
    assert close(host(prob), V["sm_y"])
    loss = torch.empty(V["sm_loss"].shape, device="cuda")
    capi.check(capi.softmax_nll_loss_fwd(prob, dev(V["sm_label"]), loss), "nll")
    assert close(host(loss), V["sm_loss"])
    dxs = dev(V["sm_dx0"])
    capi.check(capi.softmax_nll_loss_bwd(prob, dev(V["sm_label"]), dev(V["sm_dloss"]), dxs), "nll bwd")
    assert close(host(dxs), V["sm_dx"])
