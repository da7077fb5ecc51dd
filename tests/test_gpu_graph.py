"""The C ABI enqueues kernels only (no allocation, no memset, no host synchronisation), so a sequence
of calls can be captured into a HIP graph and replayed.  A forward + backward slice of the path
(pack -> conv -> batch norm/rectifier/pad -> pooling; conv backward-filter, backward-data -> halo
reduce -> unpack) is captured once and replayed several times with eager work and synchronisations
between the replays; every replay must reproduce the eager results bit for bit (all kernels are
deterministic).  Also: two eager runs of the three filter-gradient paths give identical bits."""
import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi

pytestmark = pytest.mark.gpu


def _sequence(bufs):
    K, p, N, C, H, W = bufs["dims"]
    Ht = H // K
    capi.check(capi.tiles_pack(K, p, W, H, C, N, bufs["x"], bufs["tiles"]))
    capi.check(capi.conv_fwd_tiles(bufs["tiles"], bufs["w"], bufs["ys"], N, C, C, Ht, W))
    capi.check(capi.batchnorm_fwd_tiles(bufs["ys"], bufs["scale"], bufs["shift"], bufs["act"], N, C, Ht, W, relu=1, out_halo=1,
                                        save_means=bufs["mean"], save_invstds=bufs["invstd"], ws=bufs["bn_ws"]))
    capi.check(capi.pool_fwd_tiles(capi.ADH_POOL_MAX, bufs["act"], bufs["pooled"], N, C, Ht + 2, W + 2, 3, 3, 2, 2))
    capi.check(capi.conv_bwd_filter_tiles(bufs["tiles"], bufs["dys"], bufs["dw"], N, C, C, Ht, W, ws=bufs["wg_ws"]))
    capi.check(capi.conv_bwd_data_tiles(bufs["w"], bufs["dys"], bufs["gs"], N, C, C, Ht, W))
    capi.check(capi.halo_reduce(bufs["gs"], 1, K, p, W, Ht, C, N))
    capi.check(capi.tiles_unpack(K, p, W, H, C, N, bufs["gs"], bufs["dx"]))


def _outputs(bufs):
    return [t.clone() for t in bufs["pooled"]] + [bufs["dw"].clone(), bufs["dx"].clone()] + [t.clone() for t in bufs["mean"]]


def test_graph_replays_match_eager():
    K, p, N, C, H, W = 4, 1, 4, 32, 32, 40
    Ht = H // K
    g = torch.Generator(device="cuda").manual_seed(5)
    rnd = lambda *s: torch.randn(s, device="cuda", generator=g)
    bufs = {
        "dims": (K, p, N, C, H, W), "x": rnd(N, C, H, W), "w": rnd(C, C, 3, 3) * 0.1,
        "tiles": [torch.empty((N, C, Ht + 2, W + 2), device="cuda") for _ in range(K)],
        "ys": [torch.empty((N, C, Ht, W), device="cuda") for _ in range(K)],
        "act": [torch.empty((N, C, Ht + 2, W + 2), device="cuda") for _ in range(K)],
        "pooled": [torch.empty((N, C, (Ht - 1) // 2 + 1, (W - 1) // 2 + 1), device="cuda") for _ in range(K)],
        "scale": [torch.rand(C, device="cuda", generator=g) + 0.5 for _ in range(K)],
        "shift": [torch.rand(C, device="cuda", generator=g) - 0.5 for _ in range(K)],
        "mean": [torch.empty(C, device="cuda") for _ in range(K)], "invstd": [torch.empty(C, device="cuda") for _ in range(K)],
        "dys": [rnd(N, C, Ht, W) for _ in range(K)], "gs": [torch.empty((N, C, Ht + 2, W + 2), device="cuda") for _ in range(K)],
        "dw": torch.empty((C, C, 3, 3), device="cuda"), "dx": torch.empty((N, C, H, W), device="cuda"),
        "bn_ws": torch.empty(capi.batchnorm_workspace_bytes(K, N, C) // 4, device="cuda"),
        "wg_ws": torch.empty(max(capi.conv_workspace_bytes(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, K, N, C, C, Ht, W) // 4, 1),
                             device="cuda"),
    }
    assert bufs["pooled"][0].shape[2:] == ((Ht + 2 - 3) // 2 + 1, (W + 2 - 3) // 2 + 1)
    _sequence(bufs)
    torch.cuda.synchronize()
    want = _outputs(bufs)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _sequence(bufs)  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _sequence(bufs)
    for rep in range(3):
        # eager work between the replays: scribble over every output, run an unrelated call, synchronise
        for t in bufs["pooled"] + bufs["gs"] + bufs["act"] + bufs["mean"] + [bufs["dw"], bufs["dx"]]:
            t.fill_(float("nan"))
        capi.check(capi.relu_fwd(bufs["x"], torch.empty_like(bufs["x"])))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, exp in zip(_outputs(bufs), want):
            assert torch.equal(got, exp), "replay %d differs from the eager run" % rep


def test_graph_replays_bf16_wide_channels_and_bias():
    """The bf16 convolution with more than 64 reduction channels (a launch of 128 with the sums in registers, fp32 sums
    through the workspace into a launch of 64), forward and backward-data, and the bias add and gradient, captured and
    replayed: bit for bit the eager results on every replay."""
    K, N, Cin, Cout, Ht, W = 2, 2, 192, 136, 12, 72
    g = torch.Generator(device="cuda").manual_seed(8)
    bf = lambda *s: torch.randn(s, device="cuda", generator=g).to(torch.bfloat16)
    xs, dys = [bf(N, Cin, Ht + 2, W + 2) for _ in range(K)], [bf(N, Cout, Ht, W) for _ in range(K)]
    w = (torch.randn((Cout, Cin, 3, 3), device="cuda", generator=g) * 0.05).to(torch.bfloat16)
    bias = [torch.randn(Cout, device="cuda", generator=g) for _ in range(K)]
    ys = [torch.empty((N, Cout, Ht, W), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    gs = [torch.empty((N, Cin, Ht + 2, W + 2), device="cuda", dtype=torch.bfloat16) for _ in range(K)]
    db = torch.empty(Cout, device="cuda")
    ws = torch.empty(max(capi.conv_workspace_bytes(wh, capi.ADH_BF16, K, N, Cin, Cout, Ht, W)
                         for wh in (capi.ADH_CONV_FWD, capi.ADH_CONV_BWD_DATA)) // 4 + 64, device="cuda")
    bws = torch.empty(capi.conv_bwd_bias_workspace_bytes(K, N, Cout) // 4 + 64, device="cuda")

    def sequence():
        capi.check(capi.conv_fwd_tiles(xs, w, ys, N, Cin, Cout, Ht, W, ws=ws))
        capi.check(capi.conv_bias_add_tiles(bias, ys, N, Cout, Ht, W))
        capi.check(capi.conv_bwd_data_tiles(w, dys, gs, N, Cin, Cout, Ht, W, ws=ws))
        capi.check(capi.conv_bwd_bias_tiles(dys, db, N, Cout, Ht, W, ws=bws))

    outputs = lambda: [t.clone() for t in ys + gs] + [db.clone()]
    sequence()
    torch.cuda.synchronize()
    want = outputs()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        sequence()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        sequence()
    for rep in range(3):
        for t in ys + gs + [db, ws, bws]:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, exp in zip(outputs(), want):
            assert torch.equal(got, exp), "replay %d differs from the eager run" % rep


def test_filter_gradients_are_reproducible():
    g = torch.Generator(device="cuda").manual_seed(6)
    K, N, C, Ht, W = 2, 4, 64, 14, 56
    xs = [torch.randn((N, C, Ht + 2, W + 2), device="cuda", generator=g) for _ in range(K)]
    dys = [torch.randn((N, C, Ht, W), device="cuda", generator=g) for _ in range(K)]
    ws = torch.empty(max(capi.conv_workspace_bytes(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, K, N, C, C, Ht, W) // 4, 1), device="cuda")
    a, b = torch.empty((C, C, 3, 3), device="cuda"), torch.empty((C, C, 3, 3), device="cuda")
    capi.check(capi.conv_bwd_filter_tiles(xs, dys, a, N, C, C, Ht, W, ws=ws))
    capi.check(capi.conv_bwd_filter_tiles(xs, dys, b, N, C, C, Ht, W, ws=ws))
    assert torch.equal(a, b)
    xb, db = [t.to(torch.bfloat16) for t in xs], [t.to(torch.bfloat16) for t in dys]
    wsb = torch.empty(capi.conv_workspace_bytes(capi.ADH_CONV_BWD_FILTER, capi.ADH_BF16, K, N, C, C, Ht, W) // 4 + 64, device="cuda")
    capi.check(capi.conv_bwd_filter_tiles(xb, db, a, N, C, C, Ht, W, ws=wsb))
    capi.check(capi.conv_bwd_filter_tiles(xb, db, b, N, C, C, Ht, W, ws=wsb))
    assert torch.equal(a, b)
    geo = (3, 3, 2, 2, 1, 1)
    d2 = [torch.randn((N, C, 7, 28), device="cuda", generator=g) for _ in range(K)]
    wsg = torch.empty(capi.conv2d_workspace_bytes(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, K, N, C, C, Ht + 2, W + 2, *geo) // 4,
                      device="cuda")
    capi.check(capi.conv2d_bwd_filter_tiles(xs, d2, a, N, C, C, Ht + 2, W + 2, *geo, ws=wsg))
    capi.check(capi.conv2d_bwd_filter_tiles(xs, d2, b, N, C, C, Ht + 2, W + 2, *geo, ws=wsg))
    assert torch.equal(a, b)
