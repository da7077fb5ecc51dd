"""The forward entry point that allocates nothing (adh_conv3x3_slab_fwd_tiles_static: its reordered
filter lives in an array inside the library's device image) against the entry point that takes a
workspace: same kernels, so the outputs must agree bit for bit.  Two calls in a row, the second
with a smaller input and fewer output channels, so that a stale part of the shared array would
show; then beta = 1, a shape past the array's limit, and a check that the calls really allocate
nothing."""
import ctypes

import numpy as np
import pytest
import torch

from arraydiff_cuda_amd import capi

pytestmark = pytest.mark.gpu


def _run_pair(K, N, Cin, Cout, H, W, seed, beta=0.0):
    lib = capi.lib()
    g = torch.Generator(device="cuda").manual_seed(seed)
    xs = [(torch.rand((N, Cin, H + 2, W + 2), device="cuda", generator=g) * 2 - 1).to(torch.bfloat16) for _ in range(K)]
    w = (torch.randn((Cout, Cin, 3, 3), device="cuda", generator=g) * (2.0 / (Cin * 9)) ** 0.5).to(torch.bfloat16)
    y0 = [torch.randn((N, Cout, H, W), device="cuda", generator=g).to(torch.bfloat16) for _ in range(K)]
    ya = [t.clone() for t in y0]
    yb = [t.clone() for t in y0]
    ws_bytes = capi.conv_workspace_bytes(capi.ADH_CONV_FWD, capi.ADH_BF16, K, N, Cin, Cout, H, W)
    ws = torch.empty(ws_bytes // 4 + 64, device="cuda")
    x_tbl, _k0 = capi.ptr_table([t.data_ptr() for t in xs])
    a_tbl, _k1 = capi.ptr_table([t.data_ptr() for t in ya])
    b_tbl, _k2 = capi.ptr_table([t.data_ptr() for t in yb])
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    capi.check(lib.adh_conv3x3_slab_fwd_tiles(capi.ADH_BF16, K, N, Cin, Cout, H, W, x_tbl, w.data_ptr(), a_tbl, beta,
                                              ws.data_ptr(), ws_bytes, st), "fwd with workspace")
    torch.cuda.synchronize()
    # torch's own counter sees only torch's caching allocator; the driver's free-memory figure also sees what the
    # library itself would take with hipMalloc and keep
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    capi.check(lib.adh_conv3x3_slab_fwd_tiles_static(capi.ADH_BF16, K, N, Cin, Cout, H, W, x_tbl, w.data_ptr(), b_tbl,
                                                     beta, st), "fwd, static scratch")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    for r in range(K):
        a, b = ya[r].view(torch.int16).cpu().numpy(), yb[r].view(torch.int16).cpu().numpy()
        assert not np.array_equal(a, y0[r].view(torch.int16).cpu().numpy())  # something was computed
        np.testing.assert_array_equal(a, b)


def test_static_scratch_forward_matches_workspace_forward():
    # fewer than 64 input channels: the filter is reordered into the scratch array (a 64-channel filter at an
    # aligned address is read in place), and 256 output channels write and read all 294,912 bytes of it
    print("static scratch: 2 tiles, N=2, 48->256 channels, 12x136", flush=True)
    _run_pair(2, 2, 48, 256, 12, 136, seed=14)
    print("static scratch: 2 tiles, N=2, 64->200 channels, 12x136", flush=True)
    _run_pair(2, 2, 64, 200, 12, 136, seed=11)
    print("static scratch: second call, smaller: 1 tile, N=1, 24->40 channels, 5x24", flush=True)
    _run_pair(1, 1, 24, 40, 5, 24, seed=12)
    print("static scratch: beta = 1, odd width (the four-wave kernel)", flush=True)
    _run_pair(2, 1, 64, 64, 6, 33, seed=13, beta=1.0)


def test_static_scratch_limits():
    lib = capi.lib()
    x = torch.zeros((1, 64, 6, 10), device="cuda", dtype=torch.bfloat16)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    x_tbl, _k0 = capi.ptr_table([x.data_ptr()])
    for Cin, Cout in ((64, 257), (65, 64)):
        w = torch.zeros((Cout, Cin, 3, 3), device="cuda", dtype=torch.bfloat16)
        y = torch.zeros((1, Cout, 4, 8), device="cuda", dtype=torch.bfloat16)
        y_tbl, _k1 = capi.ptr_table([y.data_ptr()])
        assert lib.adh_conv3x3_slab_fwd_tiles_static(capi.ADH_BF16, 1, 1, Cin, Cout, 4, 8, x_tbl, w.data_ptr(), y_tbl,
                                                     0.0, st) == capi.ADH_EWORKSPACE
    w = torch.zeros((64, 64, 3, 3), device="cuda")
    y = torch.zeros((1, 64, 4, 8), device="cuda")
    y_tbl, _k1 = capi.ptr_table([y.data_ptr()])
    assert lib.adh_conv3x3_slab_fwd_tiles_static(capi.ADH_F32, 1, 1, 64, 64, 4, 8, x_tbl, w.data_ptr(), y_tbl, 0.0,
                                                 st) == capi.ADH_EUNIMPL
