"""The C-ABI library loads and exports every symbol include/adh_capi.h declares; argument
validation that returns before any device work is exercised without a GPU."""
import ctypes
import os
import re

from arraydiff_cuda_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    hdr = open(os.path.join(ROOT, "include", "adh_capi.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    return sorted(set(re.findall(r"\b(adh_[a-z0-9_]+)\s*\(", hdr)))


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_symbols()
    assert len(names) >= 28
    lib = ctypes.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), "libadh.so does not export %s" % n
    assert set(names) == set(capi.SIGNATURES), "capi.SIGNATURES out of sync with the header"
    assert capi.lib().adh_version() == 1
    assert b"NULL" in capi.lib().adh_error_string(capi.ADH_ENULL)


def test_argument_errors_need_no_gpu():
    l = capi.lib()
    bogus = ctypes.c_void_p(0x1000)
    tb, keep = capi.ptr_table([0x1000, None])
    assert l.adh_halo_exchange_nchw(0, 1, 2, 1, 4, 4, 1, 1, tb, None) == capi.ADH_ENULL
    tb4, keep4 = capi.ptr_table([0x1000] * 4)
    assert l.adh_halo_exchange_nchw(0, 2, 2, 1, 4, 4, 1, 1, tb4, None) == capi.ADH_EUNIMPL
    assert l.adh_halo_exchange_nchw(7, 1, 2, 1, 4, 4, 1, 1, tb4, None) == capi.ADH_EINVAL          # dtype
    assert l.adh_halo_reduce_nchw(0, 1, 4, 3, 4, 4, 1, 1, tb4, None) == capi.ADH_EINVAL            # H < 2p
    assert l.adh_halo_exchange_nchw(0, 1, 1, 1, 4, 4, 1, 1, tb4, None) == capi.ADH_OK              # 1x1 no-op
    odd, keepo = capi.ptr_table([0x1001, 0x1000])
    assert l.adh_halo_exchange_nchw(0, 1, 2, 1, 4, 4, 1, 1, odd, None) == capi.ADH_EALIGN
    assert l.adh_tiles_pack_nchw(0, 3, 1, 4, 8, 1, 1, bogus, tb4, None) == capi.ADH_EINVAL          # H % K
    assert l.adh_tiles_pack_nchw(0, 17, 1, 4, 34, 1, 1, bogus, tb4, None) == capi.ADH_EINVAL        # > 16 tiles
    assert l.adh_slice_copy_nchw(0, 5, 1, 1, 1, bogus, 4, 4, 1, 0, 0, 0, bogus, 8, 8, 1, 0, 0, 0, None) == capi.ADH_EINVAL
    assert l.adh_conv3x3_slab_fwd(0, 1, 4, 4, 3, 3, bogus, bogus, bogus, 0.5, None, 0, None) == capi.ADH_EINVAL  # beta
    assert l.adh_conv3x3_slab_fwd(1, 1, 4, 4, 3, 3, bogus, bogus, bogus, 0.0, None, 0, None) == capi.ADH_ENULL  # bf16 needs a workspace
    assert l.adh_conv3x3_workspace_bytes(capi.ADH_CONV_FWD, 1, 1, 1, 4, 4, 3, 3) > 0
    assert l.adh_conv3x3_slab_fwd(0, 1, 4, 4, 3, 3, None, bogus, bogus, 0.0, None, 0, None) == capi.ADH_ENULL
    assert l.adh_conv3x3_slab_bwd_filter(0, 1, 4, 4, 3, 3, bogus, bogus, bogus, 0.0, bogus, 16, None) == capi.ADH_EWORKSPACE
    assert l.adh_conv3x3_workspace_bytes(capi.ADH_CONV_BWD_FILTER, 0, 4, 32, 64, 64, 14, 56) > 0
    assert l.adh_conv3x3_workspace_bytes(capi.ADH_CONV_FWD, 0, 4, 32, 64, 64, 14, 56) == 0
    assert l.adh_softmax_fwd(10, 2, None, bogus, None) == capi.ADH_ENULL
    assert l.adh_fill_f32(0, 1.0, None, None) == capi.ADH_OK                                       # empty
    assert l.adh_softmax_fwd(0, 0, None, None, None) == capi.ADH_OK
    # the shape query of the pooling over tiles without halo launches nothing
    q = l.adh_pool2d_unpadded_supported
    assert q(0, capi.ADH_POOL_MAX, 4, 32, 64, 64, 256, 3, 3, 2, 2, 1, 1) == capi.ADH_OK        # the stem's pooling
    assert q(0, capi.ADH_POOL_MAX, 4, 32, 64, 64, 8192, 3, 3, 2, 2, 1, 1) == capi.ADH_EUNIMPL  # rows too wide for a band in LDS
    assert q(0, capi.ADH_POOL_MAX, 4, 32, 64, 63, 256, 3, 3, 2, 2, 1, 1) == capi.ADH_EINVAL    # the row split does not stitch
    assert l.adh_conv_bwd_bias_workspace_bytes(4, 32, 64) > 0


def test_bf16_conv_workspace_holds_the_sums_of_every_route_that_needs_them():
    """More than 64 reduction channels at a width the eight-wave kernels do not take run one launch per 64 channels
    with fp32 sums between them: the workspace query has to count those sums whatever one launch of 128 channels
    would have needed at a friendlier width (host logic only, no GPU)."""
    l = capi.lib()
    group = 9 * 2 * 64 * 32 * 2  # bytes of the reordered filter per (64 outputs, 64 reduction channels)

    def need(which, K, N, Cin, Cout, H, W):
        cred, cout = (Cin, Cout) if which == capi.ADH_CONV_FWD else (Cout, Cin)
        oh, ow = (H, W) if which == capi.ADH_CONV_FWD else (H + 2, W + 2)
        filt = ((cout + 63) // 64) * ((cred + 63) // 64) * group
        part = K * ((N * cout * oh * ow * 4 + 255) // 256 * 256)
        return filt, part

    for (K, N, Cin, Cout, H, W) in [(2, 1, 128, 128, 9, 7), (1, 2, 100, 70, 5, 13), (3, 1, 65, 65, 3, 1), (1, 1, 128, 96, 4, 27)]:
        for which in (capi.ADH_CONV_FWD, capi.ADH_CONV_BWD_DATA):
            filt, part = need(which, K, N, Cin, Cout, H, W)
            got = l.adh_conv3x3_workspace_bytes(which, capi.ADH_BF16, K, N, Cin, Cout, H, W)
            assert got >= filt + part, (which, K, N, Cin, Cout, H, W, got, filt, part)
    # one launch of 128 channels (even width forward, a multiple of 8 backward): the filter alone
    for which in (capi.ADH_CONV_FWD, capi.ADH_CONV_BWD_DATA):
        filt, part = need(which, 2, 1, 128, 128, 9, 72)
        assert l.adh_conv3x3_workspace_bytes(which, capi.ADH_BF16, 2, 1, 128, 128, 9, 72) == filt
