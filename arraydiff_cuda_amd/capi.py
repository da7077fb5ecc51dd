"""ctypes binding of ``libadh.so``.  There is no fallback: if the library is missing, or a
call is made without a GPU, an exception is raised."""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
# ADH_LIB names another build of the library (A/B measurements); the default is the one beside this file
LIB_PATH = os.environ.get("ADH_LIB") or os.path.join(_HERE, "libadh.so")
CSRC = os.path.join(_HERE, "csrc")

ADH_F32 = 0
ADH_BF16 = 1
ADH_OK, ADH_EINVAL, ADH_EUNIMPL, ADH_ENULL, ADH_EALIGN, ADH_EWORKSPACE = 0, -1, -2, -3, -4, -5
ADH_CONV_FWD, ADH_CONV_BWD_DATA, ADH_CONV_BWD_FILTER = 0, 1, 2
ADH_POOL_AVG, ADH_POOL_MAX = 0, 1
ADH_MAX_TILES = 16

u32, u64, i32, f32, vp, sz = (ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int, ctypes.c_float,
                              ctypes.c_void_p, ctypes.c_size_t)
vpp = ctypes.POINTER(ctypes.c_void_p)

# name -> (restype, argtypes); every symbol include/adh_capi.h declares
SIGNATURES = {
    "adh_version": (i32, []),
    "adh_error_string": (ctypes.c_char_p, [i32]),
    "adh_fill_f32": (i32, [u64, f32, vp, vp]),
    "adh_add_f32": (i32, [u64, vp, vp, vp]),
    "adh_halo_exchange_nchw": (i32, [i32, u32, u32, u32, u32, u32, u32, u32, vpp, vp]),
    "adh_halo_reduce_nchw": (i32, [i32, u32, u32, u32, u32, u32, u32, u32, vpp, vp]),
    "adh_halo_exchange_nchw_rank": (i32, [i32, u32, u32, u32, u32, u32, u32, u32, u32, vpp, vp]),
    "adh_halo_reduce_nchw_rank": (i32, [i32, u32, u32, u32, u32, u32, u32, u32, u32, vpp, vp]),
    "adh_halo_pad_nchw": (i32, [i32, u32, u32, u32, u32, u32, vp, vp, vp]),
    "adh_halo_pad_add_nchw": (i32, [i32, u32, u32, u32, u32, u32, vp, vp, vp]),
    "adh_halo_unpad_nchw": (i32, [i32, u32, u32, u32, u32, u32, vp, vp, vp]),
    "adh_halo_unpad_add_nchw": (i32, [i32, u32, u32, u32, u32, u32, vp, vp, vp]),
    "adh_halo_repad_nchw": (i32, [i32, u32, u32, u32, u32, u32, u32, vp, vp, vp]),
    "adh_slice_copy_nchw": (i32, [i32, u32, u32, u32, u32, vp, u32, u32, u32, u32, u32, u32,
                                  vp, u32, u32, u32, u32, u32, u32, vp]),
    "adh_slice_add_nchw": (i32, [i32, u32, u32, u32, u32, vp, u32, u32, u32, u32, u32, u32,
                                 vp, u32, u32, u32, u32, u32, u32, vp]),
    "adh_tiles_pack_nchw": (i32, [i32, u32, u32, u32, u32, u32, u32, vp, vpp, vp]),
    "adh_tiles_unpack_nchw": (i32, [i32, u32, u32, u32, u32, u32, u32, vpp, vp, vp]),
    "adh_conv3x3_workspace_bytes": (sz, [i32, i32, u32, u32, u32, u32, u32, u32]),
    "adh_conv3x3_kernel_name": (i32, [i32, i32, u32, u32, u32, u32, u32, u32, f32, ctypes.c_char_p, sz]),
    "adh_conv3x3_slab_fwd": (i32, [i32, u32, u32, u32, u32, u32, vp, vp, vp, f32, vp, sz, vp]),
    "adh_conv3x3_slab_fwd_tiles": (i32, [i32, u32, u32, u32, u32, u32, u32, vpp, vp, vpp, f32, vp, sz, vp]),
    "adh_conv3x3_slab_fwd_tiles_unexchanged": (i32, [i32, u32, u32, u32, u32, u32, u32, vpp, vp, vpp, f32, vp, sz, vp]),
    "adh_conv3x3_slab_bwd_data_tiles_reduced": (i32, [i32, u32, u32, u32, u32, u32, u32, vp, vpp, vpp, f32, vp, sz, vp]),
    "adh_conv3x3_unpadded_fwd_tiles": (i32, [i32, u32, u32, u32, u32, u32, u32, vpp, vp, vpp, f32, vp, sz, vp]),
    "adh_conv3x3_unpadded_fwd_residual_tiles": (i32, [i32, u32, u32, u32, u32, u32, u32, vpp, vp, vpp, vpp, vp]),
    "adh_conv3x3_unpadded_bwd_data_tiles": (i32, [i32, u32, u32, u32, u32, u32, u32, vp, vpp, vpp, f32, vp, sz, vp]),
    "adh_conv3x3_unpadded_bwd_filter_tiles": (i32, [i32, u32, u32, u32, u32, u32, u32, vpp, vpp, vp, f32, vp, sz, vp]),
    "adh_conv3x3_slab_fwd_tiles_static": (i32, [i32, u32, u32, u32, u32, u32, u32, vpp, vp, vpp, f32, vp]),
    "adh_conv3x3_slab_bwd_data": (i32, [i32, u32, u32, u32, u32, u32, vp, vp, vp, f32, vp, sz, vp]),
    "adh_conv3x3_slab_bwd_data_tiles": (i32, [i32, u32, u32, u32, u32, u32, u32, vp, vpp, vpp, f32, vp, sz, vp]),
    "adh_conv3x3_slab_bwd_filter": (i32, [i32, u32, u32, u32, u32, u32, vp, vp, vp, f32, vp, sz, vp]),
    "adh_conv3x3_slab_bwd_filter_tiles": (i32, [i32, u32, u32, u32, u32, u32, u32, vpp, vpp, vp, f32, vp, sz, vp]),
    "adh_conv3x3_slab_bwd_filter_tiles_unexchanged": (i32, [i32, u32, u32, u32, u32, u32, u32, vpp, vpp, vp, f32, vp, sz,
                                                            vp]),
    "adh_conv_bias_add_tiles": (i32, [i32, u32, u32, u32, u32, u32, vpp, vpp, vp]),
    "adh_conv_bwd_bias_workspace_bytes": (sz, [u32, u32, u32]),
    "adh_conv_bwd_bias_tiles": (i32, [i32, u32, u32, u32, u32, u32, vpp, vp, f32, vp, sz, vp]),
    "adh_conv2d_workspace_bytes": (sz, [i32, i32] + [u32] * 12),
    "adh_conv2d_slab_fwd_tiles": (i32, [i32] + [u32] * 12 + [vpp, vp, vpp, f32, vp, sz, vp]),
    "adh_conv2d_slab_fwd_bias_tiles": (i32, [i32] + [u32] * 12 + [vpp, vp, vpp, vpp, f32, vp, sz, vp]),
    "adh_conv2d_slab_bwd_data_tiles": (i32, [i32] + [u32] * 12 + [vp, vpp, vpp, f32, vp, sz, vp]),
    "adh_conv2d_slab_bwd_filter_tiles": (i32, [i32] + [u32] * 12 + [vpp, vpp, vp, f32, vp, sz, vp]),
    "adh_conv2d_unpadded_workspace_bytes": (sz, [i32, i32] + [u32] * 14),
    "adh_conv2d_unpadded_fwd_tiles": (i32, [i32] + [u32] * 14 + [vpp, vp, vpp, f32, vp, sz, vp]),
    "adh_conv2d_unpadded_bwd_data_tiles": (i32, [i32] + [u32] * 14 + [vp, vpp, vpp, f32, vp, sz, vp]),
    "adh_conv2d_unpadded_bwd_filter_tiles": (i32, [i32] + [u32] * 14 + [vpp, vpp, vp, f32, vp, sz, vp]),
    "adh_batchnorm2d_workspace_bytes": (sz, [u32, u32, u32]),
    "adh_batchnorm2d_fwd_tiles": (i32, [i32, i32, u32, u32, u32, u32, u32, f32, i32, u32, vpp, vpp, vpp, vpp, vpp, vpp, vpp,
                                        vpp, vpp, vpp, vp, sz, vp]),
    "adh_batchnorm2d_bwd_tiles": (i32, [i32, u32, u32, u32, u32, u32, i32, u32, vpp, vpp, vpp, vpp, vpp, vpp, vpp, vpp, vpp,
                                        f32, f32, vp, sz, vp]),
    "adh_relu_fwd": (i32, [i32, ctypes.c_uint64, vp, vp, vp]),
    "adh_relu_bwd": (i32, [i32, ctypes.c_uint64, vp, vp, vp, f32, vp]),
    "adh_sum_fwd": (i32, [i32, u32, ctypes.c_uint64, vpp, vp, vp]),
    "adh_pool2d_slab_fwd_tiles": (i32, [i32, i32, u32, u32, u32, u32, u32, u32, u32, u32, u32, vpp, vpp, vp]),
    "adh_pool2d_slab_fwd": (i32, [i32, i32, u32, u32, u32, u32, u32, u32, u32, u32, vp, vp, vp]),
    "adh_pool2d_slab_bwd_tiles": (i32, [i32, i32, u32, u32, u32, u32, u32, u32, u32, u32, u32, vpp, vpp, vpp, vpp, f32, vp]),
    "adh_pool2d_slab_bwd": (i32, [i32, i32, u32, u32, u32, u32, u32, u32, u32, u32, vp, vp, vp, vp, f32, vp]),
    "adh_pool2d_unpadded_supported": (i32, [i32, i32] + [u32] * 11),
    "adh_pool2d_unpadded_fwd_tiles": (i32, [i32, i32] + [u32] * 11 + [vpp, vpp, vp]),
    "adh_pool2d_unpadded_bwd_tiles": (i32, [i32, i32] + [u32] * 11 + [vpp, vpp, vpp, vpp, f32, vp]),
    "adh_softmax_fwd": (i32, [u32, u32, vp, vp, vp]),
    "adh_softmax_nll_loss_fwd": (i32, [u32, u32, vp, vp, vp, vp]),
    "adh_softmax_nll_loss_bwd": (i32, [u32, u32, vp, vp, vp, vp, vp]),
    "adh_softmax_xent_fwd": (i32, [u32, u32, vp, vp, vp, vp, vp]),
    "adh_softmax_nll_loss_bwd_scaled": (i32, [u32, u32, vp, vp, vp, f32, f32, vp, vp]),
    "adh_softmax_xent_fwd_bwd": (i32, [u32, u32, vp, vp, vp, f32, vp, vp, f32, vp, vp]),
    "adh_scale_add_f32": (i32, [u64, f32, vp, f32, vp, vp]),
    "adh_add_online_f32": (i32, [u64, f32, vp, vp, vp]),
    "adh_stat_step_f32": (i32, [u64, f32, vp, vp, vp, vp]),
    "adh_flat_store_f32": (i32, [u32, vpp, ctypes.POINTER(u64), u64, vp, vp]),
    "adh_flat_load_f32": (i32, [u32, vpp, ctypes.POINTER(u64), u64, vp, vp]),
    "adh_sgd_step_f32": (i32, [u64, u32, vpp, f32, f32, f32, f32, i32, vp, vp, vp, vp, vp]),
}


def build(force=True):
    """Compile libadh.so for gfx950 with hipcc (cross-compiles without a GPU)."""
    args = ["make", "-s", "-C", CSRC, "-j8"]
    if force:
        args.append("-B")
    subprocess.check_call(args)
    return LIB_PATH


class AdhError(RuntimeError):
    def __init__(self, code, what):
        self.code = code
        super().__init__("%s failed: %d (%s)" % (what, code, lib().adh_error_string(code).decode()))


_lib = None


def lib():
    """The loaded library.  Raises if it has not been built: there is no CPU fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libadh.so is not built (%s); run __graft_entry__.build() or "
                               "`make -C arraydiff_cuda_amd/csrc`" % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)  # AttributeError if a declared symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(code, what="adh call"):
    if code != 0:
        raise AdhError(code, what)
    return code


def ptr_table(ptrs):
    """Host array of device pointers from ints / None."""
    arr = (ctypes.c_void_p * len(ptrs))(*[p if p else None for p in ptrs])
    return ctypes.cast(arr, vpp), arr


# ---------------------------------------------------------------------------
# torch-tensor convenience wrappers (tests / bench).  Tensors must live on the GPU.
# ---------------------------------------------------------------------------
def _dt(t):
    import torch
    if t.dtype == torch.float32:
        return ADH_F32
    if t.dtype == torch.bfloat16:
        return ADH_BF16
    raise TypeError("dtype %s not supported" % t.dtype)


def _dev(*ts):
    for t in ts:
        if t is not None and (not t.is_cuda or not t.is_contiguous()):
            raise ValueError("tensors must be contiguous GPU tensors")


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _tbl(ts):
    return ptr_table([t.data_ptr() for t in ts])


def fill_f32(x, v):
    _dev(x)
    return lib().adh_fill_f32(x.numel(), v, x.data_ptr(), _stream())


def add_f32(x, y):
    _dev(x, y)
    return lib().adh_add_f32(x.numel(), x.data_ptr(), y.data_ptr(), _stream())


def halo_exchange(tiles, grid_w, grid_h, p, W, H, C, N, rank=None):
    _dev(*tiles)
    tb, keep = _tbl(tiles)
    if rank is None:
        return lib().adh_halo_exchange_nchw(_dt(tiles[0]), grid_w, grid_h, p, W, H, C, N, tb, _stream())
    return lib().adh_halo_exchange_nchw_rank(_dt(tiles[0]), grid_w, grid_h, rank, p, W, H, C, N, tb, _stream())


def halo_reduce(tiles, grid_w, grid_h, p, W, H, C, N, rank=None):
    _dev(*tiles)
    tb, keep = _tbl(tiles)
    if rank is None:
        return lib().adh_halo_reduce_nchw(_dt(tiles[0]), grid_w, grid_h, p, W, H, C, N, tb, _stream())
    return lib().adh_halo_reduce_nchw_rank(_dt(tiles[0]), grid_w, grid_h, rank, p, W, H, C, N, tb, _stream())


def _padlike(name, p, W, H, C, N, a, b):
    _dev(a, b)
    return getattr(lib(), name)(_dt(a), p, W, H, C, N, a.data_ptr(), b.data_ptr(), _stream())


def halo_pad(p, W, H, C, N, x, y):
    return _padlike("adh_halo_pad_nchw", p, W, H, C, N, x, y)


def halo_pad_add(p, W, H, C, N, x, y):
    return _padlike("adh_halo_pad_add_nchw", p, W, H, C, N, x, y)


def halo_unpad(p, W, H, C, N, x, y):
    return _padlike("adh_halo_unpad_nchw", p, W, H, C, N, x, y)


def halo_unpad_add(p, W, H, C, N, x, y):
    return _padlike("adh_halo_unpad_add_nchw", p, W, H, C, N, x, y)


def halo_repad(ps, pd, W, H, C, N, x, y):
    _dev(x, y)
    return lib().adh_halo_repad_nchw(_dt(x), ps, pd, W, H, C, N, x.data_ptr(), y.data_ptr(), _stream())


def slice_nchw(add, count, N, src, src_dims, src_off, dst, dst_dims, dst_off):
    _dev(src, dst)
    fn = lib().adh_slice_add_nchw if add else lib().adh_slice_copy_nchw
    return fn(_dt(src), count[0], count[1], count[2], N, src.data_ptr(), src_dims[0], src_dims[1], src_dims[2],
              src_off[0], src_off[1], src_off[2], dst.data_ptr(), dst_dims[0], dst_dims[1], dst_dims[2],
              dst_off[0], dst_off[1], dst_off[2], _stream())


def tiles_pack(K, p, W, H, C, N, x, tiles):
    _dev(x, *tiles)
    tb, keep = _tbl(tiles)
    return lib().adh_tiles_pack_nchw(_dt(x), K, p, W, H, C, N, x.data_ptr(), tb, _stream())


def tiles_unpack(K, p, W, H, C, N, tiles, y):
    _dev(y, *tiles)
    tb, keep = _tbl(tiles)
    return lib().adh_tiles_unpack_nchw(_dt(y), K, p, W, H, C, N, tb, y.data_ptr(), _stream())


def conv_workspace_bytes(which, dtype, K, N, Cin, Cout, H, W):
    return lib().adh_conv3x3_workspace_bytes(which, dtype, K, N, Cin, Cout, H, W)


def _ws(ws):
    if ws is None:
        return None, 0
    return ws.data_ptr(), ws.numel() * ws.element_size()


def conv_fwd_tiles(xs, w, ys, N, Cin, Cout, H, W, beta=0.0, ws=None, unexchanged=False):
    """unexchanged: xs are the row tiles of one activation in rank order whose inner halo rows have not been
    exchanged; the result equals halo_exchange followed by the ordinary forward."""
    _dev(w, *xs, *ys)
    xt, k1 = _tbl(xs)
    yt, k2 = _tbl(ys)
    wp, wb = _ws(ws)
    fn = lib().adh_conv3x3_slab_fwd_tiles_unexchanged if unexchanged else lib().adh_conv3x3_slab_fwd_tiles
    return fn(_dt(xs[0]), len(xs), N, Cin, Cout, H, W, xt, w.data_ptr(), yt, beta,
                                            wp, wb, _stream())


def conv_bwd_data_tiles(w, dys, dxs, N, Cin, Cout, H, W, beta=0.0, ws=None, reduced=False):
    """reduced: dys are the row tiles of one gradient in rank order; the interior of every dx tile comes out as
    after backward-data followed by halo_reduce."""
    _dev(w, *dys, *dxs)
    dt, k1 = _tbl(dys)
    xt, k2 = _tbl(dxs)
    wp, wb = _ws(ws)
    fn = lib().adh_conv3x3_slab_bwd_data_tiles_reduced if reduced else lib().adh_conv3x3_slab_bwd_data_tiles
    return fn(_dt(dys[0]), len(dys), N, Cin, Cout, H, W, w.data_ptr(), dt, xt, beta, wp, wb, _stream())


def conv_unpadded_fwd_tiles(xs, w, ys, N, Cin, Cout, H, W, beta=0.0, ws=None):
    """xs, ys: the row tiles (H x W, no halo) of one tensor in rank order."""
    _dev(w, *xs, *ys)
    xt, k1 = _tbl(xs)
    yt, k2 = _tbl(ys)
    wp, wb = _ws(ws)
    return lib().adh_conv3x3_unpadded_fwd_tiles(_dt(xs[0]), len(xs), N, Cin, Cout, H, W, xt, w.data_ptr(), yt, beta, wp,
                                                wb, _stream())


def conv_unpadded_fwd_residual_tiles(xs, w, res, ys, N, Cin, Cout, H, W):
    """ys[t] = conv(xs, w)[t] + res[t] over tiles without halo (fp32)."""
    _dev(w, *xs, *res, *ys)
    xt, k1 = _tbl(xs)
    rt, k2 = _tbl(res)
    yt, k3 = _tbl(ys)
    return lib().adh_conv3x3_unpadded_fwd_residual_tiles(_dt(xs[0]), len(xs), N, Cin, Cout, H, W, xt, w.data_ptr(), rt, yt,
                                                         _stream())


def conv_unpadded_bwd_data_tiles(w, dys, dxs, N, Cin, Cout, H, W, beta=0.0, ws=None):
    _dev(w, *dys, *dxs)
    dt, k1 = _tbl(dys)
    xt, k2 = _tbl(dxs)
    wp, wb = _ws(ws)
    return lib().adh_conv3x3_unpadded_bwd_data_tiles(_dt(dys[0]), len(dys), N, Cin, Cout, H, W, w.data_ptr(), dt, xt,
                                                     beta, wp, wb, _stream())


def conv_unpadded_bwd_filter_tiles(xs, dys, dw, N, Cin, Cout, H, W, beta=0.0, ws=None):
    _dev(dw, *xs, *dys)
    xt, k1 = _tbl(xs)
    dt, k2 = _tbl(dys)
    wp, wb = _ws(ws)
    return lib().adh_conv3x3_unpadded_bwd_filter_tiles(_dt(xs[0]), len(xs), N, Cin, Cout, H, W, xt, dt, dw.data_ptr(),
                                                       beta, wp, wb, _stream())


def conv_bias_add_tiles(biases, ys, N, C, H, W):
    """ys[t][n,c,h,w] += biases[t][c]; biases are fp32 vectors of C (entries may repeat)."""
    _dev(*biases, *ys)
    bt, k1 = _tbl(biases)
    yt, k2 = _tbl(ys)
    return lib().adh_conv_bias_add_tiles(_dt(ys[0]), len(ys), N, C, H, W, bt, yt, _stream())


def conv_bwd_bias_workspace_bytes(K, N, C):
    return lib().adh_conv_bwd_bias_workspace_bytes(K, N, C)


def conv_bwd_bias_tiles(dys, db, N, C, H, W, beta=0.0, ws=None):
    """db[c] = beta*db[c] + sum over tiles, n, h, w of dys[t][n,c,h,w]."""
    _dev(db, *dys)
    dt, k1 = _tbl(dys)
    wp, wb = _ws(ws)
    return lib().adh_conv_bwd_bias_tiles(_dt(dys[0]), len(dys), N, C, H, W, dt, db.data_ptr(), beta, wp, wb, _stream())


def conv2d_workspace_bytes(which, dtype, K, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw):
    return lib().adh_conv2d_workspace_bytes(which, dtype, K, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw)


def conv2d_fwd_tiles(xs, w, ys, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, beta=0.0, ws=None):
    _dev(*xs, w, *ys)
    xt, k1 = _tbl(xs)
    yt, k2 = _tbl(ys)
    wp, wb = _ws(ws)
    return lib().adh_conv2d_slab_fwd_tiles(_dt(xs[0]), len(xs), N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, xt,
                                           w.data_ptr(), yt, beta, wp, wb, _stream())


def conv2d_fwd_bias_tiles(xs, w, biases, ys, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, beta=0.0, ws=None):
    """conv2d_fwd_tiles followed by ys[t] += biases[t] per channel, in the convolution's stores where its kernel can."""
    _dev(*xs, w, *biases, *ys)
    xt, k1 = _tbl(xs)
    bt, k3 = _tbl(biases)
    yt, k2 = _tbl(ys)
    wp, wb = _ws(ws)
    return lib().adh_conv2d_slab_fwd_bias_tiles(_dt(xs[0]), len(xs), N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, xt,
                                                w.data_ptr(), bt, yt, beta, wp, wb, _stream())


def conv2d_bwd_data_tiles(w, dys, dxs, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, beta=0.0, ws=None):
    _dev(w, *dys, *dxs)
    dt, k1 = _tbl(dys)
    gt, k2 = _tbl(dxs)
    wp, wb = _ws(ws)
    return lib().adh_conv2d_slab_bwd_data_tiles(_dt(dys[0]), len(dys), N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw,
                                                w.data_ptr(), dt, gt, beta, wp, wb, _stream())


def conv2d_bwd_filter_tiles(xs, dys, dw, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw_, beta=0.0, ws=None):
    _dev(*xs, *dys, dw)
    xt, k1 = _tbl(xs)
    dt, k2 = _tbl(dys)
    wp, wb = _ws(ws)
    return lib().adh_conv2d_slab_bwd_filter_tiles(_dt(xs[0]), len(xs), N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw_,
                                                  xt, dt, dw.data_ptr(), beta, wp, wb, _stream())


def conv2d_unpadded_workspace_bytes(which, dtype, K, N, Cin, Cout, H, W, kh, kw, sh, sw, dh, dw, pad_h, pad_w):
    return lib().adh_conv2d_unpadded_workspace_bytes(which, dtype, K, N, Cin, Cout, H, W, kh, kw, sh, sw, dh, dw, pad_h, pad_w)


def conv2d_unpadded_fwd_tiles(xs, w, ys, N, Cin, Cout, H, W, kh, kw, sh, sw, dh, dw, pad_h, pad_w, beta=0.0, ws=None):
    """Row tiles without halo, any window / stride / dilation: rows outside a tile come from its neighbours."""
    _dev(*xs, w, *ys)
    xt, k1 = _tbl(xs)
    yt, k2 = _tbl(ys)
    wp, wb = _ws(ws)
    return lib().adh_conv2d_unpadded_fwd_tiles(_dt(xs[0]), len(xs), N, Cin, Cout, H, W, kh, kw, sh, sw, dh, dw, pad_h, pad_w,
                                               xt, w.data_ptr(), yt, beta, wp, wb, _stream())


def conv2d_unpadded_bwd_data_tiles(w, dys, dxs, N, Cin, Cout, H, W, kh, kw, sh, sw, dh, dw, pad_h, pad_w, beta=0.0, ws=None):
    _dev(w, *dys, *dxs)
    dt, k1 = _tbl(dys)
    gt, k2 = _tbl(dxs)
    wp, wb = _ws(ws)
    return lib().adh_conv2d_unpadded_bwd_data_tiles(_dt(dys[0]), len(dys), N, Cin, Cout, H, W, kh, kw, sh, sw, dh, dw, pad_h,
                                                    pad_w, w.data_ptr(), dt, gt, beta, wp, wb, _stream())


def conv2d_unpadded_bwd_filter_tiles(xs, dys, dw, N, Cin, Cout, H, W, kh, kw, sh, sw, dh, dw_, pad_h, pad_w, beta=0.0, ws=None):
    _dev(*xs, *dys, dw)
    xt, k1 = _tbl(xs)
    dt, k2 = _tbl(dys)
    wp, wb = _ws(ws)
    return lib().adh_conv2d_unpadded_bwd_filter_tiles(_dt(xs[0]), len(xs), N, Cin, Cout, H, W, kh, kw, sh, sw, dh, dw_, pad_h,
                                                      pad_w, xt, dt, dw.data_ptr(), beta, wp, wb, _stream())


def _opt_tbl(ts):
    if ts is None:
        return None, None
    return _tbl(ts)


def batchnorm_workspace_bytes(K, N, C):
    return lib().adh_batchnorm2d_workspace_bytes(K, N, C)


def batchnorm_fwd_tiles(xs, scales, shifts, ys, N, C, H, W, eps=1e-5, relu=0, out_halo=0, training=True, fixed_means=None,
                        fixed_vars=None, run_means=None, run_vars=None, save_means=None, save_invstds=None, ws=None):
    _dev(*xs, *ys, *scales, *shifts)
    tabs = [_tbl(xs), _tbl(scales), _tbl(shifts), _opt_tbl(fixed_means), _opt_tbl(fixed_vars), _tbl(ys), _opt_tbl(run_means),
            _opt_tbl(run_vars), _opt_tbl(save_means), _opt_tbl(save_invstds)]
    wp, wb = _ws(ws)
    return lib().adh_batchnorm2d_fwd_tiles(_dt(xs[0]), 1 if training else 0, len(xs), N, C, H, W, eps, relu, out_halo,
                                           *[t[0] for t in tabs], wp, wb, _stream())


def batchnorm_bwd_tiles(xs, dys, scales, shifts, save_means, save_invstds, dxs, dscales, dshifts, N, C, H, W, relu=0,
                        dy_halo=0, beta_data=0.0, beta_param=0.0, ws=None):
    _dev(*xs, *dys, *dxs)
    tabs = [_tbl(xs), _tbl(dys), _tbl(scales), _opt_tbl(shifts), _tbl(save_means), _tbl(save_invstds), _tbl(dxs),
            _tbl(dscales), _tbl(dshifts)]
    wp, wb = _ws(ws)
    return lib().adh_batchnorm2d_bwd_tiles(_dt(xs[0]), len(xs), N, C, H, W, relu, dy_halo, *[t[0] for t in tabs],
                                           beta_data, beta_param, wp, wb, _stream())


def relu_fwd(x, y):
    _dev(x, y)
    return lib().adh_relu_fwd(_dt(x), x.numel(), x.data_ptr(), y.data_ptr(), _stream())


def relu_bwd(y, dy, dx, beta=0.0):
    _dev(y, dy, dx)
    return lib().adh_relu_bwd(_dt(y), y.numel(), y.data_ptr(), dy.data_ptr(), dx.data_ptr(), beta, _stream())


def sum_fwd(xs, y):
    _dev(*xs, y)
    xt, keep = _tbl(xs)
    return lib().adh_sum_fwd(_dt(y), len(xs), y.numel(), xt, y.data_ptr(), _stream())


def scale_add(alpha, x, beta, y):
    """y = alpha*x + beta*y over flat fp32 tensors."""
    _dev(x, y)
    return lib().adh_scale_add_f32(y.numel(), alpha, x.data_ptr(), beta, y.data_ptr(), _stream())


def add_online(alpha, x, y):
    """y = y + alpha*(x - y)."""
    _dev(x, y)
    return lib().adh_add_online_f32(y.numel(), alpha, x.data_ptr(), y.data_ptr(), _stream())


def stat_step(rate, avg_stat, running_stat, stat):
    _dev(avg_stat, running_stat, stat)
    return lib().adh_stat_step_f32(stat.numel(), rate, avg_stat.data_ptr(), running_stat.data_ptr(), stat.data_ptr(),
                                   _stream())


def _lens(arrays):
    return (u64 * len(arrays))(*[a.numel() for a in arrays])


def flat_store(arrays, flat, offset=0):
    """Copy the arrays, in order, into consecutive ranges of `flat` starting at element `offset`."""
    _dev(*arrays, flat)
    t, keep = _tbl(arrays)
    return lib().adh_flat_store_f32(len(arrays), t, _lens(arrays), offset, flat.data_ptr(), _stream())


def flat_load(arrays, flat, offset=0):
    """The inverse of flat_store: consecutive ranges of `flat` into the arrays."""
    _dev(*arrays, flat)
    t, keep = _tbl(arrays)
    return lib().adh_flat_load_f32(len(arrays), t, _lens(arrays), offset, flat.data_ptr(), _stream())


def sgd_step(grads, param, momentum_grad, lagged_param=None, sum_grad=None, l2_reg=0.0, momentum=0.0, step_size=0.0,
             next_step_size=0.0, nesterov=False):
    """One fused optimizer update over flat fp32 vectors; grads is the list of per-rank gradient vectors."""
    _dev(*grads, param, momentum_grad)
    t, keep = _tbl(grads)
    return lib().adh_sgd_step_f32(param.numel(), len(grads), t, l2_reg, momentum, step_size, next_step_size,
                                  int(bool(nesterov)), param.data_ptr(), momentum_grad.data_ptr(),
                                  lagged_param.data_ptr() if lagged_param is not None else None,
                                  sum_grad.data_ptr() if sum_grad is not None else None, _stream())


def pool_fwd_tiles(mode, xs, ys, N, C, HP, WP, wh, ww, sh, sw):
    _dev(*xs, *ys)
    xt, k1 = _tbl(xs)
    yt, k2 = _tbl(ys)
    return lib().adh_pool2d_slab_fwd_tiles(_dt(xs[0]), mode, len(xs), N, C, HP, WP, wh, ww, sh, sw, xt, yt, _stream())


def pool_bwd_tiles(mode, xs, ys, dys, dxs, N, C, HP, WP, wh, ww, sh, sw, beta=0.0):
    _dev(*xs, *ys, *dys, *dxs)
    xt, k1 = _tbl(xs)
    yt, k2 = _tbl(ys)
    dt, k3 = _tbl(dys)
    gt, k4 = _tbl(dxs)
    return lib().adh_pool2d_slab_bwd_tiles(_dt(dys[0]), mode, len(dys), N, C, HP, WP, wh, ww, sh, sw, xt, yt, dt, gt,
                                           beta, _stream())


def pool_unpadded_fwd_tiles(mode, xs, ys, N, C, H, W, wh, ww, sh, sw, pad_h, pad_w):
    """Pooling over row tiles without halo: rows outside a tile come from its neighbours, zeros outside the tensor."""
    _dev(*xs, *ys)
    xt, k1 = _tbl(xs)
    yt, k2 = _tbl(ys)
    return lib().adh_pool2d_unpadded_fwd_tiles(_dt(xs[0]), mode, len(xs), N, C, H, W, wh, ww, sh, sw, pad_h, pad_w, xt, yt,
                                               _stream())


def pool_unpadded_bwd_tiles(mode, xs, ys, dys, dxs, N, C, H, W, wh, ww, sh, sw, pad_h, pad_w, beta=0.0):
    _dev(*xs, *dys, *dxs)
    xt, k1 = _tbl(xs)
    yt, k2 = _opt_tbl(ys)
    dt, k3 = _tbl(dys)
    gt, k4 = _tbl(dxs)
    return lib().adh_pool2d_unpadded_bwd_tiles(_dt(dys[0]), mode, len(dys), N, C, H, W, wh, ww, sh, sw, pad_h, pad_w, xt, yt,
                                               dt, gt, beta, _stream())


def conv_bwd_filter_tiles(xs, dys, dw, N, Cin, Cout, H, W, beta=0.0, ws=None, unexchanged=False):
    _dev(dw, *xs, *dys)
    xt, k1 = _tbl(xs)
    dt, k2 = _tbl(dys)
    wp, wb = _ws(ws)
    fn = (lib().adh_conv3x3_slab_bwd_filter_tiles_unexchanged if unexchanged
          else lib().adh_conv3x3_slab_bwd_filter_tiles)
    return fn(_dt(xs[0]), len(xs), N, Cin, Cout, H, W, xt, dt, dw.data_ptr(), beta, wp, wb, _stream())


def softmax_fwd(x, y):
    _dev(x, y)
    N, C = x.shape
    return lib().adh_softmax_fwd(C, N, x.data_ptr(), y.data_ptr(), _stream())


def softmax_xent_fwd(x, label, y, loss):
    _dev(x, label, y, loss)
    N, C = x.shape
    return lib().adh_softmax_xent_fwd(C, N, x.data_ptr(), label.data_ptr(), y.data_ptr(), loss.data_ptr(), _stream())


def softmax_nll_loss_fwd(y, label, loss):
    _dev(y, label, loss)
    N, C = y.shape
    return lib().adh_softmax_nll_loss_fwd(C, N, y.data_ptr(), label.data_ptr(), loss.data_ptr(), _stream())


def softmax_nll_loss_bwd(y, label, dloss, dx):
    _dev(y, label, dloss, dx)
    N, C = y.shape
    return lib().adh_softmax_nll_loss_bwd(C, N, y.data_ptr(), label.data_ptr(), dloss.data_ptr(), dx.data_ptr(),
                                          _stream())


def softmax_nll_loss_bwd_scaled(y, label, dloss, dloss_all, beta, dx):
    """dx = beta*dx + dl*(y - onehot); dloss None: every example's dl is dloss_all."""
    _dev(y, label, dx)
    N, C = y.shape
    return lib().adh_softmax_nll_loss_bwd_scaled(C, N, y.data_ptr(), label.data_ptr(),
                                                 None if dloss is None else dloss.data_ptr(), dloss_all, beta,
                                                 dx.data_ptr(), _stream())


def softmax_xent_fwd_bwd(x, label, dloss, dloss_all, y, loss, beta, dx):
    _dev(x, label, y, loss, dx)
    N, C = x.shape
    return lib().adh_softmax_xent_fwd_bwd(C, N, x.data_ptr(), label.data_ptr(),
                                          None if dloss is None else dloss.data_ptr(), dloss_all, y.data_ptr(),
                                          loss.data_ptr(), beta, dx.data_ptr(), _stream())


def conv_kernel_name(which, dtype, K, N, Cin, Cout, H, W, beta=0.0):
    """Name of the kernel instance a 3x3 forward / backward-data call of this shape runs."""
    buf = ctypes.create_string_buffer(256)
    check(lib().adh_conv3x3_kernel_name(which, dtype, K, N, Cin, Cout, H, W, beta, buf, 256), "kernel name")
    return buf.value.decode()
