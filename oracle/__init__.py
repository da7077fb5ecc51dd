"""ctypes binding of the CPU oracle (``adh_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU
baseline.  The product package never imports this module.

All arrays are numpy, C-contiguous, NCHW with W fastest (numpy shape
``(N, C, H, W)``).  bf16 tensors are carried as ``uint16`` bit patterns.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F32 = 0
BF16 = 1
EXCH = 0
REDUCE = 1
OP_COPY = 0
OP_ADD = 1


def build(force=False):
    """Compile liboracle.so with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "liboracle.so"])
    return _LIB_PATH


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    lib.orc_now_seconds.restype = ctypes.c_double
    lib.orc_bf16_to_f32.restype = ctypes.c_float
    lib.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
    lib.orc_f32_to_bf16.restype = ctypes.c_uint16
    lib.orc_f32_to_bf16.argtypes = [ctypes.c_float]
    lib.orc_padded_index.restype = ctypes.c_int64
    lib.orc_padded_index.argtypes = [ctypes.c_int64] * 8
    return lib


_lib = _load()

_u32 = ctypes.c_uint32
_vp = ctypes.c_void_p


def _ptr(a):
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"], "need C-contiguous numpy"
    return ctypes.c_void_p(a.ctypes.data)


def _ptr_array(arrs):
    return (ctypes.c_void_p * len(arrs))(*[a.ctypes.data if a is not None else None for a in arrs])


def dtype_code(a):
    if a.dtype == np.float32:
        return F32
    if a.dtype == np.uint16:
        return BF16
    raise TypeError("oracle tensors are float32 or uint16 (bf16 bits), got %s" % a.dtype)


def f32_to_bf16(x):
    """Round-to-nearest-even float32 -> bf16 bit patterns (vectorised twin of orc_f32_to_bf16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def padded_index(w, h, c, n, p, W, H, C):
    return _lib.orc_padded_index(w, h, c, n, p, W, H, C)


def fill_f32(x, v):
    _lib.orc_fill_f32(ctypes.c_uint64(x.size), ctypes.c_float(v), _ptr(x))


def add_f32(x, y):
    _lib.orc_add_f32(ctypes.c_uint64(x.size), _ptr(x), _ptr(y))


def halo_op_rank(which, grid_w, grid_h, rank, p, W, H, C, N, tiles):
    dt = dtype_code(tiles[0])
    return _lib.orc_halo_op_rank(which, dt, _u32(grid_w), _u32(grid_h), _u32(rank), _u32(p), _u32(W),
                                 _u32(H), _u32(C), _u32(N), _ptr_array(tiles))


def halo_op(which, grid_w, grid_h, p, W, H, C, N, tiles):
    dt = F32
    for t in tiles:
        if t is not None:
            dt = dtype_code(t)
    return _lib.orc_halo_op(which, dt, _u32(grid_w), _u32(grid_h), _u32(p), _u32(W), _u32(H), _u32(C),
                            _u32(N), _ptr_array(tiles))


def slice_nchw(op, count, N, src, src_dims, src_off, dst, dst_dims, dst_off):
    """count/src_dims/src_off/... are (w, h, c) triples."""
    dt = dtype_code(src)
    assert dtype_code(dst) == dt
    return _lib.orc_slice_nchw(op, dt, _u32(count[0]), _u32(count[1]), _u32(count[2]), _u32(N),
                               _ptr(src), _u32(src_dims[0]), _u32(src_dims[1]), _u32(src_dims[2]),
                               _u32(src_off[0]), _u32(src_off[1]), _u32(src_off[2]),
                               _ptr(dst), _u32(dst_dims[0]), _u32(dst_dims[1]), _u32(dst_dims[2]),
                               _u32(dst_off[0]), _u32(dst_off[1]), _u32(dst_off[2]))


def _pad_like(fn, p, W, H, C, N, a, b):
    dt = dtype_code(a)
    assert dtype_code(b) == dt
    fn(dt, _u32(p), _u32(W), _u32(H), _u32(C), _u32(N), _ptr(a), _ptr(b))


def halo_pad(p, W, H, C, N, x_packed, y_padded):
    _pad_like(_lib.orc_halo_pad, p, W, H, C, N, x_packed, y_padded)


def halo_pad_add(p, W, H, C, N, x_packed, y_padded):
    _pad_like(_lib.orc_halo_pad_add, p, W, H, C, N, x_packed, y_padded)


def halo_unpad(p, W, H, C, N, x_padded, y_packed):
    _pad_like(_lib.orc_halo_unpad, p, W, H, C, N, x_padded, y_packed)


def halo_unpad_add(p, W, H, C, N, x_padded, y_packed):
    _pad_like(_lib.orc_halo_unpad_add, p, W, H, C, N, x_padded, y_packed)


def halo_repad(p_src, p_dst, W, H, C, N, x_padded, y_padded):
    dt = dtype_code(x_padded)
    _lib.orc_halo_repad(dt, _u32(p_src), _u32(p_dst), _u32(W), _u32(H), _u32(C), _u32(N),
                        _ptr(x_padded), _ptr(y_padded))


def tiles_pack(K, p, W, H, C, N, x_unsplit, tiles):
    dt = dtype_code(x_unsplit)
    scratch = np.empty((N, C, max(H // max(K, 1), 1), W), dtype=x_unsplit.dtype)
    return _lib.orc_tiles_pack(dt, _u32(K), _u32(p), _u32(W), _u32(H), _u32(C), _u32(N),
                               _ptr(x_unsplit), _ptr_array(tiles), _ptr(scratch))


def tiles_unpack(K, p, W, H, C, N, tiles, y_unsplit):
    dt = dtype_code(y_unsplit)
    scratch = np.empty((N, C, max(H // max(K, 1), 1), W), dtype=y_unsplit.dtype)
    return _lib.orc_tiles_unpack(dt, _u32(K), _u32(p), _u32(W), _u32(H), _u32(C), _u32(N),
                                 _ptr_array(tiles), _ptr(y_unsplit), _ptr(scratch))


def hardware_threads():
    """Hardware threads of this host (what std::thread::hardware_concurrency() reports)."""
    _lib.orc_hardware_threads.restype = ctypes.c_uint32
    return int(_lib.orc_hardware_threads())


def halo_op_threaded(which, grid_w, grid_h, p, W, H, C, N, tiles):
    """halo_op with one host thread per rank (the reference runs one kernel per rank)."""
    dt = dtype_code(tiles[0])
    return _lib.orc_halo_op_threaded(which, dt, _u32(grid_w), _u32(grid_h), _u32(p), _u32(W), _u32(H), _u32(C),
                                     _u32(N), _ptr_array(tiles))


def tiles_pack_threaded(K, p, W, H, C, N, x_unsplit, tiles):
    dt = dtype_code(x_unsplit)
    scratch = np.empty((max(K, 1), N, C, max(H // max(K, 1), 1), W), dtype=x_unsplit.dtype)
    return _lib.orc_tiles_pack_threaded(dt, _u32(K), _u32(p), _u32(W), _u32(H), _u32(C), _u32(N),
                                        _ptr(x_unsplit), _ptr_array(tiles), _ptr(scratch))


def tiles_unpack_threaded(K, p, W, H, C, N, tiles, y_unsplit):
    dt = dtype_code(y_unsplit)
    scratch = np.empty((max(K, 1), N, C, max(H // max(K, 1), 1), W), dtype=y_unsplit.dtype)
    return _lib.orc_tiles_unpack_threaded(dt, _u32(K), _u32(p), _u32(W), _u32(H), _u32(C), _u32(N),
                                          _ptr_array(tiles), _ptr(y_unsplit), _ptr(scratch))


def conv_slab_fwd_f32_threaded(x_pads, wt, ys):
    """conv_slab_fwd_f32 of every tile, one host thread per tile."""
    N, Cin, Hp, Wp = x_pads[0].shape
    Cout, _, k, _ = wt.shape
    H, W = Hp - k + 1, Wp - k + 1
    return _lib.orc_conv_slab_fwd_f32_threaded(_u32(len(x_pads)), _u32(N), _u32(Cin), _u32(Cout), _u32(H), _u32(W),
                                               _u32(k), _ptr_array(x_pads), _ptr(wt), _ptr_array(ys))


def conv_slab_fwd(x_pad, wt, y, beta=0.0):
    N, Cin, Hp, Wp = x_pad.shape
    Cout, _, k, _ = wt.shape
    H, W = Hp - k + 1, Wp - k + 1
    assert y.shape == (N, Cout, H, W)
    _lib.orc_conv_slab_fwd(_u32(N), _u32(Cin), _u32(Cout), _u32(H), _u32(W), _u32(k), _ptr(x_pad),
                           _ptr(wt), ctypes.c_float(beta), _ptr(y))


def conv_slab_fwd_f32(x_pad, wt, y):
    N, Cin, Hp, Wp = x_pad.shape
    Cout, _, k, _ = wt.shape
    H, W = Hp - k + 1, Wp - k + 1
    _lib.orc_conv_slab_fwd_f32(_u32(N), _u32(Cin), _u32(Cout), _u32(H), _u32(W), _u32(k),
                               _ptr(x_pad), _ptr(wt), _ptr(y))


def conv_slab_bwd_data(wt, dy, dx_pad, beta=0.0):
    N, Cout, H, W = dy.shape
    _, Cin, k, _ = wt.shape
    assert dx_pad.shape == (N, Cin, H + k - 1, W + k - 1)
    _lib.orc_conv_slab_bwd_data(_u32(N), _u32(Cin), _u32(Cout), _u32(H), _u32(W), _u32(k), _ptr(wt),
                                _ptr(dy), ctypes.c_float(beta), _ptr(dx_pad))


def conv_slab_bwd_filter(x_pad, dy, dw, beta=0.0):
    N, Cout, H, W = dy.shape
    _, Cin, k, _ = dw.shape
    assert x_pad.shape == (N, Cin, H + k - 1, W + k - 1)
    _lib.orc_conv_slab_bwd_filter(_u32(N), _u32(Cin), _u32(Cout), _u32(H), _u32(W), _u32(k),
                                  _ptr(x_pad), _ptr(dy), ctypes.c_float(beta), _ptr(dw))


def conv2d_out_dims(HP, WP, kh, kw, sh, sw, dh, dw):
    return (HP - ((kh - 1) * dh + 1)) // sh + 1, (WP - ((kw - 1) * dw + 1)) // sw + 1


def conv2d_slab_fwd(x_pad, wt, sh, sw, dh, dw, y, beta=0.0):
    """General slab conv: x_pad (N,Cin,HP,WP), wt (Cout,Cin,kh,kw), pad 0, stride (sh,sw), dilation (dh,dw)."""
    N, Cin, HP, WP = x_pad.shape
    Cout, _, kh, kw = wt.shape
    assert y.shape == (N, Cout) + conv2d_out_dims(HP, WP, kh, kw, sh, sw, dh, dw)
    _lib.orc_conv2d_slab_fwd(_u32(N), _u32(Cin), _u32(Cout), _u32(HP), _u32(WP), _u32(kh), _u32(kw), _u32(sh), _u32(sw),
                             _u32(dh), _u32(dw), _ptr(x_pad), _ptr(wt), ctypes.c_float(beta), _ptr(y))


def conv2d_slab_bwd_data(wt, dy, sh, sw, dh, dw, dx_pad, beta=0.0):
    N, Cin, HP, WP = dx_pad.shape
    Cout, _, kh, kw = wt.shape
    assert dy.shape == (N, Cout) + conv2d_out_dims(HP, WP, kh, kw, sh, sw, dh, dw)
    _lib.orc_conv2d_slab_bwd_data(_u32(N), _u32(Cin), _u32(Cout), _u32(HP), _u32(WP), _u32(kh), _u32(kw), _u32(sh),
                                  _u32(sw), _u32(dh), _u32(dw), _ptr(wt), _ptr(dy), ctypes.c_float(beta), _ptr(dx_pad))


def conv2d_slab_bwd_filter(x_pad, dy, sh, sw, dh, dw, dwt, beta=0.0):
    N, Cin, HP, WP = x_pad.shape
    Cout, _, kh, kw = dwt.shape
    assert dy.shape == (N, Cout) + conv2d_out_dims(HP, WP, kh, kw, sh, sw, dh, dw)
    _lib.orc_conv2d_slab_bwd_filter(_u32(N), _u32(Cin), _u32(Cout), _u32(HP), _u32(WP), _u32(kh), _u32(kw), _u32(sh),
                                    _u32(sw), _u32(dh), _u32(dw), _ptr(x_pad), _ptr(dy), ctypes.c_float(beta), _ptr(dwt))


def _fp(a):
    return _ptr(a) if a is not None else None


def batchnorm2d_fwd_train(x, scale, shift, eps, relu, p, y, run_mean=None, run_var=None, save_mean=None, save_invstd=None):
    N, C, H, W = x.shape
    assert y.shape == (N, C, H + 2 * p, W + 2 * p)
    _lib.orc_batchnorm2d_fwd_train(_u32(N), _u32(C), _u32(H), _u32(W), ctypes.c_float(eps), ctypes.c_int(relu), _u32(p),
                                   _ptr(x), _ptr(scale), _ptr(shift), _ptr(y), _fp(run_mean), _fp(run_var), _fp(save_mean),
                                   _fp(save_invstd))


def batchnorm2d_fwd_infer(x, scale, shift, fixed_mean, fixed_var, eps, relu, p, y):
    N, C, H, W = x.shape
    assert y.shape == (N, C, H + 2 * p, W + 2 * p)
    _lib.orc_batchnorm2d_fwd_infer(_u32(N), _u32(C), _u32(H), _u32(W), ctypes.c_float(eps), ctypes.c_int(relu), _u32(p),
                                   _ptr(x), _ptr(scale), _ptr(shift), _ptr(fixed_mean), _ptr(fixed_var), _ptr(y))


def batchnorm2d_bwd(x, dy, scale, shift, save_mean, save_invstd, relu, p, dx, dscale, dshift, beta_data=0.0, beta_param=0.0):
    N, C, H, W = x.shape
    assert dy.shape == (N, C, H + 2 * p, W + 2 * p)
    _lib.orc_batchnorm2d_bwd(_u32(N), _u32(C), _u32(H), _u32(W), ctypes.c_int(relu), _u32(p), _ptr(x), _ptr(dy), _ptr(scale),
                             _fp(shift), _ptr(save_mean), _ptr(save_invstd), ctypes.c_float(beta_data),
                             ctypes.c_float(beta_param), _ptr(dx), _ptr(dscale), _ptr(dshift))


def conv_bias_add(bias, y):
    """y[n,c,h,w] += bias[c] in place; y is (N, C, H, W) float32."""
    N, C, H, W = y.shape
    assert bias.shape == (C,)
    _lib.orc_conv_bias_add(_u32(N), _u32(C), _u32(H), _u32(W), _ptr(bias), _ptr(y))


def conv_bwd_bias(dy, db, beta=0.0):
    """db[c] = beta*db[c] + sum over n,h,w of dy[n,c,h,w]."""
    N, C, H, W = dy.shape
    assert db.shape == (C,)
    _lib.orc_conv_bwd_bias(_u32(N), _u32(C), _u32(H), _u32(W), _ptr(dy), ctypes.c_float(beta), _ptr(db))


def relu_fwd(x, y):
    _lib.orc_relu_fwd(ctypes.c_uint64(x.size), _ptr(x), _ptr(y))


def relu_bwd(y, dy, dx, beta=0.0):
    _lib.orc_relu_bwd(ctypes.c_uint64(y.size), _ptr(y), _ptr(dy), ctypes.c_float(beta), _ptr(dx))


def sum_fwd(xs, y):
    _lib.orc_sum_fwd(_u32(len(xs)), ctypes.c_uint64(y.size), _ptr_array(xs), _ptr(y))


def array_add_scaled(alpha, x, beta, y):
    """y = alpha*x + beta*y in place (flat float32)."""
    _lib.orc_array_add_scaled(ctypes.c_uint64(y.size), ctypes.c_float(alpha), _ptr(x), ctypes.c_float(beta), _ptr(y))


def array_add_online(alpha, x, y):
    """y = y + alpha*(x - y) in place."""
    _lib.orc_array_add_online(ctypes.c_uint64(y.size), ctypes.c_float(alpha), _ptr(x), _ptr(y))


def _len_array(arrs):
    return (ctypes.c_uint64 * len(arrs))(*[a.size for a in arrs])


def flat_store(arrays, flat, offset=0):
    """Arrays, in order, into consecutive ranges of flat from `offset`; returns the new offset.
    flat=None only measures."""
    _lib.orc_flat_store.restype = ctypes.c_uint64
    return _lib.orc_flat_store(_u32(len(arrays)), _ptr_array(arrays), _len_array(arrays), ctypes.c_uint64(offset),
                               _ptr(flat) if flat is not None else None)


def flat_load(arrays, flat, offset=0):
    _lib.orc_flat_load.restype = ctypes.c_uint64
    return _lib.orc_flat_load(_u32(len(arrays)), _ptr_array(arrays), _len_array(arrays), ctypes.c_uint64(offset),
                              _ptr(flat))


def sgd_step(grads, param, momentum_grad, lagged, sum_grad, l2_reg, momentum, step_size, next_step_size, nesterov):
    """The root-rank update of the parallel SGD optimizer, in place on param / momentum_grad;
    lagged may be None; sum_grad receives the reduced (and l2-regularised) gradient."""
    _lib.orc_sgd_step(ctypes.c_uint64(param.size), _u32(len(grads)), _ptr_array(grads), ctypes.c_float(l2_reg),
                      ctypes.c_float(momentum), ctypes.c_float(step_size), ctypes.c_float(next_step_size),
                      ctypes.c_int(int(bool(nesterov))), _ptr(param), _ptr(momentum_grad),
                      _ptr(lagged) if lagged is not None else None, _ptr(sum_grad))


def stat_step(rate, avg_stat, running_stat, stat):
    _lib.orc_stat_step(ctypes.c_uint64(stat.size), ctypes.c_float(rate), _ptr(avg_stat), _ptr(running_stat), _ptr(stat))


def pool_slab_fwd(mode, x_pad, wh, ww, sh, sw, y):
    """x_pad (N, C, HP, WP) float32 -> y (N, C, OH, OW); mode 1 = max, 0 = average."""
    N, C, HP, WP = x_pad.shape
    assert y.shape == (N, C, (HP - wh) // sh + 1, (WP - ww) // sw + 1)
    _lib.orc_pool_slab_fwd(ctypes.c_int(mode), _u32(N), _u32(C), _u32(HP), _u32(WP), _u32(wh), _u32(ww),
                           _u32(sh), _u32(sw), _ptr(x_pad), _ptr(y))


def pool_slab_bwd(mode, x_pad, dy, wh, ww, sh, sw, dx_pad, beta=0.0):
    N, C, HP, WP = x_pad.shape
    _lib.orc_pool_slab_bwd(ctypes.c_int(mode), _u32(N), _u32(C), _u32(HP), _u32(WP), _u32(wh), _u32(ww),
                           _u32(sh), _u32(sw), _ptr(x_pad), _ptr(dy), ctypes.c_float(beta), _ptr(dx_pad))


def softmax_fwd(x, y):
    N, C = x.shape
    _lib.orc_softmax_fwd(_u32(C), _u32(N), _ptr(x), _ptr(y))


def softmax_nll_loss_fwd(y, label, loss):
    N, C = y.shape
    assert label.dtype == np.uint32
    _lib.orc_softmax_nll_loss_fwd(_u32(C), _u32(N), _ptr(y), _ptr(label), _ptr(loss))


def softmax_nll_loss_bwd(y, label, dloss, dx):
    N, C = y.shape
    assert label.dtype == np.uint32
    _lib.orc_softmax_nll_loss_bwd(_u32(C), _u32(N), _ptr(y), _ptr(label), _ptr(dloss), _ptr(dx))


def now():
    return _lib.orc_now_seconds()
