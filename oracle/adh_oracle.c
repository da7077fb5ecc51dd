/*
 * adh_oracle.c -- CPU restatement of the spatially-parallel convolution path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against and the scalar CPU baseline timed next to them.  Nothing in
 * the shipped library links, loads or calls it.
 *
 * Every function follows the algorithm of the reference at the cited
 * file:line (paths relative to the reference tree).  Where the reference's
 * arithmetic lives in a closed-source dependency (cuDNN 7.0.5 for CUDA 9.0,
 * pinned by path in Makefile.config:2) the published definition of the routine
 * is restated and anchored on the reference's call site.
 *
 * Memory layout everywhere: NCHW, fastest dimension first,
 *   idx = w + W*(h + H*(c + C*n))            (src/kernels/spatial.cu:22-36)
 * A halo-padded tile of interior (W,H) and halo width p is a packed buffer of
 * (W+2p, H+2p, C, N); interior element (w,h) lives at padded (w+p, h+p).
 *
 * Pinning status (how each function is checked independently of this file's
 * own formulas is listed in tests/test_oracle_*.py):
 *   - index / strip movers / slices / pad / unpad : pinned by brute-force
 *     nested-loop numpy slicing and the pack == zero-padded-unsplit invariant.
 *   - halo reduce : pinned by the adjoint identity <E a, b> = <a, R b>.
 *   - conv fwd / bwd-data / bwd-filter : pinned against torch.nn.functional
 *     conv2d + autograd on the CPU, delta / box / hot-pixel closed forms.
 *   - softmax / nll : pinned against scipy.special.log_softmax and closed
 *     forms (uniform logits, shift invariance, rows sum to one).
 *   - general conv (any window / stride / dilation) : pinned against torch
 *     conv2d(stride, dilation) + autograd on the CPU and against the 3x3
 *     stride-1 functions above.
 *   - convolution bias (add, backward-bias) : pinned against torch conv2d with a
 *     bias + autograd on the CPU and numpy broadcasting / axis sums.
 *   - batch norm / rectifier / sum : pinned against torch batch_norm (training and
 *     evaluation) + relu + constant_pad + autograd on the CPU, and closed forms
 *     (normalised output has mean 0 / variance 1, dx sums to zero per channel).
 *   - pooling over the padded slab : pinned against torch max_pool2d /
 *     avg_pool2d + autograd on the CPU; which element of a window receives the
 *     max gradient when several are equal is cuDNN's choice and is parity
 *     unpinned (this file and the kernels pick the first in row-major order).
 *   - axpy / online average / flat copies / SGD step / running statistics :
 *     pinned by closed forms (geometric momentum sum under a constant gradient,
 *     (1 - step*l2)^t decay, textbook look-ahead Nesterov on a quadratic,
 *     (1 - a)^t convergence of the online average) and round trips.  Which of
 *     the two products of alpha*x + beta*y the reference's compiler fused, and
 *     the order in which NCCL summed the ranks, are parity unpinned (one ulp).
 *   - cuDNN's exact fp32 summation order for conv and softmax: parity
 *     unpinned (not reproducible by the reference itself run to run); the
 *     tolerance-vs-unsplit criterion is used instead.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_F32 0
#define ORC_BF16 1

#define ORC_OP_COPY 0
#define ORC_OP_ADD 1

#define ORC_EXCH 0
#define ORC_REDUCE 1

#define ORC_OK 0
#define ORC_EINVAL (-1)
#define ORC_EUNIMPL (-2)

/* ------------------------------------------------------------------ */
/* element helpers                                                     */
/* ------------------------------------------------------------------ */

static size_t orc_esize(int dtype) { return dtype == ORC_BF16 ? 2u : 4u; }

float orc_bf16_to_f32(uint16_t v) {
  uint32_t u = ((uint32_t)v) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* round-to-nearest-even, NaN kept quiet */
uint16_t orc_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

/* CopyMap / ReduceMap functors: include/arraydiff/kernels.hh:57-65.
 * (AtomicReduceMap :67-70 has the same result when every destination has a
 * single contributor, which holds for 1xK grids with H >= 2p.) */
static void orc_map(int op, int dtype, void *dst, const void *src) {
  if (op == ORC_OP_COPY) {
    memcpy(dst, src, orc_esize(dtype));
  } else if (dtype == ORC_F32) {
    float a, b;
    memcpy(&a, dst, 4);
    memcpy(&b, src, 4);
    a += b;
    memcpy(dst, &a, 4);
  } else {
    uint16_t a, b;
    memcpy(&a, dst, 2);
    memcpy(&b, src, 2);
    a = orc_f32_to_bf16(orc_bf16_to_f32(a) + orc_bf16_to_f32(b));
    memcpy(dst, &a, 2);
  }
}

/* NCHWLayout::Pack, src/kernels/spatial.cu:22-36 */
int64_t orc_nchw_pack(int64_t w, int64_t pitch_w, int64_t h, int64_t pitch_h,
                      int64_t c, int64_t pitch_c, int64_t n) {
  return w + pitch_w * (h + pitch_h * (c + pitch_c * n));
}

/* index of interior-relative (w,h) in a halo-padded tile,
 * src/kernels/spatial.cu:363-372 with offset_w = offset_h = halo_pad and
 * pitches = padded dims (:444-451). w in [-p, W+p), h in [-p, H+p). */
int64_t orc_padded_index(int64_t w, int64_t h, int64_t c, int64_t n, int64_t p,
                         int64_t W, int64_t H, int64_t C) {
  return orc_nchw_pack(p + w, W + 2 * p, p + h, H + 2 * p, c, C, n);
}

/* ------------------------------------------------------------------ */
/* Z1: fill / add   (src/kernels/array.cu:58-68, 83-94)                */
/* ------------------------------------------------------------------ */

void orc_fill_f32(uint64_t n, float v, float *x) {
  for (uint64_t i = 0; i < n; ++i) x[i] = v;
}

void orc_add_f32(uint64_t n, const float *x, float *y) {
  for (uint64_t i = 0; i < n; ++i) {
    float yi = y[i];
    y[i] = x[i] + yi;
  }
}

/* ------------------------------------------------------------------ */
/* H1/H2: row-halo strips, 1 x K grid                                  */
/* ------------------------------------------------------------------ */

/* One strip of W*C*N elements at a fixed row: spatial2d_map_h_slice,
 * src/kernels/spatial.cu:336-399, HSlice::Unpack<NCHW> :103-115.
 * The loop over the linear index with div/mod per element is the reference's
 * loop structure on purpose (this is also the timed CPU baseline). */
static void orc_map_h_strip(int op, int dtype, uint32_t W, uint32_t H,
                            uint32_t C, uint32_t N, uint32_t p,
                            const void *src, int32_t src_h, void *dst,
                            int32_t dst_h) {
  const size_t es = orc_esize(dtype);
  const uint32_t total = W * C * N;
  const uint32_t pw = W + 2 * p, ph = H + 2 * p;
  for (uint32_t idx = 0; idx < total; ++idx) {
    uint32_t w = idx % W;
    uint32_t c = (idx / W) % C;
    uint32_t n = (idx / W) / C;
    int64_t s = orc_nchw_pack((int64_t)p + w, pw, (int64_t)p + src_h, ph, c, C, n);
    int64_t d = orc_nchw_pack((int64_t)p + w, pw, (int64_t)p + dst_h, ph, c, C, n);
    orc_map(op, dtype, (char *)dst + (size_t)d * es,
            (const char *)src + (size_t)s * es);
  }
}

/* One strip of H*C*N elements at a fixed column: spatial2d_map_w_slice,
 * src/kernels/spatial.cu:271-334. */
static void orc_map_w_strip(int op, int dtype, uint32_t W, uint32_t H,
                            uint32_t C, uint32_t N, uint32_t p,
                            const void *src, int32_t src_w, void *dst,
                            int32_t dst_w) {
  const size_t es = orc_esize(dtype);
  const uint32_t total = H * C * N;
  const uint32_t pw = W + 2 * p, ph = H + 2 * p;
  for (uint32_t idx = 0; idx < total; ++idx) {
    uint32_t h = idx % H;
    uint32_t c = (idx / H) % C;
    uint32_t n = (idx / H) / C;
    int64_t s = orc_nchw_pack((int64_t)p + src_w, pw, (int64_t)p + h, ph, c, C, n);
    int64_t d = orc_nchw_pack((int64_t)p + dst_w, pw, (int64_t)p + h, ph, c, C, n);
    orc_map(op, dtype, (char *)dst + (size_t)d * es,
            (const char *)src + (size_t)s * es);
  }
}

/* ExchOp / ReduceOp offset tables, src/kernels/spatial.cu:175-205.
 * "next" = neighbour rank+1, "prev" = neighbour rank-1, `base` = W or H. */
static void orc_op_table(int which, int32_t base, int32_t *inc_next,
                         int32_t *src_next, int32_t *dst_next,
                         int32_t *inc_prev, int32_t *src_prev,
                         int32_t *dst_prev) {
  if (which == ORC_EXCH) {
    *inc_next = 1;  *src_next = 0;        *dst_next = base;
    *inc_prev = -1; *src_prev = base - 1; *dst_prev = -1;
  } else {
    *inc_next = -1; *src_next = -1;   *dst_next = base - 1;
    *inc_prev = 1;  *src_prev = base; *dst_prev = 0;
  }
}

/* What ONE rank's kernel does on a grid_w x grid_h grid
 * (spatial2d_1x4_halo_op_nchw_kernel, src/kernels/spatial.cu:512-594, for any
 * K; spatial2d_2x1_halo_op_nchw_kernel :654-706 for columns).  Dispatch rules
 * follow Spatial2DComm::group_end, src/spatial.cc:76-200: 1x1 is a no-op,
 * grids with both dimensions > 1 are unimplemented.  The reference has no
 * linked column reduce (src/spatial.cc:166-178); here it is defined as the
 * W-direction mirror of the row reduce, from the same ReduceOp table. */
int orc_halo_op_rank(int which, int dtype, uint32_t grid_w, uint32_t grid_h,
                     uint32_t rank, uint32_t p, uint32_t W, uint32_t H,
                     uint32_t C, uint32_t N, void *const *tiles) {
  if (grid_w == 0 || grid_h == 0 || rank >= grid_w * grid_h) return ORC_EINVAL;
  if (grid_w > 1 && grid_h > 1) return ORC_EUNIMPL;
  for (uint32_t r = 0; r < grid_w * grid_h; ++r)
    if (!tiles[r]) return ORC_EINVAL;
  if (grid_w == 1 && grid_h == 1) return ORC_OK;
  const int op = which == ORC_EXCH ? ORC_OP_COPY : ORC_OP_ADD;
  int32_t in, sn, dn, ip, sp, dp;
  if (grid_w == 1) {
    orc_op_table(which, (int32_t)H, &in, &sn, &dn, &ip, &sp, &dp);
    if (rank < grid_h - 1)
      for (uint32_t d = 0; d < p; ++d)
        orc_map_h_strip(op, dtype, W, H, C, N, p, tiles[rank + 1],
                        sn + in * (int32_t)d, tiles[rank], dn + in * (int32_t)d);
    if (rank > 0)
      for (uint32_t d = 0; d < p; ++d)
        orc_map_h_strip(op, dtype, W, H, C, N, p, tiles[rank - 1],
                        sp + ip * (int32_t)d, tiles[rank], dp + ip * (int32_t)d);
  } else {
    orc_op_table(which, (int32_t)W, &in, &sn, &dn, &ip, &sp, &dp);
    if (rank < grid_w - 1)
      for (uint32_t d = 0; d < p; ++d)
        orc_map_w_strip(op, dtype, W, H, C, N, p, tiles[rank + 1],
                        sn + in * (int32_t)d, tiles[rank], dn + in * (int32_t)d);
    if (rank > 0)
      for (uint32_t d = 0; d < p; ++d)
        orc_map_w_strip(op, dtype, W, H, C, N, p, tiles[rank - 1],
                        sp + ip * (int32_t)d, tiles[rank], dp + ip * (int32_t)d);
  }
  return ORC_OK;
}

/* All ranks, in rank order: the loop HaloExch2DOp runs, src/op.cc:2977-3000
 * (forward) and :3025-3049 (backward). */
int orc_halo_op(int which, int dtype, uint32_t grid_w, uint32_t grid_h,
                uint32_t p, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                void *const *tiles) {
  for (uint32_t r = 0; r < grid_w * grid_h; ++r) {
    int e = orc_halo_op_rank(which, dtype, grid_w, grid_h, r, p, W, H, C, N, tiles);
    if (e) return e;
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* S1/S2: window copy / add between packed NCHW tensors                 */
/* ------------------------------------------------------------------ */

/* slice2d_map_hw_nchw_packed_kernel, src/kernels/slice.cu:12-41; argument
 * checks :61-64.  Extended with a channel range (the reference's kernel is
 * the special case count_c == src_C == dst_C, src_c_off == dst_c_off == 0). */
int orc_slice_nchw(int op, int dtype, uint32_t count_w, uint32_t count_h,
                   uint32_t count_c, uint32_t N, const void *src,
                   uint32_t src_W, uint32_t src_H, uint32_t src_C,
                   uint32_t src_w_off, uint32_t src_h_off, uint32_t src_c_off,
                   void *dst, uint32_t dst_W, uint32_t dst_H, uint32_t dst_C,
                   uint32_t dst_w_off, uint32_t dst_h_off, uint32_t dst_c_off) {
  if (src_w_off + count_w > src_W || src_h_off + count_h > src_H ||
      src_c_off + count_c > src_C || dst_w_off + count_w > dst_W ||
      dst_h_off + count_h > dst_H || dst_c_off + count_c > dst_C)
    return ORC_EINVAL;
  const size_t es = orc_esize(dtype);
  const uint64_t count = (uint64_t)count_w * count_h * count_c * N;
  for (uint64_t idx = 0; idx < count; ++idx) {
    uint64_t w = idx % count_w;
    uint64_t h = (idx / count_w) % count_h;
    uint64_t c = ((idx / count_w) / count_h) % count_c;
    uint64_t n = ((idx / count_w) / count_h) / count_c;
    uint64_t s = (src_w_off + w) +
                 (uint64_t)src_W * ((src_h_off + h) +
                                    (uint64_t)src_H * ((src_c_off + c) + (uint64_t)src_C * n));
    uint64_t d = (dst_w_off + w) +
                 (uint64_t)dst_W * ((dst_h_off + h) +
                                    (uint64_t)dst_H * ((dst_c_off + c) + (uint64_t)dst_C * n));
    orc_map(op, dtype, (char *)dst + d * es, (const char *)src + s * es);
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* P1/P2/P3: pad / unpad / repad                                        */
/* ------------------------------------------------------------------ */

/* HaloPad2DOp::_forward, src/op.cc:2574-2641: zero the whole padded buffer
 * (base_as_view().set_constant(0)), then cudnnAddTensor(alpha=1, beta=0)
 * packed x -> interior of y. */
void orc_halo_pad(int dtype, uint32_t p, uint32_t W, uint32_t H, uint32_t C,
                  uint32_t N, const void *x_packed, void *y_padded) {
  const size_t es = orc_esize(dtype);
  memset(y_padded, 0, (size_t)(W + 2 * p) * (H + 2 * p) * C * N * es);
  orc_slice_nchw(ORC_OP_COPY, dtype, W, H, C, N, x_packed, W, H, C, 0, 0, 0,
                 y_padded, W + 2 * p, H + 2 * p, C, p, p, 0);
}

/* HaloUnpad2DOp::_backward, src/op.cc:2798-2870: interior(dx_padded) += dy
 * (cudnnAddTensor alpha=1, beta=1 after the first-touch zeroing). */
void orc_halo_pad_add(int dtype, uint32_t p, uint32_t W, uint32_t H, uint32_t C,
                      uint32_t N, const void *x_packed, void *y_padded) {
  orc_slice_nchw(ORC_OP_ADD, dtype, W, H, C, N, x_packed, W, H, C, 0, 0, 0,
                 y_padded, W + 2 * p, H + 2 * p, C, p, p, 0);
}

/* HaloUnpad2DOp::_forward, src/op.cc:2715-2793: y_packed = interior(x). */
void orc_halo_unpad(int dtype, uint32_t p, uint32_t W, uint32_t H, uint32_t C,
                    uint32_t N, const void *x_padded, void *y_packed) {
  orc_slice_nchw(ORC_OP_COPY, dtype, W, H, C, N, x_padded, W + 2 * p, H + 2 * p,
                 C, p, p, 0, y_packed, W, H, C, 0, 0, 0);
}

/* HaloPad2DOp::_backward, src/op.cc:2644-2712: dx_packed += interior(dy). */
void orc_halo_unpad_add(int dtype, uint32_t p, uint32_t W, uint32_t H,
                        uint32_t C, uint32_t N, const void *x_padded,
                        void *y_packed) {
  orc_slice_nchw(ORC_OP_ADD, dtype, W, H, C, N, x_padded, W + 2 * p, H + 2 * p,
                 C, p, p, 0, y_packed, W, H, C, 0, 0, 0);
}

/* HaloRepad2DOp::_forward, src/op.cc:2873-2960: interior of a p_src buffer ->
 * interior of a zeroed p_dst buffer. */
void orc_halo_repad(int dtype, uint32_t p_src, uint32_t p_dst, uint32_t W,
                    uint32_t H, uint32_t C, uint32_t N, const void *x_padded,
                    void *y_padded) {
  const size_t es = orc_esize(dtype);
  memset(y_padded, 0, (size_t)(W + 2 * p_dst) * (H + 2 * p_dst) * C * N * es);
  orc_slice_nchw(ORC_OP_COPY, dtype, W, H, C, N, x_padded, W + 2 * p_src,
                 H + 2 * p_src, C, p_src, p_src, 0, y_padded, W + 2 * p_dst,
                 H + 2 * p_dst, C, p_dst, p_dst, 0);
}

/* ------------------------------------------------------------------ */
/* pack / unpack = the op sequence the model zoo builds                 */
/* ------------------------------------------------------------------ */

/* pack: SpatialScatter2DOp::_forward (src/op.cc:2395-2429, rows
 * [r*H/K, (r+1)*H/K) of the unsplit tensor -> tile r), HaloPad2DOp::_forward,
 * then HaloExch2DOp::_forward; the order src/zoo.cc:1522-1526 wires them in.
 * H is the unsplit height; requires H % K == 0 (src/op.cc:2385-2387).
 * `scratch` must hold one unpadded tile. */
int orc_tiles_pack(int dtype, uint32_t K, uint32_t p, uint32_t W, uint32_t H,
                   uint32_t C, uint32_t N, const void *x_unsplit,
                   void *const *tiles, void *scratch) {
  if (K == 0 || H % K != 0) return ORC_EINVAL;
  const uint32_t Ht = H / K;
  for (uint32_t r = 0; r < K; ++r) {
    int e = orc_slice_nchw(ORC_OP_COPY, dtype, W, Ht, C, N, x_unsplit, W, H, C,
                           0, r * Ht, 0, scratch, W, Ht, C, 0, 0, 0);
    if (e) return e;
    orc_halo_pad(dtype, p, W, Ht, C, N, scratch, tiles[r]);
  }
  return orc_halo_op(ORC_EXCH, dtype, 1, K, p, W, Ht, C, N, tiles);
}

/* unpack: HaloUnpad2DOp::_forward then SpatialGather2DOp::_forward
 * (src/op.cc:2479-2514: tile r -> rows [r*H/K, ...) of a full tensor; the
 * zero-fill + allreduce of src/zoo.cc:1841-1842 collapses to a plain gather
 * when all tiles are in one memory). */
int orc_tiles_unpack(int dtype, uint32_t K, uint32_t p, uint32_t W, uint32_t H,
                     uint32_t C, uint32_t N, void *const *tiles,
                     void *y_unsplit, void *scratch) {
  if (K == 0 || H % K != 0) return ORC_EINVAL;
  const uint32_t Ht = H / K;
  for (uint32_t r = 0; r < K; ++r) {
    orc_halo_unpad(dtype, p, W, Ht, C, N, tiles[r], scratch);
    int e = orc_slice_nchw(ORC_OP_COPY, dtype, W, Ht, C, N, scratch, W, Ht, C,
                           0, 0, 0, y_unsplit, W, H, C, 0, r * Ht, 0);
    if (e) return e;
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------ */
/* C2/C3/C4: 3x3 (k x k) convolution over the halo-padded slab          */
/* ------------------------------------------------------------------ */

/* cudnnConvolutionForward at src/op.cc:1576-1587 with the descriptors of
 * src/op.cc:1354-1410: CUDNN_CROSS_CORRELATION, x = padded slab
 * (N,Cin,H+2p,W+2p) with conv pad 0, stride 1, filter KCRS = (Cout,Cin,k,k),
 * y packed (N,Cout,H,W), k = 2p+1:
 *   y[n,co,h,w] = beta*y + sum_{ci,kh,kw} wt[co,ci,kh,kw] * x[n,ci,h+kh,w+kw]
 * Accumulated in double, rounded once to float. */
void orc_conv_slab_fwd(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                       uint32_t W, uint32_t k, const float *x_pad,
                       const float *wt, float beta, float *y) {
  const uint32_t Hp = H + k - 1, Wp = W + k - 1;
  for (uint32_t n = 0; n < N; ++n)
    for (uint32_t co = 0; co < Cout; ++co)
      for (uint32_t h = 0; h < H; ++h)
        for (uint32_t w = 0; w < W; ++w) {
          double acc = 0.0;
          for (uint32_t ci = 0; ci < Cin; ++ci)
            for (uint32_t kh = 0; kh < k; ++kh)
              for (uint32_t kw = 0; kw < k; ++kw)
                acc += (double)wt[((co * (size_t)Cin + ci) * k + kh) * k + kw] *
                       (double)x_pad[((n * (size_t)Cin + ci) * Hp + h + kh) * Wp + w + kw];
          size_t yi = ((n * (size_t)Cout + co) * H + h) * W + w;
          y[yi] = (float)(acc + (beta != 0.0f ? (double)beta * y[yi] : 0.0));
        }
}

/* cudnnConvolutionBackwardData at src/op.cc:1701-1712 (alpha=1, beta as
 * given; the op passes beta=1 onto a slab it zeroed first, :1687-1691):
 *   dx[n,ci,h',w'] = beta*dx + sum_{co,kh,kw} wt[co,ci,kh,kw]*dy[n,co,h'-kh,w'-kw]
 * over the WHOLE padded slab h' in [0,H+k-1), w' in [0,W+k-1); dy outside
 * [0,H)x[0,W) is zero. */
void orc_conv_slab_bwd_data(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                            uint32_t W, uint32_t k, const float *wt,
                            const float *dy, float beta, float *dx_pad) {
  const uint32_t Hp = H + k - 1, Wp = W + k - 1;
  for (uint32_t n = 0; n < N; ++n)
    for (uint32_t ci = 0; ci < Cin; ++ci)
      for (uint32_t hp = 0; hp < Hp; ++hp)
        for (uint32_t wp = 0; wp < Wp; ++wp) {
          double acc = 0.0;
          for (uint32_t co = 0; co < Cout; ++co)
            for (uint32_t kh = 0; kh < k; ++kh)
              for (uint32_t kw = 0; kw < k; ++kw) {
                int64_t h = (int64_t)hp - kh, w = (int64_t)wp - kw;
                if (h < 0 || h >= (int64_t)H || w < 0 || w >= (int64_t)W) continue;
                acc += (double)wt[((co * (size_t)Cin + ci) * k + kh) * k + kw] *
                       (double)dy[((n * (size_t)Cout + co) * H + h) * W + w];
              }
          size_t xi = ((n * (size_t)Cin + ci) * Hp + hp) * Wp + wp;
          dx_pad[xi] = (float)(acc + (beta != 0.0f ? (double)beta * dx_pad[xi] : 0.0));
        }
}

/* cudnnConvolutionBackwardFilter at src/op.cc:1660-1671 (alpha=1, beta as
 * given; beta=1 onto a first-touch-zeroed dw, :1651-1654):
 *   dw[co,ci,kh,kw] = beta*dw + sum_{n,h,w} dy[n,co,h,w] * x[n,ci,h+kh,w+kw] */
void orc_conv_slab_bwd_filter(uint32_t N, uint32_t Cin, uint32_t Cout,
                              uint32_t H, uint32_t W, uint32_t k,
                              const float *x_pad, const float *dy, float beta,
                              float *dw) {
  const uint32_t Hp = H + k - 1, Wp = W + k - 1;
  for (uint32_t co = 0; co < Cout; ++co)
    for (uint32_t ci = 0; ci < Cin; ++ci)
      for (uint32_t kh = 0; kh < k; ++kh)
        for (uint32_t kw = 0; kw < k; ++kw) {
          double acc = 0.0;
          for (uint32_t n = 0; n < N; ++n)
            for (uint32_t h = 0; h < H; ++h) {
              const float *dyr = dy + ((n * (size_t)Cout + co) * H + h) * W;
              const float *xr = x_pad + ((n * (size_t)Cin + ci) * Hp + h + kh) * Wp + kw;
              for (uint32_t w = 0; w < W; ++w) acc += (double)dyr[w] * (double)xr[w];
            }
          size_t wi = ((co * (size_t)Cin + ci) * k + kh) * k + kw;
          dw[wi] = (float)(acc + (beta != 0.0f ? (double)beta * dw[wi] : 0.0));
        }
}

/* Scalar fp32 direct convolution with the loop nest of a per-output-element
 * GPU thread (float accumulate, no blocking): the timed CPU baseline for the
 * slab conv.  Same definition as orc_conv_slab_fwd. */
void orc_conv_slab_fwd_f32(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                           uint32_t W, uint32_t k, const float *x_pad,
                           const float *wt, float *y) {
  const uint32_t Hp = H + k - 1, Wp = W + k - 1;
  for (uint32_t n = 0; n < N; ++n)
    for (uint32_t co = 0; co < Cout; ++co)
      for (uint32_t h = 0; h < H; ++h)
        for (uint32_t w = 0; w < W; ++w) {
          float acc = 0.0f;
          for (uint32_t ci = 0; ci < Cin; ++ci)
            for (uint32_t kh = 0; kh < k; ++kh)
              for (uint32_t kw = 0; kw < k; ++kw)
                acc += wt[((co * (size_t)Cin + ci) * k + kh) * k + kw] *
                       x_pad[((n * (size_t)Cin + ci) * Hp + h + kh) * Wp + w + kw];
          y[((n * (size_t)Cout + co) * H + h) * W + w] = acc;
        }
}

/* ------------------------------------------------------------------ */
/* general window / stride / dilation over the halo-padded slab          */
/* ------------------------------------------------------------------ */

/* CudnnConv2DSize with halo_padded_input (src/op.cc:1354-1410): x = packed
 * (N,Cin,HP,WP) with conv pad 0, stride (sh,sw), dilation (dh,dw), filter KCRS
 * (Cout,Cin,kh,kw); output extents as cudnnGetConvolution2dForwardOutputDim,
 * OH = (HP - ((kh-1)*dh + 1)) / sh + 1 (src/op.cc:1512-1523):
 *   y[n,co,oh,ow] = beta*y + sum wt[co,ci,a,b] * x[n,ci,oh*sh + a*dh, ow*sw + b*dw] */
void orc_conv2d_slab_fwd(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t kh, uint32_t kw,
                         uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, const float *x_pad, const float *wt,
                         float beta, float *y) {
  const uint32_t OH = (HP - ((kh - 1) * dh + 1)) / sh + 1, OW = (WP - ((kw - 1) * dw + 1)) / sw + 1;
  for (uint32_t n = 0; n < N; ++n)
    for (uint32_t co = 0; co < Cout; ++co)
      for (uint32_t oh = 0; oh < OH; ++oh)
        for (uint32_t ow = 0; ow < OW; ++ow) {
          double acc = 0.0;
          for (uint32_t ci = 0; ci < Cin; ++ci)
            for (uint32_t a = 0; a < kh; ++a)
              for (uint32_t b = 0; b < kw; ++b)
                acc += (double)wt[((co * (size_t)Cin + ci) * kh + a) * kw + b] *
                       (double)x_pad[((n * (size_t)Cin + ci) * HP + oh * sh + a * dh) * WP + ow * sw + b * dw];
          size_t yi = ((n * (size_t)Cout + co) * OH + oh) * OW + ow;
          y[yi] = (float)(acc + (beta != 0.0f ? (double)beta * y[yi] : 0.0));
        }
}

/* cudnnConvolutionBackwardData (src/op.cc:1701-1712) for the same descriptors, as the adjoint of
 * the forward map written as a scatter: every (output pixel, tap) adds wt*dy onto the padded pixel
 * it read.  Padded pixels that no window reads get beta*dx. */
void orc_conv2d_slab_bwd_data(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t kh,
                              uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, const float *wt,
                              const float *dy, float beta, float *dx_pad) {
  const uint32_t OH = (HP - ((kh - 1) * dh + 1)) / sh + 1, OW = (WP - ((kw - 1) * dw + 1)) / sw + 1;
  const size_t plane = (size_t)HP * WP;
  double *g = (double *)malloc(plane * sizeof(double));
  for (uint32_t n = 0; n < N; ++n)
    for (uint32_t ci = 0; ci < Cin; ++ci) {
      for (size_t i = 0; i < plane; ++i) g[i] = 0.0;
      for (uint32_t co = 0; co < Cout; ++co)
        for (uint32_t oh = 0; oh < OH; ++oh)
          for (uint32_t ow = 0; ow < OW; ++ow) {
            const double d = dy[((n * (size_t)Cout + co) * OH + oh) * OW + ow];
            for (uint32_t a = 0; a < kh; ++a)
              for (uint32_t b = 0; b < kw; ++b)
                g[(size_t)(oh * sh + a * dh) * WP + ow * sw + b * dw] +=
                    (double)wt[((co * (size_t)Cin + ci) * kh + a) * kw + b] * d;
          }
      float *dxp = dx_pad + (n * (size_t)Cin + ci) * plane;
      for (size_t i = 0; i < plane; ++i) dxp[i] = (float)(g[i] + (beta != 0.0f ? (double)beta * dxp[i] : 0.0));
    }
  free(g);
}

/* cudnnConvolutionBackwardFilter (src/op.cc:1660-1671) for the same descriptors:
 *   dw[co,ci,a,b] = beta*dw + sum_{n,oh,ow} dy[n,co,oh,ow] * x[n,ci,oh*sh + a*dh, ow*sw + b*dw] */
void orc_conv2d_slab_bwd_filter(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t kh,
                                uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, const float *x_pad,
                                const float *dy, float beta, float *dwt) {
  const uint32_t OH = (HP - ((kh - 1) * dh + 1)) / sh + 1, OW = (WP - ((kw - 1) * dw + 1)) / sw + 1;
  for (uint32_t co = 0; co < Cout; ++co)
    for (uint32_t ci = 0; ci < Cin; ++ci)
      for (uint32_t a = 0; a < kh; ++a)
        for (uint32_t b = 0; b < kw; ++b) {
          double acc = 0.0;
          for (uint32_t n = 0; n < N; ++n)
            for (uint32_t oh = 0; oh < OH; ++oh)
              for (uint32_t ow = 0; ow < OW; ++ow)
                acc += (double)dy[((n * (size_t)Cout + co) * OH + oh) * OW + ow] *
                       (double)x_pad[((n * (size_t)Cin + ci) * HP + oh * sh + a * dh) * WP + ow * sw + b * dw];
          size_t wi = ((co * (size_t)Cin + ci) * kh + a) * kw + b;
          dwt[wi] = (float)(acc + (beta != 0.0f ? (double)beta * dwt[wi] : 0.0));
        }
}

/* ------------------------------------------------------------------ */
/* convolution bias                                                     */
/* ------------------------------------------------------------------ */

/* cudnnAddTensor(alpha = 1, bias_desc (1,C,1,1), beta = 1, y_desc) after the convolution
 * (src/op.cc:1602-1610): y[n,c,h,w] += bias[c].  One rounding per element. */
void orc_conv_bias_add(uint32_t N, uint32_t C, uint32_t H, uint32_t W, const float *bias, float *y) {
  const size_t HW = (size_t)H * W;
  for (uint32_t n = 0; n < N; ++n)
    for (uint32_t c = 0; c < C; ++c) {
      float *plane = y + ((size_t)n * C + c) * HW;
      for (size_t i = 0; i < HW; ++i) plane[i] = plane[i] + bias[c];
    }
}

/* cudnnConvolutionBackwardBias(alpha = 1, dy, beta, db) (src/op.cc:1632-1648; the reference
 * zeroes db on first touch and passes beta = 1): db[c] = beta*db[c] + sum_{n,h,w} dy[n,c,h,w].
 * Summed in double; cuDNN's order of additions is parity unpinned. */
void orc_conv_bwd_bias(uint32_t N, uint32_t C, uint32_t H, uint32_t W, const float *dy, float beta, float *db) {
  const size_t HW = (size_t)H * W;
  for (uint32_t c = 0; c < C; ++c) {
    double acc = 0.0;
    for (uint32_t n = 0; n < N; ++n) {
      const float *plane = dy + ((size_t)n * C + c) * HW;
      for (size_t i = 0; i < HW; ++i) acc += plane[i];
    }
    db[c] = (float)(acc + (beta != 0.0f ? (double)beta * db[c] : 0.0));
  }
}

/* ------------------------------------------------------------------ */
/* shard-local ops between halos: batch norm, rectifier, residual sum     */
/* ------------------------------------------------------------------ */

/* cudnnBatchNormalizationForwardTraining(CUDNN_BATCHNORM_SPATIAL, factor = 1, eps) at
 * src/op.cc:3996-4011 over one tile (N,C,H,W): per channel over m = N*H*W elements
 *   mean = sum x / m, var = sum (x-mean)^2 / m, y = scale*(x-mean)/sqrt(var+eps) + shift,
 *   running mean = mean, running variance = var*m/(m-1) (factor 1 replaces the old values),
 *   saved mean = mean, saved inverse std = 1/sqrt(var+eps).
 * relu != 0 applies CudnnActivationOp's max(y,0) (src/op.cc:3189-3250) on the way out;
 * p > 0 writes y into the interior of a tile padded by p and zeroes the border
 * (HaloPad2DOp::_forward, src/op.cc:2573-2640).  Two passes in double. */
void orc_batchnorm2d_fwd_train(uint32_t N, uint32_t C, uint32_t H, uint32_t W, float eps, int relu, uint32_t p,
                               const float *x, const float *scale, const float *shift, float *y, float *run_mean,
                               float *run_var, float *save_mean, float *save_invstd) {
  const size_t HW = (size_t)H * W, WP = W + 2 * (size_t)p, HP = H + 2 * (size_t)p;
  const double m = (double)N * (double)HW;
  for (size_t i = 0; i < (size_t)N * C * HP * WP; ++i) y[i] = 0.0f;
  for (uint32_t c = 0; c < C; ++c) {
    double s = 0.0;
    for (uint32_t n = 0; n < N; ++n)
      for (size_t i = 0; i < HW; ++i) s += x[((size_t)n * C + c) * HW + i];
    const double mean = s / m;
    double v = 0.0;
    for (uint32_t n = 0; n < N; ++n)
      for (size_t i = 0; i < HW; ++i) {
        const double d = x[((size_t)n * C + c) * HW + i] - mean;
        v += d * d;
      }
    const double var = v / m, invstd = 1.0 / sqrt(var + (double)eps);
    if (run_mean) run_mean[c] = (float)mean;
    if (run_var) run_var[c] = (float)(m > 1.0 ? var * m / (m - 1.0) : var);
    if (save_mean) save_mean[c] = (float)mean;
    if (save_invstd) save_invstd[c] = (float)invstd;
    for (uint32_t n = 0; n < N; ++n)
      for (uint32_t h = 0; h < H; ++h)
        for (uint32_t w = 0; w < W; ++w) {
          double o = (double)scale[c] * (x[((size_t)n * C + c) * HW + (size_t)h * W + w] - mean) * invstd + (double)shift[c];
          if (relu && o < 0.0) o = 0.0;
          y[((size_t)n * C + c) * HP * WP + (size_t)(h + p) * WP + w + p] = (float)o;
        }
  }
}

/* cudnnBatchNormalizationForwardInference at src/op.cc:3978-3990:
 *   y = scale*(x - fixed_mean)/sqrt(fixed_var + eps) + shift */
void orc_batchnorm2d_fwd_infer(uint32_t N, uint32_t C, uint32_t H, uint32_t W, float eps, int relu, uint32_t p,
                               const float *x, const float *scale, const float *shift, const float *fixed_mean,
                               const float *fixed_var, float *y) {
  const size_t HW = (size_t)H * W, WP = W + 2 * (size_t)p, HP = H + 2 * (size_t)p;
  for (size_t i = 0; i < (size_t)N * C * HP * WP; ++i) y[i] = 0.0f;
  for (uint32_t n = 0; n < N; ++n)
    for (uint32_t c = 0; c < C; ++c) {
      const double invstd = 1.0 / sqrt((double)fixed_var[c] + (double)eps);
      for (uint32_t h = 0; h < H; ++h)
        for (uint32_t w = 0; w < W; ++w) {
          double o = (double)scale[c] * (x[((size_t)n * C + c) * HW + (size_t)h * W + w] - (double)fixed_mean[c]) * invstd +
                     (double)shift[c];
          if (relu && o < 0.0) o = 0.0;
          y[((size_t)n * C + c) * HP * WP + (size_t)(h + p) * WP + w + p] = (float)o;
        }
    }
}

/* cudnnBatchNormalizationBackward(alpha = 1, beta as given for data and parameters) at
 * src/op.cc:4082-4097 with the saved mean / inverse std of the forward pass:
 *   dshift = sum dy', dscale = sum dy'*xhat, dx = scale*invstd*(dy' - dshift/m - xhat*dscale/m),
 * xhat = (x-mean)*invstd.  relu != 0: dy' = dy where the forward output was positive
 * (cudnnActivationBackward, src/op.cc:3252-3324); p > 0: dy is the interior of a gradient tile
 * padded by p (HaloPad2DOp::_backward, src/op.cc:2642-2712). */
void orc_batchnorm2d_bwd(uint32_t N, uint32_t C, uint32_t H, uint32_t W, int relu, uint32_t p, const float *x,
                         const float *dy, const float *scale, const float *shift, const float *save_mean,
                         const float *save_invstd, float beta_data, float beta_param, float *dx, float *dscale,
                         float *dshift) {
  const size_t HW = (size_t)H * W, WP = W + 2 * (size_t)p, HP = H + 2 * (size_t)p;
  const double m = (double)N * (double)HW;
  for (uint32_t c = 0; c < C; ++c) {
    const double mean = save_mean[c], invstd = save_invstd[c], sc = scale[c], sh = shift ? shift[c] : 0.0;
    double sd = 0.0, sdx = 0.0;
    for (int pass = 0; pass < 2; ++pass)
      for (uint32_t n = 0; n < N; ++n)
        for (uint32_t h = 0; h < H; ++h)
          for (uint32_t w = 0; w < W; ++w) {
            const size_t xi = ((size_t)n * C + c) * HW + (size_t)h * W + w;
            const double xhat = (x[xi] - mean) * invstd;
            double d = dy[((size_t)n * C + c) * HP * WP + (size_t)(h + p) * WP + w + p];
            if (relu && !(sc * xhat + sh > 0.0)) d = 0.0;
            if (pass == 0) {
              sd += d;
              sdx += d * xhat;
            } else {
              const double g = sc * invstd * (d - sd / m - xhat * sdx / m);
              dx[xi] = (float)(g + (beta_data != 0.0f ? (double)beta_data * dx[xi] : 0.0));
            }
          }
    dscale[c] = (float)(sdx + (beta_param != 0.0f ? (double)beta_param * dscale[c] : 0.0));
    dshift[c] = (float)(sd + (beta_param != 0.0f ? (double)beta_param * dshift[c] : 0.0));
  }
}

/* cudnnActivationForward / Backward with CUDNN_ACTIVATION_RELU (src/op.cc:3189-3324) */
void orc_relu_fwd(uint64_t n, const float *x, float *y) {
  for (uint64_t i = 0; i < n; ++i) y[i] = x[i] > 0.0f ? x[i] : 0.0f;
}
void orc_relu_bwd(uint64_t n, const float *y, const float *dy, float beta, float *dx) {
  for (uint64_t i = 0; i < n; ++i) dx[i] = (y[i] > 0.0f ? dy[i] : 0.0f) + (beta != 0.0f ? beta * dx[i] : 0.0f);
}
/* SumJoinOp::_forward (src/op.cc:744-806): y = x_0 + x_1 + ... in that order */
void orc_sum_fwd(uint32_t count, uint64_t n, const float *const *xs, float *y) {
  for (uint64_t i = 0; i < n; ++i) {
    float v = xs[0][i];
    for (uint32_t k = 1; k < count; ++k) v += xs[k][i];
    y[i] = v;
  }
}

/* ------------------------------------------------------------------ */
/* flat parameter vectors and the SGD update                            */
/* ------------------------------------------------------------------ */

/* arraydiff_array_add_scaled_packed_kernel (src/kernels/array.cu:97-110): y = alpha*x + beta*y.
 * The compiler of the reference contracts the expression into one fused multiply-add; the form
 * fma(alpha, x, beta*y), which contracts the first product, is fixed here.  With beta == 1 (every
 * parameter update) both possible contractions give these bits; with alpha == 1 (the momentum
 * update) the other contraction may differ in the last place. */
void orc_array_add_scaled(uint64_t n, float alpha, const float *x, float beta, float *y) {
  for (uint64_t i = 0; i < n; ++i) {
    const float yi = y[i];
    const float by = beta * yi;
    y[i] = fmaf(alpha, x[i], by);
  }
}
/* arraydiff_array_add_online_packed_kernel (src/kernels/array.cu:112-124): y = y + alpha*(x - y) */
void orc_array_add_online(uint64_t n, float alpha, const float *x, float *y) {
  for (uint64_t i = 0; i < n; ++i) {
    const float yi = y[i];
    const float d = x[i] - yi;
    y[i] = fmaf(alpha, d, yi);
  }
}
/* Op::store_val / store_grad walking the graph (src/op.cc:170-194): every array of the set is
 * copied to the writer at the running offset, which advances by the array's size. */
uint64_t orc_flat_store(uint32_t count, const float *const *arrays, const uint64_t *lens, uint64_t offset, float *flat) {
  for (uint32_t k = 0; k < count; ++k) {
    if (flat) memcpy(flat + offset, arrays[k], lens[k] * sizeof(float));
    offset += lens[k];
  }
  return offset;
}
/* Op::load_val (src/op.cc:148-158): the inverse copy */
uint64_t orc_flat_load(uint32_t count, float *const *arrays, const uint64_t *lens, uint64_t offset, const float *flat) {
  for (uint32_t k = 0; k < count; ++k) {
    memcpy(arrays[k], flat + offset, lens[k] * sizeof(float));
    offset += lens[k];
  }
  return offset;
}
/* The root-rank part of ParallelSGDOptimizer::step (include/arraydiff/optimize.hh:443-505):
 *   ncclReduce(sum) of the ranks' sum_grad vectors onto rank 0   (:443-451; summed here in rank order)
 *   sum_grad += l2_reg * param                  if l2_reg != 0   (:481-483)
 *   momentum_grad = 1*sum_grad + mu*momentum_grad                (:487)
 *   nesterov:  param += -alpha*sum_grad; lagged = param; param += -next_alpha*mu*momentum_grad  (:488-492)
 *   else:      param += -alpha*momentum_grad; lagged = param                                    (:493-496)
 * sum_grad (n floats) is rank 0's vector on entry when grads == NULL, else scratch that receives
 * the reduced gradient. */
void orc_sgd_step(uint64_t n, uint32_t num_grads, const float *const *grads, float l2_reg, float mu, float alpha,
                  float next_alpha, int nesterov, float *param, float *momentum_grad, float *lagged,
                  float *sum_grad) {
  if (grads) {
    for (uint64_t i = 0; i < n; ++i) {
      float g = grads[0][i];
      for (uint32_t r = 1; r < num_grads; ++r) g += grads[r][i];
      sum_grad[i] = g;
    }
  }
  if (l2_reg != 0.0f) orc_array_add_scaled(n, l2_reg, param, 1.0f, sum_grad);
  orc_array_add_scaled(n, 1.0f, sum_grad, mu, momentum_grad);
  if (nesterov) {
    orc_array_add_scaled(n, -alpha, sum_grad, 1.0f, param);
    if (lagged) memcpy(lagged, param, n * sizeof(float));
    orc_array_add_scaled(n, -next_alpha * mu, momentum_grad, 1.0f, param);
  } else {
    orc_array_add_scaled(n, -alpha, momentum_grad, 1.0f, param);
    if (lagged) memcpy(lagged, param, n * sizeof(float));
  }
}
/* running statistics (include/arraydiff/optimize.hh:507-514): running += rate*(avg - running); stat = running */
void orc_stat_step(uint64_t n, float rate, const float *avg_stat, float *running_stat, float *stat) {
  orc_array_add_online(n, rate, avg_stat, running_stat);
  memcpy(stat, running_stat, n * sizeof(float));
}

/* ------------------------------------------------------------------ */
/* L1/L2/L3: softmax + negative log likelihood                          */
/* ------------------------------------------------------------------ */

/* cudnnSoftmaxForward(CUDNN_SOFTMAX_ACCURATE, CUDNN_SOFTMAX_MODE_INSTANCE) on
 * (N, C, 1, 1) at src/op.cc:4129-4152: max-subtracted softmax over the C
 * classes of each row.  Computed in double, rounded once. */
void orc_softmax_fwd(uint32_t C, uint32_t N, const float *x, float *y) {
  for (uint32_t i = 0; i < N; ++i) {
    const float *xr = x + (size_t)i * C;
    float *yr = y + (size_t)i * C;
    double m = -INFINITY;
    for (uint32_t j = 0; j < C; ++j)
      if ((double)xr[j] > m) m = xr[j];
    double s = 0.0;
    for (uint32_t j = 0; j < C; ++j) s += exp((double)xr[j] - m);
    for (uint32_t j = 0; j < C; ++j) yr[j] = (float)(exp((double)xr[j] - m) / s);
  }
}

/* softmax_nll_loss_fwd_kernel, src/kernels/softmax.cu:36-54 */
void orc_softmax_nll_loss_fwd(uint32_t C, uint32_t N, const float *y,
                              const uint32_t *label, float *loss) {
  for (uint32_t i = 0; i < N; ++i) {
    float prob = y[label[i] + (size_t)C * i];
    loss[i] = -logf(prob);
  }
}

/* softmax_nll_loss_bwd_kernel, src/kernels/softmax.cu:56-78 (dx is
 * accumulated into; the label round-trips through float as in the kernel). */
void orc_softmax_nll_loss_bwd(uint32_t C, uint32_t N, const float *y,
                              const uint32_t *label, const float *dloss,
                              float *dx) {
  for (uint64_t idx = 0; idx < (uint64_t)C * N; ++idx) {
    uint32_t channel = (uint32_t)(idx % C);
    uint32_t i = (uint32_t)(idx / C);
    float y_i = y[idx];
    float label_i = (float)label[i];
    float dl = dloss[i];
    if ((uint32_t)label_i == channel)
      dx[idx] += dl * (y_i - 1.0f);
    else
      dx[idx] += dl * y_i;
  }
}

/* ------------------------------------------------------------------ */
/* timing helper for the CPU baseline (bench only)                      */
/* ------------------------------------------------------------------ */
#include <time.h>
double orc_now_seconds(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}


/* ------------------------------------------------------------------------- */
/* pooling over the halo-padded slab                                          */
/* ------------------------------------------------------------------------- */
/* CudnnPool2DOp::_forward with halo_padded_input (src/op.cc:3424-3462, 3496-3503): the padded
 * tile (WP, HP, C, N) is pooled as a plain packed tensor with pad 0; mode 1 = CUDNN_POOLING_MAX
 * (NaNs never win, CUDNN_NOT_PROPAGATE_NAN), mode 0 = AVERAGE_COUNT_INCLUDE_PADDING (divisor
 * wh*ww).  Output (OW, OH) = ((WP - ww)/sw + 1, (HP - wh)/sh + 1). */
void orc_pool_slab_fwd(int mode, uint32_t N, uint32_t C, uint32_t HP, uint32_t WP, uint32_t wh, uint32_t ww,
                       uint32_t sh, uint32_t sw, const float *x, float *y) {
  const uint32_t OH = (HP - wh) / sh + 1u, OW = (WP - ww) / sw + 1u;
  for (uint64_t pl = 0; pl < (uint64_t)N * C; ++pl) {
    const float *xp = x + pl * HP * WP;
    float *yp = y + pl * OH * OW;
    for (uint32_t oh = 0; oh < OH; ++oh)
      for (uint32_t ow = 0; ow < OW; ++ow) {
        double sum = 0.0;
        float mx = -INFINITY;
        for (uint32_t a = 0; a < wh; ++a)
          for (uint32_t b = 0; b < ww; ++b) {
            const float v = xp[(uint64_t)(oh * sh + a) * WP + ow * sw + b];
            sum += v;
            if (v > mx) mx = v;
          }
        yp[(uint64_t)oh * OW + ow] = mode ? mx : (float)(sum / (double)(wh * ww));
      }
  }
}

/* CudnnPool2DOp::_backward (src/op.cc:3548-3619): dx_pad = beta*dx_pad + pool'(dy) over the whole
 * padded tile.  MAX: a window's dy goes to its first maximum in row-major window order. */
void orc_pool_slab_bwd(int mode, uint32_t N, uint32_t C, uint32_t HP, uint32_t WP, uint32_t wh, uint32_t ww,
                       uint32_t sh, uint32_t sw, const float *x, const float *dy, float beta, float *dx) {
  const uint32_t OH = (HP - wh) / sh + 1u, OW = (WP - ww) / sw + 1u;
  const uint64_t plane = (uint64_t)HP * WP;
  double *g = (double *)malloc(plane * sizeof(double));
  for (uint64_t pl = 0; pl < (uint64_t)N * C; ++pl) {
    const float *xp = x ? x + pl * plane : NULL;
    const float *dyp = dy + pl * OH * OW;
    float *dxp = dx + pl * plane;
    for (uint64_t i = 0; i < plane; ++i) g[i] = 0.0;
    for (uint32_t oh = 0; oh < OH; ++oh)
      for (uint32_t ow = 0; ow < OW; ++ow) {
        const float d = dyp[(uint64_t)oh * OW + ow];
        if (mode) {
          float mx = -INFINITY;
          uint64_t arg = (uint64_t)(oh * sh) * WP + ow * sw;
          for (uint32_t a = 0; a < wh; ++a)
            for (uint32_t b = 0; b < ww; ++b) {
              const uint64_t i = (uint64_t)(oh * sh + a) * WP + ow * sw + b;
              if (xp[i] > mx) { mx = xp[i]; arg = i; }
            }
          g[arg] += d;
        } else {
          for (uint32_t a = 0; a < wh; ++a)
            for (uint32_t b = 0; b < ww; ++b)
              g[(uint64_t)(oh * sh + a) * WP + ow * sw + b] += (double)d / (double)(wh * ww);
        }
      }
    for (uint64_t i = 0; i < plane; ++i) dxp[i] = (float)((beta != 0.f ? (double)beta * dxp[i] : 0.0) + g[i]);
  }
  free(g);
}

/* ------------------------------------------------------------------ */
/* one host thread per rank: the timed CPU baseline's parallel form     */
/* ------------------------------------------------------------------ */

/* The reference runs one kernel per rank on that rank's own device and stream
 * (Spatial2DComm::group_end, src/spatial.cc:58-201, called once per rank at
 * src/op.cc:2990-2999).  On the host the same split is one thread per rank,
 * each running what orc_halo_op_rank / the per-rank part of pack and unpack /
 * the slab conv runs for its tile.  Results are identical to the loops above:
 * ranks write disjoint elements. */
#include <pthread.h>
#include <unistd.h>

#define ORC_MAX_RANKS 64

uint32_t orc_hardware_threads(void) {
  long n = sysconf(_SC_NPROCESSORS_ONLN);
  return n > 0 ? (uint32_t)n : 1u;
}

typedef struct {
  int kind;  /* 0 halo op, 1 scatter + pad of one tile, 2 unpad + gather of one tile, 3 slab conv fwd f32 */
  int which, dtype, status;
  uint32_t grid_w, grid_h, rank, K, p, W, H, C, N, Cout, k;
  void *const *tiles;
  const void *x_unsplit;
  void *y_unsplit, *scratch;
  const float *x_pad, *wt;
  float *y;
} orc_job;

static void *orc_job_run(void *arg) {
  orc_job *j = (orc_job *)arg;
  const uint32_t Ht = j->K ? j->H / j->K : 0;
  j->status = ORC_OK;
  switch (j->kind) {
    case 0:
      j->status = orc_halo_op_rank(j->which, j->dtype, j->grid_w, j->grid_h, j->rank, j->p, j->W, j->H, j->C, j->N, j->tiles);
      break;
    case 1:
      j->status = orc_slice_nchw(ORC_OP_COPY, j->dtype, j->W, Ht, j->C, j->N, j->x_unsplit, j->W, j->H, j->C, 0,
                                 j->rank * Ht, 0, j->scratch, j->W, Ht, j->C, 0, 0, 0);
      if (!j->status) orc_halo_pad(j->dtype, j->p, j->W, Ht, j->C, j->N, j->scratch, j->tiles[j->rank]);
      break;
    case 2:
      orc_halo_unpad(j->dtype, j->p, j->W, Ht, j->C, j->N, j->tiles[j->rank], j->scratch);
      j->status = orc_slice_nchw(ORC_OP_COPY, j->dtype, j->W, Ht, j->C, j->N, j->scratch, j->W, Ht, j->C, 0, 0, 0,
                                 j->y_unsplit, j->W, j->H, j->C, 0, j->rank * Ht, 0);
      break;
    default:
      orc_conv_slab_fwd_f32(j->N, j->C, j->Cout, j->H, j->W, j->k, j->x_pad, j->wt, j->y);
      break;
  }
  return NULL;
}

static int orc_run_jobs(orc_job *jobs, uint32_t count) {
  pthread_t th[ORC_MAX_RANKS];
  uint32_t started = 0;
  int status = ORC_OK;
  for (; started < count; ++started)
    if (pthread_create(&th[started], NULL, orc_job_run, &jobs[started]) != 0) break;
  for (uint32_t r = started; r < count; ++r) orc_job_run(&jobs[r]); /* could not start: run it here */
  for (uint32_t r = 0; r < started; ++r) pthread_join(th[r], NULL);
  for (uint32_t r = 0; r < count; ++r)
    if (jobs[r].status) status = jobs[r].status;
  return status;
}

/* orc_halo_op with one thread per rank.  An exchange only writes the caller's own halo rows and
 * reads the neighbours' interiors, a reduce only writes interiors and reads halos, so the ranks
 * do not race (the reference relies on the same fact between its per-rank kernels). */
int orc_halo_op_threaded(int which, int dtype, uint32_t grid_w, uint32_t grid_h, uint32_t p, uint32_t W, uint32_t H,
                         uint32_t C, uint32_t N, void *const *tiles) {
  const uint32_t R = grid_w * grid_h;
  if (R == 0 || R > ORC_MAX_RANKS) return ORC_EINVAL;
  orc_job jobs[ORC_MAX_RANKS];
  for (uint32_t r = 0; r < R; ++r) {
    orc_job j = {0};
    j.kind = 0; j.which = which; j.dtype = dtype; j.grid_w = grid_w; j.grid_h = grid_h; j.rank = r;
    j.p = p; j.W = W; j.H = H; j.C = C; j.N = N; j.tiles = tiles;
    jobs[r] = j;
  }
  return orc_run_jobs(jobs, R);
}

/* orc_tiles_pack / orc_tiles_unpack with one thread per tile; `scratch` holds K unpadded tiles. */
int orc_tiles_pack_threaded(int dtype, uint32_t K, uint32_t p, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                            const void *x_unsplit, void *const *tiles, void *scratch) {
  if (K == 0 || K > ORC_MAX_RANKS || H % K != 0) return ORC_EINVAL;
  const size_t tile_bytes = (size_t)N * C * (H / K) * W * orc_esize(dtype);
  orc_job jobs[ORC_MAX_RANKS];
  for (uint32_t r = 0; r < K; ++r) {
    orc_job j = {0};
    j.kind = 1; j.dtype = dtype; j.rank = r; j.K = K; j.p = p; j.W = W; j.H = H; j.C = C; j.N = N;
    j.tiles = tiles; j.x_unsplit = x_unsplit; j.scratch = (char *)scratch + r * tile_bytes;
    jobs[r] = j;
  }
  int e = orc_run_jobs(jobs, K);
  if (e) return e;
  return orc_halo_op_threaded(ORC_EXCH, dtype, 1, K, p, W, H / K, C, N, tiles);
}

int orc_tiles_unpack_threaded(int dtype, uint32_t K, uint32_t p, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                              void *const *tiles, void *y_unsplit, void *scratch) {
  if (K == 0 || K > ORC_MAX_RANKS || H % K != 0) return ORC_EINVAL;
  const size_t tile_bytes = (size_t)N * C * (H / K) * W * orc_esize(dtype);
  orc_job jobs[ORC_MAX_RANKS];
  for (uint32_t r = 0; r < K; ++r) {
    orc_job j = {0};
    j.kind = 2; j.dtype = dtype; j.rank = r; j.K = K; j.p = p; j.W = W; j.H = H; j.C = C; j.N = N;
    j.tiles = tiles; j.y_unsplit = y_unsplit; j.scratch = (char *)scratch + r * tile_bytes;
    jobs[r] = j;
  }
  return orc_run_jobs(jobs, K);
}

/* orc_conv_slab_fwd_f32 of K tiles, one thread per tile (same filter, as the ranks' equal copies). */
int orc_conv_slab_fwd_f32_threaded(uint32_t K, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                                   uint32_t k, const float *const *x_pads, const float *wt, float *const *ys) {
  if (K == 0 || K > ORC_MAX_RANKS) return ORC_EINVAL;
  orc_job jobs[ORC_MAX_RANKS];
  for (uint32_t r = 0; r < K; ++r) {
    orc_job j = {0};
    j.kind = 3; j.N = N; j.C = Cin; j.Cout = Cout; j.H = H; j.W = W; j.k = k;
    j.x_pad = x_pads[r]; j.wt = wt; j.y = ys[r];
    jobs[r] = j;
  }
  return orc_run_jobs(jobs, K);
}
