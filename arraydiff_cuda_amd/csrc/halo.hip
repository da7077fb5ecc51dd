// Data-movement kernels of the spatially-parallel path for gfx950:
// halo exchange / reduce between row (or column) tiles held in one HBM, pad / unpad /
// repad, box slices, and the fused pack (unsplit -> K halo-padded tiles) and unpack.
//
// All of these are HBM-bound copies with at most one add per element.  The two rules
// that shape them:
//   * every destination buffer that is contiguous is written with 16-byte stores by
//     consecutive lanes (a wavefront writes 1 KiB contiguous), the shifted source rows
//     are gathered with element loads that stay inside the same cache lines;
//   * one launch covers all K tiles and all planes: grid = (chunks of one plane, C,
//     N * tiles), so a launch has thousands of workgroups and only one division by a
//     launch-time constant (a mul_hi) per thread.
#include "adh_common.h"

namespace adh {

static constexpr int kBlock = 256;

// ---------------------------------------------------------------------------
// plane_gather: dst planes are contiguous (DW x DH elements each); every dst element is
// either a source element at a shifted position or zero.  Serves pack, pad, repad,
// unpack, unpad and full-row slices.
// ---------------------------------------------------------------------------
struct GatherParams {
  void *dst[ADH_MAX_TILES];
  const void *src[ADH_MAX_TILES];
  uint32_t n_dst;          // number of dst tiles; blockIdx.z = n * n_dst + r
  uint32_t DW, DH;         // dst plane dims; plane_elems = DW * DH
  uint32_t plane_elems;
  uint64_t dst_off;        // element offset of plane (c=0,n=0) in each dst buffer
  uint64_t dst_c_stride, dst_n_stride;
  int32_t off_w, off_h;    // src coords: ws = wp - off_w, gs = hp - off_h + r * row_step
  uint32_t row_step;
  uint32_t valid_w, valid_h;  // src element exists iff 0 <= ws < valid_w && 0 <= gs < valid_h
  uint32_t src_rows_per_tile; // ROW_TILED: source tile = gs / src_rows_per_tile
  uint64_t src_off;           // element offset of (ws=0, gs=0, c=0, n=0) in each src buffer
  uint64_t src_c_stride, src_n_stride;
  uint32_t src_pitch;
  FastDiv div_DW, div_rows;
};

template <typename T, int EPT>
struct VecOf;
template <>
struct VecOf<float, 4> { typedef float4 type; };
template <>
struct VecOf<float, 1> { typedef float type; };
template <>
struct VecOf<uint16_t, 8> { typedef uint4 type; };
template <>
struct VecOf<uint16_t, 1> { typedef uint16_t type; };

template <typename T, int EPT, bool ROW_TILED>
__global__ __launch_bounds__(kBlock) void plane_gather_kernel(const GatherParams P) {
  const uint32_t c = blockIdx.y;
  const uint32_t z = blockIdx.z;
  const uint32_t n = z / P.n_dst;
  const uint32_t r = z - n * P.n_dst;
  const uint32_t e0 = (blockIdx.x * kBlock + threadIdx.x) * EPT;
  if (e0 >= P.plane_elems) return;
  uint32_t hp, wp;
  P.div_DW.divmod(e0, hp, wp);
  const int32_t row_base = (int32_t)(r * P.row_step) - P.off_h;
  const uint64_t src_plane = P.src_off + c * P.src_c_stride + n * P.src_n_stride;
  union {
    typename VecOf<T, EPT>::type v;
    T e[EPT];
  } out;
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int32_t ws = (int32_t)wp - P.off_w;
    int32_t gs = (int32_t)hp + row_base;
    T val = (T)0;
    if ((uint32_t)ws < P.valid_w && (uint32_t)gs < P.valid_h) {
      uint32_t t = 0;
      if (ROW_TILED) {
        t = P.div_rows.div((uint32_t)gs);
        gs -= (int32_t)(t * P.src_rows_per_tile);
      }
      const T *s = reinterpret_cast<const T *>(P.src[t]);
      val = s[src_plane + (uint64_t)gs * P.src_pitch + (uint32_t)ws];
    }
    out.e[i] = val;
    if (++wp == P.DW) {
      wp = 0;
      ++hp;
    }
  }
  T *d = reinterpret_cast<T *>(P.dst[r]) + P.dst_off + c * P.dst_c_stride + n * P.dst_n_stride + e0;
  *reinterpret_cast<typename VecOf<T, EPT>::type *>(d) = out.v;
}

template <typename T, int EPT>
static int launch_gather_t(const GatherParams &P, uint32_t C, uint32_t N, bool row_tiled, hipStream_t st) {
  const uint32_t per_block = kBlock * EPT;
  dim3 grid((P.plane_elems + per_block - 1) / per_block, C, N * P.n_dst);
  if (grid.z > 65535u || grid.y > 65535u) return ADH_EINVAL;
  if (row_tiled)
    hipLaunchKernelGGL((plane_gather_kernel<T, EPT, true>), grid, dim3(kBlock), 0, st, P);
  else
    hipLaunchKernelGGL((plane_gather_kernel<T, EPT, false>), grid, dim3(kBlock), 0, st, P);
  return launch_status();
}

// Picks the 16-byte-store variant when every dst plane start is 16-byte aligned.
static int launch_gather(int dtype, GatherParams &P, uint32_t C, uint32_t N, bool row_tiled, hipStream_t st) {
  if (P.plane_elems == 0 || C == 0 || N == 0) return ADH_OK;
  P.div_DW = FastDiv(P.DW);
  P.div_rows = FastDiv(P.src_rows_per_tile);
  const size_t es = dtype_size(dtype);
  const uint32_t ept = (uint32_t)(16 / es);
  bool vec = (P.plane_elems % ept == 0) && (P.dst_off % ept == 0) && (P.dst_c_stride % ept == 0) &&
             (P.dst_n_stride % ept == 0);
  for (uint32_t r = 0; r < P.n_dst; ++r) vec = vec && aligned_to(P.dst[r], 16);
  if (dtype == ADH_F32)
    return vec ? launch_gather_t<float, 4>(P, C, N, row_tiled, st) : launch_gather_t<float, 1>(P, C, N, row_tiled, st);
  return vec ? launch_gather_t<uint16_t, 8>(P, C, N, row_tiled, st)
             : launch_gather_t<uint16_t, 1>(P, C, N, row_tiled, st);
}

// ---------------------------------------------------------------------------
// box_map: general window copy / add, one element per thread.
// ---------------------------------------------------------------------------
struct BoxParams {
  const void *src;
  void *dst;
  uint32_t cw, ch;  // window extents inside a plane
  uint32_t src_pitch, dst_pitch;
  uint64_t src_off, dst_off;  // element offset of window origin at (c=0, n=0)
  uint64_t src_c_stride, src_n_stride, dst_c_stride, dst_n_stride;
  FastDiv div_cw;
};

template <typename T, bool ADD>
__global__ __launch_bounds__(kBlock) void box_map_kernel(const BoxParams P) {
  const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
  if (e >= P.cw * P.ch) return;
  uint32_t h, w;
  P.div_cw.divmod(e, h, w);
  const uint32_t c = blockIdx.y, n = blockIdx.z;
  const T *s = reinterpret_cast<const T *>(P.src) + P.src_off + c * P.src_c_stride + n * P.src_n_stride +
               (uint64_t)h * P.src_pitch + w;
  T *d = reinterpret_cast<T *>(P.dst) + P.dst_off + c * P.dst_c_stride + n * P.dst_n_stride +
         (uint64_t)h * P.dst_pitch + w;
  if (ADD)
    *d = elem_add(*d, *s);
  else
    *d = *s;
}

static int launch_box(int dtype, bool add, BoxParams &P, uint32_t cc, uint32_t N, hipStream_t st) {
  if (P.cw == 0 || P.ch == 0 || cc == 0 || N == 0) return ADH_OK;
  if ((uint64_t)P.cw * P.ch >= (1ull << 31) || cc > 65535u || N > 65535u) return ADH_EINVAL;
  P.div_cw = FastDiv(P.cw);
  dim3 grid((P.cw * P.ch + kBlock - 1) / kBlock, cc, N);
  if (dtype == ADH_F32) {
    if (add) hipLaunchKernelGGL((box_map_kernel<float, true>), grid, dim3(kBlock), 0, st, P);
    else hipLaunchKernelGGL((box_map_kernel<float, false>), grid, dim3(kBlock), 0, st, P);
  } else {
    if (add) hipLaunchKernelGGL((box_map_kernel<uint16_t, true>), grid, dim3(kBlock), 0, st, P);
    else hipLaunchKernelGGL((box_map_kernel<uint16_t, false>), grid, dim3(kBlock), 0, st, P);
  }
  return launch_status();
}

// ---------------------------------------------------------------------------
// halo strips: a job moves one strip (one row of W, or one column of H, for every
// (c,n)) from a neighbour's buffer into this tile's buffer.
// ---------------------------------------------------------------------------
struct StripJob {
  uint32_t dst_tile, src_tile;
  int32_t dst_pos, src_pos;  // row (or column) index relative to the interior origin
};
static constexpr int kMaxPairs = 2 * (ADH_MAX_TILES - 1);
struct StripParams {
  void *tiles[ADH_MAX_TILES];
  StripJob pairs[kMaxPairs];
  int32_t inc[kMaxPairs];   // step of dst_pos/src_pos per delta
  uint32_t halo_pad;
  uint32_t W, H, PW, PH;    // interior and padded extents
  uint32_t run;             // W for row strips, H for column strips
  uint32_t total;           // run * C * N
  FastDiv div_run;
};

template <typename T, bool ADD, bool COLUMNS>
__global__ __launch_bounds__(kBlock) void halo_strip_kernel(const StripParams P) {
  const uint32_t idx = blockIdx.x * kBlock + threadIdx.x;
  if (idx >= P.total) return;
  const uint32_t pair = blockIdx.y / P.halo_pad;
  const int32_t delta = (int32_t)(blockIdx.y - pair * P.halo_pad);
  const StripJob job = P.pairs[pair];
  const int32_t dpos = job.dst_pos + P.inc[pair] * delta;
  const int32_t spos = job.src_pos + P.inc[pair] * delta;
  uint32_t cn, i;
  P.div_run.divmod(idx, cn, i);
  const uint64_t plane = (uint64_t)cn * P.PW * P.PH;
  uint64_t so, dof;
  if (COLUMNS) {
    const uint64_t row = (uint64_t)(P.halo_pad + i) * P.PW;
    so = plane + row + (uint32_t)((int32_t)P.halo_pad + spos);
    dof = plane + row + (uint32_t)((int32_t)P.halo_pad + dpos);
  } else {
    so = plane + (uint64_t)(uint32_t)((int32_t)P.halo_pad + spos) * P.PW + P.halo_pad + i;
    dof = plane + (uint64_t)(uint32_t)((int32_t)P.halo_pad + dpos) * P.PW + P.halo_pad + i;
  }
  const T *s = reinterpret_cast<const T *>(P.tiles[job.src_tile]) + so;
  T *d = reinterpret_cast<T *>(P.tiles[job.dst_tile]) + dof;
  if (ADD)
    *d = elem_add(*d, *s);
  else
    *d = *s;
}

// rank == UINT32_MAX: all ranks.
static int halo_op(bool reduce, int dtype, uint32_t grid_w, uint32_t grid_h, uint32_t rank, uint32_t p,
                   uint32_t W, uint32_t H, uint32_t C, uint32_t N, void *const *tiles, hipStream_t st) {
  if (!dtype_ok(dtype) || grid_w == 0 || grid_h == 0) return ADH_EINVAL;
  const uint64_t K64 = (uint64_t)grid_w * grid_h;
  if (K64 > ADH_MAX_TILES) return ADH_EINVAL;
  const uint32_t K = (uint32_t)K64;
  if (rank != UINT32_MAX && rank >= K) return ADH_EINVAL;
  if (!tiles) return ADH_ENULL;
  for (uint32_t r = 0; r < K; ++r) {
    if (!tiles[r]) return ADH_ENULL;
    if (!aligned_to(tiles[r], dtype_size(dtype))) return ADH_EALIGN;
  }
  if (grid_w > 1 && grid_h > 1) return ADH_EUNIMPL;
  if (K == 1) return ADH_OK;
  const bool columns = grid_w > 1;
  const uint32_t base = columns ? W : H;
  if (W == 0 || H == 0 || C == 0 || N == 0 || p == 0) return ADH_OK;
  if (base < p) return ADH_EINVAL;              // a strip must come from the neighbour's interior
  if (reduce && base < 2 * p) return ADH_EINVAL;  // single contributor per destination
  const uint64_t plane = (uint64_t)(W + 2 * p) * (H + 2 * p);
  const uint64_t total = (uint64_t)(columns ? H : W) * C * N;
  if (plane * C * N >= (1ull << 31) * 4 || total >= (1ull << 31)) return ADH_EINVAL;

  StripParams P;
  for (uint32_t r = 0; r < K; ++r) P.tiles[r] = tiles[r];
  uint32_t np = 0;
  for (uint32_t r = 0; r < K; ++r) {
    if (rank != UINT32_MAX && r != rank) continue;
    if (r < K - 1) {  // "next" neighbour
      P.pairs[np].dst_tile = r;
      P.pairs[np].src_tile = r + 1;
      if (!reduce) { P.inc[np] = 1;  P.pairs[np].src_pos = 0;  P.pairs[np].dst_pos = (int32_t)base; }
      else         { P.inc[np] = -1; P.pairs[np].src_pos = -1; P.pairs[np].dst_pos = (int32_t)base - 1; }
      ++np;
    }
    if (r > 0) {  // "prev" neighbour
      P.pairs[np].dst_tile = r;
      P.pairs[np].src_tile = r - 1;
      if (!reduce) { P.inc[np] = -1; P.pairs[np].src_pos = (int32_t)base - 1; P.pairs[np].dst_pos = -1; }
      else         { P.inc[np] = 1;  P.pairs[np].src_pos = (int32_t)base;     P.pairs[np].dst_pos = 0; }
      ++np;
    }
  }
  if (np == 0) return ADH_OK;
  P.halo_pad = p;
  P.W = W; P.H = H; P.PW = W + 2 * p; P.PH = H + 2 * p;
  P.run = columns ? H : W;
  P.total = (uint32_t)total;
  P.div_run = FastDiv(P.run);
  dim3 grid((P.total + kBlock - 1) / kBlock, np * p, 1);
  if (grid.y > 65535u) return ADH_EINVAL;
#define ADH_LAUNCH_STRIP(T, ADD, COL) \
  hipLaunchKernelGGL((halo_strip_kernel<T, ADD, COL>), grid, dim3(kBlock), 0, st, P)
  if (dtype == ADH_F32) {
    if (reduce) { if (columns) ADH_LAUNCH_STRIP(float, true, true); else ADH_LAUNCH_STRIP(float, true, false); }
    else        { if (columns) ADH_LAUNCH_STRIP(float, false, true); else ADH_LAUNCH_STRIP(float, false, false); }
  } else {
    if (reduce) { if (columns) ADH_LAUNCH_STRIP(uint16_t, true, true); else ADH_LAUNCH_STRIP(uint16_t, true, false); }
    else        { if (columns) ADH_LAUNCH_STRIP(uint16_t, false, true); else ADH_LAUNCH_STRIP(uint16_t, false, false); }
  }
#undef ADH_LAUNCH_STRIP
  return launch_status();
}

// ---------------------------------------------------------------------------
// fill / add
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void fill_f32_kernel(uint64_t n, float v, float *x) {
  const uint64_t stride = (uint64_t)gridDim.x * kBlock * 4;
  for (uint64_t i = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) * 4; i < n; i += stride) {
    if (i + 4 <= n) {
      *reinterpret_cast<float4 *>(x + i) = make_float4(v, v, v, v);
    } else {
      for (uint64_t j = i; j < n; ++j) x[j] = v;
    }
  }
}

__global__ __launch_bounds__(kBlock) void fill_f32_scalar_kernel(uint64_t n, float v, float *x) {
  const uint64_t stride = (uint64_t)gridDim.x * kBlock;
  for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) x[i] = v;
}

__global__ __launch_bounds__(kBlock) void add_f32_kernel(uint64_t n, const float *x, float *y) {
  const uint64_t stride = (uint64_t)gridDim.x * kBlock * 4;
  for (uint64_t i = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) * 4; i < n; i += stride) {
    if (i + 4 <= n) {
      const float4 a = *reinterpret_cast<const float4 *>(x + i);
      float4 b = *reinterpret_cast<float4 *>(y + i);
      b.x = a.x + b.x; b.y = a.y + b.y; b.z = a.z + b.z; b.w = a.w + b.w;
      *reinterpret_cast<float4 *>(y + i) = b;
    } else {
      for (uint64_t j = i; j < n; ++j) y[j] = x[j] + y[j];
    }
  }
}

__global__ __launch_bounds__(kBlock) void add_f32_scalar_kernel(uint64_t n, const float *x, float *y) {
  const uint64_t stride = (uint64_t)gridDim.x * kBlock;
  for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) y[i] = x[i] + y[i];
}

static uint32_t stream_grid(uint64_t n, uint32_t per_thread) {
  uint64_t blocks = (n + (uint64_t)kBlock * per_thread - 1) / ((uint64_t)kBlock * per_thread);
  const uint64_t cap = 256ull * 16;  // 16 workgroups per CU is plenty for a streaming loop
  if (blocks > cap) blocks = cap;
  if (blocks == 0) blocks = 1;
  return (uint32_t)blocks;
}

static bool plane_limits_ok(uint64_t plane_elems, uint64_t total_elems) {
  return plane_elems < (1ull << 31) && total_elems < (1ull << 40);
}

}  // namespace adh

using namespace adh;

extern "C" {

int adh_fill_f32(uint64_t n, float value, float *x, void *stream) {
  if (n == 0) return ADH_OK;
  if (!x) return ADH_ENULL;
  if (!aligned_to(x, 4)) return ADH_EALIGN;
  if (aligned_to(x, 16))
    hipLaunchKernelGGL(fill_f32_kernel, dim3(stream_grid(n, 4)), dim3(kBlock), 0, as_stream(stream), n, value, x);
  else
    hipLaunchKernelGGL(fill_f32_scalar_kernel, dim3(stream_grid(n, 1)), dim3(kBlock), 0, as_stream(stream), n, value, x);
  return launch_status();
}

int adh_add_f32(uint64_t n, const float *x, float *y, void *stream) {
  if (n == 0) return ADH_OK;
  if (!x || !y) return ADH_ENULL;
  if (!aligned_to(x, 4) || !aligned_to(y, 4)) return ADH_EALIGN;
  if (aligned_to(x, 16) && aligned_to(y, 16))
    hipLaunchKernelGGL(add_f32_kernel, dim3(stream_grid(n, 4)), dim3(kBlock), 0, as_stream(stream), n, x, y);
  else
    hipLaunchKernelGGL(add_f32_scalar_kernel, dim3(stream_grid(n, 1)), dim3(kBlock), 0, as_stream(stream), n, x, y);
  return launch_status();
}

int adh_halo_exchange_nchw(int dtype, uint32_t grid_w, uint32_t grid_h, uint32_t halo_pad, uint32_t W,
                           uint32_t H, uint32_t C, uint32_t N, void *const *tile_bufs, void *stream) {
  return halo_op(false, dtype, grid_w, grid_h, UINT32_MAX, halo_pad, W, H, C, N, tile_bufs, as_stream(stream));
}

int adh_halo_reduce_nchw(int dtype, uint32_t grid_w, uint32_t grid_h, uint32_t halo_pad, uint32_t W,
                         uint32_t H, uint32_t C, uint32_t N, void *const *tile_bufs, void *stream) {
  return halo_op(true, dtype, grid_w, grid_h, UINT32_MAX, halo_pad, W, H, C, N, tile_bufs, as_stream(stream));
}

int adh_halo_exchange_nchw_rank(int dtype, uint32_t grid_w, uint32_t grid_h, uint32_t rank, uint32_t halo_pad,
                                uint32_t W, uint32_t H, uint32_t C, uint32_t N, void *const *tile_bufs,
                                void *stream) {
  if (rank == UINT32_MAX) return ADH_EINVAL;
  return halo_op(false, dtype, grid_w, grid_h, rank, halo_pad, W, H, C, N, tile_bufs, as_stream(stream));
}

int adh_halo_reduce_nchw_rank(int dtype, uint32_t grid_w, uint32_t grid_h, uint32_t rank, uint32_t halo_pad,
                              uint32_t W, uint32_t H, uint32_t C, uint32_t N, void *const *tile_bufs,
                              void *stream) {
  if (rank == UINT32_MAX) return ADH_EINVAL;
  return halo_op(true, dtype, grid_w, grid_h, rank, halo_pad, W, H, C, N, tile_bufs, as_stream(stream));
}

// dst = padded (W+2q, H+2q) planes, src = interior of padded-by-ps planes (ps = 0: packed)
static int pad_like(int dtype, uint32_t ps, uint32_t q, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                    const void *x, void *y, void *stream) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if (W == 0 || H == 0 || C == 0 || N == 0) return ADH_OK;
  if (!x || !y) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  if (!aligned_to(x, es) || !aligned_to(y, es)) return ADH_EALIGN;
  const uint64_t DW = (uint64_t)W + 2 * q, DH = (uint64_t)H + 2 * q;
  const uint64_t SW = (uint64_t)W + 2 * ps, SH = (uint64_t)H + 2 * ps;
  if (!plane_limits_ok(DW * DH, DW * DH * C * N) || !plane_limits_ok(SW * SH, SW * SH * C * N)) return ADH_EINVAL;
  GatherParams P = {};
  P.dst[0] = y;
  P.src[0] = x;
  P.n_dst = 1;
  P.DW = (uint32_t)DW; P.DH = (uint32_t)DH; P.plane_elems = (uint32_t)(DW * DH);
  P.dst_off = 0; P.dst_c_stride = DW * DH; P.dst_n_stride = DW * DH * C;
  P.off_w = (int32_t)q; P.off_h = (int32_t)q; P.row_step = 0;
  P.valid_w = W; P.valid_h = H; P.src_rows_per_tile = 1;
  P.src_off = (uint64_t)ps * SW + ps; P.src_c_stride = SW * SH; P.src_n_stride = SW * SH * C;
  P.src_pitch = (uint32_t)SW;
  return launch_gather(dtype, P, C, N, false, as_stream(stream));
}

int adh_halo_pad_nchw(int dtype, uint32_t halo_pad, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                      const void *x_packed, void *y_padded, void *stream) {
  return pad_like(dtype, 0, halo_pad, W, H, C, N, x_packed, y_padded, stream);
}

int adh_halo_unpad_nchw(int dtype, uint32_t halo_pad, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                        const void *x_padded, void *y_packed, void *stream) {
  return pad_like(dtype, halo_pad, 0, W, H, C, N, x_padded, y_packed, stream);
}

int adh_halo_repad_nchw(int dtype, uint32_t pad_src, uint32_t pad_dst, uint32_t W, uint32_t H, uint32_t C,
                        uint32_t N, const void *x_padded, void *y_padded, void *stream) {
  return pad_like(dtype, pad_src, pad_dst, W, H, C, N, x_padded, y_padded, stream);
}

static int slice_op(bool add, int dtype, uint32_t cw, uint32_t ch, uint32_t cc, uint32_t N, const void *src,
                    uint32_t sW, uint32_t sH, uint32_t sC, uint32_t sw, uint32_t sh, uint32_t sc, void *dst,
                    uint32_t dW, uint32_t dH, uint32_t dC, uint32_t dw, uint32_t dh, uint32_t dc, void *stream) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if ((uint64_t)sw + cw > sW || (uint64_t)sh + ch > sH || (uint64_t)sc + cc > sC || (uint64_t)dw + cw > dW ||
      (uint64_t)dh + ch > dH || (uint64_t)dc + cc > dC)
    return ADH_EINVAL;
  if (cw == 0 || ch == 0 || cc == 0 || N == 0) return ADH_OK;
  if (!src || !dst) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  if (!aligned_to(src, es) || !aligned_to(dst, es)) return ADH_EALIGN;
  const uint64_t splane = (uint64_t)sW * sH, dplane = (uint64_t)dW * dH;
  if (!plane_limits_ok(splane, splane * sC * N) || !plane_limits_ok(dplane, dplane * dC * N)) return ADH_EINVAL;
  if (!add && cw == dW && ch == dH) {
    // dst window = whole planes: contiguous destination, 16-byte stores
    GatherParams P = {};
    P.dst[0] = dst;
    P.src[0] = src;
    P.n_dst = 1;
    P.DW = dW; P.DH = dH; P.plane_elems = (uint32_t)dplane;
    P.dst_off = (uint64_t)dc * dplane; P.dst_c_stride = dplane; P.dst_n_stride = dplane * dC;
    P.off_w = 0; P.off_h = 0; P.row_step = 0;
    P.valid_w = cw; P.valid_h = ch; P.src_rows_per_tile = 1;
    P.src_off = (uint64_t)sc * splane + (uint64_t)sh * sW + sw;
    P.src_c_stride = splane; P.src_n_stride = splane * sC; P.src_pitch = sW;
    return launch_gather(dtype, P, cc, N, false, as_stream(stream));
  }
  BoxParams B = {};
  B.src = src; B.dst = dst;
  B.cw = cw; B.ch = ch;
  B.src_pitch = sW; B.dst_pitch = dW;
  B.src_off = (uint64_t)sc * splane + (uint64_t)sh * sW + sw;
  B.dst_off = (uint64_t)dc * dplane + (uint64_t)dh * dW + dw;
  B.src_c_stride = splane; B.src_n_stride = splane * sC;
  B.dst_c_stride = dplane; B.dst_n_stride = dplane * dC;
  return launch_box(dtype, add, B, cc, N, as_stream(stream));
}

int adh_slice_copy_nchw(int dtype, uint32_t count_w, uint32_t count_h, uint32_t count_c, uint32_t N,
                        const void *src, uint32_t src_W, uint32_t src_H, uint32_t src_C, uint32_t src_w_off,
                        uint32_t src_h_off, uint32_t src_c_off, void *dst, uint32_t dst_W, uint32_t dst_H,
                        uint32_t dst_C, uint32_t dst_w_off, uint32_t dst_h_off, uint32_t dst_c_off, void *stream) {
  return slice_op(false, dtype, count_w, count_h, count_c, N, src, src_W, src_H, src_C, src_w_off, src_h_off,
                  src_c_off, dst, dst_W, dst_H, dst_C, dst_w_off, dst_h_off, dst_c_off, stream);
}

int adh_slice_add_nchw(int dtype, uint32_t count_w, uint32_t count_h, uint32_t count_c, uint32_t N,
                       const void *src, uint32_t src_W, uint32_t src_H, uint32_t src_C, uint32_t src_w_off,
                       uint32_t src_h_off, uint32_t src_c_off, void *dst, uint32_t dst_W, uint32_t dst_H,
                       uint32_t dst_C, uint32_t dst_w_off, uint32_t dst_h_off, uint32_t dst_c_off, void *stream) {
  return slice_op(true, dtype, count_w, count_h, count_c, N, src, src_W, src_H, src_C, src_w_off, src_h_off,
                  src_c_off, dst, dst_W, dst_H, dst_C, dst_w_off, dst_h_off, dst_c_off, stream);
}

int adh_halo_pad_add_nchw(int dtype, uint32_t p, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                          const void *x_packed, void *y_padded, void *stream) {
  return slice_op(true, dtype, W, H, C, N, x_packed, W, H, C, 0, 0, 0, y_padded, W + 2 * p, H + 2 * p, C, p, p, 0,
                  stream);
}

int adh_halo_unpad_add_nchw(int dtype, uint32_t p, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                            const void *x_padded, void *y_packed, void *stream) {
  return slice_op(true, dtype, W, H, C, N, x_padded, W + 2 * p, H + 2 * p, C, p, p, 0, y_packed, W, H, C, 0, 0, 0,
                  stream);
}

int adh_tiles_pack_nchw(int dtype, uint32_t K, uint32_t p, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                        const void *x_unsplit, void *const *tile_bufs, void *stream) {
  if (!dtype_ok(dtype) || K == 0 || K > ADH_MAX_TILES || H % K != 0) return ADH_EINVAL;
  if (W == 0 || H == 0 || C == 0 || N == 0) return ADH_OK;
  const uint32_t Ht = H / K;
  if (K > 1 && Ht < p) return ADH_EINVAL;
  if (!x_unsplit || !tile_bufs) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  if (!aligned_to(x_unsplit, es)) return ADH_EALIGN;
  const uint64_t DW = (uint64_t)W + 2 * p, DH = (uint64_t)Ht + 2 * p;
  if (!plane_limits_ok(DW * DH, DW * DH * C * N) || !plane_limits_ok((uint64_t)W * H, (uint64_t)W * H * C * N))
    return ADH_EINVAL;
  GatherParams P = {};
  for (uint32_t r = 0; r < K; ++r) {
    if (!tile_bufs[r]) return ADH_ENULL;
    if (!aligned_to(tile_bufs[r], es)) return ADH_EALIGN;
    P.dst[r] = tile_bufs[r];
  }
  P.src[0] = x_unsplit;
  P.n_dst = K;
  P.DW = (uint32_t)DW; P.DH = (uint32_t)DH; P.plane_elems = (uint32_t)(DW * DH);
  P.dst_off = 0; P.dst_c_stride = DW * DH; P.dst_n_stride = DW * DH * C;
  P.off_w = (int32_t)p; P.off_h = (int32_t)p; P.row_step = Ht;
  P.valid_w = W; P.valid_h = H; P.src_rows_per_tile = 1;
  P.src_off = 0; P.src_c_stride = (uint64_t)W * H; P.src_n_stride = (uint64_t)W * H * C; P.src_pitch = W;
  return launch_gather(dtype, P, C, N, false, as_stream(stream));
}

int adh_tiles_unpack_nchw(int dtype, uint32_t K, uint32_t p, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                          const void *const *tile_bufs, void *y_unsplit, void *stream) {
  if (!dtype_ok(dtype) || K == 0 || K > ADH_MAX_TILES || H % K != 0) return ADH_EINVAL;
  if (W == 0 || H == 0 || C == 0 || N == 0) return ADH_OK;
  const uint32_t Ht = H / K;
  if (!y_unsplit || !tile_bufs) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  if (!aligned_to(y_unsplit, es)) return ADH_EALIGN;
  const uint64_t SW = (uint64_t)W + 2 * p, SH = (uint64_t)Ht + 2 * p;
  if (!plane_limits_ok(SW * SH, SW * SH * C * N) || !plane_limits_ok((uint64_t)W * H, (uint64_t)W * H * C * N))
    return ADH_EINVAL;
  GatherParams P = {};
  for (uint32_t r = 0; r < K; ++r) {
    if (!tile_bufs[r]) return ADH_ENULL;
    if (!aligned_to(tile_bufs[r], es)) return ADH_EALIGN;
    P.src[r] = tile_bufs[r];
  }
  P.dst[0] = y_unsplit;
  P.n_dst = 1;
  P.DW = W; P.DH = H; P.plane_elems = (uint32_t)((uint64_t)W * H);
  P.dst_off = 0; P.dst_c_stride = (uint64_t)W * H; P.dst_n_stride = (uint64_t)W * H * C;
  P.off_w = 0; P.off_h = 0; P.row_step = 0;
  P.valid_w = W; P.valid_h = H; P.src_rows_per_tile = Ht;
  P.src_off = (uint64_t)p * SW + p; P.src_c_stride = SW * SH; P.src_n_stride = SW * SH * C;
  P.src_pitch = (uint32_t)SW;
  return launch_gather(dtype, P, C, N, true, as_stream(stream));
}

}  // extern "C"
