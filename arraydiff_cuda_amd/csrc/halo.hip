// Data-movement kernels of the spatially-parallel path for gfx950:
// halo exchange / reduce between row (or column) tiles held in one HBM, pad / unpad /
// repad, box slices, and the fused pack (unsplit -> K halo-padded tiles) and unpack.
//
// All of these are HBM-bound copies with at most one add per element.  The two rules
// that shape them:
//   * every destination buffer that is contiguous is written with aligned 16-byte stores by
//     consecutive lanes (a wavefront writes 1 KiB contiguous); the matching source run is
//     fetched with ONE 16-byte load at the source's own element alignment (padded rows are
//     shifted by 2p elements per row, so source and destination can never both be 16-byte
//     aligned); only vectors that straddle a row end fall back to element loads;
//   * one launch covers all K tiles and all planes, so a launch has thousands of
//     workgroups; index arithmetic is two or three divisions by launch-time constants
//     (mul_hi + shift) per 16 bytes.
#include "adh_common.h"

namespace adh {

static constexpr int kBlock = 256;

// ---------------------------------------------------------------------------
// row_copy: the one copy kernel behind pack, unpack, pad, unpad, repad and all slices.
//
// For every destination row (hp, c, n) of every destination buffer r:
//   source row gs = hp - off_h + r*row_step; if 0 <= gs < valid_h the W elements
//   dst[hp][off_w .. off_w+W) are copied from (or, ADD, incremented by) the source row,
//   else they are zeroed (never when ADD);
//   with ZERO_BORDER the dst columns left and right of the copied run are zeroed too.
// A thread moves one vector of EPT consecutive elements of a row with ONE 16-byte load and
// ONE 16-byte store, both at element alignment (padded rows are shifted by 2p elements per
// row, so source and destination can never both be 16-byte aligned; the hardware takes
// unaligned vector accesses, and a wavefront still touches one contiguous run per row).
// Each thread handles VPT vectors, all loads issued before the first store.
// ---------------------------------------------------------------------------
struct RowCopyParams {
  void *dst[ADH_MAX_TILES];        // per launch-row r = blockIdx.y
  const void *src[ADH_MAX_TILES];
  uint32_t W;                // elements moved per row
  uint32_t VR;               // vectors per row = ceil(W / EPT)
  uint32_t DH;               // destination rows per plane
  uint32_t C;                // planes per image (plane = c + C*n)
  uint32_t total_vectors;    // VR * DH * C * N  (per destination buffer)
  uint32_t dst_pitch, off_w; // dst row pitch and first written column
  uint32_t border_l, border_r;  // ZERO_BORDER: columns zeroed left / right of the run
  uint64_t dst_off, dst_c_stride, dst_n_stride;
  int32_t off_h;
  uint32_t row_step, valid_h;
  uint32_t src_pitch;
  uint64_t src_off, src_c_stride, src_n_stride;
  FastDiv div_VR, div_DH, div_C;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// 16 bytes at 2-byte alignment: valid for both element types (fp32 rows are 4-byte aligned)
typedef u32x4 u32x4_unaligned __attribute__((aligned(2)));

// TAIL = (W % EPT != 0): the last vector of a row is partial and is moved element-wise.
// STREAM = the transfer is larger than the on-package cache: loads and stores are marked
// non-temporal so that lines are not kept (a few percent more bandwidth from HBM, but a loss
// when the data would have stayed cache-resident, so the host decides by size).
template <typename T, bool ADD, bool ZERO_BORDER, bool TAIL, bool STREAM, int VPT>
__global__ __launch_bounds__(kBlock) void row_copy_kernel(const RowCopyParams P) {
  constexpr int EPT = 16 / sizeof(T);
  typedef u32x4_unaligned VU;
  union Pack {
    u32x4 v;
    T e[EPT];
  };
  const uint32_t r = blockIdx.y;
  const T *__restrict__ sbase = reinterpret_cast<const T *>(P.src[r]) + P.src_off;
  T *__restrict__ dbase = reinterpret_cast<T *>(P.dst[r]) + P.dst_off;
  const int32_t row_base = (int32_t)(r * P.row_step) - P.off_h;

  uint64_t so[VPT], dof[VPT];
  uint32_t cnt[VPT];   // elements of this vector inside the row (0 = no work)
  bool have_src[VPT], first[VPT];
  u32x4 in[VPT], old[VPT];

#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const uint32_t v = (blockIdx.x * VPT + k) * kBlock + threadIdx.x;
    const bool live = v < P.total_vectors;
    uint32_t row, vr, pl, hp, n, c;
    P.div_VR.divmod(live ? v : 0u, row, vr);
    P.div_DH.divmod(row, pl, hp);
    P.div_C.divmod(pl, n, c);
    const uint32_t w0 = vr * EPT;
    cnt[k] = live ? (TAIL ? min((uint32_t)EPT, P.W - w0) : (uint32_t)EPT) : 0u;
    first[k] = vr == 0;
    const int32_t gs = (int32_t)hp + row_base;
    have_src[k] = (uint32_t)gs < P.valid_h;
    so[k] = c * P.src_c_stride + n * P.src_n_stride + (uint64_t)(have_src[k] ? (uint32_t)gs : 0u) * P.src_pitch + w0;
    dof[k] = c * P.dst_c_stride + n * P.dst_n_stride + (uint64_t)hp * P.dst_pitch + P.off_w + w0;
    in[k] = u32x4{0u, 0u, 0u, 0u};
    old[k] = u32x4{0u, 0u, 0u, 0u};
  }
  // all loads first
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    // addresses are valid even for idle threads and zero rows (clamped above), so the
    // vector loads need no branch when rows have no tail
    if (!TAIL || cnt[k] == (uint32_t)EPT) {
      in[k] = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const VU *>(sbase + so[k]))
                     : *reinterpret_cast<const VU *>(sbase + so[k]);
      if (ADD) old[k] = *reinterpret_cast<const VU *>(dbase + dof[k]);
    } else if (TAIL && cnt[k] > 0) {
      Pack pi, po;
      pi.v = in[k];
      po.v = old[k];
#pragma unroll
      for (int i = 0; i < EPT - 1; ++i) {
        if ((uint32_t)i < cnt[k]) {
          pi.e[i] = sbase[so[k] + i];
          if (ADD) po.e[i] = dbase[dof[k] + i];
        }
      }
      in[k] = pi.v;
      old[k] = po.v;
    }
  }
  // Keep every load above this point (the empty asm consumes the loaded registers), so the
  // compiler cannot sink a load into its store's branch and serialise load -> wait -> store.
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    asm volatile("" : "+v"(in[k]));
    if (ADD) asm volatile("" : "+v"(old[k]));
  }
  // then all stores
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    if (cnt[k] == 0) continue;
    if (ADD && !have_src[k]) continue;
    Pack out;
    if (ADD) {
      Pack pi, po;
      pi.v = in[k];
      po.v = old[k];
#pragma unroll
      for (int i = 0; i < EPT; ++i) out.e[i] = elem_add(po.e[i], pi.e[i]);
    } else {
      out.v = have_src[k] ? in[k] : u32x4{0u, 0u, 0u, 0u};
    }
    T *d = dbase + dof[k];
    if (!TAIL || cnt[k] == (uint32_t)EPT) {
      if (STREAM) __builtin_nontemporal_store(out.v, reinterpret_cast<VU *>(d));
      else *reinterpret_cast<VU *>(d) = out.v;
    } else {
#pragma unroll
      for (int i = 0; i < EPT - 1; ++i)
        if ((uint32_t)i < cnt[k]) d[i] = out.e[i];
    }
    if (ZERO_BORDER && first[k]) {
      T *row = d - P.off_w;
      for (uint32_t i = 0; i < P.border_l; ++i) row[i] = (T)0;
      for (uint32_t i = 0; i < P.border_r; ++i) row[P.off_w + P.W + i] = (T)0;
    }
  }
}

template <typename T, bool STREAM, int VPT = 2>
static void launch_row_copy_t(bool add, bool zero_border, bool tail, const RowCopyParams &P, dim3 grid,
                              hipStream_t st) {
#define ADH_RC(A, Z, TL) hipLaunchKernelGGL((row_copy_kernel<T, A, Z, TL, STREAM, VPT>), grid, dim3(kBlock), 0, st, P)
  if (add) { if (tail) ADH_RC(true, false, true); else ADH_RC(true, false, false); }
  else if (zero_border) { if (tail) ADH_RC(false, true, true); else ADH_RC(false, true, false); }
  else { if (tail) ADH_RC(false, false, true); else ADH_RC(false, false, false); }
#undef ADH_RC
}

// N is the image count; P.C must be set.  All extents validated by the callers.
static int launch_row_copy(int dtype, bool add, bool zero_border, RowCopyParams &P, uint32_t n_dst, uint32_t N,
                           hipStream_t st) {
  if (P.W == 0 || P.DH == 0 || P.C == 0 || N == 0 || n_dst == 0) return ADH_OK;
  const uint32_t ept = (uint32_t)(16 / dtype_size(dtype));
  P.VR = (P.W + ept - 1) / ept;
  const uint64_t total = (uint64_t)P.VR * P.DH * P.C * N;
  if (total >= (1ull << 31)) return ADH_EINVAL;
  P.total_vectors = (uint32_t)total;
  P.div_VR = FastDiv(P.VR);
  P.div_DH = FastDiv(P.DH);
  P.div_C = FastDiv(P.C);
  const bool tail = P.W % ept != 0;
  // bytes read + written by the launch; above half of the 256 MB on-package cache nothing
  // would stay resident anyway
  const uint64_t moved = 2ull * P.W * P.DH * P.C * N * n_dst * dtype_size(dtype);
  const bool stream = moved > (128ull << 20);
  // Vectors per thread: two, but for bf16 transfers from and to HBM with long rows.  Measured on 1 GB transfers
  // with rows of 1000 to 4096 elements: where the destination is the skewed side (pack, pad: rows with a zeroed
  // border) one vector per thread moves 3-7 % more bytes a second than two, three or four (5.9 against 5.55 TB/s at
  // 8 tiles of 128 x 2048); where the source is (unpack, unpad, slices) three do, from 256 vectors a row on (5.88
  // against 5.60 TB/s).  fp32 rows and cache-resident sizes showed no such preference.
  int vpt = 2;
  if (stream && dtype == ADH_BF16 && !add) {
    if (zero_border && P.VR >= 120u) vpt = 1;
    else if (!zero_border && P.VR >= 256u) vpt = 3;
  }
  dim3 grid((P.total_vectors + kBlock * vpt - 1) / (kBlock * vpt), n_dst, 1);
  if (dtype == ADH_F32) {
    if (stream) launch_row_copy_t<float, true>(add, zero_border, tail, P, grid, st);
    else launch_row_copy_t<float, false>(add, zero_border, tail, P, grid, st);
  } else if (!stream) {
    launch_row_copy_t<uint16_t, false>(add, zero_border, tail, P, grid, st);
  } else if (vpt == 1) {
    launch_row_copy_t<uint16_t, true, 1>(add, zero_border, tail, P, grid, st);
  } else if (vpt == 3) {
    launch_row_copy_t<uint16_t, true, 3>(add, zero_border, tail, P, grid, st);
  } else {
    launch_row_copy_t<uint16_t, true>(add, zero_border, tail, P, grid, st);
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

// VEC elements per thread (row strips only): 16-byte accesses, which need no alignment beyond the element's.
template <typename T, bool ADD, bool COLUMNS, int VEC>
__global__ __launch_bounds__(kBlock) void halo_strip_kernel(const StripParams P) {
  const uint32_t idx = blockIdx.x * kBlock + threadIdx.x;
  if (idx >= P.total) return;
  const uint32_t pair = blockIdx.y / P.halo_pad;
  const int32_t delta = (int32_t)(blockIdx.y - pair * P.halo_pad);
  const StripJob job = P.pairs[pair];
  const int32_t dpos = job.dst_pos + P.inc[pair] * delta;
  const int32_t spos = job.src_pos + P.inc[pair] * delta;
  uint32_t cn, i;
  P.div_run.divmod(idx, cn, i);  // run is counted in groups of VEC elements
  i *= (uint32_t)VEC;
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
  if (VEC == 1) {
    if (ADD)
      *d = elem_add(*d, *s);
    else
      *d = *s;
  } else {
    struct __attribute__((packed, aligned(sizeof(T)))) Vec { T v[VEC]; };
    Vec a = *reinterpret_cast<const Vec *>(s);
    if (ADD) {
      const Vec b = *reinterpret_cast<const Vec *>(d);
#pragma unroll
      for (int k = 0; k < VEC; ++k) a.v[k] = elem_add(b.v[k], a.v[k]);
    }
    *reinterpret_cast<Vec *>(d) = a;
  }
}


// Column strips through LDS: a workgroup takes one plane of one neighbour pair, copies the source
// plane's interior rows into LDS as they lie in memory (contiguous 16-byte accesses instead of one
// element per row and lane), and then moves the halo_pad columns out of LDS to their places.  Only the
// strip's own columns of the staged rows are used; what other workgroups write elsewhere in the
// source plane meanwhile is staged but never used.
// Measured against halo_strip_kernel<.., COLUMNS = true, 1> (N=32, C=64, fp32): 14-column tiles
// 10.5 us against 9.7 (exchange) and 10.9 against 11.2 (reduce); 56-column tiles 31.0 against 19.0
// and 38.8 against 27.1; halo 3 over 64 columns 15.8 against 12.6 (exchange) and 16.3 against 19.7
// (reduce).  It fetches 1.4 to 1.7 times the bytes, because a strip only needs the line of each row
// that holds its column while the staging reads whole rows: every row of a column strip is its own
// line of memory whatever the order it is asked for in.  It pays where several columns of a row are
// read and written back (a reduce over a halo of two or more columns), and that is where halo_op
// selects it; every other column strip takes the direct kernel.
template <typename T, bool ADD>
__global__ __launch_bounds__(kBlock) void halo_column_staged_kernel(const StripParams P) {
  extern __shared__ __attribute__((aligned(16))) uint8_t staged_rows[];
  T *lds = reinterpret_cast<T *>(staged_rows);
  constexpr uint32_t kVecElems = 16 / sizeof(T);
  struct __attribute__((packed, aligned(sizeof(T)))) Vec { T v[kVecElems]; };
  const uint32_t cn = blockIdx.x, pair = blockIdx.y;
  const StripJob job = P.pairs[pair];
  const uint64_t plane = (uint64_t)cn * P.PW * P.PH;
  const T *s = reinterpret_cast<const T *>(P.tiles[job.src_tile]) + plane + (uint64_t)P.halo_pad * P.PW;
  T *d = reinterpret_cast<T *>(P.tiles[job.dst_tile]) + plane + (uint64_t)P.halo_pad * P.PW;
  const uint32_t elems = P.H * P.PW;
  for (uint32_t i = threadIdx.x * kVecElems; i < elems; i += kBlock * kVecElems) {
    if (i + kVecElems <= elems) {
      *reinterpret_cast<Vec *>(lds + i) = *reinterpret_cast<const Vec *>(s + i);
    } else {
      for (uint32_t j = i; j < elems; ++j) lds[j] = s[j];
    }
  }
  __syncthreads();
  const uint32_t count = P.H * P.halo_pad;
  for (uint32_t i = threadIdx.x; i < count; i += kBlock) {
    const uint32_t row = i / P.halo_pad;
    const int32_t delta = (int32_t)(i - row * P.halo_pad);
    const uint32_t sc = (uint32_t)((int32_t)P.halo_pad + job.src_pos + P.inc[pair] * delta);
    const uint32_t dc = (uint32_t)((int32_t)P.halo_pad + job.dst_pos + P.inc[pair] * delta);
    const T v = lds[row * P.PW + sc];
    T *dst = d + (uint64_t)row * P.PW + dc;
    if (ADD)
      *dst = elem_add(*dst, v);
    else
      *dst = v;
  }
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
  // row strips whose length is a whole number of 16-byte groups move 16 bytes per thread
  const uint32_t vec = (uint32_t)(16 / dtype_size(dtype));
  const bool wide = !columns && W % vec == 0;
  if (wide) P.run = W / vec;
  P.total = (uint32_t)(wide ? total / vec : total);
  P.div_run = FastDiv(P.run);
  if (columns && reduce && p >= 2 && (uint64_t)H * P.PW * dtype_size(dtype) <= 48u * 1024u && (uint64_t)C * N <= 0x7fffffffull) {
    const dim3 sgrid(C * N, np, 1);
    const size_t lds_bytes = (size_t)H * P.PW * dtype_size(dtype);
    if (dtype == ADH_F32) hipLaunchKernelGGL((halo_column_staged_kernel<float, true>), sgrid, dim3(kBlock), lds_bytes, st, P);
    else hipLaunchKernelGGL((halo_column_staged_kernel<uint16_t, true>), sgrid, dim3(kBlock), lds_bytes, st, P);
    return launch_status();
  }
  dim3 grid((P.total + kBlock - 1) / kBlock, np * p, 1);
  if (grid.y > 65535u) return ADH_EINVAL;
#define ADH_LAUNCH_STRIP(T, ADD, COL, V) \
  hipLaunchKernelGGL((halo_strip_kernel<T, ADD, COL, V>), grid, dim3(kBlock), 0, st, P)
  if (dtype == ADH_F32) {
    if (columns) { if (reduce) ADH_LAUNCH_STRIP(float, true, true, 1); else ADH_LAUNCH_STRIP(float, false, true, 1); }
    else if (wide) { if (reduce) ADH_LAUNCH_STRIP(float, true, false, 4); else ADH_LAUNCH_STRIP(float, false, false, 4); }
    else { if (reduce) ADH_LAUNCH_STRIP(float, true, false, 1); else ADH_LAUNCH_STRIP(float, false, false, 1); }
  } else {
    if (columns) { if (reduce) ADH_LAUNCH_STRIP(uint16_t, true, true, 1); else ADH_LAUNCH_STRIP(uint16_t, false, true, 1); }
    else if (wide) { if (reduce) ADH_LAUNCH_STRIP(uint16_t, true, false, 8); else ADH_LAUNCH_STRIP(uint16_t, false, false, 8); }
    else { if (reduce) ADH_LAUNCH_STRIP(uint16_t, true, false, 1); else ADH_LAUNCH_STRIP(uint16_t, false, false, 1); }
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
  RowCopyParams P = {};
  P.dst[0] = y;
  P.src[0] = x;
  P.W = W; P.DH = (uint32_t)DH; P.C = C;
  P.dst_pitch = (uint32_t)DW; P.off_w = q; P.border_l = q; P.border_r = q;
  P.dst_off = 0; P.dst_c_stride = DW * DH; P.dst_n_stride = DW * DH * C;
  P.off_h = (int32_t)q; P.row_step = 0; P.valid_h = H;
  P.src_pitch = (uint32_t)SW;
  P.src_off = (uint64_t)ps * SW + ps; P.src_c_stride = SW * SH; P.src_n_stride = SW * SH * C;
  return launch_row_copy(dtype, false, q > 0, P, 1, N, as_stream(stream));
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
  RowCopyParams P = {};
  P.dst[0] = dst;
  P.src[0] = src;
  P.W = cw; P.DH = ch; P.C = cc;
  P.dst_pitch = dW; P.off_w = 0;
  P.dst_off = (uint64_t)dc * dplane + (uint64_t)dh * dW + dw; P.dst_c_stride = dplane; P.dst_n_stride = dplane * dC;
  P.off_h = 0; P.row_step = 0; P.valid_h = ch;
  P.src_pitch = sW;
  P.src_off = (uint64_t)sc * splane + (uint64_t)sh * sW + sw; P.src_c_stride = splane; P.src_n_stride = splane * sC;
  return launch_row_copy(dtype, add, false, P, 1, N, as_stream(stream));
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
  RowCopyParams P = {};
  for (uint32_t r = 0; r < K; ++r) {
    if (!tile_bufs[r]) return ADH_ENULL;
    if (!aligned_to(tile_bufs[r], es)) return ADH_EALIGN;
    P.dst[r] = tile_bufs[r];
    P.src[r] = x_unsplit;
  }
  P.W = W; P.DH = (uint32_t)DH; P.C = C;
  P.dst_pitch = (uint32_t)DW; P.off_w = p; P.border_l = p; P.border_r = p;
  P.dst_off = 0; P.dst_c_stride = DW * DH; P.dst_n_stride = DW * DH * C;
  P.off_h = (int32_t)p; P.row_step = Ht; P.valid_h = H;
  P.src_pitch = W;
  P.src_off = 0; P.src_c_stride = (uint64_t)W * H; P.src_n_stride = (uint64_t)W * H * C;
  return launch_row_copy(dtype, false, p > 0, P, K, N, as_stream(stream));
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
  RowCopyParams P = {};
  for (uint32_t r = 0; r < K; ++r) {
    if (!tile_bufs[r]) return ADH_ENULL;
    if (!aligned_to(tile_bufs[r], es)) return ADH_EALIGN;
    P.src[r] = tile_bufs[r];
    P.dst[r] = reinterpret_cast<char *>(y_unsplit) + (size_t)r * Ht * W * es;  // rows [r*Ht, (r+1)*Ht)
  }
  P.W = W; P.DH = Ht; P.C = C;
  P.dst_pitch = W; P.off_w = 0;
  P.dst_off = 0; P.dst_c_stride = (uint64_t)W * H; P.dst_n_stride = (uint64_t)W * H * C;
  P.off_h = 0; P.row_step = 0; P.valid_h = Ht;
  P.src_pitch = (uint32_t)SW;
  P.src_off = (uint64_t)p * SW + p; P.src_c_stride = SW * SH; P.src_n_stride = SW * SH * C;
  return launch_row_copy(dtype, false, false, P, K, N, as_stream(stream));
}

}  // extern "C"
