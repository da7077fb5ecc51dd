// Pooling over the halo-padded slab (max / average, forward and backward): HBM-bound kernels.
//
// Banded kernels (the normal route): a block owns a band of rows of one plane.  The band of the
// padded tile is a contiguous byte range, so it is staged into LDS with 16-byte loads whatever the
// window and stride are, and the strided window reads then hit LDS instead of the vector caches.
//   forward : stage the input band, one output element per thread and step, coalesced stores.
//   backward: stage the input band and the band's dy rows; MAX first writes, per window, the
//             position of its first maximum in row-major order (one byte); then one thread per
//             element of the padded tile gathers the at most ceil(wh/sh) x ceil(ww/sw) windows
//             that contain it in a fixed order (no atomics: results are reproducible) and stores
//             dx coalesced.  y is not read: the maximum is recomputed from the staged input.
// Direct kernels (rows too wide for LDS, windows of more than 256 elements): one thread per
//   output (forward) or per padded element (backward), window reads served by the caches.
// Tiles without halo (the UNP instances of the banded kernels): the tiles are the row tiles of one tensor in rank
//   order; a block stages its band of the PADDED tile into LDS element by element, reading rows outside the
//   tile from the neighbouring tiles and zeros outside the tensor, and then works as over a padded tile.
//   Backward also takes the windows of the tiles above and below that reach into this tile (the padded plane
//   is continued upward by `up` window rows and downward as far as needed, so that they are the windows
//   0 .. up - 1 and up + OH .. of one row numbering) and stores interior pixels only: the gradient tile comes
//   out complete, as after a halo reduce and an unpad.
#include "adh_common.h"

#include <algorithm>

namespace adh {

struct PoolParams {
  const void *x[ADH_MAX_TILES];
  const void *y[ADH_MAX_TILES];
  const void *dy[ADH_MAX_TILES];
  void *out[ADH_MAX_TILES];  // y (forward) or dx_pad (backward)
  uint32_t planes;           // N * C per tile
  uint32_t HP, WP, OH, OW, wh, ww, sh, sw;
  float beta, inv_area;
  FastDiv div_sh, div_sw;
  // banded kernels
  uint32_t bands, band_rows;  // bands per plane; output rows (forward) / window rows (backward) per band
  FastDiv div_bands, div_OW, div_WP;
  // tiles without halo: the tile is H x W and WP = W + 2 pad_w; pad_top rows lie above the tile's first row in
  // the launch's row numbering (forward: pad_h, HP = H + 2 pad_h; backward: pad_h + up * sh, HP = pad_top + H +
  // pad_h); up / extra = windows of the tile above / below that reach into this tile's rows (backward)
  uint32_t H, W, pad_h, pad_w, pad_top, num_tiles, up, extra;
  // rows of W (x, dx) and OW (dy) elements are copied as 16-byte vectors when their width is a multiple of the
  // vector and the tiles are 16-byte aligned; x_items / dy_items = vectors (or elements) per row
  uint32_t x_vec, dy_vec, x_items, dy_items;
  FastDiv div_x_items, div_dy_items, div_side;
};

__device__ __forceinline__ float ld_f(const float *p, size_t i) { return p[i]; }
__device__ __forceinline__ float ld_f(const uint16_t *p, size_t i) { return bf16_bits_to_f32(p[i]); }
__device__ __forceinline__ void st_f(float *p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void st_f(uint16_t *p, size_t i, float v) { p[i] = f32_to_bf16_bits(v); }

constexpr uint32_t kPoolThreads = 256;
constexpr uint32_t kPoolBandBytes = 24u * 1024u;  // LDS aimed at per block (the backward pass: bwd_band_aim)
constexpr uint32_t kPoolMaxLds = 64u * 1024u;

// Copies nrows rows of `items` vectors (vec: 16 bytes each) or elements into LDS rows of `pitch` elements, from
// column col0 on.  src(row) is the row's first element in memory, or nullptr for a row of zeros; `any` is an
// address that can always be read (a row of zeros loads from there and drops what it loaded: no branch around
// the loads, so that several are in flight).
template <typename T, typename F>
__device__ __forceinline__ void stage_rows(T *lds, uint32_t pitch, uint32_t col0, uint32_t nrows, uint32_t items,
                                           const FastDiv &div_items, bool vec, const T *any, F src) {
  constexpr uint32_t VE = 16u / sizeof(T);
  const uint32_t n = nrows * items;
  if (vec) {
#pragma unroll 4
    for (uint32_t e = threadIdx.x; e < n; e += 256u) {
      uint32_t row, it;
      div_items.divmod(e, row, it);
      const T *sp = src(row);
      const bool have = sp != nullptr;
      uint4 v = reinterpret_cast<const uint4 *>(have ? sp : any)[have ? it : 0u];
      if (!have) v = make_uint4(0u, 0u, 0u, 0u);
      T *d = lds + row * pitch + col0 + it * VE;
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
      if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int k = 0; k < 4; ++k) reinterpret_cast<uint32_t *>(d)[k] = w[k];
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          d[2 * k] = (T)(w[k] & 0xffffu);
          d[2 * k + 1] = (T)(w[k] >> 16);
        }
      }
    }
  } else {
#pragma unroll 4
    for (uint32_t e = threadIdx.x; e < n; e += 256u) {
      uint32_t row, it;
      div_items.divmod(e, row, it);
      const T *sp = src(row);
      const bool have = sp != nullptr;
      const T v = (have ? sp : any)[have ? it : 0u];
      lds[row * pitch + col0 + it] = have ? v : (T)0;
    }
  }
}
// rows [v0, v0 + nrows) of tile `tile`'s padded plane into LDS (row pitch WP), read through the row tiles that
// carry no halo: rows outside the tile from the neighbouring tiles, zeros outside the tensor
template <typename T>
__device__ __forceinline__ void stage_virtual(T *lds, const PoolParams &P, uint32_t tile, uint32_t plane, uint32_t v0, uint32_t nrows) {
  // the three planes a row can come from (chosen per row by selects: an index into the table of tiles that
  // differs between lanes would be looked up one lane group at a time)
  const size_t plane_off = (size_t)plane * P.H * P.W;
  const T *own = reinterpret_cast<const T *>(P.x[tile]) + plane_off;
  const T *above = tile > 0u ? reinterpret_cast<const T *>(P.x[tile - 1u]) + plane_off : nullptr;
  const T *below = tile + 1u < P.num_tiles ? reinterpret_cast<const T *>(P.x[tile + 1u]) + plane_off : nullptr;
  stage_rows(lds, P.WP, P.pad_w, nrows, P.x_items, P.div_x_items, P.x_vec != 0u, own, [&](uint32_t row) -> const T * {
    int32_t r = (int32_t)(v0 + row) - (int32_t)P.pad_top;
    const T *from = own;
    if (r < 0) {
      r += (int32_t)P.H;
      from = r >= 0 ? above : nullptr;
    } else if (r >= (int32_t)P.H) {
      r -= (int32_t)P.H;
      from = r < (int32_t)P.H ? below : nullptr;
    }
    return from ? from + (size_t)(uint32_t)r * P.W : nullptr;
  });
  // the zero columns left and right of every row
  const uint32_t side = P.WP - P.W;
  for (uint32_t e = threadIdx.x; e < nrows * side; e += 256u) {
    uint32_t row, k;
    P.div_side.divmod(e, row, k);
    lds[row * P.WP + (k < P.pad_w ? k : P.W + k)] = (T)0;
  }
}

// Copies n elements from src into LDS with 16-byte loads; lds is 16-byte aligned and has room for
// n + 16 / sizeof(T) elements.  Returns the LDS address of element 0: it is shifted by the source's
// misalignment so that aligned global vectors land on aligned LDS vectors.
template <typename T>
__device__ __forceinline__ T *stage_contiguous(T *lds, const T *__restrict__ src, uint32_t n) {
  constexpr uint32_t VE = 16u / sizeof(T);
  const uint32_t tid = threadIdx.x;
  const uint32_t pad = (uint32_t)(reinterpret_cast<uintptr_t>(src) & 15u) / (uint32_t)sizeof(T);
  T *dst = lds + pad;
  const uint32_t head = min(n, (VE - pad) & (VE - 1u));
  const uint32_t nvec = (n - head) / VE;
  const uint32_t tail0 = head + nvec * VE;
  if (tid < head) dst[tid] = src[tid];
  const uint4 *gv = reinterpret_cast<const uint4 *>(src + head);
  uint4 *lv = reinterpret_cast<uint4 *>(dst + head);
#pragma unroll 4
  for (uint32_t v = tid; v < nvec; v += kPoolThreads) lv[v] = gv[v];
  if (tid < n - tail0) dst[tail0 + tid] = src[tail0 + tid];
  return dst;
}

__device__ __forceinline__ void vec_to_f32(const uint4 &v, float (&f)[4], const float *) {
  f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
}
__device__ __forceinline__ void vec_to_f32(const uint4 &v, float (&f)[8], const uint16_t *) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ uint4 f32_to_vec(const float (&f)[4], const float *) {
  return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3]));
}
__device__ __forceinline__ uint4 f32_to_vec(const float (&f)[8], const uint16_t *) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f32_to_bf16_bits(f[2 * i]) | ((uint32_t)f32_to_bf16_bits(f[2 * i + 1]) << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// dst[i] = src[i] (+ dst[i] when accumulate) for n elements with 16-byte stores; src is fp32 in LDS
// and src - (dst's misalignment in elements) is 16-byte aligned.
template <typename T>
__device__ __forceinline__ void unstage_contiguous(T *__restrict__ dst, const float *src, uint32_t n, bool accumulate) {
  constexpr uint32_t VE = 16u / sizeof(T);
  const uint32_t tid = threadIdx.x;
  const uint32_t pad = (uint32_t)(reinterpret_cast<uintptr_t>(dst) & 15u) / (uint32_t)sizeof(T);
  const uint32_t head = min(n, (VE - pad) & (VE - 1u));
  const uint32_t nvec = (n - head) / VE;
  const uint32_t tail0 = head + nvec * VE;
  if (tid < head) st_f(dst, tid, src[tid] + (accumulate ? ld_f(dst, tid) : 0.f));
  uint4 *gv = reinterpret_cast<uint4 *>(dst + head);
  const float4 *lv = reinterpret_cast<const float4 *>(src + head);
#pragma unroll 2
  for (uint32_t v = tid; v < nvec; v += kPoolThreads) {
    float f[VE];
#pragma unroll
    for (uint32_t q = 0; q < VE / 4u; ++q) {
      const float4 t = lv[v * (VE / 4u) + q];
      f[4 * q] = t.x; f[4 * q + 1] = t.y; f[4 * q + 2] = t.z; f[4 * q + 3] = t.w;
    }
    if (accumulate) {
      float o[VE];
      vec_to_f32(gv[v], o, (const T *)nullptr);
#pragma unroll
      for (uint32_t q = 0; q < VE; ++q) f[q] += o[q];
    }
    gv[v] = f32_to_vec(f, (const T *)nullptr);
  }
  if (tid < n - tail0) st_f(dst, tail0 + tid, src[tail0 + tid] + (accumulate ? ld_f(dst, tail0 + tid) : 0.f));
}

template <int WH, int WW, bool MAX, typename T>
__device__ __forceinline__ float window_reduce(const T *x, uint32_t base, uint32_t WP, uint32_t wh, uint32_t ww) {
  float acc = MAX ? -__builtin_inff() : 0.f;
  if (WH > 0) {
#pragma unroll
    for (int a = 0; a < WH; ++a)
#pragma unroll
      for (int b = 0; b < WW; ++b) {
        const float v = ld_f(x, base + a * WP + b);
        if (MAX) acc = v > acc ? v : acc;
        else acc += v;
      }
  } else {
    for (uint32_t a = 0; a < wh; ++a)
      for (uint32_t b = 0; b < ww; ++b) {
        const float v = ld_f(x, base + a * WP + b);
        if (MAX) acc = v > acc ? v : acc;
        else acc += v;
      }
  }
  return acc;
}

// grid: planes * tiles * bands; block 256.  Band b: output rows [b * band_rows, ...), input rows
// [b * band_rows * sh, last * sh + wh).
template <typename T, bool MAX, int WH, int WW, bool UNP = false>
__global__ __launch_bounds__(kPoolThreads) void pool_fwd_band_kernel(const PoolParams P) {
  extern __shared__ __align__(16) unsigned char pool_lds[];
  uint32_t pb, band;
  P.div_bands.divmod(blockIdx.x, pb, band);
  const uint32_t tile = pb / P.planes, plane = pb - tile * P.planes;
  const uint32_t oh0 = band * P.band_rows, rows = min(P.band_rows, P.OH - oh0);
  const uint32_t in_rows = (rows - 1u) * P.sh + P.wh;
  T *y = reinterpret_cast<T *>(P.out[tile]) + (size_t)plane * P.OH * P.OW + (size_t)oh0 * P.OW;
  const T *xl;
  if constexpr (UNP) {
    stage_virtual(reinterpret_cast<T *>(pool_lds), P, tile, plane, oh0 * P.sh, in_rows);
    xl = reinterpret_cast<const T *>(pool_lds);
  } else {
    const T *x = reinterpret_cast<const T *>(P.x[tile]) + (size_t)plane * P.HP * P.WP + (size_t)oh0 * P.sh * P.WP;
    xl = stage_contiguous(reinterpret_cast<T *>(pool_lds), x, in_rows * P.WP);
  }
  __syncthreads();
  const uint32_t n_out = rows * P.OW;
  for (uint32_t o = threadIdx.x; o < n_out; o += kPoolThreads) {
    uint32_t oh, ow;
    P.div_OW.divmod(o, oh, ow);
    const float acc = window_reduce<WH, WW, MAX>(xl, oh * P.sh * P.WP + ow * P.sw, P.WP, P.wh, P.ww);
    st_f(y, o, MAX ? acc : acc * P.inv_area);
  }
}

// grid: planes * tiles * bands; block 256.  Band b owns the padded rows [b * band_rows * sh,
// (b + 1) * band_rows * sh) (the last band: up to HP) and stages every window row that touches them.
// WH, WW, S > 0: window and stride (both directions) known at compile time, 0: read from P.
template <typename T, bool MAX, int WH, int WW, int S, bool UNP = false>
__global__ __launch_bounds__(kPoolThreads) void pool_bwd_band_kernel(const PoolParams PP) {
  extern __shared__ __align__(16) unsigned char pool_lds[];
  constexpr uint32_t VE = 16u / sizeof(T);
  struct Shape {
    const PoolParams &p;
    __device__ __forceinline__ uint32_t wh() const { return WH > 0 ? (uint32_t)WH : p.wh; }
    __device__ __forceinline__ uint32_t ww() const { return WW > 0 ? (uint32_t)WW : p.ww; }
    __device__ __forceinline__ uint32_t sh() const { return S > 0 ? (uint32_t)S : p.sh; }
    __device__ __forceinline__ uint32_t sw() const { return S > 0 ? (uint32_t)S : p.sw; }
    __device__ __forceinline__ uint32_t div_sh(uint32_t n) const { return S > 0 ? n / (uint32_t)S : p.div_sh.div(n); }
    __device__ __forceinline__ uint32_t div_sw(uint32_t n) const { return S > 0 ? n / (uint32_t)S : p.div_sw.div(n); }
  };
  const Shape Q{PP};
  const PoolParams &P = PP;
  uint32_t pb, band;
  P.div_bands.divmod(blockIdx.x, pb, band);
  const uint32_t tile = pb / P.planes, plane = pb - tile * P.planes;
  const uint32_t r0 = band * P.band_rows * Q.sh();
  const uint32_t r1 = band + 1u == P.bands ? P.HP : r0 + P.band_rows * Q.sh();
  // window rows that touch [r0, r1)
  // tiles without halo: window rows 0 .. up - 1 are the last windows of the tile above (none for the first
  // tile), up .. up + OH - 1 this tile's, the next `extra` the first windows of the tile below
  const uint32_t up = UNP ? P.up : 0u;
  const uint32_t w_first = UNP && tile == 0u ? up : 0u;
  const uint32_t OHv = up + P.OH + (UNP && tile + 1u < P.num_tiles ? P.extra : 0u);
  const uint32_t wr_lo = max(r0 + 1u > Q.wh() ? Q.div_sh(r0 + Q.sh() - Q.wh()) : 0u, w_first);
  const uint32_t wr_hi = min(Q.div_sh(r1 - 1u), OHv - 1u);
  if (UNP && wr_hi < wr_lo) return;  // (uniform) a band of the first tile that only the absent tile above would touch
  const uint32_t wrows = wr_hi + 1u - wr_lo;  // >= 1: r0 <= (OH - 1) * sh by the choice of bands
  const uint32_t n_win = wrows * P.OW;
  const uint32_t x_row0 = wr_lo * Q.sh(), x_rows = (wrows - 1u) * Q.sh() + Q.wh();
  // padded: the tile's padded gradient plane; tiles without halo: the H x W plane
  T *dx = reinterpret_cast<T *>(P.out[tile]) + (size_t)plane * (UNP ? P.H * P.W : P.HP * P.WP);
  // LDS: dy rows | input rows | first-maximum positions
  T *lds_dy = reinterpret_cast<T *>(pool_lds);
  const uint32_t dy_room = (n_win + VE + VE - 1u) & ~(VE - 1u);
  const T *dyl;
  if constexpr (UNP) {
    const size_t dy_plane_off = (size_t)plane * P.OH * P.OW;
    const T *own_dy = reinterpret_cast<const T *>(P.dy[tile]) + dy_plane_off;
    const T *dy_above = tile > 0u ? reinterpret_cast<const T *>(P.dy[tile - 1u]) + dy_plane_off : own_dy;
    const T *dy_below = tile + 1u < P.num_tiles ? reinterpret_cast<const T *>(P.dy[tile + 1u]) + dy_plane_off : own_dy;
    stage_rows(lds_dy, P.OW, 0u, wrows, P.dy_items, P.div_dy_items, P.dy_vec != 0u, own_dy, [&](uint32_t wr) -> const T * {
      const uint32_t row = wr_lo + wr;
      const T *from = own_dy;
      uint32_t drow = row - up;
      if (row < up) {
        from = dy_above;
        drow = P.OH - up + row;
      } else if (row >= up + P.OH) {
        from = dy_below;
        drow = row - up - P.OH;
      }
      return from + (size_t)drow * P.OW;
    });
    dyl = lds_dy;
  } else {
    const T *dy = reinterpret_cast<const T *>(P.dy[tile]) + (size_t)plane * P.OH * P.OW + (size_t)wr_lo * P.OW;
    dyl = stage_contiguous(lds_dy, dy, n_win);
  }
  // stores the owned rows' gradient g (LDS, fp32, padded pitch): all of it into the padded plane, or the
  // interior pixels into the plane without halo
  auto store_unpadded = [&](const float *g, uint32_t n_own) {
    // the owned rows that are the tile's own: rows [i0, i1) of the H x W plane
    const uint32_t i0 = r0 > P.pad_top ? r0 - P.pad_top : 0u;
    const uint32_t i1 = min(P.H, r1 > P.pad_top ? r1 - P.pad_top : 0u);
    if (i1 <= i0) return;
    const uint32_t n = (i1 - i0) * P.x_items;
    (void)n_own;
#pragma unroll 2
    for (uint32_t e = threadIdx.x; e < n; e += kPoolThreads) {
      uint32_t rb, it;
      P.div_x_items.divmod(e, rb, it);
      const uint32_t r = i0 + rb;
      const float *gs = g + (r + P.pad_top - r0) * P.WP + P.pad_w;
      T *drow = dx + (size_t)r * P.W;
      if (P.x_vec) {
        float f[VE];
#pragma unroll
        for (uint32_t k = 0; k < VE; ++k) f[k] = gs[it * VE + k];
        uint4 *dv = reinterpret_cast<uint4 *>(drow) + it;
        if (P.beta != 0.f) {
          float o[VE];
          vec_to_f32(*dv, o, (const T *)nullptr);
#pragma unroll
          for (uint32_t k = 0; k < VE; ++k) f[k] += o[k];
        }
        *dv = f32_to_vec(f, (const T *)nullptr);
      } else {
        st_f(drow, it, gs[it] + (P.beta != 0.f ? ld_f(drow, it) : 0.f));
      }
    }
  };
  if (MAX) {
    T *lds_x = lds_dy + dy_room;
    const uint32_t x_room = (x_rows * P.WP + VE + VE - 1u) & ~(VE - 1u);
    const T *xl;
    if constexpr (UNP) {
      stage_virtual(lds_x, P, tile, plane, x_row0, x_rows);
      xl = lds_x;
    } else {
      const T *x = reinterpret_cast<const T *>(P.x[tile]) + (size_t)plane * P.HP * P.WP + (size_t)x_row0 * P.WP;
      xl = stage_contiguous(lds_x, x, x_rows * P.WP);
    }
    // fp32 gradient of the owned rows, shifted like dx so that 16-byte stores line up
    const uint32_t n_own = (r1 - r0) * P.WP;
    T *dxo = dx + (size_t)r0 * P.WP;
    float *gl_base = reinterpret_cast<float *>(lds_x + x_room);
    const uint32_t gpad = UNP ? 0u : (uint32_t)(reinterpret_cast<uintptr_t>(dxo) & 15u) / (uint32_t)sizeof(T);
    float *gl = gl_base + gpad;
    for (uint32_t v = threadIdx.x; v < (gpad + n_own + 3u) / 4u; v += kPoolThreads)
      reinterpret_cast<float4 *>(gl_base)[v] = make_float4(0.f, 0.f, 0.f, 0.f);
    __syncthreads();
    // Windows whose row and column indices agree modulo ceil(wh / sh) and ceil(ww / sw) are disjoint:
    // one class at a time, every window adds its dy onto its first maximum without atomics, and an
    // element's terms are added in class order whatever the banding is.
    const uint32_t ch = (Q.wh() + Q.sh() - 1u) / Q.sh(), cw = (Q.ww() + Q.sw() - 1u) / Q.sw();
    const int32_t g_shift = ((int32_t)x_row0 - (int32_t)r0) * (int32_t)P.WP;
    for (uint32_t ca = 0; ca < ch; ++ca)
      for (uint32_t cb = 0; cb < cw; ++cb) {
        const uint32_t first_oh = wr_lo + (ca + ch - wr_lo % ch) % ch;
        const uint32_t nrow_c = first_oh <= wr_hi ? (wr_hi - first_oh) / ch + 1u : 0u;
        const uint32_t ncol_c = cb < P.OW ? (P.OW - 1u - cb) / cw + 1u : 0u;
        for (uint32_t t = threadIdx.x; t < nrow_c * ncol_c; t += kPoolThreads) {
          const uint32_t wi = t / ncol_c, wj = t - wi * ncol_c;
          const uint32_t ohl = first_oh - wr_lo + wi * ch, ow = cb + wj * cw;
          const uint32_t base = ohl * Q.sh() * P.WP + ow * Q.sw();
          float best = -__builtin_inff();
          uint32_t at = base;
          if (WH > 0) {
#pragma unroll
            for (int a = 0; a < WH; ++a)
#pragma unroll
              for (int b = 0; b < WW; ++b) {
                const float v = ld_f(xl, base + a * P.WP + b);
                if (v > best) { best = v; at = base + a * P.WP + b; }
              }
          } else {
            for (uint32_t a = 0; a < Q.wh(); ++a)
              for (uint32_t b = 0; b < Q.ww(); ++b) {
                const float v = ld_f(xl, base + a * P.WP + b);
                if (v > best) { best = v; at = base + a * P.WP + b; }
              }
          }
          const uint32_t gi = (uint32_t)((int32_t)at + g_shift);
          if (gi < n_own) gl[gi] += ld_f(dyl, ohl * P.OW + ow);
        }
        __syncthreads();
      }
    if constexpr (UNP) store_unpadded(gl, n_own);
    else unstage_contiguous(dxo, gl, n_own, P.beta != 0.f);
  } else {
    __syncthreads();
    const uint32_t n_own = (r1 - r0) * P.WP;
    for (uint32_t j = threadIdx.x; j < n_own; j += kPoolThreads) {
      uint32_t ihb, iw;
      P.div_WP.divmod(j, ihb, iw);
      const uint32_t ih = r0 + ihb;
      if constexpr (UNP) {  // interior pixels only
        if (ih < P.pad_top || ih >= P.pad_top + P.H || iw < P.pad_w || iw >= P.pad_w + P.W) continue;
      }
      const uint32_t oh_hi = min(Q.div_sh(ih), OHv - 1u);
      const uint32_t oh_lo = max(ih + 1u > Q.wh() ? Q.div_sh(ih + Q.sh() - Q.wh()) : 0u, w_first);
      const uint32_t ow_hi = min(Q.div_sw(iw), P.OW - 1u);
      const uint32_t ow_lo = iw + 1u > Q.ww() ? Q.div_sw(iw + Q.sw() - Q.ww()) : 0u;
      float g = 0.f;
      for (uint32_t oh = oh_lo; oh <= oh_hi; ++oh)
        for (uint32_t ow = ow_lo; ow <= ow_hi; ++ow) g += ld_f(dyl, (oh - wr_lo) * P.OW + ow);
      g *= P.inv_area;
      const size_t i = UNP ? (size_t)(ih - P.pad_top) * P.W + (iw - P.pad_w) : (size_t)r0 * P.WP + j;
      if (P.beta != 0.f) g += ld_f(dx, i);
      st_f(dx, i, g);
    }
  }
}

// grid: (planes * tiles, ceil(OH / 4), ceil(OW / 64)); block 64 x 4 (4 output rows share a block)
template <typename T, bool MAX>
__global__ __launch_bounds__(256) void pool_fwd_kernel(const PoolParams P) {
  const uint32_t ow = blockIdx.z * 64u + threadIdx.x;
  const uint32_t oh = blockIdx.y * 4u + threadIdx.y;
  const uint32_t tile = blockIdx.x / P.planes, plane = blockIdx.x - tile * P.planes;
  if (ow >= P.OW || oh >= P.OH) return;
  const T *x = reinterpret_cast<const T *>(P.x[tile]) + (size_t)plane * P.HP * P.WP;
  T *y = reinterpret_cast<T *>(P.out[tile]) + (size_t)plane * P.OH * P.OW;
  const size_t base = (size_t)(oh * P.sh) * P.WP + ow * P.sw;
  float acc = MAX ? -__builtin_inff() : 0.f;
  for (uint32_t a = 0; a < P.wh; ++a)
    for (uint32_t b = 0; b < P.ww; ++b) {
      const float v = ld_f(x, base + (size_t)a * P.WP + b);
      if (MAX) acc = v > acc ? v : acc;
      else acc += v;
    }
  st_f(y, (size_t)oh * P.OW + ow, MAX ? acc : acc * P.inv_area);
}

// grid: (planes * tiles, ceil(HP / 4), ceil(WP / 64))
template <typename T, bool MAX>
__global__ __launch_bounds__(256) void pool_bwd_kernel(const PoolParams P) {
  const uint32_t iw = blockIdx.z * 64u + threadIdx.x;
  const uint32_t ih = blockIdx.y * 4u + threadIdx.y;
  const uint32_t tile = blockIdx.x / P.planes, plane = blockIdx.x - tile * P.planes;
  if (iw >= P.WP || ih >= P.HP) return;
  const T *x = reinterpret_cast<const T *>(P.x[tile]) + (size_t)plane * P.HP * P.WP;
  const T *y = reinterpret_cast<const T *>(P.y[tile]) + (size_t)plane * P.OH * P.OW;
  const T *dy = reinterpret_cast<const T *>(P.dy[tile]) + (size_t)plane * P.OH * P.OW;
  T *dx = reinterpret_cast<T *>(P.out[tile]) + (size_t)plane * P.HP * P.WP;
  // windows oh with oh*sh <= ih <= oh*sh + wh - 1
  const uint32_t oh_hi = min(P.div_sh.div(ih), P.OH - 1u);
  const uint32_t oh_lo = ih + 1u > P.wh ? P.div_sh.div(ih + P.sh - P.wh) : 0u;  // ceil((ih - wh + 1) / sh)
  const uint32_t ow_hi = min(P.div_sw.div(iw), P.OW - 1u);
  const uint32_t ow_lo = iw + 1u > P.ww ? P.div_sw.div(iw + P.sw - P.ww) : 0u;
  const float xv = MAX ? ld_f(x, (size_t)ih * P.WP + iw) : 0.f;
  float g = 0.f;
  for (uint32_t oh = oh_lo; oh <= oh_hi; ++oh)
    for (uint32_t ow = ow_lo; ow <= ow_hi; ++ow) {
      const size_t o = (size_t)oh * P.OW + ow;
      if (!MAX) {
        g += ld_f(dy, o);
      } else if (xv == ld_f(y, o)) {
        // first maximum of the window?
        const uint32_t a0 = ih - oh * P.sh, b0 = iw - ow * P.sw;
        const size_t base = (size_t)(oh * P.sh) * P.WP + ow * P.sw;
        bool first = true;
        for (uint32_t a = 0; a <= a0 && first; ++a) {
          const uint32_t bend = a < a0 ? P.ww : b0;
          for (uint32_t b = 0; b < bend; ++b)
            if (ld_f(x, base + (size_t)a * P.WP + b) == xv) { first = false; break; }
        }
        if (first) g += ld_f(dy, o);
      }
    }
  if (!MAX) g *= P.inv_area;
  const size_t i = (size_t)ih * P.WP + iw;
  if (P.beta != 0.f) g += ld_f(dx, i);
  st_f(dx, i, g);
}

static int pool_check(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t HP, uint32_t WP,
                      uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw, PoolParams *P) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if (mode != ADH_POOL_AVG && mode != ADH_POOL_MAX) return ADH_EINVAL;
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if (wh == 0 || ww == 0 || sh == 0 || sw == 0 || wh > HP || ww > WP) return ADH_EINVAL;
  if ((uint64_t)HP * WP >= (1ull << 31) || (uint64_t)N * C * num_tiles > 0x7fffffffull) return ADH_EINVAL;
  P->planes = N * C;
  P->HP = HP; P->WP = WP; P->wh = wh; P->ww = ww; P->sh = sh; P->sw = sw;
  P->OH = (HP - wh) / sh + 1u;
  P->OW = (WP - ww) / sw + 1u;
  P->inv_area = 1.0f / (float)(wh * ww);
  P->div_sh = FastDiv(sh);
  P->div_sw = FastDiv(sw);
  return ADH_OK;
}

template <bool MAX>
static void launch_fwd(int dtype, const PoolParams &P, dim3 grid, hipStream_t st) {
  if (dtype == ADH_F32) hipLaunchKernelGGL((pool_fwd_kernel<float, MAX>), grid, dim3(64, 4), 0, st, P);
  else hipLaunchKernelGGL((pool_fwd_kernel<uint16_t, MAX>), grid, dim3(64, 4), 0, st, P);
}
template <bool MAX>
static void launch_bwd(int dtype, const PoolParams &P, dim3 grid, hipStream_t st) {
  if (dtype == ADH_F32) hipLaunchKernelGGL((pool_bwd_kernel<float, MAX>), grid, dim3(64, 4), 0, st, P);
  else hipLaunchKernelGGL((pool_bwd_kernel<uint16_t, MAX>), grid, dim3(64, 4), 0, st, P);
}

// ---- banded route: band size, LDS bytes, launches ----

static size_t fwd_band_lds(const PoolParams &P, size_t es, uint32_t rows) {
  return ((size_t)((rows - 1u) * P.sh + P.wh) * P.WP * es + 16u + 15u) & ~(size_t)15u;
}
static size_t bwd_band_lds(const PoolParams &P, size_t es, bool max, uint32_t rows) {
  const uint64_t wrows = std::min<uint64_t>(P.OH + P.up + P.extra, (uint64_t)rows + (P.wh - 1u) / P.sh + P.extra);
  const uint64_t n_win = wrows * P.OW;
  size_t b = ((n_win * es + 16u + 15u) & ~(size_t)15u);
  if (max) {
    const uint64_t own_rows = std::min<uint64_t>(P.HP, (uint64_t)rows * P.sh + P.wh);
    b += ((((wrows - 1u) * P.sh + P.wh) * P.WP * es + 16u + 15u) & ~(size_t)15u) + (own_rows * P.WP + 8u) * 4u;
  }
  return b;
}

// Picks the rows per band: as many as fit the LDS aimed at per block, fewer while the launch would
// have too few blocks to fill the chip.  Returns 0 when not even one row fits (direct route).
template <typename F>
static uint32_t pick_band_rows(const PoolParams &P, uint32_t num_tiles, size_t aim, F lds_bytes) {
  if (lds_bytes(1u) > kPoolMaxLds) return 0;
  uint32_t rows = 1;
  while (rows < P.OH && lds_bytes(rows + 1u) <= aim) ++rows;
  const uint64_t pt = (uint64_t)P.planes * num_tiles;
  while (rows > 1u && pt * ((P.OH + rows - 1u) / rows) < 2048u) rows = (rows + 1u) / 2u;
  if (pt * ((P.OH + rows - 1u) / rows) >= (1ull << 24)) return 0;
  return rows;
}

// The LDS a band of the backward pass aims at.  A plane that fits 48 KB whole is one band (no window row is staged
// twice: 4 tiles of 30 x 114, 0.052 ms against 0.064 in two bands); larger planes take bands of 24 KB, so that six
// workgroups per CU in different phases keep loads in flight (the max backward over 64 x 256 tiles: 0.46 ms with
// bands of 48 KB, 0.39 with 24 KB; 0.70 with 18 KB, whose bands stage too many window rows twice).
template <typename P_>
static size_t bwd_band_aim(const P_ &P, size_t es, bool is_max) {
  if (is_max && bwd_band_lds(P, es, is_max, P.OH + P.up) <= 2u * kPoolBandBytes) return 2u * kPoolBandBytes;
  return kPoolBandBytes;
}

static void set_bands(PoolParams *P, uint32_t rows) {
  P->band_rows = rows;
  P->bands = (P->OH + P->up + rows - 1u) / rows;  // (up: window rows of the tile above, backward over tiles without halo)
  P->div_bands = FastDiv(P->bands);
  P->div_OW = FastDiv(P->OW);
  P->div_WP = FastDiv(P->WP);
}

template <typename T, bool MAX, bool UNP>
static void launch_fwd_band_t(const PoolParams &P, uint32_t blocks, size_t lds, hipStream_t st) {
  if (P.wh == 3 && P.ww == 3)
    hipLaunchKernelGGL((pool_fwd_band_kernel<T, MAX, 3, 3, UNP>), dim3(blocks), dim3(kPoolThreads), lds, st, P);
  else if (P.wh == 2 && P.ww == 2)
    hipLaunchKernelGGL((pool_fwd_band_kernel<T, MAX, 2, 2, UNP>), dim3(blocks), dim3(kPoolThreads), lds, st, P);
  else
    hipLaunchKernelGGL((pool_fwd_band_kernel<T, MAX, 0, 0, UNP>), dim3(blocks), dim3(kPoolThreads), lds, st, P);
}
template <typename T, bool MAX, bool UNP>
static void launch_bwd_band_t(const PoolParams &P, uint32_t blocks, size_t lds, hipStream_t st) {
  const bool s2 = P.sh == 2 && P.sw == 2;
  if (P.wh == 3 && P.ww == 3 && s2)
    hipLaunchKernelGGL((pool_bwd_band_kernel<T, MAX, 3, 3, 2, UNP>), dim3(blocks), dim3(kPoolThreads), lds, st, P);
  else if (P.wh == 2 && P.ww == 2 && s2)
    hipLaunchKernelGGL((pool_bwd_band_kernel<T, MAX, 2, 2, 2, UNP>), dim3(blocks), dim3(kPoolThreads), lds, st, P);
  else
    hipLaunchKernelGGL((pool_bwd_band_kernel<T, MAX, 0, 0, 0, UNP>), dim3(blocks), dim3(kPoolThreads), lds, st, P);
}
template <bool UNP>
static void launch_fwd_band_u(int dtype, bool max, const PoolParams &P, uint32_t blocks, size_t lds, hipStream_t st) {
  if (dtype == ADH_F32) max ? launch_fwd_band_t<float, true, UNP>(P, blocks, lds, st) : launch_fwd_band_t<float, false, UNP>(P, blocks, lds, st);
  else max ? launch_fwd_band_t<uint16_t, true, UNP>(P, blocks, lds, st) : launch_fwd_band_t<uint16_t, false, UNP>(P, blocks, lds, st);
}
template <bool UNP>
static void launch_bwd_band_u(int dtype, bool max, const PoolParams &P, uint32_t blocks, size_t lds, hipStream_t st) {
  if (dtype == ADH_F32) max ? launch_bwd_band_t<float, true, UNP>(P, blocks, lds, st) : launch_bwd_band_t<float, false, UNP>(P, blocks, lds, st);
  else max ? launch_bwd_band_t<uint16_t, true, UNP>(P, blocks, lds, st) : launch_bwd_band_t<uint16_t, false, UNP>(P, blocks, lds, st);
}
static void launch_fwd_band(int dtype, bool max, const PoolParams &P, uint32_t blocks, size_t lds, hipStream_t st) {
  launch_fwd_band_u<false>(dtype, max, P, blocks, lds, st);
}
static void launch_bwd_band(int dtype, bool max, const PoolParams &P, uint32_t blocks, size_t lds, hipStream_t st) {
  launch_bwd_band_u<false>(dtype, max, P, blocks, lds, st);
}

// Tiles without halo: fills the padded extents and the split's fields; the same limits as the convolution over
// such tiles (H / sh output rows per tile must stitch, a window reaches the adjacent tiles only).
static int pool_check_unpadded(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                               uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw, uint32_t pad_h, uint32_t pad_w,
                               PoolParams *P) {
  if (H == 0 || W == 0 || sh == 0 || wh == 0 || pad_h > 4096u || pad_w > 4096u) return ADH_EINVAL;
  if (H % sh != 0u || 2u * pad_h >= wh || wh - 2u * pad_h > sh || pad_h > H || wh - 1u - pad_h > H) return ADH_EINVAL;
  // (backward) the windows of the tile above that reach into this tile must start inside that tile
  if (pad_h + (wh - 1u - pad_h) / sh * sh > H) return ADH_EINVAL;
  const int e = pool_check(dtype, mode, num_tiles, N, C, H + 2u * pad_h, W + 2u * pad_w, wh, ww, sh, sw, P);
  if (e) return e;
  P->H = H; P->W = W; P->pad_h = pad_h; P->pad_w = pad_w; P->pad_top = pad_h; P->num_tiles = num_tiles;
  P->div_side = FastDiv(std::max(1u, 2u * pad_w));
  return ADH_OK;
}
// rows as 16-byte vectors where widths and addresses allow
static void pool_unpadded_vectors(PoolParams *P, size_t es, uint32_t num_tiles, bool with_dy) {
  const uint32_t ve = (uint32_t)(16u / es);
  bool x_ok = P->W % ve == 0u, dy_ok = with_dy && P->OW % ve == 0u;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    x_ok = x_ok && (!P->x[t] || aligned_to(P->x[t], 16)) && (!with_dy || aligned_to(P->out[t], 16));
    dy_ok = dy_ok && aligned_to(P->dy[t], 16);
  }
  P->x_vec = x_ok ? 1u : 0u;
  P->dy_vec = dy_ok ? 1u : 0u;
  P->x_items = x_ok ? P->W / ve : P->W;
  P->dy_items = dy_ok ? P->OW / ve : P->OW;
  P->div_x_items = FastDiv(P->x_items);
  P->div_dy_items = FastDiv(std::max(1u, P->dy_items));
}
// the backward launch's row numbering: continued upward by the window rows of the tile above that reach this tile
static int pool_unpadded_bwd_rows(PoolParams *P) {
  P->extra = (P->pad_h + P->sh - 1u) / P->sh;     // windows j of the tile below with j * sh < pad_h
  P->up = (P->wh - 1u - P->pad_h) / P->sh;        // windows OH - j of the tile above with j * sh <= wh - 1 - pad_h
  P->pad_top = P->pad_h + P->up * P->sh;
  if (P->pad_top > P->H) return ADH_EINVAL;       // they start inside the tile above
  P->HP = P->pad_top + P->H + P->pad_h;
  return ADH_OK;
}

}  // namespace adh

using namespace adh;

extern "C" {

int adh_pool2d_slab_fwd_tiles(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t HP,
                              uint32_t WP, uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw,
                              const void *const *x_pad_tiles, void *const *y_tiles, void *stream) {
  PoolParams P = {};
  int e = pool_check(dtype, mode, num_tiles, N, C, HP, WP, wh, ww, sh, sw, &P);
  if (e) return e;
  if (N == 0 || C == 0) return ADH_OK;
  if (!x_pad_tiles || !y_tiles) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!x_pad_tiles[t] || !y_tiles[t]) return ADH_ENULL;
    if (!aligned_to(x_pad_tiles[t], es) || !aligned_to(y_tiles[t], es)) return ADH_EALIGN;
    P.x[t] = x_pad_tiles[t];
    P.out[t] = y_tiles[t];
  }
  const uint32_t band_rows = pick_band_rows(P, num_tiles, kPoolBandBytes, [&](uint32_t r) { return fwd_band_lds(P, es, r); });
  if (band_rows) {
    set_bands(&P, band_rows);
    launch_fwd_band(dtype, mode == ADH_POOL_MAX, P, P.planes * num_tiles * P.bands, fwd_band_lds(P, es, band_rows),
                    as_stream(stream));
    return launch_status();
  }
  const uint64_t gz = (uint64_t)P.planes * num_tiles;
  if (gz >= (1ull << 26) || (P.OH + 3u) / 4u > 65535u || (P.OW + 63u) / 64u > 65535u) return ADH_EINVAL;
  dim3 grid((uint32_t)gz, (P.OH + 3u) / 4u, (P.OW + 63u) / 64u);
  if (mode == ADH_POOL_MAX) launch_fwd<true>(dtype, P, grid, as_stream(stream));
  else launch_fwd<false>(dtype, P, grid, as_stream(stream));
  return launch_status();
}

int adh_pool2d_slab_fwd(int dtype, int mode, uint32_t N, uint32_t C, uint32_t HP, uint32_t WP, uint32_t wh,
                        uint32_t ww, uint32_t sh, uint32_t sw, const void *x_pad, void *y, void *stream) {
  const void *xs[1] = {x_pad};
  void *ys[1] = {y};
  return adh_pool2d_slab_fwd_tiles(dtype, mode, 1, N, C, HP, WP, wh, ww, sh, sw, xs, ys, stream);
}

int adh_pool2d_slab_bwd_tiles(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t HP,
                              uint32_t WP, uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw,
                              const void *const *x_pad_tiles, const void *const *y_tiles,
                              const void *const *dy_tiles, void *const *dx_pad_tiles, float beta, void *stream) {
  PoolParams P = {};
  int e = pool_check(dtype, mode, num_tiles, N, C, HP, WP, wh, ww, sh, sw, &P);
  if (e) return e;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (N == 0 || C == 0) return ADH_OK;
  if (!dy_tiles || !dx_pad_tiles) return ADH_ENULL;
  if (mode == ADH_POOL_MAX && (!x_pad_tiles || !y_tiles)) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!dy_tiles[t] || !dx_pad_tiles[t]) return ADH_ENULL;
    if (!aligned_to(dy_tiles[t], es) || !aligned_to(dx_pad_tiles[t], es)) return ADH_EALIGN;
    if (mode == ADH_POOL_MAX) {
      if (!x_pad_tiles[t] || !y_tiles[t]) return ADH_ENULL;
      if (!aligned_to(x_pad_tiles[t], es) || !aligned_to(y_tiles[t], es)) return ADH_EALIGN;
      P.x[t] = x_pad_tiles[t];
      P.y[t] = y_tiles[t];
    }
    P.dy[t] = dy_tiles[t];
    P.out[t] = dx_pad_tiles[t];
  }
  P.beta = beta;
  const bool is_max = mode == ADH_POOL_MAX;
  const uint32_t band_rows =
      wh * ww > 256u ? 0u : pick_band_rows(P, num_tiles, bwd_band_aim(P, es, is_max), [&](uint32_t r) { return bwd_band_lds(P, es, is_max, r); });
  if (band_rows) {
    set_bands(&P, band_rows);
    launch_bwd_band(dtype, is_max, P, P.planes * num_tiles * P.bands, bwd_band_lds(P, es, is_max, band_rows),
                    as_stream(stream));
    return launch_status();
  }
  const uint64_t gz = (uint64_t)P.planes * num_tiles;
  if (gz >= (1ull << 26) || (HP + 3u) / 4u > 65535u || (WP + 63u) / 64u > 65535u) return ADH_EINVAL;
  dim3 grid((uint32_t)gz, (HP + 3u) / 4u, (WP + 63u) / 64u);
  if (mode == ADH_POOL_MAX) launch_bwd<true>(dtype, P, grid, as_stream(stream));
  else launch_bwd<false>(dtype, P, grid, as_stream(stream));
  return launch_status();
}

int adh_pool2d_slab_bwd(int dtype, int mode, uint32_t N, uint32_t C, uint32_t HP, uint32_t WP, uint32_t wh,
                        uint32_t ww, uint32_t sh, uint32_t sw, const void *x_pad, const void *y, const void *dy,
                        void *dx_pad, float beta, void *stream) {
  const void *xs[1] = {x_pad};
  const void *ys[1] = {y};
  const void *dys[1] = {dy};
  void *dxs[1] = {dx_pad};
  return adh_pool2d_slab_bwd_tiles(dtype, mode, 1, N, C, HP, WP, wh, ww, sh, sw, xs, ys, dys, dxs, beta, stream);
}

int adh_pool2d_unpadded_supported(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                                  uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw, uint32_t pad_h, uint32_t pad_w) {
  PoolParams P = {};
  int e = pool_check_unpadded(dtype, mode, num_tiles, N, C, H, W, wh, ww, sh, sw, pad_h, pad_w, &P);
  if (e) return e;
  if (N == 0 || C == 0) return ADH_OK;
  const size_t es = dtype_size(dtype);
  const bool is_max = mode == ADH_POOL_MAX;
  if (!pick_band_rows(P, num_tiles, kPoolBandBytes, [&](uint32_t r) { return fwd_band_lds(P, es, r); })) return ADH_EUNIMPL;
  e = pool_unpadded_bwd_rows(&P);
  if (e) return e;
  if (wh * ww > 256u ||
      !pick_band_rows(P, num_tiles, bwd_band_aim(P, es, is_max), [&](uint32_t r) { return bwd_band_lds(P, es, is_max, r); }))
    return ADH_EUNIMPL;
  return ADH_OK;
}

int adh_pool2d_unpadded_fwd_tiles(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                                  uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw, uint32_t pad_h, uint32_t pad_w,
                                  const void *const *x_tiles, void *const *y_tiles, void *stream) {
  PoolParams P = {};
  int e = pool_check_unpadded(dtype, mode, num_tiles, N, C, H, W, wh, ww, sh, sw, pad_h, pad_w, &P);
  if (e) return e;
  if (N == 0 || C == 0) return ADH_OK;
  if (!x_tiles || !y_tiles) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!x_tiles[t] || !y_tiles[t]) return ADH_ENULL;
    if (!aligned_to(x_tiles[t], es) || !aligned_to(y_tiles[t], es)) return ADH_EALIGN;
    P.x[t] = x_tiles[t];
    P.out[t] = y_tiles[t];
  }
  pool_unpadded_vectors(&P, es, num_tiles, false);
  const uint32_t band_rows = pick_band_rows(P, num_tiles, kPoolBandBytes, [&](uint32_t r) { return fwd_band_lds(P, es, r); });
  if (!band_rows) return ADH_EUNIMPL;  // rows too wide for a band in LDS: use the padded entry points
  set_bands(&P, band_rows);
  launch_fwd_band_u<true>(dtype, mode == ADH_POOL_MAX, P, P.planes * num_tiles * P.bands, fwd_band_lds(P, es, band_rows),
                          as_stream(stream));
  return launch_status();
}

int adh_pool2d_unpadded_bwd_tiles(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                                  uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw, uint32_t pad_h, uint32_t pad_w,
                                  const void *const *x_tiles, const void *const *y_tiles, const void *const *dy_tiles,
                                  void *const *dx_tiles, float beta, void *stream) {
  PoolParams P = {};
  int e = pool_check_unpadded(dtype, mode, num_tiles, N, C, H, W, wh, ww, sh, sw, pad_h, pad_w, &P);
  if (e) return e;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (N == 0 || C == 0) return ADH_OK;
  if (!dy_tiles || !dx_tiles) return ADH_ENULL;
  const bool is_max = mode == ADH_POOL_MAX;
  if (is_max && !x_tiles) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!dy_tiles[t] || !dx_tiles[t]) return ADH_ENULL;
    if (!aligned_to(dy_tiles[t], es) || !aligned_to(dx_tiles[t], es)) return ADH_EALIGN;
    if (is_max) {
      if (!x_tiles[t]) return ADH_ENULL;
      if (!aligned_to(x_tiles[t], es)) return ADH_EALIGN;
      P.x[t] = x_tiles[t];
      P.y[t] = y_tiles ? y_tiles[t] : nullptr;  // not read: the maximum is recomputed from the staged input
    }
    P.dy[t] = dy_tiles[t];
    P.out[t] = dx_tiles[t];
  }
  P.beta = beta;
  e = pool_unpadded_bwd_rows(&P);
  if (e) return e;
  pool_unpadded_vectors(&P, es, num_tiles, true);
  const uint32_t band_rows =
      wh * ww > 256u ? 0u : pick_band_rows(P, num_tiles, bwd_band_aim(P, es, is_max), [&](uint32_t r) { return bwd_band_lds(P, es, is_max, r); });
  if (!band_rows) return ADH_EUNIMPL;
  set_bands(&P, band_rows);
  launch_bwd_band_u<true>(dtype, is_max, P, P.planes * num_tiles * P.bands, bwd_band_lds(P, es, is_max, band_rows),
                          as_stream(stream));
  return launch_status();
}

}  // extern "C"
