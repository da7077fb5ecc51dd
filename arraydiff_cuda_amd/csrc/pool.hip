// Pooling over the halo-padded slab (max / average, forward and backward): HBM-bound kernels.
//
// forward : one thread per output element, lanes along the output row; the wh x ww window reads
//           overlap between neighbouring lanes and rows and are served by the caches, so HBM sees
//           the padded tile once.
// backward: one thread per element of the padded tile (a gather, no atomics): it visits the at
//           most ceil(wh/sh) x ceil(ww/sw) windows that contain it.  For MAX it takes a window's
//           gradient if it is that window's first maximum in row-major order: its value equals the
//           stored maximum and no earlier element of the window does.
#include "adh_common.h"

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
};

__device__ __forceinline__ float ld_f(const float *p, size_t i) { return p[i]; }
__device__ __forceinline__ float ld_f(const uint16_t *p, size_t i) { return bf16_bits_to_f32(p[i]); }
__device__ __forceinline__ void st_f(float *p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void st_f(uint16_t *p, size_t i, float v) { p[i] = f32_to_bf16_bits(v); }

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

}  // extern "C"
