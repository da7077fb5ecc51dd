// bf16 entry of the 3x3 slab convolution: bf16 tensors in HBM, fp32 accumulation.
//
// Forward and backward-data run on the bf16 matrix-core kernels of conv3x3_bf16_mfma.hip, the filter
// gradient on that of conv3x3_bf16_wgrad.hip (at a width that is no multiple of 8 over copies of the
// tensors with wider rows, made here).  What those do not take (images or sums beyond the 2 GiB a
// buffer resource addresses) goes the route below: the bf16 slabs, filter and (for beta = 1) outputs
// are widened to fp32 in the caller's workspace, the fp32 MFMA kernels run on the copies, and the
// result is rounded back to bf16 (round to nearest even).  Every product is therefore exact and every sum is in
// fp32, i.e. the arithmetic of a bf16-input / fp32-accumulate matrix core, at the speed of the
// fp32 path plus three streaming passes.  The filter gradient stays fp32.
#include "adh_common.h"

namespace adh {

__global__ __launch_bounds__(256) void widen_bf16_kernel(uint64_t n, const uint16_t *__restrict__ src,
                                                        float *__restrict__ dst) {
  const uint64_t stride = (uint64_t)gridDim.x * 256u * 8u;
  for (uint64_t i = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * 8u; i < n; i += stride) {
    if (i + 8u <= n) {
      typedef uint4 U4 __attribute__((aligned(2)));
      const uint4 v = *reinterpret_cast<const U4 *>(src + i);
      float4 lo, hi;
      lo.x = __uint_as_float(v.x << 16); lo.y = __uint_as_float(v.x & 0xffff0000u);
      lo.z = __uint_as_float(v.y << 16); lo.w = __uint_as_float(v.y & 0xffff0000u);
      hi.x = __uint_as_float(v.z << 16); hi.y = __uint_as_float(v.z & 0xffff0000u);
      hi.z = __uint_as_float(v.w << 16); hi.w = __uint_as_float(v.w & 0xffff0000u);
      *reinterpret_cast<float4 *>(dst + i) = lo;
      *reinterpret_cast<float4 *>(dst + i + 4) = hi;
    } else {
      for (uint64_t j = i; j < n; ++j) dst[j] = bf16_bits_to_f32(src[j]);
    }
  }
}

__global__ __launch_bounds__(256) void narrow_bf16_kernel(uint64_t n, const float *__restrict__ src,
                                                         uint16_t *__restrict__ dst) {
  const uint64_t stride = (uint64_t)gridDim.x * 256u * 8u;
  for (uint64_t i = ((uint64_t)blockIdx.x * 256u + threadIdx.x) * 8u; i < n; i += stride) {
    if (i + 8u <= n) {
      const float4 lo = *reinterpret_cast<const float4 *>(src + i);
      const float4 hi = *reinterpret_cast<const float4 *>(src + i + 4);
      uint4 v;
      v.x = (uint32_t)f32_to_bf16_bits(lo.x) | ((uint32_t)f32_to_bf16_bits(lo.y) << 16);
      v.y = (uint32_t)f32_to_bf16_bits(lo.z) | ((uint32_t)f32_to_bf16_bits(lo.w) << 16);
      v.z = (uint32_t)f32_to_bf16_bits(hi.x) | ((uint32_t)f32_to_bf16_bits(hi.y) << 16);
      v.w = (uint32_t)f32_to_bf16_bits(hi.z) | ((uint32_t)f32_to_bf16_bits(hi.w) << 16);
      typedef uint4 U4 __attribute__((aligned(2)));
      *reinterpret_cast<U4 *>(dst + i) = v;
    } else {
      for (uint64_t j = i; j < n; ++j) dst[j] = f32_to_bf16_bits(src[j]);
    }
  }
}

// Rows of `w_src` bf16 elements copied into rows of `w_dst` >= w_src elements (w_dst even; dst 4-byte aligned),
// zeros behind: one thread per dword of the destination.
__global__ __launch_bounds__(256) void repitch_bf16_kernel(uint64_t rows, uint32_t w_src, uint32_t w_dst,
                                                          const uint16_t *__restrict__ src, uint32_t *__restrict__ dst) {
  const uint32_t row_dwords = w_dst >> 1;
  const uint64_t n = rows * row_dwords;
  const uint64_t stride = (uint64_t)gridDim.x * 256u;
  for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < n; i += stride) {
    const uint64_t r = i / row_dwords;
    const uint32_t c = (uint32_t)(i - r * row_dwords) * 2u;
    const uint16_t *p = src + r * w_src + c;
    const uint32_t lo = c < w_src ? p[0] : 0u, hi = c + 1u < w_src ? p[1] : 0u;
    dst[i] = lo | (hi << 16);
  }
}

static uint32_t cvt_grid(uint64_t n) {
  uint64_t b = (n + 2047) / 2048;
  if (b > 256ull * 32) b = 256ull * 32;
  return (uint32_t)(b ? b : 1);
}

// fp32 scratch copies live in 256-byte aligned consecutive regions of the workspace
static size_t region(uint64_t elems) { return (size_t)((elems * 4u + 255u) / 256u * 256u); }

bool conv_bf16_mfma_supported(int which, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W);
size_t conv_bf16_mfma_workspace_bytes(int which, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                                      uint32_t W);
int conv_bf16_mfma(int which, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                   const void *const *in_tiles, const void *w, void *const *out_tiles, float beta, void *workspace,
                   hipStream_t st, bool halofree = false);

bool conv_bf16_wgrad_mfma_supported(uint32_t Cin, uint32_t Cout, uint32_t W);
size_t conv_bf16_wgrad_mfma_workspace_bytes(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t W);
int conv_bf16_wgrad_mfma(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                         const void *const *x_tiles, const void *const *dy_tiles, float *dw, float beta,
                         void *workspace, hipStream_t st, bool unpadded);

// The filter gradient at a width that is no multiple of 8: the rows of x_pad and dy are copied into rows of the
// next multiple of 8 (+ 2 for x_pad) with zeros behind, and the matrix-core kernel runs on the copies: a dy that
// is zero in the added columns adds nothing to any tap.  (Not when the widened image passes the 2 GiB a buffer
// resource addresses.)
static uint32_t wgrad_wide_width(uint32_t W) { return (W + 7u) & ~7u; }
static bool wgrad_repitch_route(uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W) {
  if ((W % 8u) == 0u) return false;
  const uint32_t Wd = wgrad_wide_width(W);
  return conv_bf16_wgrad_mfma_supported(Cin, Cout, Wd) &&
         (uint64_t)(Cin > Cout ? Cin : Cout) * (H + 2ull) * (Wd + 2ull) * 2u < (1ull << 31);
}
static size_t repitch_region(uint64_t elems) { return (size_t)((elems * 2u + 255u) / 256u * 256u); }

size_t bf16_workspace_bytes(int which, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                            uint32_t W, size_t fp32_path_bytes) {
  if (which == ADH_CONV_BWD_FILTER && conv_bf16_wgrad_mfma_supported(Cin, Cout, W))
    return conv_bf16_wgrad_mfma_workspace_bytes(num_tiles, N, Cin, Cout, W);
  if (which == ADH_CONV_BWD_FILTER && wgrad_repitch_route(Cin, Cout, H, W)) {
    const uint32_t Wd = wgrad_wide_width(W);
    return num_tiles * (repitch_region((uint64_t)N * Cin * (H + 2) * (Wd + 2)) + repitch_region((uint64_t)N * Cout * H * Wd)) +
           conv_bf16_wgrad_mfma_workspace_bytes(num_tiles, N, Cin, Cout, Wd);
  }
  if (which != ADH_CONV_BWD_FILTER && conv_bf16_mfma_supported(which, Cin, Cout, H, W))
    return conv_bf16_mfma_workspace_bytes(which, num_tiles, N, Cin, Cout, H, W);
  const uint64_t slab = (uint64_t)N * Cin * (H + 2) * (W + 2), out = (uint64_t)N * Cout * H * W;
  const uint64_t filt = (uint64_t)Cin * Cout * 9u;
  size_t total = 0;
  if (which == ADH_CONV_BWD_FILTER) total = num_tiles * (region(slab) + region(out));
  else total = num_tiles * (region(slab) + region(out)) + region(filt);
  return total + (fp32_path_bytes + 255u) / 256u * 256u;
}

}  // namespace adh

using namespace adh;

// fp32 kernels of the other translation units
extern "C" size_t adh_conv3x3_workspace_bytes(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin,
                                              uint32_t Cout, uint32_t H, uint32_t W);

namespace adh {

static int widen(uint64_t n, const void *src, float *dst, hipStream_t st) {
  hipLaunchKernelGGL(widen_bf16_kernel, dim3(cvt_grid(n)), dim3(256), 0, st, n, reinterpret_cast<const uint16_t *>(src), dst);
  return launch_status();
}
static int narrow(uint64_t n, const float *src, void *dst, hipStream_t st) {
  hipLaunchKernelGGL(narrow_bf16_kernel, dim3(cvt_grid(n)), dim3(256), 0, st, n, src, reinterpret_cast<uint16_t *>(dst));
  return launch_status();
}

// which = ADH_CONV_FWD: in = x_pad tiles (slab sized), out = y tiles; ADH_CONV_BWD_DATA: in = dy
// tiles, out = dx_pad tiles.  Called by the dispatchers in conv3x3.hip for dtype == ADH_BF16.
int conv_bf16_via_f32(int which, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                      const void *const *in_tiles, const void *w, void *const *out_tiles, float beta, void *workspace,
                      size_t workspace_bytes, hipStream_t st) {
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (N == 0 || Cin == 0 || Cout == 0 || H == 0 || W == 0) return ADH_OK;
  if (!in_tiles || !out_tiles || !w) return ADH_ENULL;
  if (!aligned_to(w, 2)) return ADH_EALIGN;
  const size_t need = bf16_workspace_bytes(which, num_tiles, N, Cin, Cout, H, W, 0);
  if (!workspace) return ADH_ENULL;
  if (!aligned_to(workspace, 256)) return ADH_EALIGN;
  if (workspace_bytes < need) return ADH_EWORKSPACE;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!in_tiles[t] || !out_tiles[t]) return ADH_ENULL;
    if (!aligned_to(in_tiles[t], 2) || !aligned_to(out_tiles[t], 2)) return ADH_EALIGN;
  }
  if (conv_bf16_mfma_supported(which, Cin, Cout, H, W)) {
    // one image is addressed through a 32-bit buffer resource
    const uint64_t cmax = Cin > Cout ? Cin : Cout;
    if (cmax * (H + 2ull) * (W + 2ull) * 2u >= (1ull << 31) || (uint64_t)Cin * Cout * 18u >= (1ull << 31))
      return ADH_EINVAL;
    return conv_bf16_mfma(which, num_tiles, N, Cin, Cout, H, W, in_tiles, w, out_tiles, beta, workspace, st);
  }
  const uint64_t slab = (uint64_t)N * Cin * (H + 2) * (W + 2), outn = (uint64_t)N * Cout * H * W;
  const uint64_t in_elems = which == ADH_CONV_FWD ? slab : outn;
  const uint64_t out_elems = which == ADH_CONV_FWD ? outn : slab;
  char *ws = reinterpret_cast<char *>(workspace);
  const void *in32[ADH_MAX_TILES];
  void *out32[ADH_MAX_TILES];
  float *w32 = reinterpret_cast<float *>(ws);
  ws += region((uint64_t)Cin * Cout * 9u);
  int e = widen((uint64_t)Cin * Cout * 9u, w, w32, st);
  if (e) return e;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    float *i32 = reinterpret_cast<float *>(ws);
    ws += region(in_elems);
    float *o32 = reinterpret_cast<float *>(ws);
    ws += region(out_elems);
    if ((e = widen(in_elems, in_tiles[t], i32, st))) return e;
    if (beta != 0.f && (e = widen(out_elems, out_tiles[t], o32, st))) return e;
    in32[t] = i32;
    out32[t] = o32;
  }
  if (which == ADH_CONV_FWD)
    e = adh_conv3x3_slab_fwd_tiles(ADH_F32, num_tiles, N, Cin, Cout, H, W, in32, w32, out32, beta, nullptr, 0, st);
  else
    e = adh_conv3x3_slab_bwd_data_tiles(ADH_F32, num_tiles, N, Cin, Cout, H, W, w32, in32, out32, beta, nullptr, 0, st);
  if (e) return e;
  for (uint32_t t = 0; t < num_tiles; ++t)
    if ((e = narrow(out_elems, reinterpret_cast<const float *>(out32[t]), out_tiles[t], st))) return e;
  return ADH_OK;
}

int conv_bf16_filter_via_f32(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                             const void *const *x_tiles, const void *const *dy_tiles, float *dw, float beta,
                             void *workspace, size_t workspace_bytes, hipStream_t st) {
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (Cin == 0 || Cout == 0) return ADH_OK;
  if (!dw) return ADH_ENULL;
  if (N == 0 || H == 0 || W == 0)
    return adh_conv3x3_slab_bwd_filter_tiles(ADH_F32, num_tiles, N, Cin, Cout, H, W, x_tiles, dy_tiles, dw, beta,
                                             workspace, workspace_bytes, st);
  if (!x_tiles || !dy_tiles) return ADH_ENULL;
  if (conv_bf16_wgrad_mfma_supported(Cin, Cout, W)) {
    if (!workspace) return ADH_ENULL;
    if (!aligned_to(workspace, 256) || !aligned_to(dw, 4)) return ADH_EALIGN;
    if (workspace_bytes < conv_bf16_wgrad_mfma_workspace_bytes(num_tiles, N, Cin, Cout, W)) return ADH_EWORKSPACE;
    // one image is addressed through a 32-bit buffer resource
    if ((uint64_t)(Cin > Cout ? Cin : Cout) * (H + 2ull) * (W + 2ull) * 2u >= (1ull << 31)) return ADH_EINVAL;
    for (uint32_t t = 0; t < num_tiles; ++t) {
      if (!x_tiles[t] || !dy_tiles[t]) return ADH_ENULL;
      if (!aligned_to(x_tiles[t], 2) || !aligned_to(dy_tiles[t], 2)) return ADH_EALIGN;
    }
    return conv_bf16_wgrad_mfma(num_tiles, N, Cin, Cout, H, W, x_tiles, dy_tiles, dw, beta, workspace, st, false);
  }
  if (wgrad_repitch_route(Cin, Cout, H, W)) {
    const uint32_t Wd = wgrad_wide_width(W);
    if (!workspace) return ADH_ENULL;
    if (!aligned_to(workspace, 256) || !aligned_to(dw, 4)) return ADH_EALIGN;
    if (workspace_bytes < bf16_workspace_bytes(ADH_CONV_BWD_FILTER, num_tiles, N, Cin, Cout, H, W, 0)) return ADH_EWORKSPACE;
    const uint64_t x_rows = (uint64_t)N * Cin * (H + 2), dy_rows = (uint64_t)N * Cout * H;
    char *ws = reinterpret_cast<char *>(workspace);
    const void *xw[ADH_MAX_TILES];
    const void *dyw[ADH_MAX_TILES];
    for (uint32_t t = 0; t < num_tiles; ++t) {
      if (!x_tiles[t] || !dy_tiles[t]) return ADH_ENULL;
      if (!aligned_to(x_tiles[t], 2) || !aligned_to(dy_tiles[t], 2)) return ADH_EALIGN;
      uint32_t *a = reinterpret_cast<uint32_t *>(ws);
      ws += repitch_region(x_rows * (Wd + 2));
      uint32_t *b = reinterpret_cast<uint32_t *>(ws);
      ws += repitch_region(dy_rows * Wd);
      hipLaunchKernelGGL(repitch_bf16_kernel, dim3(cvt_grid(x_rows * (Wd + 2) * 4u)), dim3(256), 0, st, x_rows, W + 2u, Wd + 2u,
                         reinterpret_cast<const uint16_t *>(x_tiles[t]), a);
      int e = launch_status();
      if (e) return e;
      hipLaunchKernelGGL(repitch_bf16_kernel, dim3(cvt_grid(dy_rows * Wd * 4u)), dim3(256), 0, st, dy_rows, W, Wd,
                         reinterpret_cast<const uint16_t *>(dy_tiles[t]), b);
      if ((e = launch_status())) return e;
      xw[t] = a;
      dyw[t] = b;
    }
    return conv_bf16_wgrad_mfma(num_tiles, N, Cin, Cout, H, Wd, xw, dyw, dw, beta, ws, st, false);
  }
  const size_t f32_bytes = adh_conv3x3_workspace_bytes(ADH_CONV_BWD_FILTER, ADH_F32, num_tiles, N, Cin, Cout, H, W);
  if (f32_bytes == 0) return ADH_EUNIMPL;
  const size_t need = bf16_workspace_bytes(ADH_CONV_BWD_FILTER, num_tiles, N, Cin, Cout, H, W, f32_bytes);
  if (!workspace) return ADH_ENULL;
  if (!aligned_to(workspace, 256)) return ADH_EALIGN;
  if (workspace_bytes < need) return ADH_EWORKSPACE;
  const uint64_t slab = (uint64_t)N * Cin * (H + 2) * (W + 2), outn = (uint64_t)N * Cout * H * W;
  char *ws = reinterpret_cast<char *>(workspace);
  const void *x32[ADH_MAX_TILES];
  const void *dy32[ADH_MAX_TILES];
  int e;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!x_tiles[t] || !dy_tiles[t]) return ADH_ENULL;
    if (!aligned_to(x_tiles[t], 2) || !aligned_to(dy_tiles[t], 2)) return ADH_EALIGN;
    float *a = reinterpret_cast<float *>(ws);
    ws += region(slab);
    float *b = reinterpret_cast<float *>(ws);
    ws += region(outn);
    if ((e = widen(slab, x_tiles[t], a, st))) return e;
    if ((e = widen(outn, dy_tiles[t], b, st))) return e;
    x32[t] = a;
    dy32[t] = b;
  }
  return adh_conv3x3_slab_bwd_filter_tiles(ADH_F32, num_tiles, N, Cin, Cout, H, W, x32, dy32, dw, beta, ws,
                                           workspace_bytes - (size_t)(ws - reinterpret_cast<char *>(workspace)), st);
}

}  // namespace adh

namespace adh {
int conv_wgrad_f32_unpadded(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                            const void *const *x_tiles, const void *const *dy_tiles, float *dw, float beta, void *workspace,
                            size_t workspace_bytes, void *stream);
}

// The filter gradient over tiles without halo: see adh_conv3x3_unpadded_fwd_tiles.
extern "C" int adh_conv3x3_unpadded_bwd_filter_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                                     uint32_t H, uint32_t W, const void *const *x_tiles,
                                                     const void *const *dy_tiles, float *dw, float beta, void *workspace,
                                                     size_t workspace_bytes, void *stream) {
  using namespace adh;
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if (dtype == ADH_F32)
    return conv_wgrad_f32_unpadded(num_tiles, N, Cin, Cout, H, W, x_tiles, dy_tiles, dw, beta, workspace, workspace_bytes,
                                   stream);
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (Cin == 0 || Cout == 0) return ADH_OK;
  if (!dw) return ADH_ENULL;
  if (!aligned_to(dw, 4)) return ADH_EALIGN;
  if (N == 0 || H == 0 || W == 0) {
    if (beta == 0.f) return adh_fill_f32((uint64_t)Cin * Cout * 9u, 0.f, dw, stream);  // an empty sum
    return ADH_OK;
  }
  if (!x_tiles || !dy_tiles) return ADH_ENULL;
  if (!conv_bf16_wgrad_mfma_supported(Cin, Cout, W)) return ADH_EUNIMPL;  // whole 16-byte granules per row
  if (!workspace) return ADH_ENULL;
  if (!aligned_to(workspace, 256)) return ADH_EALIGN;
  if (workspace_bytes < conv_bf16_wgrad_mfma_workspace_bytes(num_tiles, N, Cin, Cout, W)) return ADH_EWORKSPACE;
  if ((uint64_t)(Cin > Cout ? Cin : Cout) * (H + 2ull) * (W + 2ull) * 2u >= (1ull << 31)) return ADH_EINVAL;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!x_tiles[t] || !dy_tiles[t]) return ADH_ENULL;
    if (!aligned_to(x_tiles[t], 16) || !aligned_to(dy_tiles[t], 2)) return ADH_EALIGN;
  }
  return conv_bf16_wgrad_mfma(num_tiles, N, Cin, Cout, H, W, x_tiles, dy_tiles, dw, beta, workspace, as_stream(stream), true);
}
