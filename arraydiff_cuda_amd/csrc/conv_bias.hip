// The bias of a convolution: y[n,c,h,w] += bias[c] after the conv (cudnnAddTensor with a (1,C,1,1)
// descriptor, src/op.cc:1602-1610) and its gradient db[c] = beta*db[c] + sum over tiles, n, h, w of dy
// (cudnnConvolutionBackwardBias, src/op.cc:1632-1648).  Both HBM-bound; one launch covers all K tiles.
//
//   conv_bias_add_kernel   16 bytes per thread where a plane is a whole number of 16-byte groups (a group
//                          then lies in one channel), one element per thread otherwise
//   conv_bias_grad_kernel  workgroup (channel, split): adds its share of the channel's planes, every thread a
//                          fixed subsequence, then a tree over the workgroup; one number per workgroup
//   conv_bias_grad_final   one thread per channel adds the splits in order (double) and applies beta:
//                          the sum does not depend on timing, repeated calls give the same bits
#include "adh_common.h"

#include <algorithm>

namespace adh {

constexpr uint32_t kBiasThreads = 256;

struct BiasParams {
  void *y[ADH_MAX_TILES];           // add: the result tiles; gradient: the dy tiles
  const float *bias[ADH_MAX_TILES];  // add: one vector per tile
  float *partial;                    // gradient: [channel][split]
  uint32_t C, HW, groups_per_plane, planes, split, tiles, N;
  FastDiv div_groups, div_C, div_N;
};

__device__ __forceinline__ float bias_ld(float v) { return v; }
__device__ __forceinline__ float bias_ld(uint16_t v) { return bf16_bits_to_f32(v); }
__device__ __forceinline__ void bias_st(float &d, float v) { d = v; }
__device__ __forceinline__ void bias_st(uint16_t &d, float v) { d = f32_to_bf16_bits(v); }

template <typename T, int VEC>
struct __attribute__((packed, aligned(sizeof(T)))) BiasVec {
  T v[VEC];
};

// grid: (ceil(planes * groups_per_plane / 256), tiles); a group = VEC consecutive elements of one plane
template <typename T, int VEC>
__global__ __launch_bounds__(kBiasThreads) void conv_bias_add_kernel(const BiasParams P) {
  const uint32_t g = blockIdx.x * kBiasThreads + threadIdx.x;
  if (g >= P.planes * P.groups_per_plane) return;
  const uint32_t plane = P.div_groups.div(g);
  const uint32_t c = plane - P.div_C.div(plane) * P.C;
  const float b = P.bias[blockIdx.y][c];
  typedef BiasVec<T, VEC> V;
  V *p = reinterpret_cast<V *>(static_cast<T *>(P.y[blockIdx.y])) + g;
  V v = *p;
#pragma unroll
  for (int i = 0; i < VEC; ++i) bias_st(v.v[i], bias_ld(v.v[i]) + b);
  *p = v;
}

// grid: (split, C).  The channel's planes (tile, n) are numbered tile-major; workgroup s takes planes
// s, s + split, ...
template <typename T, int VEC>
__global__ __launch_bounds__(kBiasThreads) void conv_bias_grad_kernel(const BiasParams P) {
  const uint32_t c = blockIdx.y, s = blockIdx.x;
  float acc[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
  typedef BiasVec<T, VEC> V;
  for (uint32_t q = s; q < P.tiles * P.N; q += P.split) {
    const uint32_t t = P.div_N.div(q), n = q - t * P.N;
    const V *p = reinterpret_cast<const V *>(static_cast<const T *>(P.y[t]) + ((size_t)n * P.C + c) * P.HW);
    for (uint32_t g = threadIdx.x; g < P.groups_per_plane; g += kBiasThreads) {
      const V v = p[g];
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[i] += bias_ld(v.v[i]);
    }
  }
  float a = acc[0];
#pragma unroll
  for (int i = 1; i < VEC; ++i) a += acc[i];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) a += __shfl_xor(a, o);
  __shared__ float red[kBiasThreads / 64];
  if ((threadIdx.x & 63u) == 0) red[threadIdx.x >> 6] = a;
  __syncthreads();
  if (threadIdx.x == 0) P.partial[(size_t)c * P.split + s] = (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ void conv_bias_grad_final(const float *partial, uint32_t C, uint32_t split, float beta, float *db) {
  const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  double a = 0.0;
  for (uint32_t s = 0; s < split; ++s) a += (double)partial[(size_t)c * split + s];
  db[c] = (float)(beta != 0.0f ? a + (double)beta * (double)db[c] : a);
}

static uint32_t bias_grad_split(uint32_t tiles, uint32_t N, uint32_t C) {
  // about four workgroups per CU over the whole launch, never more than the channel has planes
  uint32_t s = (1024 + C - 1) / C;
  return std::max(1u, std::min(s, tiles * N));
}

template <typename T>
static int bias_add_launch(BiasParams &P, bool vec_ok, uint32_t tiles, hipStream_t st) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool vec = vec_ok && P.HW % VEC == 0;
  P.groups_per_plane = vec ? P.HW / VEC : P.HW;
  P.div_groups = FastDiv(P.groups_per_plane);
  const uint64_t groups = (uint64_t)P.planes * P.groups_per_plane;
  if (groups >= (1ull << 31)) return ADH_EINVAL;
  const dim3 grid((uint32_t)((groups + kBiasThreads - 1) / kBiasThreads), tiles);
  if (vec)
    hipLaunchKernelGGL((conv_bias_add_kernel<T, VEC>), grid, dim3(kBiasThreads), 0, st, P);
  else
    hipLaunchKernelGGL((conv_bias_add_kernel<T, 1>), grid, dim3(kBiasThreads), 0, st, P);
  return launch_status();
}

template <typename T>
static int bias_grad_launch(BiasParams &P, bool vec_ok, hipStream_t st) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const bool vec = vec_ok && P.HW % VEC == 0;
  P.groups_per_plane = vec ? P.HW / VEC : P.HW;
  const dim3 grid(P.split, P.C);
  if (vec)
    hipLaunchKernelGGL((conv_bias_grad_kernel<T, VEC>), grid, dim3(kBiasThreads), 0, st, P);
  else
    hipLaunchKernelGGL((conv_bias_grad_kernel<T, 1>), grid, dim3(kBiasThreads), 0, st, P);
  return launch_status();
}

}  // namespace adh

using namespace adh;

extern "C" int adh_conv_bias_add_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                                       const float *const *bias_tiles, void *const *y_tiles, void *stream) {
  if (!dtype_ok(dtype) || num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if (!bias_tiles || !y_tiles) return ADH_ENULL;
  if (N == 0 || C == 0 || H == 0 || W == 0) return ADH_OK;
  if ((uint64_t)H * W >= (1ull << 31) || (uint64_t)N * C >= (1ull << 31)) return ADH_EINVAL;
  BiasParams P{};
  bool vec_ok = true;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!bias_tiles[t] || !y_tiles[t]) return ADH_ENULL;
    if (!aligned_to(y_tiles[t], dtype_size(dtype)) || !aligned_to(bias_tiles[t], 4)) return ADH_EALIGN;
    P.y[t] = y_tiles[t];
    P.bias[t] = bias_tiles[t];
  }
  P.C = C;
  P.HW = H * W;
  P.planes = N * C;
  P.div_C = FastDiv(C);
  return dtype == ADH_F32 ? bias_add_launch<float>(P, vec_ok, num_tiles, as_stream(stream))
                          : bias_add_launch<uint16_t>(P, vec_ok, num_tiles, as_stream(stream));
}

extern "C" size_t adh_conv_bwd_bias_workspace_bytes(uint32_t num_tiles, uint32_t N, uint32_t C) {
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES || N == 0 || C == 0) return 0;
  return (size_t)C * bias_grad_split(num_tiles, N, C) * sizeof(float);
}

extern "C" int adh_conv_bwd_bias_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                                       const void *const *dy_tiles, float *db, float beta, void *workspace,
                                       size_t workspace_bytes, void *stream) {
  if (!dtype_ok(dtype) || num_tiles == 0 || num_tiles > ADH_MAX_TILES || (beta != 0.0f && beta != 1.0f))
    return ADH_EINVAL;
  if (!dy_tiles || !db) return ADH_ENULL;
  if (C == 0) return ADH_OK;
  if ((uint64_t)H * W >= (1ull << 31) || C > 65535) return ADH_EINVAL;
  if (!aligned_to(db, 4)) return ADH_EALIGN;
  const hipStream_t st = as_stream(stream);
  if (N == 0 || H == 0 || W == 0) {  // an empty sum
    if (beta == 0.0f) {
      hipLaunchKernelGGL(conv_bias_grad_final, dim3((C + 255) / 256), dim3(256), 0, st, (const float *)nullptr, C, 0u,
                         beta, db);
      return launch_status();
    }
    return ADH_OK;
  }
  BiasParams P{};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!dy_tiles[t]) return ADH_ENULL;
    if (!aligned_to(dy_tiles[t], dtype_size(dtype))) return ADH_EALIGN;
    P.y[t] = const_cast<void *>(dy_tiles[t]);
  }
  const size_t need = adh_conv_bwd_bias_workspace_bytes(num_tiles, N, C);
  if (!workspace) return ADH_ENULL;
  if (workspace_bytes < need) return ADH_EWORKSPACE;
  if (!aligned_to(workspace, 256)) return ADH_EALIGN;
  P.partial = static_cast<float *>(workspace);
  P.C = C;
  P.N = N;
  P.HW = H * W;
  P.tiles = num_tiles;
  P.split = bias_grad_split(num_tiles, N, C);
  P.div_N = FastDiv(N);
  const int rc = dtype == ADH_F32 ? bias_grad_launch<float>(P, true, st) : bias_grad_launch<uint16_t>(P, true, st);
  if (rc != ADH_OK) return rc;
  hipLaunchKernelGGL(conv_bias_grad_final, dim3((C + 255) / 256), dim3(256), 0, st, (const float *)P.partial, C, P.split,
                     beta, db);
  return launch_status();
}
