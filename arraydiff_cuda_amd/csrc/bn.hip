// The shard-local ops between two halo exchanges: spatial batch normalisation with tile-local batch
// statistics (every rank of the reference normalises its own tile), the rectifier and the
// residual sum.  All HBM-bound.
//
// Batch norm, training forward (three launches):
//   bn_reduce_kernel<FWD>  per (tile, channel, split of the batch): sum (x - K) and sum (x - K)^2 with
//                          K = the channel's first element, so that the sums stay small next to
//                          the variance; fp32 per thread, tree over the block
//   bn_apply_kernel        first, one thread per plane of the workgroup adds the channel's splits in double:
//                          mean, 1/sqrt(var + eps), running statistics, a = scale / sqrt(var + eps) (there
//                          is no finalize launch between the two passes); then
//                          y = a*(x - mean) + shift (the difference first: the mean may be large next
//                          to the deviation), optionally max(., 0), optionally written into the interior
//                          of a halo-padded tile whose border it zeroes (BN -> ReLU -> HaloPad in
//                          one pass over the data)
// Backward mirrors it: reduce sum dy' and sum dy'*(x - mean) (dy' = dy masked by the rectifier, dy read
// from the interior of the padded gradient tile when the forward wrote a padded tile); apply works out
// the parameter gradients and three coefficients, then dx = beta*dx + k1*dy' + k2*(x - mean) + k3.
#include "adh_common.h"

#include <algorithm>

namespace adh {

constexpr uint32_t kBnThreads = 256;

struct BnParams {
  const void *x[ADH_MAX_TILES];
  const void *dy[ADH_MAX_TILES];
  void *out[ADH_MAX_TILES];  // y (forward) or dx (backward)
  const float *scale[ADH_MAX_TILES];
  const float *shift[ADH_MAX_TILES];
  const float *mean_in[ADH_MAX_TILES];    // backward / inference: saved or fixed mean
  const float *second_in[ADH_MAX_TILES];  // backward: saved 1/sqrt(var + eps); inference: fixed variance
  float *o0[ADH_MAX_TILES];               // forward: running mean;     backward: scale gradient
  float *o1[ADH_MAX_TILES];               // forward: running variance; backward: shift gradient
  float *o2[ADH_MAX_TILES];               // forward: saved mean
  float *o3[ADH_MAX_TILES];               // forward: saved 1/sqrt(var + eps)
  float *partial;                         // [tile][c][split][2]
  uint32_t N, C, H, W, HW, p, split, n_per_split, tiles, groups_per_plane, slots_log2, planes_per_pass;
  float eps, beta, beta_param;  // beta: input-gradient accumulation; beta_param: parameter-gradient accumulation
  int relu;
  FastDiv div_C, div_N, div_split, div_groups, div_cols;  // div_groups: the 16-byte groups of a plane; div_cols: row length of the index that a kernel splits into (row, column)
};

__device__ __forceinline__ float bn_ld(const float *p, size_t i) { return p[i]; }
__device__ __forceinline__ float bn_ld(const uint16_t *p, size_t i) { return bf16_bits_to_f32(p[i]); }
__device__ __forceinline__ void bn_st(float *p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void bn_st(uint16_t *p, size_t i, float v) { p[i] = f32_to_bf16_bits(v); }

// VEC elements moved by one 16-byte access at element alignment (gfx950 takes unaligned vector accesses)
template <typename T, int VEC>
struct __attribute__((packed, aligned(sizeof(T)))) BnVec {
  T v[VEC];
};
__device__ __forceinline__ float bn_f(float v) { return v; }
__device__ __forceinline__ float bn_f(uint16_t v) { return bf16_bits_to_f32(v); }
__device__ __forceinline__ void bn_t(float &d, float v) { d = v; }
__device__ __forceinline__ void bn_t(uint16_t &d, float v) { d = f32_to_bf16_bits(v); }

__device__ __forceinline__ float2 block_sum2(float a, float b) {
  __shared__ float red[2][kBnThreads / 64];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    a += __shfl_xor(a, o);
    b += __shfl_xor(b, o);
  }
  const uint32_t wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63u) == 0) {
    red[0][wave] = a;
    red[1][wave] = b;
  }
  __syncthreads();
  float2 r;
  r.x = (red[0][0] + red[0][1]) + (red[0][2] + red[0][3]);
  r.y = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
  return r;
}

// grid: tiles * C * split.  BWD = false: sums of (x - K), (x - K)^2.  BWD = true: sums of dy', dy' * (x - mean)
// (dy' = dy where a*(x - mean) + shift > 0 when the rectifier was fused, else dy), dy at the interior of a tile padded by p.
// VEC > 1: H*W (and, backward, W) are whole numbers of VEC-element groups, one 16-byte access per group.
template <typename T, bool BWD, int VEC>
__global__ __launch_bounds__(kBnThreads) void bn_reduce_kernel(const BnParams P) {
  typedef BnVec<T, VEC> Vec;
  uint32_t tc, sp, tile, c;
  P.div_split.divmod(blockIdx.x, tc, sp);
  P.div_C.divmod(tc, tile, c);
  const T *x = reinterpret_cast<const T *>(P.x[tile]);
  const uint32_t n0 = sp * P.n_per_split, n1 = min(P.N, n0 + P.n_per_split);
  const uint32_t groups = P.HW / (uint32_t)VEC;
  float s1 = 0.f, s2 = 0.f;
  if (!BWD) {
    const float K = bn_ld(x, (size_t)c * P.HW);
    // the groups of the split's planes are numbered through: a plane of a few groups (a late layer's 4 x 16 tile
    // is 16 of them) would otherwise leave most of the workgroup idle for one load latency per plane
    // (P.planes_per_pass planes at a time keep the running number below 2^31: one pass but for gigantic planes)
    for (uint32_t nb = n0; nb < n1; nb += P.planes_per_pass) {
      const uint32_t items = min(P.planes_per_pass, n1 - nb) * groups;
      for (uint32_t it = threadIdx.x; it < items; it += kBnThreads) {
        uint32_t nr, i;
        P.div_groups.divmod(it, nr, i);
        const T *pl = x + ((size_t)(nb + nr) * P.C + c) * P.HW;
        const Vec xv = *reinterpret_cast<const Vec *>(pl + (size_t)i * VEC);
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          const float v = bn_f(xv.v[k]) - K;
          s1 += v;
          s2 += v * v;
        }
      }
    }
  } else {
    const T *dy = reinterpret_cast<const T *>(P.dy[tile]);
    const uint32_t WP = P.W + 2u * P.p, HPp = P.H + 2u * P.p;
    const float a = P.relu ? P.scale[tile][c] * P.second_in[tile][c] : 0.f;
    const float mean = P.mean_in[tile][c];
    const float b = P.relu ? P.shift[tile][c] : 0.f;
    for (uint32_t nb = n0; nb < n1; nb += P.planes_per_pass) {
      const uint32_t items = min(P.planes_per_pass, n1 - nb) * groups;
      for (uint32_t it = threadIdx.x; it < items; it += kBnThreads) {
        uint32_t nr, i, h, w;
        P.div_groups.divmod(it, nr, i);
        P.div_cols.divmod(i, h, w);  // groups per row
        const T *pl = x + ((size_t)(nb + nr) * P.C + c) * P.HW;
        const T *dl = dy + ((size_t)(nb + nr) * P.C + c) * HPp * WP + (size_t)P.p * WP + P.p;
        const Vec xv = *reinterpret_cast<const Vec *>(pl + (size_t)i * VEC);
        const Vec dv = *reinterpret_cast<const Vec *>(dl + (size_t)h * WP + w * VEC);
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          const float xc = bn_f(xv.v[k]) - mean;
          float d = bn_f(dv.v[k]);
          if (P.relu && !(a * xc + b > 0.f)) d = 0.f;
          s1 += d;
          s2 += d * xc;
        }
      }
    }
  }
  const float2 r = block_sum2(s1, s2);
  if (threadIdx.x == 0) {
    P.partial[(size_t)blockIdx.x * 2u] = r.x;
    P.partial[(size_t)blockIdx.x * 2u + 1u] = r.y;
  }
}

// The five numbers the apply pass needs for one (tile, channel), worked out by ONE thread of every apply
// workgroup that touches the channel (the sums of the splits are added in double, in split order, so every
// workgroup gets the same bits).  `publish`: this thread also writes the channel's statistics (forward) or
// parameter gradients (backward); exactly one thread per (tile, channel) in the grid is told to.
//   MODE 0, training forward : cf = { a = scale / sqrt(var + eps), mean, shift }
//   MODE 1, inference        : the same from the fixed statistics
//   MODE 2, backward         : cf = { k1 = a, k2, k3, mean, shift };  dx = k1 dy' + k2 (x - mean) + k3
template <typename T, int MODE>
__device__ void bn_plane_coef(const BnParams &P, uint32_t tile, uint32_t c, bool publish, float *cf) {
  const size_t tc = (size_t)tile * P.C + c;
  if (MODE == 1) {
    const double invstd = 1.0 / sqrt((double)P.second_in[tile][c] + (double)P.eps);
    cf[0] = (float)((double)P.scale[tile][c] * invstd);
    cf[1] = P.mean_in[tile][c];
    cf[2] = P.shift[tile][c];
    return;
  }
  double s1 = 0.0, s2 = 0.0;
  for (uint32_t sp = 0; sp < P.split; ++sp) {
    s1 += (double)P.partial[(tc * P.split + sp) * 2u];
    s2 += (double)P.partial[(tc * P.split + sp) * 2u + 1u];
  }
  const double m = (double)P.N * (double)P.HW;
  if (MODE == 0) {
    const double K = (double)bn_ld(reinterpret_cast<const T *>(P.x[tile]), (size_t)c * P.HW);
    const double d = s1 / m, mean = K + d;
    double var = s2 / m - d * d;
    if (var < 0.0) var = 0.0;
    const double invstd = 1.0 / sqrt(var + (double)P.eps);
    if (publish) {
      if (P.o0[tile]) P.o0[tile][c] = (float)mean;
      if (P.o1[tile]) P.o1[tile][c] = (float)(m > 1.0 ? var * m / (m - 1.0) : var);
      if (P.o2[tile]) P.o2[tile][c] = (float)mean;
      if (P.o3[tile]) P.o3[tile][c] = (float)invstd;
    }
    cf[0] = (float)((double)P.scale[tile][c] * invstd);
    cf[1] = (float)mean;
    cf[2] = P.shift[tile][c];
  } else {
    const double mean = P.mean_in[tile][c], invstd = P.second_in[tile][c], scale = P.scale[tile][c];
    const double dshift = s1, dscale = s2 * invstd;  // sum dy' * (x - mean) * invstd
    if (publish) {
      P.o0[tile][c] = (float)((P.beta_param != 0.f ? (double)P.o0[tile][c] : 0.0) + dscale);
      P.o1[tile][c] = (float)((P.beta_param != 0.f ? (double)P.o1[tile][c] : 0.0) + dshift);
    }
    // dx = a * (dy' - dshift/m - xhat * dscale/m),  xhat = (x - mean) * invstd
    const double a = scale * invstd;
    cf[0] = (float)a;
    cf[1] = (float)(-a * invstd * dscale / m);
    cf[2] = (float)(-a * dshift / m);
    cf[3] = (float)mean;
    cf[4] = P.shift[tile][c];  // the rectifier's mask needs the forward output's sign
  }
}

// a thread moves VEC consecutive elements of the padded output
// plane (forward: any shape, the last partial group element by element) or of the packed gradient plane (backward:
// VEC > 1 needs H*W and W to be whole numbers of groups)
// MODE as in bn_plane_coef: the first U threads of the workgroup work out the coefficients of its U planes
// (there is no separate finalize launch), everyone else picks them up from LDS.
template <typename T, int MODE, int VEC>
__global__ __launch_bounds__(kBnThreads) void bn_apply_kernel(const BnParams P) {
  typedef BnVec<T, VEC> Vec;
  constexpr bool BWD = MODE == 2;
  constexpr int U = 4;  // planes per thread: a thread moves the same group of each, all loads before the first store
  // A plane of at most 128 groups (the late layers' tiles) takes P.slots = 16 .. 128 threads, and the workgroup's
  // 256 / P.slots parts take U planes each; a larger plane takes the whole workgroup, band by band (blockIdx.y).
  __shared__ float cf_s[U * 16][8];
  const uint32_t WP = P.W + 2u * P.p, HPp = P.H + 2u * P.p;
  const uint32_t total = HPp * WP;
  const uint32_t planes = P.tiles * P.N * P.C;
  const uint32_t parts = kBnThreads >> P.slots_log2;
  const uint32_t part = threadIdx.x >> P.slots_log2;
  if (threadIdx.x < (uint32_t)U * parts) {
    const uint32_t pl = blockIdx.x * U * parts + threadIdx.x;
    if (pl < planes) {
      uint32_t tn, c, tile, n;
      P.div_C.divmod(pl, tn, c);
      P.div_N.divmod(tn, tile, n);
      bn_plane_coef<T, MODE>(P, tile, c, blockIdx.y == 0u && n == 0u, cf_s[threadIdx.x]);
    }
  }
  __syncthreads();
  const uint32_t gi = blockIdx.y * kBnThreads + (threadIdx.x & ((1u << P.slots_log2) - 1u));  // group of VEC elements within a plane
  if (gi >= P.groups_per_plane) return;
  // where the group sits is the same for every plane
  uint32_t r = 0, col = 0, in_off = 0, mask = 0;
  bool whole = false;
  if (!BWD) {
    P.div_cols.divmod(gi * VEC, r, col);
    whole = VEC > 1 && r - P.p < P.H && col >= P.p && col + VEC <= P.p + P.W;  // inside one interior row
    in_off = (r - P.p) * P.W + (col - P.p);
    if (!whole) {
      uint32_t rr = r, cc = col;
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        if (rr - P.p < P.H && cc - P.p < P.W) mask |= 1u << k;
        if (++cc == WP) {
          cc = 0;
          ++rr;
        }
      }
    } else {
      mask = (1u << VEC) - 1u;
    }
  } else {
    uint32_t h, w;
    P.div_cols.divmod(gi, h, w);  // groups per row
    in_off = h * WP + w * VEC;     // within the interior of the padded gradient plane
  }
  Vec xv[U], dv[U], old[U];
  const float *cf_u[U];
  T *out_u[U];
  bool live[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const uint32_t pl = (blockIdx.x * parts + part) * U + u;
    live[u] = pl < planes;
    if (!live[u]) continue;
    uint32_t tn, c, tile, n;
    P.div_C.divmod(pl, tn, c);
    P.div_N.divmod(tn, tile, n);
    cf_u[u] = cf_s[part * U + u];
    const T *x = reinterpret_cast<const T *>(P.x[tile]) + ((size_t)n * P.C + c) * P.HW;
    if (!BWD) {
      out_u[u] = reinterpret_cast<T *>(P.out[tile]) + ((size_t)n * P.C + c) * total;
      if (whole) {
        xv[u] = *reinterpret_cast<const Vec *>(x + in_off);
      } else {
        uint32_t rr = r, cc = col;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          if (mask >> k & 1u) xv[u].v[k] = x[(size_t)(rr - P.p) * P.W + (cc - P.p)];
          if (++cc == WP) {
            cc = 0;
            ++rr;
          }
        }
      }
    } else {
      const T *dy = reinterpret_cast<const T *>(P.dy[tile]) + ((size_t)n * P.C + c) * total + (size_t)P.p * WP + P.p;
      out_u[u] = reinterpret_cast<T *>(P.out[tile]) + ((size_t)n * P.C + c) * P.HW;
      xv[u] = *reinterpret_cast<const Vec *>(x + (size_t)gi * VEC);
      dv[u] = *reinterpret_cast<const Vec *>(dy + in_off);
      if (P.beta != 0.f) old[u] = *reinterpret_cast<const Vec *>(out_u[u] + (size_t)gi * VEC);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (!live[u]) continue;
    const float *cf = cf_u[u];
    Vec out;
    if (!BWD) {
      const float a = cf[0], mean = cf[1], b = cf[2];
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        float v = 0.f;
        if (mask >> k & 1u) {
          v = a * (bn_f(xv[u].v[k]) - mean) + b;
          if (P.relu) v = v > 0.f ? v : 0.f;
        }
        bn_t(out.v[k], v);
      }
      const uint32_t o = gi * VEC;
      if (o + VEC <= total) {
        *reinterpret_cast<Vec *>(out_u[u] + o) = out;
      } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          if (o + k < total) out_u[u][o + k] = out.v[k];
      }
    } else {
      const float k1 = cf[0], k2 = cf[1], k3 = cf[2], mean = cf[3], b = cf[4];
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const float xc = bn_f(xv[u].v[k]) - mean;
        float d = bn_f(dv[u].v[k]);
        if (P.relu && !(k1 * xc + b > 0.f)) d = 0.f;
        float g = k1 * d + k2 * xc + k3;
        if (P.beta != 0.f) g += bn_f(old[u].v[k]);
        bn_t(out.v[k], g);
      }
      *reinterpret_cast<Vec *>(out_u[u] + (size_t)gi * VEC) = out;
    }
  }
}

// ---- rectifier and residual sum ----

template <typename T>
__global__ __launch_bounds__(256) void relu_fwd_kernel(uint64_t n, const T *__restrict__ x, T *__restrict__ y) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256u) {
    const float v = bn_ld(x, i);
    bn_st(y, i, v > 0.f ? v : 0.f);
  }
}
template <typename T>
__global__ __launch_bounds__(256) void relu_bwd_kernel(uint64_t n, const T *__restrict__ y, const T *__restrict__ dy,
                                                       T *__restrict__ dx, float beta) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256u) {
    float g = bn_ld(y, i) > 0.f ? bn_ld(dy, i) : 0.f;
    if (beta != 0.f) g += bn_ld(dx, i);
    bn_st(dx, i, g);
  }
}
struct SumParams {
  const void *x[ADH_MAX_TILES];
  uint32_t count;
};
template <typename T>
__global__ __launch_bounds__(256) void sum_fwd_kernel(uint64_t n, const SumParams S, T *__restrict__ y) {
  for (uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256u) {
    float v = bn_ld(reinterpret_cast<const T *>(S.x[0]), i);
    for (uint32_t k = 1; k < S.count; ++k) v += bn_ld(reinterpret_cast<const T *>(S.x[k]), i);
    bn_st(y, i, v);
  }
}

// ---- host side ----

static size_t bn_ws_bytes(uint32_t tiles, uint32_t C, uint32_t split) {
  return ((size_t)tiles * C * split * 2u + (size_t)tiles * C * 8u) * 4u;
}
static uint32_t bn_split(uint32_t tiles, uint32_t N, uint32_t C) {
  const uint64_t tc = (uint64_t)tiles * C;
  return (uint32_t)std::max<uint64_t>(1u, std::min<uint64_t>(N, (2048u + tc - 1u) / tc));
}

static int bn_common(int dtype, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W, uint32_t p,
                     void *workspace, size_t workspace_bytes, BnParams *P) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if ((uint64_t)(H + 2ull * p) * (W + 2ull * p) >= (1ull << 31) || (uint64_t)N * C * num_tiles >= (1ull << 31)) return ADH_EINVAL;
  if (p > 4096u) return ADH_EINVAL;
  P->N = N; P->C = C; P->H = H; P->W = W; P->HW = H * W; P->p = p; P->tiles = num_tiles;
  P->split = bn_split(num_tiles, N, C);
  P->n_per_split = (N + P->split - 1u) / std::max(P->split, 1u);
  P->div_C = FastDiv(C);
  P->div_split = FastDiv(P->split);
  if (N == 0 || C == 0 || H == 0 || W == 0) return ADH_OK;
  if (!workspace) return ADH_ENULL;
  if (!aligned_to(workspace, 256)) return ADH_EALIGN;
  if (workspace_bytes < bn_ws_bytes(num_tiles, C, P->split)) return ADH_EWORKSPACE;
  P->partial = reinterpret_cast<float *>(workspace);
  return ADH_OK;
}

// sets the apply kernel's work split and returns its grid: x = groups of four planes, y = bands of 256 groups of a plane
static dim3 bn_apply_grid(BnParams *P, uint32_t groups_per_plane) {
  P->groups_per_plane = groups_per_plane;
  P->div_N = FastDiv(P->N);
  // threads per plane: the whole workgroup, or for planes of at most 128 groups the power of two that holds them
  P->slots_log2 = 8;
  if (groups_per_plane <= kBnThreads / 2u) {
    P->slots_log2 = 4;
    while ((1u << P->slots_log2) < groups_per_plane) ++P->slots_log2;
  }
  const uint64_t planes = (uint64_t)P->tiles * P->N * P->C;
  const uint64_t per_block = 4u * (kBnThreads >> P->slots_log2);
  return dim3((uint32_t)((planes + per_block - 1u) / per_block), (groups_per_plane + kBnThreads - 1u) / kBnThreads);
}

}  // namespace adh

using namespace adh;

extern "C" {

size_t adh_batchnorm2d_workspace_bytes(uint32_t num_tiles, uint32_t N, uint32_t C) {
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return 0;
  return (bn_ws_bytes(num_tiles, C, bn_split(num_tiles, N, C)) + 255u) & ~(size_t)255u;
}

int adh_batchnorm2d_fwd_tiles(int dtype, int training, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                              float eps, int relu, uint32_t out_halo, const void *const *x_tiles,
                              const float *const *scale_tiles, const float *const *shift_tiles,
                              const float *const *fixed_mean_tiles, const float *const *fixed_var_tiles,
                              void *const *y_tiles, float *const *run_mean_tiles, float *const *run_var_tiles,
                              float *const *save_mean_tiles, float *const *save_invstd_tiles, void *workspace,
                              size_t workspace_bytes, void *stream) {
  BnParams P = {};
  int e = bn_common(dtype, num_tiles, N, C, H, W, out_halo, workspace, workspace_bytes, &P);
  if (e) return e;
  if (N == 0 || C == 0 || H == 0 || W == 0) return ADH_OK;
  if (!(eps >= 0.f)) return ADH_EINVAL;
  if (!x_tiles || !scale_tiles || !shift_tiles || !y_tiles) return ADH_ENULL;
  if (!training && (!fixed_mean_tiles || !fixed_var_tiles)) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!x_tiles[t] || !scale_tiles[t] || !shift_tiles[t] || !y_tiles[t]) return ADH_ENULL;
    if (!aligned_to(x_tiles[t], es) || !aligned_to(y_tiles[t], es)) return ADH_EALIGN;
    P.x[t] = x_tiles[t];
    P.out[t] = y_tiles[t];
    P.scale[t] = scale_tiles[t];
    P.shift[t] = shift_tiles[t];
    if (training) {
      P.o0[t] = run_mean_tiles ? run_mean_tiles[t] : nullptr;
      P.o1[t] = run_var_tiles ? run_var_tiles[t] : nullptr;
      P.o2[t] = save_mean_tiles ? save_mean_tiles[t] : nullptr;
      P.o3[t] = save_invstd_tiles ? save_invstd_tiles[t] : nullptr;
    } else {
      if (!fixed_mean_tiles[t] || !fixed_var_tiles[t]) return ADH_ENULL;
      P.mean_in[t] = fixed_mean_tiles[t];
      P.second_in[t] = fixed_var_tiles[t];
    }
  }
  P.eps = eps;
  P.relu = relu ? 1 : 0;
  P.div_cols = FastDiv(W + 2u * out_halo);  // the apply kernel walks the padded output plane
  hipStream_t st = as_stream(stream);
  const uint32_t tc = num_tiles * C;
  const uint32_t vec = (uint32_t)(16 / dtype_size(dtype));
  const bool wide = (H * W) % vec == 0;  // the statistics pass reads whole 16-byte groups
  P.div_groups = FastDiv(wide ? H * W / vec : H * W);
  P.planes_per_pass = std::max(1u, 0x7fffffffu / (wide ? H * W / vec : H * W));
  const uint32_t gpp = ((H + 2u * out_halo) * (W + 2u * out_halo) + vec - 1u) / vec;
  if ((gpp + kBnThreads - 1u) / kBnThreads > 65535u) return ADH_EINVAL;  // grid.y
  if (training) {
    if (dtype == ADH_F32) {
      if (wide) hipLaunchKernelGGL((bn_reduce_kernel<float, false, 4>), dim3(tc * P.split), dim3(kBnThreads), 0, st, P);
      else hipLaunchKernelGGL((bn_reduce_kernel<float, false, 1>), dim3(tc * P.split), dim3(kBnThreads), 0, st, P);
    } else {
      if (wide) hipLaunchKernelGGL((bn_reduce_kernel<uint16_t, false, 8>), dim3(tc * P.split), dim3(kBnThreads), 0, st, P);
      else hipLaunchKernelGGL((bn_reduce_kernel<uint16_t, false, 1>), dim3(tc * P.split), dim3(kBnThreads), 0, st, P);
    }
  }
  const dim3 grid = bn_apply_grid(&P, gpp);
  if (training) {
    if (dtype == ADH_F32) hipLaunchKernelGGL((bn_apply_kernel<float, 0, 4>), grid, dim3(kBnThreads), 0, st, P);
    else hipLaunchKernelGGL((bn_apply_kernel<uint16_t, 0, 8>), grid, dim3(kBnThreads), 0, st, P);
  } else {
    if (dtype == ADH_F32) hipLaunchKernelGGL((bn_apply_kernel<float, 1, 4>), grid, dim3(kBnThreads), 0, st, P);
    else hipLaunchKernelGGL((bn_apply_kernel<uint16_t, 1, 8>), grid, dim3(kBnThreads), 0, st, P);
  }
  return launch_status();
}

int adh_batchnorm2d_bwd_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W, int relu,
                              uint32_t dy_halo, const void *const *x_tiles, const void *const *dy_tiles,
                              const float *const *scale_tiles, const float *const *shift_tiles,
                              const float *const *save_mean_tiles, const float *const *save_invstd_tiles,
                              void *const *dx_tiles, float *const *dscale_tiles, float *const *dshift_tiles,
                              float beta_data, float beta_param, void *workspace, size_t workspace_bytes,
                              void *stream) {
  BnParams P = {};
  int e = bn_common(dtype, num_tiles, N, C, H, W, dy_halo, workspace, workspace_bytes, &P);
  if (e) return e;
  if ((beta_data != 0.f && beta_data != 1.f) || (beta_param != 0.f && beta_param != 1.f)) return ADH_EINVAL;
  if (N == 0 || C == 0 || H == 0 || W == 0) return ADH_OK;
  if (!x_tiles || !dy_tiles || !scale_tiles || !save_mean_tiles || !save_invstd_tiles || !dx_tiles || !dscale_tiles ||
      !dshift_tiles)
    return ADH_ENULL;
  if (relu && !shift_tiles) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!x_tiles[t] || !dy_tiles[t] || !scale_tiles[t] || !save_mean_tiles[t] || !save_invstd_tiles[t] || !dx_tiles[t] ||
        !dscale_tiles[t] || !dshift_tiles[t] || (relu && !shift_tiles[t]))
      return ADH_ENULL;
    if (!aligned_to(x_tiles[t], es) || !aligned_to(dy_tiles[t], es) || !aligned_to(dx_tiles[t], es)) return ADH_EALIGN;
    P.x[t] = x_tiles[t];
    P.dy[t] = dy_tiles[t];
    P.out[t] = dx_tiles[t];
    P.scale[t] = scale_tiles[t];
    P.shift[t] = shift_tiles ? shift_tiles[t] : scale_tiles[t];
    P.mean_in[t] = save_mean_tiles[t];
    P.second_in[t] = save_invstd_tiles[t];
    P.o0[t] = dscale_tiles[t];
    P.o1[t] = dshift_tiles[t];
  }
  P.relu = relu ? 1 : 0;
  // the reduce and apply kernels walk the packed plane in groups of `vec` elements when rows are whole groups
  const uint32_t vec = (uint32_t)(16 / dtype_size(dtype));
  const bool wide = W % vec == 0;
  P.div_cols = FastDiv(wide ? W / vec : W);
  P.div_groups = FastDiv(wide ? H * W / vec : H * W);
  P.planes_per_pass = std::max(1u, 0x7fffffffu / (wide ? H * W / vec : H * W));
  hipStream_t st = as_stream(stream);
  const uint32_t tc = num_tiles * C;
  if (((wide ? H * W / vec : H * W) + kBnThreads - 1u) / kBnThreads > 65535u) return ADH_EINVAL;  // grid.y
  const dim3 rgrid(tc * P.split), agrid = bn_apply_grid(&P, wide ? H * W / vec : H * W);
  P.beta = beta_data;
  P.beta_param = beta_param;
  if (dtype == ADH_F32) {
    if (wide) hipLaunchKernelGGL((bn_reduce_kernel<float, true, 4>), rgrid, dim3(kBnThreads), 0, st, P);
    else hipLaunchKernelGGL((bn_reduce_kernel<float, true, 1>), rgrid, dim3(kBnThreads), 0, st, P);
  } else {
    if (wide) hipLaunchKernelGGL((bn_reduce_kernel<uint16_t, true, 8>), rgrid, dim3(kBnThreads), 0, st, P);
    else hipLaunchKernelGGL((bn_reduce_kernel<uint16_t, true, 1>), rgrid, dim3(kBnThreads), 0, st, P);
  }
  if (dtype == ADH_F32) {
    if (wide) hipLaunchKernelGGL((bn_apply_kernel<float, 2, 4>), agrid, dim3(kBnThreads), 0, st, P);
    else hipLaunchKernelGGL((bn_apply_kernel<float, 2, 1>), agrid, dim3(kBnThreads), 0, st, P);
  } else {
    if (wide) hipLaunchKernelGGL((bn_apply_kernel<uint16_t, 2, 8>), agrid, dim3(kBnThreads), 0, st, P);
    else hipLaunchKernelGGL((bn_apply_kernel<uint16_t, 2, 1>), agrid, dim3(kBnThreads), 0, st, P);
  }
  return launch_status();
}

static uint32_t flat_blocks(uint64_t n) { return (uint32_t)std::min<uint64_t>((n + 1023u) / 1024u, 1u << 20); }

int adh_relu_fwd(int dtype, uint64_t n, const void *x, void *y, void *stream) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if (n == 0) return ADH_OK;
  if (!x || !y) return ADH_ENULL;
  if (!aligned_to(x, dtype_size(dtype)) || !aligned_to(y, dtype_size(dtype))) return ADH_EALIGN;
  if (dtype == ADH_F32)
    hipLaunchKernelGGL(relu_fwd_kernel<float>, dim3(flat_blocks(n)), dim3(256), 0, as_stream(stream), n,
                       reinterpret_cast<const float *>(x), reinterpret_cast<float *>(y));
  else
    hipLaunchKernelGGL(relu_fwd_kernel<uint16_t>, dim3(flat_blocks(n)), dim3(256), 0, as_stream(stream), n,
                       reinterpret_cast<const uint16_t *>(x), reinterpret_cast<uint16_t *>(y));
  return launch_status();
}

int adh_relu_bwd(int dtype, uint64_t n, const void *y, const void *dy, void *dx, float beta, void *stream) {
  if (!dtype_ok(dtype) || (beta != 0.f && beta != 1.f)) return ADH_EINVAL;
  if (n == 0) return ADH_OK;
  if (!y || !dy || !dx) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  if (!aligned_to(y, es) || !aligned_to(dy, es) || !aligned_to(dx, es)) return ADH_EALIGN;
  if (dtype == ADH_F32)
    hipLaunchKernelGGL(relu_bwd_kernel<float>, dim3(flat_blocks(n)), dim3(256), 0, as_stream(stream), n,
                       reinterpret_cast<const float *>(y), reinterpret_cast<const float *>(dy),
                       reinterpret_cast<float *>(dx), beta);
  else
    hipLaunchKernelGGL(relu_bwd_kernel<uint16_t>, dim3(flat_blocks(n)), dim3(256), 0, as_stream(stream), n,
                       reinterpret_cast<const uint16_t *>(y), reinterpret_cast<const uint16_t *>(dy),
                       reinterpret_cast<uint16_t *>(dx), beta);
  return launch_status();
}

int adh_sum_fwd(int dtype, uint32_t num_inputs, uint64_t n, const void *const *xs, void *y, void *stream) {
  if (!dtype_ok(dtype) || num_inputs == 0 || num_inputs > ADH_MAX_TILES) return ADH_EINVAL;
  if (n == 0) return ADH_OK;
  if (!xs || !y) return ADH_ENULL;
  const size_t es = dtype_size(dtype);
  SumParams S = {};
  S.count = num_inputs;
  for (uint32_t k = 0; k < num_inputs; ++k) {
    if (!xs[k]) return ADH_ENULL;
    if (!aligned_to(xs[k], es)) return ADH_EALIGN;
    S.x[k] = xs[k];
  }
  if (!aligned_to(y, es)) return ADH_EALIGN;
  if (dtype == ADH_F32)
    hipLaunchKernelGGL(sum_fwd_kernel<float>, dim3(flat_blocks(n)), dim3(256), 0, as_stream(stream), n, S,
                       reinterpret_cast<float *>(y));
  else
    hipLaunchKernelGGL(sum_fwd_kernel<uint16_t>, dim3(flat_blocks(n)), dim3(256), 0, as_stream(stream), n, S,
                       reinterpret_cast<uint16_t *>(y));
  return launch_status();
}

}  // extern "C"
