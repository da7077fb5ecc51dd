// Flat parameter vectors and the SGD update on them: the device side of the optimizer that drives
// the spatially-parallel graph (include/arraydiff/optimize.hh:262-586 in the reference).
//
// The reference keeps, per rank, flat vectors param / batch_sum_grad / sum_grad / stat ... of
// param_dim (stat_dim) floats.  Every step it (1) copies each parameter and gradient array into
// them one cudaMemcpy at a time (store_val / store_grad, src/op.cc:148-194), (2) sums the
// gradient vectors of all ranks onto rank 0 (ncclReduce, optimize.hh:443-451), (3) runs three
// to five whole-vector axpy kernels (src/kernels/array.cu:97-124) for l2, momentum and the
// parameter update, and (4) copies the result back into every array (load_val).  Here
//   (1), (4) are one launch per vector: a segment table travels in the kernel arguments;
//   (2), (3) are ONE pass: the kernel reads the K gradient vectors, the parameters and the
//            momentum once and writes momentum, parameters and the lagged copy once.
// All of it is HBM-bound streaming; 16-byte accesses, nothing staged.
//
// The arithmetic is fixed (and restated by the CPU oracle) as one fused multiply-add per axpy,
// y <- fma(alpha, x, beta*y), which with beta == 1 is what every use in the optimizer reduces to.
#include "adh_common.h"

// Every multiply-add in this file is either an explicit fma or two separately rounded operations:
// the compiler must not fuse on its own, or the bits would depend on its choices.
#pragma clang fp contract(off)

namespace adh {

constexpr int kOptBlock = 256;
constexpr int kOptUnroll = 4;                                  // float4 per thread per trip
constexpr uint32_t kChunk = kOptBlock * 4 * kOptUnroll;        // floats per workgroup trip
constexpr int kFlatSegs = 48;                                  // segments per launch

struct __attribute__((packed, aligned(4))) UFloat4 {
  float x, y, z, w;
};

// ---------------------------------------------------------------------------
// y = alpha*x + beta*y and y = y + alpha*(x - y)   (src/kernels/array.cu:97-124)
// ---------------------------------------------------------------------------
template <bool ONLINE>
__device__ __forceinline__ float axpy_elem(float alpha, float beta, float x, float y) {
  return ONLINE ? __fmaf_rn(alpha, x - y, y) : __fmaf_rn(alpha, x, beta * y);
}

template <bool ONLINE, bool VEC>
__global__ __launch_bounds__(kOptBlock) void axpy_kernel(uint64_t n, float alpha, float beta, const float *x,
                                                         float *y, float *copy) {
  if (VEC) {
    const uint64_t stride = (uint64_t)gridDim.x * kOptBlock * 4;
    for (uint64_t i = ((uint64_t)blockIdx.x * kOptBlock + threadIdx.x) * 4; i < n; i += stride) {
      if (i + 4 <= n) {
        const float4 a = *reinterpret_cast<const float4 *>(x + i);
        float4 b = *reinterpret_cast<float4 *>(y + i);
        b.x = axpy_elem<ONLINE>(alpha, beta, a.x, b.x);
        b.y = axpy_elem<ONLINE>(alpha, beta, a.y, b.y);
        b.z = axpy_elem<ONLINE>(alpha, beta, a.z, b.z);
        b.w = axpy_elem<ONLINE>(alpha, beta, a.w, b.w);
        *reinterpret_cast<float4 *>(y + i) = b;
        if (copy) *reinterpret_cast<float4 *>(copy + i) = b;
      } else {
        for (uint64_t j = i; j < n; ++j) {
          const float v = axpy_elem<ONLINE>(alpha, beta, x[j], y[j]);
          y[j] = v;
          if (copy) copy[j] = v;
        }
      }
    }
  } else {
    const uint64_t stride = (uint64_t)gridDim.x * kOptBlock;
    for (uint64_t i = (uint64_t)blockIdx.x * kOptBlock + threadIdx.x; i < n; i += stride) {
      const float v = axpy_elem<ONLINE>(alpha, beta, x[i], y[i]);
      y[i] = v;
      if (copy) copy[i] = v;
    }
  }
}

static uint32_t opt_grid(uint64_t n, uint32_t per_thread) {
  uint64_t blocks = (n + (uint64_t)kOptBlock * per_thread - 1) / ((uint64_t)kOptBlock * per_thread);
  const uint64_t cap = 256ull * 16;
  if (blocks > cap) blocks = cap;
  if (blocks == 0) blocks = 1;
  return (uint32_t)blocks;
}

template <bool ONLINE>
static int axpy_launch(uint64_t n, float alpha, float beta, const float *x, float *y, float *copy,
                       hipStream_t stream) {
  if (n == 0) return ADH_OK;
  if (!x || !y) return ADH_ENULL;
  if (!aligned_to(x, 4) || !aligned_to(y, 4) || (copy && !aligned_to(copy, 4))) return ADH_EALIGN;
  const bool vec = aligned_to(x, 16) && aligned_to(y, 16) && (!copy || aligned_to(copy, 16));
  if (vec)
    hipLaunchKernelGGL((axpy_kernel<ONLINE, true>), dim3(opt_grid(n, 4)), dim3(kOptBlock), 0, stream, n, alpha, beta,
                       x, y, copy);
  else
    hipLaunchKernelGGL((axpy_kernel<ONLINE, false>), dim3(opt_grid(n, 1)), dim3(kOptBlock), 0, stream, n, alpha,
                       beta, x, y, copy);
  return launch_status();
}

// ---------------------------------------------------------------------------
// the fused SGD step
// ---------------------------------------------------------------------------
struct SgdParams {
  uint64_t n;
  const float *grads[ADH_MAX_TILES];
  uint32_t num_grads;
  int use_l2, nesterov;
  float l2, mu, neg_step, neg_next_step_mu;
  float *param, *momentum, *lagged, *sum_grad;
};

struct SgdOut {
  float p, m, lag, g;
};

__device__ __forceinline__ SgdOut sgd_elem(const SgdParams &P, float g, float p, float m) {
  if (P.use_l2) g = __fmaf_rn(P.l2, p, g);                 // sum_grad += l2_reg * param
  const float mu_m = P.mu * m;                             // rounded product, then the rounded sum:
  m = g + mu_m;                                            // momentum = fma(1, sum_grad, mu * momentum)
  SgdOut o;
  o.g = g;
  o.m = m;
  if (P.nesterov) {
    const float q = __fmaf_rn(P.neg_step, g, p);           // param -= step * sum_grad
    o.lag = q;                                             // lagged copy taken between the two updates
    o.p = __fmaf_rn(P.neg_next_step_mu, m, q);             // param -= next_step * mu * momentum
  } else {
    o.p = __fmaf_rn(P.neg_step, m, p);                     // param -= step * momentum
    o.lag = o.p;
  }
  return o;
}

// KG > 0: exactly KG gradient vectors, all of whose loads are issued before the first add (a loop over a
// run-time count waits for each vector in turn); KG = 0: any count.
template <bool VEC, int KG>
__global__ __launch_bounds__(kOptBlock) void sgd_step_kernel(SgdParams P) {
  if (VEC) {
    const uint64_t stride = (uint64_t)gridDim.x * kOptBlock * 4;
    for (uint64_t i = ((uint64_t)blockIdx.x * kOptBlock + threadIdx.x) * 4; i < P.n; i += stride) {
      if (i + 4 <= P.n) {
        float4 g;
        if constexpr (KG > 0) {
          float4 gv[KG];
#pragma unroll
          for (int r = 0; r < KG; ++r) gv[r] = *reinterpret_cast<const float4 *>(P.grads[r] + i);
          g = gv[0];
#pragma unroll
          for (int r = 1; r < KG; ++r) {                     // rank order: the result does not depend on timing
            g.x += gv[r].x; g.y += gv[r].y; g.z += gv[r].z; g.w += gv[r].w;
          }
        } else {
          g = *reinterpret_cast<const float4 *>(P.grads[0] + i);
          for (uint32_t r = 1; r < P.num_grads; ++r) {
            const float4 h = *reinterpret_cast<const float4 *>(P.grads[r] + i);
            g.x += h.x; g.y += h.y; g.z += h.z; g.w += h.w;
          }
        }
        const float4 p = *reinterpret_cast<const float4 *>(P.param + i);
        const float4 m = *reinterpret_cast<const float4 *>(P.momentum + i);
        const SgdOut a = sgd_elem(P, g.x, p.x, m.x), b = sgd_elem(P, g.y, p.y, m.y);
        const SgdOut c = sgd_elem(P, g.z, p.z, m.z), d = sgd_elem(P, g.w, p.w, m.w);
        *reinterpret_cast<float4 *>(P.momentum + i) = make_float4(a.m, b.m, c.m, d.m);
        *reinterpret_cast<float4 *>(P.param + i) = make_float4(a.p, b.p, c.p, d.p);
        if (P.lagged) *reinterpret_cast<float4 *>(P.lagged + i) = make_float4(a.lag, b.lag, c.lag, d.lag);
        if (P.sum_grad) *reinterpret_cast<float4 *>(P.sum_grad + i) = make_float4(a.g, b.g, c.g, d.g);
      } else {
        for (uint64_t j = i; j < P.n; ++j) {
          float g = P.grads[0][j];
          for (uint32_t r = 1; r < P.num_grads; ++r) g += P.grads[r][j];
          const SgdOut o = sgd_elem(P, g, P.param[j], P.momentum[j]);
          P.momentum[j] = o.m;
          P.param[j] = o.p;
          if (P.lagged) P.lagged[j] = o.lag;
          if (P.sum_grad) P.sum_grad[j] = o.g;
        }
      }
    }
  } else {
    const uint64_t stride = (uint64_t)gridDim.x * kOptBlock;
    for (uint64_t j = (uint64_t)blockIdx.x * kOptBlock + threadIdx.x; j < P.n; j += stride) {
      float g = P.grads[0][j];
      for (uint32_t r = 1; r < P.num_grads; ++r) g += P.grads[r][j];
      const SgdOut o = sgd_elem(P, g, P.param[j], P.momentum[j]);
      P.momentum[j] = o.m;
      P.param[j] = o.p;
      if (P.lagged) P.lagged[j] = o.lag;
      if (P.sum_grad) P.sum_grad[j] = o.g;
    }
  }
}

// ---------------------------------------------------------------------------
// many arrays <-> one flat vector
// ---------------------------------------------------------------------------
struct FlatSegTable {
  const float *array[kFlatSegs];
  uint64_t flat_off[kFlatSegs];        // element offset of the segment inside the flat vector
  uint32_t len[kFlatSegs];             // elements (< 2^31 per array)
  uint32_t first_block[kFlatSegs + 1]; // workgroups [first_block[s], first_block[s+1]) serve segment s
  uint32_t count;
};

// One workgroup moves up to kChunk consecutive floats of one segment.  The array side is 16-byte
// aligned when VEC (checked on the host); the flat side sits at an arbitrary element offset and is
// accessed through an element-aligned 16-byte type.
template <bool TO_FLAT, bool VEC>
__global__ __launch_bounds__(kOptBlock) void flat_copy_kernel(FlatSegTable T, float *flat) {
  const uint32_t b = blockIdx.x;
  uint32_t lo = 0, hi = T.count;  // binary search, uniform over the workgroup
  while (hi - lo > 1) {
    const uint32_t mid = (lo + hi) >> 1;
    if (T.first_block[mid] <= b) lo = mid; else hi = mid;
  }
  const uint32_t s = lo;
  const uint32_t len = T.len[s];
  const uint32_t begin = (b - T.first_block[s]) * kChunk;
  const uint32_t end = min(len, begin + kChunk);
  float *arr = const_cast<float *>(T.array[s]);
  float *fl = flat + T.flat_off[s];
  if (VEC) {
#pragma unroll
    for (int u = 0; u < kOptUnroll; ++u) {
      const uint32_t i = begin + (u * kOptBlock + threadIdx.x) * 4;
      if (i + 4 <= end) {
        if (TO_FLAT) {
          const float4 v = *reinterpret_cast<const float4 *>(arr + i);
          UFloat4 o; o.x = v.x; o.y = v.y; o.z = v.z; o.w = v.w;
          *reinterpret_cast<UFloat4 *>(fl + i) = o;
        } else {
          const UFloat4 v = *reinterpret_cast<const UFloat4 *>(fl + i);
          *reinterpret_cast<float4 *>(arr + i) = make_float4(v.x, v.y, v.z, v.w);
        }
      } else {
        for (uint32_t j = i; j < end; ++j) {
          if (TO_FLAT) fl[j] = arr[j]; else arr[j] = fl[j];
        }
      }
    }
  } else {
    for (uint32_t j = begin + threadIdx.x; j < end; j += kOptBlock) {
      if (TO_FLAT) fl[j] = arr[j]; else arr[j] = fl[j];
    }
  }
}

template <bool TO_FLAT>
static int flat_copy(uint32_t num, const float *const *arrays, const uint64_t *lens, uint64_t flat_offset,
                     float *flat, hipStream_t stream) {
  if (num == 0) return ADH_OK;
  if (!arrays || !lens || !flat) return ADH_ENULL;
  if (!aligned_to(flat, 4)) return ADH_EALIGN;
  for (uint32_t s = 0; s < num; ++s) {
    if (lens[s] >= (1ull << 31)) return ADH_EINVAL;
    if (lens[s] && !arrays[s]) return ADH_ENULL;
    if (!aligned_to(arrays[s], 4)) return ADH_EALIGN;
  }
  uint64_t off = flat_offset;
  uint32_t s = 0;
  while (s < num) {
    FlatSegTable T;
    T.count = 0;
    uint32_t blocks = 0;
    bool vec = true;
    while (s < num && T.count < (uint32_t)kFlatSegs) {
      const uint64_t len = lens[s];
      if (len) {
        const uint32_t c = T.count++;
        T.array[c] = arrays[s];
        T.flat_off[c] = off;
        T.len[c] = (uint32_t)len;
        T.first_block[c] = blocks;
        blocks += (uint32_t)((len + kChunk - 1) / kChunk);
        vec = vec && aligned_to(arrays[s], 16);
      }
      off += len;
      ++s;
    }
    if (T.count == 0) continue;
    T.first_block[T.count] = blocks;
    for (uint32_t c = T.count; c < (uint32_t)kFlatSegs; ++c) {
      T.array[c] = nullptr; T.flat_off[c] = 0; T.len[c] = 0; T.first_block[c + 1] = blocks;
    }
    if (vec)
      hipLaunchKernelGGL((flat_copy_kernel<TO_FLAT, true>), dim3(blocks), dim3(kOptBlock), 0, stream, T, flat);
    else
      hipLaunchKernelGGL((flat_copy_kernel<TO_FLAT, false>), dim3(blocks), dim3(kOptBlock), 0, stream, T, flat);
    const int st = launch_status();
    if (st != ADH_OK) return st;
  }
  return ADH_OK;
}

}  // namespace adh

using namespace adh;

extern "C" {

int adh_scale_add_f32(uint64_t n, float alpha, const float *x, float beta, float *y, void *stream) {
  return axpy_launch<false>(n, alpha, beta, x, y, nullptr, as_stream(stream));
}

int adh_add_online_f32(uint64_t n, float alpha, const float *x, float *y, void *stream) {
  return axpy_launch<true>(n, alpha, 0.f, x, y, nullptr, as_stream(stream));
}

int adh_stat_step_f32(uint64_t n, float rate, const float *avg_stat, float *running_stat, float *stat,
                      void *stream) {
  if (n && !stat) return ADH_ENULL;
  return axpy_launch<true>(n, rate, 0.f, avg_stat, running_stat, stat, as_stream(stream));
}

int adh_flat_store_f32(uint32_t num_arrays, const float *const *arrays, const uint64_t *lens, uint64_t flat_offset,
                       float *flat, void *stream) {
  return flat_copy<true>(num_arrays, arrays, lens, flat_offset, flat, as_stream(stream));
}

int adh_flat_load_f32(uint32_t num_arrays, float *const *arrays, const uint64_t *lens, uint64_t flat_offset,
                      const float *flat, void *stream) {
  return flat_copy<false>(num_arrays, arrays, lens, flat_offset, const_cast<float *>(flat), as_stream(stream));
}

int adh_sgd_step_f32(uint64_t n, uint32_t num_grads, const float *const *grads, float l2_reg, float momentum,
                     float step_size, float next_step_size, int nesterov, float *param, float *momentum_grad,
                     float *lagged_param, float *sum_grad, void *stream) {
  if (n == 0) return ADH_OK;
  if (num_grads == 0 || num_grads > ADH_MAX_TILES) return ADH_EINVAL;
  if (!grads || !param || !momentum_grad) return ADH_ENULL;
  SgdParams P;
  P.n = n;
  P.num_grads = num_grads;
  bool vec = aligned_to(param, 16) && aligned_to(momentum_grad, 16) && (!lagged_param || aligned_to(lagged_param, 16)) &&
             (!sum_grad || aligned_to(sum_grad, 16));
  if (!aligned_to(param, 4) || !aligned_to(momentum_grad, 4) || !aligned_to(lagged_param, 4) || !aligned_to(sum_grad, 4))
    return ADH_EALIGN;
  for (uint32_t r = 0; r < ADH_MAX_TILES; ++r) {
    P.grads[r] = r < num_grads ? grads[r] : nullptr;
    if (r < num_grads) {
      if (!grads[r]) return ADH_ENULL;
      if (!aligned_to(grads[r], 4)) return ADH_EALIGN;
      vec = vec && aligned_to(grads[r], 16);
      // the gradient vectors are read while the outputs are written: they must not be the outputs,
      // except that sum_grad may be grads[0] (every element is read before it is written)
      if (grads[r] == param || grads[r] == momentum_grad || grads[r] == lagged_param) return ADH_EINVAL;
      if (r > 0 && grads[r] == sum_grad) return ADH_EINVAL;
    }
  }
  P.use_l2 = l2_reg != 0.f;
  P.nesterov = nesterov != 0;
  P.l2 = l2_reg;
  P.mu = momentum;
  P.neg_step = -step_size;
  P.neg_next_step_mu = -next_step_size * momentum;
  P.param = param;
  P.momentum = momentum_grad;
  P.lagged = lagged_param;
  P.sum_grad = sum_grad;
  const dim3 grid(opt_grid(n, vec ? 4 : 1)), block(kOptBlock);
  if (!vec)
    hipLaunchKernelGGL((sgd_step_kernel<false, 0>), grid, block, 0, as_stream(stream), P);
  else if (num_grads == 1)
    hipLaunchKernelGGL((sgd_step_kernel<true, 1>), grid, block, 0, as_stream(stream), P);
  else if (num_grads == 2)
    hipLaunchKernelGGL((sgd_step_kernel<true, 2>), grid, block, 0, as_stream(stream), P);
  else if (num_grads == 4)
    hipLaunchKernelGGL((sgd_step_kernel<true, 4>), grid, block, 0, as_stream(stream), P);
  else if (num_grads == 8)
    hipLaunchKernelGGL((sgd_step_kernel<true, 8>), grid, block, 0, as_stream(stream), P);
  else
    hipLaunchKernelGGL((sgd_step_kernel<true, 0>), grid, block, 0, as_stream(stream), P);
  return launch_status();
}

}  // extern "C"
