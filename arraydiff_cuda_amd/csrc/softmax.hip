// Row-wise softmax and negative log likelihood for gfx950.
//
// A workgroup of four wavefronts owns one row: the row is read once into registers (up to
// 2048 classes, 8 per thread; longer rows are re-read from cache), the max and the sum are
// reduced with cross-lane shuffles inside each wavefront and combined across the four through
// 16 bytes of LDS, and y is written once.  A row of 1000 fp32 logits is 4 KB, so the kernel is
// latency bound: four waves per row shorten every thread's chain of loads, exponentials and
// divisions to a quarter of what one wave per row had (256 x 1000: 4.0 -> 3.5 us per launch).
#include <math.h>

#include "adh_common.h"

namespace adh {

static constexpr int kWave = 64;
static constexpr int kRowThreads = 256;  // four wavefronts per row
static constexpr int kCached = 8;        // register-cached elements per thread -> rows up to 2048

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// y = softmax(x) per row; if LOSS, also loss[row] = -logf(y[row, label[row]]) computed
// from the rounded fp32 y, i.e. exactly what a separate nll pass over y would produce.
// max / sum over the workgroup: shuffles inside a wavefront, then the four partial results through LDS
__device__ __forceinline__ float block_max(float v, float *red) {
  v = wave_max(v);
  if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = v;
  __syncthreads();
  v = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  return v;
}
__device__ __forceinline__ float block_sum(float v, float *red) {
  v = wave_sum(v);
  if ((threadIdx.x & (kWave - 1)) == 0) red[threadIdx.x / kWave] = v;
  __syncthreads();
  v = (red[0] + red[1]) + (red[2] + red[3]);
  __syncthreads();
  return v;
}

// beta*old + dl*(y - [at the label]) with every product and sum rounded on its own (no fused multiply-add), so
// that the fused kernel and the separate one give the same bits
__device__ __forceinline__ float nll_grad(float dl, float yv, bool at_label, float beta, float old) {
  const float g = __fmul_rn(dl, at_label ? __fsub_rn(yv, 1.0f) : yv);
  return beta != 0.f ? __fadd_rn(old, g) : g;
}

// the gradient of the loss with respect to the logits, written in the same pass (GRAD):
// dx[row, j] = beta * dx[row, j] + g * (y - [j == label]), g = dloss ? dloss[row] : dloss_all,
// evaluated like nll_loss_bwd_kernel below
struct RowGrad {
  const float *dloss;
  float dloss_all;
  float beta;
  float *dx;
};

template <bool LOSS, bool GRAD>
__global__ __launch_bounds__(kRowThreads) void softmax_row_kernel(uint32_t C, uint32_t N, const float *__restrict__ x,
                                                           const uint32_t *__restrict__ label,
                                                           float *__restrict__ y, float *__restrict__ loss,
                                                           const RowGrad G) {
  __shared__ float red[kRowThreads / kWave];
  const uint32_t row = blockIdx.x;
  const uint32_t lane = threadIdx.x;
  if (row >= N) return;
  const float *xr = x + (uint64_t)row * C;
  float *yr = y + (uint64_t)row * C;
  float *dxr = GRAD ? G.dx + (uint64_t)row * C : nullptr;
  const float dl = GRAD ? (G.dloss ? G.dloss[row] : G.dloss_all) : 0.f;
  auto grad = [&](uint32_t j, float yv, uint32_t lab) {
    dxr[j] = nll_grad(dl, yv, lab == j, G.beta, dxr[j]);
  };
  const bool cached = C <= (uint32_t)(kRowThreads * kCached);
  float v[kCached];
  float m = -INFINITY;
  if (cached) {
#pragma unroll
    for (int k = 0; k < kCached; ++k) {
      const uint32_t j = lane + k * kRowThreads;
      v[k] = j < C ? xr[j] : -INFINITY;
      m = fmaxf(m, v[k]);
    }
  } else {
    for (uint32_t j = lane; j < C; j += kRowThreads) m = fmaxf(m, xr[j]);
  }
  m = block_max(m, red);
  float s = 0.f;
  if (cached) {
#pragma unroll
    for (int k = 0; k < kCached; ++k) {
      v[k] = expf(v[k] - m);  // exp(-inf) = 0 for the padding lanes
      s += v[k];
    }
  } else {
    for (uint32_t j = lane; j < C; j += kRowThreads) s += expf(xr[j] - m);
  }
  s = block_sum(s, red);
  const uint32_t lab = LOSS ? label[row] : 0u;
  if (cached) {
#pragma unroll
    for (int k = 0; k < kCached; ++k) {
      const uint32_t j = lane + k * kRowThreads;
      if (j < C) {
        const float yv = v[k] / s;
        yr[j] = yv;
        if (LOSS && j == lab) loss[row] = -logf(yv);
        if (GRAD) grad(j, yv, lab);
      }
    }
  } else {
    for (uint32_t j = lane; j < C; j += kRowThreads) {
      const float yv = expf(xr[j] - m) / s;
      yr[j] = yv;
      if (LOSS && j == lab) loss[row] = -logf(yv);
      if (GRAD) grad(j, yv, lab);
    }
  }
  if (LOSS && lab >= C && lane == 0) loss[row] = NAN;  // label outside [0, C)
}

__global__ __launch_bounds__(256) void nll_loss_fwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ y,
                                                          const uint32_t *__restrict__ label,
                                                          float *__restrict__ loss) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i >= N) return;
  const uint32_t lab = label[i];
  loss[i] = lab < C ? -logf(y[lab + (uint64_t)C * i]) : NAN;
}

// dx[i,j] = beta*dx[i,j] + dl * (y[i,j] - [j == label[i]]), dl = dloss ? dloss[i] : dloss_all, beta 0 or 1;
// grid = (chunks of a row, rows)
__global__ __launch_bounds__(256) void nll_loss_bwd_kernel(uint32_t C, uint32_t N, const float *__restrict__ y,
                                                          const uint32_t *__restrict__ label,
                                                          const float *__restrict__ dloss, float dloss_all, float beta,
                                                          float *__restrict__ dx) {
  const uint32_t j = blockIdx.x * 256 + threadIdx.x;
  const uint32_t i = blockIdx.y;
  if (j >= C || i >= N) return;
  const uint64_t idx = (uint64_t)i * C + j;
  const float yv = y[idx];
  const float dl = dloss ? dloss[i] : dloss_all;
  dx[idx] = nll_grad(dl, yv, label[i] == j, beta, dx[idx]);
}

static int nll_loss_bwd(uint32_t C, uint32_t N, const float *y, const uint32_t *label, const float *dloss, float dloss_all,
                        float beta, float *dx, hipStream_t st) {
  // rows beyond the grid.y limit: split the launch
  for (uint32_t i0 = 0; i0 < N; i0 += 65535u) {
    const uint32_t rows = (N - i0) < 65535u ? (N - i0) : 65535u;
    hipLaunchKernelGGL(nll_loss_bwd_kernel, dim3((C + 255) / 256, rows), dim3(256), 0, st, C, rows, y + (uint64_t)i0 * C,
                       label + i0, dloss ? dloss + i0 : nullptr, dloss_all, beta, dx + (uint64_t)i0 * C);
  }
  return launch_status();
}

}  // namespace adh

using namespace adh;

extern "C" {

int adh_softmax_fwd(uint32_t C, uint32_t N, const float *x, float *y, void *stream) {
  if (C == 0 || N == 0) return ADH_OK;
  if (!x || !y) return ADH_ENULL;
  if (!aligned_to(x, 4) || !aligned_to(y, 4)) return ADH_EALIGN;
  if (x == y && C > 2048u) return ADH_EINVAL;  // rows past 2048 classes are read again after y is written
  hipLaunchKernelGGL((softmax_row_kernel<false, false>), dim3(N), dim3(kRowThreads), 0, as_stream(stream), C, N, x,
                     (const uint32_t *)nullptr, y, (float *)nullptr, RowGrad{});
  return launch_status();
}

int adh_softmax_xent_fwd(uint32_t C, uint32_t N, const float *x, const uint32_t *label, float *y, float *loss,
                         void *stream) {
  if (C == 0 || N == 0) return ADH_OK;
  if (!x || !y || !label || !loss) return ADH_ENULL;
  if (!aligned_to(x, 4) || !aligned_to(y, 4) || !aligned_to(label, 4) || !aligned_to(loss, 4)) return ADH_EALIGN;
  if (x == y && C > 2048u) return ADH_EINVAL;
  hipLaunchKernelGGL((softmax_row_kernel<true, false>), dim3(N), dim3(kRowThreads), 0, as_stream(stream), C, N, x, label, y,
                     loss, RowGrad{});
  return launch_status();
}

int adh_softmax_xent_fwd_bwd(uint32_t C, uint32_t N, const float *x, const uint32_t *label, const float *dloss,
                             float dloss_all, float *y, float *loss, float beta, float *dx, void *stream) {
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (C == 0 || N == 0) return ADH_OK;
  if (!x || !y || !label || !loss || !dx) return ADH_ENULL;
  if (!aligned_to(x, 4) || !aligned_to(y, 4) || !aligned_to(label, 4) || !aligned_to(loss, 4) || !aligned_to(dx, 4) ||
      !aligned_to(dloss, 4))
    return ADH_EALIGN;
  if (x == y && C > 2048u) return ADH_EINVAL;
  if (dx == y || (dx == x && C > 2048u)) return ADH_EINVAL;  // y is an output of its own; long rows re-read x
  RowGrad G = {dloss, dloss_all, beta, dx};
  hipLaunchKernelGGL((softmax_row_kernel<true, true>), dim3(N), dim3(kRowThreads), 0, as_stream(stream), C, N, x, label, y,
                     loss, G);
  return launch_status();
}

int adh_softmax_nll_loss_fwd(uint32_t C, uint32_t N, const float *y, const uint32_t *label, float *loss,
                             void *stream) {
  if (C == 0 || N == 0) return ADH_OK;
  if (!y || !label || !loss) return ADH_ENULL;
  if (!aligned_to(y, 4) || !aligned_to(label, 4) || !aligned_to(loss, 4)) return ADH_EALIGN;
  hipLaunchKernelGGL(nll_loss_fwd_kernel, dim3((N + 255) / 256), dim3(256), 0, as_stream(stream), C, N, y, label,
                     loss);
  return launch_status();
}

int adh_softmax_nll_loss_bwd(uint32_t C, uint32_t N, const float *y, const uint32_t *label, const float *dloss,
                             float *dx, void *stream) {
  if (C == 0 || N == 0) return ADH_OK;
  if (!y || !label || !dloss || !dx) return ADH_ENULL;
  if (!aligned_to(y, 4) || !aligned_to(label, 4) || !aligned_to(dloss, 4) || !aligned_to(dx, 4)) return ADH_EALIGN;
  return nll_loss_bwd(C, N, y, label, dloss, 0.f, 1.f, dx, as_stream(stream));
}

int adh_softmax_nll_loss_bwd_scaled(uint32_t C, uint32_t N, const float *y, const uint32_t *label, const float *dloss,
                                    float dloss_all, float beta, float *dx, void *stream) {
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (C == 0 || N == 0) return ADH_OK;
  if (!y || !label || !dx) return ADH_ENULL;
  if (!aligned_to(y, 4) || !aligned_to(label, 4) || !aligned_to(dloss, 4) || !aligned_to(dx, 4)) return ADH_EALIGN;
  return nll_loss_bwd(C, N, y, label, dloss, dloss_all, beta, dx, as_stream(stream));
}

}  // extern "C"
