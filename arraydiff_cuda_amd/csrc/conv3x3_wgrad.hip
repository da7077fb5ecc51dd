// Backward-filter of the 3x3 slab convolution on the gfx950 matrix cores (fp32 MFMA):
//   dw[co][ci][a][b] = beta*dw + sum_{tile,n,h,w} dy[n][co][h][w] * x_pad[n][ci][h+a][w+b]
//
// GEMM view: D[co][ci] (one 16x16 tile per tap) += A[co][pixel] * B[pixel][ci], the reduction
// runs over pixels, 4 consecutive pixels of one row per v_mfma_f32_16x16x4_f32.
//   * a workgroup (4 waves) owns a run of output rows of one image and ALL 64 x 64 x 9
//     filter taps: wave v owns output channels [16v,16v+16) x 4 ci-tiles x 9 taps = 36
//     accumulator tiles (144 accumulator registers), so dy is read once per workgroup and
//     every A operand feeds 36 MFMAs.
//   * rows stream through LDS: the slab rows live in a 4-slot ring (row y in slot y%4), so
//     each new output row loads exactly one new slab row and one dy row while the previous
//     row is being multiplied; channel strides are 4 (mod 64) so the 16 channels x 4 pixels
//     of one operand read hit 64 different banks.
//   * every workgroup writes its partial 64x64x9 block to the workspace and a second kernel
//     sums the partials in a fixed order: the result is deterministic (no float atomics).
#include "adh_common.h"

namespace adh {

typedef float floatx4 __attribute__((ext_vector_type(4)));

static constexpr int kWgThreads = 256;
static constexpr int kPitch = 64;                 // floats per staged row
static constexpr int kXStride = 4 * kPitch + 4;   // slab ring: 4 rows per channel, == 4 (mod 64)
static constexpr int kDStride = 2 * kPitch + 4;   // dy double buffer: 2 rows per channel
// the last k-step reads columns up to 4*ceil(W/4)+1, which must stay inside the row
static constexpr int kMaxW = kPitch - 4;

struct WgradParams {
  const float *x[ADH_MAX_TILES];
  const float *dy[ADH_MAX_TILES];
  float *partial;            // [num_blocks][64*64*9] in (co, ci, tap) order, co/ci local to the group
  uint32_t num_tiles, N, Cin, Cout, H, W;
  uint32_t rows_per_block, chunks_per_plane;  // grid.x = chunks_per_plane * N * num_tiles
  uint32_t ci_groups;        // grid.y = ci_groups * co_groups
  FastDiv div_chunks, div_tiles, div_ci_groups;
};

__global__ __launch_bounds__(kWgThreads, 1) void conv3x3_wgrad_f32_kernel(const WgradParams P) {
  __shared__ float xs[64 * kXStride];
  __shared__ float dys[64 * kDStride];

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u, wv = tid >> 6, g = lane >> 4, l16 = lane & 15u;

  uint32_t plane, chunk;
  P.div_chunks.divmod(blockIdx.x, plane, chunk);
  uint32_t n, t;
  P.div_tiles.divmod(plane, n, t);
  uint32_t cog, cig;
  P.div_ci_groups.divmod(blockIdx.y, cog, cig);
  const uint32_t r0 = chunk * P.rows_per_block;
  const uint32_t r1 = min(r0 + P.rows_per_block, P.H);
  const uint32_t WP = P.W + 2u, HP = P.H + 2u;
  const uint32_t ci0 = cig * 64u, co0 = cog * 64u;
  const float *__restrict__ x = P.x[t] + ((uint64_t)n * P.Cin) * HP * WP;
  const float *__restrict__ dy = P.dy[t] + ((uint64_t)n * P.Cout) * P.H * P.W;

  // ---- staging: lane = column, wave v loads channels v, v+4, ... (16 per row) ----
  const bool xcol_ok = lane < WP;
  const bool dcol_ok = lane < P.W;
  float xst[16], dst_[16];
  auto load_x_row = [&](uint32_t y) {  // slab row y (clamped; masked at store)
    const uint32_t off = min(y, HP - 1u) * WP + (xcol_ok ? lane : 0u);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const uint32_t ci = min(ci0 + wv + 4u * i, P.Cin - 1u);
      xst[i] = x[(uint64_t)ci * HP * WP + off];
    }
  };
  auto store_x_row = [&](uint32_t y) {
    const bool row_ok = xcol_ok && y < HP;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const uint32_t cl = wv + 4u * i;
      xs[cl * kXStride + (y & 3u) * kPitch + lane] = (row_ok && ci0 + cl < P.Cin) ? xst[i] : 0.f;
    }
  };
  auto load_dy_row = [&](uint32_t r) {
    const uint32_t off = min(r, P.H - 1u) * P.W + (dcol_ok ? lane : 0u);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const uint32_t co = min(co0 + wv + 4u * i, P.Cout - 1u);
      dst_[i] = dy[(uint64_t)co * P.H * P.W + off];
    }
  };
  auto store_dy_row = [&](uint32_t r) {
    const bool row_ok = dcol_ok && r < r1;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const uint32_t cl = wv + 4u * i;
      dys[cl * kDStride + (r & 1u) * kPitch + lane] = (row_ok && co0 + cl < P.Cout) ? dst_[i] : 0.f;
    }
  };

  floatx4 acc[4][9];
#pragma unroll
  for (int ct = 0; ct < 4; ++ct)
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) acc[ct][tap] = floatx4{0.f, 0.f, 0.f, 0.f};

  // prologue: slab rows r0, r0+1, r0+2 and dy row r0
  load_x_row(r0);
  store_x_row(r0);
  load_x_row(r0 + 1);
  store_x_row(r0 + 1);
  load_x_row(r0 + 2);
  load_dy_row(r0);
  store_x_row(r0 + 2);
  store_dy_row(r0);
  __syncthreads();

  const uint32_t ksteps = (P.W + 3u) / 4u;
  const uint32_t a_lane = (16u * wv + l16) * kDStride + g;
  const uint32_t b_lane = l16 * kXStride + g;

  for (uint32_t r = r0; r < r1; ++r) {
    const bool more = r + 1 < r1;  // uniform
    if (more) {
      load_x_row(r + 3);
      load_dy_row(r + 1);
    }
    const float *arow = dys + a_lane + (r & 1u) * kPitch;
    const float *brow0 = xs + b_lane + ((r + 0u) & 3u) * kPitch;
    const float *brow1 = xs + b_lane + ((r + 1u) & 3u) * kPitch;
    const float *brow2 = xs + b_lane + ((r + 2u) & 3u) * kPitch;
#pragma unroll 2
    for (uint32_t ks = 0; ks < ksteps; ++ks) {
      const float a = arow[4u * ks];
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
#pragma unroll
        for (int kw = 0; kw < 3; ++kw) {
          const float b0 = brow0[ct * 16 * kXStride + 4u * ks + kw];
          const float b1 = brow1[ct * 16 * kXStride + 4u * ks + kw];
          const float b2 = brow2[ct * 16 * kXStride + 4u * ks + kw];
          acc[ct][0 + kw] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b0, acc[ct][0 + kw], 0, 0, 0);
          acc[ct][3 + kw] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b1, acc[ct][3 + kw], 0, 0, 0);
          acc[ct][6 + kw] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b2, acc[ct][6 + kw], 0, 0, 0);
        }
      }
    }
    if (more) {
      store_x_row(r + 3);   // slot (r+3)%4 held row r-1, last read one barrier ago
      store_dy_row(r + 1);
    }
    __syncthreads();
  }

  // ---- epilogue: lane holds D[co = 4g+i][ci = l16] of each (ct, tap) tile ----
  const uint32_t block_lin = blockIdx.y * gridDim.x + blockIdx.x;
  float *__restrict__ part = P.partial + (uint64_t)block_lin * (64u * 64u * 9u);
#pragma unroll
  for (int ct = 0; ct < 4; ++ct)
#pragma unroll
    for (int tap = 0; tap < 9; ++tap)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t co_l = 16u * wv + 4u * g + i, ci_l = 16u * ct + l16;
        part[(co_l * 64u + ci_l) * 9u + tap] = acc[ct][tap][i];
      }
}

// dw[co][ci][tap] = beta*dw + sum over the pixel-chunk partials of its (co,ci) group, in
// block order (deterministic).
struct WgradReduceParams {
  const float *partial;
  float *dw;
  uint32_t Cin, Cout, blocks_x, ci_groups;
  float beta;
  FastDiv div9, div_cin;
};

__global__ __launch_bounds__(256) void conv3x3_wgrad_reduce_kernel(const WgradReduceParams P) {
  const uint32_t e = blockIdx.x * 256u + threadIdx.x;
  if (e >= P.Cout * P.Cin * 9u) return;
  uint32_t cc, tap, co, ci;
  P.div9.divmod(e, cc, tap);
  P.div_cin.divmod(cc, co, ci);
  const uint32_t grp = (co >> 6) * P.ci_groups + (ci >> 6);
  const uint32_t local = (((co & 63u) * 64u) + (ci & 63u)) * 9u + tap;
  const float *p = P.partial + ((uint64_t)grp * P.blocks_x) * (64u * 64u * 9u) + local;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  uint32_t b = 0;
  for (; b + 4 <= P.blocks_x; b += 4) {
    s0 += p[(uint64_t)(b + 0) * 36864u];
    s1 += p[(uint64_t)(b + 1) * 36864u];
    s2 += p[(uint64_t)(b + 2) * 36864u];
    s3 += p[(uint64_t)(b + 3) * 36864u];
  }
  for (; b < P.blocks_x; ++b) s0 += p[(uint64_t)b * 36864u];
  float s = (s0 + s1) + (s2 + s3);
  if (P.beta != 0.f) s += P.beta * P.dw[e];
  P.dw[e] = s;
}

struct WgradPlan {
  uint32_t rows_per_block, chunks_per_plane, blocks_x, groups;
  size_t workspace_bytes;
};

static bool wgrad_plan(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                       WgradPlan *plan) {
  if (W > (uint32_t)kMaxW) return false;
  const uint64_t planes = (uint64_t)num_tiles * N;
  const uint32_t groups = ((Cin + 63u) / 64u) * ((Cout + 63u) / 64u);
  // aim at >= 256 workgroups (one per CU) with as few partial blocks as that allows
  uint32_t chunks = 1;
  while (planes * chunks * groups < 256 && chunks < H) ++chunks;
  uint32_t rows = (H + chunks - 1) / chunks;
  chunks = (H + rows - 1) / rows;
  if (planes * chunks > 0x7fffffffull) return false;
  plan->rows_per_block = rows;
  plan->chunks_per_plane = chunks;
  plan->blocks_x = (uint32_t)(planes * chunks);
  plan->groups = groups;
  plan->workspace_bytes = (size_t)plan->blocks_x * groups * 36864u * sizeof(float);
  return true;
}

}  // namespace adh

using namespace adh;

extern "C" {

size_t adh_conv3x3_workspace_bytes(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                   uint32_t H, uint32_t W) {
  if (which != ADH_CONV_BWD_FILTER || dtype != ADH_F32) return 0;
  if (num_tiles == 0 || N == 0 || Cin == 0 || Cout == 0 || H == 0 || W == 0) return 0;
  WgradPlan plan;
  if (!wgrad_plan(num_tiles, N, Cin, Cout, H, W, &plan)) return 0;
  return plan.workspace_bytes;
}

int adh_conv3x3_slab_bwd_filter_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                      uint32_t H, uint32_t W, const void *const *x_pad_tiles,
                                      const void *const *dy_tiles, float *dw, float beta, void *workspace,
                                      size_t workspace_bytes, void *stream) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if (dtype != ADH_F32) return ADH_EUNIMPL;
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (Cin == 0 || Cout == 0) return ADH_OK;
  if (!dw) return ADH_ENULL;
  if (!aligned_to(dw, 4)) return ADH_EALIGN;
  hipStream_t st = as_stream(stream);
  if (N == 0 || H == 0 || W == 0) {
    // empty sum: dw = beta * dw
    if (beta == 0.f) return adh_fill_f32((uint64_t)Cin * Cout * 9u, 0.f, dw, stream);
    return ADH_OK;
  }
  if (!x_pad_tiles || !dy_tiles) return ADH_ENULL;
  WgradPlan plan;
  if (!wgrad_plan(num_tiles, N, Cin, Cout, H, W, &plan)) return ADH_EUNIMPL;
  if (!workspace) return ADH_ENULL;
  if (!aligned_to(workspace, 4)) return ADH_EALIGN;
  if (workspace_bytes < plan.workspace_bytes) return ADH_EWORKSPACE;
  WgradParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!x_pad_tiles[t] || !dy_tiles[t]) return ADH_ENULL;
    if (!aligned_to(x_pad_tiles[t], 4) || !aligned_to(dy_tiles[t], 4)) return ADH_EALIGN;
    P.x[t] = reinterpret_cast<const float *>(x_pad_tiles[t]);
    P.dy[t] = reinterpret_cast<const float *>(dy_tiles[t]);
  }
  P.partial = reinterpret_cast<float *>(workspace);
  P.num_tiles = num_tiles; P.N = N; P.Cin = Cin; P.Cout = Cout; P.H = H; P.W = W;
  P.rows_per_block = plan.rows_per_block;
  P.chunks_per_plane = plan.chunks_per_plane;
  P.ci_groups = (Cin + 63u) / 64u;
  P.div_chunks = FastDiv(plan.chunks_per_plane);
  P.div_tiles = FastDiv(num_tiles);
  P.div_ci_groups = FastDiv(P.ci_groups);
  dim3 grid(plan.blocks_x, plan.groups, 1);
  if (grid.y > 65535u) return ADH_EINVAL;
  hipLaunchKernelGGL(conv3x3_wgrad_f32_kernel, grid, dim3(kWgThreads), 0, st, P);
  int e = launch_status();
  if (e) return e;
  WgradReduceParams R = {};
  R.partial = P.partial; R.dw = dw; R.Cin = Cin; R.Cout = Cout;
  R.blocks_x = plan.blocks_x; R.ci_groups = P.ci_groups; R.beta = beta;
  R.div9 = FastDiv(9); R.div_cin = FastDiv(Cin);
  const uint32_t total = Cin * Cout * 9u;
  hipLaunchKernelGGL(conv3x3_wgrad_reduce_kernel, dim3((total + 255u) / 256u), dim3(256), 0, st, R);
  return launch_status();
}

int adh_conv3x3_slab_bwd_filter(int dtype, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                                const void *x_pad, const void *dy, float *dw, float beta, void *workspace,
                                size_t workspace_bytes, void *stream) {
  const void *xs[1] = {x_pad};
  const void *dys[1] = {dy};
  return adh_conv3x3_slab_bwd_filter_tiles(dtype, 1, N, Cin, Cout, H, W, xs, dys, dw, beta, workspace,
                                           workspace_bytes, stream);
}

}  // extern "C"
