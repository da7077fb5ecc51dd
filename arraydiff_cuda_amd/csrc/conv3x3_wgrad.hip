// Backward-filter of the 3x3 slab convolution on the gfx950 matrix cores (fp32 MFMA):
//   dw[co][ci][a][b] = beta*dw + sum_{tile,n,h,w} dy[n][co][h][w] * x_pad[n][ci][h+a][w+b]
//
// GEMM view: D[co][ci] (one 16x16 tile per tap) += A[co][pixel] * B[pixel][ci], the reduction
// runs over pixels, 4 consecutive pixels of one row per v_mfma_f32_16x16x4_f32.
//   * a workgroup (8 waves, two per SIMD) owns a run of output rows of one image, 32 output
//     channels, 64 input channels and all 9 taps: wave = (co tile, ci tile), 9 accumulator tiles.
//     Halving the output channels per workgroup halves the partial block it has to write.
//   * rows stream through LDS: the slab rows live in a 4-slot ring (4 separate arrays so that
//     every phase of the 4x unrolled row loop names its slots statically), each new output row
//     loads exactly one new slab row and one dy row, asynchronously and register-free with
//     buffer_load ... lds, while the previous row is being multiplied; lanes past the row end
//     carry an out-of-range offset and the hardware writes zero.  Channel pitch 68 floats
//     (== 4 mod 64): the 16 channels x 4 pixels of one operand read hit 64 different banks.
//     Column tiles of at most 36 pixels take pitch 44 instead (16 channels x 44 floats fall on 16
//     different groups of four banks too): the rings then need 56 KB, two workgroups share a CU and
//     each one's waits (first rows of a plane, the barrier after a row, the partial block's stores)
//     are the other's matrix-core time.
//   * LDS reads of k-step s+1 are interleaved 1:1 with the MFMAs of k-step s (two-deep register
//     buffer, pinned with scheduling-group barriers).
//   * every workgroup writes its partial 32x64x9 block to the workspace and a second kernel
//     sums the partials in a fixed order: the result is deterministic (no float atomics).
#include "adh_common.h"

namespace adh {

typedef float floatx4 __attribute__((ext_vector_type(4)));

static constexpr int kWgWaves = 8;
static constexpr int kWgThreads = 64 * kWgWaves;
// floats per staged channel row (PITCH): 68 or 44.  A row is one load of min(64, PITCH) lanes, and the k-steps
// run in pairs: the last one reads columns up to 8 * ceil(ceil(W / 4) / 2) + 1 < PITCH.
static constexpr int kMaxW = 60;        // widest column tile at pitch 68
static constexpr int kMaxWNarrow = 40;  // at pitch 44
static constexpr int kPartialFloats = 32 * 64 * 9;
static constexpr int kWgBufferFlags = 0x00020000;
static constexpr uint32_t kWgOutOfRange = 0x80000000u;

struct WgradParams {
  const float *x[ADH_MAX_TILES];
  const float *dy[ADH_MAX_TILES];
  float *partial;            // [grid.y][grid.x][32*64*9] in (co, ci, tap) order, local to the group
  uint32_t num_tiles, N, Cin, Cout, H, W;
  uint32_t rows_per_block, chunks_per_plane;  // row chunks of a plane
  uint32_t planes_per_block;                  // image planes a workgroup walks (same rows and columns of each)
  uint32_t cols_per_block, col_tiles;         // column tiles of a plane (<= kMaxW columns each)
  // grid.x = col_tiles * chunks_per_plane * ceil(N * num_tiles / planes_per_block)
  uint32_t ci_groups;        // grid.y = co_halves * ci_groups, co_halves = ceil(Cout/32)
  // the tiles are the row tiles of one activation in rank order: slab row 0 of tile t > 0 is read from
  // tile t-1's last interior row and slab row H+1 of tile t < num_tiles-1 from tile t+1's first
  // interior row, which is what a halo exchange would have copied there
  int32_t rows_from_neighbours;
  // x carries no halo (H x W like dy): slab row y is x row y - 1, slab column c is x column c - 1, what lies
  // outside is zero or, for rows -1 and H with rows_from_neighbours, the neighbouring tile's last / first row
  int32_t unpadded;
  FastDiv div_chunks, div_tiles, div_ci_groups, div_cols;
};

template <int PITCH>
__global__ __launch_bounds__(kWgThreads, PITCH == 44 ? 2 : 1) void conv3x3_wgrad_f32_kernel(const WgradParams P) {
  constexpr int kRowPitch = PITCH;
  constexpr int kXSlotFloats = 64 * kRowPitch, kDSlotFloats = 32 * kRowPitch;
  __shared__ float xs0[kXSlotFloats];
  __shared__ float xs1[kXSlotFloats];
  __shared__ float xs2[kXSlotFloats];
  __shared__ float xs3[kXSlotFloats];
  __shared__ float dys0[kDSlotFloats];
  __shared__ float dys1[kDSlotFloats];

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u, g = lane >> 4, l16 = lane & 15u;
  const uint32_t wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t ot = wv & 1u;   // co tile inside the 32-channel half
  const uint32_t ct = wv >> 1;   // ci tile

  uint32_t rest, ctile, pgroup, chunk;
  P.div_cols.divmod(blockIdx.x, rest, ctile);
  P.div_chunks.divmod(rest, pgroup, chunk);
  uint32_t coh, cig;
  P.div_ci_groups.divmod(blockIdx.y, coh, cig);
  const uint32_t r0 = chunk * P.rows_per_block;
  const uint32_t r1 = min(r0 + P.rows_per_block, P.H);
  const uint32_t WP = P.unpadded ? P.W : P.W + 2u, HP = P.unpadded ? P.H : P.H + 2u;  // an x plane in memory
  const uint32_t ci0 = cig * 64u, co0 = coh * 32u;

  // columns 64..67 of every staged row are read by the last k-steps of wide rows but never
  // written by the 64-lane loads: clear them once
  if constexpr (PITCH > 64) {
    for (uint32_t i = tid; i < 64u * 4u; i += kWgThreads) {
      const uint32_t o = (i >> 2) * kRowPitch + 64u + (i & 3u);
      xs0[o] = 0.f; xs1[o] = 0.f; xs2[o] = 0.f; xs3[o] = 0.f;
    }
  }
  // a load writes one dword per lane from the row's start on: lanes past the pitch would land in the next
  // channel's row, so they are switched off (a lane that is switched off writes nothing)
  const bool row_lane = PITCH >= 64 || lane < (uint32_t)PITCH;

  // ---- staging: one 64-lane load = one channel row; wave v loads slab channels [8v,8v+8) and
  // dy channels [4v,4v+4) ----
  const uint32_t w0 = ctile * P.cols_per_block;
  const uint32_t tw = min(P.cols_per_block, P.W - w0);  // columns of this workgroup
  uint32_t x_voff = lane < tw + 2u ? (w0 + lane) * 4u : kWgOutOfRange;
  if (P.unpadded) {
    const int32_t col = (int32_t)(w0 + lane) - 1;
    x_voff = (lane < tw + 2u && col >= 0 && col < (int32_t)P.W) ? (uint32_t)col * 4u : kWgOutOfRange;
  }
  const uint32_t d_voff = lane < tw ? (w0 + lane) * 4u : kWgOutOfRange;
  const bool ragged_c = (ci0 + 64u > P.Cin) || (co0 + 32u > P.Cout);  // uniform
  // The image plane (tile, image) the workgroup stands at; it walks planes_per_block of them with the same
  // accumulators.  A slab row is uniform over the workgroup, and so is the image it comes from.
  const int x_bytes = (int)(P.Cin * HP * WP * 4u), dy_bytes = (int)(P.Cout * P.H * P.W * 4u);
  __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.x[0]), 0, 0, kWgBufferFlags);
  __amdgpu_buffer_rsrc_t rsrc_dy = rsrc_x, rsrc_above = rsrc_x, rsrc_below = rsrc_x;
  bool from_above = false, from_below = false;
  auto open_plane = [&](uint32_t plane) {
    uint32_t n, t;
    P.div_tiles.divmod(plane, n, t);
    const uint64_t x_img = ((uint64_t)n * P.Cin) * HP * WP;
    rsrc_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.x[t] + x_img), 0, x_bytes, kWgBufferFlags);
    rsrc_dy = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.dy[t] + ((uint64_t)n * P.Cout) * P.H * P.W), 0,
                                                dy_bytes, kWgBufferFlags);
    from_above = P.rows_from_neighbours && t > 0u;
    from_below = P.rows_from_neighbours && t + 1u < P.num_tiles;
    rsrc_above = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.x[from_above ? t - 1u : t] + x_img), 0, x_bytes,
                                                   kWgBufferFlags);
    rsrc_below = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.x[from_below ? t + 1u : t] + x_img), 0, x_bytes,
                                                   kWgBufferFlags);
  };
  auto stage_x_row = [&](float *slot, uint32_t y) {  // slab row y of the 64 input channels
    __amdgpu_buffer_rsrc_t rsrc = rsrc_x;
    bool none = false;  // a row of zeros
    if (P.unpadded) {
      if (y == 0u) {
        rsrc = rsrc_above;
        none = !from_above;
        y = P.H - 1u;
      } else if (y == P.H + 1u) {
        rsrc = rsrc_below;
        none = !from_below;
        y = 0u;
      } else {
        y -= 1u;
      }
    } else if (from_above && y == 0u) {
      rsrc = rsrc_above;
      y = P.H;
    } else if (from_below && y == HP - 1u) {
      rsrc = rsrc_below;
      y = 1u;
    }
    if (!row_lane) return;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t cl = wv * 8u + i;
      uint32_t voff = none ? kWgOutOfRange : x_voff;
      uint32_t ci = ci0 + cl;
      if (ragged_c && ci >= P.Cin) {
        voff = kWgOutOfRange;
        ci = 0;
      }
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, slot + cl * kRowPitch, 4, voff,
                                               __builtin_amdgcn_readfirstlane((ci * HP + y) * WP * 4u), 0, 0);
    }
  };
  auto stage_dy_row = [&](float *slot, uint32_t r) {  // output row r of the 32 output channels
    if (!row_lane) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t cl = wv * 4u + i;
      uint32_t voff = d_voff;
      uint32_t co = co0 + cl;
      if (ragged_c && co >= P.Cout) {
        voff = kWgOutOfRange;
        co = 0;
      }
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_dy, slot + cl * kRowPitch, 4, voff,
                                               __builtin_amdgcn_readfirstlane((co * P.H + r) * P.W * 4u), 0, 0);
    }
  };

  floatx4 acc[9];
#pragma unroll
  for (int tap = 0; tap < 9; ++tap) acc[tap] = floatx4{0.f, 0.f, 0.f, 0.f};

  const uint32_t ksteps = (tw + 3u) / 4u;
  const uint32_t npairs = (ksteps + 1u) / 2u;   // an odd tail k-step multiplies the zero columns
  const uint32_t a_lane = (16u * ot + l16) * kRowPitch + g;
  const uint32_t b_lane = (16u * ct + l16) * kRowPitch + g;

  // one output row: dyr = its dy slot, b0/b1/b2 = the slab rows r, r+1, r+2
  auto compute_row = [&](const float *dyr, const float *b0, const float *b1, const float *b2) {
    float a[2], b[2][9];
    auto read_operands = [&](int buf, uint32_t ks) {
      const uint32_t col = 4u * ks;
      a[buf] = dyr[a_lane + col];
#pragma unroll
      for (int kw = 0; kw < 3; ++kw) {
        b[buf][0 + kw] = b0[b_lane + col + kw];
        b[buf][3 + kw] = b1[b_lane + col + kw];
        b[buf][6 + kw] = b2[b_lane + col + kw];
      }
    };
    auto step = [&](int cur, uint32_t next_ks) {
      read_operands(cur ^ 1, next_ks);
#pragma unroll
      for (int tap = 0; tap < 9; ++tap)
        acc[tap] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[cur], b[cur][tap], acc[tap], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // the A read
#pragma unroll
      for (int tap = 0; tap < 9; ++tap) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    read_operands(0, 0);
    const uint32_t last = 2u * npairs - 1u;
    for (uint32_t kp = 0; kp < npairs; ++kp) {
      step(0, 2u * kp + 1u);
      step(1, min(2u * kp + 2u, last));  // the final prefetch is not used; keep it in range
    }
  };

  const uint32_t plane0 = pgroup * P.planes_per_block;
  const uint32_t plane1 = min(plane0 + P.planes_per_block, P.num_tiles * P.N);
  for (uint32_t plane = plane0; plane < plane1; ++plane) {
    open_plane(plane);
    // prologue: slab rows r0, r0+1, r0+2 -> slots 0,1,2 and dy row r0 -> slot 0
    stage_x_row(xs0, r0);
    stage_x_row(xs1, r0 + 1u);
    stage_x_row(xs2, r0 + 2u);
    stage_dy_row(dys0, r0);
    __syncthreads();

    // four rows per trip: each phase names its ring slots statically
    for (uint32_t r = r0;;) {
      if (r + 1u < r1) { stage_x_row(xs3, r + 3u); stage_dy_row(dys1, r + 1u); }
      __builtin_amdgcn_sched_barrier(0);
      compute_row(dys0, xs0, xs1, xs2);
      __syncthreads();
      if (++r == r1) break;
      if (r + 1u < r1) { stage_x_row(xs0, r + 3u); stage_dy_row(dys0, r + 1u); }
      __builtin_amdgcn_sched_barrier(0);
      compute_row(dys1, xs1, xs2, xs3);
      __syncthreads();
      if (++r == r1) break;
      if (r + 1u < r1) { stage_x_row(xs1, r + 3u); stage_dy_row(dys1, r + 1u); }
      __builtin_amdgcn_sched_barrier(0);
      compute_row(dys0, xs2, xs3, xs0);
      __syncthreads();
      if (++r == r1) break;
      if (r + 1u < r1) { stage_x_row(xs2, r + 3u); stage_dy_row(dys0, r + 1u); }
      __builtin_amdgcn_sched_barrier(0);
      compute_row(dys1, xs3, xs0, xs1);
      __syncthreads();
      if (++r == r1) break;
    }
  }

  // ---- epilogue: lane holds D[co = 4g+i][ci = l16] of each tap tile ----
  const uint32_t block_lin = blockIdx.y * gridDim.x + blockIdx.x;
  float *__restrict__ part = P.partial + (uint64_t)block_lin * kPartialFloats;
#pragma unroll
  for (int tap = 0; tap < 9; ++tap)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t co_l = 16u * ot + 4u * g + i, ci_l = 16u * ct + l16;
      part[(co_l * 64u + ci_l) * 9u + tap] = acc[tap][i];
    }
}


// The same filter gradient for a window whose taps lie DIL rows and columns apart (stride 1, tiles padded by DIL):
//   dw[co][ci][a][b] = beta*dw + sum dy[n][co][h][w] * x_pad[n][ci][h + DIL a][w + DIL b]
// Output row r meets the slab rows r, r + DIL and r + 2 DIL, so the ring holds 2 DIL + 2 slab rows (the 2 DIL + 1
// in use and the one arriving) and the row loop is unrolled once per slot; column tiles of at most 56 pixels at
// pitch 68 (the last k-step reads column 8 * ceil(ceil(tw / 4) / 2) - 1 + 2 DIL).  Everything else as above.
static constexpr int kMaxWDil = 56;

template <int V>
struct WgPhase {
  static constexpr int value = V;
};

template <int DIL>
__global__ __launch_bounds__(kWgThreads, 1) void conv3x3_wgrad_dil_f32_kernel(const WgradParams P) {
  static_assert(DIL == 3, "eight ring slots are declared below");
  constexpr int kRowPitch = 68, NS = 2 * DIL + 2;
  constexpr int kXSlotFloats = 64 * kRowPitch, kDSlotFloats = 32 * kRowPitch;
  __shared__ float xs0[kXSlotFloats];
  __shared__ float xs1[kXSlotFloats];
  __shared__ float xs2[kXSlotFloats];
  __shared__ float xs3[kXSlotFloats];
  __shared__ float xs4[kXSlotFloats];
  __shared__ float xs5[kXSlotFloats];
  __shared__ float xs6[kXSlotFloats];
  __shared__ float xs7[kXSlotFloats];
  __shared__ float dys0[kDSlotFloats];
  __shared__ float dys1[kDSlotFloats];
  float *const xs[NS] = {xs0, xs1, xs2, xs3, xs4, xs5, xs6, xs7};
  float *const dys[2] = {dys0, dys1};

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u, g = lane >> 4, l16 = lane & 15u;
  const uint32_t wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t ot = wv & 1u;   // co tile inside the 32-channel half
  const uint32_t ct = wv >> 1;   // ci tile

  uint32_t rest, ctile, pgroup, chunk;
  P.div_cols.divmod(blockIdx.x, rest, ctile);
  P.div_chunks.divmod(rest, pgroup, chunk);
  uint32_t coh, cig;
  P.div_ci_groups.divmod(blockIdx.y, coh, cig);
  const uint32_t r0 = chunk * P.rows_per_block;
  const uint32_t r1 = min(r0 + P.rows_per_block, P.H);
  const uint32_t WP = P.W + 2u * DIL, HP = P.H + 2u * DIL;
  const uint32_t ci0 = cig * 64u, co0 = coh * 32u;

  // columns 64..67 of every staged slab row are read by the last k-steps of wide rows but never written by the
  // 64-lane loads: clear them once
  for (uint32_t i = tid; i < 64u * 4u; i += kWgThreads) {
    const uint32_t o = (i >> 2) * kRowPitch + 64u + (i & 3u);
    xs0[o] = 0.f; xs1[o] = 0.f; xs2[o] = 0.f; xs3[o] = 0.f;
    xs4[o] = 0.f; xs5[o] = 0.f; xs6[o] = 0.f; xs7[o] = 0.f;
  }

  const uint32_t w0 = ctile * P.cols_per_block;
  const uint32_t tw = min(P.cols_per_block, P.W - w0);  // columns of this workgroup
  const uint32_t x_voff = lane < tw + 2u * DIL ? (w0 + lane) * 4u : kWgOutOfRange;
  const uint32_t d_voff = lane < tw ? (w0 + lane) * 4u : kWgOutOfRange;
  const bool ragged_c = (ci0 + 64u > P.Cin) || (co0 + 32u > P.Cout);  // uniform
  const int x_bytes = (int)(P.Cin * HP * WP * 4u), dy_bytes = (int)(P.Cout * P.H * P.W * 4u);
  __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.x[0]), 0, 0, kWgBufferFlags);
  __amdgpu_buffer_rsrc_t rsrc_dy = rsrc_x;
  auto open_plane = [&](uint32_t plane) {
    uint32_t n, t;
    P.div_tiles.divmod(plane, n, t);
    rsrc_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.x[t] + ((uint64_t)n * P.Cin) * HP * WP), 0, x_bytes,
                                               kWgBufferFlags);
    rsrc_dy = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.dy[t] + ((uint64_t)n * P.Cout) * P.H * P.W), 0,
                                                dy_bytes, kWgBufferFlags);
  };
  auto stage_x_row = [&](float *slot, uint32_t y) {  // slab row y of the 64 input channels; wave v loads channels [8v, 8v+8)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t cl = wv * 8u + i;
      uint32_t voff = x_voff;
      uint32_t ci = ci0 + cl;
      if (ragged_c && ci >= P.Cin) {
        voff = kWgOutOfRange;
        ci = 0;
      }
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, slot + cl * kRowPitch, 4, voff,
                                               __builtin_amdgcn_readfirstlane((ci * HP + y) * WP * 4u), 0, 0);
    }
  };
  auto stage_dy_row = [&](float *slot, uint32_t r) {  // output row r of the 32 output channels; wave v loads [4v, 4v+4)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t cl = wv * 4u + i;
      uint32_t voff = d_voff;
      uint32_t co = co0 + cl;
      if (ragged_c && co >= P.Cout) {
        voff = kWgOutOfRange;
        co = 0;
      }
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_dy, slot + cl * kRowPitch, 4, voff,
                                               __builtin_amdgcn_readfirstlane((co * P.H + r) * P.W * 4u), 0, 0);
    }
  };

  floatx4 acc[9];
#pragma unroll
  for (int tap = 0; tap < 9; ++tap) acc[tap] = floatx4{0.f, 0.f, 0.f, 0.f};

  const uint32_t ksteps = (tw + 3u) / 4u;
  const uint32_t npairs = (ksteps + 1u) / 2u;   // an odd tail k-step multiplies the zero columns
  const uint32_t a_lane = (16u * ot + l16) * kRowPitch + g;
  const uint32_t b_lane = (16u * ct + l16) * kRowPitch + g;

  // one output row: dyr = its dy slot, b0/b1/b2 = the slab rows r, r + DIL, r + 2 DIL
  auto compute_row = [&](const float *dyr, const float *b0, const float *b1, const float *b2) {
    float a[2], b[2][9];
    auto read_operands = [&](int buf, uint32_t ks) {
      const uint32_t col = 4u * ks;
      a[buf] = dyr[a_lane + col];
#pragma unroll
      for (int kw = 0; kw < 3; ++kw) {
        b[buf][0 + kw] = b0[b_lane + col + kw * DIL];
        b[buf][3 + kw] = b1[b_lane + col + kw * DIL];
        b[buf][6 + kw] = b2[b_lane + col + kw * DIL];
      }
    };
    auto step = [&](int cur, uint32_t next_ks) {
      read_operands(cur ^ 1, next_ks);
#pragma unroll
      for (int tap = 0; tap < 9; ++tap)
        acc[tap] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[cur], b[cur][tap], acc[tap], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // the A read
#pragma unroll
      for (int tap = 0; tap < 9; ++tap) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    read_operands(0, 0);
    const uint32_t last = 2u * npairs - 1u;
    for (uint32_t kp = 0; kp < npairs; ++kp) {
      step(0, 2u * kp + 1u);
      step(1, min(2u * kp + 2u, last));  // the final prefetch is not used; keep it in range
    }
  };

  // phase PH = (r - r0) mod NS: slab row y of the chunk lives in slot (y - r0) mod NS
  auto phase = [&](auto tag, uint32_t r) {
    constexpr int PH = decltype(tag)::value;
    if (r + 1u < r1) {
      stage_x_row(xs[(PH + 2 * DIL + 1) % NS], r + 2u * DIL + 1u);
      stage_dy_row(dys[(PH + 1) & 1], r + 1u);
    }
    __builtin_amdgcn_sched_barrier(0);
    compute_row(dys[PH & 1], xs[PH], xs[(PH + DIL) % NS], xs[(PH + 2 * DIL) % NS]);
    __syncthreads();
  };

  const uint32_t plane0 = pgroup * P.planes_per_block;
  const uint32_t plane1 = min(plane0 + P.planes_per_block, P.num_tiles * P.N);
  for (uint32_t plane = plane0; plane < plane1; ++plane) {
    open_plane(plane);
    // prologue: slab rows r0 .. r0 + 2 DIL -> slots 0 .. 2 DIL and dy row r0 -> slot 0
#pragma unroll
    for (int y = 0; y <= 2 * DIL; ++y) stage_x_row(xs[y], r0 + (uint32_t)y);
    stage_dy_row(dys0, r0);
    __syncthreads();
    for (uint32_t r = r0;;) {
      phase(WgPhase<0>(), r);
      if (++r == r1) break;
      phase(WgPhase<1>(), r);
      if (++r == r1) break;
      phase(WgPhase<2>(), r);
      if (++r == r1) break;
      phase(WgPhase<3>(), r);
      if (++r == r1) break;
      phase(WgPhase<4>(), r);
      if (++r == r1) break;
      phase(WgPhase<5>(), r);
      if (++r == r1) break;
      phase(WgPhase<6>(), r);
      if (++r == r1) break;
      phase(WgPhase<7>(), r);
      if (++r == r1) break;
    }
  }

  // ---- epilogue: lane holds D[co = 4g+i][ci = l16] of each tap tile ----
  const uint32_t block_lin = blockIdx.y * gridDim.x + blockIdx.x;
  float *__restrict__ part = P.partial + (uint64_t)block_lin * kPartialFloats;
#pragma unroll
  for (int tap = 0; tap < 9; ++tap)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t co_l = 16u * ot + 4u * g + i, ci_l = 16u * ct + l16;
      part[(co_l * 64u + ci_l) * 9u + tap] = acc[tap][i];
    }
}

// dw[co][ci][tap] = beta*dw + sum over the pixel-chunk partials of its (co half, ci group), in
// a fixed order (deterministic): 4 lanes-groups each sum a quarter of the partials, then the
// quarters are combined through LDS in index order.
struct WgradReduceParams {
  const float *partial;
  float *dw;
  uint32_t Cin, Cout, blocks_x, ci_groups, total;
  float beta;
  FastDiv div9, div_cin;
};

__global__ __launch_bounds__(256) void conv3x3_wgrad_reduce_kernel(const WgradReduceParams P) {
  __shared__ float part[4][64];
  const uint32_t q = threadIdx.x >> 6, j = threadIdx.x & 63u;
  const uint32_t e = blockIdx.x * 64u + j;
  float s = 0.f;
  if (e < P.total) {
    uint32_t cc, tap, co, ci;
    P.div9.divmod(e, cc, tap);
    P.div_cin.divmod(cc, co, ci);
    const uint32_t grp = (co >> 5) * P.ci_groups + (ci >> 6);
    const uint32_t local = (((co & 31u) * 64u) + (ci & 63u)) * 9u + tap;
    const float *p = P.partial + ((uint64_t)grp * P.blocks_x) * kPartialFloats + local;
    const uint32_t per = (P.blocks_x + 3u) / 4u;
    const uint32_t b0 = q * per, b1 = min(b0 + per, P.blocks_x);
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    uint32_t b = b0;
    for (; b + 4u <= b1; b += 4u) {
      s0 += p[(uint64_t)(b + 0u) * kPartialFloats];
      s1 += p[(uint64_t)(b + 1u) * kPartialFloats];
      s2 += p[(uint64_t)(b + 2u) * kPartialFloats];
      s3 += p[(uint64_t)(b + 3u) * kPartialFloats];
    }
    for (; b < b1; ++b) s0 += p[(uint64_t)b * kPartialFloats];
    s = (s0 + s1) + (s2 + s3);
  }
  part[q][j] = s;
  __syncthreads();
  if (q == 0 && e < P.total) {
    float r = (part[0][j] + part[1][j]) + (part[2][j] + part[3][j]);
    if (P.beta != 0.f) r += P.beta * P.dw[e];
    P.dw[e] = r;
  }
}

struct WgradPlan {
  uint32_t rows_per_block, chunks_per_plane, planes_per_block, cols_per_block, col_tiles, blocks_x, groups;
  bool narrow;  // column tiles of at most kMaxWNarrow pixels: row pitch 44, two workgroups per CU
  size_t workspace_bytes;
};

// Row chunks per plane and planes per workgroup for column tiles of `cols` pixels, `per_cu` workgroups sharing a
// CU.  A workgroup spends 576 matrix-core cycles per k-step of four columns (9 MFMAs of 32 cycles, two waves a SIMD)
// on every row, about 4000 cycles per plane waiting for its first rows, and about 19000 cycles on being launched
// and on writing the partial block that the second kernel then reads back; workgroups that share a CU share its
// matrix cores, and one's waits are the other's multiplications.  Every partial block is 74 KB written and read
// once more, about 100 cycles of the whole chip's memory bandwidth.  Returns the least modelled time.
static double wgrad_plan_rows(uint64_t planes, uint64_t per_chunk, uint32_t H, uint32_t cols, uint32_t per_cu,
                              uint32_t *best_chunks, uint32_t *best_ppb) {
  const double row_cycles = 576.0 * ((cols + 3u) / 4u) * per_cu;
  const double plane_cycles = per_cu > 1u ? 1000.0 : 4000.0, block_cycles = per_cu > 1u ? 8000.0 : 19000.0;
  const uint64_t slots = 256ull * per_cu;
  double best_cost = 1e300;
  *best_chunks = 1;
  *best_ppb = 1;
  for (uint32_t chunks = 1; chunks <= H; ++chunks) {
    const uint32_t rows = (H + chunks - 1) / chunks;
    if ((H + rows - 1) / rows != chunks) continue;  // same row count as a smaller chunk number
    for (uint64_t ppb = 1; ppb <= planes; ++ppb) {
      const uint64_t pgroups = (planes + ppb - 1) / ppb;
      if ((planes + pgroups - 1) / pgroups != ppb) continue;  // same group count as a smaller number of planes
      const uint64_t blocks = per_chunk * chunks * pgroups;
      const double cost = (double)((blocks + slots - 1) / slots) * ((double)ppb * (rows * row_cycles + plane_cycles) + block_cycles) +
                          100.0 * (double)blocks;
      if (cost < best_cost) {
        best_cost = cost;
        *best_chunks = chunks;
        *best_ppb = (uint32_t)ppb;
      }
      if (blocks < slots) break;  // more planes per workgroup only leave more CUs idle
    }
    if (per_chunk * chunks * planes >= 16u * slots) break;
  }
  return best_cost;
}

static bool wgrad_plan(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                       WgradPlan *plan) {
  const uint64_t planes = (uint64_t)num_tiles * N;
  const uint32_t groups = ((Cin + 63u) / 64u) * ((Cout + 31u) / 32u);
  uint32_t chunks[2], ppb[2], col_tiles[2], cols[2];
  double cost[2];
  for (int narrow = 0; narrow < 2; ++narrow) {
    const uint32_t max_w = narrow ? kMaxWNarrow : kMaxW;
    col_tiles[narrow] = (W + max_w - 1) / max_w;
    cols[narrow] = (W + col_tiles[narrow] - 1) / col_tiles[narrow];
    cost[narrow] = wgrad_plan_rows(planes, (uint64_t)col_tiles[narrow] * groups, H, cols[narrow], narrow ? 2u : 1u,
                                   &chunks[narrow], &ppb[narrow]);
  }
  const int pick = cost[1] <= cost[0] ? 1 : 0;
  const uint32_t rows = (H + chunks[pick] - 1) / chunks[pick];
  const uint64_t blocks_x = ((planes + ppb[pick] - 1) / ppb[pick]) * chunks[pick] * col_tiles[pick];
  if (blocks_x > 0x7fffffffull) return false;
  // one image of x / dy is addressed through a 32-bit buffer resource
  if ((uint64_t)Cin * (H + 2) * (W + 2) * 4u >= (1ull << 31) || (uint64_t)Cout * H * W * 4u >= (1ull << 31)) return false;
  plan->rows_per_block = rows;
  plan->chunks_per_plane = chunks[pick];
  plan->planes_per_block = ppb[pick];
  plan->cols_per_block = cols[pick];
  plan->col_tiles = col_tiles[pick];
  plan->narrow = pick == 1;
  plan->blocks_x = (uint32_t)blocks_x;
  plan->groups = groups;
  plan->workspace_bytes = (size_t)plan->blocks_x * groups * kPartialFloats * sizeof(float);
  return true;
}


// the plan of the dilated kernel: column tiles of at most kMaxWDil pixels, one workgroup per CU
static bool wgrad_dil_plan(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W, uint32_t dil,
                           WgradPlan *plan) {
  if (dil != 3u || num_tiles == 0 || N == 0 || Cin == 0 || Cout == 0 || H == 0 || W == 0) return false;
  const uint64_t planes = (uint64_t)num_tiles * N;
  const uint32_t groups = ((Cin + 63u) / 64u) * ((Cout + 31u) / 32u);
  if (groups > 65535u) return false;
  const uint32_t col_tiles = (W + kMaxWDil - 1) / kMaxWDil;
  const uint32_t cols = (W + col_tiles - 1) / col_tiles;
  uint32_t chunks = 1, ppb = 1;
  wgrad_plan_rows(planes, (uint64_t)col_tiles * groups, H, cols, 1u, &chunks, &ppb);
  const uint64_t blocks_x = ((planes + ppb - 1) / ppb) * chunks * col_tiles;
  if (blocks_x > 0x7fffffffull) return false;
  if ((uint64_t)Cin * (H + 2ull * dil) * (W + 2ull * dil) * 4u >= (1ull << 31) || (uint64_t)Cout * H * W * 4u >= (1ull << 31) ||
      (uint64_t)Cin * Cout * 9u >= (1ull << 31))
    return false;
  plan->rows_per_block = (H + chunks - 1) / chunks;
  plan->chunks_per_plane = chunks;
  plan->planes_per_block = ppb;
  plan->cols_per_block = cols;
  plan->col_tiles = col_tiles;
  plan->narrow = false;
  plan->blocks_x = (uint32_t)blocks_x;
  plan->groups = groups;
  plan->workspace_bytes = (size_t)plan->blocks_x * groups * kPartialFloats * sizeof(float);
  return true;
}

// The filter gradient of the 3x3 window at stride 1 with dilation 3 over fp32 tiles padded by 3 (the reference's
// tools/microbench_spatial_conv.cc:25-32).  H, W: the interior (= dy) extents.  Workspace 0 / ADH_EUNIMPL (and
// nothing launched) for another dilation and for images beyond a buffer resource's 2 GiB: the general kernel serves
// those.  Arguments are the caller's, already validated.
size_t conv3x3_dilated_wgrad_workspace(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                                       uint32_t dil) {
  WgradPlan plan;
  return wgrad_dil_plan(num_tiles, N, Cin, Cout, H, W, dil, &plan) ? plan.workspace_bytes : 0;
}
int conv3x3_dilated_wgrad_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W, uint32_t dil,
                              const void *const *x_tiles, const void *const *dy_tiles, float *dw, float beta, void *workspace,
                              hipStream_t st) {
  WgradPlan plan;
  if (!wgrad_dil_plan(num_tiles, N, Cin, Cout, H, W, dil, &plan)) return ADH_EUNIMPL;
  WgradParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    P.x[t] = reinterpret_cast<const float *>(x_tiles[t]);
    P.dy[t] = reinterpret_cast<const float *>(dy_tiles[t]);
  }
  P.partial = reinterpret_cast<float *>(workspace);
  P.num_tiles = num_tiles; P.N = N; P.Cin = Cin; P.Cout = Cout; P.H = H; P.W = W;
  P.rows_per_block = plan.rows_per_block;
  P.chunks_per_plane = plan.chunks_per_plane;
  P.planes_per_block = plan.planes_per_block;
  P.cols_per_block = plan.cols_per_block;
  P.col_tiles = plan.col_tiles;
  P.div_cols = FastDiv(plan.col_tiles);
  P.ci_groups = (Cin + 63u) / 64u;
  P.div_chunks = FastDiv(plan.chunks_per_plane);
  P.div_tiles = FastDiv(num_tiles);
  P.div_ci_groups = FastDiv(P.ci_groups);
  hipLaunchKernelGGL(conv3x3_wgrad_dil_f32_kernel<3>, dim3(plan.blocks_x, plan.groups, 1), dim3(kWgThreads), 0, st, P);
  int e = launch_status();
  if (e) return e;
  WgradReduceParams R = {};
  R.partial = P.partial; R.dw = dw; R.Cin = Cin; R.Cout = Cout;
  R.blocks_x = plan.blocks_x; R.ci_groups = P.ci_groups; R.beta = beta;
  R.total = Cin * Cout * 9u;
  R.div9 = FastDiv(9); R.div_cin = FastDiv(Cin);
  hipLaunchKernelGGL(conv3x3_wgrad_reduce_kernel, dim3((R.total + 63u) / 64u), dim3(256), 0, st, R);
  return launch_status();
}

size_t bf16_workspace_bytes(int which, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                            uint32_t W, size_t fp32_path_bytes);
int conv_bf16_filter_via_f32(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                             const void *const *x_tiles, const void *const *dy_tiles, float *dw, float beta,
                             void *workspace, size_t workspace_bytes, hipStream_t st);

}  // namespace adh

using namespace adh;

extern "C" {

size_t adh_conv3x3_workspace_bytes(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                   uint32_t H, uint32_t W) {
  if (num_tiles == 0 || N == 0 || Cin == 0 || Cout == 0 || H == 0 || W == 0) return 0;
  size_t f32_bytes = 0;
  if (which == ADH_CONV_BWD_FILTER) {
    WgradPlan plan;
    if (!wgrad_plan(num_tiles, N, Cin, Cout, H, W, &plan)) return 0;
    f32_bytes = plan.workspace_bytes;
  }
  if (dtype == ADH_BF16) return bf16_workspace_bytes(which, num_tiles, N, Cin, Cout, H, W, f32_bytes);
  return dtype == ADH_F32 ? f32_bytes : 0;
}

static int wgrad_entry(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                       const void *const *x_pad_tiles, const void *const *dy_tiles, float *dw, float beta,
                       void *workspace, size_t workspace_bytes, void *stream, bool rows_from_neighbours,
                       bool unpadded = false) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if (unpadded && dtype != ADH_F32) return ADH_EINVAL;  // the bf16 form has an entry of its own
  if (dtype == ADH_BF16 && rows_from_neighbours) {
    // the bf16 kernels stream their rows from one image: exchange first, then the ordinary path
    const int rc = adh_halo_exchange_nchw(dtype, 1, num_tiles, 1, W, H, Cin, N,
                                          const_cast<void *const *>(reinterpret_cast<const void *const *>(x_pad_tiles)),
                                          stream);
    if (rc != ADH_OK) return rc;
  }
  if (dtype == ADH_BF16)
    return conv_bf16_filter_via_f32(num_tiles, N, Cin, Cout, H, W, x_pad_tiles, dy_tiles, dw, beta, workspace,
                                    workspace_bytes, as_stream(stream));
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
  if ((uint64_t)Cin * Cout * 9u >= (1ull << 31)) return ADH_EINVAL;
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
  P.planes_per_block = plan.planes_per_block;
  P.cols_per_block = plan.cols_per_block;
  P.col_tiles = plan.col_tiles;
  P.div_cols = FastDiv(plan.col_tiles);
  P.ci_groups = (Cin + 63u) / 64u;
  P.div_chunks = FastDiv(plan.chunks_per_plane);
  P.div_tiles = FastDiv(num_tiles);
  P.div_ci_groups = FastDiv(P.ci_groups);
  P.rows_from_neighbours = rows_from_neighbours ? 1 : 0;
  P.unpadded = unpadded ? 1 : 0;
  dim3 grid(plan.blocks_x, plan.groups, 1);
  if (grid.y > 65535u) return ADH_EINVAL;
  if (plan.narrow)
    hipLaunchKernelGGL(conv3x3_wgrad_f32_kernel<44>, grid, dim3(kWgThreads), 0, st, P);
  else
    hipLaunchKernelGGL(conv3x3_wgrad_f32_kernel<68>, grid, dim3(kWgThreads), 0, st, P);
  int e = launch_status();
  if (e) return e;
  WgradReduceParams R = {};
  R.partial = P.partial; R.dw = dw; R.Cin = Cin; R.Cout = Cout;
  R.blocks_x = plan.blocks_x; R.ci_groups = P.ci_groups; R.beta = beta;
  R.total = Cin * Cout * 9u;
  R.div9 = FastDiv(9); R.div_cin = FastDiv(Cin);
  hipLaunchKernelGGL(conv3x3_wgrad_reduce_kernel, dim3((R.total + 63u) / 64u), dim3(256), 0, st, R);
  return launch_status();
}

int adh_conv3x3_slab_bwd_filter_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                      uint32_t H, uint32_t W, const void *const *x_pad_tiles,
                                      const void *const *dy_tiles, float *dw, float beta, void *workspace,
                                      size_t workspace_bytes, void *stream) {
  return wgrad_entry(dtype, num_tiles, N, Cin, Cout, H, W, x_pad_tiles, dy_tiles, dw, beta, workspace, workspace_bytes,
                     stream, false);
}

int adh_conv3x3_slab_bwd_filter_tiles_unexchanged(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin,
                                                  uint32_t Cout, uint32_t H, uint32_t W,
                                                  const void *const *x_pad_tiles, const void *const *dy_tiles,
                                                  float *dw, float beta, void *workspace, size_t workspace_bytes,
                                                  void *stream) {
  return wgrad_entry(dtype, num_tiles, N, Cin, Cout, H, W, x_pad_tiles, dy_tiles, dw, beta, workspace, workspace_bytes,
                     stream, true);
}

}  // extern "C"

// the fp32 leg of adh_conv3x3_unpadded_bwd_filter_tiles
namespace adh {
int conv_wgrad_f32_unpadded(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                            const void *const *x_tiles, const void *const *dy_tiles, float *dw, float beta, void *workspace,
                            size_t workspace_bytes, void *stream) {
  return wgrad_entry(ADH_F32, num_tiles, N, Cin, Cout, H, W, x_tiles, dy_tiles, dw, beta, workspace, workspace_bytes, stream,
                     true, true);
}
}  // namespace adh

extern "C" {

int adh_conv3x3_slab_bwd_filter(int dtype, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                                const void *x_pad, const void *dy, float *dw, float beta, void *workspace,
                                size_t workspace_bytes, void *stream) {
  const void *xs[1] = {x_pad};
  const void *dys[1] = {dy};
  return adh_conv3x3_slab_bwd_filter_tiles(dtype, 1, N, Cin, Cout, H, W, xs, dys, dw, beta, workspace,
                                           workspace_bytes, stream);
}

}  // extern "C"
