// Filter gradient of the 3x3 slab convolution on the bf16 matrix cores, for up to 64 input and
// 64 output channels and image widths that are a multiple of eight:
//   dw[co][ci][kh][kw] = sum over images, rows h, columns w of dy[co][h][w] * x_pad[ci][h+kh][w+kw]
//
// The reduction runs over pixels, and eight neighbouring pixels of a channel row are 16
// contiguous bytes in NCHW, so both MFMA operands come straight from rows as they lie in memory:
// A = dy (m = output channel, k = 32 columns), B = x_pad (k = 32 columns, n = input channel).
// Rows are copied into LDS by `buffer_load ... lds` with 16 bytes per lane (asynchronous, no
// registers), one row of x_pad and one of dy per stage, six stages (five rows in flight).
//
// A workgroup of eight waves (two per SIMD) walks down a 64-column strip of one image.  A wave
// owns one tile of 16 input channels, one half of the output channels (two tiles of 16) and all
// nine taps: 18 accumulator tiles, fed by both 32-column halves of the strip.  x_pad row r meets
// the dy rows r, r-1, r-2 (taps kh = 0, 1, 2); the three dy rows are kept in registers, so each
// row step reads four dy operands and two x operands from LDS for 36 MFMAs.  The x operand for
// column shift kw = 1 is made from the aligned 16 bytes and the next dword with four funnel
// shifts, kw = 2 is the same five dwords taken one further: 16-byte LDS reads that are not
// 16-byte aligned run nine times slower.
//
// Every wave keeps its sums over all the strips it visits and writes them once, its part of the
// workgroup's partial filter; a second kernel adds the partials in a fixed order.
#include <utility>

#include "adh_common.h"

namespace adh {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWgCols = 64;                       // dy columns per strip
constexpr int kWgLanes = 9;                       // 16-byte lanes per channel row in LDS
constexpr int kWgPitch = kWgLanes * 16;           // 144 bytes: 66 x_pad columns, or 64 dy columns + pad
constexpr int kWgRegion = 64 * kWgPitch;          // 9216 bytes: 64 channel rows
constexpr int kWgStages = 6;                      // rows in LDS: the one being fetched + five on their way
constexpr uint32_t kWgOutOfRange = 0x80000000u;
constexpr uint32_t kWgPartialFloats = 64u * 64u * 9u;

struct WgradBf16Params {
  const uint16_t *x[ADH_MAX_TILES];
  const uint16_t *dy[ADH_MAX_TILES];
  float *partial;  // [gridDim.y][gridDim.x][8 waves][9 taps][2 output-channel tiles][64 lanes][4]
  uint32_t N, Cin, Cout, H, W;
  // More than 64 channels on either side: blockIdx.y numbers the pairs (block of 64 output channels,
  // block of 64 input channels), input block fastest; every pair is a problem of its own.
  uint32_t ci_blocks;
  // UNP instance: x carries no halo (H x W like dy); the tiles are the row tiles of one tensor in rank
  // order, and a tile's rows -1 and H are its neighbours' last and first rows
  uint32_t num_tiles;
  uint32_t strips, items;
  FastDiv div_strips, div_N;
};

template <int V>
struct WgTag { static constexpr int value = V; };

// UNP: x has no halo.  The x row of a stage is then the unpadded row r - 1 (from a neighbouring tile at the
// tile's ends, zeros at the tensor's), and a strip's 64 dy columns meet x columns c0 - 1 .. c0 + 64: ten
// aligned granules from c0 - 8 per channel row (pitch 160 bytes), the operand for column shift kw = 0 made from
// the aligned 16 bytes and the dword BEFORE them, kw = 2 from the dword after.
template <bool UNP>
__global__ __launch_bounds__(512, 1) void conv3x3_bf16_wgrad_kernel(WgradBf16Params P) {
  constexpr int kXLanes = UNP ? 10 : kWgLanes;          // 16-byte lanes per x channel row
  constexpr int kXPitch = kXLanes * 16;
  constexpr int kXRegion = 64 * kXPitch;                // 64 channel rows of x
  constexpr int kStageBytes = kXRegion + kWgRegion;     // x row, then dy row
  constexpr int kDmaPerStage = kStageBytes / 1024;      // 18 (19) wave-wide copies
  // one array per stage: the compiler can then tell the asynchronous writes of one stage from
  // the reads of another
  __shared__ __attribute__((aligned(16))) uint8_t stage0[kStageBytes];
  __shared__ __attribute__((aligned(16))) uint8_t stage1[kStageBytes];
  __shared__ __attribute__((aligned(16))) uint8_t stage2[kStageBytes];
  __shared__ __attribute__((aligned(16))) uint8_t stage3[kStageBytes];
  __shared__ __attribute__((aligned(16))) uint8_t stage4[kStageBytes];
  __shared__ __attribute__((aligned(16))) uint8_t stage5[kStageBytes];
  __shared__ __attribute__((aligned(16))) uint8_t spare[1024];
  uint8_t *const stages[kWgStages] = {stage0, stage1, stage2, stage3, stage4, stage5};

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t cit = wv & 3u, coh = wv >> 2;  // input-channel tile, output-channel half

  floatx4 acc[3][3][2];
#pragma unroll
  for (int kh = 0; kh < 3; ++kh)
#pragma unroll
    for (int kw = 0; kw < 3; ++kw)
#pragma unroll
      for (int cot = 0; cot < 2; ++cot) acc[kh][kw][cot] = (floatx4){0.f, 0.f, 0.f, 0.f};

  // operand addresses inside a stage, for the left 32 columns (+ 64 bytes for the right ones)
  // (UNP: the row in LDS starts eight columns left of the strip)
  const uint32_t b_off = (16u * cit + l16) * kXPitch + g * 16u + (UNP ? 16u : 0u);
  const uint32_t a_off = kXRegion + (32u * coh + l16) * kWgPitch + g * 16u;  // + cot * 16 * kWgPitch

  // copies this wave issues per stage: numbers wv, wv + 8, wv + 16 of the 18 (19)
  const uint32_t HP = UNP ? P.H : P.H + 2u, WP = UNP ? P.W : P.W + 2u;  // extents of an x plane in memory
  const uint32_t last_row = P.H + 1u;

  // Workgroups are dealt to the eight XCDs (each with its own L2) in turn.  Renumber them so
  // that an XCD works on neighbouring strips: those share the 128-byte lines at strip borders.
  uint32_t vblock = blockIdx.x;
  if ((gridDim.x & 7u) == 0u) vblock = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const uint32_t co_blk = blockIdx.y / P.ci_blocks, ci_blk = blockIdx.y - co_blk * P.ci_blocks;
  const uint32_t ci0 = 64u * ci_blk, co0 = 64u * co_blk;
  for (uint32_t item = vblock; item < P.items; item += gridDim.x) {
    uint32_t strip, plane, tile, n;
    P.div_strips.divmod(item, plane, strip);
    P.div_N.divmod(plane, tile, n);
    const uint32_t c0 = strip * kWgCols;
    const uint16_t *x_img = P.x[tile] + (size_t)n * P.Cin * HP * WP;
    const uint16_t *dy_img = P.dy[tile] + (size_t)n * P.Cout * P.H * P.W;
    const __amdgpu_buffer_rsrc_t rsrc_x =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(x_img), 0, P.Cin * HP * WP * 2u, 0x00020000);
    const bool has_up = UNP && tile > 0u, has_dn = UNP && tile + 1u < P.num_tiles;
    const __amdgpu_buffer_rsrc_t rsrc_up = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(P.x[has_up ? tile - 1u : tile] + (size_t)n * P.Cin * HP * WP), 0, P.Cin * HP * WP * 2u,
        0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_dn = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(P.x[has_dn ? tile + 1u : tile] + (size_t)n * P.Cin * HP * WP), 0, P.Cin * HP * WP * 2u,
        0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_dy =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(dy_img), 0, P.Cout * P.H * P.W * 2u, 0x00020000);

    // Every wave issues three copies per row, numbers wv, wv + 8 and wv + 16 of the stage's 18
    // (numbers 18 and up write zeros to a spare kilobyte: the same instruction count in every
    // wave keeps the row loop free of branches and the wait counts exact).  Per-lane source
    // offsets of row 0; out of range where the channel, the piece or the column does not exist.
    uint32_t voff[3], rows_q[3], pitch_q[3], dst_q[3];
    bool isx_q[3];
#pragma unroll
    for (int q = 0; q < 3; ++q) {
      const uint32_t k = wv + 8u * q;  // uniform
      isx_q[q] = k < (uint32_t)kXLanes;
      const uint32_t j = (isx_q[q] ? k : k - (uint32_t)kXLanes) * 64u + lane;  // lane slot within the x or dy region
      const uint32_t lanes_per_row = isx_q[q] ? (uint32_t)kXLanes : (uint32_t)kWgLanes;
      const uint32_t ch = j / lanes_per_row, piece = j - ch * lanes_per_row;
      const uint32_t col = c0 + piece * 8u;
      uint32_t vx;
      if (UNP) {
        const int32_t xcol = (int32_t)col - 8;  // whole granules lie inside or outside a row (W is a multiple of 8)
        vx = (ci0 + ch < P.Cin && xcol >= 0 && xcol < (int32_t)P.W) ? ((ci0 + ch) * HP * WP + (uint32_t)xcol) * 2u : kWgOutOfRange;
      } else {
        vx = ci0 + ch < P.Cin ? ((ci0 + ch) * HP * WP + col) * 2u : kWgOutOfRange;
      }
      const uint32_t vd =
          (co0 + ch < P.Cout && piece < 8u && col < P.W) ? ((co0 + ch) * P.H * P.W + col) * 2u : kWgOutOfRange;
      voff[q] = isx_q[q] ? vx : vd;
      rows_q[q] = k >= (uint32_t)kDmaPerStage ? 0u : (isx_q[q] ? P.H + 2u : P.H);
      pitch_q[q] = isx_q[q] ? WP * 2u : P.W * 2u;
      dst_q[q] = k * 1024u;
    }

    auto dma_row = [&](uint32_t r, uint8_t *stage) {
#pragma unroll
      for (int q = 0; q < 3; ++q) {
        uint8_t *dst = dst_q[q] < (uint32_t)kStageBytes ? stage + dst_q[q] : spare;
        uint32_t v = r < rows_q[q] ? voff[q] : kWgOutOfRange;
        if (UNP && isx_q[q]) {
          // stage row r holds x row r - 1: the neighbour's last row, the tile's own rows, the other neighbour's first
          __amdgpu_buffer_rsrc_t rs = rsrc_x;
          uint32_t row = r - 1u;
          if (r == 0u) {
            rs = rsrc_up;
            row = P.H - 1u;
            if (!has_up) v = kWgOutOfRange;
          } else if (r == P.H + 1u) {
            rs = rsrc_dn;
            row = 0u;
            if (!has_dn) v = kWgOutOfRange;
          }
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, (__attribute__((address_space(3))) void *)dst, 16, v,
                                                   __builtin_amdgcn_readfirstlane(row * pitch_q[q]), 0, 0);
        } else {
          __builtin_amdgcn_raw_ptr_buffer_load_lds(isx_q[q] ? rsrc_x : rsrc_dy, (__attribute__((address_space(3))) void *)dst,
                                                   16, v, __builtin_amdgcn_readfirstlane(r * pitch_q[q]), 0, 0);
        }
      }
    };

    // dy rows as A operands (two column halves x two output-channel tiles each): rows r, r-1, r-2
    // in use plus row r+1 arriving, in four slots; x_pad rows as five dwords per column half, the
    // row in use and the row arriving
    u32x4 win[4][2][2];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int cot = 0; cot < 2; ++cot) win[a][kb][cot] = (u32x4){0u, 0u, 0u, 0u};
    u32x4 xb[2][2];
    uint32_t xe[2][2], xm[2][2];  // the dword after the 16 bytes; UNP: and the one before

    // operands of row r from its stage: dy row r -> window slot r mod 4, x_pad row r -> parity r mod 2
    auto fetch = [&](auto ph) {
      constexpr int PH = decltype(ph)::value;
      const uint8_t *src = stages[PH % kWgStages];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        xb[PH % 2][kb] = *reinterpret_cast<const u32x4 *>(src + b_off + kb * 64);
        xe[PH % 2][kb] = *reinterpret_cast<const uint32_t *>(src + b_off + kb * 64 + 16);
        if (UNP) xm[PH % 2][kb] = *reinterpret_cast<const uint32_t *>(src + b_off + kb * 64 - 4);
      }
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int cot = 0; cot < 2; ++cot)
          win[PH % 4][kb][cot] = *reinterpret_cast<const u32x4 *>(src + a_off + cot * 16 * kWgPitch + kb * 64);
    };
    // waits until this wave's copies (three per row) of all rows but the newest `behind` have landed
    auto wait_rows = [&](uint32_t behind) {
      if (behind >= 4u) {
        __builtin_amdgcn_s_waitcnt(0x0F70 | 12);
      } else {
        switch (behind) {
          case 0: __builtin_amdgcn_s_waitcnt(0x0F70 | 0); break;
          case 1: __builtin_amdgcn_s_waitcnt(0x0F70 | 3); break;
          case 2: __builtin_amdgcn_s_waitcnt(0x0F70 | 6); break;
          default: __builtin_amdgcn_s_waitcnt(0x0F70 | 9); break;
        }
      }
    };

    __syncthreads();  // the previous item's last rows have been read
#pragma unroll
    for (int q = 0; q < kWgStages; ++q)
      if ((uint32_t)q <= last_row) dma_row((uint32_t)q, stages[q]);
    wait_rows(last_row < (uint32_t)(kWgStages - 1) ? last_row : (uint32_t)(kWgStages - 1));
    __syncthreads();
    fetch(WgTag<0>());

    // One row: the MFMAs of row r run on operands fetched a step ago, while the operands of row
    // r + 1 are fetched.  PH = r mod 12 gives the stage (mod 6), the window slot (mod 4) and the
    // x_pad register set (mod 2).
    auto step = [&](auto ph, uint32_t r) {
      constexpr int PH = decltype(ph)::value;
      if (r < last_row) {
        // row r + 1 must have landed; rows r + 2 .. r + 5 may stay in flight
        const uint32_t rest = last_row - (r + 1u);
        wait_rows(rest < (uint32_t)(kWgStages - 2) ? rest : (uint32_t)(kWgStages - 2));
      }
      // Row r + 1 is complete in LDS (every wave has waited for its own copies of it) and
      // everybody has fetched row r.  Not __syncthreads(): the compiler would put vmcnt(0) before
      // it and the rows meant to stay in flight would be waited for at every step.
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      if (r + (uint32_t)kWgStages <= last_row) dma_row(r + (uint32_t)kWgStages, stages[PH % kWgStages]);
      if (r < last_row) fetch(WgTag<(PH + 1) % 12>());

#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const u32x4 b0 = xb[PH % 2][kb];
        const uint32_t b4 = xe[PH % 2][kb];
        u32x4 b1;
        b1[0] = __builtin_amdgcn_alignbit(b0[1], b0[0], 16);
        b1[1] = __builtin_amdgcn_alignbit(b0[2], b0[1], 16);
        b1[2] = __builtin_amdgcn_alignbit(b0[3], b0[2], 16);
        b1[3] = __builtin_amdgcn_alignbit(b4, b0[3], 16);
        const u32x4 b2 = (u32x4){b0[1], b0[2], b0[3], b4};
        u32x4 bm;  // UNP: one column to the left
        if (UNP) {
          bm[0] = __builtin_amdgcn_alignbit(b0[0], xm[PH % 2][kb], 16);
          bm[1] = __builtin_amdgcn_alignbit(b0[1], b0[0], 16);
          bm[2] = __builtin_amdgcn_alignbit(b0[2], b0[1], 16);
          bm[3] = __builtin_amdgcn_alignbit(b0[3], b0[2], 16);
        }
        // column shifts kw = 0, 1, 2: padded x: 0, +1, +2 columns from the strip's first; unpadded: -1, 0, +1
        const u32x4 bs[3] = {UNP ? bm : b0, UNP ? b0 : b1, UNP ? b1 : b2};
#pragma unroll
        for (int kh = 0; kh < 3; ++kh) {
          const int slot = (PH + 4 - kh) % 4;  // dy row r - kh
#pragma unroll
          for (int kw = 0; kw < 3; ++kw)
#pragma unroll
            for (int cot = 0; cot < 2; ++cot)
              acc[kh][kw][cot] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                  __builtin_bit_cast(bf16x8, win[slot][kb][cot]), __builtin_bit_cast(bf16x8, bs[kw]),
                  acc[kh][kw][cot], 0, 0, 0);
        }
      }
    };

    for (uint32_t r = 0; r <= last_row; r += 12u) {
      step(WgTag<0>(), r);
      if (r + 1u <= last_row) step(WgTag<1>(), r + 1u);
      if (r + 2u <= last_row) step(WgTag<2>(), r + 2u);
      if (r + 3u <= last_row) step(WgTag<3>(), r + 3u);
      if (r + 4u <= last_row) step(WgTag<4>(), r + 4u);
      if (r + 5u <= last_row) step(WgTag<5>(), r + 5u);
      if (r + 6u <= last_row) step(WgTag<6>(), r + 6u);
      if (r + 7u <= last_row) step(WgTag<7>(), r + 7u);
      if (r + 8u <= last_row) step(WgTag<8>(), r + 8u);
      if (r + 9u <= last_row) step(WgTag<9>(), r + 9u);
      if (r + 10u <= last_row) step(WgTag<10>(), r + 10u);
      if (r + 11u <= last_row) step(WgTag<11>(), r + 11u);
    }
  }

  // D[m = 4 g + i][n = l16]: output channel 32 coh + 16 cot + 4 g + i, input channel 16 cit + l16.
  // The partial is written in register order, [wave][tap][cot][lane][i], 16 contiguous bytes per
  // lane: in filter order every lane would write lone floats 36 bytes apart, which costs five
  // times the bytes in partial-sector writes.
  floatx4 *part = reinterpret_cast<floatx4 *>(P.partial + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * kWgPartialFloats) +
                  wv * (18u * 64u) + lane;
#pragma unroll
  for (int kh = 0; kh < 3; ++kh)
#pragma unroll
    for (int kw = 0; kw < 3; ++kw)
#pragma unroll
      for (int cot = 0; cot < 2; ++cot) part[((kh * 3 + kw) * 2 + cot) * 64] = acc[kh][kw][cot];
}

// dw[co][ci][tap] = beta * dw + sum over partials, in a fixed order.  A workgroup takes 64
// consecutive elements in the partials' register order (coalesced reads), four quarters of the
// partials in parallel, and scatters the 64 sums to their places in the filter.
__global__ __launch_bounds__(256) void conv3x3_bf16_wgrad_reduce_kernel(const float *__restrict__ partial,
                                                                        uint32_t num_partials, float *dw, uint32_t Cin,
                                                                        uint32_t Cout, uint32_t ci_blocks, float beta) {
  __shared__ float part[4][64];
  const uint32_t q = threadIdx.x >> 6, j = threadIdx.x & 63u;
  const uint32_t e = blockIdx.x * 64u + j;  // < kWgPartialFloats: the grid covers it exactly
  const uint32_t co_blk = blockIdx.y / ci_blocks, ci_blk = blockIdx.y - co_blk * ci_blocks;
  {
    const float *p = partial + (size_t)blockIdx.y * num_partials * kWgPartialFloats + e;
    const uint32_t per = (num_partials + 3u) / 4u;
    const uint32_t b0 = q * per, b1 = min(b0 + per, num_partials);
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    uint32_t b = b0;
    for (; b + 4u <= b1; b += 4u) {
      s0 += p[(size_t)(b + 0u) * kWgPartialFloats];
      s1 += p[(size_t)(b + 1u) * kWgPartialFloats];
      s2 += p[(size_t)(b + 2u) * kWgPartialFloats];
      s3 += p[(size_t)(b + 3u) * kWgPartialFloats];
    }
    for (; b < b1; ++b) s0 += p[(size_t)b * kWgPartialFloats];
    part[q][j] = (s0 + s1) + (s2 + s3);
  }
  __syncthreads();
  if (q == 0) {
    // e = (((wave * 9 + tap) * 2 + cot) * 64 + lane) * 4 + i
    const uint32_t i = e & 3u, lane = (e >> 2) & 63u, cot = (e >> 8) & 1u;
    const uint32_t wt = e >> 9, tap = wt % 9u, wave = wt / 9u;
    const uint32_t co = 64u * co_blk + 32u * (wave >> 2) + 16u * cot + 4u * (lane >> 4) + i;
    const uint32_t ci = 64u * ci_blk + 16u * (wave & 3u) + (lane & 15u);
    if (co < Cout && ci < Cin) {
      float *d = dw + ((size_t)co * Cin + ci) * 9u + tap;
      float r = (part[0][j] + part[1][j]) + (part[2][j] + part[3][j]);
      if (beta != 0.f) r += beta * *d;
      *d = r;
    }
  }
}

static uint32_t wgrad_bf16_blocks(uint64_t items) {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
    n = 256;
  return (uint32_t)(items < (uint64_t)n ? items : (uint64_t)n);
}

bool conv_bf16_wgrad_mfma_supported(uint32_t Cin, uint32_t Cout, uint32_t W) {
  return (W % 8u) == 0u && (uint64_t)((Cin + 63u) / 64u) * ((Cout + 63u) / 64u) <= 65535u;
}

static uint64_t wgrad_bf16_items(uint32_t num_tiles, uint32_t N, uint32_t W) {
  return (uint64_t)num_tiles * N * ((W + kWgCols - 1) / kWgCols);
}

size_t conv_bf16_wgrad_mfma_workspace_bytes(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t W) {
  const size_t pairs = (size_t)((Cin + 63u) / 64u) * ((Cout + 63u) / 64u);
  return pairs * wgrad_bf16_blocks(wgrad_bf16_items(num_tiles, N, W)) * kWgPartialFloats * sizeof(float);
}

// Arguments are validated by the caller (pointers, alignment, workspace size, extents > 0).
int conv_bf16_wgrad_mfma(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                         const void *const *x_tiles, const void *const *dy_tiles, float *dw, float beta,
                         void *workspace, hipStream_t st, bool unpadded) {
  WgradBf16Params P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    P.x[t] = reinterpret_cast<const uint16_t *>(x_tiles[t]);
    P.dy[t] = reinterpret_cast<const uint16_t *>(dy_tiles[t]);
  }
  P.partial = reinterpret_cast<float *>(workspace);
  P.N = N; P.Cin = Cin; P.Cout = Cout; P.H = H; P.W = W;
  P.strips = (W + kWgCols - 1) / kWgCols;
  const uint64_t items = wgrad_bf16_items(num_tiles, N, W);
  if (items >= (1ull << 31)) return ADH_EINVAL;
  P.items = (uint32_t)items;
  P.div_strips = FastDiv(P.strips);
  P.div_N = FastDiv(N);
  const uint32_t blocks = wgrad_bf16_blocks(items);
  P.ci_blocks = (Cin + 63u) / 64u;
  const uint32_t pairs = P.ci_blocks * ((Cout + 63u) / 64u);
  P.num_tiles = num_tiles;
  if (unpadded)
    hipLaunchKernelGGL(conv3x3_bf16_wgrad_kernel<true>, dim3(blocks, pairs), dim3(512), 0, st, P);
  else
    hipLaunchKernelGGL(conv3x3_bf16_wgrad_kernel<false>, dim3(blocks, pairs), dim3(512), 0, st, P);
  int e = launch_status();
  if (e) return e;
  hipLaunchKernelGGL(conv3x3_bf16_wgrad_reduce_kernel, dim3(kWgPartialFloats / 64u, pairs), dim3(256), 0, st,
                     reinterpret_cast<const float *>(workspace), blocks, dw, Cin, Cout, P.ci_blocks, beta);
  return launch_status();
}

}  // namespace adh
