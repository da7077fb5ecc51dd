// Forward convolution of an input with very few channels (an image: 1-3) over halo-padded tiles, fp32 matrix cores:
// the stem of a network (7x7 over RGB).  The general kernel multiplies four channels per step, so three channels
// waste a quarter of every step, and it stages the filter tap group by tap group between barriers.  Here the
// reduction index is the flattened (channel, tap) pair, k = (c kh + a) kw + b < 148: the 147 pairs of a 7x7x3 window
// are 37 steps of 4 with one pair of padding; the whole filter of 64 output channels (38 KB) and the input patch of
// 256 output pixels (8 rows x 32 columns) are staged once, and the multiplications then run without a barrier.
// v_mfma_f32_16x16x4_f32 takes the pixels as its row operand (a lane ends up with four neighbouring pixels of one
// output channel); lane group g of a step reads the patch at the offset of ITS pair, kept in a register per step.
#include "adh_common.h"

#include <algorithm>

namespace adh {

constexpr uint32_t kThinThreads = 256;
constexpr uint32_t kThinSteps = 37;            // reduction steps of 4 pairs
constexpr uint32_t kThinK = 4u * kThinSteps;   // 148
constexpr uint32_t kThinBR = 8, kThinBC = 32;  // a workgroup's output pixels
constexpr uint32_t kThinCo = 64;               // output channels per workgroup
// odd, so that the filter's transposing store (64 consecutive pairs of one output channel per wave) spreads over
// the banks; 38.5 KB of filter and a 6 KB patch let three workgroups share a CU
constexpr uint32_t kThinWPitch = kThinCo + 1u;
constexpr uint32_t kThinTiles = 4;  // 8 x 32 pixel tiles (one below the other) per workgroup and staged filter

struct ThinParams {
  const float *x[ADH_MAX_TILES];
  float *y[ADH_MAX_TILES];
  const float *w;
  const float *bias[ADH_MAX_TILES];  // forward: added to every pixel of its output channel after beta * y; null: none
  uint32_t N, C, M, HP, WP, OH, OW, kh, kw, sh, sw;
  uint32_t KK;            // C * kh * kw pairs
  uint32_t PRH, PRW, PP;  // patch rows, columns, floats per channel
  uint32_t NBR, NBC, MG;  // row blocks, column blocks, output-channel groups
  float beta;
  FastDiv div_NBC, div_NBR, div_MG, div_N, div_PRW, div_PP, div_kw, div_khw;
};

typedef float thin_floatx4 __attribute__((ext_vector_type(4)));

// VEC: output rows are whole groups of four pixels at 16-byte aligned addresses.  PJ: patch elements per thread
// (C * PP <= 256 PJ; 8 for a 7x7 window at stride 1, 17 at stride 2)
template <bool VEC, int PJ>
__global__ __launch_bounds__(kThinThreads, 2) void conv_thin_fwd_kernel(const ThinParams P) {
  extern __shared__ __align__(16) float thin_lds[];
  float *wl = thin_lds;                             // [kThinK][kThinWPitch]
  float *patch = thin_lds + kThinK * kThinWPitch;   // [C][PP]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wp = wave & 1u, wm = wave >> 1;  // pixel half (rows 4 wp .. 4 wp + 3), output-channel half

  uint32_t r1, r2, r3, bc, br, mg, n, tile;
  P.div_NBC.divmod(blockIdx.x, r1, bc);
  P.div_NBR.divmod(r1, r2, br);
  P.div_MG.divmod(r2, r3, mg);
  P.div_N.divmod(r3, tile, n);
  const uint32_t j0 = bc * kThinBC, m0 = mg * kThinCo;
  const float *x = P.x[tile] + (size_t)n * P.C * P.HP * P.WP;

  // ---- the filter: w[co][k] for the group's output channels, stored [k][co].  All loads first, then the stores:
  // a loop of load -> store pairs would pay one memory latency per element
  {
    constexpr int WJ = (int)(kThinCo * kThinK / kThinThreads);  // 37
    float wtmp[WJ];
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const uint32_t e = tid + (uint32_t)j * kThinThreads;
      const uint32_t co_l = e / kThinK, k = e - co_l * kThinK;
      const bool ok = k < P.KK && m0 + co_l < P.M;
      wtmp[j] = P.w[ok ? (size_t)(m0 + co_l) * P.KK + k : (size_t)0];
    }
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const uint32_t e = tid + (uint32_t)j * kThinThreads;
      const uint32_t co_l = e / kThinK, k = e - co_l * kThinK;
      const bool ok = k < P.KK && m0 + co_l < P.M;
      wl[k * kThinWPitch + co_l] = ok ? wtmp[j] : 0.f;
    }
  }
  // ---- where lane group g's pair of step q lies in the patch
  uint32_t koff[kThinSteps];
#pragma unroll
  for (int q = 0; q < (int)kThinSteps; ++q) {
    const uint32_t k = 4u * (uint32_t)q + g;
    uint32_t c, t, a, b;
    P.div_khw.divmod(k, c, t);
    P.div_kw.divmod(t, a, b);
    koff[q] = k < P.KK ? c * P.PP + a * P.PRW + b : 0u;
  }
  // this lane's pixel of each of its wave's eight 16-pixel tiles: tile pt is columns 16 (pt % 2) .. of row 4 wp + pt / 2
  uint32_t pixoff[8];
#pragma unroll
  for (int pt = 0; pt < 8; ++pt) {
    const uint32_t row = 4u * wp + (uint32_t)(pt >> 1), col = 16u * (uint32_t)(pt & 1) + l16;
    pixoff[pt] = row * P.sh * P.PRW + col * P.sw;
  }
  const float *b_base = wl + g * kThinWPitch + wm * 32u + l16;

  float *y = P.y[tile] + (size_t)n * P.M * P.OH * P.OW;
  const float *const bias_t = P.bias[tile];
  // a tile's patch: PJ elements per thread, loaded a tile ahead (in flight while the tile before is multiplied)
  const uint32_t total = P.C * P.PP;
  float ptmp[PJ];
  uint32_t pok = 0;
  auto load_patch = [&](uint32_t i0) {
    pok = 0;
#pragma unroll
    for (int j = 0; j < PJ; ++j) {
      const uint32_t e = tid + (uint32_t)j * kThinThreads;
      uint32_t c, e2, pr, pc;
      P.div_PP.divmod(e, c, e2);
      P.div_PRW.divmod(e2, pr, pc);
      const uint32_t row = i0 * P.sh + pr, col = j0 * P.sw + pc;
      const bool ok = e < total && row < P.HP && col < P.WP;
      pok |= ok ? 1u << j : 0u;
      ptmp[j] = x[ok ? ((size_t)c * P.HP + row) * P.WP + col : (size_t)0];
    }
  };
  load_patch(br * kThinTiles * kThinBR);
#pragma unroll 1
  for (uint32_t tt = 0; tt < kThinTiles; ++tt) {
    const uint32_t i0 = (br * kThinTiles + tt) * kThinBR;
    if (i0 >= P.OH) break;
    if (tt > 0u) __syncthreads();  // every wave is done with the patch before
#pragma unroll
    for (int j = 0; j < PJ; ++j) {
      const uint32_t e = tid + (uint32_t)j * kThinThreads;
      if (e < total) patch[e] = ((pok >> j) & 1u) ? ptmp[j] : 0.f;
    }
    thin_floatx4 acc[8][2];
#pragma unroll
    for (int pt = 0; pt < 8; ++pt)
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) acc[pt][ct] = thin_floatx4{0.f, 0.f, 0.f, 0.f};
    // The 37 x 8 operand addresses koff + pixoff are the same for every tile; computed once outside this loop they
    // would need 296 registers.  A zero the compiler cannot see through keeps the sums inside.
    uint32_t here = 0;
    asm volatile("" : "+v"(here));
    uint32_t pix_t[8];
#pragma unroll
    for (int pt = 0; pt < 8; ++pt) pix_t[pt] = pixoff[pt] + here;

    __syncthreads();  // the patch (and, the first time, the filter) is in place
    if (tt + 1u < kThinTiles && i0 + kThinBR < P.OH) load_patch(i0 + kThinBR);
#pragma unroll
    for (int q = 0; q < (int)kThinSteps; ++q) {
      float a[8], b[2];
#pragma unroll
      for (int pt = 0; pt < 8; ++pt) a[pt] = patch[koff[q] + pix_t[pt]];
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) b[ct] = b_base[(4 * q) * (int)kThinWPitch + 16 * ct];
#pragma unroll
      for (int pt = 0; pt < 8; ++pt)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) acc[pt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[pt], b[ct], acc[pt][ct], 0, 0, 0);
    }

    // ---- the lane holds pixels 4 g .. 4 g + 3 of each tile for channel l16 of each channel tile
#pragma unroll
    for (int pt = 0; pt < 8; ++pt) {
      const uint32_t row = i0 + 4u * wp + (uint32_t)(pt >> 1), col = j0 + 16u * (uint32_t)(pt & 1) + 4u * g;
      if (row >= P.OH || col >= P.OW) continue;
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) {
        const uint32_t m = m0 + wm * 32u + 16u * (uint32_t)ct + l16;
        if (m >= P.M) continue;
        float *o = y + ((size_t)m * P.OH + row) * P.OW + col;
        thin_floatx4 v = acc[pt][ct];
        const float bias = bias_t ? bias_t[m] : 0.f;
        if (VEC) {
          if (P.beta != 0.f) v += *reinterpret_cast<const thin_floatx4 *>(o);
          if (bias_t) v += bias;
          *reinterpret_cast<thin_floatx4 *>(o) = v;
        } else {
#pragma unroll
          for (int k = 0; k < 4; ++k)
            if (col + (uint32_t)k < P.OW) {
              float e = P.beta != 0.f ? o[k] + v[k] : v[k];
              if (bias_t) e += bias;
              o[k] = e;
            }
        }
      }
    }
  }
}

// Forward over halo-padded fp32 tiles of HP x WP for at most three input channels and Cin kh kw <= 148, any stride,
// no dilation; bias_tiles (or null): one vector of Cout floats per tile, added in the stores (y = beta * y + conv +
// bias, the order of a separate add after the convolution).  ADH_EUNIMPL: not a shape this kernel serves; nothing
// launched.
int conv_thin_fwd_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t OH,
                      uint32_t OW, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, const void *const *x_tiles,
                      const void *w, void *const *y_tiles, float beta, hipStream_t st, const float *const *bias_tiles) {
  if (Cin == 0 || Cin > 3u || Cin * kh * kw > kThinK) return ADH_EUNIMPL;
  if (!aligned_to(w, 4)) return ADH_EUNIMPL;
  bool vec = OW % 4u == 0u;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!aligned_to(x_tiles[t], 4) || !aligned_to(y_tiles[t], 4)) return ADH_EUNIMPL;
    vec = vec && aligned_to(y_tiles[t], 16);
  }
  ThinParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    P.x[t] = reinterpret_cast<const float *>(x_tiles[t]);
    P.y[t] = reinterpret_cast<float *>(y_tiles[t]);
    P.bias[t] = bias_tiles ? bias_tiles[t] : nullptr;
  }
  P.w = reinterpret_cast<const float *>(w);
  P.N = N; P.C = Cin; P.M = Cout; P.HP = HP; P.WP = WP; P.OH = OH; P.OW = OW;
  P.kh = kh; P.kw = kw; P.sh = sh; P.sw = sw;
  P.KK = Cin * kh * kw;
  P.PRH = (kThinBR - 1u) * sh + kh;
  P.PRW = (kThinBC - 1u) * sw + kw;
  P.PP = P.PRH * P.PRW;
  const size_t lds = (size_t)(kThinK * kThinWPitch + Cin * P.PP) * sizeof(float);
  if (lds > 64u * 1024u || Cin * P.PP > 17u * kThinThreads) return ADH_EUNIMPL;
  const bool small = Cin * P.PP <= 8u * kThinThreads;
  P.NBR = (OH + kThinBR * kThinTiles - 1u) / (kThinBR * kThinTiles); P.NBC = (OW + kThinBC - 1u) / kThinBC; P.MG = (Cout + kThinCo - 1u) / kThinCo;
  P.beta = beta;
  P.div_NBC = FastDiv(P.NBC); P.div_NBR = FastDiv(P.NBR); P.div_MG = FastDiv(P.MG); P.div_N = FastDiv(N);
  P.div_PRW = FastDiv(P.PRW); P.div_PP = FastDiv(P.PP); P.div_kw = FastDiv(kw); P.div_khw = FastDiv(kh * kw);
  const uint64_t blocks = (uint64_t)num_tiles * N * P.MG * P.NBR * P.NBC;
  if (blocks == 0 || blocks >= (1ull << 31)) return ADH_EUNIMPL;
  const dim3 grid((uint32_t)blocks), block(kThinThreads);
  if (vec && small) hipLaunchKernelGGL((conv_thin_fwd_kernel<true, 8>), grid, block, lds, st, P);
  else if (vec) hipLaunchKernelGGL((conv_thin_fwd_kernel<true, 17>), grid, block, lds, st, P);
  else if (small) hipLaunchKernelGGL((conv_thin_fwd_kernel<false, 8>), grid, block, lds, st, P);
  else hipLaunchKernelGGL((conv_thin_fwd_kernel<false, 17>), grid, block, lds, st, P);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// backward-filter of the same convolutions: dw[co][k] = beta dw + sum over pixels of dy[co][px] * x[pair k at px], a
// matrix product whose reduction runs over the pixels and whose columns are the (channel, tap) pairs (ten tiles of
// 16 for a 7x7x3 window: 147 of 160 columns real).  A workgroup owns 64 output channels x all pairs and a run of
// 64-pixel chunks (2 rows x 32 columns); each of its four waves takes 16 output channels: one dy operand per step
// serves the ten column tiles.  The sums go to part[split][co][k] (the filter's own layout) and a second kernel adds
// the splits in a fixed order.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kThinWgRows = 2, kThinWgCols = 32, kThinWgPx = kThinWgRows * kThinWgCols;
constexpr uint32_t kThinWgYPitch = kThinWgPx + 4u;
constexpr int kThinKT = 10;  // column tiles: up to 160 pairs

struct ThinWgradParams {
  const float *x[ADH_MAX_TILES];
  const float *dy[ADH_MAX_TILES];
  float *part;
  uint32_t N, C, M, HP, WP, OH, OW, kh, kw, sh, sw, KK;
  uint32_t PRH, PRW, PP;
  uint32_t NRC, NCC, MG;  // row chunks and column chunks per image and tile, output-channel groups
  uint32_t chunks, chunks_per_split;
  FastDiv div_MG, div_NCC, div_NRC, div_N, div_PRW, div_PP, div_kw, div_khw;
};

int split_sum_launch(const float *part, float *dw, uint32_t elems, uint32_t nsplit, float beta, hipStream_t st);

// PJ: patch elements per thread (C * PP <= 256 PJ)
template <int PJ>
__global__ __launch_bounds__(kThinThreads, 2) void conv_thin_wgrad_kernel(const ThinWgradParams P) {
  extern __shared__ __align__(16) float thin_lds[];
  float *yl = thin_lds;                               // [64 co][kThinWgYPitch]
  float *patch = thin_lds + kThinCo * kThinWgYPitch;  // [C][PP]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
  uint32_t split, mg;
  P.div_MG.divmod(blockIdx.x, split, mg);
  const uint32_t m0 = mg * kThinCo;
  const uint32_t c_lo = split * P.chunks_per_split, c_hi = min(P.chunks, c_lo + P.chunks_per_split);
  const uint32_t total = P.C * P.PP;

  // what a thread stages of a chunk: pixel tid % 64 of dy for output channels tid / 64 + 4 j; patch elements tid + 256 j
  const uint32_t ypx = tid & 63u, yrow = ypx >> 5, ycol = ypx & 31u;
  uint32_t p_rel[PJ], p_rc[PJ];  // offset in the image of the element for the chunk at (0, 0); patch row << 16 | column
#pragma unroll
  for (int j = 0; j < PJ; ++j) {
    const uint32_t e = tid + (uint32_t)j * kThinThreads;
    uint32_t c, e2, pr, pc;
    P.div_PP.divmod(e, c, e2);
    P.div_PRW.divmod(e2, pr, pc);
    p_rel[j] = (c * P.HP + pr) * P.WP + pc;
    p_rc[j] = pr << 16 | pc;
  }

  float ypre[16], ppre[PJ];
  uint32_t y_ok = 0, p_ok = 0;
  auto load_chunk = [&](uint32_t ch) {
    uint32_t q1, q2, cc, rc, n, tile;
    P.div_NCC.divmod(ch, q1, cc);
    P.div_NRC.divmod(q1, q2, rc);
    P.div_N.divmod(q2, tile, n);
    const uint32_t i0 = rc * kThinWgRows, j0 = cc * kThinWgCols;
    const float *yb = P.dy[tile] + (size_t)n * P.M * P.OH * P.OW;
    y_ok = i0 + yrow < P.OH && j0 + ycol < P.OW ? 1u : 0u;
    const uint32_t y_off = y_ok ? (i0 + yrow) * P.OW + j0 + ycol : 0u;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const uint32_t co = min(m0 + wave + 4u * (uint32_t)j, P.M - 1u);
      ypre[j] = yb[y_ok ? (size_t)co * P.OH * P.OW + y_off : (size_t)0];
    }
    const float *xb = P.x[tile] + (size_t)n * P.C * P.HP * P.WP;
    const uint32_t base = i0 * P.sh * P.WP + j0 * P.sw;
    p_ok = 0;
#pragma unroll
    for (int j = 0; j < PJ; ++j) {
      const uint32_t e = tid + (uint32_t)j * kThinThreads;
      const bool ok = e < total && i0 * P.sh + (p_rc[j] >> 16) < P.HP && j0 * P.sw + (p_rc[j] & 0xffffu) < P.WP;
      p_ok |= ok ? 1u << j : 0u;
      ppre[j] = xb[ok ? base + p_rel[j] : 0u];
    }
  };
  auto store_chunk = [&]() {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const uint32_t cl = wave + 4u * (uint32_t)j;
      yl[cl * kThinWgYPitch + ypx] = y_ok && m0 + cl < P.M ? ypre[j] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < PJ; ++j) {
      const uint32_t e = tid + (uint32_t)j * kThinThreads;
      if (e < total) patch[e] = ((p_ok >> j) & 1u) ? ppre[j] : 0.f;
    }
  };

  // column l16 of column tile kt is pair kt * 16 + l16: where it lies in the patch (a pair that does not exist reads
  // the patch's first element: its column of the result is never stored)
  uint32_t kB[kThinKT];
#pragma unroll
  for (int kt = 0; kt < kThinKT; ++kt) {
    const uint32_t k = 16u * (uint32_t)kt + l16;
    uint32_t c, t, a, b;
    P.div_khw.divmod(k, c, t);
    P.div_kw.divmod(t, a, b);
    kB[kt] = k < P.KK ? c * P.PP + a * P.PRW + b : 0u;
  }
  const float *a_base = yl + (wave * 16u + l16) * kThinWgYPitch + g;

  thin_floatx4 acc[kThinKT];
#pragma unroll
  for (int kt = 0; kt < kThinKT; ++kt) acc[kt] = thin_floatx4{0.f, 0.f, 0.f, 0.f};

  if (c_lo < c_hi) load_chunk(c_lo);
#pragma unroll 1
  for (uint32_t ch = c_lo; ch < c_hi; ++ch) {
    __syncthreads();
    store_chunk();
    __syncthreads();
    if (ch + 1u < c_hi) load_chunk(ch + 1u);
    // the sums kB + pixel offset are the same for every chunk: a zero the compiler cannot see through keeps them
    // from being worked out (160 registers) ahead of the loop
    uint32_t here = 0;
    asm volatile("" : "+v"(here));
    // Two operand sets take turns: the reads of step q + 1 are issued, then the multiplications of step q (left
    // to itself the compiler waits for every read right before the multiplication that uses it).
    auto fetch = [&](int q, float &a, float (&b)[kThinKT]) {
      // pixels 4 q .. 4 q + 3: row q / 8, columns 4 (q % 8) ..; this lane reads pixel g of them
      const uint32_t px_off = (uint32_t)(q >> 3) * P.sh * P.PRW + (4u * (uint32_t)(q & 7) + g) * P.sw + here;
      a = a_base[4 * q];
#pragma unroll
      for (int kt = 0; kt < kThinKT; ++kt) b[kt] = patch[kB[kt] + px_off];
    };
    auto multiply = [&](float a, const float (&b)[kThinKT]) {
#pragma unroll
      for (int kt = 0; kt < kThinKT; ++kt) acc[kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b[kt], acc[kt], 0, 0, 0);
    };
    constexpr int kSteps = (int)kThinWgPx / 4;
    float a0, a1, b0[kThinKT], b1[kThinKT];
    fetch(0, a0, b0);
#pragma unroll
    for (int q = 0; q < kSteps; q += 2) {
      fetch(q + 1, a1, b1);
      __builtin_amdgcn_sched_barrier(0);
      multiply(a0, b0);
      __builtin_amdgcn_sched_barrier(0);
      fetch(q + 2 < kSteps ? q + 2 : kSteps - 1, a0, b0);  // past the end: the last step again, so that every pass has the same reads in flight
      __builtin_amdgcn_sched_barrier(0);
      multiply(a1, b1);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // the lane holds output channels 4 g .. 4 g + 3 of its wave's 16 for pair l16 of each column tile
  float *part = P.part + (size_t)split * P.M * P.KK;
#pragma unroll
  for (int kt = 0; kt < kThinKT; ++kt) {
    const uint32_t k = 16u * (uint32_t)kt + l16;
    if (k >= P.KK) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const uint32_t co = m0 + wave * 16u + 4u * g + (uint32_t)r;
      if (co < P.M) part[(size_t)co * P.KK + k] = acc[kt][r];
    }
  }
}

struct ThinWgradPlan {
  uint32_t nsplit, chunks, chunks_per_split, PRH, PRW;
  size_t part_bytes, lds;
};

static bool thin_wgrad_plan(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP,
                            uint32_t OH, uint32_t OW, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw,
                            ThinWgradPlan *plan) {
  if (Cin == 0 || Cin > 3u || Cin * kh * kw > 16u * (uint32_t)kThinKT || N == 0 || OH == 0 || OW == 0) return false;
  plan->PRH = (kThinWgRows - 1u) * sh + kh;
  plan->PRW = (kThinWgCols - 1u) * sw + kw;
  if (plan->PRH >= (1u << 16) || plan->PRW >= (1u << 16)) return false;
  const uint32_t total = Cin * plan->PRH * plan->PRW;
  if (total > 8u * kThinThreads) return false;
  plan->lds = (size_t)(kThinCo * kThinWgYPitch + total) * sizeof(float);
  if ((uint64_t)Cin * HP * WP >= (1ull << 31) || (uint64_t)Cout * Cin * kh * kw >= (1ull << 31)) return false;
  const uint64_t chunks = (uint64_t)num_tiles * N * ((OH + kThinWgRows - 1u) / kThinWgRows) * ((OW + kThinWgCols - 1u) / kThinWgCols);
  if (chunks >= (1ull << 31)) return false;
  plan->chunks = (uint32_t)chunks;
  const uint32_t mg = (Cout + kThinCo - 1u) / kThinCo;
  // two workgroups per CU; at least sixteen chunks each
  const uint32_t nsplit = std::max(1u, std::min(plan->chunks / 16u, (512u + mg - 1u) / mg));
  plan->chunks_per_split = (plan->chunks + nsplit - 1u) / nsplit;
  plan->nsplit = (plan->chunks + plan->chunks_per_split - 1u) / plan->chunks_per_split;
  plan->part_bytes = (size_t)plan->nsplit * Cout * Cin * kh * kw * sizeof(float);
  return true;
}

// the partial sums of conv_thin_wgrad_try (0: not a shape it serves)
size_t conv_thin_wgrad_workspace(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP,
                                 uint32_t OH, uint32_t OW, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw) {
  ThinWgradPlan plan;
  if (!thin_wgrad_plan(num_tiles, N, Cin, Cout, HP, WP, OH, OW, kh, kw, sh, sw, &plan)) return 0;
  return plan.part_bytes;
}

// Filter gradient over halo-padded fp32 tiles for at most three input channels and Cin kh kw <= 160, any stride, no
// dilation.  `workspace` holds conv_thin_wgrad_workspace bytes.  ADH_EUNIMPL: not served; nothing launched.
int conv_thin_wgrad_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t OH,
                        uint32_t OW, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, const void *const *x_tiles,
                        const void *const *dy_tiles, float *dwt, float beta, void *workspace, hipStream_t st) {
  ThinWgradPlan plan;
  if (!thin_wgrad_plan(num_tiles, N, Cin, Cout, HP, WP, OH, OW, kh, kw, sh, sw, &plan)) return ADH_EUNIMPL;
  ThinWgradParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!aligned_to(x_tiles[t], 4) || !aligned_to(dy_tiles[t], 4)) return ADH_EUNIMPL;
    P.x[t] = reinterpret_cast<const float *>(x_tiles[t]);
    P.dy[t] = reinterpret_cast<const float *>(dy_tiles[t]);
  }
  P.part = reinterpret_cast<float *>(workspace);
  P.N = N; P.C = Cin; P.M = Cout; P.HP = HP; P.WP = WP; P.OH = OH; P.OW = OW;
  P.kh = kh; P.kw = kw; P.sh = sh; P.sw = sw; P.KK = Cin * kh * kw;
  P.PRH = plan.PRH; P.PRW = plan.PRW; P.PP = plan.PRH * plan.PRW;
  P.NRC = (OH + kThinWgRows - 1u) / kThinWgRows; P.NCC = (OW + kThinWgCols - 1u) / kThinWgCols;
  P.MG = (Cout + kThinCo - 1u) / kThinCo;
  P.chunks = plan.chunks; P.chunks_per_split = plan.chunks_per_split;
  P.div_MG = FastDiv(P.MG); P.div_NCC = FastDiv(P.NCC); P.div_NRC = FastDiv(P.NRC); P.div_N = FastDiv(N);
  P.div_PRW = FastDiv(P.PRW); P.div_PP = FastDiv(P.PP); P.div_kw = FastDiv(kw); P.div_khw = FastDiv(kh * kw);
  const uint64_t blocks = (uint64_t)plan.nsplit * P.MG;
  if (blocks >= (1ull << 31)) return ADH_EUNIMPL;
  if (Cin * P.PP <= 4u * kThinThreads)
    hipLaunchKernelGGL((conv_thin_wgrad_kernel<4>), dim3((uint32_t)blocks), dim3(kThinThreads), plan.lds, st, P);
  else
    hipLaunchKernelGGL((conv_thin_wgrad_kernel<8>), dim3((uint32_t)blocks), dim3(kThinThreads), plan.lds, st, P);
  const int e = launch_status();
  if (e) return e;
  return split_sum_launch(P.part, dwt, Cout * P.KK, plan.nsplit, beta, st);
}

}  // namespace adh
