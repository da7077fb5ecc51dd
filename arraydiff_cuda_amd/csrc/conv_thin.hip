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
  uint32_t N, C, M, HP, WP, OH, OW, kh, kw, sh, sw;
  uint32_t KK;            // C * kh * kw pairs
  uint32_t PRH, PRW, PP;  // patch rows, columns, floats per channel
  uint32_t NBR, NBC, MG;  // row blocks, column blocks, output-channel groups
  float beta;
  FastDiv div_NBC, div_NBR, div_MG, div_N, div_PRW, div_PP, div_kw, div_khw;
};

typedef float thin_floatx4 __attribute__((ext_vector_type(4)));

// VEC: output rows are whole groups of four pixels at 16-byte aligned addresses
template <bool VEC>
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
  // a tile's patch: at most 8 elements per thread, loaded a tile ahead (in flight while the tile before is multiplied)
  const uint32_t total = P.C * P.PP;
  float ptmp[8];
  uint32_t pok = 0;
  auto load_patch = [&](uint32_t i0) {
    pok = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
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
    for (int j = 0; j < 8; ++j) {
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
        if (VEC) {
          if (P.beta != 0.f) v += *reinterpret_cast<const thin_floatx4 *>(o);
          *reinterpret_cast<thin_floatx4 *>(o) = v;
        } else {
#pragma unroll
          for (int k = 0; k < 4; ++k)
            if (col + (uint32_t)k < P.OW) o[k] = P.beta != 0.f ? o[k] + v[k] : v[k];
        }
      }
    }
  }
}

// Forward over halo-padded fp32 tiles of HP x WP for at most three input channels and Cin kh kw <= 148, any stride,
// no dilation.  ADH_EUNIMPL: not a shape this kernel serves; nothing launched.
int conv_thin_fwd_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t OH,
                      uint32_t OW, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, const void *const *x_tiles,
                      const void *w, void *const *y_tiles, float beta, hipStream_t st) {
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
  }
  P.w = reinterpret_cast<const float *>(w);
  P.N = N; P.C = Cin; P.M = Cout; P.HP = HP; P.WP = WP; P.OH = OH; P.OW = OW;
  P.kh = kh; P.kw = kw; P.sh = sh; P.sw = sw;
  P.KK = Cin * kh * kw;
  P.PRH = (kThinBR - 1u) * sh + kh;
  P.PRW = (kThinBC - 1u) * sw + kw;
  P.PP = P.PRH * P.PRW;
  const size_t lds = (size_t)(kThinK * kThinWPitch + Cin * P.PP) * sizeof(float);
  if (lds > 64u * 1024u || Cin * P.PP > 8u * kThinThreads) return ADH_EUNIMPL;
  P.NBR = (OH + kThinBR * kThinTiles - 1u) / (kThinBR * kThinTiles); P.NBC = (OW + kThinBC - 1u) / kThinBC; P.MG = (Cout + kThinCo - 1u) / kThinCo;
  P.beta = beta;
  P.div_NBC = FastDiv(P.NBC); P.div_NBR = FastDiv(P.NBR); P.div_MG = FastDiv(P.MG); P.div_N = FastDiv(N);
  P.div_PRW = FastDiv(P.PRW); P.div_PP = FastDiv(P.PP); P.div_kw = FastDiv(kw); P.div_khw = FastDiv(kh * kw);
  const uint64_t blocks = (uint64_t)num_tiles * N * P.MG * P.NBR * P.NBC;
  if (blocks == 0 || blocks >= (1ull << 31)) return ADH_EUNIMPL;
  if (vec) hipLaunchKernelGGL((conv_thin_fwd_kernel<true>), dim3((uint32_t)blocks), dim3(kThinThreads), lds, st, P);
  else hipLaunchKernelGGL((conv_thin_fwd_kernel<false>), dim3((uint32_t)blocks), dim3(kThinThreads), lds, st, P);
  return launch_status();
}

}  // namespace adh
