// 3x3 convolution at stride 2 with padding 1 over row tiles WITHOUT halo, fp32 matrix cores: backward-data.
//
// A gradient pixel dx[h][w] receives dy[i'][j'] through tap (a, b) when h = 2 i' + a - 1 and w = 2 j' + b - 1.  The
// 2 x 2 pixels dx[2i .. 2i+1][2j .. 2j+1] (a "quad", one per dy pixel (i, j)) therefore need, per channel pair,
//   dx[2i  ][2j  ] : tap (1,1) dy[i][j]
//   dx[2i  ][2j+1] : tap (1,0) dy[i][j+1] + tap (1,2) dy[i][j]
//   dx[2i+1][2j  ] : tap (0,1) dy[i+1][j] + tap (2,1) dy[i][j]
//   dx[2i+1][2j+1] : tap (0,0) dy[i+1][j+1] + tap (0,2) dy[i+1][j] + tap (2,0) dy[i][j+1] + tap (2,2) dy[i][j]
// nine multiplications of the dy patch (shifted by 0 or 1) with one tap each, into four accumulator sets.  The
// general kernel makes the four sets four workgroups that stage the same dy patch four times, hold 1, 2, 2 and 4
// taps, and write every cache line of dx in four pieces; here a workgroup owns 64 quads x 64 input channels, stages
// the dy patch and the filter rows (read as the caller holds them) once per 16 output channels, and a lane, which
// ends up with four neighbouring quads of one channel, writes two rows of eight consecutive pixels.
// dy row OH of a tile is the first row of the tile below (zero below the last tile); dy column OW is zero.
#include "adh_common.h"

#include <algorithm>

namespace adh {

constexpr uint32_t kS2Threads = 256;
constexpr uint32_t kS2CC = 16;       // output channels (the reduction) per staged chunk
constexpr uint32_t kS2Quads = 64;    // quads per workgroup
constexpr uint32_t kS2BM = 64;       // input channels per workgroup
constexpr uint32_t kS2WPitch = kS2BM * 9u + 16u;  // floats per staged output channel of the filter

struct S2BwdParams {
  const float *dy[ADH_MAX_TILES];
  float *dx[ADH_MAX_TILES];
  const float *w;
  uint32_t num_tiles, N, Cin, Cout;
  uint32_t OH, OW;          // a dy tile; the gradient tile is 2 OH x 2 OW
  uint32_t QR, QC, NBI;     // a workgroup's quads: NBI images x QR rows x QC columns (= 64)
  uint32_t PRW, PPI, PPITCH;  // patch row width (QC + 1), floats per image ((QR + 1) PRW), per staged channel
  uint32_t RB, CB, NG, MG;  // row blocks and column blocks per image and tile, image groups, input-channel groups
  float beta;
  FastDiv div_MG, div_CB, div_RB, div_NG;
};

typedef float s2_floatx4 __attribute__((ext_vector_type(4)));

static bool s2_quads(uint32_t OH, uint32_t OW, uint32_t *QR, uint32_t *QC, uint32_t *NBI);

// PJ: patch elements a thread stages per chunk (kS2CC * NBI * PPI <= 256 PJ)
template <int PJ>
__global__ __launch_bounds__(kS2Threads, 2) void conv3x3s2_bwd_data_kernel(const S2BwdParams P) {
  constexpr int WJ = (int)(kS2CC * kS2BM * 9u / 4u / kS2Threads);  // 16-byte filter pieces a thread stages per chunk
  extern __shared__ __align__(16) float s2_lds[];
  float *wl = s2_lds;                        // [kS2CC][kS2WPitch]
  float *patch = s2_lds + kS2CC * kS2WPitch;  // [kS2CC][PPITCH]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wq = wave & 1u, wm = wave >> 1;  // quad half, channel half

  uint32_t vb = blockIdx.x;
  if ((gridDim.x & 7u) == 0u) vb = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  uint32_t r1, r2, r3, mg, cb, rb, ng, tile;
  P.div_MG.divmod(vb, r1, mg);
  P.div_CB.divmod(r1, r2, cb);
  P.div_RB.divmod(r2, r3, rb);
  P.div_NG.divmod(r3, tile, ng);
  const uint32_t n0 = ng * P.NBI, i0 = rb * P.QR, j0 = cb * P.QC, m0 = mg * kS2BM;
  const uint32_t y_plane = P.OH * P.OW;
  const size_t y_image = (size_t)P.Cout * y_plane;

  // ---- staging: the thread's patch elements (output channel within the chunk, place in the patch) and where
  // they come from; an element outside the tensor points at the tile's first element and is replaced by zero
  const float *p_ptr[PJ];
  uint32_t p_dst[PJ];      // where the element goes in LDS (no place: past the end, never stored)
  uint32_t p_ok = 0;       // bit j: the element lies inside the tensor
  uint32_t p_k = 0;        // 4 bits per element: its output channel within the chunk
  const uint32_t pp = P.NBI * P.PPI;
  constexpr uint32_t kNoPlace = 0xffffffffu;
#pragma unroll
  for (int j = 0; j < PJ; ++j) {
    const uint32_t f = tid + (uint32_t)j * kS2Threads;
    const uint32_t k = f / pp, e = f - k * pp;
    const uint32_t b = e / P.PPI, e2 = e - b * P.PPI;
    const uint32_t pr = e2 / P.PRW, pc = e2 - pr * P.PRW;
    const uint32_t row = i0 + pr, col = j0 + pc;
    bool ok = k < kS2CC && n0 + b < P.N && col < P.OW && row <= P.OH;
    uint32_t from = tile, rr = row;
    if (row >= P.OH) {  // the row below the tile
      rr = 0;
      from = tile + 1u < P.num_tiles ? tile + 1u : tile;
      ok = ok && tile + 1u < P.num_tiles;
    }
    p_ptr[j] = P.dy[from] + (ok ? (size_t)(n0 + b) * y_image + rr * P.OW + col : (size_t)0);
    p_dst[j] = k < kS2CC ? k * P.PPITCH + e : kNoPlace;
    p_ok |= ok ? 1u << j : 0u;
    p_k |= (k & 15u) << (4 * j);
  }
  // the filter: for output channel co0 + k the 576 consecutive floats from input channel m0 on, 16 bytes at a
  // time (Cin is a multiple of 4, so a piece lies wholly inside or outside the filter)
  const uint32_t w_row = m0 * 9u, w_end = P.Cin * 9u;
  float ppre[PJ];
  s2_floatx4 wpre[WJ];
  uint32_t pre_co = 0;
  // (an element that does not exist loads one that does and becomes zero on the way to LDS: the selects sit on
  // the addresses, never on the loaded values, which nothing may touch before the multiplications they overlap)
  auto load_chunk = [&](uint32_t co0) {
    pre_co = co0;
#pragma unroll
    for (int j = 0; j < PJ; ++j) {
      const uint32_t co = min(co0 + ((p_k >> (4 * j)) & 15u), P.Cout - 1u);
      ppre[j] = p_ptr[j][((p_ok >> j) & 1u) ? (size_t)co * y_plane : (size_t)0];
    }
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const uint32_t f = tid + (uint32_t)j * kS2Threads;
      const uint32_t k = f / (kS2BM * 9u / 4u), rr = (f - k * (kS2BM * 9u / 4u)) * 4u;
      const uint32_t co = min(co0 + k, P.Cout - 1u);
      wpre[j] = *reinterpret_cast<const s2_floatx4 *>(P.w + (w_row + rr < w_end ? co * w_end + w_row + rr : 0u));
    }
  };
  auto store_chunk = [&]() {
#pragma unroll
    for (int j = 0; j < PJ; ++j) {
      const uint32_t k = (p_k >> (4 * j)) & 15u;
      if (p_dst[j] != kNoPlace) patch[p_dst[j]] = ((p_ok >> j) & 1u) && pre_co + k < P.Cout ? ppre[j] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const uint32_t f = tid + (uint32_t)j * kS2Threads;
      const uint32_t k = f / (kS2BM * 9u / 4u), rr = (f - k * (kS2BM * 9u / 4u)) * 4u;
      const bool ok = w_row + rr < w_end && pre_co + k < P.Cout;
      *reinterpret_cast<s2_floatx4 *>(wl + k * kS2WPitch + rr) = ok ? wpre[j] : s2_floatx4{0.f, 0.f, 0.f, 0.f};
    }
  };

  // ---- this lane's quads: quad l16 of each of its wave's two 16-quad tiles, as an offset into a patch plane
  uint32_t q_off[2];
#pragma unroll
  for (int pt = 0; pt < 2; ++pt) {
    const uint32_t q = wq * 32u + (uint32_t)pt * 16u + l16;
    const uint32_t per = P.QR * P.QC;
    const uint32_t b = q / per, q2 = q - b * per;
    const uint32_t qi = q2 / P.QC, qj = q2 - qi * P.QC;
    q_off[pt] = b * P.PPI + qi * P.PRW + qj + g * P.PPITCH;
  }
  const float *b_base = wl + g * kS2WPitch + (wm * 32u + l16) * 9u;

  // acc[class 2 pr + pc][quad tile][channel tile]
  s2_floatx4 acc[4][2][2];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int pt = 0; pt < 2; ++pt)
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) acc[c][pt][ct] = s2_floatx4{0.f, 0.f, 0.f, 0.f};

  load_chunk(0);
  for (uint32_t co0 = 0; co0 < P.Cout; co0 += kS2CC) {
    __syncthreads();
    store_chunk();
    __syncthreads();
    if (co0 + kS2CC < P.Cout) load_chunk(co0 + kS2CC);
#pragma unroll
    for (int kk = 0; kk < (int)kS2CC / 4; ++kk) {
      // the patch at the four shifts (di, dj), then tap by tap
      float a[2][2][2];
#pragma unroll
      for (int di = 0; di < 2; ++di)
#pragma unroll
        for (int dj = 0; dj < 2; ++dj)
#pragma unroll
          for (int pt = 0; pt < 2; ++pt) a[di][dj][pt] = patch[(uint32_t)(4 * kk) * P.PPITCH + q_off[pt] + (uint32_t)di * P.PRW + (uint32_t)dj];
#pragma unroll
      for (int ta = 0; ta < 3; ++ta)
#pragma unroll
        for (int tb = 0; tb < 3; ++tb) {
          float b[2];
#pragma unroll
          for (int ct = 0; ct < 2; ++ct) b[ct] = b_base[(4 * kk) * (int)kS2WPitch + ct * 144 + ta * 3 + tb];
          const int cls = (ta == 1 ? 0 : 2) + (tb == 1 ? 0 : 1);
          const int di = ta == 0 ? 1 : 0, dj = tb == 0 ? 1 : 0;
#pragma unroll
          for (int pt = 0; pt < 2; ++pt)
#pragma unroll
            for (int ct = 0; ct < 2; ++ct)
              acc[cls][pt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[di][dj][pt], b[ct], acc[cls][pt][ct], 0, 0, 0);
        }
    }
  }

  // ---- the lane holds quads 4 g .. 4 g + 3 of each tile (one dy row: QC is a multiple of 4) for channel l16 of
  // each channel tile: two rows of eight consecutive gradient pixels
  const uint32_t W = 2u * P.OW;
  const size_t x_plane = (size_t)(2u * P.OH) * W;
#pragma unroll
  for (int pt = 0; pt < 2; ++pt) {
    const uint32_t q = wq * 32u + (uint32_t)pt * 16u + 4u * g;
    const uint32_t per = P.QR * P.QC;
    const uint32_t b = q / per, q2 = q - b * per;
    const uint32_t qi = q2 / P.QC, qj = q2 - qi * P.QC;
    if (b >= P.NBI || n0 + b >= P.N || i0 + qi >= P.OH || j0 + qj >= P.OW) continue;
    float *o_px = P.dx[tile] + (size_t)(n0 + b) * P.Cin * x_plane + (size_t)(2u * (i0 + qi)) * W + 2u * (j0 + qj);
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
      const uint32_t m = m0 + wm * 32u + (uint32_t)ct * 16u + l16;
      if (m >= P.Cin) continue;
      float *o = o_px + (size_t)m * x_plane;
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        const s2_floatx4 e = acc[2 * pr][pt][ct], d = acc[2 * pr + 1][pt][ct];
        s2_floatx4 lo = {e[0], d[0], e[1], d[1]}, hi = {e[2], d[2], e[3], d[3]};
        float *row = o + (size_t)pr * W;
        if (P.beta != 0.f) {
          lo += *reinterpret_cast<const s2_floatx4 *>(row);
          hi += *reinterpret_cast<const s2_floatx4 *>(row + 4);
        }
        *reinterpret_cast<s2_floatx4 *>(row) = lo;
        *reinterpret_cast<s2_floatx4 *>(row + 4) = hi;
      }
    }
  }
}

// Backward-data of a 3x3 window at stride 2, padding 1, over fp32 tiles of H x W without halo (dy tiles of
// H/2 x W/2).  ADH_EUNIMPL: not a shape this kernel serves (the caller takes the general kernel); nothing launched.
int conv3x3s2_bwd_data_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                           const void *w, const void *const *dy_tiles, void *const *dx_tiles, float beta,
                           hipStream_t st) {
  if (H % 2u != 0u || W % 2u != 0u || H == 0 || W == 0) return ADH_EUNIMPL;
  const uint32_t OH = H / 2u, OW = W / 2u;
  uint32_t QR, QC, NBI;
  if (!s2_quads(OH, OW, &QR, &QC, &NBI)) return ADH_EUNIMPL;
  if (!aligned_to(w, 16) || Cin % 4u != 0u) return ADH_EUNIMPL;
  for (uint32_t t = 0; t < num_tiles; ++t)
    if (!aligned_to(dx_tiles[t], 16) || !aligned_to(dy_tiles[t], 4)) return ADH_EUNIMPL;
  if ((uint64_t)Cin * Cout * 9u >= (1ull << 31) || (uint64_t)H * W >= (1ull << 30)) return ADH_EUNIMPL;

  S2BwdParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    P.dy[t] = reinterpret_cast<const float *>(dy_tiles[t]);
    P.dx[t] = reinterpret_cast<float *>(dx_tiles[t]);
  }
  P.w = reinterpret_cast<const float *>(w);
  P.num_tiles = num_tiles; P.N = N; P.Cin = Cin; P.Cout = Cout;
  P.OH = OH; P.OW = OW;
  P.QR = QR; P.QC = QC; P.NBI = NBI;
  P.PRW = QC + 1u;
  P.PPI = (QR + 1u) * P.PRW;
  const uint32_t pp = NBI * P.PPI;
  // the four shifted reads of a wave cover runs of 16 consecutive floats in 4 channel planes: planes 16 banks apart
  P.PPITCH = (pp + 63u) / 64u * 64u + 16u;
  P.RB = OH / QR; P.CB = OW / QC; P.NG = (N + NBI - 1u) / NBI; P.MG = (Cin + kS2BM - 1u) / kS2BM;
  P.beta = beta;
  P.div_MG = FastDiv(P.MG); P.div_CB = FastDiv(P.CB); P.div_RB = FastDiv(P.RB); P.div_NG = FastDiv(P.NG);
  const uint64_t blocks = (uint64_t)num_tiles * P.NG * P.RB * P.CB * P.MG;
  if (blocks == 0 || blocks >= (1ull << 31)) return ADH_EUNIMPL;
  const uint32_t pj = (kS2CC * pp + kS2Threads - 1u) / kS2Threads;
  const size_t lds = (size_t)(kS2CC * kS2WPitch + kS2CC * P.PPITCH) * sizeof(float);
  if (lds > 64u * 1024u) return ADH_EUNIMPL;
  if (pj <= 6u)
    hipLaunchKernelGGL((conv3x3s2_bwd_data_kernel<6>), dim3((uint32_t)blocks), dim3(kS2Threads), lds, st, P);
  else if (pj <= 8u)
    hipLaunchKernelGGL((conv3x3s2_bwd_data_kernel<8>), dim3((uint32_t)blocks), dim3(kS2Threads), lds, st, P);
  else
    return ADH_EUNIMPL;
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// forward: y[co][i][j] = sum over ci and taps of w[co][ci][a][b] * x[ci][2 i + a - 1][2 j + b - 1]
// A workgroup owns 64 output pixels (NBI images x QR rows x QC columns) x 64 output channels and stages, per 16
// input channels, the (2 QR + 1) x (2 QC + 1) input patch of every image and the filter rows as the caller holds
// them.  A patch row is stored with its even columns first and its odd columns after them, so that the 16
// pixels of a matrix tile read 16 consecutive floats for every tap.  Input row -1 of a tile is the last row of
// the tile above (zero above the first tile); column -1 is zero.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kS2FwdWPitch = kS2CC * 9u + 4u;  // floats per staged output channel: 16 input channels x 9 taps

struct S2FwdParams {
  const float *x[ADH_MAX_TILES];
  float *y[ADH_MAX_TILES];
  const float *w;
  uint32_t num_tiles, N, Cin, Cout;
  uint32_t OH, OW;
  uint32_t QR, QC, NBI;
  uint32_t PRW, PPI, PPITCH;  // patch row width (2 QC + 1), floats per image ((2 QR + 1) PRW), per staged channel
  uint32_t RB, CB, NG, MG;
  float beta;
  FastDiv div_MG, div_CB, div_RB, div_NG, div_PPI, div_PRW;
};

// NP: patch places a thread stages (NBI * PPI <= 128 NP); threads 0-127 stage them for the chunk's first eight
// input channels, threads 128-255 for the other eight
template <int NP>
__global__ __launch_bounds__(kS2Threads, 2) void conv3x3s2_fwd_kernel(const S2FwdParams P) {
  constexpr int WJ = (int)(kS2BM * kS2CC * 9u / 4u / kS2Threads);  // 16-byte filter pieces per thread and chunk
  constexpr uint32_t kRowPieces = kS2CC * 9u / 4u;                  // pieces per output channel
  extern __shared__ __align__(16) float s2_lds[];
  float *wl = s2_lds;                            // [kS2BM][kS2FwdWPitch]
  float *patch = s2_lds + kS2BM * kS2FwdWPitch;  // [kS2CC][PPITCH]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wq = wave & 1u, wm = wave >> 1;

  uint32_t vb = blockIdx.x;
  if ((gridDim.x & 7u) == 0u) vb = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  uint32_t r1, r2, r3, mg, cb, rb, ng, tile;
  P.div_MG.divmod(vb, r1, mg);
  P.div_CB.divmod(r1, r2, cb);
  P.div_RB.divmod(r2, r3, rb);
  P.div_NG.divmod(r3, tile, ng);
  const uint32_t n0 = ng * P.NBI, i0 = rb * P.QR, j0 = cb * P.QC, m0 = mg * kS2BM;
  const uint32_t H = 2u * P.OH, W = 2u * P.OW;
  const uint32_t x_plane = H * W;
  const float *x_own = P.x[tile];
  const float *x_up = P.x[tile > 0u ? tile - 1u : tile];

  // ---- staging: the thread's places in the patch (the same for each of its eight channels).  Offsets are relative
  // to the tile, or to the tile above for input row -1
  const uint32_t half = tid >> 7, t128 = tid & 127u;
  uint32_t p_off[NP], p_dst[NP];
  uint32_t p_ok = 0, p_up = 0, p_has = 0;  // inside the tensor / from the tile above / a place of the patch
  const uint32_t even_cols = P.QC + 1u;
  const uint32_t pp = P.NBI * P.PPI;
#pragma unroll
  for (int j = 0; j < NP; ++j) {
    const uint32_t e = t128 + (uint32_t)j * 128u;
    uint32_t b, e2, pr, pc;
    P.div_PPI.divmod(e, b, e2);
    P.div_PRW.divmod(e2, pr, pc);
    const int32_t row = (int32_t)(2u * i0 + pr) - 1, col = (int32_t)(2u * j0 + pc) - 1;
    const bool has = e < pp;
    bool ok = has && n0 + b < P.N && col >= 0;
    const bool up = row < 0;
    if (up) ok = ok && tile > 0u;
    const uint32_t rr = up ? H - 1u : (uint32_t)row;
    p_off[j] = ok ? (n0 + b) * P.Cin * x_plane + rr * W + (uint32_t)col : 0u;
    // even columns of the patch row first, odd ones after them
    p_dst[j] = b * P.PPI + pr * P.PRW + ((pc & 1u) ? even_cols + (pc >> 1) : (pc >> 1));
    p_ok |= ok ? 1u << j : 0u;
    p_up |= (ok && up) ? 1u << j : 0u;
    p_has |= has ? 1u << j : 0u;
  }
  const uint32_t w_end = P.Cin * 9u;

  float ppre[NP][8];
  s2_floatx4 wpre[WJ];
  uint32_t pre_ci = 0;
  auto load_chunk = [&](uint32_t ci0) {
    pre_ci = ci0;
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      const float *base = ((p_up >> j) & 1u) ? x_up : x_own;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const uint32_t ci = min(ci0 + half * 8u + (uint32_t)c, P.Cin - 1u);
        ppre[j][c] = base[((p_ok >> j) & 1u) ? p_off[j] + ci * x_plane : 0u];
      }
    }
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const uint32_t f = tid + (uint32_t)j * kS2Threads;
      const uint32_t co_l = f / kRowPieces, rr = (f - co_l * kRowPieces) * 4u;
      const uint32_t co = min(m0 + co_l, P.Cout - 1u);
      const uint32_t at = ci0 * 9u + rr;  // within the output channel's Cin * 9 floats
      wpre[j] = *reinterpret_cast<const s2_floatx4 *>(P.w + (at < w_end ? co * w_end + at : 0u));
    }
  };
  auto store_chunk = [&]() {
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      if (!((p_has >> j) & 1u)) continue;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const uint32_t k = half * 8u + (uint32_t)c;
        patch[k * P.PPITCH + p_dst[j]] = ((p_ok >> j) & 1u) && pre_ci + k < P.Cin ? ppre[j][c] : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < WJ; ++j) {
      const uint32_t f = tid + (uint32_t)j * kS2Threads;
      const uint32_t co_l = f / kRowPieces, rr = (f - co_l * kRowPieces) * 4u;
      const bool ok = pre_ci * 9u + rr < w_end && m0 + co_l < P.Cout;
      *reinterpret_cast<s2_floatx4 *>(wl + co_l * kS2FwdWPitch + rr) = ok ? wpre[j] : s2_floatx4{0.f, 0.f, 0.f, 0.f};
    }
  };

  // ---- this lane's pixels: pixel l16 of each of its wave's two 16-pixel tiles
  uint32_t q_off[2];
#pragma unroll
  for (int pt = 0; pt < 2; ++pt) {
    const uint32_t q = wq * 32u + (uint32_t)pt * 16u + l16;
    const uint32_t per = P.QR * P.QC;
    const uint32_t b = q / per, q2 = q - b * per;
    const uint32_t qi = q2 / P.QC, qj = q2 - qi * P.QC;
    q_off[pt] = b * P.PPI + 2u * qi * P.PRW + qj + g * P.PPITCH;
  }
  const float *b_base = wl + (wm * 32u + l16) * kS2FwdWPitch + g * 9u;
  // where tap column tb = 0, 1, 2 lies relative to the pixel's place in the even half of a patch row
  const uint32_t tap_col[3] = {0u, even_cols, 1u};

  s2_floatx4 acc[2][2];
#pragma unroll
  for (int pt = 0; pt < 2; ++pt)
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) acc[pt][ct] = s2_floatx4{0.f, 0.f, 0.f, 0.f};

  load_chunk(0);
  for (uint32_t ci0 = 0; ci0 < P.Cin; ci0 += kS2CC) {
    __syncthreads();
    store_chunk();
    __syncthreads();
    if (ci0 + kS2CC < P.Cin) load_chunk(ci0 + kS2CC);
#pragma unroll
    for (int kk = 0; kk < (int)kS2CC / 4; ++kk) {
#pragma unroll
      for (int ta = 0; ta < 3; ++ta)
#pragma unroll
        for (int tb = 0; tb < 3; ++tb) {
          float a[2], b[2];
#pragma unroll
          for (int pt = 0; pt < 2; ++pt)
            a[pt] = patch[(uint32_t)(4 * kk) * P.PPITCH + q_off[pt] + (uint32_t)ta * P.PRW + tap_col[tb]];
#pragma unroll
          for (int ct = 0; ct < 2; ++ct) b[ct] = b_base[ct * 16 * (int)kS2FwdWPitch + kk * 36 + ta * 3 + tb];
#pragma unroll
          for (int pt = 0; pt < 2; ++pt)
#pragma unroll
            for (int ct = 0; ct < 2; ++ct)
              acc[pt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[pt], b[ct], acc[pt][ct], 0, 0, 0);
        }
    }
  }

  // ---- the lane holds pixels 4 g .. 4 g + 3 of each tile (one output row) for channel l16 of each channel tile
  const size_t y_plane = (size_t)P.OH * P.OW;
#pragma unroll
  for (int pt = 0; pt < 2; ++pt) {
    const uint32_t q = wq * 32u + (uint32_t)pt * 16u + 4u * g;
    const uint32_t per = P.QR * P.QC;
    const uint32_t b = q / per, q2 = q - b * per;
    const uint32_t qi = q2 / P.QC, qj = q2 - qi * P.QC;
    if (n0 + b >= P.N) continue;
    float *o_px = P.y[tile] + (size_t)(n0 + b) * P.Cout * y_plane + (size_t)(i0 + qi) * P.OW + (j0 + qj);
#pragma unroll
    for (int ct = 0; ct < 2; ++ct) {
      const uint32_t m = m0 + wm * 32u + (uint32_t)ct * 16u + l16;
      if (m >= P.Cout) continue;
      float *o = o_px + (size_t)m * y_plane;
      s2_floatx4 v = acc[pt][ct];
      if (P.beta != 0.f) v += *reinterpret_cast<const s2_floatx4 *>(o);
      *reinterpret_cast<s2_floatx4 *>(o) = v;
    }
  }
}

// the split of a tile's H/2 x W/2 output pixels into workgroups of 64: rows of 8 or 16 pixels
static bool s2_quads(uint32_t OH, uint32_t OW, uint32_t *QR, uint32_t *QC, uint32_t *NBI) {
  if (OW != 8u && OW % 16u != 0u) return false;
  *QC = std::min(OW, 16u);
  *QR = std::min(OH, kS2Quads / *QC);
  while (*QR > 1u && OH % *QR != 0u) --*QR;
  if ((kS2Quads / *QC) % *QR != 0u) return false;
  *NBI = kS2Quads / (*QC * *QR);
  return true;
}

// Forward of a 3x3 window at stride 2, padding 1, over fp32 tiles of H x W without halo (y tiles of H/2 x W/2).
// ADH_EUNIMPL: not a shape this kernel serves; nothing launched.
int conv3x3s2_fwd_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                      const void *const *x_tiles, const void *w, void *const *y_tiles, float beta, hipStream_t st) {
  if (H % 2u != 0u || W % 2u != 0u || H == 0 || W == 0) return ADH_EUNIMPL;
  const uint32_t OH = H / 2u, OW = W / 2u;
  uint32_t QR, QC, NBI;
  if (!s2_quads(OH, OW, &QR, &QC, &NBI)) return ADH_EUNIMPL;
  // With few input channels a workgroup's set-up and its first chunk, which nothing overlaps, weigh more than
  // what the kernel saves: 64 -> 128 on 32x128 tiles 0.23-0.24 ms against the general kernel's 0.22, 128 -> 256 on
  // 16x64 0.215-0.225 against 0.205; 256 -> 512 on 8x32 0.21 against 0.36, 512 -> 512 on 4x16 0.13 against 0.27.
  if (Cin < 256u) return ADH_EUNIMPL;
  if (!aligned_to(w, 16) || Cin % 4u != 0u) return ADH_EUNIMPL;
  for (uint32_t t = 0; t < num_tiles; ++t)
    if (!aligned_to(y_tiles[t], 16) || !aligned_to(x_tiles[t], 4)) return ADH_EUNIMPL;
  if ((uint64_t)Cin * Cout * 9u >= (1ull << 31) || (uint64_t)N * Cin * H * W >= (1ull << 31)) return ADH_EUNIMPL;

  S2FwdParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    P.x[t] = reinterpret_cast<const float *>(x_tiles[t]);
    P.y[t] = reinterpret_cast<float *>(y_tiles[t]);
  }
  P.w = reinterpret_cast<const float *>(w);
  P.num_tiles = num_tiles; P.N = N; P.Cin = Cin; P.Cout = Cout;
  P.OH = OH; P.OW = OW;
  P.QR = QR; P.QC = QC; P.NBI = NBI;
  P.PRW = 2u * QC + 1u;
  P.PPI = (2u * QR + 1u) * P.PRW;
  const uint32_t pp = NBI * P.PPI;
  P.PPITCH = (pp + 63u) / 64u * 64u + 16u;
  P.RB = OH / QR; P.CB = OW / QC; P.NG = (N + NBI - 1u) / NBI; P.MG = (Cout + kS2BM - 1u) / kS2BM;
  P.beta = beta;
  P.div_MG = FastDiv(P.MG); P.div_CB = FastDiv(P.CB); P.div_RB = FastDiv(P.RB); P.div_NG = FastDiv(P.NG);
  P.div_PPI = FastDiv(P.PPI); P.div_PRW = FastDiv(P.PRW);
  const uint64_t blocks = (uint64_t)num_tiles * P.NG * P.RB * P.CB * P.MG;
  if (blocks == 0 || blocks >= (1ull << 31)) return ADH_EUNIMPL;
  const size_t lds = (size_t)(kS2BM * kS2FwdWPitch + kS2CC * P.PPITCH) * sizeof(float);
  if (lds > 64u * 1024u || pp > 3u * 128u) return ADH_EUNIMPL;
  hipLaunchKernelGGL((conv3x3s2_fwd_kernel<3>), dim3((uint32_t)blocks), dim3(kS2Threads), lds, st, P);
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// backward-filter: dw[co][ci][a][b] = beta dw + sum over tiles, n, i, j of dy[n][co][i][j] * x[n][ci][2i+a-1][2j+b-1]
// Per tap a matrix product whose reduction runs over the pixels.  A workgroup owns 64 output channels x 32 input
// channels x 9 taps and a run of 32-pixel chunks (NBI images x QR rows x QC columns of dy); per chunk it stages the
// dy pixels and the input patch (rows split into even and odd columns, as in the forward kernel), and each wave
// multiplies four consecutive pixels of a row at a time: one dy operand serves all nine taps.  The sums go to
// part[split][tap][co][ci]; a second kernel adds the splits in a fixed order and writes the filter's own layout.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kS2WgPx = 32;   // pixels per chunk
constexpr uint32_t kS2WgCo = 64;   // output channels per workgroup
constexpr uint32_t kS2WgCi = 32;   // input channels per workgroup
constexpr uint32_t kS2WgYPitch = kS2WgPx + 4u;

struct S2WgradParams {
  const float *x[ADH_MAX_TILES];
  const float *dy[ADH_MAX_TILES];
  float *part;
  uint32_t num_tiles, N, Cin, Cout;
  uint32_t OH, OW;
  uint32_t QR, QC, NBI;
  uint32_t PRW, PPI, XP;     // patch row width, floats per image, per staged input channel (4 mod 64)
  uint32_t RB, CB, NG;
  uint32_t COB, CIB;         // blocks of output / input channels
  uint32_t chunks, chunks_per_split;
  FastDiv div_CIB, div_COB, div_CB, div_RB, div_NG, div_PPI, div_PRW;
};

__global__ __launch_bounds__(kS2Threads, 2) void conv3x3s2_wgrad_kernel(const S2WgradParams P) {
  constexpr int NP = 3;  // patch places per lane (NBI * PPI <= 192), each for eight input channels
  extern __shared__ __align__(16) float s2_lds[];
  float *yl = s2_lds;                               // [kS2WgCo][kS2WgYPitch]
  float *xl = s2_lds + kS2WgCo * kS2WgYPitch;       // [kS2WgCi][XP]

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wo = wave & 1u, wi = wave >> 1;  // output-channel half (32), input-channel half (16)

  uint32_t vb = blockIdx.x;
  if ((gridDim.x & 7u) == 0u) vb = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  uint32_t r1, cib, cob, split;
  P.div_CIB.divmod(vb, r1, cib);
  P.div_COB.divmod(r1, split, cob);
  const uint32_t co0 = cob * kS2WgCo, ci0 = cib * kS2WgCi;
  const uint32_t c_lo = split * P.chunks_per_split, c_hi = min(P.chunks, c_lo + P.chunks_per_split);
  const uint32_t H = 2u * P.OH, W = 2u * P.OW;
  const uint32_t x_plane = H * W, y_plane = P.OH * P.OW;
  const uint32_t pp = P.NBI * P.PPI;
  const uint32_t even_cols = P.QC + 1u;

  // ---- what a thread stages is the same for every chunk but for the chunk's place in the tensor
  // dy: pixel tid % 32 of the chunk for output channels tid / 32 + 8 c
  const uint32_t ypx = tid & (kS2WgPx - 1u), yco = tid >> 5;
  uint32_t y_b, y_rel;
  {
    const uint32_t per = P.QR * P.QC;
    y_b = ypx / per;
    const uint32_t q2 = ypx - y_b * per, qi = q2 / P.QC, qj = q2 - qi * P.QC;
    y_rel = y_b * P.Cout * y_plane + qi * P.OW + qj;
  }
  // x: patch places lane + 64 j for input channels 8 wave + c
  uint32_t x_rel[NP], x_dst[NP], x_b[NP];
  uint32_t x_has = 0, x_row0 = 0, x_col0 = 0;  // bit j: a place of the patch / in its first row / in its first column
#pragma unroll
  for (int j = 0; j < NP; ++j) {
    const uint32_t e = lane + 64u * (uint32_t)j;
    uint32_t b, e2, pr, pc;
    P.div_PPI.divmod(e, b, e2);
    P.div_PRW.divmod(e2, pr, pc);
    x_b[j] = b;
    x_rel[j] = b * P.Cin * x_plane + pr * W + pc;
    x_dst[j] = b * P.PPI + pr * P.PRW + ((pc & 1u) ? even_cols + (pc >> 1) : (pc >> 1));
    x_has |= e < pp ? 1u << j : 0u;
    x_row0 |= pr == 0u ? 1u << j : 0u;
    x_col0 |= pc == 0u ? 1u << j : 0u;
  }

  float ypre[8], xpre[NP][8];
  uint32_t pre_y_ok = 0, pre_x_ok = 0;
  auto load_chunk = [&](uint32_t c) {
    uint32_t q1, q2, cb, rb, ng, tile;
    P.div_CB.divmod(c, q1, cb);
    P.div_RB.divmod(q1, q2, rb);
    P.div_NG.divmod(q2, tile, ng);
    const uint32_t n0 = ng * P.NBI, i0 = rb * P.QR, j0 = cb * P.QC;
    const float *yb = P.dy[tile] + (size_t)n0 * P.Cout * y_plane + i0 * P.OW + j0;
    pre_y_ok = n0 + y_b < P.N ? 1u : 0u;
#pragma unroll
    for (int cc = 0; cc < 8; ++cc) {
      const uint32_t co = min(co0 + yco + 8u * (uint32_t)cc, P.Cout - 1u);
      ypre[cc] = yb[pre_y_ok ? y_rel + co * y_plane : 0u];
    }
    // the patch starts one row above and one column left of the chunk's first input pixel
    const float *x_own = P.x[tile];
    const float *x_up = P.x[tile > 0u ? tile - 1u : tile];
    const int32_t base = (int32_t)(n0 * P.Cin * x_plane) + ((int32_t)(2u * i0) - 1) * (int32_t)W + (int32_t)(2u * j0) - 1;
    pre_x_ok = 0;
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      const bool up = i0 == 0u && ((x_row0 >> j) & 1u);
      const bool left = j0 == 0u && ((x_col0 >> j) & 1u);
      const bool ok = ((x_has >> j) & 1u) && n0 + x_b[j] < P.N && !left && (!up || tile > 0u);
      pre_x_ok |= ok ? 1u << j : 0u;
      // row -1 of this tile is row H - 1 of the tile above; a place outside the tensor reads the tile's first element
      const float *xb = ok && up ? x_up + x_plane : x_own;
      const int32_t off = ok ? base + (int32_t)x_rel[j] : 0;
#pragma unroll
      for (int cc = 0; cc < 8; ++cc) {
        const uint32_t ci = min(ci0 + 8u * wave + (uint32_t)cc, P.Cin - 1u);
        xpre[j][cc] = xb[off + (ok ? (int32_t)(ci * x_plane) : 0)];
      }
    }
  };
  auto store_chunk = [&]() {
#pragma unroll
    for (int cc = 0; cc < 8; ++cc) {
      const uint32_t cl = yco + 8u * (uint32_t)cc;
      yl[cl * kS2WgYPitch + ypx] = pre_y_ok && co0 + cl < P.Cout ? ypre[cc] : 0.f;
    }
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      if (!((x_has >> j) & 1u)) continue;
#pragma unroll
      for (int cc = 0; cc < 8; ++cc) {
        const uint32_t cl = 8u * wave + (uint32_t)cc;
        xl[cl * P.XP + x_dst[j]] = ((pre_x_ok >> j) & 1u) && ci0 + cl < P.Cin ? xpre[j][cc] : 0.f;
      }
    }
  };

  // ---- the eight groups of four consecutive pixels of a chunk: where the group's first pixel lies in the even half
  // of its patch row (this lane reads pixel g of the group)
  uint32_t goff[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const uint32_t p = 4u * (uint32_t)q, per = P.QR * P.QC;
    const uint32_t b = p / per, q2 = p - b * per, qi = q2 / P.QC, qj = q2 - qi * P.QC;
    goff[q] = b * P.PPI + 2u * qi * P.PRW + qj + g;
  }
  const float *a_base = yl + (wo * 32u + l16) * kS2WgYPitch + g;
  const float *b_base = xl + (wi * 16u + l16) * P.XP;
  const uint32_t tap_col[3] = {0u, even_cols, 1u};

  s2_floatx4 acc[9][2];
#pragma unroll
  for (int t = 0; t < 9; ++t)
#pragma unroll
    for (int ot = 0; ot < 2; ++ot) acc[t][ot] = s2_floatx4{0.f, 0.f, 0.f, 0.f};

  if (c_lo < c_hi) load_chunk(c_lo);
  for (uint32_t c = c_lo; c < c_hi; ++c) {
    __syncthreads();
    store_chunk();
    __syncthreads();
    if (c + 1u < c_hi) load_chunk(c + 1u);
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      float a[2];
#pragma unroll
      for (int ot = 0; ot < 2; ++ot) a[ot] = a_base[ot * 16 * (int)kS2WgYPitch + 4 * q];
#pragma unroll
      for (int ta = 0; ta < 3; ++ta)
#pragma unroll
        for (int tb = 0; tb < 3; ++tb) {
          const float b = b_base[goff[q] + (uint32_t)ta * P.PRW + tap_col[tb]];
#pragma unroll
          for (int ot = 0; ot < 2; ++ot)
            acc[ta * 3 + tb][ot] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[ot], b, acc[ta * 3 + tb][ot], 0, 0, 0);
        }
    }
  }

  // ---- the lane holds output channels 4 g .. 4 g + 3 of each tile for input channel l16, per tap
  const uint32_t ci = ci0 + wi * 16u + l16;
  const size_t taps_stride = (size_t)P.Cout * P.Cin;
  float *part = P.part + (size_t)split * 9u * taps_stride;
  if (ci < P.Cin) {
#pragma unroll
    for (int t = 0; t < 9; ++t)
#pragma unroll
      for (int ot = 0; ot < 2; ++ot)
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const uint32_t co = co0 + wo * 32u + (uint32_t)ot * 16u + 4u * g + (uint32_t)k;
          if (co < P.Cout) part[(size_t)t * taps_stride + (size_t)co * P.Cin + ci] = acc[t][ot][k];
        }
  }
}

// dw[pair][tap] = beta dw + sum over the splits of part[split][tap][pair]: a workgroup takes 64 (co, ci) pairs; its
// four waves take every fourth split each, and the four sums are added in order (the same bits on every run)
__global__ __launch_bounds__(256) void conv3x3s2_wgrad_reduce_kernel(const float *part, float *dw, uint32_t pairs,
                                                                     uint32_t nsplit, float beta) {
  __shared__ float sums[4][9][64];
  const uint32_t l = threadIdx.x & 63u, sg = threadIdx.x >> 6;
  const uint32_t pair = blockIdx.x * 64u + l;
  float s[9];
#pragma unroll
  for (int t = 0; t < 9; ++t) s[t] = 0.f;
  if (pair < pairs)
    for (uint32_t sp = sg; sp < nsplit; sp += 4u)
#pragma unroll
      for (int t = 0; t < 9; ++t) s[t] += part[((size_t)sp * 9u + (uint32_t)t) * pairs + pair];
#pragma unroll
  for (int t = 0; t < 9; ++t) sums[sg][t][l] = s[t];
  __syncthreads();
  // the block's 64 x 9 results are consecutive in dw
  for (uint32_t e = threadIdx.x; e < 576u; e += 256u) {
    const uint32_t pl = e / 9u, t = e - pl * 9u;
    if (blockIdx.x * 64u + pl >= pairs) continue;
    const float total = ((sums[0][t][pl] + sums[1][t][pl]) + sums[2][t][pl]) + sums[3][t][pl];
    const size_t o = (size_t)blockIdx.x * 576u + e;
    dw[o] = beta != 0.f ? dw[o] + total : total;
  }
}

struct S2WgradPlan {
  uint32_t QR, QC, NBI, nsplit, chunks, chunks_per_split;
  size_t part_bytes;
};

static bool s2_wgrad_plan(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                          S2WgradPlan *plan) {
  if (H % 2u != 0u || W % 2u != 0u || H == 0 || W == 0 || N == 0) return false;
  const uint32_t OH = H / 2u, OW = W / 2u;
  if (OW != 8u && OW % 16u != 0u) return false;
  plan->QC = std::min(OW, 16u);
  plan->QR = std::min(OH, kS2WgPx / plan->QC);
  while (plan->QR > 1u && OH % plan->QR != 0u) --plan->QR;
  if ((kS2WgPx / plan->QC) % plan->QR != 0u) return false;
  plan->NBI = kS2WgPx / (plan->QC * plan->QR);
  if (plan->NBI * (2u * plan->QR + 1u) * (2u * plan->QC + 1u) > 192u) return false;
  if ((uint64_t)Cin * Cout * 9u >= (1ull << 31) || (uint64_t)N * Cin * H * W >= (1ull << 31)) return false;
  const uint64_t chunks = (uint64_t)num_tiles * ((N + plan->NBI - 1u) / plan->NBI) * (OH / plan->QR) * (OW / plan->QC);
  if (chunks == 0 || chunks >= (1ull << 31)) return false;
  plan->chunks = (uint32_t)chunks;
  const uint32_t out_tiles = ((Cout + kS2WgCo - 1u) / kS2WgCo) * ((Cin + kS2WgCi - 1u) / kS2WgCi);
  // two workgroups per CU, and at least four chunks each: every split writes and re-reads a whole filter gradient
  const uint32_t nsplit = std::max(1u, std::min(plan->chunks / 4u, (512u + out_tiles - 1u) / out_tiles));
  plan->chunks_per_split = (plan->chunks + nsplit - 1u) / nsplit;
  plan->nsplit = (plan->chunks + plan->chunks_per_split - 1u) / plan->chunks_per_split;
  plan->part_bytes = (size_t)plan->nsplit * 9u * Cout * Cin * sizeof(float);
  return true;
}

// the partial sums of conv3x3s2_wgrad_try (0: not a shape it serves)
size_t conv3x3s2_wgrad_workspace(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W) {
  S2WgradPlan plan;
  if (!s2_wgrad_plan(num_tiles, N, Cin, Cout, H, W, &plan)) return 0;
  return plan.part_bytes;
}

// Filter gradient of a 3x3 window at stride 2, padding 1, over fp32 tiles of H x W without halo.  `workspace` holds
// conv3x3s2_wgrad_workspace bytes.  ADH_EUNIMPL: not a shape this kernel serves; nothing launched.
int conv3x3s2_wgrad_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                        const void *const *x_tiles, const void *const *dy_tiles, float *dwt, float beta, void *workspace,
                        hipStream_t st) {
  S2WgradPlan plan;
  if (!s2_wgrad_plan(num_tiles, N, Cin, Cout, H, W, &plan)) return ADH_EUNIMPL;
  S2WgradParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!aligned_to(x_tiles[t], 4) || !aligned_to(dy_tiles[t], 4)) return ADH_EUNIMPL;
    P.x[t] = reinterpret_cast<const float *>(x_tiles[t]);
    P.dy[t] = reinterpret_cast<const float *>(dy_tiles[t]);
  }
  P.part = reinterpret_cast<float *>(workspace);
  P.num_tiles = num_tiles; P.N = N; P.Cin = Cin; P.Cout = Cout;
  P.OH = H / 2u; P.OW = W / 2u;
  P.QR = plan.QR; P.QC = plan.QC; P.NBI = plan.NBI;
  P.PRW = 2u * plan.QC + 1u;
  P.PPI = (2u * plan.QR + 1u) * P.PRW;
  const uint32_t pp = plan.NBI * P.PPI;
  P.XP = (pp + 63u) / 64u * 64u + 4u;
  P.RB = P.OH / plan.QR; P.CB = P.OW / plan.QC; P.NG = (N + plan.NBI - 1u) / plan.NBI;
  P.COB = (Cout + kS2WgCo - 1u) / kS2WgCo; P.CIB = (Cin + kS2WgCi - 1u) / kS2WgCi;
  P.chunks = plan.chunks; P.chunks_per_split = plan.chunks_per_split;
  P.div_CIB = FastDiv(P.CIB); P.div_COB = FastDiv(P.COB); P.div_CB = FastDiv(P.CB); P.div_RB = FastDiv(P.RB);
  P.div_NG = FastDiv(P.NG); P.div_PPI = FastDiv(P.PPI); P.div_PRW = FastDiv(P.PRW);
  const uint64_t blocks = (uint64_t)plan.nsplit * P.COB * P.CIB;
  if (blocks >= (1ull << 31)) return ADH_EUNIMPL;
  const size_t lds = (size_t)(kS2WgCo * kS2WgYPitch + kS2WgCi * P.XP) * sizeof(float);
  if (lds > 64u * 1024u) return ADH_EUNIMPL;
  hipLaunchKernelGGL(conv3x3s2_wgrad_kernel, dim3((uint32_t)blocks), dim3(kS2Threads), lds, st, P);
  int e = launch_status();
  if (e) return e;
  const uint32_t pairs = Cout * Cin;
  hipLaunchKernelGGL(conv3x3s2_wgrad_reduce_kernel, dim3((pairs + 63u) / 64u), dim3(256), 0, st, P.part, dwt, pairs,
                     plan.nsplit, beta);
  return launch_status();
}

}  // namespace adh
