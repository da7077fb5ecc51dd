// 1x1 convolution (the projection shortcut of a residual block) at stride 1 or 2 on the fp32 matrix cores,
// forward and backward-data: a plain matrix product over channels,
//   forward      : y[n][m][i][j]      (+)= sum over c of w[m][c] * x[n][c][i s][j s]
//   backward-data: dx[n][c][i s][j s] (+)= sum over m of w[m][c] * dy[n][m][i][j];  with beta = 0 the pixels of dx
//                  that no output pixel reads (odd rows and columns at stride 2) become zero in the same pass.
// The general kernel serves these shapes too, but a window of one tap leaves it two barriers for every few
// multiplications, and at stride 2 its backward pass scatters single floats; here a workgroup multiplies a
// block of pixels by a block of channels over ALL reduction channels, 32 at a time, and a lane stores four
// neighbouring pixels at once.
//
// The "pixels" are the sample points (i, j) of every image of every tile, numbered tile by tile, image by image,
// row by row, so that small tiles (2 x 8 in the last stage of a row-split ResNet) still fill a workgroup.
// v_mfma_f32_16x16x4_f32 takes the pixels as its row operand: a lane ends up with four consecutive pixels of one
// channel.  Reads the filter as the caller holds it: no reordering kernel, no workspace.
#include "adh_common.h"

#include <algorithm>

namespace adh {

constexpr uint32_t kPwThreads = 256;
constexpr uint32_t kPwKC = 32;  // reduction channels per staged chunk

struct PwParams {
  const float *in[ADH_MAX_TILES];
  float *out[ADH_MAX_TILES];
  const float *w;
  uint32_t num_tiles, N;
  uint32_t K, M;                    // reduction channels, produced channels
  uint32_t w_k_stride, w_m_stride;  // distance in w of two reduction channels / two produced channels
  uint32_t GI, GJ;                  // sample points per image and tile: the rows and columns of y (dy)
  uint32_t in_plane, in_W;          // elements per channel plane and per row of the operand tensor
  uint32_t out_plane, out_W;        // the same of the produced tensor
  uint32_t total_px;                // num_tiles * N * GI * GJ
  uint32_t MG;                      // blocks of produced channels
  float beta;
  FastDiv div_GJ, div_GI, div_N, div_MG;
};

typedef float pw_floatx4 __attribute__((ext_vector_type(4)));

// PT, CT: 16-wide pixel / channel tiles per wave (the workgroup's four waves form a 2 x 2 grid: 32 PT pixels by
// 32 CT channels).  BWD: backward-data (the filter is read along its input channels, the output is strided).
// S: the stride (1 or 2).
template <int PT, int CT, bool BWD, int S>
__global__ __launch_bounds__(kPwThreads, 2) void conv1x1_kernel(const PwParams P) {
  constexpr uint32_t BP = 32u * PT, BM = 32u * CT;
  // pitches that spread a wave's 64 operand reads over 64 banks: lane (l16, g) reads pixel l16 of channel g, or
  // channel l16 at reduction index g
  constexpr uint32_t XP = BP + 16u;
  constexpr uint32_t WP = BWD ? BM + 16u : kPwKC + 4u;
  constexpr uint32_t W_ROWS = BWD ? kPwKC : BM;
  constexpr int XN = (int)(kPwKC * BP / kPwThreads);  // staged operand elements per thread and chunk
  constexpr int WN = (int)(kPwKC * BM / kPwThreads);
  constexpr uint32_t XK_STEP = kPwThreads / BP;       // channels between a thread's operand elements
  __shared__ float xl[kPwKC * XP];
  __shared__ float wl[W_ROWS * WP];
  __shared__ const float *in_tbl[ADH_MAX_TILES];
  __shared__ float *out_tbl[ADH_MAX_TILES];

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wp = wave & 1u, wc = wave >> 1;
  if (tid < P.num_tiles) {
    in_tbl[tid] = P.in[tid];
    out_tbl[tid] = P.out[tid];
  }
  __syncthreads();

  // Workgroups are dealt to the eight XCDs in turn; renumber them so that the channel blocks of one pixel
  // block, which read the same pixels, share an XCD's cache.
  uint32_t vb = blockIdx.x;
  if ((gridDim.x & 7u) == 0u) vb = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  uint32_t pb, mg;
  P.div_MG.divmod(vb, pb, mg);
  const uint32_t p0 = pb * BP, m0 = mg * BM;

  auto decode = [&](uint32_t p, uint32_t &tile, uint32_t &n, uint32_t &i, uint32_t &j) {
    uint32_t r, r2;
    P.div_GJ.divmod(p, r, j);
    P.div_GI.divmod(r, r2, i);
    P.div_N.divmod(r2, tile, n);
  };

  // ---- staging: this thread's pixel (the same for all its operand elements) and filter elements
  const uint32_t xp = tid & (BP - 1u), xk0 = tid / BP;
  const bool x_live = p0 + xp < P.total_px;
  const float *x_ptr;
  {
    uint32_t tile, n, i, j;
    decode(x_live ? p0 + xp : 0u, tile, n, i, j);
    const uint32_t step = BWD ? 1u : (uint32_t)S;
    x_ptr = in_tbl[tile] + (size_t)n * P.K * P.in_plane + (size_t)(i * step) * P.in_W + j * step;
  }
  uint32_t w_off[WN];   // offset in w of the element's produced channel; lanes outside the filter take channel 0
  uint32_t w_ok = 0;    // bit e: the produced channel exists
#pragma unroll
  for (int e = 0; e < WN; ++e) {
    const uint32_t f = tid + (uint32_t)e * kPwThreads;
    const uint32_t mm = BWD ? f % BM : f / kPwKC;
    const bool ok = m0 + mm < P.M;
    w_off[e] = ok ? (m0 + mm) * P.w_m_stride : 0u;
    w_ok |= ok ? 1u << e : 0u;
  }

  float xpre[XN], wpre[WN];
  uint32_t pre_k0 = 0;
  // (what does not exist loads an element that does and is replaced by zero on the way to LDS: a branch or a
  // select next to the loads would make the wave wait for them before the multiplications they overlap)
  auto load_chunk = [&](uint32_t k0) {
    pre_k0 = k0;
#pragma unroll
    for (int e = 0; e < XN; ++e) {
      const uint32_t k = min(k0 + xk0 + (uint32_t)e * XK_STEP, P.K - 1u);
      xpre[e] = x_ptr[(size_t)k * P.in_plane];
    }
#pragma unroll
    for (int e = 0; e < WN; ++e) {
      const uint32_t f = tid + (uint32_t)e * kPwThreads;
      const uint32_t kk = BWD ? f / BM : f % kPwKC;
      wpre[e] = P.w[w_off[e] + min(k0 + kk, P.K - 1u) * P.w_k_stride];
    }
  };
  auto store_chunk = [&]() {
#pragma unroll
    for (int e = 0; e < XN; ++e) {
      const uint32_t kl = xk0 + (uint32_t)e * XK_STEP;
      xl[kl * XP + xp] = x_live && pre_k0 + kl < P.K ? xpre[e] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < WN; ++e) {
      const uint32_t f = tid + (uint32_t)e * kPwThreads;
      const uint32_t kk = BWD ? f / BM : f % kPwKC, mm = BWD ? f % BM : f / kPwKC;
      const bool ok = ((w_ok >> e) & 1u) != 0u && pre_k0 + kk < P.K;
      wl[BWD ? kk * WP + mm : mm * WP + kk] = ok ? wpre[e] : 0.f;
    }
  };

  pw_floatx4 acc[PT][CT];
#pragma unroll
  for (int pt = 0; pt < PT; ++pt)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc[pt][ct] = pw_floatx4{0.f, 0.f, 0.f, 0.f};

  const float *a_base = xl + g * XP + wp * (16u * PT) + l16;
  const float *b_base = BWD ? wl + g * WP + wc * (16u * CT) + l16 : wl + (wc * (16u * CT) + l16) * WP + g;

  load_chunk(0);
  for (uint32_t k0 = 0; k0 < P.K; k0 += kPwKC) {
    __syncthreads();  // every wave is done with the chunk before
    store_chunk();
    __syncthreads();
    if (k0 + kPwKC < P.K) load_chunk(k0 + kPwKC);  // on its way while this chunk is multiplied
#pragma unroll
    for (int q = 0; q < (int)kPwKC / 4; ++q) {
      float a[PT], b[CT];
#pragma unroll
      for (int pt = 0; pt < PT; ++pt) a[pt] = a_base[(4 * q) * XP + 16 * pt];
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) b[ct] = BWD ? b_base[(4 * q) * WP + 16 * ct] : b_base[(16 * ct) * WP + 4 * q];
#pragma unroll
      for (int pt = 0; pt < PT; ++pt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          acc[pt][ct] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[pt], b[ct], acc[pt][ct], 0, 0, 0);
    }
  }

  // ---- the lane holds pixels 4 g .. 4 g + 3 of each pixel tile (one row: GJ is a multiple of 4) for channel l16
  // of each channel tile
#pragma unroll
  for (int pt = 0; pt < PT; ++pt) {
    const uint32_t p = p0 + wp * (16u * PT) + 16u * pt + 4u * g;
    if (p >= P.total_px) continue;
    uint32_t tile, n, i, j;
    decode(p, tile, n, i, j);
    const uint32_t so = BWD ? (uint32_t)S : 1u;
    float *o_px = out_tbl[tile] + (size_t)n * P.M * P.out_plane + (size_t)(i * so) * P.out_W + j * so;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const uint32_t m = m0 + wc * (16u * CT) + 16u * ct + l16;
      if (m >= P.M) continue;
      float *o = o_px + (size_t)m * P.out_plane;
      const pw_floatx4 v = acc[pt][ct];
      if constexpr (!BWD || S == 1) {
        pw_floatx4 r = v;
        if (P.beta != 0.f) r += *reinterpret_cast<const pw_floatx4 *>(o);
        *reinterpret_cast<pw_floatx4 *>(o) = r;
      } else {
        pw_floatx4 lo = {v[0], 0.f, v[1], 0.f}, hi = {v[2], 0.f, v[3], 0.f};
        if (P.beta != 0.f) {
          lo += *reinterpret_cast<const pw_floatx4 *>(o);
          hi += *reinterpret_cast<const pw_floatx4 *>(o + 4);
        } else {
          // the row between this one and the next sample row belongs to no output pixel
          const pw_floatx4 z = {0.f, 0.f, 0.f, 0.f};
          *reinterpret_cast<pw_floatx4 *>(o + P.out_W) = z;
          *reinterpret_cast<pw_floatx4 *>(o + P.out_W + 4) = z;
        }
        *reinterpret_cast<pw_floatx4 *>(o) = lo;
        *reinterpret_cast<pw_floatx4 *>(o + 4) = hi;
      }
    }
  }
}

template <bool BWD, int S>
static void conv1x1_launch_tile(const PwParams &P, uint32_t pt, uint32_t ct, uint32_t blocks, hipStream_t st) {
  if (pt == 4u && ct == 4u)
    hipLaunchKernelGGL((conv1x1_kernel<4, 4, BWD, S>), dim3(blocks), dim3(kPwThreads), 0, st, P);
  else if (pt == 4u)
    hipLaunchKernelGGL((conv1x1_kernel<4, 2, BWD, S>), dim3(blocks), dim3(kPwThreads), 0, st, P);
  else
    hipLaunchKernelGGL((conv1x1_kernel<2, 2, BWD, S>), dim3(blocks), dim3(kPwThreads), 0, st, P);
}

// Forward (bwd false: in = x tiles of H x W, out = y tiles of OH x OW) or backward-data (in = dy tiles, out = dx
// tiles) of a 1x1 convolution at stride s.  ADH_EUNIMPL: not a shape these kernels serve (the caller falls back
// to the general kernel); nothing was launched then.
int conv1x1_try(bool bwd, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                uint32_t OH, uint32_t OW, uint32_t s, const void *const *in_tiles, const void *w,
                void *const *out_tiles, float beta, hipStream_t st) {
  if (s != 1u && s != 2u) return ADH_EUNIMPL;
  if (OW % 4u != 0u) return ADH_EUNIMPL;
  // backward: the sample rows and columns and the ones between them must make up the whole gradient tile
  if (bwd && (H != s * OH || W != s * OW)) return ADH_EUNIMPL;
  const uint64_t total = (uint64_t)num_tiles * N * OH * OW;
  if (total == 0 || total >= (1ull << 31)) return ADH_EUNIMPL;
  if (!aligned_to(w, 4)) return ADH_EUNIMPL;
  for (uint32_t t = 0; t < num_tiles; ++t)
    if (!aligned_to(out_tiles[t], 16) || !aligned_to(in_tiles[t], 4)) return ADH_EUNIMPL;

  PwParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    P.in[t] = reinterpret_cast<const float *>(in_tiles[t]);
    P.out[t] = reinterpret_cast<float *>(out_tiles[t]);
  }
  P.w = reinterpret_cast<const float *>(w);
  P.num_tiles = num_tiles;
  P.N = N;
  P.GI = OH; P.GJ = OW;
  if (!bwd) {
    P.K = Cin; P.M = Cout;
    P.w_k_stride = 1; P.w_m_stride = Cin;
    P.in_plane = H * W; P.in_W = W;
    P.out_plane = OH * OW; P.out_W = OW;
  } else {
    P.K = Cout; P.M = Cin;
    P.w_k_stride = Cin; P.w_m_stride = 1;
    P.in_plane = OH * OW; P.in_W = OW;
    P.out_plane = H * W; P.out_W = W;
  }
  if ((uint64_t)Cin * Cout >= (1ull << 31)) return ADH_EUNIMPL;
  P.total_px = (uint32_t)total;
  P.beta = beta;
  // the largest block of pixels and channels that still gives every CU two workgroups
  uint32_t ct = P.M > 64u ? 4u : 2u, pt = 4u;
  auto blocks_of = [&](uint32_t pt_, uint32_t ct_) {
    return (uint64_t)((total + 32u * pt_ - 1u) / (32u * pt_)) * ((P.M + 32u * ct_ - 1u) / (32u * ct_));
  };
  if (blocks_of(pt, ct) < 512u) pt = ct = 2u;
  const uint64_t blocks = blocks_of(pt, ct);
  if (blocks >= (1ull << 31)) return ADH_EUNIMPL;
  P.MG = (P.M + 32u * ct - 1u) / (32u * ct);
  P.div_GJ = FastDiv(P.GJ);
  P.div_GI = FastDiv(P.GI);
  P.div_N = FastDiv(N);
  P.div_MG = FastDiv(P.MG);
  if (!bwd) {
    if (s == 1u) conv1x1_launch_tile<false, 1>(P, pt, ct, (uint32_t)blocks, st);
    else conv1x1_launch_tile<false, 2>(P, pt, ct, (uint32_t)blocks, st);
  } else {
    if (s == 1u) conv1x1_launch_tile<true, 1>(P, pt, ct, (uint32_t)blocks, st);
    else conv1x1_launch_tile<true, 2>(P, pt, ct, (uint32_t)blocks, st);
  }
  return launch_status();
}

// ---------------------------------------------------------------------------------------------
// backward-filter of a 1x1 window at any stride:
//   dw[co][ci] = beta dw[co][ci] + sum over tiles, n, i, j of dy[n][co][i][j] * x[n][ci][i sh][j sw]
// a matrix product whose reduction runs over the pixels.  The pixels are dealt to `nsplit` workgroups per block of
// the filter gradient in runs of 32-pixel chunks; each writes its sums to part[split][co][ci] and a second kernel
// adds the splits in a fixed order: the same bits on every run.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kPwPC = 32;  // pixels per staged chunk

struct PwWgradParams {
  const float *x[ADH_MAX_TILES];
  const float *dy[ADH_MAX_TILES];
  float *part;
  uint32_t num_tiles, N, Cin, Cout;
  uint32_t GI, GJ;             // rows and columns of a dy tile
  uint32_t x_plane, x_W, sh, sw;
  uint32_t y_plane;
  uint32_t total_px, chunks_per_split;
  uint32_t CIB, COB;           // blocks of input / output channels
  FastDiv div_GJ, div_GI, div_N, div_CIB, div_COB;
};

// OT, IT: 16-wide tiles of output / input channels per wave; the four waves form a 2 x 2 grid
template <int OT, int IT>
__global__ __launch_bounds__(kPwThreads, 2) void conv1x1_wgrad_kernel(const PwWgradParams P) {
  constexpr uint32_t BCO = 32u * OT, BCI = 32u * IT;
  constexpr uint32_t LP = kPwPC + 4u;  // lane (l16, g) reads pixel g of channel l16: 64 banks
  constexpr int YN = (int)(BCO / 8u), XN = (int)(BCI / 8u);
  __shared__ float yl[BCO * LP];
  __shared__ float xl[BCI * LP];
  __shared__ const float *x_tbl[ADH_MAX_TILES];
  __shared__ const float *y_tbl[ADH_MAX_TILES];

  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wo = wave & 1u, wi = wave >> 1;
  if (tid < P.num_tiles) {
    x_tbl[tid] = P.x[tid];
    y_tbl[tid] = P.dy[tid];
  }
  __syncthreads();

  // the blocks of one split read the same pixels: keep them on one XCD
  uint32_t vb = blockIdx.x;
  if ((gridDim.x & 7u) == 0u) vb = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  uint32_t r, cib, cob, split;
  P.div_CIB.divmod(vb, r, cib);
  P.div_COB.divmod(r, split, cob);
  const uint32_t co0 = cob * BCO, ci0 = cib * BCI;

  const uint32_t px = tid & (kPwPC - 1u), ch0 = tid >> 5;  // this thread's pixel of a chunk and first channel
  const uint32_t chunk0 = split * P.chunks_per_split;
  const uint32_t nchunks =
      min(P.chunks_per_split, (P.total_px + kPwPC - 1u) / kPwPC > chunk0 ? (P.total_px + kPwPC - 1u) / kPwPC - chunk0 : 0u);

  float ypre[YN], xpre[XN];
  bool pre_live = false;
  auto load_chunk = [&](uint32_t c) {
    const uint32_t p = (chunk0 + c) * kPwPC + px;
    pre_live = p < P.total_px;
    uint32_t q, q2, tile, n, i, j;
    P.div_GJ.divmod(pre_live ? p : 0u, q, j);
    P.div_GI.divmod(q, q2, i);
    P.div_N.divmod(q2, tile, n);
    const float *yp = y_tbl[tile] + (size_t)n * P.Cout * P.y_plane + i * P.GJ + j;
    const float *xp = x_tbl[tile] + (size_t)n * P.Cin * P.x_plane + (size_t)(i * P.sh) * P.x_W + j * P.sw;
#pragma unroll
    for (int e = 0; e < YN; ++e) ypre[e] = yp[(size_t)min(co0 + ch0 + 8u * e, P.Cout - 1u) * P.y_plane];
#pragma unroll
    for (int e = 0; e < XN; ++e) xpre[e] = xp[(size_t)min(ci0 + ch0 + 8u * e, P.Cin - 1u) * P.x_plane];
  };
  auto store_chunk = [&]() {
#pragma unroll
    for (int e = 0; e < YN; ++e) yl[(ch0 + 8u * e) * LP + px] = pre_live && co0 + ch0 + 8u * e < P.Cout ? ypre[e] : 0.f;
#pragma unroll
    for (int e = 0; e < XN; ++e) xl[(ch0 + 8u * e) * LP + px] = pre_live && ci0 + ch0 + 8u * e < P.Cin ? xpre[e] : 0.f;
  };

  pw_floatx4 acc[OT][IT];
#pragma unroll
  for (int ot = 0; ot < OT; ++ot)
#pragma unroll
    for (int it = 0; it < IT; ++it) acc[ot][it] = pw_floatx4{0.f, 0.f, 0.f, 0.f};
  const float *a_base = yl + (wo * (16u * OT) + l16) * LP + g;
  const float *b_base = xl + (wi * (16u * IT) + l16) * LP + g;

  if (nchunks > 0u) load_chunk(0);
  for (uint32_t c = 0; c < nchunks; ++c) {
    __syncthreads();
    store_chunk();
    __syncthreads();
    if (c + 1u < nchunks) load_chunk(c + 1u);
#pragma unroll
    for (int q = 0; q < (int)kPwPC / 4; ++q) {
      float a[OT], b[IT];
#pragma unroll
      for (int ot = 0; ot < OT; ++ot) a[ot] = a_base[(16 * ot) * LP + 4 * q];
#pragma unroll
      for (int it = 0; it < IT; ++it) b[it] = b_base[(16 * it) * LP + 4 * q];
#pragma unroll
      for (int ot = 0; ot < OT; ++ot)
#pragma unroll
        for (int it = 0; it < IT; ++it)
          acc[ot][it] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[ot], b[it], acc[ot][it], 0, 0, 0);
    }
  }

  // the lane holds output channels 4 g .. 4 g + 3 of each tile for input channel l16
  float *part = P.part + (size_t)split * P.Cout * P.Cin;
#pragma unroll
  for (int ot = 0; ot < OT; ++ot)
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const uint32_t ci = ci0 + wi * (16u * IT) + 16u * it + l16;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t co = co0 + wo * (16u * OT) + 16u * ot + 4u * g + k;
        if (co < P.Cout && ci < P.Cin) part[(size_t)co * P.Cin + ci] = acc[ot][it][k];
      }
    }
}

// dw[e] = beta dw[e] + part[0][e] + part[1][e] + ...: four waves take every fourth split each (in four interleaved
// chains), then the four sums are added in order: a fixed order, the same bits on every run
__global__ __launch_bounds__(256) void conv1x1_wgrad_reduce_kernel(const float *part, float *dw, uint32_t elems,
                                                                   uint32_t nsplit, float beta) {
  __shared__ float sums[4][64];
  const uint32_t e = blockIdx.x * 64u + (threadIdx.x & 63u), sg = threadIdx.x >> 6;
  float s = 0.f;
  if (e < elems) {
    // four loads in flight per thread: with a few hundred splits a chain of single loads is all latency
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    uint32_t sp = sg;
    for (; sp + 12u < nsplit; sp += 16u) {
      s0 += part[(size_t)sp * elems + e];
      s1 += part[(size_t)(sp + 4u) * elems + e];
      s2 += part[(size_t)(sp + 8u) * elems + e];
      s3 += part[(size_t)(sp + 12u) * elems + e];
    }
    for (; sp < nsplit; sp += 4u) s0 += part[(size_t)sp * elems + e];
    s = (s0 + s1) + (s2 + s3);
  }
  sums[sg][threadIdx.x & 63u] = s;
  __syncthreads();
  if (sg == 0u && e < elems) {
    const uint32_t l = threadIdx.x;
    const float total = ((sums[0][l] + sums[1][l]) + sums[2][l]) + sums[3][l];
    dw[e] = beta != 0.f ? dw[e] + total : total;
  }
}

// dw[e] = beta dw[e] + the sum over the splits of part[split][e], for any kernel whose partial sums have the
// filter gradient's own layout
int split_sum_launch(const float *part, float *dw, uint32_t elems, uint32_t nsplit, float beta, hipStream_t st) {
  hipLaunchKernelGGL(conv1x1_wgrad_reduce_kernel, dim3((elems + 63u) / 64u), dim3(256), 0, st, part, dw, elems, nsplit, beta);
  return launch_status();
}

struct PwWgradPlan {
  uint32_t ot, it, nsplit, chunks_per_split;
  size_t part_bytes;
};

static bool conv1x1_wgrad_plan(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t OH, uint32_t OW,
                               PwWgradPlan *plan) {
  const uint64_t total = (uint64_t)num_tiles * N * OH * OW;
  if (total == 0 || total >= (1ull << 31) || (uint64_t)Cin * Cout >= (1ull << 31)) return false;
  plan->ot = Cout > 64u ? 4u : 2u;
  plan->it = Cin > 64u ? 4u : 2u;
  const uint32_t cob = (Cout + 32u * plan->ot - 1u) / (32u * plan->ot), cib = (Cin + 32u * plan->it - 1u) / (32u * plan->it);
  const uint32_t chunks = (uint32_t)((total + kPwPC - 1u) / kPwPC);
  // Every workgroup writes a whole block of the gradient and the second kernel reads it again: one workgroup per
  // CU, and at least four chunks each (more splits measured slower: 64 -> 128 channels over 131072 pixels 67 us with
  // 512 splits, 54 with 256).
  const uint32_t nsplit = std::max(1u, std::min(chunks / 4u, (256u + cob * cib - 1u) / (cob * cib)));
  plan->chunks_per_split = (chunks + nsplit - 1u) / nsplit;
  plan->nsplit = (chunks + plan->chunks_per_split - 1u) / plan->chunks_per_split;
  plan->part_bytes = (size_t)plan->nsplit * Cout * Cin * sizeof(float);
  return true;
}

// the partial sums of conv1x1_wgrad_try (0: not a shape it serves)
size_t conv1x1_wgrad_workspace(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t OH, uint32_t OW) {
  PwWgradPlan plan;
  if (!conv1x1_wgrad_plan(num_tiles, N, Cin, Cout, OH, OW, &plan)) return 0;
  return plan.part_bytes;
}

// x tiles of H x W, dy tiles of OH x OW, a 1x1 window at stride (sh, sw), fp32.  ADH_EUNIMPL: not served, nothing
// launched.  `workspace` holds conv1x1_wgrad_workspace bytes.
int conv1x1_wgrad_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W, uint32_t OH,
                      uint32_t OW, uint32_t sh, uint32_t sw, const void *const *x_tiles, const void *const *dy_tiles,
                      float *dwt, float beta, void *workspace, hipStream_t st) {
  PwWgradPlan plan;
  if (!conv1x1_wgrad_plan(num_tiles, N, Cin, Cout, OH, OW, &plan)) return ADH_EUNIMPL;
  PwWgradParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!aligned_to(x_tiles[t], 4) || !aligned_to(dy_tiles[t], 4)) return ADH_EUNIMPL;
    P.x[t] = reinterpret_cast<const float *>(x_tiles[t]);
    P.dy[t] = reinterpret_cast<const float *>(dy_tiles[t]);
  }
  P.part = reinterpret_cast<float *>(workspace);
  P.num_tiles = num_tiles; P.N = N; P.Cin = Cin; P.Cout = Cout;
  P.GI = OH; P.GJ = OW;
  P.x_plane = H * W; P.x_W = W; P.sh = sh; P.sw = sw;
  P.y_plane = OH * OW;
  P.total_px = num_tiles * N * OH * OW;
  P.chunks_per_split = plan.chunks_per_split;
  P.COB = (Cout + 32u * plan.ot - 1u) / (32u * plan.ot);
  P.CIB = (Cin + 32u * plan.it - 1u) / (32u * plan.it);
  P.div_GJ = FastDiv(OW); P.div_GI = FastDiv(OH); P.div_N = FastDiv(N);
  P.div_CIB = FastDiv(P.CIB); P.div_COB = FastDiv(P.COB);
  const uint64_t blocks = (uint64_t)plan.nsplit * P.COB * P.CIB;
  if (blocks >= (1ull << 31)) return ADH_EUNIMPL;
  if (plan.ot == 4u && plan.it == 4u)
    hipLaunchKernelGGL((conv1x1_wgrad_kernel<4, 4>), dim3((uint32_t)blocks), dim3(kPwThreads), 0, st, P);
  else if (plan.ot == 4u)
    hipLaunchKernelGGL((conv1x1_wgrad_kernel<4, 2>), dim3((uint32_t)blocks), dim3(kPwThreads), 0, st, P);
  else if (plan.it == 4u)
    hipLaunchKernelGGL((conv1x1_wgrad_kernel<2, 4>), dim3((uint32_t)blocks), dim3(kPwThreads), 0, st, P);
  else
    hipLaunchKernelGGL((conv1x1_wgrad_kernel<2, 2>), dim3((uint32_t)blocks), dim3(kPwThreads), 0, st, P);
  int e = launch_status();
  if (e) return e;
  const uint32_t elems = Cout * Cin;
  hipLaunchKernelGGL(conv1x1_wgrad_reduce_kernel, dim3((elems + 63u) / 64u), dim3(256), 0, st, P.part, dwt, elems,
                     plan.nsplit, beta);
  return launch_status();
}

}  // namespace adh
