// General slab convolution on the fp32 matrix cores: any window, stride and dilation, forward and
// backward-data (the 7x7 stem, stride-2 3x3, 1x1 projections and dilated 3x3 of the networks that
// feed halo-padded tiles to a convolution).  The 3x3 / stride-1 case has kernels of its own.
//
// One kernel serves both passes as a "tap correlation":
//   out[m][o_r + i*so_r][o_c + j*so_c] (+)= sum over c and taps t of
//       Wt[t][c][m] * in[c][i*si_r + off_r[t]][j*si_c + off_c[t]]          (zero outside `in`)
//   forward      : in = padded tile, m = output channel, taps = all (a, b) with offsets (a*dh, b*dw),
//                  si = stride, so = 1.
//   backward-data: in = dy, m = input channel, out = the whole padded gradient tile.  Padded pixels
//                  with the same residues (h' mod sh, w' mod sw) receive the same subset of taps, so
//                  each residue class is a stride-1 correlation of dy with the taps that satisfy
//                  a*dh = h' (mod sh), b*dw = w' (mod sw), offsets (h' - a*dh) / sh: up to sh*sw
//                  sub-problems in one launch, written with output stride (sh, sw).
// Implicit GEMM: M = 64 output channels per block, N = 256 output pixels per block (BR rows x BC columns, 16 n-tiles
// of 16 consecutive pixels in row-major order, 4 per wave), K = (tap, channel) in groups of 4 channels for
// v_mfma_f32_16x16x4_f32.  Per channel chunk the input patch is staged in LDS once; the filter,
// rewritten beforehand to [m group][chunk][tap][channel][m] in the workspace, is staged per tap
// group.  bf16 tensors are widened while staging and rounded when stored: the arithmetic is fp32.
#include "adh_common.h"

#include <algorithm>

namespace adh {

constexpr int kGenMaxTaps = 64;
constexpr int kGenMaxSub = 16;
constexpr uint32_t kGenThreads = 256;
constexpr uint32_t kGenLdsBytes = 64u * 1024u;

struct GenSub {
  uint32_t t0, t1;            // taps of this sub-problem
  uint32_t GI, GJ, o_r, o_c;  // output sub-grid and where it starts
  int32_t min_r, min_c;       // smallest tap offsets
  uint32_t PR, PC;            // patch rows / columns
  uint32_t nbj, blk0;         // block columns, first block of this sub-problem within an image
};

struct ConvGenParams {
  const void *in[ADH_MAX_TILES];
  void *out[ADH_MAX_TILES];
  const float *wt;
  uint32_t N, C, M, MG, in_H, in_W, out_H, out_W;
  uint32_t si_r, si_c, so_r, so_c;
  uint32_t CC, nchunks, ntaps, TG;
  uint32_t BR, BC;  // a block's output pixels per image: BR rows x BC columns, numbered row by row, 16 per n-tile
  // When an image's share (BR * BC = `live` pixels) fills at most half of the block's 256 pixel slots, the
  // block takes NB consecutive images: slot f is pixel f % live of image f / live.  NG = ceil(N / NB) image
  // groups per tile.  PPI: patch elements per image and channel; PP >= NB * PPI: pitch of a channel plane.
  uint32_t NB, NG, live, PPI;
  uint32_t PCP, PP, w_lds_floats;
  uint32_t nsub, blocks_per_image;
  // the tiles are the row tiles of one tensor in rank order and carry no halo (the NBR instances of the kernel):
  // input rows -in_H .. -1 of tile t > 0 are the last rows of tile t - 1, rows in_H .. 2 in_H - 1 of tile
  // t < num_tiles - 1 the first rows of tile t + 1; what lies outside the tensor is zero
  uint32_t num_tiles;
  // ksplit > 1: the channel chunks are dealt to ksplit workgroups per block of pixels; each writes its fp32 sums
  // to part[split][tile] (laid out like an output tile) and a second kernel adds them in a fixed order
  uint32_t ksplit, chunks_per_split;
  float *part;
  uint64_t part_tile_elems;
  float beta;
  FastDiv div_bpi, div_MG, div_N, div_PCP, div_BC, div_live, div_PPI, div_ksplit;
  GenSub sub[kGenMaxSub];
  int16_t off_r[kGenMaxTaps], off_c[kGenMaxTaps];
};

struct FilterGenParams {
  const void *w;
  float *wt;
  uint32_t M, C, m_stride, c_stride, MG, MW, nchunks, CC, ntaps;
  uint16_t tap_index[kGenMaxTaps];
};

typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float gen_ld(const float *p, size_t i) { return p[i]; }
__device__ __forceinline__ float gen_ld(const uint16_t *p, size_t i) { return bf16_bits_to_f32(p[i]); }
// base: the same address in every lane (it travels in scalar registers); boff: the lane's byte offset
__device__ __forceinline__ float gen_ld_b(const float *base, uint32_t boff) {
  return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(base) + boff);
}
__device__ __forceinline__ float gen_ld_b(const uint16_t *base, uint32_t boff) {
  return bf16_bits_to_f32(*reinterpret_cast<const uint16_t *>(reinterpret_cast<const char *>(base) + boff));
}
// p: the lane's own address
__device__ __forceinline__ float gen_ld_p(const float *, const char *p) { return *reinterpret_cast<const float *>(p); }
__device__ __forceinline__ float gen_ld_p(const uint16_t *, const char *p) {
  return bf16_bits_to_f32(*reinterpret_cast<const uint16_t *>(p));
}
__device__ __forceinline__ void gen_st(float *p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void gen_st(uint16_t *p, size_t i, float v) { p[i] = f32_to_bf16_bits(v); }

// wt[((mg * nchunks + ch) * ntaps + t) * CC + c][m] = w[(mg*MW + m) * m_stride + (ch*CC + c) * c_stride + tap_index[t]]
template <typename T>
__global__ __launch_bounds__(256) void conv_gen_filter_kernel(const FilterGenParams F) {
  const uint32_t total = F.MG * F.nchunks * F.ntaps * F.CC * F.MW;
  for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    const uint32_t m = e % F.MW;
    uint32_t r = e / F.MW;
    const uint32_t c = r % F.CC;
    r /= F.CC;
    const uint32_t t = r % F.ntaps;
    r /= F.ntaps;
    const uint32_t ch = r % F.nchunks, mg = r / F.nchunks;
    const uint32_t mm = mg * F.MW + m, cc = ch * F.CC + c;
    float v = 0.f;
    if (mm < F.M && cc < F.C)
      v = gen_ld(reinterpret_cast<const T *>(F.w), (size_t)mm * F.m_stride + (size_t)cc * F.c_stride + F.tap_index[t]);
    F.wt[e] = v;
  }
}

// CC: channels per chunk (4, 8, 16 or 32: the more, the fewer barriers; the smaller the patch must be); MT: 16-wide m-tiles per block (1, 2 or 4).
// The next (chunk, tap group)'s patch and filter rows are loaded into registers while the current
// one is multiplied; they go to LDS after the barrier that ends the current one.  The register
// budget is held to half the file, so that two workgroups share a CU and hide each other's barriers.
// NBR: the input tiles carry no halo and rows outside a tile are read from the neighbouring tiles (P.num_tiles):
// a staged element then has an address of its own instead of an offset from the tile's.
template <typename T, int CC, int MT, bool NBR = false>
__global__ __launch_bounds__(kGenThreads, 2) void conv_gen_kernel(const ConvGenParams P) {
  constexpr uint32_t MW = 16u * MT;                         // m per block
  constexpr uint32_t WPITCH = MT == 1 ? 16u : MW + 16u;     // filter row pitch: the 4 channel groups 16 banks apart
  constexpr int PFC = 32 / CC;                              // staging registers per channel plane: PP <= 256 * PFC
  constexpr int WF = 6;                                     // float4 filter registers: TG * CC * MW / 4 <= 256 * WF
  constexpr uint32_t LOG2_CQ = CC == 32 ? 3u : CC == 16 ? 2u : CC == 8 ? 1u : 0u;  // log2 of the chunk's groups of 4 channels
  extern __shared__ __align__(16) float gen_lds[];
  float *wl = gen_lds;
  float *patch = gen_lds + P.w_lds_floats;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;

  // block -> (tile, image, m group, sub-problem, block row, block column), split of the channel chunks
  uint32_t outer, inner, bid = blockIdx.x, ks = 0;
  if (P.ksplit > 1u) P.div_ksplit.divmod(blockIdx.x, bid, ks);
  const uint32_t ch_lo = ks * P.chunks_per_split, ch_hi = min(P.nchunks, ch_lo + P.chunks_per_split);
  P.div_bpi.divmod(bid, outer, inner);
  uint32_t img, mg;
  P.div_MG.divmod(outer, img, mg);
  uint32_t tile, ng;
  P.div_N.divmod(img, tile, ng);
  const uint32_t n = ng * P.NB;  // first image of this block
  uint32_t s = 0;
  while (s + 1u < P.nsub && inner >= P.sub[s + 1u].blk0) ++s;
  const GenSub &S = P.sub[s];
  const uint32_t local = inner - S.blk0;
  const uint32_t bi = local / S.nbj, bj = local - bi * S.nbj;

  const T *src = reinterpret_cast<const T *>(P.in[tile]) + (size_t)n * P.C * P.in_H * P.in_W;
  T *dst = reinterpret_cast<T *>(P.out[tile]) + (size_t)n * P.M * P.out_H * P.out_W;

  // this wave's four n-tiles: 16 consecutive pixels each of the block's BR x BC pixels numbered row by row;
  // slots past the last pixel compute pixel 0 again and store nothing
  uint32_t pix[4], row_q[4], col_q[4], img_q[4];
  bool live_q[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const uint32_t f = ((wave * 4u + q) << 4) + l16;
    uint32_t fi;
    P.div_live.divmod(f, img_q[q], fi);
    P.div_BC.divmod(fi, row_q[q], col_q[q]);
    live_q[q] = img_q[q] < P.NB && n + img_q[q] < P.N;
    pix[q] = live_q[q] ? img_q[q] * P.PPI + row_q[q] * P.si_r * P.PCP + col_q[q] * P.si_c : 0u;
    pix[q] += g * P.PP;
  }
  floatx4 acc[4][MT];
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[q][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // where this thread's PFC elements of a channel plane come from (-1: outside the input or the patch)
  const int32_t in_r0 = (int32_t)(bi * P.BR * P.si_r) + S.min_r;
  const int32_t in_c0 = (int32_t)(bj * P.BC * P.si_c) + S.min_c;
  const size_t plane = (size_t)P.in_H * P.in_W;
  const int32_t image_elems = (int32_t)(P.C * (uint32_t)plane);  // only used when NB > 1 (the host bounds NB * C * plane)
  // a byte offset into the channel plane of the block's first image, and a bit per element that exists; the
  // elements that do not (outside the input or the patch) load offset 0 and are replaced by zero
  uint32_t src_boff[PFC], src_ok = 0;
  const char *src_ptr[NBR ? PFC : 1];  // NBR: the element's address in channel 0 of the block's first image
#pragma unroll
  for (int j = 0; j < PFC; ++j) {
    const uint32_t e = tid + j * kGenThreads;
    uint32_t b, ei, r, col;
    P.div_PPI.divmod(e, b, ei);
    P.div_PCP.divmod(ei, r, col);
    const int32_t gr = in_r0 + (int32_t)r, gc = in_c0 + (int32_t)col;
    bool ok = b < P.NB && n + b < P.N && r < S.PR && col < S.PC && gc >= 0 && gc < (int32_t)P.in_W;
    if constexpr (!NBR) {
      ok = ok && gr >= 0 && gr < (int32_t)P.in_H;
      src_boff[j] = ok ? (uint32_t)((int32_t)b * image_elems + gr * (int32_t)P.in_W + gc) * (uint32_t)sizeof(T) : 0u;
    } else {
      int32_t row = gr;
      uint32_t from = tile;
      if (gr < 0) {
        row = gr + (int32_t)P.in_H;
        ok = ok && tile > 0u;
        from = tile > 0u ? tile - 1u : tile;
      } else if (gr >= (int32_t)P.in_H) {
        row = gr - (int32_t)P.in_H;
        ok = ok && tile + 1u < P.num_tiles;
        from = tile + 1u < P.num_tiles ? tile + 1u : tile;
      }
      ok = ok && row >= 0 && row < (int32_t)P.in_H;
      const T *base = reinterpret_cast<const T *>(P.in[from]) + (size_t)n * P.C * P.in_H * P.in_W;
      src_boff[j] = 0u;
      src_ptr[j] = reinterpret_cast<const char *>(base) +
                   (ok ? (size_t)((int32_t)b * image_elems + row * (int32_t)P.in_W + gc) * sizeof(T) : (size_t)0);
    }
    src_ok |= ok ? 1u << j : 0u;
  }

  float pre[CC * PFC];
  floatx4 wpre[WF];
  uint32_t pre_ch = 0;  // the chunk in `pre`
  // (what does not exist is replaced by zero in store_patch, not here: a use of the loaded values next to
  // the loads would make the wave wait for them before the multiplications they are meant to overlap)
  auto load_patch = [&](uint32_t ch) {
    pre_ch = ch;
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const size_t chan = (size_t)min(ch * CC + c, P.C - 1u) * plane;
      const T *pl = src + chan;
#pragma unroll
      for (int j = 0; j < PFC; ++j) {
        if constexpr (NBR) pre[c * PFC + j] = gen_ld_p(src, src_ptr[j] + chan * sizeof(T));
        else pre[c * PFC + j] = gen_ld_b(pl, src_boff[j]);
      }
    }
  };
  auto store_patch = [&]() {
#pragma unroll
    for (int c = 0; c < CC; ++c) {
      const bool chan = pre_ch * CC + c < P.C;
#pragma unroll
      for (int j = 0; j < PFC; ++j) {
        const uint32_t e = tid + j * kGenThreads;
        if (e < P.PP) patch[c * P.PP + e] = chan && ((src_ok >> j) & 1u) != 0u ? pre[c * PFC + j] : 0.f;
      }
    }
  };
  auto load_filter = [&](uint32_t ch, uint32_t tg0, uint32_t ntg) {
    const floatx4 *wsrc =
        reinterpret_cast<const floatx4 *>(P.wt + ((size_t)(mg * P.nchunks + ch) * P.ntaps + tg0) * CC * MW);
    const uint32_t n4 = ntg * CC * (MW / 4u);
#pragma unroll
    for (int k = 0; k < WF; ++k) {
      // no branch and no default value: either would put a wait for the patch loads here (lanes past the end
      // load the last piece again; store_filter drops it)
      const uint32_t e = tid + k * kGenThreads;
      wpre[k] = wsrc[min(e, n4 - 1u)];
    }
  };
  auto store_filter = [&](uint32_t ntg) {
    const uint32_t n4 = ntg * CC * (MW / 4u);
#pragma unroll
    for (int k = 0; k < WF; ++k) {
      const uint32_t e = tid + k * kGenThreads;
      if (e < n4) *reinterpret_cast<floatx4 *>(wl + (e / (MW / 4u)) * WPITCH + (e % (MW / 4u)) * 4u) = wpre[k];
    }
  };

  const uint32_t ntaps_s = S.t1 - S.t0;
  if (ntaps_s > 0 && ch_lo < ch_hi) {
    const uint32_t ngroups = (ntaps_s + P.TG - 1u) / P.TG;
    const uint32_t total = (ch_hi - ch_lo) * ngroups;
    uint32_t ch = ch_lo, gi = 0;
    load_patch(ch_lo);
    load_filter(ch_lo, S.t0, min(P.TG, ntaps_s));
    for (uint32_t it = 0; it < total; ++it) {
      const uint32_t tg0 = S.t0 + gi * P.TG;
      const uint32_t ntg = min(P.TG, S.t1 - tg0);
      __syncthreads();  // every wave is done with the filter rows (and, at a new chunk, the patch)
      if (gi == 0) store_patch();
      store_filter(ntg);
      // lane L keeps the patch offset of tap tg0 + L
      int32_t delta_vec = 0;
      if (lane < ntg)
        delta_vec = ((int32_t)P.off_r[tg0 + lane] - S.min_r) * (int32_t)P.PCP + ((int32_t)P.off_c[tg0 + lane] - S.min_c);
      __syncthreads();
      // the next (chunk, tap group) is on its way from memory while this one is multiplied
      if (++gi == ngroups) {
        gi = 0;
        ++ch;
      }
      if (it + 1u < total) {
        if (gi == 0) load_patch(ch);
        const uint32_t tn0 = S.t0 + gi * P.TG;
        load_filter(ch, tn0, min(P.TG, S.t1 - tn0));
      }
      const uint32_t steps = ntg << LOG2_CQ;
      float a_cur[MT], b_cur[4], a_nxt[MT], b_nxt[4];
      auto fetch = [&](uint32_t step, float (&a)[MT], float (&b)[4]) {
        const uint32_t t = step >> LOG2_CQ, cq = step & ((CC >> 2) - 1u);
        const int32_t delta = __builtin_amdgcn_readlane(delta_vec, (int)t);
        const float *wrow = wl + (t * CC + (cq << 2) + g) * WPITCH + l16;
        const float *prow = patch + (cq << 2) * P.PP + delta;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) a[mt] = wrow[mt * 16];
#pragma unroll
        for (int q = 0; q < 4; ++q) b[q] = prow[pix[q]];
      };
      auto multiply = [&](const float (&a)[MT], const float (&b)[4]) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[q][mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[mt], b[q], acc[q][mt], 0, 0, 0);
      };
      // two operand sets take turns: the reads of one step are in flight during the other step's multiplications
      fetch(0, a_cur, b_cur);
      // (a fetch past the last step repeats the last one: every pass has the same number of reads in flight, so
      // the wait before a multiplication can leave the newer set outstanding)
      // The scheduling barriers keep a set's reads together ahead of the other set's multiplications.
      for (uint32_t step = 0; step < steps; step += 2u) {
        fetch(min(step + 1u, steps - 1u), a_nxt, b_nxt);
        __builtin_amdgcn_sched_barrier(0);
        multiply(a_cur, b_cur);
        __builtin_amdgcn_sched_barrier(0);
        if (step + 1u >= steps) break;
        fetch(min(step + 2u, steps - 1u), a_cur, b_cur);
        __builtin_amdgcn_sched_barrier(0);
        multiply(a_nxt, b_nxt);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // the lane holds D[m = 4g + i][n = l16] of each 16 x 16 tile
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const uint32_t i = bi * P.BR + row_q[q], j = bj * P.BC + col_q[q];
    if (!live_q[q] || i >= S.GI || j >= S.GJ) continue;
    const size_t pix_out = (size_t)img_q[q] * P.M * P.out_H * P.out_W + (size_t)(S.o_r + i * P.so_r) * P.out_W + (S.o_c + j * P.so_c);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t m = mg * MW + mt * 16u + g * 4u + k;
        if (m >= P.M) continue;
        const size_t o = (size_t)m * P.out_H * P.out_W + pix_out;
        float v = acc[q][mt][k];
        if (P.ksplit > 1u) {
          P.part[((size_t)ks * P.num_tiles + tile) * P.part_tile_elems + (size_t)n * P.M * P.out_H * P.out_W + o] = v;
          continue;
        }
        if (P.beta != 0.f) v += gen_ld(dst, o);
        gen_st(dst, o, v);
      }
  }
}

// out[tile][e] = beta * out[tile][e] + part[0][tile][e] + part[1][tile][e] + ... (a fixed order: reproducible)
struct SplitReduceParams {
  void *out[ADH_MAX_TILES];
  const float *part;
  uint64_t tile_elems;
  uint32_t num_tiles, ksplit;
  float beta;
};
template <typename T>
__global__ __launch_bounds__(256) void conv_gen_split_reduce_kernel(const SplitReduceParams R) {
  const uint32_t tile = blockIdx.y;
  T *out = reinterpret_cast<T *>(R.out[tile]);
  for (uint64_t e = (uint64_t)blockIdx.x * 256u + threadIdx.x; e < R.tile_elems; e += (uint64_t)gridDim.x * 256u) {
    float v = R.part[(size_t)tile * R.tile_elems + e];
    for (uint32_t k = 1; k < R.ksplit; ++k) v += R.part[((size_t)k * R.num_tiles + tile) * R.tile_elems + e];
    if (R.beta != 0.f) v += gen_ld(out, e);
    gen_st(out, e, v);
  }
}

// ---- host side: tap tables, tiling, launches ----

struct GenPlan {
  ConvGenParams P;
  FilterGenParams F;
  size_t lds_bytes, wt_bytes, part_bytes;  // part_bytes: the partial sums of a launch whose channel chunks are split
  uint32_t MT, num_tiles;
  bool nbr;  // tiles without halo: the kernel instances that read rows from the neighbouring tiles
};
// a launch of fewer blocks than this (two per compute unit) is split finer
constexpr uint64_t kGenFillBlocks = 512;

// The part of the tiling that depends on the block's width in output channels (16 * plan->MT); BR and BC are set.
static int gen_tile_plan(GenPlan *plan, uint32_t max_taps) {
  ConvGenParams &P = plan->P;
  const uint32_t MW = 16u * plan->MT, wpitch = plan->MT == 1u ? 16u : MW + 16u;
  P.MG = (P.M + MW - 1u) / MW;
  uint32_t max_PR, max_PC, bpi;
  size_t patch_bytes;
  // channels per chunk: 8 (4 when there are fewer), or 16 / 32 when the channel count is (nearly) a multiple and the
  // patch is small enough for a thread's 32 staging registers without giving up images per block
  // (a last chunk padded with zero channels is accepted when the padding is under an eighth of the channels)
  auto pads_little = [&](uint32_t cc) { return ((P.C + cc - 1u) / cc * cc - P.C) * 8u <= P.C; };
  P.CC = pads_little(32u) ? 32u : pads_little(16u) ? 16u : P.C >= 8u ? 8u : 4u;
  for (;;) {
    max_PR = 1; max_PC = 1; bpi = 0;
    for (uint32_t s = 0; s < P.nsub; ++s) {
      GenSub &S = P.sub[s];
      int32_t lo_r = 0, hi_r = 0, lo_c = 0, hi_c = 0;
      for (uint32_t t = S.t0; t < S.t1; ++t) {
        if (t == S.t0) {
          lo_r = hi_r = P.off_r[t];
          lo_c = hi_c = P.off_c[t];
        }
        lo_r = std::min<int32_t>(lo_r, P.off_r[t]);
        hi_r = std::max<int32_t>(hi_r, P.off_r[t]);
        lo_c = std::min<int32_t>(lo_c, P.off_c[t]);
        hi_c = std::max<int32_t>(hi_c, P.off_c[t]);
      }
      S.min_r = lo_r;
      S.min_c = lo_c;
      S.PR = (P.BR - 1u) * P.si_r + (uint32_t)(hi_r - lo_r) + 1u;
      S.PC = (P.BC - 1u) * P.si_c + (uint32_t)(hi_c - lo_c) + 1u;
      max_PR = std::max(max_PR, S.PR);
      max_PC = std::max(max_PC, S.PC);
      S.nbj = (S.GJ + P.BC - 1u) / P.BC;
      S.blk0 = bpi;
      bpi += S.nbj * ((S.GI + P.BR - 1u) / P.BR);
    }
    if (bpi == 0) return ADH_EINVAL;
    P.PCP = max_PC;
    P.PPI = max_PR * P.PCP;
    P.live = P.BR * P.BC;
    // images per block: as many as fill the 256 pixel slots, fit LDS and the staging registers, and keep
    // the byte offsets of a block's images within 32 bits
    uint32_t nb = P.live <= 128u ? std::min(256u / P.live, std::max(P.N, 1u)) : 1u;
    while (nb > 1u && (uint64_t)nb * P.C * P.in_H * P.in_W >= (1ull << 30)) --nb;
    bool fits = false;
    for (;; --nb) {
      // plane pitch: the four channel groups of a read start 16 banks apart
      uint32_t pp = nb * P.PPI;
      while (pp % 64u != 16u) ++pp;
      P.PP = pp;
      patch_bytes = (size_t)P.CC * P.PP * 4u;
      // a thread stages 32 / CC elements of each channel plane
      fits = P.PP <= 256u * (32u / P.CC) && patch_bytes + (size_t)P.CC * wpitch * 4u <= kGenLdsBytes;
      if (fits || nb == 1u || P.CC > 8u) break;
    }
    P.NB = nb;
    if (fits) break;
    if (P.CC > 4u) {
      P.CC /= 2u;  // half the channels per chunk: twice the room per plane
      continue;
    }
    if (P.BR == 1u) return ADH_EUNIMPL;
    P.BR -= 1u;  // fewer rows per block: the n-tiles of the dropped rows idle
    P.CC = P.C >= 8u ? 8u : 4u;
  }
  P.nchunks = (P.C + P.CC - 1u) / P.CC;
  P.blocks_per_image = bpi;
  // taps per group: what fits LDS, a lane per tap, and six float4 staging registers per thread
  P.TG = (uint32_t)std::min<size_t>(std::min<uint32_t>(std::max(max_taps, 1u), 64u),
                                    (kGenLdsBytes - patch_bytes) / ((size_t)P.CC * wpitch * 4u));
  P.TG = std::min<uint32_t>(P.TG, 256u * 6u / (P.CC * MW / 4u));
  P.w_lds_floats = P.TG * P.CC * wpitch;
  P.div_PCP = FastDiv(P.PCP);
  P.div_BC = FastDiv(P.BC);
  P.div_live = FastDiv(P.live);
  P.div_PPI = FastDiv(P.PPI);
  P.NG = (P.N + P.NB - 1u) / P.NB;
  plan->lds_bytes = (size_t)P.w_lds_floats * 4u + patch_bytes;
  plan->wt_bytes = (size_t)P.MG * P.nchunks * P.ntaps * P.CC * MW * 4u;
  P.div_bpi = FastDiv(bpi);
  P.div_MG = FastDiv(P.MG);
  P.div_N = FastDiv(P.NG);
  FilterGenParams &F = plan->F;
  F.M = P.M;
  F.C = P.C;
  F.MG = P.MG;
  F.MW = MW;
  F.nchunks = P.nchunks;
  F.CC = P.CC;
  F.ntaps = P.ntaps;
  return ADH_OK;
}

// Fills the tiling fields of `plan` once the sub-problems' taps and grids are set.  Returns an error code.
static int gen_finish_plan(GenPlan *plan) {
  ConvGenParams &P = plan->P;
  uint32_t max_GJ = 0, max_taps = 0;
  for (uint32_t s = 0; s < P.nsub; ++s) {
    max_GJ = std::max(max_GJ, P.sub[s].GJ);
    max_taps = std::max(max_taps, P.sub[s].t1 - P.sub[s].t0);
  }
  uint32_t max_GI = 0;
  for (uint32_t s = 0; s < P.nsub; ++s) max_GI = std::max(max_GI, P.sub[s].GI);
  // block columns: the whole row when it has at most 64 pixels, else the width in [32, 64] that wastes least
  if (max_GJ <= 64u) {
    P.BC = std::max(max_GJ, 1u);
  } else {
    double best = -1.0;
    for (uint32_t bc = 64u; bc >= 32u; --bc) {
      const double used = (double)((256u / bc) * bc) / 256.0 * (double)max_GJ / (double)(((max_GJ + bc - 1u) / bc) * bc);
      if (used > best + 1e-9) { best = used; P.BC = bc; }
    }
  }
  P.BR = std::max(1u, std::min(256u / P.BC, std::max(max_GI, 1u)));
  // Fewer rows per block when that fills the 256 pixel slots better: a 9-row grid in blocks of 7 rows leaves the
  // second block two rows, in blocks of 3 rows (two images per block) nothing.  Modelled time per pixel: the
  // reciprocal of the filled share of the slots, times 1 + 0.39 * (patch rows staged per row of pixels); the
  // factor is fitted to stride-2 backward-data on 17x65 and 9x33 grids, and a lower block must win by a tenth.
  // Only where the input is read at stride 1 (backward-data, stride-1 forward): a strided forward's patch has
  // si_r rows per row of pixels, lower blocks push it out of the wider chunks, and the model does not hold
  // (7x28 outputs of a stride-2 3x3: 9 one-row images per block ran 1.8 times slower than one 7-row image).
  if (P.si_r == 1u) {
    uint32_t span_r = 0;
    for (uint32_t s = 0; s < P.nsub; ++s) {
      int32_t lo = 0, hi = 0;
      for (uint32_t t = P.sub[s].t0; t < P.sub[s].t1; ++t) {
        if (t == P.sub[s].t0) lo = hi = P.off_r[t];
        lo = std::min<int32_t>(lo, P.off_r[t]);
        hi = std::max<int32_t>(hi, P.off_r[t]);
      }
      span_r = std::max(span_r, (uint32_t)(hi - lo));
    }
    const uint32_t gi = std::max(max_GI, 1u);
    auto modelled = [&](uint32_t br) {
      const uint32_t live = br * P.BC;
      const uint32_t nb = live <= 128u ? std::min(256u / live, std::max(P.N, 1u)) : 1u;
      const double filled = (double)gi / (double)(((gi + br - 1u) / br) * br) * (double)(nb * live) / 256.0;
      const double patch_rows = (double)((br - 1u) * P.si_r + span_r + 1u) / (double)(br * P.si_r);
      return (1.0 + 0.39 * patch_rows) / filled;
    };
    uint32_t best = P.BR;
    for (uint32_t br = P.BR; br >= 1u; --br)
      if (modelled(br) < modelled(best) - 1e-9) best = br;
    if (modelled(best) < 0.9 * modelled(P.BR)) P.BR = best;
  }
  // Output channels per block: 64, or fewer when there are no more of them, or when the launch would
  // leave compute units idle (a block's time is mostly the latency of staging its chunks, whatever its
  // width, so narrower blocks on more units finish sooner).
  plan->MT = P.M <= 16u ? 1u : P.M <= 32u ? 2u : 4u;
  // Many channels over few, full blocks of pixels (512 channels on the 4x16 or 2x8 tiles of a net split over ranks):
  // blocks of 64 output channels whose channel chunks are dealt to 2, 4 or 8 workgroups run ahead of narrower blocks,
  // as each staged patch serves four times the output channels (3x3, 512 -> 512, 32 images, 4 tiles: 4x16 tiles 0.39 ms
  // with 2 workgroups per block against 0.44 for blocks of 32 channels; 2x8 tiles 0.13 ms with 8 against 0.20 for
  // blocks of 16 channels in 3).  Powers of two only: 3 and 6 ran slower than 2 and 4.
  uint32_t wide_split = 0;
  if (plan->MT == 4u) {
    const int e = gen_tile_plan(plan, max_taps);
    if (e) return e;
    const uint64_t blocks = (uint64_t)std::max(plan->num_tiles, 1u) * P.NG * P.MG * P.blocks_per_image;
    if (blocks < kGenFillBlocks && P.nchunks >= 16u && P.NB * P.live >= 128u) {
      wide_split = 2;
      while (blocks * wide_split < kGenFillBlocks && P.nchunks / (wide_split * 2u) >= 4u) wide_split *= 2u;
    }
  }
  for (; wide_split == 0u; plan->MT /= 2u) {
    const int e = gen_tile_plan(plan, max_taps);
    if (e) return e;
    const uint64_t blocks = (uint64_t)std::max(plan->num_tiles, 1u) * P.NG * P.MG * P.blocks_per_image;
    if (plan->MT == 1u || blocks >= kGenFillBlocks) break;
  }
  // Still a thin launch at 16 output channels per block (the late layers of a net split over ranks: a 2x8 tile
  // with 512 channels makes 256 workgroups, one wave per SIMD, each waiting for its next chunk with nothing else
  // to run): deal the channel chunks to up to four workgroups per block of pixels, three of which share a CU,
  // and add their sums in a second kernel.
  const uint64_t blocks = (uint64_t)std::max(plan->num_tiles, 1u) * P.NG * P.MG * P.blocks_per_image;
  P.ksplit = 1;
  if (wide_split)
    P.ksplit = wide_split;
  else if (blocks < kGenFillBlocks && P.nchunks >= 8u)
    P.ksplit = (uint32_t)std::min<uint64_t>(std::min<uint64_t>(4u, P.nchunks / 4u), (768u + blocks - 1u) / blocks);
  P.chunks_per_split = (P.nchunks + P.ksplit - 1u) / P.ksplit;
  P.ksplit = (P.nchunks + P.chunks_per_split - 1u) / P.chunks_per_split;  // no split without chunks
  P.div_ksplit = FastDiv(P.ksplit);
  P.part_tile_elems = (uint64_t)P.N * P.M * P.out_H * P.out_W;
  plan->part_bytes = P.ksplit > 1u ? (size_t)P.ksplit * std::max(plan->num_tiles, 1u) * P.part_tile_elems * 4u : 0u;
  return ADH_OK;
}

struct GenShape {
  uint32_t N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, OH, OW;
};

// conv1x1.hip: forward / backward-data of a 1x1 window at stride 1 or 2 in fp32; ADH_EUNIMPL (and nothing
// launched) for a shape it does not serve
int conv1x1_try(bool bwd, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                uint32_t OH, uint32_t OW, uint32_t s, const void *const *in_tiles, const void *w,
                void *const *out_tiles, float beta, hipStream_t st);

size_t conv1x1_wgrad_workspace(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t OH, uint32_t OW);
int conv1x1_wgrad_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W, uint32_t OH,
                      uint32_t OW, uint32_t sh, uint32_t sw, const void *const *x_tiles, const void *const *dy_tiles,
                      float *dwt, float beta, void *workspace, hipStream_t st);

// conv3x3s2.hip: backward-data of a 3x3 window at stride 2, padding 1, over fp32 tiles of H x W without halo
int conv3x3s2_bwd_data_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                           const void *w, const void *const *dy_tiles, void *const *dx_tiles, float beta,
                           hipStream_t st);

int conv3x3s2_fwd_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                      const void *const *x_tiles, const void *w, void *const *y_tiles, float beta, hipStream_t st);

size_t conv3x3s2_wgrad_workspace(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W);
int conv3x3s2_wgrad_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                        const void *const *x_tiles, const void *const *dy_tiles, float *dwt, float beta, void *workspace,
                        hipStream_t st);
static bool gen_is_3x3s2_unpadded(int dtype, const GenShape &g, bool unpadded, uint32_t pad_h, uint32_t pad_w) {
  return dtype == ADH_F32 && unpadded && g.kh == 3u && g.kw == 3u && g.sh == 2u && g.sw == 2u && g.dh == 1u && g.dw == 1u &&
         pad_h == 1u && pad_w == 1u;
}

// conv3x3.hip: the 3x3 window at stride 1 with dilation 3 over fp32 tiles padded by 3, forward and backward-data
static bool gen_is_3x3_dilated(int dtype, const GenShape &g, bool unpadded) {
  return dtype == ADH_F32 && !unpadded && g.kh == 3u && g.kw == 3u && g.sh == 1u && g.sw == 1u && g.dh == g.dw && g.dh > 1u;
}
int conv3x3_dilated_try(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                        uint32_t W, uint32_t dil, const void *const *in_tiles, const void *w, void *const *out_tiles,
                        float beta, hipStream_t st);
// conv3x3_wgrad.hip: its filter gradient
size_t conv3x3_dilated_wgrad_workspace(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                                       uint32_t dil);
int conv3x3_dilated_wgrad_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W, uint32_t dil,
                              const void *const *x_tiles, const void *const *dy_tiles, float *dw, float beta, void *workspace,
                              hipStream_t st);
// conv_thin.hip: forward over halo-padded fp32 tiles for at most three input channels (a network's stem)
int conv_thin_fwd_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t OH,
                      uint32_t OW, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, const void *const *x_tiles,
                      const void *w, void *const *y_tiles, float beta, hipStream_t st, const float *const *bias_tiles);

size_t conv_thin_wgrad_workspace(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP,
                                 uint32_t OH, uint32_t OW, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw);
int conv_thin_wgrad_try(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t OH,
                        uint32_t OW, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, const void *const *x_tiles,
                        const void *const *dy_tiles, float *dwt, float beta, void *workspace, hipStream_t st);
static bool gen_is_thin(int dtype, const GenShape &g, bool unpadded) {
  return dtype == ADH_F32 && !unpadded && g.dh == 1u && g.dw == 1u && g.Cin <= 3u && (g.kh > 1u || g.kw > 1u);
}

// a window of one tap reads no neighbour and no padding: tiles with and without halo are the same thing
static bool gen_is_pointwise(int dtype, const GenShape &g, bool unpadded, uint32_t pad_h, uint32_t pad_w) {
  return dtype == ADH_F32 && g.kh == 1u && g.kw == 1u && g.sh == g.sw && (!unpadded || (pad_h == 0u && pad_w == 0u));
}
// the filter gradient's kernel takes any pair of strides
static bool gen_is_pointwise_wgrad(int dtype, const GenShape &g, bool unpadded, uint32_t pad_h, uint32_t pad_w) {
  return dtype == ADH_F32 && g.kh == 1u && g.kw == 1u && (!unpadded || (pad_h == 0u && pad_w == 0u));
}

static int gen_check_shape(uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP,
                           uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, GenShape *g) {
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if (kh == 0 || kw == 0 || sh == 0 || sw == 0 || dh == 0 || dw == 0) return ADH_EINVAL;
  if ((uint64_t)kh * kw > (uint64_t)kGenMaxTaps) return ADH_EUNIMPL;
  if ((uint64_t)sh * sw > (uint64_t)kGenMaxSub) return ADH_EUNIMPL;
  const uint64_t eh = (uint64_t)(kh - 1u) * dh + 1u, ew = (uint64_t)(kw - 1u) * dw + 1u;
  if (eh > HP || ew > WP || eh > 4096u || ew > 4096u) return ADH_EINVAL;
  // a lane's byte offset within a channel plane (within a block's images when it takes several) is 32 bits wide
  if ((uint64_t)HP * WP >= (1ull << 30) || Cin >= (1u << 24) || Cout >= (1u << 24)) return ADH_EINVAL;
  *g = GenShape{N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, (uint32_t)((HP - eh) / sh + 1u), (uint32_t)((WP - ew) / sw + 1u)};
  return ADH_OK;
}

// pad_h, pad_w: the input tile carries no halo (it is g.HP - 2 pad_h rows by g.WP - 2 pad_w columns) and the taps
// reach pad_h rows and pad_w columns before its first pixel
static int gen_plan_fwd(const GenShape &g, GenPlan *plan, uint32_t pad_h = 0, uint32_t pad_w = 0) {
  ConvGenParams &P = plan->P;
  P.N = g.N; P.C = g.Cin; P.M = g.Cout;
  P.in_H = g.HP - 2u * pad_h; P.in_W = g.WP - 2u * pad_w; P.out_H = g.OH; P.out_W = g.OW;
  P.si_r = g.sh; P.si_c = g.sw; P.so_r = 1; P.so_c = 1;
  P.ntaps = g.kh * g.kw;
  P.nsub = 1;
  for (uint32_t a = 0; a < g.kh; ++a)
    for (uint32_t b = 0; b < g.kw; ++b) {
      const uint32_t t = a * g.kw + b;
      P.off_r[t] = (int16_t)((int32_t)(a * g.dh) - (int32_t)pad_h);
      P.off_c[t] = (int16_t)((int32_t)(b * g.dw) - (int32_t)pad_w);
      plan->F.tap_index[t] = (uint16_t)t;
    }
  GenSub &S = P.sub[0];
  S.t0 = 0; S.t1 = P.ntaps; S.GI = g.OH; S.GJ = g.OW; S.o_r = 0; S.o_c = 0;
  plan->F.m_stride = g.Cin * g.kh * g.kw;
  plan->F.c_stride = g.kh * g.kw;
  return gen_finish_plan(plan);
}

// pad_h, pad_w (with `unpadded`): the gradient tile carries no halo: only the pixels pad_h .. pad_h + H - 1 by
// pad_w .. pad_w + W - 1 of the padded gradient are computed, and they are stored from (0, 0) on.
static int gen_plan_bwd_data(const GenShape &g, GenPlan *plan, bool unpadded = false, uint32_t pad_h = 0, uint32_t pad_w = 0) {
  ConvGenParams &P = plan->P;
  if (!unpadded) pad_h = pad_w = 0;
  const uint32_t H = g.HP - 2u * pad_h, W = g.WP - 2u * pad_w;  // the gradient tile
  P.N = g.N; P.C = g.Cout; P.M = g.Cin;
  P.in_H = g.OH; P.in_W = g.OW; P.out_H = H; P.out_W = W;
  P.si_r = 1; P.si_c = 1; P.so_r = g.sh; P.so_c = g.sw;
  P.ntaps = g.kh * g.kw;
  uint32_t nsub = 0, t = 0;
  for (uint32_t pr = 0; pr < g.sh && pr < g.HP; ++pr)
    for (uint32_t pc = 0; pc < g.sw && pc < g.WP; ++pc) {
      GenSub &S = P.sub[nsub++];
      // the class's first padded row / column inside the tile: pr + sh * i0 >= pad_h
      const uint32_t i0 = pad_h > pr ? (pad_h - pr + g.sh - 1u) / g.sh : 0u;
      const uint32_t j0 = pad_w > pc ? (pad_w - pc + g.sw - 1u) / g.sw : 0u;
      const uint32_t r_first = pr + g.sh * i0 - pad_h, c_first = pc + g.sw * j0 - pad_w;
      S.t0 = t;
      for (uint32_t a = 0; a < g.kh; ++a)
        for (uint32_t b = 0; b < g.kw; ++b) {
          if ((a * g.dh) % g.sh != pr || (b * g.dw) % g.sw != pc) continue;
          // dy row of padded row h' = pr + sh * (i0 + i) under tap a: (h' - a*dh) / sh = i + i0 + (pr - a*dh) / sh
          P.off_r[t] = (int16_t)((int32_t)i0 + ((int32_t)pr - (int32_t)(a * g.dh)) / (int32_t)g.sh);
          P.off_c[t] = (int16_t)((int32_t)j0 + ((int32_t)pc - (int32_t)(b * g.dw)) / (int32_t)g.sw);
          plan->F.tap_index[t] = (uint16_t)(a * g.kw + b);
          ++t;
        }
      S.t1 = t;
      S.GI = r_first < H ? (H - r_first + g.sh - 1u) / g.sh : 0u;
      S.GJ = c_first < W ? (W - c_first + g.sw - 1u) / g.sw : 0u;
      S.o_r = r_first;
      S.o_c = c_first;
    }
  P.nsub = nsub;
  plan->F.m_stride = g.kh * g.kw;
  plan->F.c_stride = g.Cin * g.kh * g.kw;
  return gen_finish_plan(plan);
}

template <typename T, int CC, bool NBR>
static void launch_gen_cc(const GenPlan &plan, uint32_t blocks, hipStream_t st) {
  if (plan.MT == 1u)
    hipLaunchKernelGGL((conv_gen_kernel<T, CC, 1, NBR>), dim3(blocks), dim3(kGenThreads), plan.lds_bytes, st, plan.P);
  else if (plan.MT == 2u)
    hipLaunchKernelGGL((conv_gen_kernel<T, CC, 2, NBR>), dim3(blocks), dim3(kGenThreads), plan.lds_bytes, st, plan.P);
  else
    hipLaunchKernelGGL((conv_gen_kernel<T, CC, 4, NBR>), dim3(blocks), dim3(kGenThreads), plan.lds_bytes, st, plan.P);
}
template <typename T, bool NBR>
static void launch_gen_nbr(const GenPlan &plan, uint32_t blocks, hipStream_t st) {
  if (plan.P.CC == 32u) launch_gen_cc<T, 32, NBR>(plan, blocks, st);
  else if (plan.P.CC == 16u) launch_gen_cc<T, 16, NBR>(plan, blocks, st);
  else if (plan.P.CC == 8u) launch_gen_cc<T, 8, NBR>(plan, blocks, st);
  else launch_gen_cc<T, 4, NBR>(plan, blocks, st);
}
template <typename T>
static void launch_gen(const GenPlan &plan, uint32_t blocks, hipStream_t st) {
  if (plan.nbr) launch_gen_nbr<T, true>(plan, blocks, st);
  else launch_gen_nbr<T, false>(plan, blocks, st);
}

static int gen_check_workspace(const GenPlan &plan, const void *workspace, size_t workspace_bytes) {
  if (!workspace) return ADH_ENULL;
  if (!aligned_to(workspace, 256)) return ADH_EALIGN;
  const size_t wt_room = (plan.wt_bytes + 255u) & ~(size_t)255u;
  if (workspace_bytes < wt_room + plan.part_bytes) return ADH_EWORKSPACE;
  return ADH_OK;
}

static int gen_launch(int dtype, GenPlan *plan, uint32_t num_tiles, const void *w, void *workspace,
                      size_t workspace_bytes, hipStream_t st) {
  ConvGenParams &P = plan->P;
  const int ws = gen_check_workspace(*plan, workspace, workspace_bytes);
  if (ws) return ws;
  const size_t wt_room = (plan->wt_bytes + 255u) & ~(size_t)255u;
  const uint64_t blocks = (uint64_t)num_tiles * P.NG * P.MG * P.blocks_per_image * P.ksplit;
  if (blocks == 0) return ADH_OK;
  if (blocks >= (1ull << 24)) return ADH_EINVAL;
  plan->F.w = w;
  plan->F.wt = reinterpret_cast<float *>(workspace);
  P.wt = plan->F.wt;
  P.num_tiles = num_tiles;
  P.part = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + wt_room);
  const uint32_t fblocks = (uint32_t)std::min<size_t>(1024, (plan->wt_bytes / 4u + 255u) / 256u);
  if (dtype == ADH_F32) {
    hipLaunchKernelGGL(conv_gen_filter_kernel<float>, dim3(fblocks), dim3(256), 0, st, plan->F);
    launch_gen<float>(*plan, (uint32_t)blocks, st);
  } else {
    hipLaunchKernelGGL(conv_gen_filter_kernel<uint16_t>, dim3(fblocks), dim3(256), 0, st, plan->F);
    launch_gen<uint16_t>(*plan, (uint32_t)blocks, st);
  }
  if (P.ksplit > 1u) {
    SplitReduceParams R = {};
    for (uint32_t t = 0; t < num_tiles; ++t) R.out[t] = P.out[t];
    R.part = P.part;
    R.tile_elems = P.part_tile_elems;
    R.num_tiles = num_tiles;
    R.ksplit = P.ksplit;
    R.beta = P.beta;
    const uint32_t rb = (uint32_t)std::min<uint64_t>((P.part_tile_elems + 255u) / 256u, 2048u);
    if (dtype == ADH_F32)
      hipLaunchKernelGGL(conv_gen_split_reduce_kernel<float>, dim3(rb, num_tiles), dim3(256), 0, st, R);
    else
      hipLaunchKernelGGL(conv_gen_split_reduce_kernel<uint16_t>, dim3(rb, num_tiles), dim3(256), 0, st, R);
  }
  return launch_status();
}

}  // namespace adh

// ---------------------------------------------------------------------------------------------
// backward-filter for any window / stride / dilation
//   dw[co][ci][a][b] = beta*dw + sum over tiles, n, oh, ow of dy[n][co][oh][ow] * x[n][ci][oh*sh + a*dh][ow*sw + b*dw]
// GEMM per tap: M = 64 output channels, N = 16 input channels, K = output pixels, four consecutive
// pixels of a row per v_mfma_f32_16x16x4_f32.  A block owns (64 co, 16 ci, a group of T <= 9 taps)
// and every PS-th unit of pixels (R output rows x OWT columns of one image); per unit it stages the dy
// tile and the input patch in LDS, the next unit's loads already in flight in registers, and each of
// its four waves multiplies the whole unit for its own 16 output channels, keeping T accumulator
// tiles.  Every wave writes its sums in register order to the workspace; a second kernel adds the PS
// partial sums in a fixed order (deterministic) and scatters them to KCRS.
// ---------------------------------------------------------------------------------------------
namespace adh {

constexpr uint32_t kWgGenThreads = 256;

struct WgradGenParams {
  const void *x[ADH_MAX_TILES];
  const void *dy[ADH_MAX_TILES];
  float *partial;
  uint32_t N, Cin, Cout, HP, WP, OH, OW, sh, sw;
  uint32_t T, ntg, ntaps, COG, CIT;
  uint32_t R, OWT, nrb, ncb, units, PS;
  // A unit is R x OWT pixels of one image, or, when that is a whole image of at most 32 pixel slots, of NBU
  // consecutive images (unit pixel f is pixel f % img_pix of image f / img_pix; the images' patches lie side by
  // side in a plane, PPI apart).  NG = ceil(N / NBU) image groups per tile.
  uint32_t NBU, NG, img_pix, PPI;
  uint32_t PR, PC, PCP, PP, DP, dy_lds_floats;
  // the NBR instances: x carries no halo (HP x WP is the tile itself), the taps reach pad_h rows and pad_w columns
  // before its first pixel, rows outside the tile are the neighbouring row tiles' (tiles in rank order), what
  // lies outside the tensor is zero
  uint32_t pad_h, pad_w, num_tiles;
  FastDiv div_COG, div_CIT, div_ntg, div_ncb, div_nrb, div_N, div_OWT, div_PC, div_PR, div_img_pix, div_PRPC;
  int16_t off_r[kGenMaxTaps], off_c[kGenMaxTaps];
};

// PACKED (few input channels, e.g. the 3-channel stem): the 16 columns of an accumulator tile are 16
// (tap, input channel) pairs, pair q = 16 t + column = tap * Cin + ci, instead of 16 input channels of one tap;
// all taps then fit one block and no matrix column is spent on channels that do not exist.
template <typename T, int TAPS, bool PACKED, bool NBR = false>
__global__ __launch_bounds__(kWgGenThreads, 2) void conv_gen_wgrad_kernel(const WgradGenParams P) {
  extern __shared__ __align__(16) float gen_lds[];
  float *dyl = gen_lds;
  float *patch = gen_lds + P.dy_lds_floats;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, l16 = lane & 15u, g = lane >> 4;
  uint32_t rest, rest2, cog, cit, tg, ps;
  P.div_COG.divmod(blockIdx.x, rest, cog);
  P.div_CIT.divmod(rest, rest2, cit);
  P.div_ntg.divmod(rest2, ps, tg);

  // lane L keeps the patch offset of tap tg * TAPS + L (absent taps of the last group read tap 0's place)
  int32_t delta_vec = 0;
  if (!PACKED) {
    const uint32_t t = tg * TAPS + lane;
    if (lane < (uint32_t)TAPS && t < P.ntaps) delta_vec = (int32_t)P.off_r[t] * (int32_t)P.PCP + (int32_t)P.off_c[t];
  }
  // PACKED: this lane's (tap, channel) pair of every tile, as an offset into the patch (absent pairs read place 0)
  int32_t pair_off[PACKED ? TAPS : 1];
  if (PACKED) {
#pragma unroll
    for (int t = 0; t < TAPS; ++t) {
      const uint32_t q = (uint32_t)t * 16u + l16;
      const uint32_t tap = q / P.Cin, ci = q - tap * P.Cin;
      pair_off[t] = tap < P.ntaps ? (int32_t)(ci * P.PP) + (int32_t)P.off_r[tap] * (int32_t)P.PCP + (int32_t)P.off_c[tap] : 0;
    }
  }
  // wave w owns output channels 16 w .. 16 w + 15 of the block's 64: one accumulator tile per tap
  floatx4 acc[TAPS];
#pragma unroll
  for (int t = 0; t < TAPS; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const uint32_t unit_pix = P.NBU * P.img_pix, ksteps = unit_pix >> 2;
  // only the channels that exist are staged; lanes of absent channels read channel 0 and their sums are dropped
  const uint32_t planes = min(16u, P.Cin - cit * 16u);
  const uint32_t my_plane = l16 < planes ? l16 : 0u;
  // What a thread stages is the same for every unit: the lane's pixel of the dy tile (a unit has at most 64
  // pixels) for the wave's 16 output channels, and up to two (row, column) places of every patch plane.
  // Loads take a base address that is the same in every lane (the unit's origin in the channel plane) plus the
  // lane's 32-bit byte offset; places outside the tensors load offset 0 and are replaced by zero.
  const uint32_t wave_u = (uint32_t)__builtin_amdgcn_readfirstlane((int)wave);
  uint32_t dy_b, dy_p, dy_r, dy_c;
  P.div_img_pix.divmod(lane, dy_b, dy_p);
  P.div_OWT.divmod(dy_p, dy_r, dy_c);
  const bool dy_lane = lane < unit_pix;
  const uint32_t dy_boff = (dy_b * P.Cout * P.OH * P.OW + dy_r * P.OW + dy_c) * (uint32_t)sizeof(T);
  const int32_t co_lim = (int32_t)P.Cout - (int32_t)(cog * 64u + wave_u * 16u);  // the wave's channels that exist
  constexpr int KP = 2;  // NBU * PR * PC <= 512
  uint32_t pr_rc[KP], pr_b[KP], pr_lds[KP], x_boff[KP];
#pragma unroll
  for (int k = 0; k < KP; ++k) {
    const uint32_t e = tid + k * kWgGenThreads;
    uint32_t b, ei, r, col;
    P.div_PRPC.divmod(e, b, ei);
    P.div_PC.divmod(ei, r, col);
    pr_rc[k] = b < P.NBU ? (r << 16) | col : 0xffffffffu;
    pr_b[k] = b;
    pr_lds[k] = b * P.PPI + r * P.PCP + col;
    x_boff[k] = (b * P.Cin * P.HP * P.WP + r * P.WP + col) * (uint32_t)sizeof(T);
  }
  const size_t x_plane = (size_t)P.HP * P.WP, dy_plane = (size_t)P.OH * P.OW;
  // A unit travels memory -> registers -> LDS; the next unit's loads are in flight while this one is multiplied.
  float dy_pre[16], x_pre[KP][16];
  uint32_t pre_in = 0;  // bit 0: the dy pixel exists; bit 1 + k: patch place k exists (of the unit in the registers)
  // channels that do not exist load an existing one's place (no branch around a load); store_unit drops them
  const int32_t dy_c0 = co_lim > 0 ? 0 : -(int32_t)(wave_u * 16u), dy_cmax = co_lim > 0 ? co_lim - 1 : 0;
  auto load_unit = [&](uint32_t u) {
    uint32_t r2, r3, cb, rb, n, tile;
    P.div_ncb.divmod(u, r2, cb);
    P.div_nrb.divmod(r2, r3, rb);
    P.div_N.divmod(r3, tile, n);
    n *= P.NBU;  // the unit's first image
    const uint32_t oh0 = rb * P.R, ow0 = cb * P.OWT;
    const T *xs = reinterpret_cast<const T *>(P.x[tile]) + ((size_t)n * P.Cin + cit * 16u) * x_plane +
                  (size_t)oh0 * P.sh * P.WP + (size_t)ow0 * P.sw;
    const T *ds = reinterpret_cast<const T *>(P.dy[tile]) + ((size_t)n * P.Cout + cog * 64u + wave_u * 16u) * dy_plane +
                  (size_t)oh0 * P.OW + ow0;
    const bool dy_in = dy_lane && n + dy_b < P.N && oh0 + dy_r < P.OH && ow0 + dy_c < P.OW;
    pre_in = dy_in ? 1u : 0u;
    const uint32_t dy_off = dy_in ? dy_boff : 0u;
#pragma unroll
    for (int c = 0; c < 16; ++c)
      dy_pre[c] = gen_ld_b(ds + (ptrdiff_t)(dy_c0 + min(c, dy_cmax)) * (ptrdiff_t)dy_plane, dy_off);
#pragma unroll
    for (int k = 0; k < KP; ++k) {
      if constexpr (!NBR) {
        const bool in = pr_rc[k] != 0xffffffffu && n + pr_b[k] < P.N && oh0 * P.sh + (pr_rc[k] >> 16) < P.HP &&
                        ow0 * P.sw + (pr_rc[k] & 0xffffu) < P.WP;
        pre_in |= in ? 2u << k : 0u;
        const uint32_t off = in ? x_boff[k] : 0u;
#pragma unroll
        for (int c = 0; c < 16; ++c) x_pre[k][c] = gen_ld_b(xs + (size_t)min((uint32_t)c, planes - 1u) * x_plane, off);
      } else {
        // the place's row and column in the tile; a row outside it is the neighbouring tile's
        const int32_t gr = (int32_t)(oh0 * P.sh + (pr_rc[k] >> 16)) - (int32_t)P.pad_h;
        const int32_t gc = (int32_t)(ow0 * P.sw + (pr_rc[k] & 0xffffu)) - (int32_t)P.pad_w;
        int32_t row = gr;
        uint32_t from = tile;
        bool in = pr_rc[k] != 0xffffffffu && n + pr_b[k] < P.N && gc >= 0 && gc < (int32_t)P.WP;
        if (gr < 0) {
          row = gr + (int32_t)P.HP;
          in = in && tile > 0u;
          from = tile > 0u ? tile - 1u : tile;
        } else if (gr >= (int32_t)P.HP) {
          row = gr - (int32_t)P.HP;
          in = in && tile + 1u < P.num_tiles;
          from = tile + 1u < P.num_tiles ? tile + 1u : tile;
        }
        in = in && row >= 0 && row < (int32_t)P.HP;
        pre_in |= in ? 2u << k : 0u;
        // a place that does not exist loads the first element of the unit's first image instead
        const char *px = reinterpret_cast<const char *>(reinterpret_cast<const T *>(P.x[from]) + ((size_t)n * P.Cin + cit * 16u) * x_plane) +
                         (in ? ((size_t)pr_b[k] * P.Cin * x_plane + (size_t)row * P.WP + (size_t)gc) * sizeof(T) : (size_t)0);
#pragma unroll
        for (int c = 0; c < 16; ++c)
          x_pre[k][c] = gen_ld_p(xs, px + (size_t)min((uint32_t)c, planes - 1u) * x_plane * sizeof(T));
      }
    }
  };
  auto store_unit = [&]() {
    if (dy_lane) {
      const bool in = (pre_in & 1u) != 0u;
#pragma unroll
      for (int c = 0; c < 16; ++c) dyl[(wave * 16u + c) * P.DP + lane] = in && c < co_lim ? dy_pre[c] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < KP; ++k) {
      if (pr_rc[k] == 0xffffffffu) continue;
      const bool in = ((pre_in >> (1 + k)) & 1u) != 0u;
#pragma unroll
      for (uint32_t c = 0; c < 16u; ++c)
        if (c < planes) patch[c * P.PP + pr_lds[k]] = in ? x_pre[k][c] : 0.f;
    }
  };
  const float *arow = dyl + (wave * 16u + l16) * P.DP + g;
  const float *bpl_g = patch + (PACKED ? 0u : my_plane * P.PP) + g * P.sw;
  // the operands of k-step ks: four consecutive pixels of the unit, one per lane group
  auto fetch = [&](uint32_t ks, float &a, float (&b)[TAPS]) {
    // the step's four pixels lie in one row (OWT is a multiple of 4): where the first one is is the same in every
    // lane and is worked out on the scalar unit; the lane adds its own pixel (bpl_g)
    uint32_t img, ip, r, c;
    P.div_img_pix.divmod(ks << 2, img, ip);
    P.div_OWT.divmod(ip, r, c);
    const float *brow = bpl_g + (img * P.PPI + r * P.sh * P.PCP + c * P.sw);
    a = arow[ks << 2];
#pragma unroll
    for (int t = 0; t < TAPS; ++t) b[t] = PACKED ? brow[pair_off[t]] : brow[__builtin_amdgcn_readlane(delta_vec, t)];
  };
  if (ps < P.units) load_unit(ps);
  for (uint32_t u = ps; u < P.units; u += P.PS) {
    __syncthreads();  // every wave is done with the previous unit
    store_unit();
    __syncthreads();
    if (u + P.PS < P.units) load_unit(u + P.PS);
    // two operand sets take turns: the reads of one k-step are in flight during the other's multiplications
    float a_cur, a_nxt = 0.f, b_cur[TAPS], b_nxt[TAPS];
    fetch(0, a_cur, b_cur);
    // (a fetch past the last k-step repeats the last one: every pass has the same number of reads in flight, so
    // the wait before a multiplication can leave the newer set outstanding)
    for (uint32_t ks = 0; ks < ksteps; ks += 2u) {
      fetch(min(ks + 1u, ksteps - 1u), a_nxt, b_nxt);
      __builtin_amdgcn_sched_barrier(0);  // keeps a set's reads together ahead of the other set's multiplications
#pragma unroll
      for (int t = 0; t < TAPS; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_cur, b_cur[t], acc[t], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (ks + 1u >= ksteps) break;
      fetch(min(ks + 2u, ksteps - 1u), a_cur, b_cur);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < TAPS; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a_nxt, b_nxt[t], acc[t], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // partial[ps][cog][cit][tg][t][mt = wave][lane][4]
  const size_t block_part = ((size_t)(cog * P.CIT + cit) * P.ntg + tg) * TAPS * 1024u;
  const size_t stride = (size_t)P.COG * P.CIT * P.ntg * TAPS * 1024u;
  float *dstp = P.partial + (size_t)ps * stride + block_part;
#pragma unroll
  for (int t = 0; t < TAPS; ++t) *reinterpret_cast<floatx4 *>(dstp + (t * 4 + wave) * 256u + lane * 4u) = acc[t];
}

struct WgradGenReduceParams {
  const float *partial;
  float *dw;
  uint32_t Cin, Cout, ntaps, T, ntg, COG, CIT, nparts, packed;
  float beta;
};

// 64 elements per workgroup; the partial sums of an element are dealt to four threads (part p to thread p % 4),
// whose sums are then added in thread order: a fixed order, so the result has fixed bits.
__global__ __launch_bounds__(256) void conv_gen_wgrad_reduce_kernel(const WgradGenReduceParams Q) {
  __shared__ float part_sum[4][64];
  const size_t stride = (size_t)Q.COG * Q.CIT * Q.ntg * Q.T * 1024u;
  const uint32_t slice = threadIdx.x >> 6, le = threadIdx.x & 63u;
  for (size_t e0 = (size_t)blockIdx.x * 64u; e0 < stride; e0 += (size_t)gridDim.x * 64u) {
    const size_t e = e0 + le;  // stride is a multiple of 1024: every e is in range
    const uint32_t i = (uint32_t)(e & 3u), lane = (uint32_t)((e >> 2) & 63u), mt = (uint32_t)((e >> 8) & 3u);
    size_t r = e >> 10;
    const uint32_t t = (uint32_t)(r % Q.T);
    r /= Q.T;
    const uint32_t tg = (uint32_t)(r % Q.ntg);
    r /= Q.ntg;
    const uint32_t cit = (uint32_t)(r % Q.CIT), cog = (uint32_t)(r / Q.CIT);
    const uint32_t co = cog * 64u + mt * 16u + (lane >> 4) * 4u + i;
    uint32_t ci = cit * 16u + (lane & 15u), tap = tg * Q.T + t;
    if (Q.packed) {  // column = pair tap * Cin + ci
      const uint32_t q = t * 16u + (lane & 15u);
      tap = q / Q.Cin;
      ci = q - tap * Q.Cin;
    }
    const bool real = co < Q.Cout && ci < Q.Cin && tap < Q.ntaps;
    float sum = 0.f;
    if (real)
      for (uint32_t p = slice; p < Q.nparts; p += 4u) sum += Q.partial[(size_t)p * stride + e];
    __syncthreads();  // the previous round's sums have been read
    part_sum[slice][le] = sum;
    __syncthreads();
    if (slice == 0u && real) {
      sum = ((part_sum[0][le] + part_sum[1][le]) + part_sum[2][le]) + part_sum[3][le];
      float *out = Q.dw + ((size_t)co * Q.Cin + ci) * Q.ntaps + tap;
      *out = Q.beta != 0.f ? *out + sum : sum;
    }
  }
}

struct WgradGenPlan {
  WgradGenParams P;
  size_t lds_bytes, partial_bytes;
  uint32_t blocks, nparts;
  bool packed, nbr;
};

// pad_h, pad_w (with `unpadded`): x carries no halo and is g.HP - 2 pad_h rows by g.WP - 2 pad_w columns
static int gen_plan_wgrad(const GenShape &g, uint32_t num_tiles, WgradGenPlan *plan, bool unpadded = false, uint32_t pad_h = 0,
                          uint32_t pad_w = 0) {
  WgradGenParams &P = plan->P;
  if (!unpadded) pad_h = pad_w = 0;
  plan->nbr = unpadded;
  P.pad_h = pad_h; P.pad_w = pad_w; P.num_tiles = num_tiles;
  P.N = g.N; P.Cin = g.Cin; P.Cout = g.Cout; P.HP = g.HP - 2u * pad_h; P.WP = g.WP - 2u * pad_w; P.OH = g.OH; P.OW = g.OW;
  P.sh = g.sh; P.sw = g.sw;
  P.ntaps = g.kh * g.kw;
  P.T = P.ntaps == 1u ? 1u : P.ntaps <= 4u ? 4u : 9u;
  P.ntg = (P.ntaps + P.T - 1u) / P.T;
  // few input channels and several taps: (tap, channel) pairs share the matrix columns, 4 or 10 tiles of 16
  const uint32_t pairs = P.ntaps * g.Cin;
  plan->packed = g.Cin <= 8u && P.ntaps > 1u && pairs <= 160u;
  if (plan->packed) {
    P.T = pairs <= 64u ? 4u : 10u;
    P.ntg = 1;
  }
  for (uint32_t a = 0; a < g.kh; ++a)
    for (uint32_t b = 0; b < g.kw; ++b) {
      P.off_r[a * g.kw + b] = (int16_t)(a * g.dh);
      P.off_c[a * g.kw + b] = (int16_t)(b * g.dw);
    }
  P.COG = (g.Cout + 63u) / 64u;
  P.CIT = plan->packed ? 1u : (g.Cin + 15u) / 16u;
  P.OWT = std::min<uint32_t>((g.OW + 3u) & ~3u, 64u);
  P.R = std::max<uint32_t>(1u, std::min<uint32_t>(g.OH, 64u / P.OWT));
  const uint32_t span_r = (g.kh - 1u) * g.dh + 1u, span_c = (g.kw - 1u) * g.dw + 1u;
  for (;;) {
    P.PR = (P.R - 1u) * g.sh + span_r;
    P.PC = (P.OWT - 1u) * g.sw + span_c;
    P.PCP = P.PC;
    P.PPI = P.PR * P.PCP;
    P.nrb = (g.OH + P.R - 1u) / P.R;
    P.ncb = (g.OW + P.OWT - 1u) / P.OWT;
    P.img_pix = P.R * P.OWT;
    // several images per unit when a whole image takes at most half of a unit's 64 pixel slots; the images of a
    // unit are reached from one base address by 32-bit byte offsets
    P.NBU = P.nrb == 1u && P.ncb == 1u && P.img_pix <= 32u ? std::min(64u / P.img_pix, std::max(g.N, 1u)) : 1u;
    while (P.NBU > 1u && (P.NBU * P.PR * P.PC > 512u ||
                          (uint64_t)P.NBU * std::max((uint64_t)g.Cin * g.HP * g.WP, (uint64_t)g.Cout * g.OH * g.OW) >= (1ull << 30)))
      --P.NBU;
    uint32_t pp = P.NBU * P.PPI;
    while (pp % 64u != 4u * std::min<uint32_t>(g.sw, 4u) % 64u) ++pp;  // 16 channels x 4 pixels on distinct banks
    P.PP = pp;
    uint32_t dp = P.NBU * P.img_pix;
    while (dp % 64u != 4u) ++dp;
    P.DP = dp;
    P.dy_lds_floats = 64u * P.DP;
    plan->lds_bytes = ((size_t)P.dy_lds_floats + 16u * (size_t)P.PP) * 4u;
    if (plan->lds_bytes <= kGenLdsBytes && P.NBU * P.PR * P.PC <= 512u) break;  // a thread stages up to two places per plane
    if (P.R > 1u) P.R /= 2u;
    else if (P.OWT > 4u) P.OWT = ((P.OWT / 2u) + 3u) & ~3u;
    else return ADH_EUNIMPL;
  }
  P.NG = (g.N + P.NBU - 1u) / P.NBU;
  const uint64_t units = (uint64_t)num_tiles * P.NG * P.nrb * P.ncb;
  if (units == 0 || units >= (1ull << 31)) return ADH_EINVAL;
  P.units = (uint32_t)units;
  const uint64_t fixed = (uint64_t)P.COG * P.CIT * P.ntg;
  const size_t stride_bytes = (size_t)fixed * P.T * 1024u * 4u;
  uint64_t ps = std::max<uint64_t>(1u, 1024u / fixed);  // about four workgroups per CU: they hide each other's staging
  if (P.T > 9u) ps = std::max<uint64_t>(1u, 512u / fixed);  // the ten-tile variant: two workgroups per CU, one round
  ps = std::min<uint64_t>(ps, units);
  while (ps > 1u && ps * stride_bytes > (256ull << 20)) ps /= 2u;
  if (fixed * ps >= (1ull << 24)) return ADH_EINVAL;
  P.PS = (uint32_t)ps;
  plan->nparts = P.PS;
  plan->blocks = (uint32_t)(fixed * ps);
  plan->partial_bytes = (size_t)plan->nparts * stride_bytes;
  P.div_COG = FastDiv(P.COG); P.div_CIT = FastDiv(P.CIT); P.div_ntg = FastDiv(P.ntg);
  P.div_ncb = FastDiv(P.ncb); P.div_nrb = FastDiv(P.nrb); P.div_N = FastDiv(P.NG);
  P.div_OWT = FastDiv(P.OWT); P.div_PC = FastDiv(P.PC); P.div_PR = FastDiv(P.PR);
  P.div_img_pix = FastDiv(P.img_pix); P.div_PRPC = FastDiv(P.PR * P.PC);
  return ADH_OK;
}

template <typename T, bool NBR>
static void launch_wgrad_gen_nbr(const WgradGenPlan &plan, hipStream_t st) {
  const WgradGenParams &P = plan.P;
  if (plan.packed && P.T == 4u)
    hipLaunchKernelGGL((conv_gen_wgrad_kernel<T, 4, true, NBR>), dim3(plan.blocks), dim3(kWgGenThreads), plan.lds_bytes, st, P);
  else if (plan.packed)
    hipLaunchKernelGGL((conv_gen_wgrad_kernel<T, 10, true, NBR>), dim3(plan.blocks), dim3(kWgGenThreads), plan.lds_bytes, st, P);
  else if (P.T == 1u)
    hipLaunchKernelGGL((conv_gen_wgrad_kernel<T, 1, false, NBR>), dim3(plan.blocks), dim3(kWgGenThreads), plan.lds_bytes, st, P);
  else if (P.T == 4u)
    hipLaunchKernelGGL((conv_gen_wgrad_kernel<T, 4, false, NBR>), dim3(plan.blocks), dim3(kWgGenThreads), plan.lds_bytes, st, P);
  else
    hipLaunchKernelGGL((conv_gen_wgrad_kernel<T, 9, false, NBR>), dim3(plan.blocks), dim3(kWgGenThreads), plan.lds_bytes, st, P);
}
template <typename T>
static void launch_wgrad_gen(const WgradGenPlan &plan, hipStream_t st) {
  if (plan.nbr) launch_wgrad_gen_nbr<T, true>(plan, st);
  else launch_wgrad_gen_nbr<T, false>(plan, st);
}

}  // namespace adh

using namespace adh;

namespace {

// Tiles without halo: the extents the padded form of the same convolution would have, and whether the row split
// is one the kernels serve.  H, W: the tile.  The tile's output must be H / sh rows (then any number of row tiles
// stitches to the unsplit output), and the taps may reach into the neighbouring tiles only.
int unpadded_geometry(uint32_t H, uint32_t W, uint32_t kh, uint32_t sh, uint32_t dh, uint32_t pad_h, uint32_t pad_w,
                      uint32_t *HP, uint32_t *WP) {
  if (H == 0 || W == 0 || sh == 0 || kh == 0 || dh == 0) return ADH_EINVAL;
  if (pad_h > 4096u || pad_w > 4096u) return ADH_EINVAL;
  const uint64_t eh = (uint64_t)(kh - 1u) * dh + 1u;
  if (H % sh != 0u) return ADH_EINVAL;
  // floor((H + 2 pad_h - eh) / sh) + 1 == H / sh
  if (2ull * pad_h >= eh || eh - 2ull * pad_h > sh) return ADH_EINVAL;
  if (pad_h > H || eh - 1u - pad_h > H) return ADH_EINVAL;
  *HP = H + 2u * pad_h;
  *WP = W + 2u * pad_w;
  return ADH_OK;
}

size_t conv2d_workspace(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP,
                        uint32_t WP, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw,
                        bool unpadded, uint32_t pad_h, uint32_t pad_w) {
  GenShape g;
  if (!dtype_ok(dtype) || gen_check_shape(num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, &g)) return 0;
  if (N == 0 || Cin == 0 || Cout == 0) return 0;
  if (which == ADH_CONV_BWD_FILTER) {
    WgradGenPlan wp = {};
    if (gen_plan_wgrad(g, num_tiles, &wp, unpadded, pad_h, pad_w)) return 0;
    size_t bytes = wp.partial_bytes;
    if (gen_is_pointwise_wgrad(dtype, g, unpadded, pad_h, pad_w))
      bytes = std::max(bytes, conv1x1_wgrad_workspace(num_tiles, N, Cin, Cout, g.OH, g.OW));
    if (gen_is_3x3s2_unpadded(dtype, g, unpadded, pad_h, pad_w))
      bytes = std::max(bytes, conv3x3s2_wgrad_workspace(num_tiles, N, Cin, Cout, g.HP - 2u, g.WP - 2u));
    if (gen_is_thin(dtype, g, unpadded))
      bytes = std::max(bytes, conv_thin_wgrad_workspace(num_tiles, N, Cin, Cout, g.HP, g.WP, g.OH, g.OW, kh, kw, sh, sw));
    if (gen_is_3x3_dilated(dtype, g, unpadded))
      bytes = std::max(bytes, conv3x3_dilated_wgrad_workspace(num_tiles, N, Cin, Cout, g.OH, g.OW, g.dh));
    return (bytes + 255u) & ~(size_t)255u;
  }
  GenPlan plan = {};
  plan.num_tiles = num_tiles;
  int e = ADH_EINVAL;
  if (which == ADH_CONV_FWD) e = gen_plan_fwd(g, &plan, unpadded ? pad_h : 0u, unpadded ? pad_w : 0u);
  else if (which == ADH_CONV_BWD_DATA) e = gen_plan_bwd_data(g, &plan, unpadded, pad_h, pad_w);
  if (e) return 0;
  return ((plan.wt_bytes + 255u) & ~(size_t)255u) + ((plan.part_bytes + 255u) & ~(size_t)255u);
}

int conv2d_fwd(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP,
               uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, bool unpadded, uint32_t pad_h,
               uint32_t pad_w, const void *const *x_tiles, const void *w, void *const *y_tiles, float beta, void *workspace,
               size_t workspace_bytes, void *stream, const float *const *bias_tiles = nullptr, bool *bias_added = nullptr) {
  // bias_tiles: added by the launch itself where the kernel that serves the shape can (*bias_added says so)
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  GenShape g;
  int e = gen_check_shape(num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, &g);
  if (e) return e;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (N == 0 || Cout == 0) return ADH_OK;
  if (Cin == 0) return ADH_EINVAL;
  if (!x_tiles || !y_tiles || !w) return ADH_ENULL;
  GenPlan plan = {};
  plan.num_tiles = num_tiles;
  plan.nbr = unpadded;
  e = gen_plan_fwd(g, &plan, unpadded ? pad_h : 0u, unpadded ? pad_w : 0u);
  if (e) return e;
  const size_t es = dtype_size(dtype);
  if (!aligned_to(w, es)) return ADH_EALIGN;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!x_tiles[t] || !y_tiles[t]) return ADH_ENULL;
    if (!aligned_to(x_tiles[t], es) || !aligned_to(y_tiles[t], es)) return ADH_EALIGN;
    plan.P.in[t] = x_tiles[t];
    plan.P.out[t] = y_tiles[t];
  }
  plan.P.beta = beta;
  if (gen_is_pointwise(dtype, g, unpadded, pad_h, pad_w)) {
    e = gen_check_workspace(plan, workspace, workspace_bytes);  // not used, but the contract is one for all shapes
    if (e) return e;
    e = conv1x1_try(false, num_tiles, N, Cin, Cout, g.HP, g.WP, g.OH, g.OW, g.sh, x_tiles, w, y_tiles, beta, as_stream(stream));
    if (e != ADH_EUNIMPL) return e;
  }
  if (gen_is_thin(dtype, g, unpadded)) {
    e = gen_check_workspace(plan, workspace, workspace_bytes);
    if (e) return e;
    e = conv_thin_fwd_try(num_tiles, N, Cin, Cout, g.HP, g.WP, g.OH, g.OW, kh, kw, sh, sw, x_tiles, w, y_tiles, beta,
                          as_stream(stream), bias_tiles);
    if (e == ADH_OK && bias_tiles && bias_added) *bias_added = true;
    if (e != ADH_EUNIMPL) return e;
  }
  if (gen_is_3x3_dilated(dtype, g, unpadded)) {
    e = gen_check_workspace(plan, workspace, workspace_bytes);
    if (e) return e;
    e = conv3x3_dilated_try(ADH_CONV_FWD, dtype, num_tiles, N, Cin, Cout, g.OH, g.OW, g.dh, x_tiles, w, y_tiles, beta,
                            as_stream(stream));
    if (e != ADH_EUNIMPL) return e;
  }
  if (dtype == ADH_F32 && unpadded && kh == 3u && kw == 3u && sh == 2u && sw == 2u && dh == 1u && dw == 1u && pad_h == 1u &&
      pad_w == 1u) {
    e = gen_check_workspace(plan, workspace, workspace_bytes);
    if (e) return e;
    e = conv3x3s2_fwd_try(num_tiles, N, Cin, Cout, g.HP - 2u, g.WP - 2u, x_tiles, w, y_tiles, beta, as_stream(stream));
    if (e != ADH_EUNIMPL) return e;
  }
  return gen_launch(dtype, &plan, num_tiles, w, workspace, workspace_bytes, as_stream(stream));
}

int conv2d_bwd_data(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP,
                    uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, bool unpadded,
                    uint32_t pad_h, uint32_t pad_w, const void *w, const void *const *dy_tiles, void *const *dx_tiles,
                    float beta, void *workspace, size_t workspace_bytes, void *stream) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  GenShape g;
  int e = gen_check_shape(num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, &g);
  if (e) return e;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (N == 0 || Cin == 0) return ADH_OK;
  if (Cout == 0) return ADH_EINVAL;
  if (!dy_tiles || !dx_tiles || !w) return ADH_ENULL;
  GenPlan plan = {};
  plan.num_tiles = num_tiles;
  plan.nbr = unpadded;
  e = gen_plan_bwd_data(g, &plan, unpadded, pad_h, pad_w);
  if (e) return e;
  const size_t es = dtype_size(dtype);
  if (!aligned_to(w, es)) return ADH_EALIGN;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!dy_tiles[t] || !dx_tiles[t]) return ADH_ENULL;
    if (!aligned_to(dy_tiles[t], es) || !aligned_to(dx_tiles[t], es)) return ADH_EALIGN;
    plan.P.in[t] = dy_tiles[t];
    plan.P.out[t] = dx_tiles[t];
  }
  plan.P.beta = beta;
  if (gen_is_pointwise(dtype, g, unpadded, pad_h, pad_w)) {
    e = gen_check_workspace(plan, workspace, workspace_bytes);
    if (e) return e;
    e = conv1x1_try(true, num_tiles, N, Cin, Cout, g.HP, g.WP, g.OH, g.OW, g.sh, dy_tiles, w, dx_tiles, beta, as_stream(stream));
    if (e != ADH_EUNIMPL) return e;
  }
  if (gen_is_3x3_dilated(dtype, g, unpadded)) {
    e = gen_check_workspace(plan, workspace, workspace_bytes);
    if (e) return e;
    e = conv3x3_dilated_try(ADH_CONV_BWD_DATA, dtype, num_tiles, N, Cin, Cout, g.OH, g.OW, g.dh, dy_tiles, w, dx_tiles, beta,
                            as_stream(stream));
    if (e != ADH_EUNIMPL) return e;
  }
  if (dtype == ADH_F32 && unpadded && kh == 3u && kw == 3u && sh == 2u && sw == 2u && dh == 1u && dw == 1u && pad_h == 1u &&
      pad_w == 1u) {
    e = gen_check_workspace(plan, workspace, workspace_bytes);
    if (e) return e;
    e = conv3x3s2_bwd_data_try(num_tiles, N, Cin, Cout, g.HP - 2u, g.WP - 2u, w, dy_tiles, dx_tiles, beta, as_stream(stream));
    if (e != ADH_EUNIMPL) return e;
  }
  return gen_launch(dtype, &plan, num_tiles, w, workspace, workspace_bytes, as_stream(stream));
}

int conv2d_bwd_filter(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP,
                      uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, bool unpadded,
                      uint32_t pad_h, uint32_t pad_w, const void *const *x_tiles, const void *const *dy_tiles, float *dwt,
                      float beta, void *workspace, size_t workspace_bytes, void *stream) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  GenShape g;
  int e = gen_check_shape(num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, &g);
  if (e) return e;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (Cin == 0 || Cout == 0) return ADH_OK;
  if (!dwt) return ADH_ENULL;
  if (!aligned_to(dwt, 4)) return ADH_EALIGN;
  hipStream_t st = as_stream(stream);
  if (N == 0) {  // an empty sum
    if (beta == 0.f) return adh_fill_f32((uint64_t)Cout * Cin * kh * kw, 0.f, dwt, stream);
    return ADH_OK;
  }
  if (!x_tiles || !dy_tiles) return ADH_ENULL;
  WgradGenPlan plan = {};
  e = gen_plan_wgrad(g, num_tiles, &plan, unpadded, pad_h, pad_w);
  if (e) return e;
  const size_t es = dtype_size(dtype);
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!x_tiles[t] || !dy_tiles[t]) return ADH_ENULL;
    if (!aligned_to(x_tiles[t], es) || !aligned_to(dy_tiles[t], es)) return ADH_EALIGN;
    plan.P.x[t] = x_tiles[t];
    plan.P.dy[t] = dy_tiles[t];
  }
  if (!workspace) return ADH_ENULL;
  if (!aligned_to(workspace, 256)) return ADH_EALIGN;
  if (workspace_bytes < plan.partial_bytes) return ADH_EWORKSPACE;
  if (gen_is_pointwise_wgrad(dtype, g, unpadded, pad_h, pad_w)) {
    const size_t need = conv1x1_wgrad_workspace(num_tiles, N, Cin, Cout, g.OH, g.OW);
    if (need != 0) {
      if (workspace_bytes < need) return ADH_EWORKSPACE;
      e = conv1x1_wgrad_try(num_tiles, N, Cin, Cout, g.HP, g.WP, g.OH, g.OW, g.sh, g.sw, x_tiles, dy_tiles, dwt, beta,
                            workspace, st);
      if (e != ADH_EUNIMPL) return e;
    }
  }
  if (gen_is_thin(dtype, g, unpadded)) {
    const size_t need = conv_thin_wgrad_workspace(num_tiles, N, Cin, Cout, g.HP, g.WP, g.OH, g.OW, kh, kw, sh, sw);
    if (need != 0) {
      if (workspace_bytes < need) return ADH_EWORKSPACE;
      e = conv_thin_wgrad_try(num_tiles, N, Cin, Cout, g.HP, g.WP, g.OH, g.OW, kh, kw, sh, sw, x_tiles, dy_tiles, dwt, beta,
                              workspace, st);
      if (e != ADH_EUNIMPL) return e;
    }
  }
  if (gen_is_3x3_dilated(dtype, g, unpadded)) {
    const size_t need = conv3x3_dilated_wgrad_workspace(num_tiles, N, Cin, Cout, g.OH, g.OW, g.dh);
    if (need != 0) {
      if (workspace_bytes < need) return ADH_EWORKSPACE;
      e = conv3x3_dilated_wgrad_try(num_tiles, N, Cin, Cout, g.OH, g.OW, g.dh, x_tiles, dy_tiles, dwt, beta, workspace, st);
      if (e != ADH_EUNIMPL) return e;
    }
  }
  if (gen_is_3x3s2_unpadded(dtype, g, unpadded, pad_h, pad_w)) {
    const size_t need = conv3x3s2_wgrad_workspace(num_tiles, N, Cin, Cout, g.HP - 2u, g.WP - 2u);
    if (need != 0) {
      if (workspace_bytes < need) return ADH_EWORKSPACE;
      e = conv3x3s2_wgrad_try(num_tiles, N, Cin, Cout, g.HP - 2u, g.WP - 2u, x_tiles, dy_tiles, dwt, beta, workspace, st);
      if (e != ADH_EUNIMPL) return e;
    }
  }
  plan.P.partial = reinterpret_cast<float *>(workspace);
  if (dtype == ADH_F32) launch_wgrad_gen<float>(plan, st);
  else launch_wgrad_gen<uint16_t>(plan, st);
  WgradGenReduceParams Q;
  Q.partial = plan.P.partial;
  Q.dw = dwt;
  Q.Cin = Cin; Q.Cout = Cout; Q.ntaps = plan.P.ntaps; Q.T = plan.P.T; Q.ntg = plan.P.ntg;
  Q.COG = plan.P.COG; Q.CIT = plan.P.CIT; Q.nparts = plan.nparts;
  Q.packed = plan.packed ? 1u : 0u;
  Q.beta = beta;
  const size_t stride = (size_t)Q.COG * Q.CIT * Q.ntg * Q.T * 1024u;
  hipLaunchKernelGGL(conv_gen_wgrad_reduce_kernel, dim3((uint32_t)std::min<size_t>((stride + 63u) / 64u, 65535u)),
                     dim3(256), 0, st, Q);
  return launch_status();
}

}  // namespace

extern "C" {

size_t adh_conv2d_workspace_bytes(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                  uint32_t HP, uint32_t WP, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw,
                                  uint32_t dh, uint32_t dw) {
  return conv2d_workspace(which, dtype, num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, false, 0, 0);
}

int adh_conv2d_slab_fwd_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP,
                              uint32_t WP, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw,
                              const void *const *x_pad_tiles, const void *w, void *const *y_tiles, float beta,
                              void *workspace, size_t workspace_bytes, void *stream) {
  return conv2d_fwd(dtype, num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, false, 0, 0, x_pad_tiles, w, y_tiles, beta,
                    workspace, workspace_bytes, stream);
}

int adh_conv2d_slab_fwd_bias_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP,
                                   uint32_t WP, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw,
                                   const void *const *x_pad_tiles, const void *w, const float *const *bias_tiles,
                                   void *const *y_tiles, float beta, void *workspace, size_t workspace_bytes, void *stream) {
  if (!bias_tiles) return ADH_ENULL;
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!bias_tiles[t]) return ADH_ENULL;
    if (!aligned_to(bias_tiles[t], 4)) return ADH_EALIGN;
  }
  bool added = false;
  const int e = conv2d_fwd(dtype, num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, false, 0, 0, x_pad_tiles, w, y_tiles,
                           beta, workspace, workspace_bytes, stream, bias_tiles, &added);
  if (e != ADH_OK || added || N == 0 || Cout == 0) return e;
  // the shape has been checked by the convolution: the output extents follow from it
  const uint32_t OH = (HP - ((kh - 1u) * dh + 1u)) / sh + 1u, OW = (WP - ((kw - 1u) * dw + 1u)) / sw + 1u;
  return adh_conv_bias_add_tiles(dtype, num_tiles, N, Cout, OH, OW, bias_tiles, y_tiles, stream);
}

int adh_conv2d_slab_bwd_data_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP,
                                   uint32_t WP, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh,
                                   uint32_t dw, const void *w, const void *const *dy_tiles, void *const *dx_pad_tiles,
                                   float beta, void *workspace, size_t workspace_bytes, void *stream) {
  return conv2d_bwd_data(dtype, num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, false, 0, 0, w, dy_tiles,
                         dx_pad_tiles, beta, workspace, workspace_bytes, stream);
}

int adh_conv2d_slab_bwd_filter_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP,
                                     uint32_t WP, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh,
                                     uint32_t dw, const void *const *x_pad_tiles, const void *const *dy_tiles,
                                     float *dwt, float beta, void *workspace, size_t workspace_bytes, void *stream) {
  return conv2d_bwd_filter(dtype, num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, false, 0, 0, x_pad_tiles, dy_tiles,
                           dwt, beta, workspace, workspace_bytes, stream);
}

size_t adh_conv2d_unpadded_workspace_bytes(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin,
                                           uint32_t Cout, uint32_t H, uint32_t W, uint32_t kh, uint32_t kw, uint32_t sh,
                                           uint32_t sw, uint32_t dh, uint32_t dw, uint32_t pad_h, uint32_t pad_w) {
  uint32_t HP, WP;
  if (unpadded_geometry(H, W, kh, sh, dh, pad_h, pad_w, &HP, &WP)) return 0;
  return conv2d_workspace(which, dtype, num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, true, pad_h, pad_w);
}

int adh_conv2d_unpadded_fwd_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                                  uint32_t W, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw,
                                  uint32_t pad_h, uint32_t pad_w, const void *const *x_tiles, const void *w,
                                  void *const *y_tiles, float beta, void *workspace, size_t workspace_bytes, void *stream) {
  uint32_t HP, WP;
  const int e = unpadded_geometry(H, W, kh, sh, dh, pad_h, pad_w, &HP, &WP);
  if (e) return e;
  return conv2d_fwd(dtype, num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, true, pad_h, pad_w, x_tiles, w, y_tiles,
                    beta, workspace, workspace_bytes, stream);
}

int adh_conv2d_unpadded_bwd_data_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                                       uint32_t W, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh,
                                       uint32_t dw, uint32_t pad_h, uint32_t pad_w, const void *w,
                                       const void *const *dy_tiles, void *const *dx_tiles, float beta, void *workspace,
                                       size_t workspace_bytes, void *stream) {
  uint32_t HP, WP;
  const int e = unpadded_geometry(H, W, kh, sh, dh, pad_h, pad_w, &HP, &WP);
  if (e) return e;
  return conv2d_bwd_data(dtype, num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, true, pad_h, pad_w, w, dy_tiles,
                         dx_tiles, beta, workspace, workspace_bytes, stream);
}

int adh_conv2d_unpadded_bwd_filter_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                                         uint32_t W, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh,
                                         uint32_t dw, uint32_t pad_h, uint32_t pad_w, const void *const *x_tiles,
                                         const void *const *dy_tiles, float *dwt, float beta, void *workspace,
                                         size_t workspace_bytes, void *stream) {
  uint32_t HP, WP;
  const int e = unpadded_geometry(H, W, kh, sh, dh, pad_h, pad_w, &HP, &WP);
  if (e) return e;
  return conv2d_bwd_filter(dtype, num_tiles, N, Cin, Cout, HP, WP, kh, kw, sh, sw, dh, dw, true, pad_h, pad_w, x_tiles,
                           dy_tiles, dwt, beta, workspace, workspace_bytes, stream);
}

}  // extern "C"
