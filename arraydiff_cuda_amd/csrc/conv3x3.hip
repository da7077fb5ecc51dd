// 3x3 convolution over the halo-padded slab on the gfx950 matrix cores (fp32 MFMA).
//
// One kernel serves forward and backward-data, both written as
//   out[o][oh][ow] = beta*out + sum_{k,a,b} Wt(o,k,a,b) * in[k][oh + a - pad][ow + b - pad]
// (zero outside the input plane):
//   forward       : in = padded slab x (H+2, W+2), out = y (H, W),        pad = 0,
//                   Wt(o=co,k=ci,a,b) = w[co][ci][a][b]
//   backward-data : in = dy (H, W),  out = WHOLE padded slab dx (H+2, W+2), pad = 2,
//                   Wt(o=ci,k=co,a,b) = w[co][ci][2-a][2-b]
//
// Mapping to the hardware (wave64, v_mfma_f32_16x16x4_f32):
//   * implicit GEMM D[o][pixel] += A[o][k] * B[k][pixel]; the MFMA "column" dimension is
//     the pixel, so lane%16 walks consecutive output pixels and stores are contiguous runs.
//   * a workgroup (4 waves) owns R output rows x TW columns of one image for 64 output
//     channels; wave v owns output channels [16v, 16v+16) and ALL NT = ceil(R*TW/16) pixel
//     tiles, so the four matrix pipes of a CU carry identical work (NT accumulators of 4
//     VGPRs each per wave).
//   * the reduction runs over chunks of 8 input channels.  The (R+2) x (TW+2) input patch of
//     a chunk is staged once in LDS (pitch 64 floats, channel stride = 16 mod 64 banks so the
//     four k-groups of an MFMA read disjoint banks) and reused by all 9 taps, all 4 waves and
//     all 64 output channels: each input element is fetched from HBM once per workgroup.
//     Every B operand is one ds_read_b32 at lane_base + compile-time immediate.
//   * the 64 x 8 x 9 weights of a chunk are staged in LDS too (read from global in memory
//     order, coalesced); an A operand is one ds_read_b32 per NT MFMAs.
//   * staging is asynchronous and register-free: global_load_lds writes each lane's dword
//     straight into LDS.  The loads of chunk c+1 are issued before the MFMAs of chunk c into
//     the other buffer pair; one barrier per chunk.
#include <stdio.h>

#include "adh_common.h"

namespace adh {

typedef float floatx4 __attribute__((ext_vector_type(4)));

static constexpr int kChunk = 8;        // reduction channels per LDS stage
static constexpr int kLdsPitch = 64;    // floats per staged patch row
static constexpr int kMaxTW = kLdsPitch - 2;
static constexpr int kWBufFloats = 64 * kChunk * 9;  // weights of one chunk in LDS
// word 3 of a gfx9-family buffer resource: 32-bit data format, raw (unstructured) addressing
static constexpr int kBufferFlags = 0x00020000;
// a byte offset no resource of at most 2 GiB contains: such a lane loads zero
static constexpr uint32_t kOutOfRange = 0x80000000u;

struct ConvParams {
  const float *in[ADH_MAX_TILES];
  float *out[ADH_MAX_TILES];
  const float *w;
  uint32_t num_tiles, N;
  uint32_t Cred, Cout;      // reduction channels / output channels of this pass
  uint32_t IH, IW, OH, OW;  // input and output plane extents
  int32_t pad;              // input row = oh + a - pad
  uint32_t R, TW;           // workgroup tile: R output rows x TW output columns
  uint32_t tiles_x;         // ceil(OW / TW); grid.x = tiles_x * ceil(OH / R)
  uint32_t w_out_stride, w_red_stride;  // weight address = o*w_out_stride + k*w_red_stride + tap'
  int32_t w_flip;           // tap' = w_flip ? 8 - tap : tap
  // The tiles are the row tiles of one activation, in rank order, and two input rows come from the
  // neighbouring tiles: row nb_lo of tile t > 0 is tile t-1's row nb_above, row nb_hi of tile
  // t < num_tiles-1 is tile t+1's row nb_below.  Forward (padded input whose inner halo rows nobody
  // exchanged): rows 0 and IH-1 are the neighbours' last and first interior rows, IH-2 and 1.
  // Backward-data (unpadded dy): rows -1 and IH are the neighbours' rows IH-1 and 0, which makes
  // the interior of the gradient tile complete, as after a halo reduce.
  int32_t rows_from_neighbours, nb_lo, nb_hi, nb_above, nb_below;
  float beta;
  // res[t] set (with beta = 1): the value added to the result is read from res[t], a tensor laid out like out[t],
  // instead of from out[t] itself: out = conv(in) + res, the residual sum of a block in the convolution's stores
  const float *res[ADH_MAX_TILES];
  FastDiv div_tiles_x, div_TW;
};

// staged patch rows (>= R + 2): 12, or 20 in the tall variant of the kernel, which is a few percent slower per
// flop (more rows to stage per wave) and is chosen where taller tiles waste fewer pixel slots, or 10 in the
// short variant of the 16-tile kernel: its buffers then take 77 KB, two workgroups share a CU and the waits of
// one (its first chunk, the barrier after every chunk, its stores) are the other's matrix-core time
static constexpr int kPatchRows = 12;
static constexpr int kPatchRowsTall = 20;
static constexpr int kPatchRowsShort = 10;
static constexpr int kMaxR = kPatchRows - 2;
static constexpr int kMaxRTall = kPatchRowsTall - 2;
static constexpr int kMaxRShort = kPatchRowsShort - 2;

template <int V>
struct IntTag {
  static constexpr int value = V;
};

// NT    = pixel tiles of 16 per workgroup (R*TW <= 16*NT)
// WAVES = 4: wave v owns output channels [16v,16v+16) and all NT tiles;
//         8: two waves per SIMD, waves v and v+4 share the channels and split the tiles
//            (ceil(NT/2) and the rest), which hides LDS latency and barrier skew behind the
//            other wave's MFMAs while every SIMD still carries exactly NT tile-MFMAs per k-step
// FLIP  = false: forward (weights walked as w[o][k][tap]); true: backward-data
//         (weights walked as w[k][o][8-tap]).
// DIL   = dilation of the window: tap (a, b) reads the input DIL * a rows and DIL * b columns on (pad counts input
//         pixels: 0 forward over a slab padded by DIL, 2 * DIL backward-data); the staged patch is then
//         (R + 2 DIL) x (TW + 2 DIL), which must fit PROWS rows of 64 floats.
template <int NT, int WAVES, bool FLIP, int PROWS, int DIL = 1>
__global__ __launch_bounds__(64 * WAVES, PROWS == kPatchRowsShort ? 2 : 1) void conv3x3_f32_kernel(const ConvParams P) {
  constexpr int kChanStride = PROWS * kLdsPitch + 16;  // == 16 (mod 64)
  constexpr int kPatchFloats = kChunk * kChanStride;
  constexpr int kThreads = 64 * WAVES;
  constexpr int G = WAVES / 4;                 // pixel groups
  constexpr int NTA = (NT + G - 1) / G;        // tiles of every group but the last
  constexpr int NTL = NT - (G - 1) * NTA;      // tiles of the last group
  constexpr int RROWS = (PROWS + WAVES - 1) / WAVES;
  constexpr int WLOADS = kWBufFloats / kThreads;
  static_assert(kWBufFloats % kThreads == 0 && NTL > 0, "bad configuration");
  // two patch buffers and two weight buffers as separate arrays: the compiler can then tell
  // that the LDS reads of one buffer never alias the asynchronous writes into the other
  __shared__ float patch0[kPatchFloats];
  __shared__ float patch1[kPatchFloats];
  __shared__ float wbuf0[kWBufFloats];
  __shared__ float wbuf1[kWBufFloats];

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u, g = lane >> 4, l16 = lane & 15u;
  // the wave index is uniform; saying so keeps LDS destinations of the async loads in SGPRs
  const uint32_t wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t ot = wv & 3u;   // output-channel tile of this wave
  const uint32_t pg = wv >> 2;   // pixel group of this wave

  const uint32_t ty = P.div_tiles_x.div(blockIdx.x);
  const uint32_t tx = blockIdx.x - ty * P.tiles_x;
  const uint32_t n = blockIdx.z / P.num_tiles;
  const uint32_t t = blockIdx.z - n * P.num_tiles;
  const uint32_t oh0 = ty * P.R, ow0 = tx * P.TW;
  const uint32_t o_blk = blockIdx.y * 64u;
  const uint64_t in_plane = (uint64_t)P.IH * P.IW;
  const uint64_t out_plane = (uint64_t)P.OH * P.OW;
  const float *__restrict__ in = P.in[t] + (uint64_t)n * P.Cred * in_plane;
  // `added` is `out` itself unless a residual is given, and a residual may be the result tensor: neither may be
  // declared free of aliases (an element is read, then written, by the same lane)
  float *out = P.out[t] + (uint64_t)n * P.Cout * out_plane;
  const float *added = P.res[t] ? P.res[t] + (uint64_t)n * P.Cout * out_plane : out;

  const uint32_t rows_here = min(P.R, P.OH - oh0);
  const uint32_t cols_here = min(P.TW, P.OW - ow0);
  const uint32_t npix = P.R * P.TW;
  const uint32_t nchunks = (P.Cred + kChunk - 1) / kChunk;
  const bool ragged_k = (P.Cred % kChunk) != 0;

  // ---- patch staging: lane = patch column, wave = patch row (mod WAVES); global -> LDS
  // without passing through registers (buffer_load ... lds: each lane's dword lands at
  // base + 4*lane).  Buffer addressing: a 128-bit resource (SGPRs) for this image, one 32-bit
  // VGPR offset per lane that never changes, and the channel offset in an SGPR - no per-load
  // address math and no branches: a lane whose element lies outside the input plane carries
  // an offset beyond the resource's size, for which the hardware writes ZERO into LDS. ----
  const int32_t iw = (int32_t)(ow0 + lane) - P.pad;
  const bool col_ok = lane < P.TW + 2u * DIL && iw >= 0 && iw < (int32_t)P.IW;
  const uint32_t patch_rows = P.R + 2u * DIL;
  uint32_t row_voff[RROWS];
  // a patch row is one wave's, so the image it is read from is a wave-uniform choice: one buffer
  // resource per patch row of this wave
  __amdgpu_buffer_rsrc_t rsrc_row[RROWS];
#pragma unroll
  for (int rr = 0; rr < RROWS; ++rr) {
    const uint32_t prow = wv + (uint32_t)WAVES * rr;
    int32_t ih = (int32_t)(oh0 + prow) - P.pad;
    const bool ok = col_ok && prow < patch_rows;
    const float *src = in;
    bool ok_row = ih >= 0 && ih < (int32_t)P.IH;
    if (P.rows_from_neighbours) {
      if (ih == P.nb_lo && t > 0u) {
        src = P.in[t - 1u] + (uint64_t)n * P.Cred * in_plane;
        ih = P.nb_above;
        ok_row = true;
      } else if (ih == P.nb_hi && t + 1u < P.num_tiles) {
        src = P.in[t + 1u] + (uint64_t)n * P.Cred * in_plane;
        ih = P.nb_below;
        ok_row = true;
      }
    }
    row_voff[rr] = ok && ok_row ? ((uint32_t)ih * P.IW + (uint32_t)iw) * 4u : kOutOfRange;
    rsrc_row[rr] = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(src), 0,
                                                     (int)(P.Cred * (uint32_t)in_plane * 4u), kBufferFlags);
  }
  auto stage_patch = [&](float *buf, uint32_t k0) {
    const bool ragged = ragged_k && k0 + kChunk > P.Cred;  // uniform: a ragged last chunk
#pragma unroll
    for (int rr = 0; rr < RROWS; ++rr) {
      const uint32_t prow = wv + (uint32_t)WAVES * rr;
      if (PROWS % WAVES != 0 && prow >= (uint32_t)PROWS) continue;  // wave-uniform
#pragma unroll
      for (int kl = 0; kl < kChunk; ++kl) {
        float *dst = buf + kl * kChanStride + prow * kLdsPitch;
        if (!ragged) {
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_row[rr], dst, 4, row_voff[rr], (k0 + kl) * (uint32_t)in_plane * 4u, 0, 0);
        } else {  // channels past Cred are loaded as zero
          const bool k_ok = k0 + kl < P.Cred;
          const uint32_t soff = __builtin_amdgcn_readfirstlane(min(k0 + kl, P.Cred - 1u) * (uint32_t)in_plane * 4u);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_row[rr], dst, 4, k_ok ? row_voff[rr] : kOutOfRange, soff, 0, 0);
        }
      }
    }
  };

  // ---- weight staging: the 4608 floats of a chunk in memory order, also global -> LDS
  // directly.  forward: wl[o][72] (72 contiguous floats per output channel);
  // backward-data: wl[k][576] (576 contiguous floats per reduction channel). ----
  uint32_t w_voff[WLOADS];  // byte offset inside the chunk's weight block, out of range if the
                            // element's output channel does not exist
#pragma unroll
  for (int i = 0; i < WLOADS; ++i) {
    const uint32_t f = tid + (uint32_t)kThreads * i;
    uint32_t o_l, goff;
    if (FLIP) {
      const uint32_t k_l = f / 576u;
      const uint32_t rem = f - k_l * 576u;
      o_l = rem / 9u;
      goff = k_l * P.w_red_stride + rem;
    } else {
      o_l = f / 72u;
      goff = o_l * P.w_out_stride + (f - o_l * 72u);
    }
    w_voff[i] = (o_blk + o_l < P.Cout) ? goff * 4u : kOutOfRange;
  }
  const uint32_t w_blk = FLIP ? o_blk * 9u : o_blk * P.w_out_stride;
  const uint32_t w_chunk_stride = FLIP ? kChunk * P.w_red_stride : kChunk * 9u;
  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(P.w), 0, (int)(P.Cout * P.Cred * 36u), kBufferFlags);
  auto stage_weights = [&](float *wl, uint32_t c) {
    const uint32_t soff = (w_blk + c * w_chunk_stride) * 4u;
    const bool ragged = ragged_k && (c + 1u) * kChunk > P.Cred;  // uniform
#pragma unroll
    for (int i = 0; i < WLOADS; ++i) {
      uint32_t voff = w_voff[i];
      if (ragged) {
        const uint32_t f = tid + (uint32_t)kThreads * i;
        const uint32_t k_l = FLIP ? f / 576u : (f % 72u) / 9u;
        if (c * kChunk + k_l >= P.Cred) voff = kOutOfRange;
      }
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, wl + kThreads * i + 64u * wv, 4, voff, soff, 0, 0);
    }
  };
  // A[o = 16*ot + l16][k = 4*kk + g][tap]
  const uint32_t a_lane = FLIP ? (16u * ot + l16) * 9u + g * 576u : (16u * ot + l16) * 72u + g * 9u;

  auto a_off = [](int s_) {
    const int kk = s_ / 9, tap = s_ % 9;
    return FLIP ? kk * 4 * 576 + (8 - tap) : kk * 36 + tap;
  };
  auto b_off = [](int s_) {
    const int kk = s_ / 9, tap = s_ % 9;
    return kk * 4 * kChanStride + (tap / 3) * DIL * kLdsPitch + (tap % 3) * DIL;
  };

  // Everything that depends on the number of pixel tiles this wave owns.
  auto run = [&](auto cnt_tag, uint32_t tile0) {
    constexpr int CNT = decltype(cnt_tag)::value;

    // LDS float offset of this lane's pixel in each pixel tile (+ the lane's k-group plane)
    uint32_t pix[CNT];
#pragma unroll
    for (int j = 0; j < CNT; ++j) {
      uint32_t q = 16u * (tile0 + j) + l16;
      if (q >= npix) q = 0;
      uint32_t r_, c_;
      P.div_TW.divmod(q, r_, c_);
      pix[j] = g * kChanStride + r_ * kLdsPitch + c_;
    }

    floatx4 acc[CNT];
#pragma unroll
    for (int j = 0; j < CNT; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};

    // One chunk = 18 k-steps (2 groups of 4 channels x 9 taps), CNT MFMAs each.  The operands
    // of k-step s+1 are read from LDS while the MFMAs of k-step s issue, one ds_read per MFMA,
    // into the other half of a two-deep register buffer; the scheduling-group barriers pin
    // that interleaving (left alone, the scheduler hoists hundreds of reads and spills).
    auto compute = [&](const float *cur, const float *wcur) {
      float a[2], b[2][CNT];
      a[0] = wcur[a_lane + a_off(0)];
#pragma unroll
      for (int j = 0; j < CNT; ++j) b[0][j] = cur[pix[j] + b_off(0)];
#pragma unroll
      for (int s_ = 0; s_ < 18; ++s_) {
        const int cb = s_ & 1, nb = cb ^ 1;
        if (s_ + 1 < 18) a[nb] = wcur[a_lane + a_off(s_ + 1)];
#pragma unroll
        for (int j = 0; j < CNT; ++j) {
          if (s_ + 1 < 18) b[nb][j] = cur[pix[j] + b_off(s_ + 1)];
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[cb], b[cb][j], acc[j], 0, 0, 0);
        }
        if (s_ + 1 < 18) {
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // the A read
#pragma unroll
          for (int j = 0; j < CNT; ++j) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };

    // two chunks per trip so that each phase names its buffers statically
    for (uint32_t c = 0;;) {
      if (c + 1 < nchunks) {
        stage_patch(patch1, (c + 1) * kChunk);
        stage_weights(wbuf1, c + 1);
      }
      __builtin_amdgcn_sched_barrier(0);  // keep the async loads ahead of the matrix work
      compute(patch0, wbuf0);
      __syncthreads();
      if (++c == nchunks) break;
      if (c + 1 < nchunks) {
        stage_patch(patch0, (c + 1) * kChunk);
        stage_weights(wbuf0, c + 1);
      }
      __builtin_amdgcn_sched_barrier(0);
      compute(patch1, wbuf1);
      __syncthreads();
      if (++c == nchunks) break;
    }

    // ---- epilogue: lane holds D[o = 4*g + i][pixel = l16] of each tile ----
    const uint32_t o_d = o_blk + 16u * ot + 4u * g;
#pragma unroll
    for (int j = 0; j < CNT; ++j) {
      const uint32_t q = 16u * (tile0 + j) + l16;
      uint32_t r_, c_;
      P.div_TW.divmod(q, r_, c_);
      if (q < npix && r_ < rows_here && c_ < cols_here) {
        const uint64_t at = (uint64_t)o_d * out_plane + (uint64_t)(oh0 + r_) * P.OW + ow0 + c_;
        float *dst = out + at;
        const float *src = added + at;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (o_d + i < P.Cout) {
            float v = acc[j][i];
            if (P.beta != 0.f) v += P.beta * src[(uint64_t)i * out_plane];
            dst[(uint64_t)i * out_plane] = v;
          }
        }
      }
    }
  };

  stage_patch(patch0, 0);
  stage_weights(wbuf0, 0);
  __syncthreads();  // the compiler waits for the outstanding LDS-bound loads before the barrier

  if (G == 1 || NTL == NTA) {
    run(IntTag<NTA>(), pg * NTA);
  } else if (pg < (uint32_t)(G - 1)) {   // wave-uniform
    run(IntTag<NTA>(), pg * NTA);
  } else {
    run(IntTag<NTL>(), pg * NTA);
  }
}

// ---------------------------------------------------------------------------
// host side: tile selection and launch
// ---------------------------------------------------------------------------
struct ConvTile {
  int nt;          // pixel tiles per workgroup (template instance)
  uint32_t R, TW;  // output rows / columns per workgroup
  uint64_t blocks;
};

static const int kNtVariants[] = {8, 16, 25, 29};

// staged patch rows of the instance that serves R output rows per workgroup
static int patch_rows_for(int nt, uint32_t R) {
  if (nt == 8) return kPatchRows;  // the four-wave variant has one form
  if (R > (uint32_t)kMaxR) return kPatchRowsTall;
  return nt == 16 && R <= (uint32_t)kMaxRShort ? kPatchRowsShort : kPatchRows;
}

// Picks (NT, R, TW) minimising the modelled time: a workgroup's time is proportional to NT / rate(NT) and 256 CUs
// run one workgroup each per round.  Rates measured at full tiles, relative to NT = 25 (115-120 TFLOP/s): the
// four-wave variant (NT = 8) stages the same filter chunk for a third of the pixels, 0.68; NT = 16 alone on a
// CU 0.9; NT = 29 0.95; the tall variant 0.95 of its NT's.  The short variant of NT = 16 runs two workgroups per
// CU, each at half the pace of NT = 16 at rate 1.0 (125-133 TFLOP/s at 8 x 32 tiles); a last round that leaves
// every CU one workgroup runs like NT = 16 alone.
static ConvTile choose_tile(uint32_t OH, uint32_t OW, uint64_t planes, uint32_t o_groups) {
  ConvTile best = {0, 0, 0, 0};
  double best_cost = 1e300;
  for (int nt : kNtVariants) {
    const uint32_t cap = 16u * nt;
    const uint32_t max_cols = OW < (uint32_t)kMaxTW ? OW : (uint32_t)kMaxTW;
    const uint32_t ncol0 = (OW + max_cols - 1) / max_cols;
    for (uint32_t ncol = ncol0; ncol <= OW; ++ncol) {
      const uint32_t TW = (OW + ncol - 1) / ncol;
      // the widest few column tilings, and for the 16-tile variants everything down to 24 columns (8 x 32 fills it)
      if (ncol > ncol0 + 2 && !(nt == 16 && TW >= 24u)) break;
      if (TW == 0 || TW > (uint32_t)kMaxTW || TW > cap) continue;
      uint32_t Rmax = cap / TW;
      const uint32_t max_r = nt == 8 ? (uint32_t)kMaxR : (uint32_t)kMaxRTall;  // the four-wave variant has no tall form
      if (Rmax > max_r) Rmax = max_r;
      if (Rmax > OH) Rmax = OH;
      for (uint32_t R = 1; R <= Rmax; ++R) {
        const uint64_t tiles_y = (OH + R - 1) / R;
        const uint64_t blocks = tiles_y * ncol * planes * o_groups;
        const int prows = patch_rows_for(nt, R);
        double cost;
        if (prows == kPatchRowsShort) {
          const uint64_t rest = blocks % 512;
          cost = (double)(blocks / 512) * 2.0 * nt + (rest == 0 ? 0.0 : rest <= 256 ? nt / 0.9 : 2.0 * nt);
        } else {
          const double rate = (nt == 8 ? 0.68 : nt == 16 ? 0.9 : nt == 29 ? 0.95 : 1.0) * (prows == kPatchRowsTall ? 0.95 : 1.0);
          cost = (double)((blocks + 255) / 256) * nt / rate;
        }
        cost += 1e-6 * (double)blocks * nt;  // prefers fewer, fuller workgroups when rounds tie
        if (cost < best_cost) {
          best_cost = cost;
          best.nt = nt; best.R = R; best.TW = TW; best.blocks = blocks;
        }
      }
    }
  }
  return best;
}

template <int NT, int WAVES, int PROWS>
static void launch_conv_rows(const ConvParams &P, dim3 grid, hipStream_t st) {
  if (P.w_flip)
    hipLaunchKernelGGL((conv3x3_f32_kernel<NT, WAVES, true, PROWS>), grid, dim3(64 * WAVES), 0, st, P);
  else
    hipLaunchKernelGGL((conv3x3_f32_kernel<NT, WAVES, false, PROWS>), grid, dim3(64 * WAVES), 0, st, P);
}
template <int NT, int WAVES>
static void launch_conv(const ConvParams &P, dim3 grid, hipStream_t st) {
  const int prows = patch_rows_for(NT, P.R);
  if (WAVES == 8 && prows == kPatchRowsTall) launch_conv_rows<NT, WAVES, (WAVES == 8 ? kPatchRowsTall : kPatchRows)>(P, grid, st);
  else if (NT == 16 && prows == kPatchRowsShort) launch_conv_rows<NT, WAVES, (NT == 16 ? kPatchRowsShort : kPatchRows)>(P, grid, st);
  else launch_conv_rows<NT, WAVES, kPatchRows>(P, grid, st);
}

int conv_bf16_via_f32(int which, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                      const void *const *in_tiles, const void *w, void *const *out_tiles, float beta, void *workspace,
                      size_t workspace_bytes, hipStream_t st);

// which: ADH_CONV_FWD or ADH_CONV_BWD_DATA.  H, W are the interior extents.
static int conv_direct(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                       uint32_t W, const void *const *in_tiles, const void *w, void *const *out_tiles, float beta,
                       hipStream_t st, bool rows_from_neighbours = false, bool unpadded = false,
                       const void *const *res_tiles = nullptr) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if (dtype != ADH_F32) return ADH_EUNIMPL;
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (N == 0 || Cin == 0 || Cout == 0 || H == 0 || W == 0) return ADH_OK;
  if (!in_tiles || !out_tiles || !w) return ADH_ENULL;
  if (!aligned_to(w, 4)) return ADH_EALIGN;
  const uint64_t HP = (uint64_t)H + 2, WP = (uint64_t)W + 2;
  if (HP * WP >= (1ull << 31) || (uint64_t)N * num_tiles > 65535ull) return ADH_EINVAL;
  // one image and the filter are each addressed through a 32-bit buffer resource
  const uint64_t cmax = Cin > Cout ? Cin : Cout;
  if (cmax * HP * WP * 4u >= (1ull << 31) || (uint64_t)Cin * Cout * 36u >= (1ull << 31)) return ADH_EINVAL;
  ConvParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!in_tiles[t] || !out_tiles[t]) return ADH_ENULL;
    if (!aligned_to(in_tiles[t], 4) || !aligned_to(out_tiles[t], 4)) return ADH_EALIGN;
    P.in[t] = reinterpret_cast<const float *>(in_tiles[t]);
    P.out[t] = reinterpret_cast<float *>(out_tiles[t]);
    if (res_tiles) {
      if (!res_tiles[t]) return ADH_ENULL;
      if (!aligned_to(res_tiles[t], 4)) return ADH_EALIGN;
      P.res[t] = reinterpret_cast<const float *>(res_tiles[t]);
    }
  }
  P.w = reinterpret_cast<const float *>(w);
  P.num_tiles = num_tiles;
  P.N = N;
  P.beta = res_tiles ? 1.f : beta;
  P.rows_from_neighbours = rows_from_neighbours ? 1 : 0;
  if (which == ADH_CONV_FWD) {
    P.nb_lo = 0; P.nb_hi = (int32_t)H + 1; P.nb_above = (int32_t)H; P.nb_below = 1;
  } else {
    P.nb_lo = -1; P.nb_hi = (int32_t)H; P.nb_above = (int32_t)H - 1; P.nb_below = 0;
  }
  if (which == ADH_CONV_FWD) {
    P.Cred = Cin; P.Cout = Cout;
    P.IH = (uint32_t)HP; P.IW = (uint32_t)WP; P.OH = H; P.OW = W;
    P.pad = 0;
    P.w_out_stride = Cin * 9u; P.w_red_stride = 9u; P.w_flip = 0;
  } else {
    P.Cred = Cout; P.Cout = Cin;
    P.IH = H; P.IW = W; P.OH = (uint32_t)HP; P.OW = (uint32_t)WP;
    P.pad = 2;
    P.w_out_stride = 9u; P.w_red_stride = Cin * 9u; P.w_flip = 1;
  }
  if (unpadded) {
    // neither side carries a halo: the unsplit convolution with zero padding 1, restricted to the tile; rows -1
    // and H come from the neighbouring tiles (zero columns and the tensor's own border through the range check)
    P.IH = P.OH = H; P.IW = P.OW = W;
    P.pad = 1;
    P.rows_from_neighbours = 1;
    P.nb_lo = -1; P.nb_hi = (int32_t)H; P.nb_above = (int32_t)H - 1; P.nb_below = 0;
  }
  const uint32_t o_groups = (P.Cout + 63u) / 64u;
  const ConvTile tile = choose_tile(P.OH, P.OW, (uint64_t)N * num_tiles, o_groups);
  if (tile.nt == 0) return ADH_EINVAL;
  P.R = tile.R; P.TW = tile.TW;
  P.tiles_x = (P.OW + P.TW - 1) / P.TW;
  const uint32_t tiles_y = (P.OH + P.R - 1) / P.R;
  P.div_tiles_x = FastDiv(P.tiles_x);
  P.div_TW = FastDiv(P.TW);
  dim3 grid(P.tiles_x * tiles_y, o_groups, N * num_tiles);
  switch (tile.nt) {
    case 8: launch_conv<8, 4>(P, grid, st); break;
    case 16: launch_conv<16, 8>(P, grid, st); break;
    case 25: launch_conv<25, 8>(P, grid, st); break;
    case 29: launch_conv<29, 8>(P, grid, st); break;
    default: return ADH_EINVAL;
  }
  return launch_status();
}

// name of the kernel instance conv_direct launches for a shape (fp32)
static int conv_direct_kernel_name(int which, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                                   uint32_t W, char *name, size_t name_bytes) {
  const uint32_t OH = which == ADH_CONV_FWD ? H : H + 2u, OW = which == ADH_CONV_FWD ? W : W + 2u;
  const uint32_t cout_k = which == ADH_CONV_FWD ? Cout : Cin;
  const ConvTile tile = choose_tile(OH, OW, (uint64_t)N * num_tiles, (cout_k + 63u) / 64u);
  if (tile.nt == 0) return ADH_EINVAL;
  const int waves = tile.nt == 8 ? 4 : 8;
  const int prows = patch_rows_for(tile.nt, tile.R);
  snprintf(name, name_bytes, "conv3x3_f32_kernel<%d, %d, %s, %d, 1>", tile.nt, waves, which == ADH_CONV_FWD ? "false" : "true", prows);
  return ADH_OK;
}

// The 3x3 window at stride 1 with dilation 3 over fp32 tiles padded by 3 (the convolution of the reference's
// tools/microbench_spatial_conv.cc:25-32), forward (x_pad tiles -> y tiles) and backward-data (dy tiles -> the
// whole padded dx tiles): the kernel above with its taps three rows and columns apart, 25 pixel tiles per
// workgroup over a patch of up to 20 rows.  H, W: the interior (= output) extents.  ADH_EUNIMPL (and nothing
// launched) for another dilation or dtype and for launches of fewer workgroups than CUs, which the general
// kernel spreads better.  Arguments are the caller's, already validated.
int conv3x3_dilated_try(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                        uint32_t W, uint32_t dil, const void *const *in_tiles, const void *w, void *const *out_tiles,
                        float beta, hipStream_t st) {
  constexpr uint32_t D = 3, NT = 25;
  if (dtype != ADH_F32 || dil != D) return ADH_EUNIMPL;
  const uint64_t HP = (uint64_t)H + 2u * D, WP = (uint64_t)W + 2u * D;
  const uint64_t cmax = Cin > Cout ? Cin : Cout;
  if ((uint64_t)N * num_tiles > 65535ull || cmax * HP * WP * 4u >= (1ull << 31) || (uint64_t)Cin * Cout * 36u >= (1ull << 31))
    return ADH_EUNIMPL;
  ConvParams P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    P.in[t] = reinterpret_cast<const float *>(in_tiles[t]);
    P.out[t] = reinterpret_cast<float *>(out_tiles[t]);
  }
  P.w = reinterpret_cast<const float *>(w);
  P.num_tiles = num_tiles;
  P.N = N;
  P.beta = beta;
  if (which == ADH_CONV_FWD) {
    P.Cred = Cin; P.Cout = Cout;
    P.IH = (uint32_t)HP; P.IW = (uint32_t)WP; P.OH = H; P.OW = W;
    P.pad = 0;
    P.w_out_stride = Cin * 9u; P.w_red_stride = 9u; P.w_flip = 0;
  } else {
    P.Cred = Cout; P.Cout = Cin;
    P.IH = H; P.IW = W; P.OH = (uint32_t)HP; P.OW = (uint32_t)WP;
    P.pad = 2 * (int32_t)D;
    P.w_out_stride = 9u; P.w_red_stride = Cin * 9u; P.w_flip = 1;
  }
  // R output rows x TW columns per workgroup: R + 2 D <= 20 patch rows, TW + 2 D <= 64 patch columns, R * TW <= 16 NT;
  // the fewest workgroups win (every workgroup costs the same NT tile-MFMAs per k-step), then the fewest pixels
  const uint32_t max_r = (uint32_t)kPatchRowsTall - 2u * D, max_tw = (uint32_t)kLdsPitch - 2u * D;
  uint64_t best_blocks = ~0ull;
  uint32_t best_r = 0, best_tw = 0;
  for (uint32_t R = 1; R <= max_r && R <= P.OH; ++R)
    for (uint32_t TW = 1; TW <= max_tw && TW <= P.OW && R * TW <= 16u * NT; ++TW) {
      const uint64_t blocks = (uint64_t)((P.OH + R - 1) / R) * ((P.OW + TW - 1) / TW);
      if (blocks < best_blocks || (blocks == best_blocks && R * TW < best_r * best_tw)) {
        best_blocks = blocks; best_r = R; best_tw = TW;
      }
    }
  const uint32_t o_groups = (P.Cout + 63u) / 64u;
  if (best_r == 0 || best_blocks * N * num_tiles * o_groups < 256u || best_blocks >= (1ull << 31)) return ADH_EUNIMPL;
  P.R = best_r; P.TW = best_tw;
  P.tiles_x = (P.OW + P.TW - 1) / P.TW;
  P.div_tiles_x = FastDiv(P.tiles_x);
  P.div_TW = FastDiv(P.TW);
  const dim3 grid((uint32_t)best_blocks, o_groups, N * num_tiles);
  if (P.w_flip)
    hipLaunchKernelGGL((conv3x3_f32_kernel<(int)NT, 8, true, kPatchRowsTall, (int)D>), grid, dim3(512), 0, st, P);
  else
    hipLaunchKernelGGL((conv3x3_f32_kernel<(int)NT, 8, false, kPatchRowsTall, (int)D>), grid, dim3(512), 0, st, P);
  return launch_status();
}

const char *conv_bf16_kernel_name(int which, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W, float beta);
int conv_bf16_unpadded(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                       const void *const *in_tiles, const void *w, void *const *out_tiles, float beta, void *workspace,
                       size_t workspace_bytes, hipStream_t st);

}  // namespace adh

using namespace adh;

extern "C" {

int adh_conv3x3_kernel_name(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                            uint32_t H, uint32_t W, float beta, char *name, size_t name_bytes) {
  if (!name || name_bytes == 0) return ADH_ENULL;
  if (which != ADH_CONV_FWD && which != ADH_CONV_BWD_DATA) return ADH_EINVAL;
  if (num_tiles == 0 || N == 0 || Cin == 0 || Cout == 0 || H == 0 || W == 0) return ADH_EINVAL;
  if (dtype == ADH_BF16) {
    snprintf(name, name_bytes, "%s", conv_bf16_kernel_name(which, Cin, Cout, H, W, beta));
    return ADH_OK;
  }
  if (dtype != ADH_F32) return ADH_EINVAL;
  return conv_direct_kernel_name(which, num_tiles, N, Cin, Cout, H, W, name, name_bytes);
}

int adh_conv3x3_slab_fwd_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                               uint32_t W, const void *const *x_pad_tiles, const void *w, void *const *y_tiles,
                               float beta, void *workspace, size_t workspace_bytes, void *stream) {
  if (dtype == ADH_BF16)
    return conv_bf16_via_f32(ADH_CONV_FWD, num_tiles, N, Cin, Cout, H, W, x_pad_tiles, w, y_tiles, beta, workspace,
                             workspace_bytes, as_stream(stream));
  return conv_direct(ADH_CONV_FWD, dtype, num_tiles, N, Cin, Cout, H, W, x_pad_tiles, w, y_tiles, beta,
                     as_stream(stream));
}

int adh_conv3x3_slab_fwd_tiles_unexchanged(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                           uint32_t H, uint32_t W, const void *const *x_pad_tiles, const void *w,
                                           void *const *y_tiles, float beta, void *workspace, size_t workspace_bytes,
                                           void *stream) {
  if (dtype == ADH_BF16) {
    // the bf16 kernels stream their rows from one image: exchange first, then the ordinary forward
    const int rc = adh_halo_exchange_nchw(dtype, 1, num_tiles, 1, W, H, Cin, N,
                                          const_cast<void *const *>(reinterpret_cast<const void *const *>(x_pad_tiles)),
                                          stream);
    if (rc != ADH_OK) return rc;
    return adh_conv3x3_slab_fwd_tiles(dtype, num_tiles, N, Cin, Cout, H, W, x_pad_tiles, w, y_tiles, beta, workspace,
                                      workspace_bytes, stream);
  }
  return conv_direct(ADH_CONV_FWD, dtype, num_tiles, N, Cin, Cout, H, W, x_pad_tiles, w, y_tiles, beta,
                     as_stream(stream), true);
}

int adh_conv3x3_slab_fwd(int dtype, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                         const void *x_pad, const void *w, void *y, float beta, void *workspace,
                         size_t workspace_bytes, void *stream) {
  const void *xs[1] = {x_pad};
  void *ys[1] = {y};
  return adh_conv3x3_slab_fwd_tiles(dtype, 1, N, Cin, Cout, H, W, xs, w, ys, beta, workspace, workspace_bytes, stream);
}

int adh_conv3x3_slab_bwd_data_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                    uint32_t H, uint32_t W, const void *w, const void *const *dy_tiles,
                                    void *const *dx_pad_tiles, float beta, void *workspace, size_t workspace_bytes,
                                    void *stream) {
  if (dtype == ADH_BF16)
    return conv_bf16_via_f32(ADH_CONV_BWD_DATA, num_tiles, N, Cin, Cout, H, W, dy_tiles, w, dx_pad_tiles, beta,
                             workspace, workspace_bytes, as_stream(stream));
  return conv_direct(ADH_CONV_BWD_DATA, dtype, num_tiles, N, Cin, Cout, H, W, dy_tiles, w, dx_pad_tiles, beta,
                     as_stream(stream));
}

int adh_conv3x3_slab_bwd_data_tiles_reduced(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                            uint32_t H, uint32_t W, const void *w, const void *const *dy_tiles,
                                            void *const *dx_pad_tiles, float beta, void *workspace,
                                            size_t workspace_bytes, void *stream) {
  if (dtype == ADH_BF16) {
    // the bf16 kernels stream their rows from one image: the ordinary backward-data, then the reduce
    if (beta != 0.f) return ADH_EUNIMPL;  // a reduce after accumulating would add the old halo rows again
    const int rc = adh_conv3x3_slab_bwd_data_tiles(dtype, num_tiles, N, Cin, Cout, H, W, w, dy_tiles, dx_pad_tiles, beta,
                                                   workspace, workspace_bytes, stream);
    if (rc != ADH_OK) return rc;
    return adh_halo_reduce_nchw(dtype, 1, num_tiles, 1, W, H, Cin, N, dx_pad_tiles, stream);
  }
  return conv_direct(ADH_CONV_BWD_DATA, dtype, num_tiles, N, Cin, Cout, H, W, dy_tiles, w, dx_pad_tiles, beta,
                     as_stream(stream), true);
}

int adh_conv3x3_unpadded_fwd_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                                   uint32_t W, const void *const *x_tiles, const void *w, void *const *y_tiles, float beta,
                                   void *workspace, size_t workspace_bytes, void *stream) {
  if (dtype == ADH_F32)
    return conv_direct(ADH_CONV_FWD, dtype, num_tiles, N, Cin, Cout, H, W, x_tiles, w, y_tiles, beta, as_stream(stream),
                       true, true);
  return conv_bf16_unpadded(ADH_CONV_FWD, dtype, num_tiles, N, Cin, Cout, H, W, x_tiles, w, y_tiles, beta, workspace,
                            workspace_bytes, as_stream(stream));
}

int adh_conv3x3_unpadded_fwd_residual_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                                            uint32_t W, const void *const *x_tiles, const void *w,
                                            const void *const *res_tiles, void *const *y_tiles, void *stream) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if (dtype != ADH_F32) return ADH_EUNIMPL;
  if (!res_tiles) return ADH_ENULL;
  return conv_direct(ADH_CONV_FWD, dtype, num_tiles, N, Cin, Cout, H, W, x_tiles, w, y_tiles, 1.f, as_stream(stream), true,
                     true, res_tiles);
}

int adh_conv3x3_unpadded_bwd_data_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                                        uint32_t W, const void *w, const void *const *dy_tiles, void *const *dx_tiles,
                                        float beta, void *workspace, size_t workspace_bytes, void *stream) {
  if (dtype == ADH_F32)
    return conv_direct(ADH_CONV_BWD_DATA, dtype, num_tiles, N, Cin, Cout, H, W, dy_tiles, w, dx_tiles, beta,
                       as_stream(stream), true, true);
  return conv_bf16_unpadded(ADH_CONV_BWD_DATA, dtype, num_tiles, N, Cin, Cout, H, W, dy_tiles, w, dx_tiles, beta, workspace,
                            workspace_bytes, as_stream(stream));
}

int adh_conv3x3_slab_bwd_data(int dtype, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                              const void *w, const void *dy, void *dx_pad, float beta, void *workspace,
                              size_t workspace_bytes, void *stream) {
  const void *dys[1] = {dy};
  void *dxs[1] = {dx_pad};
  return adh_conv3x3_slab_bwd_data_tiles(dtype, 1, N, Cin, Cout, H, W, w, dys, dxs, beta, workspace, workspace_bytes,
                                         stream);
}

}  // extern "C"
