// 3x3 slab convolution on the bf16 matrix cores (v_mfma_f32_16x16x32_bf16), forward and backward-data,
// for reductions of MORE than 64 channels: 128 reduction channels per pass with the sums in registers, where
// the eight-wave kernel of conv3x3_bf16_w8.hip takes one pass per 64 and hands fp32 sums through memory.
//
// What the 64-channel kernel keeps in registers is a wave's filter share, 9 taps x 64 reduction channels x 32
// output channels = 144 registers; twice the reduction does not fit.  Here a wave owns HALF the output channels
// and TWICE the reduction, 9 x 128 x 16 in the same 144 registers, and the eight waves of a workgroup are eight
// tiles of 16 output channels: a workgroup produces 128 output channels of a strip, so that the input rows it
// stages (and transposes, the expensive part) serve twice the matrix work.  Per step, four output rows of a
// 32-column strip:
//   * every wave multiplies all four rows x both 16-column tiles for its 16 output channels: 8 accumulator
//     tiles, 144 operand reads (6 input rows x 3 column shifts x 4 blocks of 32 channels x 2 column tiles) and
//     288 MFMAs: half an operand read per MFMA against a third in the 64-channel kernel, while everything else
//     a step does (copies, transposition, ring writes, stores, the barrier) is spread over twice the MFMAs;
//   * input rows arrive by `buffer_load ... lds` in memory order [channel][pixel] into a staging area of the
//     wave's own: 16 channels x 4 rows x 5 granules of 8 pixels (6 over tiles without halo) are exactly 5 (6)
//     copies of 64 lanes x 16 bytes; rows, channels and granules that do not exist carry an out-of-range offset
//     and arrive as zeros;
//   * the wave turns its staging area into the ring's [pixel][channel] order with the transposing LDS read
//     (ds_read_b64_tr_b16), two reads and one 16-byte ring write per 16 pixels x 8 channels and lane group.
//     The ring holds ten rows of 34 pixels (32 output columns and the window's two more) at a pixel pitch of
//     288 bytes (128 channels + 32 bytes: measured, 16-byte operand reads of 16 neighbouring pixels run at the
//     linear rate of 4.5 cycles per wave instruction at pitches of 160 and 288 bytes and conflict two-way at
//     272, 304 and 320); staged pixels outside those 34 are written to a dummy kilobyte;
//   * one barrier per step, LDS only, after a wave's last ring access of the step.
// More than 128 reduction channels: one pass per 128 with fp32 sums between them (a quarter of the traffic of
// passes of 64), a remainder of at most 64 channels by the 64-channel kernel, which shares the layout of the sums.
// Work items, the row-group sequence across items, the filter layouts and the output path (a swap between lane
// rows turns the MFMA's 4 + 4 columns per lane into 8 neighbouring ones) are those of the 64-channel kernel.
#include "conv3x3_bf16_mfma.h"

namespace adh {

constexpr int kK2Threads = 512;
constexpr int kK2StripCols = 32;
constexpr int kK2PxBytes = 288;
constexpr int kK2RowPx = 34;
constexpr int kK2RowBytes = kK2RowPx * kK2PxBytes;       // 9792
constexpr int kK2RingRows = 10;                           // 6 rows in use + 4 rows being written
constexpr int kK2RingBytes = kK2RingRows * kK2RowBytes;   // 97920

typedef short s16x4 __attribute__((ext_vector_type(4)));
#define ADH_LDS __attribute__((address_space(3)))

static __device__ __forceinline__ u32x2 k2_read_tr(const uint8_t *p) {
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((ADH_LDS s16x4 *)p));
}
static __device__ __forceinline__ uint32_t k2_wrap(uint32_t s) { return s >= (uint32_t)kK2RingRows ? s - (uint32_t)kK2RingRows : s; }

// BETA: the old output is added (in the first pass).  PIN: the sums of the passes before this one are read from
// P.part and added.  POUT: the sums go to P.part as fp32 instead of to the output as bf16 (a later pass follows).
// HF (P.pad == 1): neither the input nor the output carries a halo; rows -1 and IH come from the neighbouring
// tiles (P.neighbour_rows), and a row is staged from eight columns left of the strip in six granules.
template <bool BETA, bool PIN, bool POUT, bool HF>
__global__ __launch_bounds__(kK2Threads, 1) void conv3x3_bf16_k128_kernel(ConvBf16Params P) {
  static_assert(!(BETA && PIN), "the old output is added in the first pass, which reads no sums");
  constexpr int G = HF ? 6 : 5;                 // granules of a staged row = copies per row group
  constexpr int kRawWave = G * 1024;
  constexpr int kChanBytes = G * 16;            // a channel row in the staging area
  constexpr int kRowStage = 16 * kChanBytes;    // 16 channels of one row
  __shared__ __attribute__((aligned(16))) uint8_t raw[8 * kRawWave];
  __shared__ __attribute__((aligned(16))) uint8_t ring[kK2RingBytes];
  __shared__ __attribute__((aligned(16))) uint8_t dummy[1024];

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wv = __builtin_amdgcn_readfirstlane(tid >> 6);  // tile of 16 output channels
  const uint32_t grp = blockIdx.y;                               // group of 128 output channels

  uint32_t vblock = blockIdx.x;
  if ((gridDim.x & 7u) == 0u) vblock = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const uint32_t total = P.whole_items + P.pieces;
  if (vblock >= total) return;

  // this wave's filter share in B-operand order: lane (n = l16: output channel, k-block = g: 8 reduction channels)
  // of block kb of 32 reduction channels
  const uint32_t co0 = grp * 128u + 16u * wv + l16;
  u32x4 wreg[9][4];
  if (P.w_direct) {
    // straight from the filter as the caller holds it (forward, (Cout, Cin, 3, 3), Cin a multiple of 64, 16-byte
    // aligned): eight reduction channels x nine taps of one output channel are 72 consecutive elements
    const __amdgpu_buffer_rsrc_t rsrcW = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(P.w_direct), 0, (int)(P.Cout * P.Cred * 18u), 0x00020000);
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const uint32_t ci = P.chan0 + 32u * kb + 8u * g;
      const uint32_t off = (co0 < P.Cout && ci < P.Cred) ? (co0 * P.Cred + ci) * 18u : kOutOfRange;
      uint32_t d[36];
#pragma unroll
      for (int q = 0; q < 9; ++q) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrcW, off, 16 * q, 0);
        d[4 * q + 0] = v[0]; d[4 * q + 1] = v[1]; d[4 * q + 2] = v[2]; d[4 * q + 3] = v[3];
      }
#pragma unroll
      for (int tap = 0; tap < 9; ++tap) {
        u32x4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int klo = 18 * j + tap, khi = klo + 9;
          const uint32_t sel = ((khi & 1) ? 0x07060000u : 0x05040000u) | ((klo & 1) ? 0x00000302u : 0x00000100u);
          r[j] = __builtin_amdgcn_perm(d[khi >> 1], d[klo >> 1], sel);
        }
        wreg[tap][kb] = r;
      }
    }
  } else {
    // the transformed copy, [group of 64 outputs][pass of 64][tap][half][64 out][32 red]: this pass is the two
    // passes of 64 from P.pass on; a group of 64 outputs past the last one holds nothing
    const uint32_t grp64 = grp * 2u + (wv >> 2), o64 = 16u * (wv & 3u) + l16;
    const bool have = grp64 * 64u < P.Cout;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const uint32_t pass64 = P.pass + (uint32_t)(kb >> 1);
      const u32x4 *wt = reinterpret_cast<const u32x4 *>(P.wt + ((size_t)grp64 * P.passes + pass64) * kWtGroupElems);
#pragma unroll
      for (int tap = 0; tap < 9; ++tap)
        wreg[tap][kb] = (have && pass64 < P.passes) ? wt[((tap * 2 + (kb & 1)) * 64 + (int)o64) * 4 + (int)g] : (u32x4){0u, 0u, 0u, 0u};
    }
  }

  const uint32_t plane_bytes = P.IH * P.IW * 2u;
  const uint32_t image_bytes = P.Cred * plane_bytes;
  // staged pixel of the strip's first output column at tap column 0: the staged row starts eight columns left of
  // the strip whenever the input has no halo of its own (pad 1: unpadded in and out; pad 2: backward-data into a
  // padded slab); the ring holds staged pixels xoff .. xoff + 33 as its pixels 0 .. 33
  const int32_t xoff = P.pad ? 8 - P.pad : 0;
  const int32_t col_back = P.pad ? 8 : 0;

  // ---- requests: copy q of a group moves staging slots 64 q + lane; slot = (row * 16 + channel) * G + granule
  uint32_t ld_off[6];  // G of them are used
  uint32_t ld_rows = 0;  // 3 bits per copy: row of the group, bit 2 = the slot's channel exists
  uint32_t ld_gran = 0;  // 3 bits per copy: granule
#pragma unroll
  for (int q = 0; q < G; ++q) {
    const uint32_t slot = 64u * q + lane;
    const uint32_t row = slot / (16u * G), rem = slot - row * (16u * G), ch = rem / (uint32_t)G, gran = rem - ch * (uint32_t)G;
    const uint32_t chan = 16u * wv + ch;
    const bool ok = chan < P.cred_pass;
    ld_off[q] = (P.chan0 + chan) * plane_bytes + row * P.IW * 2u + gran * 16u;
    ld_rows |= ((row & 3u) | (ok ? 4u : 0u)) << (3 * q);
    ld_gran |= gran << (3 * q);
  }
  uint8_t *const raw_wave = raw + wv * kRawWave;

  // ---- turning the staging area into ring order.  A unit is 16 pixels x 8 channels of one row: inside a group of
  // 16 lanes, source lane 4 e + q reads channel e (second read: e + 4) at pixels 4 q .. 4 q + 3 of the block, and
  // lane i receives pixel i's four channels.  Lane group g takes channel half g & 1 of the wave's 16.
  //   padded (G = 5): rounds 0-3 handle row t, pixel block g >> 1; round 4 the eight-pixel tails (pixels 32-39) of
  //     rows 2 (g >> 1) and 2 (g >> 1) + 1: source lanes q < 2 read the first row, q >= 2 the second, so lanes
  //     0-7 receive the first row's pixels 32 + i and lanes 8-15 the second row's pixels 32 + i - 8
  //   no halo (G = 6): round t handles row 2 (t / 3) + (g >> 1), pixel block t % 3
  const uint32_t chb = 8u * (g & 1u);
  const uint32_t tr_lane = (chb + (l16 >> 2)) * kChanBytes + (l16 & 3u) * 8u;
  const uint8_t *const trA = raw_wave + tr_lane + (g >> 1) * (HF ? (uint32_t)kRowStage : 32u);
  const uint8_t *const tr4 = raw_wave + (2u * (g >> 1) + ((l16 & 3u) >> 1)) * kRowStage + (chb + (l16 >> 2)) * kChanBytes +
                             64u + (l16 & 1u) * 8u;
  const uint32_t wr_chan = 32u * wv + 2u * chb;  // byte offset of the unit's eight channels inside a ring pixel
  uint8_t *const wr_dummy = dummy + lane * 16u;

  uint32_t tb = 0;  // ring slot the next transposed group starts at
  struct TrPair { u32x2 lo, hi; };
  auto tr_read = [&](auto tag, TrPair &T) {
    constexpr int t = decltype(tag)::value;
    const uint8_t *src;
    if constexpr (HF) src = trA + (t / 3) * 2 * kRowStage + (t % 3) * 32;
    else if constexpr (t < 4) src = trA + t * kRowStage;
    else src = tr4;
    T.lo = k2_read_tr(src);
    T.hi = k2_read_tr(src + 4 * kChanBytes);
  };
  auto tr_write = [&](auto tag, const TrPair &T) {
    constexpr int t = decltype(tag)::value;
    const u32x4 v = {T.lo[0], T.lo[1], T.hi[0], T.hi[1]};
    int32_t px;
    uint32_t row;
    if constexpr (HF) {
      px = (t % 3) * 16 + (int32_t)l16 - xoff;
      row = 2u * (t / 3) + (g >> 1);
    } else if constexpr (t < 4) {
      px = (int32_t)((g >> 1) * 16u + l16) - xoff;
      row = (uint32_t)t;
    } else {
      px = 32 + (int32_t)(l16 & 7u) - xoff;
      row = 2u * (g >> 1) + (l16 >> 3);
    }
    uint8_t *const dst = ring + k2_wrap(tb + row) * kK2RowBytes + (uint32_t)px * kK2PxBytes + wr_chan;
    *reinterpret_cast<u32x4 *>((px >= 0 && px < kK2RowPx) ? dst : wr_dummy) = v;
  };

  // ---- the loader's place in the sequence of row groups: work item, group -1 .. steps - 1
  // (group k holds the item's ring-relative rows 4 k + 2 .. 4 k + 5; rows -2, -1 are never used)
  uint32_t workL = vblock;
  int32_t grpL = -1, stepsL = 0;
  int32_t arow0L = 0, colL = 0;  // input row of ring-relative row 0, input column of staged pixel 0
  uint32_t okL = 0;              // bit q: copy q of this lane exists for this item (channel, granule column)
  __amdgpu_buffer_rsrc_t rsrcL = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(P.in[0]), 0, 0, 0x00020000);
  __amdgpu_buffer_rsrc_t rsrcUp = rsrcL, rsrcDn = rsrcL;
  bool hasUpL = false, hasDnL = false;

  auto decode = [&](uint32_t work, uint32_t &tile, uint32_t &n, uint32_t &c0, uint32_t &r_begin, uint32_t &r_end) {
    uint32_t item, seg = 0, seg_steps = P.steps_per_item;
    if (work < P.whole_items) {
      item = work;
    } else {
      uint32_t it;
      P.div_rest.divmod(work - P.whole_items, seg, it);
      item = P.whole_items + it;
      seg_steps = P.seg_steps;
    }
    uint32_t strip, plane;
    P.div_strips.divmod(item, plane, strip);
    P.div_N.divmod(plane, tile, n);
    c0 = strip * kK2StripCols;
    r_begin = seg * seg_steps * kStepRows;
    r_end = min(P.OH, r_begin + seg_steps * kStepRows);
  };

  auto loader_open = [&]() {
    uint32_t tile, n, c0, r_begin, r_end;
    decode(workL, tile, n, c0, r_begin, r_end);
    stepsL = (int32_t)((r_end - r_begin + kStepRows - 1) / kStepRows);
    arow0L = (int32_t)r_begin - P.pad;
    colL = (int32_t)c0 - col_back;
    const size_t img_off = (size_t)n * P.Cred * P.IH * P.IW;
    rsrcL = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(P.in[tile] + img_off), 0, image_bytes, 0x00020000);
    if (P.neighbour_rows) {
      hasUpL = tile > 0u;
      hasDnL = tile + 1u < P.num_tiles;
      rsrcUp = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(P.in[hasUpL ? tile - 1u : tile] + img_off), 0,
                                                 image_bytes, 0x00020000);
      rsrcDn = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(P.in[hasDnL ? tile + 1u : tile] + img_off), 0,
                                                 image_bytes, 0x00020000);
    }
    okL = 0;
#pragma unroll
    for (int q = 0; q < G; ++q) {
      const int32_t col = colL + 8 * (int32_t)((ld_gran >> (3 * q)) & 7u);
      const bool ok = ((ld_rows >> (3 * q)) & 4u) && col >= 0 && col < (int32_t)P.IW;
      okL |= (ok ? 1u : 0u) << q;
    }
    grpL = -1;
  };
  // Copy q of the loader's current group.  Once all work has been requested okL is zero and the copies only write
  // zeros, which go to ring rows nobody reads: the sequence needs no branches.  NBR: the group holds a row that
  // comes from a neighbouring tile; the lanes of that row take an instruction of their own with the neighbour's
  // buffer (lanes that are switched off write nothing to LDS).
  auto request = [&](auto tag, auto nbr_tag) {
    constexpr int q = decltype(tag)::value;
    constexpr bool NBR = decltype(nbr_tag)::value != 0;
    const int32_t first = arow0L + 4 * grpL + 2;
    const int32_t base = (first * (int32_t)P.IW + colL) * 2;
    const int32_t arow = first + (int32_t)((ld_rows >> (3 * q)) & 3u);
    const bool ok = ((okL >> q) & 1u) && (uint32_t)arow < P.IH;
    const uint32_t v = ok ? ld_off[q] + (uint32_t)base : kOutOfRange;
    if constexpr (!NBR) {
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcL, (ADH_LDS void *)(raw_wave + q * 1024), 16, v, 0, 0, 0);
    } else {
      const bool slot = ((okL >> q) & 1u) != 0u;
      const bool up = slot && hasUpL && arow == -1, dn = slot && hasDnL && arow == (int32_t)P.IH;
      if (up) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcUp, (ADH_LDS void *)(raw_wave + q * 1024), 16,
                                                 ld_off[q] + (uint32_t)base + plane_bytes, 0, 0, 0);
      } else if (dn) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcDn, (ADH_LDS void *)(raw_wave + q * 1024), 16,
                                                 ld_off[q] + (uint32_t)base - plane_bytes, 0, 0, 0);
      } else {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcL, (ADH_LDS void *)(raw_wave + q * 1024), 16, v, 0, 0, 0);
      }
    }
  };
  auto group_has_neighbour_row = [&]() -> bool {
    if (!P.neighbour_rows || workL >= total) return false;
    const int32_t first = arow0L + 4 * grpL + 2;
    return (hasUpL && first <= -1 && -1 <= first + 3) || (hasDnL && first <= (int32_t)P.IH && (int32_t)P.IH <= first + 3);
  };
  auto loader_advance = [&]() {
    if (workL >= total) return;
    if (++grpL == stepsL) {
      workL += gridDim.x;
      if (workL < total)
        loader_open();
      else
        okL = 0;
    }
  };

  // ---- the multiplying side's place: work item and step
  uint32_t workC = vblock;
  int32_t stepC = -2, stepsC;
  uint32_t c0C, r_beginC, r_endC;
  // after the swap between lane rows a lane holds eight neighbouring columns of its output channel
  const uint32_t ocol_lane = ((g & 1u) ? 16u : 0u) + (g >> 1) * 8u;  // + first column of the strip
  const bool okc = co0 < P.Cout;
  const uint32_t out_image_bytes = P.Cout * P.OH * P.OW * 2u;
  const uint32_t orow_bytes = P.OW * 2u;
  const uint32_t ooff_lane = (co0 * P.OH * P.OW + ocol_lane) * 2u;  // + (row * OW + first column) * 2
  uint16_t *out_imgC = nullptr;
  __amdgpu_buffer_rsrc_t rsrcC = __builtin_amdgcn_make_buffer_rsrc(P.out[0], 0, 0, 0x00020000);
  // the fp32 sums between passes: the lane's own four columns of accumulator [row][column tile] at
  // (co0, row, c0 + 16 cti + 4 g): 16 bytes per lane, 64 per output channel and lane row
  constexpr bool PART = PIN || POUT;
  const uint32_t poff_lane = (co0 * P.OH * P.OW + 4u * g) * 4u;  // + (row * OW + first column) * 4
  const uint32_t prow_bytes = 2u * orow_bytes;
  float *part_imgC = nullptr;
  __amdgpu_buffer_rsrc_t rsrcP = __builtin_amdgcn_make_buffer_rsrc(P.out[0], 0, 0, 0x00020000);
  bool wholeC = false;  // every lane of the wave stores eight whole columns of an existing channel
  auto compute_open = [&]() {
    uint32_t tile, n;
    decode(workC, tile, n, c0C, r_beginC, r_endC);
    stepsC = (int32_t)((r_endC - r_beginC + kStepRows - 1) / kStepRows);
    out_imgC = P.out[tile] + (size_t)n * P.Cout * P.OH * P.OW;
    rsrcC = __builtin_amdgcn_make_buffer_rsrc(out_imgC, 0, out_image_bytes, 0x00020000);
    if constexpr (PART) {
      part_imgC = P.part[tile] + (size_t)n * P.Cout * P.OH * P.OW;
      rsrcP = __builtin_amdgcn_make_buffer_rsrc(part_imgC, 0, 2u * out_image_bytes, 0x00020000);
    }
    wholeC = __builtin_amdgcn_ballot_w64(!(c0C + ocol_lane + 7u < P.OW && okc)) == 0ull;
  };
  compute_open();

  // operand reads: ring pixel (16 cti + l16 + kw) of a row, channels 32 kb + 8 g .. + 7
  const uint32_t read_lane = l16 * kK2PxBytes + g * 16u;

  // one output row of the step, lane by lane: edge strips and channel remainders
  auto store_guarded = [&](const u32x4 &pk, uint32_t row) {
    const uint32_t ocol = c0C + ocol_lane;
    if (!okc) return;
    uint16_t *p = out_imgC + ((size_t)co0 * P.OH + row) * P.OW + ocol;
    if (ocol + 7u < P.OW) {
      *reinterpret_cast<u32x4_unaligned *>(p) = pk;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (ocol + e < P.OW) p[e] = (uint16_t)(pk[e >> 1] >> ((e & 1) * 16));
    }
  };
  auto load_old_guarded = [&](uint32_t row) -> u32x4 {
    const uint32_t ocol = c0C + ocol_lane;
    u32x4 o = {0u, 0u, 0u, 0u};
    if (okc) {
      const uint16_t *p = out_imgC + ((size_t)co0 * P.OH + row) * P.OW + ocol;
      if (ocol + 7u < P.OW) {
        o = *reinterpret_cast<const u32x4_unaligned *>(p);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (ocol + e < P.OW) o[e >> 1] |= (uint32_t)p[e] << ((e & 1) * 16);
      }
    }
    return o;
  };
  // the fp32 sums of one output row, element by element: stored, or added to the accumulators
  auto part_guarded = [&](floatx4 (&a)[2], uint32_t row, bool store) {
    if (!okc) return;
#pragma unroll
    for (int cti = 0; cti < 2; ++cti) {
      const uint32_t col = c0C + 16u * cti + 4u * g;
      float *p = part_imgC + ((size_t)co0 * P.OH + row) * P.OW + col;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (col + e < P.OW) {
          if (store)
            p[e] = a[cti][e];
          else
            a[cti][e] += p[e];
        }
    }
  };

  // The matrix part of a step: 144 operand reads, each fetched kAhead reads before its MFMAs.  Rounds 0-47 read
  // input rows 0 and 1 in turn (one and two MFMAs), rounds 48-71 row 2, rounds 72-95 row 3 (three each), rounds
  // 96-143 rows 4 and 5 in turn (two and one): output row 0 is complete after round 71, row 1 after round 95.
  // With SIDE everything else a wave does in a phase is dealt out between the rounds one instruction at a time.
  auto compute = [&](uint32_t sb, auto side_tag, auto nbr_tag, uint32_t row0, uint32_t nrows, bool after_plain) {
    constexpr bool SIDE = decltype(side_tag)::value != 0;
    const uint32_t cur_off = ooff_lane + (row0 * P.OW + c0C) * 2u;
    const uint32_t pcur = poff_lane + (row0 * P.OW + c0C) * 4u;
    uint32_t off[4], poff[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      off[r] = nrows > (uint32_t)r ? cur_off + (uint32_t)r * orow_bytes : kOutOfRange;
      poff[r] = nrows > (uint32_t)r ? pcur + (uint32_t)r * prow_bytes : kOutOfRange;
    }
    floatx4 acc[4][2];  // [row][column tile]
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int cti = 0; cti < 2; ++cti) acc[r][cti] = (floatx4){0.f, 0.f, 0.f, 0.f};
    floatx4 pin[2][2];  // [row & 1][column tile]: the earlier passes' sums
    u32x4 old[2];       // [row & 1]: old output values for beta = 1
    constexpr int kReads = 144, kAhead = (BETA || PIN) ? 3 : 4;
    const uint8_t *row_ptr[6];
#pragma unroll
    for (int ir = 0; ir < 6; ++ir) row_ptr[ir] = ring + k2_wrap(sb + (uint32_t)ir) * kK2RowBytes + read_lane;
    u32x4 abuf[kAhead + 1];
    TrPair trp[2];
    auto fetch = [&](int t) {
      const int ir = t < 48 ? (t & 1) : t < 72 ? 2 : t < 96 ? 3 : 4 + (t & 1);
      const int j = t < 48 ? t >> 1 : t < 72 ? t - 48 : t < 96 ? t - 72 : (t - 96) >> 1;
      const int kw = j >> 3, kb = (j >> 1) & 3, cti = j & 1;
      abuf[t % (kAhead + 1)] = *reinterpret_cast<const u32x4 *>(row_ptr[ir] + (cti * 16 + kw) * kK2PxBytes + kb * 64);
    };
#pragma unroll
    for (int t = 0; t < kAhead; ++t) fetch(t);
    __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
    // The copies of the group to transpose have landed: everything but the previous step's stores, which were
    // issued after them (memory instructions of a wave complete in order).  After a phase without MFMAs nothing
    // was issued after the copies, and the wait is for all of them.
    if (SIDE) {
      if (after_plain)
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      else
        __builtin_amdgcn_s_waitcnt(POUT ? 0x0F78 : 0x0F74);  // vmcnt(8) : vmcnt(4)
    }
    // packs output row r back to store order through the swap between lane rows and stores it
    auto pack_row = [&](auto tag) {
      constexpr int r = decltype(tag)::value;
      floatx4 v0 = acc[r][0], v1 = acc[r][1];
      if constexpr (BETA) {
        u32x4 o;
        if constexpr (SIDE) o = old[r & 1];
        else o = load_old_guarded(row0 + r);
        const u32x2 s0 = __builtin_amdgcn_permlane16_swap(o[0], o[2], false, false);
        const u32x2 s1 = __builtin_amdgcn_permlane16_swap(o[1], o[3], false, false);
        v0[0] += __uint_as_float(s0[0] << 16);
        v0[1] += __uint_as_float(s0[0] & 0xffff0000u);
        v0[2] += __uint_as_float(s1[0] << 16);
        v0[3] += __uint_as_float(s1[0] & 0xffff0000u);
        v1[0] += __uint_as_float(s0[1] << 16);
        v1[1] += __uint_as_float(s0[1] & 0xffff0000u);
        v1[2] += __uint_as_float(s1[1] << 16);
        v1[3] += __uint_as_float(s1[1] & 0xffff0000u);
      }
      if constexpr (PIN) {
        if constexpr (SIDE) {
          v0 += pin[r & 1][0];
          v1 += pin[r & 1][1];
        } else {
          floatx4 a[2] = {v0, v1};
          if ((uint32_t)r < nrows) part_guarded(a, row0 + r, false);
          v0 = a[0];
          v1 = a[1];
        }
      }
      if constexpr (POUT) {
        if constexpr (SIDE) {
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v0), rsrcP, poff[r], 0, 0);
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v1), rsrcP, poff[r] + 64u, 0, 0);
        } else {
          floatx4 a[2] = {v0, v1};
          if ((uint32_t)r < nrows) part_guarded(a, row0 + r, true);
        }
        return;
      }
      const u32x2 q0 = __builtin_amdgcn_permlane16_swap(pack_bf16x2(v0[0], v0[1]), pack_bf16x2(v1[0], v1[1]), false, false);
      const u32x2 q1 = __builtin_amdgcn_permlane16_swap(pack_bf16x2(v0[2], v0[3]), pack_bf16x2(v1[2], v1[3]), false, false);
      const u32x4 pk = {q0[0], q1[0], q0[1], q1[1]};
      if constexpr (SIDE) {
        __builtin_amdgcn_raw_buffer_store_b128(pk, rsrcC, off[r], 0, 0);
      } else {
        if ((uint32_t)r < nrows) store_guarded(pk, row0 + r);
      }
    };
    auto round = [&](auto tag) {
      constexpr int t = decltype(tag)::value;
      if constexpr (t + kAhead < kReads) {
        fetch(t + kAhead);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      constexpr int ir = t < 48 ? (t & 1) : t < 72 ? 2 : t < 96 ? 3 : 4 + (t & 1);
      constexpr int j = t < 48 ? t >> 1 : t < 72 ? t - 48 : t < 96 ? t - 72 : (t - 96) >> 1;
      constexpr int kw = j >> 3, kb = (j >> 1) & 3, cti = j & 1;
      const bf16x8 a = __builtin_bit_cast(bf16x8, abuf[t % (kAhead + 1)]);
      constexpr int kh_lo = ir - 3 > 0 ? ir - 3 : 0;
      constexpr int kh_hi = ir < 2 ? ir : 2;
#pragma unroll
      for (int kh = kh_lo; kh <= kh_hi; ++kh)
        acc[ir - kh][cti] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, wreg[kh * 3 + kw][kb]),
                                                                    acc[ir - kh][cti], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, kh_hi - kh_lo + 1, 0);
      if constexpr (SIDE) {
        // rounds 0, 4, .. : transposing read pair t / 4; rounds 3, 7, .. : ring write (t - 3) / 4
        if constexpr (t % 4 == 0 && t / 4 < G) {
          tr_read(IntTag<t / 4>(), trp[(t / 4) % 2]);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        if constexpr (t % 4 == 3 && t / 4 < G) {
          tr_write(IntTag<t / 4>(), trp[(t / 4) % 2]);
          __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
        // rounds 26, 29, .. : copy of the next row group (every transposing read has returned)
        if constexpr (t >= 26 && (t - 26) % 3 == 0 && (t - 26) / 3 < G) {
          request(IntTag<(t - 26) / 3>(), nbr_tag);
          if constexpr (!decltype(nbr_tag)::value) __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
        // old values (beta = 1) and the earlier passes' sums: rows 0 and 1 before their packing, rows 2 and 3 once
        // the registers of rows 0 and 1 are free again
        if constexpr (BETA && (t == 50 || t == 58 || t == 114 || t == 122)) {
          constexpr int r = t == 50 ? 0 : t == 58 ? 1 : t == 114 ? 2 : 3;
          old[r & 1] = __builtin_amdgcn_raw_buffer_load_b128(rsrcC, off[r], 0, 0);
          __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
        if constexpr (PIN && (t == 50 || t == 54 || t == 58 || t == 62 || t == 114 || t == 118 || t == 122 || t == 126)) {
          constexpr int i = t < 100 ? (t - 50) / 4 : 4 + (t - 114) / 4, r = i >> 1, cti2 = i & 1;
          pin[r & 1][cti2] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsrcP, poff[r] + 64u * cti2, 0, 0));
          __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
        // output rows 0 and 1 are packed and stored while rows 2 and 3 are still being multiplied
        if constexpr (t == 80 || t == 106) {
          pack_row(IntTag<t == 80 ? 0 : 1>());
          __builtin_amdgcn_sched_group_barrier(0x010, POUT ? 2 : 1, 0);
        }
      }
    };
    for_each_int(std::make_integer_sequence<int, kReads>(), round);
    __builtin_amdgcn_sched_barrier(0);
    // every ring read and write of the phase is done (the operands have been multiplied)
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!SIDE) {
      for_each_int(std::make_integer_sequence<int, 4>(), pack_row);
    } else {
      pack_row(IntTag<2>());
      pack_row(IntTag<3>());
    }
  };

  // the same side work in one piece, for the phases that cannot take the interleaved form
  auto move_rows_plain = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    TrPair T[6];
    for_each_int(std::make_integer_sequence<int, G>(), [&](auto tag) { tr_read(tag, T[decltype(tag)::value]); });
    for_each_int(std::make_integer_sequence<int, G>(), [&](auto tag) { tr_write(tag, T[decltype(tag)::value]); });
    for_each_int(std::make_integer_sequence<int, G>(), [&](auto tag) { request(tag, IntTag<HF ? 1 : 0>()); });
  };

  // One phase per step, plus one without MFMAs at the start of every item and a second one at the very start.  In
  // phase f a wave transposes row group f + 1 (requested in phase f - 1) into the four ring slots that the step's
  // six input rows leave free, requests group f + 2 and multiplies step f; the phase's barrier publishes the ring
  // rows written in it and frees the ones read in it.
  uint32_t sb = 4;  // ring slot of the first input row of the step multiplied in this phase
  loader_open();
  for_each_int(std::make_integer_sequence<int, G>(), [&](auto tag) { request(tag, IntTag<HF ? 1 : 0>()); });
  loader_advance();
  auto phase_barrier = [&]() {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): LDS only
    __builtin_amdgcn_s_barrier();
  };
  bool after_plain = true;  // the last phase issued its copies last: no stores after them
  for (;;) {
    if (stepC >= 0) {
      const uint32_t row0 = r_beginC + (uint32_t)stepC * kStepRows;
      const uint32_t nrows = min(4u, r_endC - row0);
      if (wholeC) {
        bool nbr = false;
        if constexpr (HF) nbr = group_has_neighbour_row();
        if constexpr (HF) {
          if (nbr) compute(sb, IntTag<1>(), IntTag<1>(), row0, nrows, after_plain);
          else compute(sb, IntTag<1>(), IntTag<0>(), row0, nrows, after_plain);
        } else {
          compute(sb, IntTag<1>(), IntTag<0>(), row0, nrows, after_plain);
        }
        after_plain = false;
      } else {
        move_rows_plain();
        compute(sb, IntTag<0>(), IntTag<0>(), row0, nrows, false);
        after_plain = true;  // its stores are conditional: count on none
      }
    } else {
      move_rows_plain();
      phase_barrier();
      after_plain = true;
    }
    loader_advance();
    sb = k2_wrap(sb + kStepRows);
    tb = k2_wrap(tb + kStepRows);
    if (++stepC == stepsC) {
      workC += gridDim.x;
      if (workC >= total) break;
      compute_open();
      stepC = -1;
    }
  }
}

// Shapes: those of the eight-wave 64-channel kernel (rows on a 4-byte boundary, on 16 bytes where the input has no
// halo of its own; byte offsets inside the buffer range check's 31 bits), more than 64 reduction and output channels.
bool conv_bf16_k128_takes(const ConvBf16Params &P, uint32_t num_tiles) {
  if (P.Cred <= 64u || P.Cout <= 64u) return false;
  return conv_bf16_w8_takes(P, num_tiles);
}

// launches the pass of 128 reduction channels from P.chan0 on
int conv_bf16_k128_launch(const ConvBf16Params &P, uint32_t gx, uint32_t groups128, hipStream_t st) {
  const dim3 grid(gx, groups128), block(kK2Threads);
  const bool first = P.first_pass != 0u, last = P.last_pass != 0u, beta = P.beta != 0.f;
#define ADH_K128(B, PI, PO)                                                                                       \
  do {                                                                                                            \
    if (P.pad == 1)                                                                                               \
      hipLaunchKernelGGL((conv3x3_bf16_k128_kernel<B, PI, PO, true>), grid, block, 0, st, P);                     \
    else                                                                                                          \
      hipLaunchKernelGGL((conv3x3_bf16_k128_kernel<B, PI, PO, false>), grid, block, 0, st, P);                    \
  } while (0)
  if (first && last) {
    if (beta) ADH_K128(true, false, false); else ADH_K128(false, false, false);
  } else if (first) {
    if (beta) ADH_K128(true, false, true); else ADH_K128(false, false, true);
  } else if (!last) {
    ADH_K128(false, true, true);
  } else {
    ADH_K128(false, true, false);
  }
#undef ADH_K128
  return launch_status();
}

}  // namespace adh
