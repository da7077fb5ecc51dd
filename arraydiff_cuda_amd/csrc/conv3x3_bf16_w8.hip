// 3x3 slab convolution on the bf16 matrix cores (v_mfma_f32_16x16x32_bf16), forward and
// backward-data, for up to 64 reduction channels: the eight-wave kernel, two waves per SIMD.
//
// A persistent workgroup of eight waves walks work items (image, 64-column strip, row segment)
// four output rows at a time, like the four-wave kernel of conv3x3_bf16_mfma.hip, and keeps the
// strip's input rows in LDS as a ring of ten rows in [pixel][channel] order, so that the matrix
// operand of 16 pixels x 32 channels is one 16-byte LDS read per lane at any column shift.  What
// differs is how rows get there and how the work is cut:
//
// * Rows arrive by `buffer_load ... lds` (16 bytes per lane, asynchronous, no registers) in the
//   order they have in memory, [channel][pixel]: every wave copies eight channels x four rows x
//   nine 8-pixel granules into a staging area of its own.  Rows, channels and granules that do
//   not exist get an out-of-range offset and arrive as zeros.
// * The wave then turns its own staging area into ring order with the transposing LDS read
//   (ds_read_b64_tr_b16: inside a group of 16 lanes, four lanes read one channel's 16 pixels and
//   every lane receives one pixel's four channels): two such reads and one 16-byte write per
//   16 pixels x 8 channels per lane group, no byte permutes, no masks.  Because a wave only ever
//   refills the staging area it has just read, one barrier per step is enough.
// * A wave owns 32 output channels x 32 columns x 2 rows: 48 operand reads and 144 MFMAs per
//   step, its filter share (9 taps x 64 x 32) in 144 registers; 8 accumulator tiles.  That fits
//   256 registers, so two waves share a SIMD.  Everything else a wave does in a step (its copies,
//   its transposition, its stores) is dealt out between the MFMA rounds one instruction at a
//   time: issued in a burst, memory instructions fill the memory pipeline's queue and the wave
//   stands at the next one with its MFMAs behind it.
// * The SIMD gives the matrix pipe to its older wave first, so waves 0-3 (row pair 0) finish
//   their rounds early and waves 4-7 late.  One barrier per step, after a wave's last ring
//   access: the early waves pack and store before it (they would wait anyway), the late ones
//   after it, while the early ones already multiply the next step.
// * `__syncthreads()` would wait for the copies in flight (the compiler puts vmcnt(0) before the
//   barrier); the barrier here waits for LDS only, and the wait for a row group's copies counts
//   the stores issued after them (memory instructions of a wave complete in order).
// * The sequence of row groups runs on across work items (the first rows of the next item are
//   requested during the last steps of the current one); an item costs one step without MFMAs.
//
// Forward takes the halo-padded input as it is (strip columns c0 .. c0 + 71).  Backward-data
// reads the unpadded gradient from column c0 - 8 (granules stay 16-byte aligned and are wholly
// inside or outside a row when the width is a multiple of 8) and finds its first column six
// pixels into the ring row.
#include "conv3x3_bf16_mfma.h"

namespace adh {

constexpr int kW8Threads = 512;
constexpr int kW8PxBytes = 160;                          // 64 channels + 32 bytes: measured, 16-byte reads of 16 neighbouring pixels run at the linear rate (4.5 cycles per wave; 8 at 144 bytes)
constexpr int kW8RowPx = 72;                             // nine granules of eight pixels
constexpr int kW8RingRows = 10;                          // 6 rows in use + 4 rows being written: a ring of 115200 bytes (157760 with 73-pixel rows)
constexpr int kW8RawCh = 144;                            // a channel row in the staging area: 72 pixels
constexpr int kW8Copies = 5;                             // 4 rows x 8 channels x 9 granules = 288 lanes of 5 x 64
constexpr int kW8RawWave = kW8Copies * 1024;
constexpr int kW8RawBytes = 8 * kW8RawWave;              // 40960

typedef short s16x4 __attribute__((ext_vector_type(4)));
#define ADH_LDS __attribute__((address_space(3)))

static __device__ __forceinline__ u32x2 lds_read_tr(const uint8_t *p) {
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((ADH_LDS s16x4 *)p));
}

static __device__ __forceinline__ uint32_t wrap_slot(uint32_t s) { return s >= (uint32_t)kW8RingRows ? s - (uint32_t)kW8RingRows : s; }

// BETA: the old output is added (in the first pass).  PIN: the sums of the passes before this one are read from
// P.part and added.  POUT: the sums go to P.part as fp32 instead of to the output as bf16 (a later pass follows).
// HF (P.pad == 1): neither the input nor the output carries a halo.  An output strip of 64 columns then needs
// input columns c0 - 1 .. c0 + 64, one more than the nine granules from c0 - 8 hold: the 32 lanes that copy 4
// leaves idle fetch the tenth granule of every row and channel into the idle tail of the staging area, and a
// sixth transposing read turns its first pixel into ring pixel 72 (rows of 73 pixels).  Rows -1 and IH come
// from the neighbouring tiles (P.neighbour_rows).
template <bool BETA, bool PIN = false, bool POUT = false, bool HF = false>
__global__ __launch_bounds__(kW8Threads, 1) void conv3x3_bf16_w8_kernel(ConvBf16Params P) {
  static_assert(!(BETA && PIN), "the old output is added in the first pass, which reads no sums");
  constexpr int kRowBytes = (HF ? kW8RowPx + 1 : kW8RowPx) * kW8PxBytes;
  constexpr int kRingBytes = kW8RingRows * kRowBytes;
  constexpr int kGroups = HF ? 6 : 5;  // transposing read pairs (and ring writes) per row group
  __shared__ __attribute__((aligned(16))) uint8_t raw[kW8RawBytes];
  __shared__ __attribute__((aligned(16))) uint8_t ring[kRingBytes];

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t h = wv & 1u, cw = (wv >> 1) & 1u, rp = wv >> 2;  // output-channel half, column half, row pair
  const uint32_t grp = blockIdx.y;

  // Workgroups are dealt to the eight XCDs (each with its own L2) in turn.  Renumber them so
  // that an XCD works on neighbouring strips: those share the 128-byte lines at strip borders.
  uint32_t vblock = blockIdx.x;
  if ((gridDim.x & 7u) == 0u) vblock = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const uint32_t total = P.whole_items + P.pieces;
  if (vblock >= total) return;

  // this wave's filter share, in B-operand order: lane (n = l16, k-block = g)
  u32x4 wreg[9][2][2];
  if (P.w_direct) {
    // Straight from the filter as the caller holds it (forward, (Cout, Cin, 3, 3), Cin a multiple of 64, 16-byte
    // aligned): the lane's eight reduction channels x nine taps of one output channel are 72 consecutive
    // elements, nine aligned 16-byte loads; what is left is to turn [channel][tap] into [tap][channel] in
    // registers, one byte permute per dword.  No reordering kernel runs before this one.
    const __amdgpu_buffer_rsrc_t rsrcW = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t *>(P.w_direct), 0, (int)(P.Cout * P.Cred * 18u), 0x00020000);
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int ct = 0; ct < 2; ++ct) {
        const uint32_t co = grp * 64u + 32u * h + 16u * ct + l16;
        const uint32_t ci = P.chan0 + 32u * half + 8u * g;
        // an output channel that does not exist lies past the end of the filter and loads as zero
        const uint32_t off = co < P.Cout ? (co * P.Cred + ci) * 18u : kOutOfRange;
        uint32_t d[36];
#pragma unroll
        for (int q = 0; q < 9; ++q) {
          const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrcW, off, 16 * q, 0);
          d[4 * q + 0] = v[0]; d[4 * q + 1] = v[1]; d[4 * q + 2] = v[2]; d[4 * q + 3] = v[3];
        }
        // element k = 9 * channel + tap sits in dword k / 2, half k % 2
#pragma unroll
        for (int tap = 0; tap < 9; ++tap) {
          u32x4 r;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int klo = 18 * j + tap, khi = klo + 9;
            // v_perm_b32 picks bytes from {first operand: bytes 4-7, second operand: bytes 0-3}
            const uint32_t sel = ((khi & 1) ? 0x07060000u : 0x05040000u) | ((klo & 1) ? 0x00000302u : 0x00000100u);
            r[j] = __builtin_amdgcn_perm(d[khi >> 1], d[klo >> 1], sel);
          }
          wreg[tap][half][ct] = r;
        }
      }
  } else {
    const u32x4 *wt = reinterpret_cast<const u32x4 *>(P.wt + ((size_t)grp * P.passes + P.pass) * kWtGroupElems);
#pragma unroll
    for (int tap = 0; tap < 9; ++tap)
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
          wreg[tap][half][ct] = wt[((tap * 2 + half) * 64 + (int)(32u * h + 16u * ct + l16)) * 4 + (int)g];
  }

  const uint32_t plane_bytes = P.IH * P.IW * 2u;
  const uint32_t image_bytes = P.Cred * plane_bytes;
  // ring pixel of the strip's first output column at tap column 0: the staged row starts eight columns left of
  // the strip whenever the input has no halo of its own (pad 1: unpadded in and out; pad 2: backward-data into a padded slab)
  const uint32_t xoff = P.pad ? 8u - (uint32_t)P.pad : 0u;
  const int32_t col_back = P.pad ? 8 : 0;       // the staged row starts this many columns left of the strip

  // ---- requests: copy q of a group moves staging slots 64 q + lane; slot = (row * 8 + channel) * 9 + granule
  uint32_t ld_off[kW8Copies];   // byte offset of the slot's granule for row 0 of the group and strip column 0
  uint32_t ld_rows = 0;         // 3 bits per copy: row of the group, bit 2 = the slot exists and so does its channel
  uint32_t ld_gran = 0;         // 4 bits per copy: granule
#pragma unroll
  for (int q = 0; q < kW8Copies; ++q) {
    const uint32_t slot = 64u * q + lane;
    uint32_t row = slot / 72u, rem = slot - row * 72u, ch = rem / 9u, gran = rem - ch * 9u;
    if (HF && slot >= 288u) {  // the tenth granule: slot 288 + 8 row + channel
      row = (slot - 288u) >> 3;
      ch = slot & 7u;
      gran = 9u;
    }
    const uint32_t chan = 8u * wv + ch;
    const bool ok = (HF || slot < 288u) && chan < P.cred_pass;
    ld_off[q] = (P.chan0 + chan) * plane_bytes + row * P.IW * 2u + gran * 16u;
    ld_rows |= ((row & 3u) | (ok ? 4u : 0u)) << (3 * q);
    ld_gran |= gran << (4 * q);
  }
  uint8_t *const raw_wave = raw + wv * kW8RawWave;

  // ---- turning the staging area into ring order.  Lane (j = l16, g): rounds 0-3 handle row t,
  // pixel block g; round 4 handles row g, pixel block 4 (pixels 64-71; its lanes 8-15 of a group
  // hold pixels 72-79, which do not exist, and write to the unused tail of the staging area).  A
  // transposing read takes channel j / 4 (+ 4 in the second read) at pixels 16 b + 4 (j % 4) and
  // returns pixel 16 b + j.
  const uint32_t tr_lane = (l16 >> 2) * kW8RawCh + (l16 & 3u) * 8u;
  const uint8_t *const tr03 = raw_wave + tr_lane + g * 32u;                  // + t * 8 * kW8RawCh
  const uint8_t *const tr4 = raw_wave + tr_lane + g * 8u * kW8RawCh + 128u;
  const uint32_t wr03 = (16u * g + l16) * kW8PxBytes + wv * 16u;             // + slot(row t) * kRowBytes
  const uint32_t wr4 = (64u + l16) * kW8PxBytes + wv * 16u;                  // + slot(row g) * kRowBytes
  uint8_t *const wr4_dummy = raw_wave + 288 * 16 + ((l16 & 7u) + 8u * g) * 16u;
  // HF, round 5: row g's tenth granule, [channel][8 pixels] at slot 288 + 8 g + channel; lane 0 of the group
  // receives its first pixel (the reads of the other lanes run on into the next slots and are not used)
  const uint8_t *const tr5 = raw_wave + (288u + 8u * g + (l16 >> 2)) * 16u + (l16 & 3u) * 8u;
  const uint32_t wr5 = (uint32_t)kW8RowPx * kW8PxBytes + wv * 16u;           // + slot(row g) * kRowBytes

  uint32_t tb = 0;  // ring slot the next transposed group starts at
  struct TrPair { u32x2 lo, hi; };
  auto tr_read = [&](auto tag, TrPair &T) {
    constexpr int t = decltype(tag)::value;
    if constexpr (t < 4) {
      T.lo = lds_read_tr(tr03 + t * 8 * kW8RawCh);
      T.hi = lds_read_tr(tr03 + t * 8 * kW8RawCh + 4 * kW8RawCh);
    } else if constexpr (t == 4) {
      T.lo = lds_read_tr(tr4);
      T.hi = lds_read_tr(tr4 + 4 * kW8RawCh);
    } else {
      T.lo = lds_read_tr(tr5);
      T.hi = lds_read_tr(tr5 + 4 * 16);
    }
  };
  auto tr_write = [&](auto tag, const TrPair &T) {
    constexpr int t = decltype(tag)::value;
    const u32x4 v = {T.lo[0], T.lo[1], T.hi[0], T.hi[1]};
    if constexpr (t < 4) {
      *reinterpret_cast<u32x4 *>(ring + wrap_slot(tb + (uint32_t)t) * kRowBytes + wr03) = v;
    } else if constexpr (t == 4) {
      uint8_t *const dst = ring + wrap_slot(tb + g) * kRowBytes + wr4;
      *reinterpret_cast<u32x4 *>(l16 < 8u ? dst : wr4_dummy) = v;
    } else {
      if (l16 == 0u) *reinterpret_cast<u32x4 *>(ring + wrap_slot(tb + g) * kRowBytes + wr5) = v;
    }
  };

  // ---- the loader's place in the sequence of row groups: work item, group -1 .. steps - 1
  // (group k holds the item's ring-relative rows 4 k + 2 .. 4 k + 5; rows -2, -1 are never used)
  uint32_t workL = vblock;
  int32_t grpL = -1, stepsL = 0;
  int32_t arow0L = 0, colL = 0;          // input row of ring-relative row 0, input column of staged pixel 0
  uint32_t okL = 0;                      // 5 bits: copy q of this lane exists for this item (slot, channel, granule column)
  __amdgpu_buffer_rsrc_t rsrcL = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(P.in[0]), 0, 0, 0x00020000);
  // P.neighbour_rows: the tiles are the row tiles of one tensor in rank order and carry no halo; input row -1 of
  // tile t > 0 is the last row of tile t - 1 and input row IH of tile t < tiles - 1 the first row of tile t + 1
  __amdgpu_buffer_rsrc_t rsrcUp = rsrcL, rsrcDn = rsrcL;
  bool hasUpL = false, hasDnL = false;

  // decodes a work number into (tile, image, first column, first and last output row)
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
    c0 = strip * kStripCols;
    r_begin = seg * seg_steps * kStepRows;
    r_end = min(P.OH, r_begin + seg_steps * kStepRows);
  };

  auto loader_open = [&]() {
    uint32_t tile, n, c0, r_begin, r_end;
    decode(workL, tile, n, c0, r_begin, r_end);
    stepsL = (int32_t)((r_end - r_begin + kStepRows - 1) / kStepRows);
    arow0L = (int32_t)r_begin - P.pad;
    colL = (int32_t)c0 - col_back;
    const uint16_t *in_img = P.in[tile] + (size_t)n * P.Cred * P.IH * P.IW;
    rsrcL = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(in_img), 0, image_bytes, 0x00020000);
    if (P.neighbour_rows) {
      hasUpL = tile > 0u;
      hasDnL = tile + 1u < P.num_tiles;
      const size_t img_off = (size_t)n * P.Cred * P.IH * P.IW;
      rsrcUp = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(P.in[hasUpL ? tile - 1u : tile] + img_off), 0,
                                                 image_bytes, 0x00020000);
      rsrcDn = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(P.in[hasDnL ? tile + 1u : tile] + img_off), 0,
                                                 image_bytes, 0x00020000);
    }
    okL = 0;
#pragma unroll
    for (int q = 0; q < kW8Copies; ++q) {
      const int32_t col = colL + 8 * (int32_t)((ld_gran >> (4 * q)) & 15u);
      const bool ok = ((ld_rows >> (3 * q)) & 4u) && col >= 0 && col < (int32_t)P.IW;
      okL |= (ok ? 1u : 0u) << q;
    }
    grpL = -1;
  };
  // Copy q of the loader's current group.  Once all work has been requested okL is zero and the
  // copies only write zeros, which go to ring rows nobody reads: the sequence needs no branches.
  // NBR: the group holds a row that comes from a neighbouring tile.  A copy instruction has one buffer, so the
  // lanes of that row take an instruction of their own with the neighbour's (lanes that are switched off write
  // nothing to LDS); one image plane further on or back turns row -1 into the neighbour's last row and row IH
  // into its first.
  auto request = [&](auto tag, auto nbr_tag) {
    constexpr int q = decltype(tag)::value;
    constexpr bool NBR = decltype(nbr_tag)::value != 0;
    const int32_t first = arow0L + 4 * grpL + 2;   // input row of the group's first row
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
  // does the group the loader stands at hold a neighbour's row?  (the same in every lane)
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
  // The MFMA leaves a lane with four neighbouring columns of one output channel in each of its
  // two column tiles; a swap between lane rows (v_permlane16_swap) turns that into eight
  // neighbouring columns, so a store moves 16 bytes per lane and four lanes fill a 64-byte run.
  const uint32_t ocol_lane = 32u * cw + ((g & 1u) ? 16u : 0u) + (g >> 1) * 8u;  // + first column of the strip
  const uint32_t co0 = grp * 64u + 32u * h + l16;
  const bool okct[2] = {co0 < P.Cout, co0 + 16u < P.Cout};
  const uint32_t out_image_bytes = P.Cout * P.OH * P.OW * 2u;
  const uint32_t ct_bytes = 16u * P.OH * P.OW * 2u, orow_bytes = P.OW * 2u;
  const uint32_t ooff_lane = (co0 * P.OH * P.OW + ocol_lane) * 2u;  // + (row * OW + first column) * 2
  uint16_t *out_imgC = nullptr;
  __amdgpu_buffer_rsrc_t rsrcC = __builtin_amdgcn_make_buffer_rsrc(P.out[0], 0, 0, 0x00020000);
  // the fp32 sums between passes: the lane's own four columns of accumulator [row][column tile][channel tile]
  // at (co0 + 16 ct, row, c0 + 32 cw + 16 cti + 4 g): 16 bytes per lane, 64 per output channel and lane row
  constexpr bool PART = PIN || POUT;
  const uint32_t poff_lane = (co0 * P.OH * P.OW + 32u * cw + 4u * g) * 4u;  // + (row * OW + first column) * 4
  const uint32_t pct_bytes = 2u * ct_bytes, prow_bytes = 2u * orow_bytes;
  float *part_imgC = nullptr;
  __amdgpu_buffer_rsrc_t rsrcP = __builtin_amdgcn_make_buffer_rsrc(P.out[0], 0, 0, 0x00020000);
  bool wholeC = false;  // every lane of the wave stores eight whole columns of two existing channels
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
    wholeC = __builtin_amdgcn_ballot_w64(!(c0C + ocol_lane + 7u < P.OW && okct[0] && okct[1])) == 0ull;
  };
  compute_open();

  // operand reads: pixel (32 cw + 16 cti + l16 + kw + xoff) of a ring row, channels 8 g .. 8 g + 7 of a half
  const uint32_t read_lane = (32u * cw + l16 + xoff) * kW8PxBytes + g * 16u;

  u32x4 pk[2][2], old[2][2];  // [channel tile][row of the pair]: packed results, old values for beta = 1

  // stores the packed results of a step lane by lane: edge strips and channel remainders
  auto store_guarded = [&](uint32_t row0, uint32_t nrows) {
    const uint32_t ocol = c0C + ocol_lane;
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int r = 0; r < 2; ++r)
        if ((uint32_t)r < nrows && okct[ct]) {
          uint16_t *p = out_imgC + ((size_t)(co0 + 16u * ct) * P.OH + row0 + r) * P.OW + ocol;
          if (ocol + 7u < P.OW) {
            *reinterpret_cast<u32x4_unaligned *>(p) = pk[ct][r];
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (ocol + e < P.OW) p[e] = (uint16_t)(pk[ct][r][e >> 1] >> ((e & 1) * 16));
          }
        }
  };
  auto load_old_guarded = [&](uint32_t row0, uint32_t nrows) {
    const uint32_t ocol = c0C + ocol_lane;
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        old[ct][r] = (u32x4){0u, 0u, 0u, 0u};
        if ((uint32_t)r < nrows && okct[ct]) {
          const uint16_t *p = out_imgC + ((size_t)(co0 + 16u * ct) * P.OH + row0 + r) * P.OW + ocol;
          if (ocol + 7u < P.OW) {
            old[ct][r] = *reinterpret_cast<const u32x4_unaligned *>(p);
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (ocol + e < P.OW) old[ct][r][e >> 1] |= (uint32_t)p[e] << ((e & 1) * 16);
          }
        }
      }
  };

  // the fp32 sums between passes, element by element: stored, or added to the accumulators
  auto part_guarded = [&](floatx4 (&acc)[2][2][2], uint32_t row0, uint32_t nrows, bool store) {
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
      for (int cti = 0; cti < 2; ++cti)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
          if ((uint32_t)r < nrows && okct[ct]) {
            const uint32_t col = c0C + 32u * cw + 16u * cti + 4u * g;
            float *p = part_imgC + ((size_t)(co0 + 16u * ct) * P.OH + row0 + r) * P.OW + col;
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (col + e < P.OW) {
                if (store)
                  p[e] = acc[r][cti][ct][e];
                else
                  acc[r][cti][ct][e] += p[e];
              }
          }
  };

  // The matrix part of a step: 48 operand reads (input row, column shift, channel half, column
  // tile), each fetched kAhead reads before its MFMAs; then the results are packed to bf16 and
  // stored.  Rounds alternate between an input row that feeds one output row of the pair (two
  // MFMAs) and one that feeds both (four), so that the reads run an even 240 or more matrix
  // cycles ahead.  With SIDE everything else a wave does in a phase is dealt out between the
  // rounds, one instruction at a time, so that no wave ever stands at a queue of memory
  // instructions while its matrix pipe idles: the five transposing read pairs and ring writes
  // of the row group that has landed, the five copies of the next group, and for beta = 1 the
  // four loads of old values (buffer loads and stores: a row that does not exist gets an
  // out-of-range offset, so the sequence has no branches).
  auto compute = [&](uint32_t sb, auto side_tag, auto bar_tag, auto nbr_tag, uint32_t row0, uint32_t nrows, bool barrier_owed,
                     bool after_plain) {
    constexpr bool SIDE = decltype(side_tag)::value != 0;
    // 1: this phase's barrier comes between the rounds and the packing; 2: the previous phase's barrier, if still
    // owed, comes after the first operand fetches (row pair 0 only: they read rows that step shares with this one)
    constexpr int BAR = decltype(bar_tag)::value;
    const uint32_t cur_off = ooff_lane + (row0 * P.OW + c0C) * 2u;
    const uint32_t off0 = nrows > 0u ? cur_off : kOutOfRange, off1 = nrows > 1u ? cur_off + orow_bytes : kOutOfRange;
    const uint32_t pcur = poff_lane + (row0 * P.OW + c0C) * 4u;
    const uint32_t poff0 = nrows > 0u ? pcur : kOutOfRange, poff1 = nrows > 1u ? pcur + prow_bytes : kOutOfRange;
    floatx4 pin[2][2];  // [channel tile][column tile]: the earlier passes' sums of the output row being finished
    floatx4 acc[2][2][2];  // [row][column tile][channel tile]
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
      for (int cti = 0; cti < 2; ++cti)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) acc[r][cti][ct] = (floatx4){0.f, 0.f, 0.f, 0.f};
    constexpr int kReads = 48, kAhead = HF ? ((BETA || PIN) ? 2 : 2) : ((BETA || PIN) ? 3 : 4);
    const uint8_t *row_ptr[4];
#pragma unroll
    for (int ir = 0; ir < 4; ++ir) row_ptr[ir] = ring + wrap_slot(sb + 2u * rp + (uint32_t)ir) * kRowBytes + read_lane;
    u32x4 abuf[kAhead + 1];
    TrPair trp[2];
    // round t reads input row 0, 1, 0, 1, .. for t < 24 (two and four MFMAs in turn), then row 2
    // for twelve rounds and row 3 for the last twelve: output row 0 of the pair is complete after
    // round 35 and is packed and stored between the two-MFMA rounds of row 3
    auto fetch = [&](int t) {
      const int ir = t < 24 ? (t & 1) : t / 12, j = t < 24 ? t >> 1 : t % 12, kw = j >> 2, half = (j >> 1) & 1, cti = j & 1;
      abuf[t % (kAhead + 1)] =
          *reinterpret_cast<const u32x4 *>(row_ptr[ir] + (cti * 16 + kw) * kW8PxBytes + half * 64);
    };
#pragma unroll
    for (int t = 0; t < kAhead; ++t) fetch(t);
    __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
    if constexpr (BAR == 2) {
      if (barrier_owed) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // The copies of the group to transpose have landed: everything but the previous step's four
    // stores, which were issued after them (memory instructions complete in order).
    // (eight stores when the sums go out as fp32).  After a phase without MFMAs nothing was issued after the
    // copies, and the wait is for all of them.
    if (SIDE) {
      if (after_plain)
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      else
        __builtin_amdgcn_s_waitcnt(POUT ? 0x0F78 : 0x0F74);  // vmcnt(8) : vmcnt(4)
    }
    // packs tile i (row i / 2 of the pair, channel tile i % 2) back to store order through the
    // swap between lane rows and, in the interleaved form, stores it
    auto pack_tile = [&](auto tag) {
      constexpr int r = decltype(tag)::value >> 1, ct = decltype(tag)::value & 1;
      floatx4 v0 = acc[r][0][ct], v1 = acc[r][1][ct];
      if (BETA) {
        // the old values, back in the MFMA's arrangement: the swap is its own inverse
        const u32x2 s0 = __builtin_amdgcn_permlane16_swap(old[ct][r][0], old[ct][r][2], false, false);
        const u32x2 s1 = __builtin_amdgcn_permlane16_swap(old[ct][r][1], old[ct][r][3], false, false);
        v0[0] += __uint_as_float(s0[0] << 16);
        v0[1] += __uint_as_float(s0[0] & 0xffff0000u);
        v0[2] += __uint_as_float(s1[0] << 16);
        v0[3] += __uint_as_float(s1[0] & 0xffff0000u);
        v1[0] += __uint_as_float(s0[1] << 16);
        v1[1] += __uint_as_float(s0[1] & 0xffff0000u);
        v1[2] += __uint_as_float(s1[1] << 16);
        v1[3] += __uint_as_float(s1[1] & 0xffff0000u);
      }
      if constexpr (PIN && SIDE) {
        v0 += pin[ct][0];
        v1 += pin[ct][1];
      }
      if constexpr (POUT) {
        if constexpr (SIDE) {
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v0), rsrcP, r ? poff1 : poff0, ct ? pct_bytes : 0u, 0);
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v1), rsrcP, (r ? poff1 : poff0) + 64u,
                                                 ct ? pct_bytes : 0u, 0);
        } else {
          acc[r][0][ct] = v0;
          acc[r][1][ct] = v1;
        }
        return;
      }
      const u32x2 q0 = __builtin_amdgcn_permlane16_swap(pack_bf16x2(v0[0], v0[1]), pack_bf16x2(v1[0], v1[1]), false, false);
      const u32x2 q1 = __builtin_amdgcn_permlane16_swap(pack_bf16x2(v0[2], v0[3]), pack_bf16x2(v1[2], v1[3]), false, false);
      pk[ct][r] = (u32x4){q0[0], q1[0], q0[1], q1[1]};
      if constexpr (SIDE)
        __builtin_amdgcn_raw_buffer_store_b128(pk[ct][r], rsrcC, r ? off1 : off0, ct ? ct_bytes : 0u, 0);
    };
    auto round = [&](auto tag) {
      constexpr int t = decltype(tag)::value;
      if constexpr (t + kAhead < kReads) {
        fetch(t + kAhead);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      constexpr int ir = t < 24 ? (t & 1) : t / 12, j = t < 24 ? t >> 1 : t % 12, kw = j >> 2, half = (j >> 1) & 1, cti = j & 1;
      const bf16x8 a = __builtin_bit_cast(bf16x8, abuf[t % (kAhead + 1)]);
      constexpr int kh_lo = ir - 1 > 0 ? ir - 1 : 0;
      constexpr int kh_hi = ir < 2 ? ir : 2;
#pragma unroll
      for (int kh = kh_lo; kh <= kh_hi; ++kh) {
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
          acc[ir - kh][cti][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              a, __builtin_bit_cast(bf16x8, wreg[kh * 3 + kw][half][ct]), acc[ir - kh][cti][ct], 0, 0, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 2 * (kh_hi - kh_lo + 1), 0);
      if constexpr (SIDE) {
        // rounds 0, 2, .., 8 (HF: 10): transposing read pair t / 2; rounds 3, 5, .., 11 (13): ring write (t - 3) / 2
        if constexpr (t % 2 == 0 && t <= 2 * (kGroups - 1)) {
          tr_read(IntTag<t / 2>(), trp[(t / 2) % 2]);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        if constexpr (t >= 3 && t % 2 == 1 && t <= 2 * kGroups + 1) {
          tr_write(IntTag<(t - 3) / 2>(), trp[((t - 3) / 2) % 2]);
          __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
        // rounds 13, 15, .., 21 (HF: 15 .. 23): copy of the next row group (every transposing read has returned)
        constexpr int kReq0 = HF ? 15 : 13;
        if constexpr (t >= kReq0 && t % 2 == 1 && t <= kReq0 + 8) {
          request(IntTag<(t - kReq0) / 2>(), nbr_tag);
          if constexpr (!decltype(nbr_tag)::value) __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
        // rounds 38 and 42: output row 0, complete since round 35, is packed and stored
        if constexpr (t == 38 || t == 42) {
          pack_tile(IntTag<(t - 38) / 4>());
          __builtin_amdgcn_sched_group_barrier(0x010, POUT ? 2 : 1, 0);
        }
        // the earlier passes' sums: output row 0 in rounds 24, 27, 30, 33; row 1 once row 0's have been used
        // (rounds 39, 40 after the packing in round 38; rounds 43, 44 after the one in round 42)
        if constexpr (PIN && t >= 24 && (t - 24) % 3 == 0 && t <= 33) {
          constexpr int i = (t - 24) / 3, ct = i >> 1, cti = i & 1;
          pin[ct][cti] = __builtin_bit_cast(
              floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsrcP, poff0 + 64u * cti, ct ? pct_bytes : 0u, 0));
          __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
        if constexpr (PIN && (t == 39 || t == 40 || t == 43 || t == 44)) {
          constexpr int ct = t > 41 ? 1 : 0, cti = (t == 40 || t == 44) ? 1 : 0;
          pin[ct][cti] = __builtin_bit_cast(
              floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsrcP, poff1 + 64u * cti, ct ? pct_bytes : 0u, 0));
          __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
        // rounds 24, 27, 30, 33: old value (t - 24) / 3 of this step, row 0 first
        if constexpr (BETA && t >= 24 && (t - 24) % 3 == 0 && t <= 33) {
          constexpr int i = (t - 24) / 3, ct = i & 1, r = i >> 1;
          old[ct][r] = __builtin_amdgcn_raw_buffer_load_b128(rsrcC, r ? off1 : off0, ct ? ct_bytes : 0u, 0);
          __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
      }
    };
    for_each_int(std::make_integer_sequence<int, kReads>(), round);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (BAR == 1) {
      // every ring read and write of the phase is done (the operands have been multiplied)
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (!SIDE) {
      if constexpr (PIN) part_guarded(acc, row0, nrows, false);
      for_each_int(std::make_integer_sequence<int, 4>(), pack_tile);
      if constexpr (POUT)
        part_guarded(acc, row0, nrows, true);
      else
        store_guarded(row0, nrows);
    } else {
      pack_tile(IntTag<2>());
      pack_tile(IntTag<3>());
    }
  };

  // the same side work in one piece, for the phases that cannot take the interleaved form
  auto move_rows_plain = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    TrPair T[kGroups];
    for_each_int(std::make_integer_sequence<int, kGroups>(), [&](auto tag) { tr_read(tag, T[decltype(tag)::value]); });
    for_each_int(std::make_integer_sequence<int, kGroups>(), [&](auto tag) { tr_write(tag, T[decltype(tag)::value]); });
    for_each_int(std::make_integer_sequence<int, 5>(), [&](auto tag) { request(tag, IntTag<HF ? 1 : 0>()); });
  };

  // One phase per step, plus one without MFMAs at the start of every item and a second one at the
  // very start.  In phase f a wave transposes row group f + 1 (requested in phase f - 1) into
  // the four ring slots that the step's six input rows leave free, requests group f + 2 and
  // multiplies step f; the phase's barrier publishes the ring rows written in it and frees the
  // ones read in it.
  uint32_t sb = 4;  // ring slot of the first input row of the step multiplied in this phase
  loader_open();
  for_each_int(std::make_integer_sequence<int, 5>(), [&](auto tag) { request(tag, IntTag<HF ? 1 : 0>()); });
  loader_advance();
  // Every wave passes one barrier per phase, after its last ring access of the phase.
  auto phase_barrier = [&]() {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): LDS only; __syncthreads() would also wait for the copies in flight
    __builtin_amdgcn_s_barrier();
  };
  // Row pair 0 (the older wave of every SIMD, which finishes its rounds early) owes each phase's barrier
  // until the next phase has fetched its first operands: those come from the two rows a step shares
  // with the one before it, which no wave overwrites meanwhile.  Its matrix pipe then starts the moment
  // the late waves arrive.  Row pair 1 passes the barrier between its rounds and its packing.
  bool barrier_owed = false;
  bool after_plain = true;  // the last phase issued its copies last: no stores after them
  for (;;) {
    const bool fast = stepC >= 0 && wholeC;
    if (barrier_owed && !(fast && rp == 0u)) {
      phase_barrier();
      barrier_owed = false;
    }
    bool barrier_done = false;
    if (stepC >= 0) {
      const uint32_t row0 = r_beginC + (uint32_t)stepC * kStepRows + 2u * rp;  // this wave's first output row
      const uint32_t nrows = row0 >= r_endC ? 0u : min(2u, r_endC - row0);
      if (wholeC) {
        // (the few steps whose next row group holds a neighbour's row run a second instance of the step)
        bool nbr = false;
        if constexpr (HF) nbr = group_has_neighbour_row();
        if (rp == 0u) {
          if constexpr (HF) {
            if (nbr) compute(sb, IntTag<1>(), IntTag<2>(), IntTag<1>(), row0, nrows, barrier_owed, after_plain);
            else compute(sb, IntTag<1>(), IntTag<2>(), IntTag<0>(), row0, nrows, barrier_owed, after_plain);
          } else {
            compute(sb, IntTag<1>(), IntTag<2>(), IntTag<0>(), row0, nrows, barrier_owed, after_plain);
          }
          barrier_owed = false;
        } else {
          if constexpr (HF) {
            if (nbr) compute(sb, IntTag<1>(), IntTag<1>(), IntTag<1>(), row0, nrows, false, after_plain);
            else compute(sb, IntTag<1>(), IntTag<1>(), IntTag<0>(), row0, nrows, false, after_plain);
          } else {
            compute(sb, IntTag<1>(), IntTag<1>(), IntTag<0>(), row0, nrows, false, after_plain);
          }
          barrier_done = true;
        }
        after_plain = false;
      } else {
        if (BETA) load_old_guarded(row0, nrows);
        move_rows_plain();
        compute(sb, IntTag<0>(), IntTag<0>(), IntTag<0>(), row0, nrows, false, false);
        after_plain = true;  // its stores are conditional: count on none
      }
    } else {
      move_rows_plain();
      after_plain = true;
    }
    loader_advance();
    if (!barrier_done) {
      if (rp == 0u)
        barrier_owed = true;
      else
        phase_barrier();
    }
    sb = wrap_slot(sb + kStepRows);
    tb = wrap_slot(tb + kStepRows);
    if (++stepC == stepsC) {
      workC += gridDim.x;
      if (workC >= total) break;
      compute_open();
      stepC = -1;
    }
  }
  if (barrier_owed) phase_barrier();
}

// Shapes of the eight-wave kernel: input and output rows that start on a 4-byte boundary (input
// rows on 16 bytes for backward-data, whose granules must lie wholly inside or outside a row),
// images whose byte offsets fit the buffer range check's 31 bits.
bool conv_bf16_w8_takes(const ConvBf16Params &P, uint32_t num_tiles) {
  if (P.pad ? (P.IW % 8u) != 0u : (P.IW % 2u) != 0u) return false;
  if (P.neighbour_rows && P.IH == 0u) return false;
  const uint64_t image_bytes = (uint64_t)P.Cred * P.IH * P.IW * 2u;
  if (image_bytes >= (1ull << 31)) return false;
  if ((uint64_t)P.Cout * P.OH * P.OW * 2u >= (1ull << 31) || (P.OW % 2u) != 0u) return false;
  const size_t a = P.pad ? 16 : 4;
  for (uint32_t t = 0; t < num_tiles; ++t)
    if (!aligned_to(P.in[t], a) || !aligned_to(P.out[t], 4)) return false;
  if (P.Cred > 64u) {
    // the fp32 sums between passes are addressed like the output, at four bytes an element
    if ((uint64_t)P.Cout * P.OH * P.OW * 4u >= (1ull << 31)) return false;
    for (uint32_t t = 0; t < num_tiles; ++t)
      if (P.part[t] && !aligned_to(P.part[t], 16)) return false;
  }
  return true;
}

int conv_bf16_w8_launch(const ConvBf16Params &P, uint32_t gx, uint32_t groups, hipStream_t st) {
  const dim3 grid(gx, groups), block(kW8Threads);
  const bool first = P.first_pass != 0u, last = P.last_pass != 0u;
  if (P.pad == 1) {  // no halo on either side
    if (first && last) {
      if (P.beta != 0.f)
        hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<true, false, false, true>), grid, block, 0, st, P);
      else
        hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<false, false, false, true>), grid, block, 0, st, P);
    } else if (first) {
      if (P.beta != 0.f)
        hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<true, false, true, true>), grid, block, 0, st, P);
      else
        hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<false, false, true, true>), grid, block, 0, st, P);
    } else if (!last) {
      hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<false, true, true, true>), grid, block, 0, st, P);
    } else {
      hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<false, true, false, true>), grid, block, 0, st, P);
    }
    return launch_status();
  }
  if (first && last) {
    if (P.beta != 0.f)
      hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<true>), grid, block, 0, st, P);
    else
      hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<false>), grid, block, 0, st, P);
  } else if (first) {
    if (P.beta != 0.f)
      hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<true, false, true>), grid, block, 0, st, P);
    else
      hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<false, false, true>), grid, block, 0, st, P);
  } else if (!last) {
    hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<false, true, true>), grid, block, 0, st, P);
  } else {
    hipLaunchKernelGGL((conv3x3_bf16_w8_kernel<false, true, false>), grid, block, 0, st, P);
  }
  return launch_status();
}

}  // namespace adh
