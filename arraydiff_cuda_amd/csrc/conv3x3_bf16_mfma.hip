// 3x3 slab convolution on the bf16 matrix cores (v_mfma_f32_16x16x32_bf16), forward and
// backward-data, for up to 64 reduction channels per launch (more: one launch per 64, fp32 sums
// between them), any width and alignment.
//
// Shape of the computation.  A workgroup of four waves (one per SIMD, which leaves each wave the
// whole register file) is persistent: it walks work items (image, 64-column strip, row segment)
// and, inside an item, steps down the strip four output rows at a time.  The input rows of the
// strip live in LDS as a ring of ten rows in [pixel][channel] order, so each input row is fetched
// from HBM once per strip; only the one-pixel column halo of a strip is read twice.  NCHW rows
// are turned into that order on the way in: a thread loads eight channels x eight pixels (eight
// 16-byte buffer loads), transposes the 8x8 block of 16-bit values with byte permutes and writes
// eight 16-byte LDS pieces.
//
// A wave owns 32 output channels x 32 columns x 4 rows.  Its share of the filter, 9 taps x 64
// reduction channels x 32 output channels, is loaded once per kernel into 144 registers in matrix
// operand order and never touches LDS.  Per step a wave reads 6 input rows x 3 column shifts x
// 2 channel halves x 2 column tiles = 72 pixel operands and issues 288 MFMAs: an operand read
// for input row r serves the output rows r, r-1, r-2 (taps kh = 0, 1, 2).
//
// What bounds the kernel is the number of global-memory instructions, not their bytes: an
// instruction that touches 16 separate short runs costs the memory pipeline the same whatever
// the run length.  Hence 64-column strips (128-byte runs per channel row on the way in) and, on
// the way out, a swap between lane rows that turns the MFMA's four columns per lane into eight,
// so that four lanes fill a 64-byte run per store.
//
// Out-of-range rows, channels and buffer ends are handled by the buffer resource's range check
// (out-of-range dwords read as zero); out-of-range columns by per-dword masks.
#include "conv3x3_bf16_mfma.h"

namespace adh {

constexpr int kRingRows = 10;                         // 6 rows in use + 4 rows being written
constexpr int kPatchCols = kStripCols + 2;            // 66
// LDS layout of a ring row: pixel px sits in slot px + px / 8 (one empty slot after every eight
// pixels), 160 bytes per slot (64 channels + 32 bytes of padding).  Measured on gfx950 with four
// waves: the 16-byte operand reads of 16 neighbouring pixels run at the rate of a linear read,
// and the loader's writes (eight lanes eight pixels apart) at 64 cycles instead of the 256 of a
// dense 144-byte layout.
constexpr int kPxPitch = 160;
constexpr int kRowSlots = kPatchCols + kPatchCols / 8;   // 74
constexpr int kRowPitch = kRowSlots * kPxPitch;       // 11840
constexpr int kRingBytes = kRingRows * kRowPitch;     // 118400
__host__ __device__ constexpr int px_slot(int px) { return px + (px >> 3); }

// filter (Cout, Cin, 3, 3) -> matrix-operand order.  flip = 0 (forward): out = Cout index,
// red = Cin index, tap as is.  flip = 1 (backward-data): out = Cin index, red = Cout index,
// tap mirrored.  Channels beyond the real extents are zero.
// Reduction channels come in passes of 64: wt[group][pass][tap][half][64 out][32 red].
__global__ __launch_bounds__(256) void conv3x3_bf16_filter_kernel(const uint16_t *__restrict__ w, uint16_t *__restrict__ wt,
                                                                  uint32_t Cin, uint32_t Cout, uint32_t flip,
                                                                  uint32_t passes, uint32_t total) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= total) return;
  const uint32_t r = i & 31u, o = (i >> 5) & 63u, half = (i >> 11) & 1u;
  const uint32_t tg = i >> 12, tap = tg % 9u, gp = tg / 9u, pass = gp % passes, grp = gp / passes;
  const uint32_t oc = grp * 64u + o, rc = pass * 64u + half * 32u + r;
  uint16_t v = 0;
  if (!flip) {
    if (oc < Cout && rc < Cin) v = w[((uint64_t)oc * Cin + rc) * 9u + tap];
  } else {
    if (oc < Cin && rc < Cout) v = w[((uint64_t)rc * Cin + oc) * 9u + (8u - tap)];
  }
  wt[i] = v;
}

// More than 64 reduction channels: one launch per 64 (P.pass), the sums travelling between the launches as fp32
// in P.part (PIN: this launch adds the sums of the earlier ones, POUT: it leaves its sums there instead of
// rounding them into the output).  BETA (old output added) belongs to the first launch.
template <bool BETA, bool PIN, bool POUT>
__global__ __launch_bounds__(256, 1) void conv3x3_bf16_kernel(ConvBf16Params P) {
  __shared__ __attribute__((aligned(16))) uint8_t ring[kRingBytes];

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t h = wv & 1u, cw = wv >> 1;  // output-channel half, column half of the strip
  const uint32_t grp = blockIdx.y;

  // this wave's filter share, in B-operand order: lane (n = l16, k-block = g)
  u32x4 wreg[9][2][2];
  {
    const u32x4 *wt = reinterpret_cast<const u32x4 *>(P.wt + ((size_t)grp * P.passes + P.pass) * kWtGroupElems);
#pragma unroll
    for (int tap = 0; tap < 9; ++tap)
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
          wreg[tap][half][ct] = wt[((tap * 2 + half) * 64 + (int)(32u * h + 16u * ct + l16)) * 4 + (int)g];
  }

  // loader role of this thread: one input row, eight channels, eight pixels; and for the two
  // tail pixels of a row (patch columns 64, 65) one channel
  const uint32_t lrow = tid >> 6, chg = (tid >> 3) & 7u, pxb = tid & 7u, tch = tid & 63u;
  const uint32_t plane_bytes = P.IH * P.IW * 2u;
  const uint32_t image_bytes = P.Cred * plane_bytes;
  uint32_t chvalid = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) chvalid |= (chg * 8u + j < P.cred_pass ? 1u : 0u) << j;
  const uint32_t tkeep = tch < P.cred_pass ? 0xffffffffu : 0u;
  // the image's last channel, counted from this launch's first (beyond 63: it belongs to a later launch)
  const uint32_t last_chan = P.Cred - 1u - P.chan0;

  // operand reads: pixel (32 cw + 16 cti + l16 + kw) of a ring row, channels 8 g .. 8 g + 7 of a half
  uint32_t read_lane_off[2][3];
#pragma unroll
  for (int cti = 0; cti < 2; ++cti)
#pragma unroll
    for (int kw = 0; kw < 3; ++kw)
      read_lane_off[cti][kw] = (uint32_t)px_slot((int)(32u * cw + 16u * cti + l16) + kw) * kPxPitch + g * 16u;

  // Workgroups are dealt to the eight XCDs (each with its own L2) in turn.  Renumber them so
  // that an XCD works on neighbouring strips: those share the 128-byte lines at strip borders.
  uint32_t vblock = blockIdx.x;
  if ((gridDim.x & 7u) == 0u) vblock = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  for (uint32_t work = vblock; work < P.whole_items + P.pieces; work += gridDim.x) {
    uint32_t item, seg = 0, seg_steps = P.steps_per_item;
    if (work < P.whole_items) {
      item = work;
    } else {
      // pieces of the left-over items, item index fastest: neighbouring workgroups get
      // neighbouring strips at the same rows
      uint32_t it;
      P.div_rest.divmod(work - P.whole_items, seg, it);
      item = P.whole_items + it;
      seg_steps = P.seg_steps;
    }
    uint32_t strip, plane, tile, n;
    P.div_strips.divmod(item, plane, strip);
    P.div_N.divmod(plane, tile, n);
    const int32_t c0 = (int32_t)(strip * kStripCols);
    const uint32_t r_begin = seg * seg_steps * kStepRows;
    const uint32_t r_end = min(P.OH, r_begin + seg_steps * kStepRows);
    const uint32_t nsteps = (r_end - r_begin + kStepRows - 1) / kStepRows;
    const uint16_t *in_img = P.in[tile] + (size_t)n * P.Cred * P.IH * P.IW;
    uint16_t *out_img = P.out[tile] + (size_t)n * P.Cout * P.OH * P.OW;
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(in_img), 0, image_bytes, 0x00020000);

    // columns of this thread's pixel block and their masks (two pixels per dword)
    const int32_t icol0 = c0 - P.pad + (int32_t)(pxb * 8u);
    uint32_t md[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int32_t ca = icol0 + 2 * d, cb2 = ca + 1;
      md[d] = ((ca >= 0 && ca < (int32_t)P.IW) ? 0x0000ffffu : 0u) | ((cb2 >= 0 && cb2 < (int32_t)P.IW) ? 0xffff0000u : 0u);
    }
    const int32_t tcol0 = c0 - P.pad + kStripCols;  // tail pixels
    const uint32_t mt = ((tcol0 >= 0 && tcol0 < (int32_t)P.IW) ? 0x0000ffffu : 0u) |
                        ((tcol0 + 1 >= 0 && tcol0 + 1 < (int32_t)P.IW) ? 0xffff0000u : 0u);
    const int32_t arow0 = (int32_t)r_begin - P.pad;  // input row of ring-relative row 0
    // byte offset of (channel chg*8, input row arow0 + lrow, column icol0); may be negative
    const int32_t vbase = (int32_t)(((P.chan0 + chg * 8u) * P.IH) * P.IW * 2u) + ((arow0 + (int32_t)lrow) * (int32_t)P.IW + icol0) * 2;
    const int32_t tbase = (int32_t)(((P.chan0 + tch) * P.IH) * P.IW * 2u) + ((arow0 + (int32_t)lrow) * (int32_t)P.IW + tcol0) * 2;

    // per-channel load offsets and keep-masks (all ones for a channel that exists)
    uint32_t vch[8], vkeep[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      vch[j] = (uint32_t)vbase + (uint32_t)j * plane_bytes;
      vkeep[j] = ((chvalid >> j) & 1u) ? 0xffffffffu : 0u;
    }

    // registers of a load round
    struct LoadRegs {
      u32x4 ld[8];
      uint32_t lt;
    };
    LoadRegs L0, L1;

    // one load of a round: k < 8 the k-th channel of the pixel block, k = 8 the tail; offsets
    // of absent rows and channels are replaced by one that is always out of range
    auto load_one = [&](auto tag, int32_t row0, LoadRegs &L) {
      constexpr int k = decltype(tag)::value;
      const int32_t i = row0 + (int32_t)lrow;
      const int32_t arow = arow0 + i;
      const uint32_t rowkeep = (i >= 0 && arow >= 0 && arow < (int32_t)P.IH) ? 0xffffffffu : 0u;
      const uint32_t step_off = (uint32_t)(row0 * (int32_t)P.IW * 2);
      if constexpr (k < 8) {
        const uint32_t keep = vkeep[k] & rowkeep;
        L.ld[k] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, ((vch[k] + step_off) & keep) | (kOutOfRange & ~keep), 0, 0);
      } else {
        const uint32_t keep = tkeep & rowkeep;
        L.lt = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (((uint32_t)tbase + step_off) & keep) | (kOutOfRange & ~keep), 0, 0);
      }
    };
    auto issue = [&](int32_t row0, LoadRegs &L) {
      for_each_int(std::make_integer_sequence<int, 9>(), [&](auto tag) { load_one(tag, row0, L); });
    };

    // the pieces of a row in ring order: eight pixels of eight channels each, plus this thread's
    // channel of the two tail pixels
    struct Transposed {
      u32x4 px[8];
      uint32_t tail;
      uint32_t dst, tdst;
    };
    // patches up what the range check dropped and works out where the row goes in the ring; the
    // caller makes sure that ring row row0 + lrow is not negative
    auto transpose_prepare = [&](int32_t row0, LoadRegs &L, Transposed &T) {
      const int32_t i = row0 + (int32_t)lrow;
      {
        const int32_t arow = arow0 + i;
        // A load that starts left of the image's first element (channel 0, left column halo: the
        // first row, and the second row of an image one column wide) has a negative offset and is
        // dropped as a whole: redo it dword by dword.  icol0 is a multiple of two pixels below zero,
        // so a dword that straddles the image's start holds no column of this row.
        const int32_t voff = vbase + row0 * (int32_t)P.IW * 2;
        if (arow >= 0 && chg == 0 && P.chan0 == 0u && voff < 0 && (chvalid & 1u)) {
#pragma unroll
          for (int d = 0; d < 4; ++d)
            L.ld[0][d] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, voff + 4 * d >= 0 ? (uint32_t)(voff + 4 * d) : kOutOfRange, 0, 0);
        }
        // The range check drops a dword that straddles the end of the image even though its low
        // half is the image's last element: fetch that element on its own.
        if (arow == (int32_t)P.IH - 1) {
          if (chg == last_chan >> 3) {
            const uint32_t j = last_chan & 7u;
            const uint32_t v = (uint32_t)(vbase + row0 * (int32_t)P.IW * 2) + j * plane_bytes;
            const uint32_t gap = image_bytes - 2u - v;  // distance of the last element from the load start
            if (gap < 16u && (gap & 3u) == 0u) {
              const uint32_t e = __builtin_amdgcn_raw_buffer_load_b16(rsrc, image_bytes - 2u, 0, 0) & 0xffffu;
              const uint32_t d = gap >> 2;
#pragma unroll
              for (int jj = 0; jj < 8; ++jj)
#pragma unroll
                for (int dd = 0; dd < 4; ++dd) L.ld[jj][dd] |= ((uint32_t)jj == j && (uint32_t)dd == d) ? e : 0u;
            }
          }
          if (tch == last_chan && (uint32_t)(tbase + row0 * (int32_t)P.IW * 2) == image_bytes - 2u)
            L.lt |= __builtin_amdgcn_raw_buffer_load_b16(rsrc, image_bytes - 2u, 0, 0) & 0xffffu;
        }
      }
      const uint32_t slot = (uint32_t)i % (uint32_t)kRingRows;
      T.dst = slot * kRowPitch + (uint32_t)px_slot((int)(pxb * 8u)) * kPxPitch + chg * 16u;
      T.tdst = slot * kRowPitch + px_slot(kStripCols) * kPxPitch + tch * 2u;
    };
    // piece d of the transposition: dword d of the eight channel registers -> pixels 2d, 2d + 1
    // (d = 0 also takes the tail along)
    auto transpose_piece = [&](auto tag, const LoadRegs &L, Transposed &T) {
      constexpr int d = decltype(tag)::value;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t lo = L.ld[2 * q][d] & md[d], hi = L.ld[2 * q + 1][d] & md[d];
        T.px[2 * d][q] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        T.px[2 * d + 1][q] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);
      }
      if constexpr (d == 0) T.tail = L.lt & mt;
    };
    // LDS write number w of a transposed row piece: 0..7 the pixels of the block, 8 and 9 the tail
    auto ring_write = [&](auto tag, const Transposed &T) {
      constexpr int w = decltype(tag)::value;
      if constexpr (w < 8)
        *reinterpret_cast<u32x4 *>(ring + T.dst + w * kPxPitch) = T.px[w];
      else
        *reinterpret_cast<uint16_t *>(ring + T.tdst + (w - 8) * kPxPitch) = (uint16_t)(T.tail >> ((w - 8) * 16));
    };
    auto commit = [&](int32_t row0, LoadRegs &L) {
      if (row0 + (int32_t)lrow < 0) return;
      Transposed T;
      transpose_prepare(row0, L, T);
      for_each_int(std::make_integer_sequence<int, 4>(), [&](auto tag) { transpose_piece(tag, L, T); });
      for_each_int(std::make_integer_sequence<int, 10>(), [&](auto tag) { ring_write(tag, T); });
    };

    // ring-relative rows 0 .. kStepRows + 1 of the first step
    issue(2 - kStepRows, L0);
    issue(2, L1);
    commit(2 - kStepRows, L0);
    commit(2, L1);
    if (nsteps > 1) issue(kStepRows + 2, L0);  // rows of step 1, committed at the start of step 0
    __syncthreads();

    // Output.  The MFMA leaves a lane with four neighbouring columns of one output channel in
    // each of its two column tiles; a swap between lane rows (v_permlane16_swap) turns that into
    // eight neighbouring columns, so a store moves 16 bytes per lane and four lanes fill a
    // 64-byte run.  The packed result of a step is stored during the next step.
    const uint32_t ocol = (uint32_t)c0 + 32u * cw + ((g & 1u) ? 16u : 0u) + (g >> 1) * 8u;
    const uint32_t co0 = grp * 64u + 32u * h + l16;
    const bool ok_ct[2] = {co0 < P.Cout, co0 + 16u < P.Cout};
    const bool full_cols = ocol + 7u < P.OW;
    const size_t ct_stride = (size_t)16u * P.OH * P.OW;
    uint16_t *const olane = out_img + (size_t)co0 * P.OH * P.OW + ocol;
    u32x4 pk[2][kStepRows], old[2][kStepRows];
    // the fp32 sums between launches, [image][output channel][row][column] per tile: a lane's four columns of
    // column tile cti start at pcol[cti], as the MFMA leaves them
    float *const part_lane = (PIN || POUT) ? P.part[tile] + ((size_t)n * P.Cout + co0) * P.OH * P.OW : nullptr;
    const uint32_t pcol[2] = {(uint32_t)c0 + 32u * cw + 4u * g, (uint32_t)c0 + 32u * cw + 16u + 4u * g};
    floatx4 pin[kStepRows][2][2];

    // common case, decided per wave: all rows of a step, both channel tiles, eight whole columns
    const bool lanes_whole = __builtin_amdgcn_ballot_w64(!(full_cols && ok_ct[0] && ok_ct[1])) == 0ull;

    auto store_packed = [&](uint32_t row0, uint32_t nrows) {
      uint16_t *obase = olane + (size_t)row0 * P.OW;
      if (full_cols) {
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
          for (int r = 0; r < kStepRows; ++r)
            if ((uint32_t)r < nrows && ok_ct[ct])
              *reinterpret_cast<u32x4_unaligned *>(obase + ct * ct_stride + (size_t)r * P.OW) = pk[ct][r];
      } else if (ocol < P.OW) {
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
          for (int r = 0; r < kStepRows; ++r)
            if ((uint32_t)r < nrows && ok_ct[ct]) {
              uint16_t *p = obase + ct * ct_stride + (size_t)r * P.OW;
#pragma unroll
              for (int e = 0; e < 8; ++e)
                if (ocol + e < P.OW) p[e] = (uint16_t)(pk[ct][r][e >> 1] >> ((e & 1) * 16));
            }
      }
    };
    auto load_old = [&](uint32_t row0, uint32_t nrows) {
      if (!BETA) return;
      const uint16_t *obase = olane + (size_t)row0 * P.OW;
#pragma unroll
      for (int ct = 0; ct < 2; ++ct)
#pragma unroll
        for (int r = 0; r < kStepRows; ++r) {
          old[ct][r] = (u32x4){0u, 0u, 0u, 0u};
          if ((uint32_t)r < nrows && ok_ct[ct]) {
            const uint16_t *p = obase + ct * ct_stride + (size_t)r * P.OW;
            if (full_cols) {
              old[ct][r] = *reinterpret_cast<const u32x4_unaligned *>(p);
            } else if (ocol < P.OW) {
#pragma unroll
              for (int e = 0; e < 8; ++e)
                if (ocol + e < P.OW) old[ct][r][e >> 1] |= (uint32_t)p[e] << ((e & 1) * 16);
            }
          }
        }
    };

    auto load_pin = [&](uint32_t row0, uint32_t nrows) {
      if (!PIN) return;
#pragma unroll
      for (int r = 0; r < kStepRows; ++r)
#pragma unroll
        for (int cti = 0; cti < 2; ++cti)
#pragma unroll
          for (int ct = 0; ct < 2; ++ct) {
            pin[r][cti][ct] = (floatx4){0.f, 0.f, 0.f, 0.f};
            if ((uint32_t)r < nrows && ok_ct[ct]) {
              const float *p = part_lane + ct * ct_stride + (size_t)(row0 + r) * P.OW + pcol[cti];
#pragma unroll
              for (int j = 0; j < 4; ++j)
                if (pcol[cti] + j < P.OW) pin[r][cti][ct][j] = p[j];
            }
          }
    };

    uint32_t sb = 0;  // ring slot of this step's first input row
    uint32_t prev_row0 = 0, prev_nrows = 0;

    // The matrix part of a step: 72 operand reads (input row, column shift, channel half, column
    // tile), each fetched kAhead reads before its MFMAs so that the LDS latency hides behind the
    // matrix pipe; then the results are packed to bf16.  kVm global-memory instructions and kLds
    // ring writes are spread over the rounds: issued in a burst they would fill the memory
    // pipeline's queue and hold every wave of the workgroup at the same point.
    // (row0, nrows, whole: where the sums of a POUT launch go; whole = every lane of the wave stores all of its
    // columns, rows and channel tiles)
    auto compute = [&](auto vm_tag, auto &&vm_op, auto lds_tag, auto &&lds_op, auto &&valu_op, uint32_t row0,
                       uint32_t nrows, bool whole) {
      constexpr int kVm = decltype(vm_tag)::value;
      constexpr int kLds = decltype(lds_tag)::value;
      floatx4 acc[kStepRows][2][2];
#pragma unroll
      for (int r = 0; r < kStepRows; ++r)
#pragma unroll
        for (int cti = 0; cti < 2; ++cti)
#pragma unroll
          for (int ct = 0; ct < 2; ++ct) acc[r][cti][ct] = (floatx4){0.f, 0.f, 0.f, 0.f};
      constexpr int kReads = (kStepRows + 2) * 12, kAhead = 3;
      uint32_t row_addr[kStepRows + 2];
#pragma unroll
      for (int ir = 0; ir < kStepRows + 2; ++ir) {
        uint32_t slot = sb + (uint32_t)ir;
        slot = slot >= (uint32_t)kRingRows ? slot - (uint32_t)kRingRows : slot;
        row_addr[ir] = slot * kRowPitch;
      }
      u32x4 pk_next[2][kStepRows];
      // packs output row r of this step to bf16 in store order
      auto pack_row = [&](auto rtag) {
        constexpr int r = decltype(rtag)::value;
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) {
          floatx4 v0 = acc[r][0][ct], v1 = acc[r][1][ct];
          if (PIN) {
            v0 += pin[r][0][ct];
            v1 += pin[r][1][ct];
          }
          if (BETA) {
            // back to the MFMA's arrangement: the swap is its own inverse
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
          if constexpr (POUT) {
            float *p0 = part_lane + ct * ct_stride + (size_t)(row0 + r) * P.OW + pcol[0];
            float *p1 = part_lane + ct * ct_stride + (size_t)(row0 + r) * P.OW + pcol[1];
            if (whole) {
              *reinterpret_cast<floatx4_a4 *>(p0) = v0;
              *reinterpret_cast<floatx4_a4 *>(p1) = v1;
            } else if ((uint32_t)r < nrows && ok_ct[ct]) {
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                if (pcol[0] + j < P.OW) p0[j] = v0[j];
                if (pcol[1] + j < P.OW) p1[j] = v1[j];
              }
            }
            continue;
          }
          const u32x2 q0 = __builtin_amdgcn_permlane16_swap(pack_bf16x2(v0[0], v0[1]), pack_bf16x2(v1[0], v1[1]), false, false);
          const u32x2 q1 = __builtin_amdgcn_permlane16_swap(pack_bf16x2(v0[2], v0[3]), pack_bf16x2(v1[2], v1[3]), false, false);
          pk_next[ct][r] = (u32x4){q0[0], q1[0], q0[1], q1[1]};
        }
      };
      u32x4 abuf[kAhead + 1];
      auto fetch = [&](int t) {
        const int ir = t / 12, kw = (t % 12) >> 2, half = (t >> 1) & 1, cti = t & 1;
        abuf[t % (kAhead + 1)] =
            *reinterpret_cast<const u32x4 *>(ring + row_addr[ir] + read_lane_off[cti][kw] + half * 64);
      };
#pragma unroll
      for (int t = 0; t < kAhead; ++t) fetch(t);
      __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
      auto round = [&](auto tag) {
        constexpr int t = decltype(tag)::value;
        if constexpr (t + kAhead < kReads) {
          fetch(t + kAhead);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        constexpr int ir = t / 12, kw = (t % 12) >> 2, half = (t >> 1) & 1, cti = t & 1;
        const bf16x8 a = __builtin_bit_cast(bf16x8, abuf[t % (kAhead + 1)]);
        constexpr int kh_lo = ir - (kStepRows - 1) > 0 ? ir - (kStepRows - 1) : 0;
        constexpr int kh_hi = ir < 2 ? ir : 2;
#pragma unroll
        for (int kh = kh_lo; kh <= kh_hi; ++kh) {
#pragma unroll
          for (int ct = 0; ct < 2; ++ct)
            acc[ir - kh][cti][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                a, __builtin_bit_cast(bf16x8, wreg[kh * 3 + kw][half][ct]), acc[ir - kh][cti][ct], 0, 0, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * (kh_hi - kh_lo + 1), 0);
        // Rounds 0..3: the four pieces of the transposition of the rows loaded a step ago (they
        // read the registers the loads below refill).  Ring write w goes after round 6 w + 4,
        // memory instruction i after round 4 + floor(i * (kReads - 4) / kVm).
        if constexpr (kLds > 0 && t < 4) valu_op(IntTag<t>());
        if constexpr (t >= 4 && (t - 4) % 6 == 0 && (t - 4) / 6 < kLds) {
          lds_op(IntTag<(t - 4) / 6>());
          __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
        if constexpr (kVm > 0 && t >= 4) {
          constexpr int span = kReads - 4, u = t - 4;
          constexpr int i = (u * kVm + span - 1) / span;  // first i with i * span >= u * kVm
          if constexpr (i < kVm && (i * span) / kVm == u) {
            vm_op(IntTag<i>());
            __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
          }
        }
        // an output row is complete once the input row two below it has been through; its
        // packing is dealt out over the next rounds
      };
      for_each_int(std::make_integer_sequence<int, kReads>(), round);
      __builtin_amdgcn_sched_barrier(0);
      for_each_int(std::make_integer_sequence<int, kStepRows>(), pack_row);
      // pk itself is still being stored while the rounds run
#pragma unroll
      for (int ct = 0; ct < 2; ++ct)
#pragma unroll
        for (int r = 0; r < kStepRows; ++r) pk[ct][r] = pk_next[ct][r];
    };

    // One step.  The rows of step s + 1, requested a whole step ago, are turned into ring order
    // first (they go to slots this step does not read); then the rows of step s + 2 are
    // requested.  Every wait on memory therefore only covers requests that are a step old.
    for (uint32_t s = 0; s < nsteps; ++s) {
      const bool more = s + 1 < nsteps, more2 = s + 2 < nsteps;
      const int32_t next_row0 = (int32_t)((s + 1) * kStepRows) + 2;
      const uint32_t row0 = r_begin + s * kStepRows;
      const uint32_t nrows = r_end - row0;  // rows >= nrows of this step do not exist
      const bool fast = lanes_whole && s > 0 && nrows >= (uint32_t)kStepRows;
      Transposed T;
      if (fast)
        transpose_prepare(next_row0, L0, T);  // transposed and written to the ring between the MFMAs below
      else if (more)
        commit(next_row0, L0);
      // Everything still in flight here (the previous step's stores) is a step old.  Draining it
      // explicitly keeps the compiler from guarding register reuse further down with waits that
      // would also cover the requests this step is about to issue.
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      if (fast) {
        // straight-line variant: every memory instruction is unconditional (rows requested
        // past the end of the segment are never used)
        uint16_t *const sbase = olane + (size_t)prev_row0 * P.OW;
        const uint16_t *const obase = olane + (size_t)row0 * P.OW;
        const float *const pbase = part_lane + (size_t)row0 * P.OW;
        // the memory instructions of a step, in issue order: the sums of the earlier launches and the old output
        // (both needed when the rows are packed), the rows of the step after next, the previous step's stores
        constexpr int kPinN = PIN ? 4 * kStepRows : 0, kOldN = BETA ? 2 * kStepRows : 0, kStoreN = POUT ? 0 : 2 * kStepRows;
        compute(IntTag<kPinN + kOldN + 9 + kStoreN>(), [&](auto tag) {
          constexpr int t = decltype(tag)::value;
          if constexpr (t < kPinN) {
            constexpr int ct = t & 1, cti = (t >> 1) & 1, r = t >> 2;
            pin[r][cti][ct] = *reinterpret_cast<const floatx4_a4 *>(pbase + ct * ct_stride + (size_t)r * P.OW + pcol[cti]);
          } else if constexpr (t < kPinN + kOldN) {
            constexpr int u = t - kPinN;
            constexpr int ct = u & 1, r = u >> 1;
            old[ct][r] = *reinterpret_cast<const u32x4_unaligned *>(obase + ct * ct_stride + (size_t)r * P.OW);
          } else if constexpr (t < kPinN + kOldN + 9) {
            load_one(IntTag<t - kPinN - kOldN>(), next_row0 + kStepRows, L0);
          } else {
            constexpr int u = t - kPinN - kOldN - 9;
            constexpr int ct = u / kStepRows, r = u % kStepRows;
            *reinterpret_cast<u32x4_unaligned *>(sbase + ct * ct_stride + (size_t)r * P.OW) = pk[ct][r];
          }
        }, IntTag<10>(), [&](auto tag) { ring_write(tag, T); }, [&](auto tag) { transpose_piece(tag, L0, T); }, row0, nrows, true);
      } else {
        if (more2) issue(next_row0 + kStepRows, L0);
        if (!POUT && s > 0) store_packed(prev_row0, prev_nrows);
        load_old(row0, nrows);
        load_pin(row0, nrows);
        compute(IntTag<0>(), [](auto) {}, IntTag<0>(), [](auto) {}, [](auto) {}, row0, nrows, false);
      }
      prev_row0 = row0;
      prev_nrows = nrows;
      __syncthreads();
      sb += kStepRows;
      sb = sb >= (uint32_t)kRingRows ? sb - (uint32_t)kRingRows : sb;
    }
    if (!POUT) store_packed(prev_row0, prev_nrows);
  }
}

static int g_num_cus = 0;
static int num_cus() {
  if (g_num_cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      g_num_cus = n;
    else
      g_num_cus = 256;
  }
  return g_num_cus;
}

// Up to 64 reduction channels: any shape.  More: several launches with fp32 sums between them, which the
// eight-wave kernels address through a buffer resource: the sums of one image have to lie inside 2 GiB.
// (The eight-wave kernels need rows on a 4-byte boundary (forward: even width) or whole 16-byte granules
// (backward-data: a width that is a multiple of 8) and aligned tiles; other shapes take the four-wave kernel
// once per 64 reduction channels.)
bool conv_bf16_mfma_supported(int which, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W) {
  const uint32_t cred = which == ADH_CONV_FWD ? Cin : Cout;
  if (cred <= 64u) return true;
  const uint32_t cout_k = which == ADH_CONV_FWD ? Cout : Cin;
  const uint64_t oh = which == ADH_CONV_FWD ? H : H + 2ull, ow = which == ADH_CONV_FWD ? W : W + 2ull;
  return cout_k * oh * ow * 4u < (1ull << 31);
}
// widths whose rows the eight-wave kernels take
static bool conv_bf16_w8_width(int which, uint32_t W) { return which == ADH_CONV_FWD ? (W % 2u) == 0u : (W % 8u) == 0u; }
static uint32_t conv_bf16_passes(int which, uint32_t Cin, uint32_t Cout) {
  return ((which == ADH_CONV_FWD ? Cin : Cout) + 63u) / 64u;
}
// More than 64 reduction AND more than 64 output channels: launches of 128 reduction channels by the kernel of
// conv3x3_bf16_k128.hip while more than 64 are left, then at most 64 by the eight-wave kernel.  Otherwise one
// launch of the eight-wave kernel per 64.
static bool conv_bf16_uses_k128(int which, uint32_t Cin, uint32_t Cout) { return Cin > 64u && Cout > 64u; }
// (a width the eight-wave kernels do not take: one launch of the four-wave kernel per 64)
static uint32_t conv_bf16_launches(int which, uint32_t Cin, uint32_t Cout, uint32_t W) {
  const uint32_t cred = which == ADH_CONV_FWD ? Cin : Cout;
  if (!conv_bf16_uses_k128(which, Cin, Cout) || !conv_bf16_w8_width(which, W)) return (cred + 63u) / 64u;
  uint32_t n = 0, rem = cred;
  while (rem > 64u) {
    rem -= rem < 128u ? rem : 128u;
    ++n;
  }
  return n + (rem ? 1u : 0u);
}

// name of the kernel a bf16 forward / backward-data call over padded tiles runs, for tiles aligned to 16 bytes
// (template arguments: old output added, sums of earlier passes read, sums written for a later pass, tiles without halo)
const char *conv_bf16_kernel_name(int which, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W, float beta) {
  if (!conv_bf16_mfma_supported(which, Cin, Cout, H, W)) return "widen_bf16_kernel + conv3x3_f32_kernel + narrow_bf16_kernel";
  if (!conv_bf16_w8_width(which, W)) {
    if (conv_bf16_passes(which, Cin, Cout) > 1u)
      return beta != 0.f ? "conv3x3_bf16_kernel<true, false, true> + <false, true, true> per middle 64 reduction channels + <false, true, false>"
                         : "conv3x3_bf16_kernel<false, false, true> + <false, true, true> per middle 64 reduction channels + <false, true, false>";
    return beta != 0.f ? "conv3x3_bf16_kernel<true, false, false>" : "conv3x3_bf16_kernel<false, false, false>";
  }
  if (conv_bf16_uses_k128(which, Cin, Cout)) {
    if (conv_bf16_launches(which, Cin, Cout, W) == 1u)
      return beta != 0.f ? "conv3x3_bf16_k128_kernel<true, false, false, false>" : "conv3x3_bf16_k128_kernel<false, false, false, false>";
    return "conv3x3_bf16_k128_kernel per 128 reduction channels (fp32 sums between the launches) + conv3x3_bf16_w8_kernel for a rest of at most 64";
  }
  if (conv_bf16_passes(which, Cin, Cout) > 1u)
    return beta != 0.f ? "conv3x3_bf16_w8_kernel<true, false, true, false> + <false, true, true, false> per middle pass + <false, true, false, false>"
                       : "conv3x3_bf16_w8_kernel<false, false, true, false> + <false, true, true, false> per middle pass + <false, true, false, false>";
  return beta != 0.f ? "conv3x3_bf16_w8_kernel<true, false, false, false>" : "conv3x3_bf16_w8_kernel<false, false, false, false>";
}

// the four-wave kernel over the reduction channels P.chan0 .. P.chan0 + P.cred_pass - 1
static int conv_bf16_w4_launch(const ConvBf16Params &P, uint32_t gx, uint32_t groups, hipStream_t st) {
  const dim3 grid(gx, groups), block(256);
  const bool first = P.first_pass != 0u, last = P.last_pass != 0u, beta = P.beta != 0.f;
  if (!(first && last) && !P.part[0]) return ADH_ENULL;  // sums between launches need their buffers
  if (first && last) {
    if (beta) hipLaunchKernelGGL((conv3x3_bf16_kernel<true, false, false>), grid, block, 0, st, P);
    else hipLaunchKernelGGL((conv3x3_bf16_kernel<false, false, false>), grid, block, 0, st, P);
  } else if (first) {
    if (beta) hipLaunchKernelGGL((conv3x3_bf16_kernel<true, false, true>), grid, block, 0, st, P);
    else hipLaunchKernelGGL((conv3x3_bf16_kernel<false, false, true>), grid, block, 0, st, P);
  } else if (!last) {
    hipLaunchKernelGGL((conv3x3_bf16_kernel<false, true, true>), grid, block, 0, st, P);
  } else {
    hipLaunchKernelGGL((conv3x3_bf16_kernel<false, true, false>), grid, block, 0, st, P);
  }
  return launch_status();
}

// the reordered filter, then (more than one pass) the fp32 sums of every tile, each region 256-byte aligned
static size_t filter_region_bytes(int which, uint32_t Cin, uint32_t Cout) {
  const uint32_t cout_k = which == ADH_CONV_FWD ? Cout : Cin;
  return (size_t)((cout_k + 63u) / 64u) * conv_bf16_passes(which, Cin, Cout) * kWtGroupElems * 2u;
}
static size_t part_region_bytes(int which, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W) {
  const uint64_t cout_k = which == ADH_CONV_FWD ? Cout : Cin;
  const uint64_t oh = which == ADH_CONV_FWD ? H : H + 2ull, ow = which == ADH_CONV_FWD ? W : W + 2ull;
  return (size_t)((N * cout_k * oh * ow * 4u + 255u) / 256u * 256u);
}
size_t conv_bf16_mfma_workspace_bytes(int which, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H,
                                      uint32_t W) {
  size_t bytes = filter_region_bytes(which, Cin, Cout);
  if (conv_bf16_launches(which, Cin, Cout, W) > 1u) bytes += (size_t)num_tiles * part_region_bytes(which, N, Cin, Cout, H, W);
  return bytes;
}

// which = ADH_CONV_FWD: in = x_pad tiles, out = y tiles; ADH_CONV_BWD_DATA: in = dy tiles,
// out = dx_pad tiles.  Arguments are validated by the caller.
// halofree: no tile carries a halo (in and out are H x W), the tiles are the row tiles of one tensor in rank order
// and a tile's rows -1 and H are its neighbours' last and first rows (zeros at the tensor's own border): the
// unsplit convolution with zero padding, restricted to the tile.  Only shapes the eight-wave kernel takes
// (ADH_EUNIMPL otherwise).
int conv_bf16_mfma(int which, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                   const void *const *in_tiles, const void *w, void *const *out_tiles, float beta, void *workspace,
                   hipStream_t st, bool halofree) {
  ConvBf16Params P = {};
  for (uint32_t t = 0; t < num_tiles; ++t) {
    P.in[t] = reinterpret_cast<const uint16_t *>(in_tiles[t]);
    P.out[t] = reinterpret_cast<uint16_t *>(out_tiles[t]);
  }
  P.wt = reinterpret_cast<const uint16_t *>(workspace);
  P.N = N;
  P.beta = beta;
  if (which == ADH_CONV_FWD) {
    P.Cred = Cin; P.Cout = Cout;
    P.IH = H + 2; P.IW = W + 2; P.OH = H; P.OW = W;
    P.pad = 0;
  } else {
    P.Cred = Cout; P.Cout = Cin;
    P.IH = H; P.IW = W; P.OH = H + 2; P.OW = W + 2;
    P.pad = 2;
  }
  if (halofree) {
    P.IH = P.OH = H; P.IW = P.OW = W;
    P.pad = 1;
    P.neighbour_rows = 1;
    P.num_tiles = num_tiles;
  }
  const uint32_t groups = (P.Cout + 63u) / 64u;
  P.passes = conv_bf16_passes(which, Cin, Cout);
  P.pass = 0;
  P.chan0 = 0;
  P.cred_pass = P.Cred < 64u ? P.Cred : 64u;
  P.first_pass = P.last_pass = 1;
  const uint32_t launches = conv_bf16_launches(which, Cin, Cout, W);
  if (launches > 1u) {
    uint8_t *part = reinterpret_cast<uint8_t *>(workspace) + filter_region_bytes(which, Cin, Cout);
    const size_t per_tile = part_region_bytes(which, N, Cin, Cout, H, W);
    for (uint32_t t = 0; t < num_tiles; ++t) P.part[t] = reinterpret_cast<float *>(part + t * per_tile);
  }
  if (halofree && !conv_bf16_w8_takes(P, num_tiles)) return ADH_EUNIMPL;
  // the forward pass of the eight-wave kernel can read the caller's filter itself
  const bool direct = which == ADH_CONV_FWD && (Cin % 64u) == 0u && aligned_to(w, 16) && (P.IW % 2u) == 0u;
  int e = ADH_OK;
  if (!direct) {
    const uint32_t total = groups * P.passes * kWtGroupElems;
    hipLaunchKernelGGL(conv3x3_bf16_filter_kernel, dim3((total + 255u) / 256u), dim3(256), 0, st,
                       reinterpret_cast<const uint16_t *>(w), reinterpret_cast<uint16_t *>(workspace), Cin, Cout,
                       which == ADH_CONV_FWD ? 0u : 1u, P.passes, total);
    e = launch_status();
    if (e) return e;
  }

  const uint32_t cus = (uint32_t)num_cus();
  // work items and their division among `gx` persistent workgroups per group of output channels, for strips of
  // `strip_cols` columns
  auto plan = [&](uint32_t strip_cols, uint32_t out_groups, uint32_t min_seg_steps, uint32_t *gx_out) -> int {
    P.strips = (P.OW + strip_cols - 1) / strip_cols;
    const uint64_t base_items = (uint64_t)N * num_tiles * P.strips;
    if (base_items >= (1ull << 30)) return ADH_EINVAL;
    P.items = (uint32_t)base_items;
    P.steps_per_item = (P.OH + kStepRows - 1) / kStepRows;
    uint32_t gx = cus / out_groups ? cus / out_groups : 1u;
    if (gx > P.items * P.steps_per_item) gx = P.items * P.steps_per_item;
    // whole items while they go round evenly; the rest in row segments of at least `min_seg_steps` steps
    // (a segment re-reads two input rows and pays for filling the ring again)
    P.whole_items = P.items / gx * gx;
    const uint32_t rest = P.items - P.whole_items;
    P.seg_steps = P.steps_per_item;
    P.segs = 1;
    if (rest) {
      const uint32_t want_segs = gx / rest;  // >= 1
      uint32_t seg_steps = (P.steps_per_item + want_segs - 1) / want_segs;
      if (seg_steps < min_seg_steps) seg_steps = P.steps_per_item < min_seg_steps ? P.steps_per_item : min_seg_steps;
      P.seg_steps = seg_steps;
      P.segs = (P.steps_per_item + seg_steps - 1) / seg_steps;
    }
    P.pieces = rest * P.segs;
    P.div_strips = FastDiv(P.strips);
    P.div_N = FastDiv(N);
    P.div_rest = FastDiv(rest ? rest : 1u);
    *gx_out = gx;
    return ADH_OK;
  };
  const bool w8 = conv_bf16_w8_takes(P, num_tiles);
  uint32_t gx = 0;
  // the eight-wave kernel starts an item with one step without MFMAs; the four-wave one fills its ring first
  e = plan(kStripCols, groups, w8 ? 2u : 4u, &gx);
  if (e) return e;
  if (direct && w8) {
    P.w_direct = reinterpret_cast<const uint16_t *>(w);
  } else if (direct) {
    // the four-wave kernel takes this shape after all (tile alignment): it needs the transformed copy
    const uint32_t total = groups * P.passes * kWtGroupElems;
    hipLaunchKernelGGL(conv3x3_bf16_filter_kernel, dim3((total + 255u) / 256u), dim3(256), 0, st,
                       reinterpret_cast<const uint16_t *>(w), reinterpret_cast<uint16_t *>(workspace), Cin, Cout, 0u,
                       P.passes, total);
    e = launch_status();
    if (e) return e;
  }
  if (P.passes > 1u) {
    if (!w8) {
      // odd widths, tiles off the eight-wave kernels' alignment: the four-wave kernel once per 64 channels.  The
      // workspace holds the sums between the launches unless the width promised one launch of 128 channels: then
      // it is the tiles' alignment that keeps the eight-wave kernels away, and there is no room for the sums.
      if (launches <= 1u) return ADH_EALIGN;
      for (uint32_t pass = 0; pass < P.passes; ++pass) {
        ConvBf16Params Q = P;
        Q.pass = pass;
        Q.chan0 = 64u * pass;
        Q.cred_pass = P.Cred - Q.chan0 < 64u ? P.Cred - Q.chan0 : 64u;
        Q.first_pass = pass == 0u ? 1u : 0u;
        Q.last_pass = pass + 1u == P.passes ? 1u : 0u;
        e = conv_bf16_w4_launch(Q, gx, groups, st);
        if (e) return e;
      }
      return ADH_OK;
    }
    const bool k128 = conv_bf16_uses_k128(which, Cin, Cout) && conv_bf16_k128_takes(P, num_tiles);
    uint32_t gx128 = 0;
    const uint32_t groups128 = (P.Cout + 127u) / 128u;
    const ConvBf16Params plan64 = P;  // the plan for 64-column strips, kept for a last launch of at most 64 channels
    if (k128) {
      e = plan(kStripColsK128, groups128, 2u, &gx128);
      if (e) return e;
    }
    ConvBf16Params plan128 = P;
    uint32_t chan = 0, launch = 0;
    while (chan < P.Cred) {
      const uint32_t rem = P.Cred - chan;
      const bool wide = k128 && rem > 64u;
      ConvBf16Params Q = wide ? plan128 : plan64;
      Q.chan0 = chan;
      Q.pass = chan / 64u;
      Q.cred_pass = wide ? (rem < 128u ? rem : 128u) : (rem < 64u ? rem : 64u);
      Q.first_pass = launch == 0u ? 1u : 0u;
      Q.last_pass = chan + Q.cred_pass >= P.Cred ? 1u : 0u;
      e = wide ? conv_bf16_k128_launch(Q, gx128, groups128, st) : conv_bf16_w8_launch(Q, gx, groups, st);
      if (e) return e;
      chan += Q.cred_pass;
      ++launch;
    }
    return ADH_OK;
  }
  if (conv_bf16_w8_takes(P, num_tiles)) return conv_bf16_w8_launch(P, gx, groups, st);
  return conv_bf16_w4_launch(P, gx, groups, st);
}

}  // namespace adh

// ---------------------------------------------------------------------------
// the forward entry point that allocates nothing
// ---------------------------------------------------------------------------
namespace {

constexpr uint32_t kStaticGroups = 4;  // reordered filter of up to 256 output channels
constexpr size_t kStaticScratchBytes = (size_t)kStaticGroups * adh::kWtGroupElems * 2u;  // 294,912 bytes
constexpr int kStaticMaxDevices = 64;

// The reordered filter of adh_conv3x3_slab_fwd_tiles_static lives here instead of in a caller's
// workspace.  Every GPU the library runs on holds its own copy of the array until the process ends.
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

// Device address of `scratch` on each device, looked up once per device with that device current.
// In host code the array's name is only a handle for this lookup, never a device address.
static void *g_scratch_ptr[kStaticMaxDevices];
static int g_scratch_lock = 0;

static int static_scratch(void **out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kStaticMaxDevices) return ADH_EINVAL;
  while (__atomic_exchange_n(&g_scratch_lock, 1, __ATOMIC_ACQUIRE)) {
  }
  void *p = g_scratch_ptr[dev];
  int status = ADH_OK;
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      status = e != hipSuccess ? (int)e : ADH_ENULL;
      p = nullptr;
    } else {
      g_scratch_ptr[dev] = p;
    }
  }
  __atomic_store_n(&g_scratch_lock, 0, __ATOMIC_RELEASE);
  *out = p;
  return status;
}

}  // namespace

extern "C" int adh_conv3x3_slab_fwd_tiles_static(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                                 uint32_t H, uint32_t W, const void *const *x_pad_tiles,
                                                 const void *w, void *const *y_tiles, float beta, void *stream) {
  using namespace adh;
  if (dtype != ADH_BF16) return ADH_EUNIMPL;
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  // beyond the static array: more than 256 output channels; beyond the matrix-core kernel: more than 64 input channels
  if (Cout > 64u * kStaticGroups || Cin > 64u) return ADH_EWORKSPACE;
  if (N == 0 || Cin == 0 || Cout == 0 || H == 0 || W == 0) return ADH_OK;
  if (!x_pad_tiles || !y_tiles || !w) return ADH_ENULL;
  if (!aligned_to(w, 2)) return ADH_EALIGN;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!x_pad_tiles[t] || !y_tiles[t]) return ADH_ENULL;
    if (!aligned_to(x_pad_tiles[t], 2) || !aligned_to(y_tiles[t], 2)) return ADH_EALIGN;
  }
  const uint64_t cmax = Cin > Cout ? Cin : Cout;
  if (cmax * (H + 2ull) * (W + 2ull) * 2u >= (1ull << 31) || (uint64_t)Cin * Cout * 18u >= (1ull << 31)) return ADH_EINVAL;
  void *ws = nullptr;
  const int e = static_scratch(&ws);
  if (e) return e;
  return conv_bf16_mfma(ADH_CONV_FWD, num_tiles, N, Cin, Cout, H, W, x_pad_tiles, w, y_tiles, beta, ws, as_stream(stream),
                        false);
}

// ---------------------------------------------------------------------------
// convolution over row tiles that carry no halo (bf16; the entry points are in conv3x3.hip)
// ---------------------------------------------------------------------------
namespace adh {
int conv_bf16_unpadded(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                       const void *const *in_tiles, const void *w, void *const *out_tiles, float beta, void *workspace,
                       size_t workspace_bytes, hipStream_t st) {
  if (!dtype_ok(dtype)) return ADH_EINVAL;
  if (dtype != ADH_BF16) return ADH_EUNIMPL;
  if (num_tiles == 0 || num_tiles > ADH_MAX_TILES) return ADH_EINVAL;
  if (beta != 0.f && beta != 1.f) return ADH_EINVAL;
  if (N == 0 || Cin == 0 || Cout == 0 || H == 0 || W == 0) return ADH_OK;
  if (!in_tiles || !out_tiles || !w) return ADH_ENULL;
  if ((W % 8u) != 0u) return ADH_EUNIMPL;  // whole 16-byte granules per row
  if (!aligned_to(w, 2)) return ADH_EALIGN;
  for (uint32_t t = 0; t < num_tiles; ++t) {
    if (!in_tiles[t] || !out_tiles[t]) return ADH_ENULL;
    if (!aligned_to(in_tiles[t], 16) || !aligned_to(out_tiles[t], 4)) return ADH_EALIGN;
  }
  const uint64_t cmax = Cin > Cout ? Cin : Cout;
  if (cmax * (H + 2ull) * (W + 2ull) * 2u >= (1ull << 31) || (uint64_t)Cin * Cout * 18u >= (1ull << 31)) return ADH_EINVAL;
  if (!conv_bf16_mfma_supported(which, Cin, Cout, H, W)) return ADH_EUNIMPL;
  // the same workspace as the padded entry point of this pass (the transformed filter; the sums between passes)
  const size_t need = conv_bf16_mfma_workspace_bytes(which, num_tiles, N, Cin, Cout, H, W);
  if (!workspace) return ADH_ENULL;
  if (!aligned_to(workspace, 256)) return ADH_EALIGN;
  if (workspace_bytes < need) return ADH_EWORKSPACE;
  return conv_bf16_mfma(which, num_tiles, N, Cin, Cout, H, W, in_tiles, w, out_tiles, beta, workspace, st, true);
}
}  // namespace adh
