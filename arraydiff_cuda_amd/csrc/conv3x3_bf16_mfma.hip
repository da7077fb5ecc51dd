// 3x3 slab convolution on the bf16 matrix cores (v_mfma_f32_16x16x32_bf16), forward and
// backward-data, for up to 64 reduction channels.
//
// Shape of the computation.  A workgroup of four waves is persistent: it walks work items
// (image, 32-column strip, row segment) and, inside an item, steps down the strip eight output
// rows at a time.  The input rows of the strip live in LDS as a ring of 18 rows in
// [pixel][channel] order (144 bytes per pixel: 64 channels + 16 bytes of padding, which makes the
// 16-byte operand reads of 16 neighbouring pixels hit 64 distinct banks), so each input row is
// fetched from HBM exactly once per strip; only the one-pixel column halo of a strip is read twice.
// NCHW rows are turned into that order on the way in: a thread loads eight channels x eight
// pixels (eight 16-byte buffer loads), transposes the 8x8 block of 16-bit values with byte
// permutes and writes eight 16-byte LDS rows.
//
// A wave owns 32 output channels x 16 columns x 8 rows.  Its share of the filter, 9 taps x 64
// reduction channels x 32 output channels, is loaded once per kernel into 144 registers in matrix
// operand order and never touches LDS.  Per step a wave reads 10 input rows x 3 column shifts x
// 2 channel halves = 60 pixel operands and issues 288 MFMAs: an operand read for input row r
// serves the output rows r, r-1, r-2 (taps kh = 0, 1, 2).
//
// Out-of-range rows, channels and buffer ends are handled by the buffer resource's range check
// (out-of-range dwords read as zero); out-of-range columns by per-dword masks.
#include "adh_common.h"

namespace adh {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef u32x2 u32x2_unaligned __attribute__((aligned(2)));

constexpr int kStripCols = 32;                        // output columns per work item
constexpr int kStepRows = 8;                          // output rows per step
constexpr int kRingRows = 18;                         // 10 rows in use + 8 rows in flight
constexpr int kPatchCols = kStripCols + 2;            // 34
constexpr int kPxPitch = 144;                         // bytes per pixel in LDS
constexpr int kRowPitch = kPatchCols * kPxPitch;      // 4896
constexpr int kRingBytes = kRingRows * kRowPitch;     // 88128
constexpr uint32_t kOutOfRange = 0x80000000u;
constexpr uint32_t kWtGroupElems = 9u * 2u * 64u * 32u;  // transformed filter elements per group of 64 outputs

struct ConvBf16Params {
  const uint16_t *in[ADH_MAX_TILES];
  uint16_t *out[ADH_MAX_TILES];
  const uint16_t *wt;       // transformed filter: [group][tap][half][64 out][32 red]
  uint32_t N, Cred, Cout;   // reduction and output channel counts as the kernel sees them
  uint32_t IH, IW, OH, OW;
  int32_t pad;              // input row/col = output row/col + tap - pad
  float beta;
  uint32_t strips, segs, seg_rows, items;
  FastDiv div_strips, div_segs, div_N;
};

// filter (Cout, Cin, 3, 3) -> matrix-operand order.  flip = 0 (forward): out = Cout index,
// red = Cin index, tap as is.  flip = 1 (backward-data): out = Cin index, red = Cout index,
// tap mirrored.  Channels beyond the real extents are zero.
__global__ __launch_bounds__(256) void conv3x3_bf16_filter_kernel(const uint16_t *__restrict__ w, uint16_t *__restrict__ wt,
                                                                  uint32_t Cin, uint32_t Cout, uint32_t flip,
                                                                  uint32_t total) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i >= total) return;
  const uint32_t r = i & 31u, o = (i >> 5) & 63u, half = (i >> 11) & 1u;
  const uint32_t tg = i >> 12, tap = tg % 9u, grp = tg / 9u;
  const uint32_t oc = grp * 64u + o, rc = half * 32u + r;
  uint16_t v = 0;
  if (!flip) {
    if (oc < Cout && rc < Cin) v = w[((uint64_t)oc * Cin + rc) * 9u + tap];
  } else {
    if (oc < Cin && rc < Cout) v = w[((uint64_t)rc * Cin + oc) * 9u + (8u - tap)];
  }
  wt[i] = v;
}

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  return (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
}

__global__ __launch_bounds__(256, 1) void conv3x3_bf16_kernel(ConvBf16Params P) {
  __shared__ __attribute__((aligned(16))) uint8_t ring[kRingBytes];

  const uint32_t tid = threadIdx.x;
  const uint32_t lane = tid & 63u, l16 = lane & 15u, g = lane >> 4;
  const uint32_t wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t h = wv & 1u, cb = wv >> 1;
  const uint32_t grp = blockIdx.y;

  // this wave's filter share, in B-operand order: lane (n = l16, k-block = g)
  u32x4 wreg[9][2][2];
  {
    const u32x4 *wt = reinterpret_cast<const u32x4 *>(P.wt + (size_t)grp * kWtGroupElems);
#pragma unroll
    for (int tap = 0; tap < 9; ++tap)
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
          wreg[tap][half][ct] = wt[((tap * 2 + half) * 64 + (int)(32u * h + 16u * ct + l16)) * 4 + (int)g];
  }

  // loader role of this thread: one input row, eight channels, eight pixels
  const uint32_t lrow = tid >> 5, chg = (tid >> 2) & 7u, pxb = tid & 3u;
  const uint32_t plane_bytes = P.IH * P.IW * 2u;
  const uint32_t image_bytes = P.Cred * plane_bytes;
  uint32_t chvalid = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) chvalid |= (chg * 8u + j < P.Cred ? 1u : 0u) << j;

  const uint32_t read_lane_base = (16u * cb + l16) * kPxPitch + g * 16u;

  for (uint32_t item = blockIdx.x; item < P.items; item += gridDim.x) {
    uint32_t strip, t1, seg, plane, tile, n;
    P.div_strips.divmod(item, t1, strip);
    P.div_segs.divmod(t1, plane, seg);
    P.div_N.divmod(plane, tile, n);
    const int32_t c0 = (int32_t)(strip * kStripCols);
    const uint32_t r_begin = seg * P.seg_rows;
    const uint32_t r_end = r_begin + P.seg_rows < P.OH ? r_begin + P.seg_rows : P.OH;
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
    const int32_t tcol0 = c0 - P.pad + kStripCols;  // tail pixels 32, 33
    const uint32_t mt = ((tcol0 >= 0 && tcol0 < (int32_t)P.IW) ? 0x0000ffffu : 0u) |
                        ((tcol0 + 1 >= 0 && tcol0 + 1 < (int32_t)P.IW) ? 0xffff0000u : 0u);
    const int32_t arow0 = (int32_t)r_begin - P.pad;  // input row of ring-relative row 0
    // byte offset of (channel chg*8, input row arow0 + lrow, column icol0); may be negative
    const int32_t vbase = (int32_t)((chg * 8u * P.IH) * P.IW * 2u) + ((arow0 + (int32_t)lrow) * (int32_t)P.IW + icol0) * 2;
    const int32_t tbase = vbase + (tcol0 - icol0) * 2;

    u32x4 ld[8];
    uint32_t lt[8];

    auto issue = [&](int32_t row0) {
      const int32_t i = row0 + (int32_t)lrow;
      const int32_t arow = arow0 + i;
      const bool ok = i >= 0 && arow >= 0 && arow < (int32_t)P.IH;
      const uint32_t v = (uint32_t)(vbase + row0 * (int32_t)P.IW * 2);
      const uint32_t t = (uint32_t)(tbase + row0 * (int32_t)P.IW * 2);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const bool okj = ok && ((chvalid >> j) & 1u);
        ld[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, okj ? v + (uint32_t)j * plane_bytes : kOutOfRange, 0, 0);
      }
      if (pxb == 0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const bool okj = ok && ((chvalid >> j) & 1u);
          lt[j] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, okj ? t + (uint32_t)j * plane_bytes : kOutOfRange, 0, 0);
        }
      }
    };

    auto commit = [&](int32_t row0) {
      const int32_t i = row0 + (int32_t)lrow;
      if (i < 0) return;
      // The range check drops a dword that straddles the end of the image even though its low
      // half is the image's last element: fetch that element on its own.
      {
        const int32_t arow = arow0 + i;
        // A load that starts left of the image's first element (first row of channel 0, left
        // column halo) has a negative offset and is dropped as a whole: redo it dword by dword.
        // icol0 is a multiple of two pixels below zero, so the in-range part starts on a dword.
        if (arow == 0 && chg == 0 && icol0 < 0 && (chvalid & 1u)) {
          const int32_t v = vbase + row0 * (int32_t)P.IW * 2;
#pragma unroll
          for (int d = 0; d < 4; ++d)
            ld[0][d] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, v + 4 * d >= 0 ? (uint32_t)(v + 4 * d) : kOutOfRange, 0, 0);
        }
        if (arow == (int32_t)P.IH - 1 && chg == (P.Cred - 1u) >> 3) {
          const uint32_t j = (P.Cred - 1u) & 7u;
          const uint32_t v = (uint32_t)(vbase + row0 * (int32_t)P.IW * 2) + j * plane_bytes;
          const uint32_t gap = image_bytes - 2u - v;  // distance of the last element from the load start
          if (gap < 16u && (gap & 3u) == 0u) {
            const uint32_t e = __builtin_amdgcn_raw_buffer_load_b16(rsrc, image_bytes - 2u, 0, 0) & 0xffffu;
            const uint32_t d = gap >> 2;
#pragma unroll
            for (int jj = 0; jj < 8; ++jj)
#pragma unroll
              for (int dd = 0; dd < 4; ++dd)
                if ((uint32_t)jj == j && (uint32_t)dd == d) ld[jj][dd] |= e;
          }
          if (pxb == 0) {
            const uint32_t t = (uint32_t)(tbase + row0 * (int32_t)P.IW * 2) + j * plane_bytes;
            if (t == image_bytes - 2u) {
              const uint32_t e = __builtin_amdgcn_raw_buffer_load_b16(rsrc, image_bytes - 2u, 0, 0) & 0xffffu;
#pragma unroll
              for (int jj = 0; jj < 8; ++jj)
                if ((uint32_t)jj == j) lt[jj] |= e;
            }
          }
        }
      }
      const uint32_t slot = (uint32_t)i % (uint32_t)kRingRows;
      uint8_t *dst = ring + slot * kRowPitch + (pxb * 8u) * kPxPitch + chg * 16u;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        u32x4 even, odd;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t lo = ld[2 * q][d] & md[d], hi = ld[2 * q + 1][d] & md[d];
          even[q] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
          odd[q] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);
        }
        *reinterpret_cast<u32x4 *>(dst + (2 * d) * kPxPitch) = even;
        *reinterpret_cast<u32x4 *>(dst + (2 * d + 1) * kPxPitch) = odd;
      }
      if (pxb == 0) {
        u32x4 even, odd;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t lo = lt[2 * q] & mt, hi = lt[2 * q + 1] & mt;
          even[q] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
          odd[q] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);
        }
        uint8_t *td = ring + slot * kRowPitch + kStripCols * kPxPitch + chg * 16u;
        *reinterpret_cast<u32x4 *>(td) = even;
        *reinterpret_cast<u32x4 *>(td + kPxPitch) = odd;
      }
    };

    // ring-relative rows 0..9 of the first step
    issue(2 - kStepRows);
    commit(2 - kStepRows);
    issue(2);
    commit(2);
    __syncthreads();

    uint32_t sb = 0;  // ring slot of this step's first input row
    for (uint32_t s = 0; s < nsteps; ++s) {
      const bool more = s + 1 < nsteps;
      const int32_t next_row0 = (int32_t)((s + 1) * kStepRows) + 2;
      if (more) issue(next_row0);

      floatx4 acc[kStepRows][2];
#pragma unroll
      for (int r = 0; r < kStepRows; ++r)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) acc[r][ct] = (floatx4){0.f, 0.f, 0.f, 0.f};

#pragma unroll
      for (int ir = 0; ir < kStepRows + 2; ++ir) {
        uint32_t slot = sb + (uint32_t)ir;
        slot = slot >= (uint32_t)kRingRows ? slot - (uint32_t)kRingRows : slot;
        const uint8_t *src = ring + slot * kRowPitch + read_lane_base;
#pragma unroll
        for (int kw = 0; kw < 3; ++kw) {
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const u32x4 a = *reinterpret_cast<const u32x4 *>(src + kw * kPxPitch + half * 64);
#pragma unroll
            for (int kh = 0; kh < 3; ++kh) {
              const int orow = ir - kh;
              if (orow < 0 || orow >= kStepRows) continue;
#pragma unroll
              for (int ct = 0; ct < 2; ++ct)
                acc[orow][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, wreg[kh * 3 + kw][half][ct]),
                    acc[orow][ct], 0, 0, 0);
            }
          }
        }
      }

      // results: lane (l16, g) holds output channel l16 of its tile, columns 4g..4g+3
      {
        const uint32_t col = (uint32_t)c0 + 16u * cb + 4u * g;
        const uint32_t row0 = r_begin + s * kStepRows;
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) {
          const uint32_t co = grp * 64u + 32u * h + 16u * ct + l16;
          if (co < P.Cout && col < P.OW) {
            uint16_t *orow_ptr = out_img + ((size_t)co * P.OH + row0) * P.OW + col;
            const bool full = col + 3u < P.OW;
#pragma unroll
            for (int r = 0; r < kStepRows; ++r) {
              if (row0 + r < r_end) {
                uint16_t *p = orow_ptr + (size_t)r * P.OW;
                floatx4 v = acc[r][ct];
                if (full) {
                  if (P.beta != 0.f) {
                    const u32x2 old = *reinterpret_cast<const u32x2_unaligned *>(p);
                    v[0] += __uint_as_float(old[0] << 16);
                    v[1] += __uint_as_float(old[0] & 0xffff0000u);
                    v[2] += __uint_as_float(old[1] << 16);
                    v[3] += __uint_as_float(old[1] & 0xffff0000u);
                  }
                  u32x2 o;
                  o[0] = pack_bf16x2(v[0], v[1]);
                  o[1] = pack_bf16x2(v[2], v[3]);
                  *reinterpret_cast<u32x2_unaligned *>(p) = o;
                } else {
#pragma unroll
                  for (int e = 0; e < 4; ++e)
                    if (col + e < P.OW) {
                      float f = v[e];
                      if (P.beta != 0.f) f += bf16_bits_to_f32(p[e]);
                      p[e] = f32_to_bf16_bits(f);
                    }
                }
              }
            }
          }
        }
      }

      if (more) commit(next_row0);
      __syncthreads();
      sb += kStepRows;
      sb = sb >= (uint32_t)kRingRows ? sb - (uint32_t)kRingRows : sb;
    }
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

bool conv_bf16_mfma_supported(int which, uint32_t Cin, uint32_t Cout) {
  const uint32_t cred = which == ADH_CONV_FWD ? Cin : Cout;
  return cred <= 64u;
}

size_t conv_bf16_mfma_workspace_bytes(int which, uint32_t Cin, uint32_t Cout) {
  const uint32_t cout_k = which == ADH_CONV_FWD ? Cout : Cin;
  return (size_t)((cout_k + 63u) / 64u) * kWtGroupElems * 2u;
}

// which = ADH_CONV_FWD: in = x_pad tiles, out = y tiles; ADH_CONV_BWD_DATA: in = dy tiles,
// out = dx_pad tiles.  Arguments are validated by the caller.
int conv_bf16_mfma(int which, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                   const void *const *in_tiles, const void *w, void *const *out_tiles, float beta, void *workspace,
                   hipStream_t st) {
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
  const uint32_t groups = (P.Cout + 63u) / 64u;
  const uint32_t total = groups * kWtGroupElems;
  hipLaunchKernelGGL(conv3x3_bf16_filter_kernel, dim3((total + 255u) / 256u), dim3(256), 0, st,
                     reinterpret_cast<const uint16_t *>(w), reinterpret_cast<uint16_t *>(workspace), Cin, Cout,
                     which == ADH_CONV_FWD ? 0u : 1u, total);
  int e = launch_status();
  if (e) return e;

  const uint32_t cus = (uint32_t)num_cus();
  P.strips = (P.OW + kStripCols - 1) / kStripCols;
  const uint64_t base_items = (uint64_t)N * num_tiles * P.strips;
  // split the rows of a strip into segments while that evens out the load over the CUs; a
  // segment re-reads two input rows, so keep it at 16 rows or more
  uint32_t segs = 1;
  const uint32_t max_segs = (P.OH + 15u) / 16u;
  const uint64_t want = 4ull * cus / groups;
  while (segs < max_segs && base_items * segs < want) ++segs;
  uint32_t seg_rows = (P.OH + segs - 1) / segs;
  seg_rows = (seg_rows + kStepRows - 1) / kStepRows * kStepRows;
  segs = (P.OH + seg_rows - 1) / seg_rows;
  P.segs = segs;
  P.seg_rows = seg_rows;
  const uint64_t items = base_items * segs;
  if (items >= (1ull << 31)) return ADH_EINVAL;
  P.items = (uint32_t)items;
  P.div_strips = FastDiv(P.strips);
  P.div_segs = FastDiv(P.segs);
  P.div_N = FastDiv(N);
  uint32_t gx = cus / groups ? cus / groups : 1u;
  if (gx > P.items) gx = P.items;
  hipLaunchKernelGGL(conv3x3_bf16_kernel, dim3(gx, groups), dim3(256), 0, st, P);
  return launch_status();
}

}  // namespace adh
