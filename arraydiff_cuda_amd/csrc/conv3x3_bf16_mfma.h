// Declarations shared by the bf16 matrix-core 3x3 slab convolution kernels (conv3x3_bf16_mfma.hip: four waves,
// any shape; conv3x3_bf16_w8.hip: eight waves, even widths; conv3x3_bf16_k128.hip: 128 reduction channels per launch).
#ifndef ADH_CONV3X3_BF16_MFMA_H
#define ADH_CONV3X3_BF16_MFMA_H

#include <utility>

#include "adh_common.h"

namespace adh {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef floatx4 floatx4_a4 __attribute__((aligned(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef u32x4 u32x4_unaligned __attribute__((aligned(2)));

constexpr int kStripCols = 64;                        // output columns per work item
constexpr int kStepRows = 4;                          // output rows per step
constexpr uint32_t kOutOfRange = 0x80000000u;
constexpr uint32_t kWtGroupElems = 9u * 2u * 64u * 32u;  // transformed filter elements per group of 64 outputs

struct ConvBf16Params {
  const uint16_t *in[ADH_MAX_TILES];
  uint16_t *out[ADH_MAX_TILES];
  const uint16_t *wt;       // transformed filter: [group][pass][tap][half][64 out][32 red]
  uint32_t N, Cred, Cout;   // reduction and output channel counts as the kernel sees them
  // More than 64 reduction channels take one launch per 64 (a pass): the pass multiplies channels
  // chan0 .. chan0 + cred_pass - 1 and hands its sums to the next one as fp32 in `part`
  // ([image][output channel][row][column] per tile); the last pass rounds to bf16 into `out`.
  // (`pass` counts in 64 channels, the unit of the transformed filter's layout; the kernel of
  // conv3x3_bf16_k128.hip multiplies two such units per launch.  first_pass / last_pass: this launch reads no
  // sums / rounds to bf16.)
  uint32_t pass, passes, chan0, cred_pass, first_pass, last_pass;
  float *part[ADH_MAX_TILES];
  // the eight-wave kernel reads the filter as the caller holds it (no transformed copy): forward, a
  // multiple of 64 input channels, 16-byte aligned; else null
  const uint16_t *w_direct;
  // the eight-wave kernel over tiles without halo (pad 1): rows -1 and IH come from the neighbouring tiles
  uint32_t neighbour_rows, num_tiles;
  uint32_t IH, IW, OH, OW;
  int32_t pad;              // input row/col = output row/col + tap - pad
  float beta;
  // An item is a strip of an image (strip index fastest).  The first `whole_items` are dealt to
  // the workgroups in turn, top to bottom each; what is left over (fewer items than workgroups)
  // is cut into row segments of `seg_steps` steps so that it spreads over all of them.
  uint32_t strips, items, whole_items, steps_per_item, seg_steps, segs, pieces;
  FastDiv div_strips, div_N, div_rest;
};

template <int V>
struct IntTag { static constexpr int value = V; };
template <int... T, typename F>
__device__ __forceinline__ void for_each_int(std::integer_sequence<int, T...>, F &&f) {
  (f(IntTag<T>()), ...);
}

// two floats -> two bf16 (round to nearest even) in one dword: one v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  const floatx2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// the eight-wave kernel: shapes it takes, and its launch (grid.x workgroups per output group)
bool conv_bf16_w8_takes(const ConvBf16Params &P, uint32_t num_tiles);
// launches the pass of up to 64 reduction channels from P.chan0 on
int conv_bf16_w8_launch(const ConvBf16Params &P, uint32_t gx, uint32_t groups, hipStream_t st);
// the kernel for more than 64 reduction channels (128 per pass, 128 output channels per workgroup, 32-column
// strips): shapes it takes, and its launch (grid.x workgroups per group of 128 output channels)
constexpr int kStripColsK128 = 32;
bool conv_bf16_k128_takes(const ConvBf16Params &P, uint32_t num_tiles);
int conv_bf16_k128_launch(const ConvBf16Params &P, uint32_t gx, uint32_t groups128, hipStream_t st);

}  // namespace adh

#endif
