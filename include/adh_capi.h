/*
 * adh_capi.h -- C ABI of the MI355X (gfx950) spatially-parallel convolution path.
 *
 * This is the launcher-level seam of the reference
 * (include/arraydiff/kernels.hh:72-262 plus the cuDNN calls in src/op.cc):
 * free functions taking raw device pointers, uint32 extents and a stream, which
 * enqueue work asynchronously and own nothing.  Differences, on purpose:
 *   - every function returns int: 0 = ok, <0 = ADH_E* argument error (nothing was
 *     enqueued), >0 = a hipError_t from the launch.  Nothing aborts.
 *   - one launch serves all K tiles that live in this GPU's memory, where the
 *     reference launched one kernel per rank; `*_rank` variants do one rank's share
 *     so that a per-rank caller (Spatial2DComm::group_end) keeps its call shape.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *
 * Layout: NCHW with W fastest, idx = w + W*(h + H*(c + C*n))
 * (src/kernels/spatial.cu:22-36).  A halo-padded tile of interior (W,H) and halo p
 * is a packed (W+2p, H+2p, C, N) buffer; "tile pointers" are BASE pointers of such
 * buffers (what GPUBatchArray::base_as_view().dptr() returns,
 * include/arraydiff/array_gpu.hh:544-548).  Pointer tables (`void* const*`) are
 * HOST arrays of DEVICE pointers; they are read before the call returns.
 *
 * Re-entrant and callable from any host thread: a call reads its arguments and enqueues work, and
 * nothing a call leaves behind changes the result of another.  The library's only process-wide state
 * is two caches filled on first use, the current device's compute-unit count (the persistent kernels'
 * grid size) and the per-device address of the scratch array of adh_conv3x3_slab_fwd_tiles_static;
 * that one entry point shares its scratch between calls and is the exception noted where it is declared.
 */
#ifndef ADH_CAPI_H
#define ADH_CAPI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ADH_VERSION 1

/* element types (Spatial2DDataType in include/arraydiff/spatial.hh:25-29 has
 * FLOAT/DOUBLE/HALF and only FLOAT is implemented, src/spatial.cc:76-78) */
#define ADH_F32 0
#define ADH_BF16 1

/* error codes */
#define ADH_OK 0
#define ADH_EINVAL (-1)  /* bad extent, window out of bounds, H % K != 0, too many tiles */
#define ADH_EUNIMPL (-2) /* combination the reference asserts "unimplemented" on, e.g. 2x2 grid */
#define ADH_ENULL (-3)   /* a required pointer is NULL (src/spatial.cc:71-73) */
#define ADH_EALIGN (-4)  /* pointer not aligned to its element size */
#define ADH_EWORKSPACE (-5) /* workspace too small; see *_workspace_bytes */

#define ADH_MAX_TILES 16 /* ARRAYDIFF_MAX_PEERS is 8, include/arraydiff/spatial.hh:11 */

int adh_version(void);
const char *adh_error_string(int code);

/* ---- Z1: whole-buffer fill / accumulate ---------------------------------- */
/* array_set_constant_packed<float>, src/kernels/array.cu:58-68,155-164 */
int adh_fill_f32(uint64_t n, float value, float *x, void *stream);
/* array_add_packed<float> (y += x), src/kernels/array.cu:83-94,199-208 */
int adh_add_f32(uint64_t n, const float *x, float *y, void *stream);

/* ---- H1/H2/H3: halo exchange / reduce ------------------------------------- */
/* spatial2d_1x{2,4}_halo_exch_nchw, src/kernels/spatial.cu:455-485,596-623 (rows),
 * spatial2d_2x1_halo_exch_nchw :708-731 (columns), for any K <= ADH_MAX_TILES.
 * grid_w x grid_h follows Spatial2DComm::group_end, src/spatial.cc:76-135:
 * 1x1 no-op, 1xK rows, Kx1 columns, both > 1 -> ADH_EUNIMPL.
 * W,H are one tile's interior extents; tile_bufs[r], r = r_w + grid_w*r_h. */
int adh_halo_exchange_nchw(int dtype, uint32_t grid_w, uint32_t grid_h, uint32_t halo_pad,
                           uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                           void *const *tile_bufs, void *stream);
/* spatial2d_1x{2,4}_halo_reduce_nchw, src/kernels/spatial.cu:487-510,625-652.
 * Plain (non-atomic) adds: needs H >= 2*halo_pad (W >= 2*halo_pad for columns) so each
 * destination has one contributor, else ADH_EINVAL.  Column reduce (declared but never
 * linked in the reference, src/spatial.cc:166-178) is the W mirror of the row reduce. */
int adh_halo_reduce_nchw(int dtype, uint32_t grid_w, uint32_t grid_h, uint32_t halo_pad,
                         uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                         void *const *tile_bufs, void *stream);
/* one rank's share of the above (what one reference kernel launch did) */
int adh_halo_exchange_nchw_rank(int dtype, uint32_t grid_w, uint32_t grid_h, uint32_t rank,
                                uint32_t halo_pad, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                                void *const *tile_bufs, void *stream);
int adh_halo_reduce_nchw_rank(int dtype, uint32_t grid_w, uint32_t grid_h, uint32_t rank,
                              uint32_t halo_pad, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                              void *const *tile_bufs, void *stream);

/* ---- P1/P2/P3: pad / unpad (the strided cudnnAddTensor uses) -------------- */
/* HaloPad2DOp::_forward, src/op.cc:2574-2641: whole padded buffer zeroed, interior = x.
 * One pass instead of memset + AddTensor. */
int adh_halo_pad_nchw(int dtype, uint32_t halo_pad, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                      const void *x_packed, void *y_padded, void *stream);
/* HaloUnpad2DOp::_backward, src/op.cc:2798-2870: interior(y_padded) += x_packed */
int adh_halo_pad_add_nchw(int dtype, uint32_t halo_pad, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                          const void *x_packed, void *y_padded, void *stream);
/* HaloUnpad2DOp::_forward, src/op.cc:2715-2793: y_packed = interior(x_padded) */
int adh_halo_unpad_nchw(int dtype, uint32_t halo_pad, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                        const void *x_padded, void *y_packed, void *stream);
/* HaloPad2DOp::_backward, src/op.cc:2644-2712: y_packed += interior(x_padded) */
int adh_halo_unpad_add_nchw(int dtype, uint32_t halo_pad, uint32_t W, uint32_t H, uint32_t C, uint32_t N,
                            const void *x_padded, void *y_packed, void *stream);
/* HaloRepad2DOp::_forward, src/op.cc:2873-2960: interior of a p_src buffer -> interior of a
 * p_dst buffer whose border is zeroed */
int adh_halo_repad_nchw(int dtype, uint32_t pad_src, uint32_t pad_dst, uint32_t W, uint32_t H,
                        uint32_t C, uint32_t N, const void *x_padded, void *y_padded, void *stream);

/* ---- S1/S2: box copy / add between packed NCHW tensors -------------------- */
/* slice2d_copy_hw_nchw_packed / slice2d_add_hw_nchw_packed, src/kernels/slice.cu:43-105,
 * extended by a channel range (the reference's call is count_c == src_C == dst_C, c offsets 0).
 * Window bounds are checked like slice.cu:61-64 but reported as ADH_EINVAL. */
int adh_slice_copy_nchw(int dtype, uint32_t count_w, uint32_t count_h, uint32_t count_c, uint32_t N,
                        const void *src, uint32_t src_W, uint32_t src_H, uint32_t src_C,
                        uint32_t src_w_off, uint32_t src_h_off, uint32_t src_c_off,
                        void *dst, uint32_t dst_W, uint32_t dst_H, uint32_t dst_C,
                        uint32_t dst_w_off, uint32_t dst_h_off, uint32_t dst_c_off, void *stream);
int adh_slice_add_nchw(int dtype, uint32_t count_w, uint32_t count_h, uint32_t count_c, uint32_t N,
                       const void *src, uint32_t src_W, uint32_t src_H, uint32_t src_C,
                       uint32_t src_w_off, uint32_t src_h_off, uint32_t src_c_off,
                       void *dst, uint32_t dst_W, uint32_t dst_H, uint32_t dst_C,
                       uint32_t dst_w_off, uint32_t dst_h_off, uint32_t dst_c_off, void *stream);

/* ---- fused pack / unpack --------------------------------------------------- */
/* pack = SpatialScatter2DOp::_forward (src/op.cc:2396-2429) + HaloPad2DOp::_forward +
 * HaloExch2DOp::_forward (src/op.cc:2963-3003) in one pass: unsplit (W,H,C,N) -> K padded
 * tiles of (W+2p, H/K+2p, C, N), halo rows filled from the neighbouring rows, border zero.
 * H is the UNSPLIT height, H % K == 0 (src/op.cc:2385-2387), H/K >= halo_pad. */
int adh_tiles_pack_nchw(int dtype, uint32_t K, uint32_t halo_pad, uint32_t W, uint32_t H, uint32_t C,
                        uint32_t N, const void *x_unsplit, void *const *tile_bufs, void *stream);
/* unpack = HaloUnpad2DOp::_forward + SpatialGather2DOp::_forward (src/op.cc:2480-2514):
 * interiors of K padded tiles -> unsplit tensor; halo contents are ignored. */
int adh_tiles_unpack_nchw(int dtype, uint32_t K, uint32_t halo_pad, uint32_t W, uint32_t H, uint32_t C,
                          uint32_t N, const void *const *tile_bufs, void *y_unsplit, void *stream);

/* ---- C2/C3/C4: 3x3 convolution over the halo-padded slab ------------------ */
/* All three: cross-correlation, stride 1, dilation 1, conv pad 0 over a slab padded by 1
 * (Conv2DShape.halo_padded_input, src/op.cc:1354-1410), filter KCRS (Cout,Cin,3,3),
 * no bias (adh_conv_bias_add_tiles / adh_conv_bwd_bias_tiles below).  beta is 0 (overwrite) or 1
 * (accumulate), the two values the reference passes.
 * `*_tiles` variants run K slabs of identical shape in one launch.  Workspace may be NULL
 * when the matching *_workspace_bytes query returns 0; otherwise it must be 256-byte aligned.
 * ADH_BF16: x, w, y, dy, dx are bf16 in memory, sums are fp32, results rounded to nearest even;
 * dw stays fp32.  The bf16 entry needs a workspace for all three passes.  Shapes and routes in bf16
 * (forward / backward-data; "reduction channels" are Cin forward and Cout backward):
 *   - up to 64 reduction channels: one launch on the bf16 matrix cores for any width and alignment;
 *   - more than 64 reduction channels, even width (forward) or a width that is a multiple of 8
 *     (backward-data), tiles aligned to 4 (16) bytes: the matrix cores, 128 reduction channels per launch
 *     with the sums in registers when there are also more than 64 output channels (fp32 sums pass through
 *     the workspace only between such launches: 256 channels are two), else 64 per launch;
 *   - more than 64 reduction channels at any other width (odd; backward-data at a width that is no multiple
 *     of 8): the four-wave matrix-core kernel once per 64 reduction channels with fp32 sums through the
 *     workspace, 2.5-3.5 times slower than the route above (128 -> 128 channels on 64 x 255 tiles 340-430
 *     TFLOP/s against 1020-1180 at 64 x 256; 512 -> 512 on 7 x 7 tiles 45-60).  Tiles off that alignment
 *     take the same route when the reduction needs more than one launch anyway; where the width promises ONE
 *     launch of 128 channels the workspace has no room for the sums and the call returns ADH_EALIGN;
 *   - the sums of one image beyond 2 GiB (Cout * H * W * 4 bytes): the tensors are widened to fp32 in the
 *     workspace and the fp32 kernels run, about ten times slower.
 * Backward-data into PADDED slabs is the form the reference's graph needs (cudnnConvolutionBackwardData
 * writes the whole padded slab, src/op.cc:1701-1712) and the compatibility path here: rows of W + 2
 * bf16 elements start 4 bytes further into a 64-byte sector with every row, so every store straddles
 * two sectors and the launch moves 1.2-1.4 times its bytes (0.33 of the matrix peak at 64 channels
 * where the forward reaches 0.45).  adh_conv3x3_unpadded_bwd_data_tiles, whose rows are aligned, is the
 * fast form (0.44; 0.54 at 128 channels) and also replaces the halo reduce and the unpad pass. */
#define ADH_CONV_FWD 0
#define ADH_CONV_BWD_DATA 1
#define ADH_CONV_BWD_FILTER 2
size_t adh_conv3x3_workspace_bytes(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin,
                                   uint32_t Cout, uint32_t H, uint32_t W);
/* Name of the kernel instance a forward or backward-data call of this shape is routed to (tile
 * buffers aligned to 16 bytes), written to `name`; for tools that match timings against a
 * profiler's kernel trace.  Plays the part of the algorithm the reference reads back from
 * cudnnFindConvolution*Algorithm and prints (src/op.cc:1463-1507). */
int adh_conv3x3_kernel_name(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                            uint32_t H, uint32_t W, float beta, char *name, size_t name_bytes);
/* cudnnConvolutionForward at src/op.cc:1576-1587:
 * y[n,co,h,w] = beta*y + sum_{ci,kh,kw} w[co,ci,kh,kw] * x_pad[n,ci,h+kh,w+kw] */
int adh_conv3x3_slab_fwd(int dtype, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                         const void *x_pad, const void *w, void *y, float beta,
                         void *workspace, size_t workspace_bytes, void *stream);
int adh_conv3x3_slab_fwd_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                               uint32_t H, uint32_t W, const void *const *x_pad_tiles, const void *w,
                               void *const *y_tiles, float beta, void *workspace,
                               size_t workspace_bytes, void *stream);
/* HaloExch2DOp::_forward (src/op.cc:2963-3007) and the cudnnConvolutionForward of its consumer
 * (src/op.cc:1576-1587) in one launch: x_pad_tiles are the row tiles of ONE activation in rank order
 * (a 1 x num_tiles grid, halo width 1) whose inner halo rows have NOT been exchanged.  The result
 * equals adh_halo_exchange_nchw followed by adh_conv3x3_slab_fwd_tiles, bit for bit: tile t reads
 * its top halo row from tile t-1's last interior row and its bottom halo row from tile t+1's first.
 * fp32 leaves the inner halo rows of x_pad unread and unwritten; bf16 exchanges and then convolves
 * (two launches, the halo rows are refreshed).  The outer halo rows are read from each tile itself;
 * the corner elements of an inner halo row, which an exchange does not touch, are taken from the
 * neighbour's halo columns: both are zero after HaloPad2DOp, and must be equal for the equality to hold. */
int adh_conv3x3_slab_fwd_tiles_unexchanged(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                           uint32_t H, uint32_t W, const void *const *x_pad_tiles,
                                           const void *w, void *const *y_tiles, float beta, void *workspace,
                                           size_t workspace_bytes, void *stream);
/* adh_conv3x3_slab_fwd_tiles for callers that cannot allocate and have no workspace to pass (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  dtype must be ADH_BF16 with Cin <= 64 and Cout <= 256 (else
 * ADH_EWORKSPACE): the reordered filter, which the other entry point keeps in the caller's
 * workspace, goes to a 294,912-byte array inside the library's device image, one copy per GPU,
 * held until the process ends.  The call allocates and frees nothing.  Unlike every other entry
 * point it is not re-entrant: all calls on a GPU share that GPU's array (each call rewrites the
 * part it uses before reading it), so calls that overlap on one GPU, on any streams, race. */
int adh_conv3x3_slab_fwd_tiles_static(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                      uint32_t H, uint32_t W, const void *const *x_pad_tiles, const void *w,
                                      void *const *y_tiles, float beta, void *stream);
/* cudnnConvolutionBackwardData at src/op.cc:1701-1712: writes the WHOLE padded slab
 * dx_pad[n,ci,h',w'] = beta*dx_pad + sum_{co,kh,kw} w[co,ci,kh,kw] * dy[n,co,h'-kh,w'-kw] */
int adh_conv3x3_slab_bwd_data(int dtype, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                              const void *w, const void *dy, void *dx_pad, float beta,
                              void *workspace, size_t workspace_bytes, void *stream);
int adh_conv3x3_slab_bwd_data_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                    uint32_t H, uint32_t W, const void *w, const void *const *dy_tiles,
                                    void *const *dx_pad_tiles, float beta, void *workspace,
                                    size_t workspace_bytes, void *stream);
/* cudnnConvolutionBackwardData of the conv (src/op.cc:1701-1712) and HaloExch2DOp::_backward of
 * its producer (the halo reduce, src/op.cc:3009-3052) in one launch: dy_tiles are the row tiles of
 * ONE gradient in rank order (a 1 x num_tiles grid, halo width 1).  The interior of every
 * dx_pad tile equals adh_conv3x3_slab_bwd_data_tiles followed by adh_halo_reduce_nchw up to the
 * order of the additions (tile t also multiplies the last dy row of tile t-1 and the first of tile
 * t+1); the inner halo rows of dx_pad hold partial sums nobody should read (HaloPad2DOp's
 * backward reads the interior).  fp32: one launch, any beta in {0, 1}.  bf16: backward-data, then
 * the reduce (two launches; beta = 1 returns ADH_EUNIMPL). */
int adh_conv3x3_slab_bwd_data_tiles_reduced(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin,
                                            uint32_t Cout, uint32_t H, uint32_t W, const void *w,
                                            const void *const *dy_tiles, void *const *dx_pad_tiles,
                                            float beta, void *workspace, size_t workspace_bytes,
                                            void *stream);
/* The whole forward chain HaloPad2DOp -> HaloExch2DOp -> CudnnConv2DOp (src/op.cc:2574-2641, 2963-3007,
 * 1576-1587) and the whole backward chain conv backward-data -> halo reduce -> HaloPad2DOp::_backward
 * (src/op.cc:1701-1712, 3009-3052, 2643-2700) as ONE launch each over row tiles that carry NO halo:
 * x_tiles / y_tiles / dy_tiles / dx_tiles are the K row tiles (H x W each, packed NCHW) of one tensor in
 * rank order.  A tile's rows -1 and H are read from its neighbours' last and first rows, the tensor's own
 * border is zero: tile t of the result is rows [t*H, (t+1)*H) of the unsplit 3x3 convolution with zero
 * padding 1 (forward: y = beta*y + conv(x, w); backward-data: dx = beta*dx + conv^T(dy, w)).  No padded
 * copy of the activation or of its gradient exists, so the pad, exchange, reduce and unpad passes and
 * their buffers disappear.  fp32: any shape the padded entry points take, no workspace.  bf16: W a
 * multiple of 8 and 16-byte aligned tiles (the bf16 matrix-core kernel; other widths return
 * ADH_EUNIMPL: use the padded entry points), workspace as for adh_conv3x3_slab_fwd_tiles /
 * adh_conv3x3_slab_bwd_data_tiles of the same shape. */
int adh_conv3x3_unpadded_fwd_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                   uint32_t H, uint32_t W, const void *const *x_tiles, const void *w,
                                   void *const *y_tiles, float beta, void *workspace, size_t workspace_bytes,
                                   void *stream);
/* The sum that closes a residual block, JoinOp<SumJoin> after the block's second CudnnConv2DOp
 * (src/zoo.cc:577-652: x + conv(...); src/op.cc:744-867), in the convolution's own stores:
 * y = conv(x, w) + res over tiles without halo, res_tiles laid out like y_tiles (H x W x Cout x N each, packed;
 * res_tiles[t] may be y_tiles[t] itself, but must not overlap another tile of y).  fp32 only (other dtypes:
 * ADH_EUNIMPL), no workspace. */
int adh_conv3x3_unpadded_fwd_residual_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                            uint32_t H, uint32_t W, const void *const *x_tiles, const void *w,
                                            const void *const *res_tiles, void *const *y_tiles, void *stream);
int adh_conv3x3_unpadded_bwd_data_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                        uint32_t H, uint32_t W, const void *w, const void *const *dy_tiles,
                                        void *const *dx_tiles, float beta, void *workspace,
                                        size_t workspace_bytes, void *stream);
/* the filter gradient of the same convolution (cudnnConvolutionBackwardFilter, src/op.cc:1660-1671, over
 * the tiles HaloPad2DOp and HaloExch2DOp would have prepared): dw = beta*dw + sum over tiles of
 * dy (*) x with x read as above.  Workspace as for adh_conv3x3_slab_bwd_filter_tiles. */
int adh_conv3x3_unpadded_bwd_filter_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                          uint32_t H, uint32_t W, const void *const *x_tiles,
                                          const void *const *dy_tiles, float *dw, float beta, void *workspace,
                                          size_t workspace_bytes, void *stream);
/* cudnnConvolutionBackwardFilter at src/op.cc:1660-1671:
 * dw[co,ci,kh,kw] = beta*dw + sum_{tiles,n,h,w} dy[n,co,h,w] * x_pad[n,ci,h+kh,w+kw]
 * (the sum over tiles is what ParallelSGDOptimizer's ncclReduce did across ranks,
 * include/arraydiff/optimize.hh:443-451).  dw is always fp32.  Deterministic.
 * ADH_BF16: the matrix-core kernel reads rows of whole 16-byte granules; at a width that is no multiple
 * of 8 the rows of x_pad and dy are first copied into the workspace at the next such width with zeros
 * behind (a zero dy adds nothing to any tap), one more pass over both tensors. */
int adh_conv3x3_slab_bwd_filter(int dtype, uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W,
                                const void *x_pad, const void *dy, float *dw, float beta,
                                void *workspace, size_t workspace_bytes, void *stream);
int adh_conv3x3_slab_bwd_filter_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin,
                                      uint32_t Cout, uint32_t H, uint32_t W,
                                      const void *const *x_pad_tiles, const void *const *dy_tiles,
                                      float *dw, float beta, void *workspace, size_t workspace_bytes,
                                      void *stream);
/* the filter gradient over tiles whose inner halo rows were never exchanged (the backward of a
 * forward that went through adh_conv3x3_slab_fwd_tiles_unexchanged): equals adh_halo_exchange_nchw
 * followed by adh_conv3x3_slab_bwd_filter_tiles, bit for bit. */
int adh_conv3x3_slab_bwd_filter_tiles_unexchanged(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin,
                                                  uint32_t Cout, uint32_t H, uint32_t W,
                                                  const void *const *x_pad_tiles, const void *const *dy_tiles,
                                                  float *dw, float beta, void *workspace,
                                                  size_t workspace_bytes, void *stream);

/* ---- convolution bias ------------------------------------------------------- */
/* cudnnAddTensor(alpha = 1, bias_desc (1,C,1,1), beta = 1, y_desc) after the forward convolution of a
 * CudnnConv2DOp built with a bias (src/op.cc:1602-1610; the stem of the spatial nets, src/zoo.cc:1548):
 * y[n,c,h,w] += bias[c] over the K packed (N,C,H,W) result tiles in one launch.  Every rank of the
 * reference holds its own bias vector: bias_tiles[t] is the fp32 vector of C added to y_tiles[t] (the
 * entries may all be one pointer).  y is f32 or bf16 (sum in fp32, one rounding). */
int adh_conv_bias_add_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                            const float *const *bias_tiles, void *const *y_tiles, void *stream);
/* cudnnConvolutionBackwardBias(alpha = 1, dy, beta, db) at src/op.cc:1632-1648:
 * db[c] = beta*db[c] + sum_{tiles,n,h,w} dy[n,c,h,w], beta 0 or 1 (the reference zeroes db on first touch
 * and passes 1); the sum over tiles is what ParallelSGDOptimizer's ncclReduce did across ranks
 * (include/arraydiff/optimize.hh:443-451).  db is fp32.  The workspace (256-byte aligned,
 * adh_conv_bwd_bias_workspace_bytes) holds partial sums that a second kernel adds in a fixed order:
 * repeated calls give the same bits. */
size_t adh_conv_bwd_bias_workspace_bytes(uint32_t num_tiles, uint32_t N, uint32_t C);
int adh_conv_bwd_bias_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                            const void *const *dy_tiles, float *db, float beta, void *workspace,
                            size_t workspace_bytes, void *stream);

/* ---- general window / stride / dilation over the halo-padded slab ------------ */
/* The other consumers of halo-padded input (CudnnConv2DSize with halo_padded_input,
 * src/op.cc:1354-1410; the 7x7 stem src/zoo.cc:1528-1538, stride-2 3x3 src/zoo.cc:692-697, the
 * dilated 3x3 of tools/microbench_spatial_conv.cc:25-32) and, with HP x WP the extents of a
 * packed unpadded tensor, the 1x1 projections (src/zoo.cc:680-690): x_pad is a packed
 * (N,Cin,HP,WP) tensor convolved with conv pad 0, filter KCRS (Cout,Cin,kh,kw), stride (sh,sw),
 * dilation (dh,dw); OH = (HP - ((kh-1)*dh + 1)) / sh + 1, likewise OW
 * (cudnnGetConvolution2dForwardOutputDim, src/op.cc:1512-1523).  kh*kw <= 64, sh*sw <= 16,
 * HP*WP < 2^30 (ADH_EINVAL beyond).
 * fp32 arithmetic on the matrix cores; ADH_BF16 tensors are widened on load and rounded on store.
 * The workspace (adh_conv2d_workspace_bytes, 256-byte aligned) holds the rewritten filter and, for thin
 * launches whose channel chunks are dealt to several workgroups, their fp32 partial sums (added in a
 * fixed order by a second kernel: results are reproducible).  In fp32, 1x1 windows at stride 1 or 2, windows
 * over at most three input channels (a stem) and the 3x3 window at stride 1 with dilation 3 (the reference's
 * microbenchmark) are served by kernels of their own behind these entry points, chosen by shape and alignment;
 * arguments, workspace query and error codes are the same for every shape. */
size_t adh_conv2d_workspace_bytes(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin,
                                  uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t kh, uint32_t kw,
                                  uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw);
/* cudnnConvolutionForward at src/op.cc:1576-1587:
 * y[n,co,oh,ow] = beta*y + sum_{ci,a,b} w[co,ci,a,b] * x_pad[n,ci,oh*sh + a*dh, ow*sw + b*dw] */
int adh_conv2d_slab_fwd_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                              uint32_t HP, uint32_t WP, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw,
                              uint32_t dh, uint32_t dw, const void *const *x_pad_tiles, const void *w,
                              void *const *y_tiles, float beta, void *workspace, size_t workspace_bytes,
                              void *stream);
/* The same followed by the bias (cudnnConvolutionForward + cudnnAddTensor, src/op.cc:1576-1610):
 * y = beta*y + conv(x_pad, w) + bias[co], bias_tiles one fp32 vector of Cout per tile (entries may repeat).  Where the
 * kernel that serves the shape can, the bias is added in its stores (windows over at most three input channels: a
 * network's stem); elsewhere adh_conv_bias_add_tiles follows the convolution on the same stream.  Either way the
 * result has the bits of the two separate calls. */
int adh_conv2d_slab_fwd_bias_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                   uint32_t HP, uint32_t WP, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw,
                                   uint32_t dh, uint32_t dw, const void *const *x_pad_tiles, const void *w,
                                   const float *const *bias_tiles, void *const *y_tiles, float beta,
                                   void *workspace, size_t workspace_bytes, void *stream);
/* cudnnConvolutionBackwardData at src/op.cc:1701-1712: the adjoint of the above, written over the
 * WHOLE padded tile (padded pixels that no window reads get beta*dx_pad) */
int adh_conv2d_slab_bwd_data_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                   uint32_t HP, uint32_t WP, uint32_t kh, uint32_t kw, uint32_t sh,
                                   uint32_t sw, uint32_t dh, uint32_t dw, const void *w,
                                   const void *const *dy_tiles, void *const *dx_pad_tiles, float beta,
                                   void *workspace, size_t workspace_bytes, void *stream);

/* cudnnConvolutionBackwardFilter at src/op.cc:1660-1671 for the same descriptors:
 * dw[co,ci,a,b] = beta*dw + sum_{tiles,n,oh,ow} dy[n,co,oh,ow] * x_pad[n,ci,oh*sh + a*dh, ow*sw + b*dw];
 * dw is always fp32; the workspace holds partial sums that are added in a fixed order. */
int adh_conv2d_slab_bwd_filter_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                     uint32_t HP, uint32_t WP, uint32_t kh, uint32_t kw, uint32_t sh,
                                     uint32_t sw, uint32_t dh, uint32_t dw, const void *const *x_pad_tiles,
                                     const void *const *dy_tiles, float *dwt, float beta, void *workspace,
                                     size_t workspace_bytes, void *stream);

/* The same three passes over row tiles that carry NO halo, for any window / stride / dilation: the chains
 * HaloPad2DOp -> HaloExch2DOp -> CudnnConv2DOp and conv backward-data -> halo reduce -> HaloPad2DOp::_backward
 * (src/op.cc:2574-2641, 2963-3007, 1576-1587; 1701-1712, 3009-3052, 2643-2700) as one convolution launch each
 * (the strided 3x3 and the 7x7 stem of src/zoo.cc:692-697, 1528-1538 without their pad, exchange, reduce and unpad
 * passes).  x_tiles / dx_tiles are the K row tiles (H x W, packed NCHW) of one tensor in rank order, y_tiles /
 * dy_tiles the row tiles (H / sh rows, OW = (W + 2 pad_w - ((kw-1)*dw + 1)) / sw + 1 columns) of the result.  Rows
 * a window reaches outside a tile are read from the neighbouring tiles, the tensor's own border is zero
 * padding (pad_h, pad_w): tile t of y is rows [t*H/sh, (t+1)*H/sh) of the unsplit convolution with that padding;
 * backward-data computes the tile's own gradient completely (what the reduce would have added comes from the
 * neighbours' dy rows) and never the halo pixels' (a 4 x 16 tile has 64 pixels, its padded form 108).
 * Limits: H a multiple of sh; 0 < (kh-1)*dh + 1 - 2 pad_h <= sh (then H / sh output rows per tile stitch to the
 * unsplit output: 3x3 pad 1 at stride 1 or 2, 7x7 pad 3, 1x1 pad 0 ...); pad_h <= H and (kh-1)*dh - pad_h <= H
 * (a window reaches the adjacent tiles only); otherwise as the padded entry points above with HP = H + 2 pad_h,
 * WP = W + 2 pad_w.  ADH_EINVAL outside these limits. */
size_t adh_conv2d_unpadded_workspace_bytes(int which, int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin,
                                           uint32_t Cout, uint32_t H, uint32_t W, uint32_t kh, uint32_t kw,
                                           uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, uint32_t pad_h,
                                           uint32_t pad_w);
int adh_conv2d_unpadded_fwd_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                  uint32_t H, uint32_t W, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw,
                                  uint32_t dh, uint32_t dw, uint32_t pad_h, uint32_t pad_w,
                                  const void *const *x_tiles, const void *w, void *const *y_tiles, float beta,
                                  void *workspace, size_t workspace_bytes, void *stream);
int adh_conv2d_unpadded_bwd_data_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                       uint32_t H, uint32_t W, uint32_t kh, uint32_t kw, uint32_t sh, uint32_t sw,
                                       uint32_t dh, uint32_t dw, uint32_t pad_h, uint32_t pad_w, const void *w,
                                       const void *const *dy_tiles, void *const *dx_tiles, float beta,
                                       void *workspace, size_t workspace_bytes, void *stream);
int adh_conv2d_unpadded_bwd_filter_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t Cin, uint32_t Cout,
                                         uint32_t H, uint32_t W, uint32_t kh, uint32_t kw, uint32_t sh,
                                         uint32_t sw, uint32_t dh, uint32_t dw, uint32_t pad_h, uint32_t pad_w,
                                         const void *const *x_tiles, const void *const *dy_tiles, float *dwt,
                                         float beta, void *workspace, size_t workspace_bytes, void *stream);

/* ---- the shard-local ops between two halo exchanges ------------------------- */
/* CudnnBatchNorm2DOp (src/op.cc:3907-4100) over K tiles in one call; as in the reference every
 * tile (rank) has its own parameters and normalises with its OWN batch statistics over
 * m = N*H*W elements per channel.  x, dx are packed (N,C,H,W); scale, shift, statistics and
 * parameter gradients are fp32 vectors of C per tile (tables of K device pointers).
 * training != 0: cudnnBatchNormalizationForwardTraining(SPATIAL, factor = 1, eps)
 *   (src/op.cc:3996-4011): y = scale*(x-mean)/sqrt(var+eps) + shift; run_mean = mean,
 *   run_var = var*m/(m-1), save_mean = mean, save_invstd = 1/sqrt(var+eps) (any of the four
 *   tables, or entries, may be NULL).  training == 0: ...ForwardInference with fixed_mean /
 *   fixed_var (src/op.cc:3978-3990).
 * Fusions that have no counterpart in the reference (it ran three ops and three passes):
 *   relu != 0 applies CudnnActivationOp's max(y,0) (src/op.cc:3189-3250) on the way out;
 *   out_halo = p > 0 writes y into the interior of a (N,C,H+2p,W+2p) tile and zeroes its border,
 *   i.e. HaloPad2DOp::_forward (src/op.cc:2573-2640); with relu = 0, out_halo = 0 it is the plain op.
 * The workspace (adh_batchnorm2d_workspace_bytes, 256-byte aligned) holds partial sums. */
size_t adh_batchnorm2d_workspace_bytes(uint32_t num_tiles, uint32_t N, uint32_t C);
int adh_batchnorm2d_fwd_tiles(int dtype, int training, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H,
                              uint32_t W, float eps, int relu, uint32_t out_halo, const void *const *x_tiles,
                              const float *const *scale_tiles, const float *const *shift_tiles,
                              const float *const *fixed_mean_tiles, const float *const *fixed_var_tiles,
                              void *const *y_tiles, float *const *run_mean_tiles, float *const *run_var_tiles,
                              float *const *save_mean_tiles, float *const *save_invstd_tiles, void *workspace,
                              size_t workspace_bytes, void *stream);
/* cudnnBatchNormalizationBackward (src/op.cc:4082-4097) with the saved statistics:
 *   dshift = beta_param*dshift + sum dy', dscale = beta_param*dscale + sum dy'*xhat,
 *   dx = beta_data*dx + scale*invstd*(dy' - sum dy'/m - xhat * sum dy'*xhat / m).
 * relu != 0: dy' = dy where the fused forward output was positive (cudnnActivationBackward,
 * src/op.cc:3252-3324; the mask is recomputed from x, y is not read); dy_halo = p > 0: dy is the
 * interior of a gradient tile padded by p (HaloPad2DOp::_backward, src/op.cc:2642-2712).
 * shift_tiles is only read when relu != 0. */
int adh_batchnorm2d_bwd_tiles(int dtype, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                              int relu, uint32_t dy_halo, const void *const *x_tiles, const void *const *dy_tiles,
                              const float *const *scale_tiles, const float *const *shift_tiles,
                              const float *const *save_mean_tiles, const float *const *save_invstd_tiles,
                              void *const *dx_tiles, float *const *dscale_tiles, float *const *dshift_tiles,
                              float beta_data, float beta_param, void *workspace, size_t workspace_bytes,
                              void *stream);
/* CudnnActivationOp with kReluAct: cudnnActivationForward (src/op.cc:3236-3246), y = max(x, 0)
 * (x == y allowed: relu_in_place), and cudnnActivationBackward (src/op.cc:3313-3322),
 * dx = beta*dx + (y > 0 ? dy : 0). */
int adh_relu_fwd(int dtype, uint64_t n, const void *x, void *y, void *stream);
int adh_relu_bwd(int dtype, uint64_t n, const void *y, const void *dy, void *dx, float beta, void *stream);
/* SumJoinOp::_forward (src/op.cc:744-806): y = x_0 + x_1 + ... (the residual join); its backward
 * is adh_add_f32 / adh_slice_add_nchw of dy onto every input gradient. */
int adh_sum_fwd(int dtype, uint32_t num_inputs, uint64_t n, const void *const *xs, void *y, void *stream);

/* ---- pooling over the halo-padded slab ------------------------------------- */
/* CudnnPool2DOp with Pool2DShape::halo_padded_input (include/arraydiff/op.hh:2917-2925): the
 * padded tile (N, C, HP, WP) with HP = H + 2*pad_h, WP = W + 2*pad_w is handed to cuDNN as a plain
 * packed tensor with pooling pad 0 (src/op.cc:3424-3462), so the halo (neighbour rows after an
 * exchange, zeros at the image border) takes part as ordinary data.  Output extents are
 * OH = (HP - wh) / sh + 1, OW = (WP - ww) / sw + 1 (cudnnGetPooling2dForwardOutputDim).
 * ADH_POOL_MAX = CUDNN_POOLING_MAX, ADH_POOL_AVG = CUDNN_POOLING_AVERAGE_COUNT_INCLUDE_PADDING
 * (every window lies inside the padded tensor, so the divisor is always wh*ww).
 * fwd, cudnnPoolingForward beta 0 (src/op.cc:3496-3503): y = pool(x_pad).
 * bwd, cudnnPoolingBackward (src/op.cc:3610-3619): dx_pad = beta*dx_pad + pool'(dy), over the
 * WHOLE padded tile (the reference zeroes it on first touch and calls with beta 1).  For MAX the
 * gradient of a window goes to its first maximum in row-major window order; NaNs never win.
 * dtype f32 or bf16 (arithmetic in fp32).  beta is 0 or 1.  One launch covers all tiles. */
#define ADH_POOL_AVG 0 /* kAveragePool, include/arraydiff/op.hh:2912-2915 */
#define ADH_POOL_MAX 1 /* kMaxPool */
int adh_pool2d_slab_fwd_tiles(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t HP,
                              uint32_t WP, uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw,
                              const void *const *x_pad_tiles, void *const *y_tiles, void *stream);
int adh_pool2d_slab_fwd(int dtype, int mode, uint32_t N, uint32_t C, uint32_t HP, uint32_t WP, uint32_t wh,
                        uint32_t ww, uint32_t sh, uint32_t sw, const void *x_pad, void *y, void *stream);
int adh_pool2d_slab_bwd_tiles(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t HP,
                              uint32_t WP, uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw,
                              const void *const *x_pad_tiles, const void *const *y_tiles,
                              const void *const *dy_tiles, void *const *dx_pad_tiles, float beta, void *stream);
int adh_pool2d_slab_bwd(int dtype, int mode, uint32_t N, uint32_t C, uint32_t HP, uint32_t WP, uint32_t wh,
                        uint32_t ww, uint32_t sh, uint32_t sw, const void *x_pad, const void *y, const void *dy,
                        void *dx_pad, float beta, void *stream);
/* The chains HaloPad2DOp -> HaloExch2DOp -> CudnnPool2DOp and pooling backward -> halo reduce ->
 * HaloPad2DOp::_backward (src/zoo.cc:1562-1574 with src/op.cc:2574-2700, 2963-3052, 3496-3503, 3610-3619) as ONE
 * launch each over row tiles that carry NO halo: x_tiles / dx_tiles are the K row tiles (H x W, packed NCHW) of
 * one tensor in rank order, y_tiles / dy_tiles the tiles (H / sh rows, OW = (W + 2 pad_w - ww) / sw + 1 columns) of
 * the result.  Rows a window reaches outside a tile are read from the neighbouring tiles; outside the tensor a
 * window sees ZEROS, which take part as data exactly as the zeroed halo of the padded tile does (a window of
 * negative values at the border has maximum 0, and its gradient then belongs to no pixel).  Backward computes the
 * tile's own gradient completely: the windows of the tile below that reach into this tile are evaluated here too.
 * Limits: H a multiple of sh, 0 < wh - 2 pad_h <= sh, pad_h + floor((wh - 1 - pad_h) / sh) * sh <= H and
 * wh - 1 - pad_h <= H (windows, the neighbours' too, touch adjacent tiles only; ADH_EINVAL otherwise); a band
 * of window rows must fit in LDS (rows of up to a few thousand elements; ADH_EUNIMPL beyond: use the padded entry
 * points).  y_tiles of the backward call is not read (the maximum is recomputed) and may be NULL. */
/* ADH_OK when both calls below take this shape, else the code they would return (ADH_EINVAL: the row split does
 * not stitch; ADH_EUNIMPL: a band of window rows does not fit LDS), without launching anything: for callers that
 * choose between this form and pad -> exchange -> pooling over padded tiles when they build a graph. */
int adh_pool2d_unpadded_supported(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
                                  uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw, uint32_t pad_h, uint32_t pad_w);
int adh_pool2d_unpadded_fwd_tiles(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H,
                                  uint32_t W, uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw, uint32_t pad_h,
                                  uint32_t pad_w, const void *const *x_tiles, void *const *y_tiles, void *stream);
int adh_pool2d_unpadded_bwd_tiles(int dtype, int mode, uint32_t num_tiles, uint32_t N, uint32_t C, uint32_t H,
                                  uint32_t W, uint32_t wh, uint32_t ww, uint32_t sh, uint32_t sw, uint32_t pad_h,
                                  uint32_t pad_w, const void *const *x_tiles, const void *const *y_tiles,
                                  const void *const *dy_tiles, void *const *dx_tiles, float beta, void *stream);

/* ---- L1/L2/L3: softmax + negative log likelihood (fp32) ------------------- */
/* cudnnSoftmaxForward(ACCURATE, MODE_INSTANCE) on (N,C,1,1), src/op.cc:4129-4152 
 * In place (y == x) is allowed up to 2048 classes; beyond that a row is read again after y
 * has been written and the call returns ADH_EINVAL. */
int adh_softmax_fwd(uint32_t C, uint32_t N, const float *x, float *y, void *stream);
/* softmax_nll_loss_fwd<float>, src/kernels/softmax.cu:36-54,86-89 */
int adh_softmax_nll_loss_fwd(uint32_t C, uint32_t N, const float *y, const uint32_t *label,
                             float *loss, void *stream);
/* softmax_nll_loss_bwd<float>, src/kernels/softmax.cu:56-78,92-95: dx += dloss*(y - onehot) */
int adh_softmax_nll_loss_bwd(uint32_t C, uint32_t N, const float *y, const uint32_t *label,
                             const float *dloss, float *dx, void *stream);
/* CudnnSoftmaxNLLLossOp::_forward, src/op.cc:4118-4163, in one kernel: y and loss together */
int adh_softmax_xent_fwd(uint32_t C, uint32_t N, const float *x, const uint32_t *label, float *y,
                         float *loss, void *stream);
/* softmax_nll_loss_bwd with the two launches the reference puts before it folded in
 * (src/op.cc:4165-4188: the gradient is zeroed on first touch, then the kernel adds):
 * dx = beta*dx + dl*(y - onehot), beta 0 or 1, dl = dloss ? dloss[i] : dloss_all (a loss that is the
 * gradient sink seeds every example with one number, src/zoo.cc:1877-1878). */
int adh_softmax_nll_loss_bwd_scaled(uint32_t C, uint32_t N, const float *y, const uint32_t *label,
                                    const float *dloss, float dloss_all, float beta, float *dx,
                                    void *stream);
/* CudnnSoftmaxNLLLossOp::_forward and ::_backward (src/op.cc:4118-4188) in ONE kernel, for callers
 * that know the loss gradient when the logits arrive (a training step whose loss is the sink):
 * y and loss as adh_softmax_xent_fwd, dx as adh_softmax_nll_loss_bwd_scaled, bit for bit.
 * dx may alias x up to 2048 classes; it may not alias y. */
int adh_softmax_xent_fwd_bwd(uint32_t C, uint32_t N, const float *x, const uint32_t *label,
                             const float *dloss, float dloss_all, float *y, float *loss, float beta,
                             float *dx, void *stream);

/* ---- flat parameter vectors and the SGD update (fp32) ---------------------- */
/* array_add_scaled_packed<float>, src/kernels/array.cu:97-110,211-222: y = alpha*x + beta*y,
 * evaluated as fma(alpha, x, beta*y). */
int adh_scale_add_f32(uint64_t n, float alpha, const float *x, float beta, float *y, void *stream);
/* array_add_online_packed<float>, src/kernels/array.cu:112-124,224-234: y = y + alpha*(x - y),
 * evaluated as fma(alpha, x - y, y). */
int adh_add_online_f32(uint64_t n, float alpha, const float *x, float *y, void *stream);
/* The running-statistics update of ParallelSGDOptimizer::step (include/arraydiff/optimize.hh:507-514):
 * running_stat += rate*(avg_stat - running_stat); stat = running_stat, in one pass. */
int adh_stat_step_f32(uint64_t n, float rate, const float *avg_stat, float *running_stat, float *stat,
                      void *stream);
/* Op::store_val / store_grad (src/op.cc:170-194) and Op::load_val (src/op.cc:148-158) for one flat
 * vector: the arrays, in the order given, occupy consecutive ranges of `flat` starting at element
 * flat_offset (array i of lens[i] floats; a zero length is skipped).  store copies arrays -> flat,
 * load copies flat -> arrays.  One launch per 48 arrays instead of one copy per array. */
int adh_flat_store_f32(uint32_t num_arrays, const float *const *arrays, const uint64_t *lens, uint64_t flat_offset,
                       float *flat, void *stream);
int adh_flat_load_f32(uint32_t num_arrays, float *const *arrays, const uint64_t *lens, uint64_t flat_offset,
                      const float *flat, void *stream);
/* The parameter update of ParallelSGDOptimizer::step (include/arraydiff/optimize.hh:443-505) in one pass
 * over flat vectors of n floats:
 *   g = grads[0] + grads[1] + ... + grads[num_grads-1]      (the ncclReduce to rank 0, in rank order)
 *   if l2_reg != 0:  g = fma(l2_reg, param, g)
 *   momentum_grad = g + momentum*momentum_grad              (product rounded, then the sum)
 *   nesterov:  param = fma(-step_size, g, param); lagged_param = param;
 *              param = fma(-next_step_size*momentum, momentum_grad, param)
 *   else:      param = fma(-step_size, momentum_grad, param); lagged_param = param
 * lagged_param and sum_grad (receives g) may be NULL.  sum_grad may be grads[0]; no other aliasing.
 * 1 <= num_grads <= ADH_MAX_TILES. */
int adh_sgd_step_f32(uint64_t n, uint32_t num_grads, const float *const *grads, float l2_reg, float momentum,
                     float step_size, float next_step_size, int nesterov, float *param, float *momentum_grad,
                     float *lagged_param, float *sum_grad, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ADH_CAPI_H */
