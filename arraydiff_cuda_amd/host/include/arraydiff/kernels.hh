// Launcher-level seam: the reference's templated host launchers
// (include/arraydiff/kernels.hh:72-262), kept by name and argument order, each forwarding to the
// C ABI of libadh.so (include/adh_capi.h).  Only the `float` instantiations exist in the
// reference (src/kernels/*.cu) and here.  A launcher that fails throws AdhError where the
// reference's launch would have gone unchecked.
#ifndef ARRAYDIFF_KERNELS_HH
#define ARRAYDIFF_KERNELS_HH

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

#include "adh_capi.h"

namespace arraydiff {

void adh_check(int code, const char *what);

// src/kernels/array.cu:155-164, 199-208
template <typename T>
void array_set_constant_packed(uint32_t dim, T constant, T *x, hipStream_t stream);
template <>
inline void array_set_constant_packed<float>(uint32_t dim, float constant, float *x, hipStream_t stream) {
  adh_check(adh_fill_f32(dim, constant, x, stream), "array_set_constant_packed");
}
template <typename T>
void array_add_packed(uint32_t dim, const T *x, T *y, hipStream_t stream);
template <>
inline void array_add_packed<float>(uint32_t dim, const float *x, float *y, hipStream_t stream) {
  adh_check(adh_add_f32(dim, x, y, stream), "array_add_packed");
}

// src/kernels/array.cu:97-124, 211-234
template <typename T>
void array_add_scaled_packed(uint32_t dim, T alpha, T beta, const T *x, T *y, hipStream_t stream);
template <>
inline void array_add_scaled_packed<float>(uint32_t dim, float alpha, float beta, const float *x, float *y,
                                           hipStream_t stream) {
  adh_check(adh_scale_add_f32(dim, alpha, x, beta, y, stream), "array_add_scaled_packed");
}
template <typename T>
void array_add_online_packed(uint32_t dim, T alpha, const T *x, T *y, hipStream_t stream);
template <>
inline void array_add_online_packed<float>(uint32_t dim, float alpha, const float *x, float *y, hipStream_t stream) {
  adh_check(adh_add_online_f32(dim, alpha, x, y, stream), "array_add_online_packed");
}

// src/kernels/spatial.cu:455-510 (1x2), 596-652 (1x4), 708-731 (2x1): rank-wise launchers
namespace detail {
inline void halo_rank(bool reduce, uint32_t grid_w, uint32_t grid_h, uint32_t rank, uint32_t halo_pad, uint32_t w,
                      uint32_t h, uint32_t c, uint32_t n, float *const *bufs, hipStream_t stream) {
  void *tiles[ADH_MAX_TILES];
  for (uint32_t i = 0; i < grid_w * grid_h; ++i) tiles[i] = bufs[i];
  adh_check(reduce ? adh_halo_reduce_nchw_rank(ADH_F32, grid_w, grid_h, rank, halo_pad, w, h, c, n, tiles, stream)
                   : adh_halo_exchange_nchw_rank(ADH_F32, grid_w, grid_h, rank, halo_pad, w, h, c, n, tiles, stream),
            reduce ? "spatial2d halo reduce" : "spatial2d halo exchange");
}
}  // namespace detail

template <typename T>
void spatial2d_1x2_halo_exch_nchw(uint32_t rank, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
                                  uint32_t num_channels, uint32_t batch_size, T *x_0_with_halo, T *x_1_with_halo,
                                  hipStream_t stream) {
  T *b[2] = {x_0_with_halo, x_1_with_halo};
  detail::halo_rank(false, 1, 2, rank, halo_pad, base_width, base_height, num_channels, batch_size, b, stream);
}
template <typename T>
void spatial2d_1x2_halo_reduce_nchw(uint32_t rank, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
                                    uint32_t num_channels, uint32_t batch_size, T *x_0_with_halo, T *x_1_with_halo,
                                    hipStream_t stream) {
  T *b[2] = {x_0_with_halo, x_1_with_halo};
  detail::halo_rank(true, 1, 2, rank, halo_pad, base_width, base_height, num_channels, batch_size, b, stream);
}
template <typename T>
void spatial2d_1x4_halo_exch_nchw(uint32_t rank, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
                                  uint32_t num_channels, uint32_t batch_size, T *x_0_with_halo, T *x_1_with_halo,
                                  T *x_2_with_halo, T *x_3_with_halo, hipStream_t stream) {
  T *b[4] = {x_0_with_halo, x_1_with_halo, x_2_with_halo, x_3_with_halo};
  detail::halo_rank(false, 1, 4, rank, halo_pad, base_width, base_height, num_channels, batch_size, b, stream);
}
template <typename T>
void spatial2d_1x4_halo_reduce_nchw(uint32_t rank, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
                                    uint32_t num_channels, uint32_t batch_size, T *x_0_with_halo, T *x_1_with_halo,
                                    T *x_2_with_halo, T *x_3_with_halo, hipStream_t stream) {
  T *b[4] = {x_0_with_halo, x_1_with_halo, x_2_with_halo, x_3_with_halo};
  detail::halo_rank(true, 1, 4, rank, halo_pad, base_width, base_height, num_channels, batch_size, b, stream);
}
template <typename T>
void spatial2d_2x1_halo_exch_nchw(uint32_t rank, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
                                  uint32_t num_channels, uint32_t batch_size, T *x_0_with_halo, T *x_1_with_halo,
                                  hipStream_t stream) {
  T *b[2] = {x_0_with_halo, x_1_with_halo};
  detail::halo_rank(false, 2, 1, rank, halo_pad, base_width, base_height, num_channels, batch_size, b, stream);
}
// declared but never linked in the reference (src/spatial.cc:166-178); defined here
template <typename T>
void spatial2d_2x1_halo_reduce_nchw(uint32_t rank, uint32_t halo_pad, uint32_t base_width, uint32_t base_height,
                                    uint32_t num_channels, uint32_t batch_size, T *x_0_with_halo, T *x_1_with_halo,
                                    hipStream_t stream) {
  T *b[2] = {x_0_with_halo, x_1_with_halo};
  detail::halo_rank(true, 2, 1, rank, halo_pad, base_width, base_height, num_channels, batch_size, b, stream);
}

// src/kernels/slice.cu:43-105
template <typename T>
void slice2d_copy_hw_nchw_packed(uint32_t count_w, uint32_t count_h, uint32_t src_width, uint32_t src_height,
                                 uint32_t dst_width, uint32_t dst_height, uint32_t channels, uint32_t batch_size,
                                 const T *src, uint32_t src_w_off, uint32_t src_h_off, T *dst, uint32_t dst_w_off,
                                 uint32_t dst_h_off, hipStream_t stream) {
  adh_check(adh_slice_copy_nchw(ADH_F32, count_w, count_h, channels, batch_size, src, src_width, src_height, channels,
                                src_w_off, src_h_off, 0, dst, dst_width, dst_height, channels, dst_w_off, dst_h_off, 0,
                                stream),
            "slice2d_copy_hw_nchw_packed");
}
template <typename T>
void slice2d_add_hw_nchw_packed(uint32_t count_w, uint32_t count_h, uint32_t src_width, uint32_t src_height,
                                uint32_t dst_width, uint32_t dst_height, uint32_t channels, uint32_t batch_size,
                                const T *src, uint32_t src_w_off, uint32_t src_h_off, T *dst, uint32_t dst_w_off,
                                uint32_t dst_h_off, hipStream_t stream) {
  adh_check(adh_slice_add_nchw(ADH_F32, count_w, count_h, channels, batch_size, src, src_width, src_height, channels,
                               src_w_off, src_h_off, 0, dst, dst_width, dst_height, channels, dst_w_off, dst_h_off, 0,
                               stream),
            "slice2d_add_hw_nchw_packed");
}

// src/kernels/softmax.cu:86-95 (softmax_fwd there is a debug stub; here it is the real
// max-subtracted softmax that cudnnSoftmaxForward provided, src/op.cc:4129-4152)
template <typename T>
void softmax_fwd(uint32_t num_channels, uint32_t batch_size, const T *x, T *y, hipStream_t stream) {
  adh_check(adh_softmax_fwd(num_channels, batch_size, x, y, stream), "softmax_fwd");
}
template <typename T>
void softmax_nll_loss_fwd(uint32_t num_channels, uint32_t batch_size, const T *y, const uint32_t *label, T *loss,
                          hipStream_t stream) {
  adh_check(adh_softmax_nll_loss_fwd(num_channels, batch_size, y, label, loss, stream), "softmax_nll_loss_fwd");
}
template <typename T>
void softmax_nll_loss_bwd(uint32_t num_channels, uint32_t batch_size, const T *y, const uint32_t *label,
                          const T *dloss, T *dx, hipStream_t stream) {
  adh_check(adh_softmax_nll_loss_bwd(num_channels, batch_size, y, label, dloss, dx, stream), "softmax_nll_loss_bwd");
}

}  // namespace arraydiff

#endif
