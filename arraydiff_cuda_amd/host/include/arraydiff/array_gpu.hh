// Device arrays of the spatial path.
//
// Mirrors the parts of the reference's GPUMemory / GPUArray / GPUBatchArray that the path uses
// (include/arraydiff/array_gpu.hh:27-65, 67-287, 289-492, 494-689): an array is
// (memory, dim, offset, stride), all fastest-dimension-first; a halo-padded batch array has
// dim = (W,H,C), offset = (p,p,0), stride = packed stride of (W+2p, H+2p, C); as_view() points
// at the interior origin, base_as_view() at the padded buffer base with dims (W+2p,H+2p,C,N).
// Unlike the reference (which never frees, array_gpu.hh:105-109) memory is released when the
// last owner goes away.
#ifndef ARRAYDIFF_ARRAY_GPU_HH
#define ARRAYDIFF_ARRAY_GPU_HH

#include "arraydiff/array_abstract.hh"
#include "arraydiff/context.hh"
#include "arraydiff/kernels.hh"

#include <cassert>
#include <cstdint>
#include <memory>
#include <stdexcept>

namespace arraydiff {

// hipMalloc / hipFree / copies, out of line so that this header needs no HIP launch syntax
void *gpu_alloc_bytes(size_t bytes);
void gpu_free_bytes(void *p);
void gpu_copy_h2d(void *dst, const void *src, size_t bytes, hipStream_t stream);
void gpu_copy_d2h(void *dst, const void *src, size_t bytes, hipStream_t stream);
void gpu_copy_d2d(void *dst, const void *src, size_t bytes, hipStream_t stream);

template <typename T>
class GPUMemory {
public:
  GPUMemory() : size_(0) {}
  // sizes are rounded up to 4 KiB like the reference (array_gpu.hh:37-44)
  GPUMemory(size_t size, GPUContext *ctx) : size_(size) {
    (void)ctx;
    const size_t bytes = (size * sizeof(T) + 4095) / 4096 * 4096;
    ptr_ = std::shared_ptr<void>(gpu_alloc_bytes(bytes ? bytes : 4096), gpu_free_bytes);
  }
  void reallocate(size_t size, GPUContext *ctx) { *this = GPUMemory<T>(size, ctx); }
  // array_gpu.hh:46-65
  static GPUMemory Zeros(size_t size, GPUContext *ctx) {
    static_assert(sizeof(T) == 4, "Zeros is a 32-bit fill");
    GPUMemory m(size, ctx);
    GPUConn conn = ctx->conn();
    m.set_constant(T(), conn);
    return m;
  }
  // whole-vector arithmetic of the optimizers (array_gpu.hh:150-215); ranges are checked here
  void set_constant(T c, GPUConn &conn) {
    float f;
    __builtin_memcpy(&f, &c, 4);
    array_set_constant_packed<float>((uint32_t)size_, f, reinterpret_cast<float *>(dptr()), conn.stream());
  }
  void add(GPUMemory<T> src, size_t buf_sz, size_t dst_offset, size_t src_offset, GPUConn &conn) {
    check_range(src, buf_sz, dst_offset, src_offset);
    array_add_packed<T>((uint32_t)buf_sz, src.dptr() + src_offset, dptr() + dst_offset, conn.stream());
  }
  void add_scaled(T alpha, GPUMemory<T> src, T beta, size_t buf_sz, size_t dst_offset, size_t src_offset, GPUConn &conn) {
    check_range(src, buf_sz, dst_offset, src_offset);
    array_add_scaled_packed<T>((uint32_t)buf_sz, alpha, beta, src.dptr() + src_offset, dptr() + dst_offset, conn.stream());
  }
  void add_online(T alpha, GPUMemory<T> src, size_t buf_sz, size_t dst_offset, size_t src_offset, GPUConn &conn) {
    check_range(src, buf_sz, dst_offset, src_offset);
    array_add_online_packed<T>((uint32_t)buf_sz, alpha, src.dptr() + src_offset, dptr() + dst_offset, conn.stream());
  }
  void copy(GPUMemory<T> src, size_t buf_sz, size_t dst_offset, size_t src_offset, GPUConn &conn) {
    check_range(src, buf_sz, dst_offset, src_offset);
    gpu_copy_d2d(dptr() + dst_offset, src.dptr() + src_offset, buf_sz * sizeof(T), conn.stream());
  }

  T *dptr() const { return static_cast<T *>(ptr_.get()); }
  uintptr_t dptr_addr() const { return reinterpret_cast<uintptr_t>(ptr_.get()); }
  size_t size() const { return size_; }

  void load_sync(const T *src, size_t offset, size_t count, GPUConn &conn) {
    assert(offset + count <= size_);
    gpu_copy_h2d(dptr() + offset, src, count * sizeof(T), conn.stream());
    conn.sync();
  }
  void store_sync(T *dst, size_t offset, size_t count, GPUConn &conn) {
    assert(offset + count <= size_);
    gpu_copy_d2h(dst, dptr() + offset, count * sizeof(T), conn.stream());
    conn.sync();
  }

private:
  void check_range(const GPUMemory<T> &src, size_t n, size_t dst_offset, size_t src_offset) const {
    if (dst_offset + n > size_ || src_offset + n > src.size_) throw std::out_of_range("GPUMemory: range outside the buffer");
  }
  std::shared_ptr<void> ptr_;
  size_t size_;
};

// A strided view (or, through the owning constructor, a dense owner) of device memory.
template <typename Dim, typename T>
class GPUArray {
public:
  typedef GPUContext Ctx;
  typedef Dim Shape;

  static GPUArray Zeros(Dim dim, GPUContext *ctx) {
    GPUArray arr(dim, ctx);
    GPUConn conn = ctx->conn();
    arr.set_constant(static_cast<T>(0), conn);
    return arr;
  }

  GPUArray() {}
  GPUArray(Dim dim, GPUContext *ctx)
      : mem_(dim.flat_size(), ctx), dim_(dim), offset_(Dim::Zero()), stride_(dim.packed_stride()) {}
  GPUArray(GPUMemory<T> mem, Dim dim, Dim offset, Dim stride) : mem_(mem), dim_(dim), offset_(offset), stride_(stride) {}

  Dim dim() const { return dim_; }
  Dim offset() const { return offset_; }
  Dim stride() const { return stride_; }
  bool is_packed() const { return offset_.is_zero() && dim_.is_packed(stride_); }

  // pointer to element `offset` (array_gpu.hh:329-341)
  T *dptr() const { return mem_.dptr() + offset_.to_index(stride_); }
  T *base_dptr() const { return mem_.dptr(); }

  // Fills stride.minor()*dim.minor() elements from the BASE pointer, whatever the view
  // (array_gpu.hh:361-368): on a padded array this clears interior and halo alike.
  void set_constant(T c, GPUConn &conn) {
    static_assert(sizeof(T) == 4, "set_constant is a 32-bit fill");
    float f;
    __builtin_memcpy(&f, &c, 4);
    array_set_constant_packed<float>((uint32_t)(stride_.minor() * dim_.minor()), f,
                                     reinterpret_cast<float *>(mem_.dptr()), conn.stream());
  }
  // y += x for two dense arrays of the same extent (array_gpu.hh:369-382)
  void add(const GPUArray &x, GPUConn &conn) {
    assert(is_packed() && x.is_packed() && dim_ == x.dim_);
    array_add_packed<float>((uint32_t)dim_.flat_size(), reinterpret_cast<const float *>(x.dptr()),
                            reinterpret_cast<float *>(dptr()), conn.stream());
  }
  void load_sync(const T *src, GPUConn &conn) {
    assert(is_packed());
    mem_.load_sync(src, 0, dim_.flat_size(), conn);
  }
  void store_sync(T *dst, GPUConn &conn) {
    assert(is_packed());
    mem_.store_sync(dst, 0, dim_.flat_size(), conn);
  }

private:
  GPUMemory<T> mem_;
  Dim dim_, offset_, stride_;
};

template <typename Dim, typename T>
class GPUBatchArray {
public:
  typedef GPUContext Ctx;
  typedef Dim Shape;
  typedef typename Dim::Upper Upper;

  static GPUBatchArray Zeros(Dim dim, size_t batch_capacity, GPUContext *ctx) {
    GPUBatchArray arr(dim, batch_capacity, ctx);
    GPUConn conn = ctx->conn();
    arr.as_view().set_constant(static_cast<T>(0), conn);
    return arr;
  }
  // GPUBatchArray::ZerosPadded, array_gpu.hh:508-519
  static GPUBatchArray ZerosPadded(Dim dim, Dim offset, Dim stride, size_t batch_capacity, GPUContext *ctx) {
    if (offset.is_zero() && dim.is_packed(stride)) return Zeros(dim, batch_capacity, ctx);
    GPUBatchArray arr(dim, offset, stride, batch_capacity, ctx);
    GPUConn conn = ctx->conn();
    arr.base_as_view().set_constant(static_cast<T>(0), conn);
    return arr;
  }

  GPUBatchArray(Dim dim, size_t batch_capacity, GPUContext *ctx)
      : dim_(dim), offset_(Dim::Zero()), stride_(dim.packed_stride()), batch_cap_(batch_capacity),
        batch_size_(batch_capacity), mem_(dim.flat_size() * batch_capacity, ctx) {
    assert(batch_capacity >= 1);
  }
  GPUBatchArray(Dim dim, Dim offset, Dim stride, size_t batch_capacity, GPUContext *ctx)
      : dim_(dim), offset_(offset), stride_(stride), batch_cap_(batch_capacity), batch_size_(batch_capacity),
        mem_(stride.minor() * dim.minor() * batch_capacity, ctx) {
    assert(batch_capacity >= 1);
  }

  // interior view: dims (dim, batch), offset (offset, 0)
  GPUArray<Upper, T> as_view() {
    return GPUArray<Upper, T>(mem_, dim_.append(batch_size_), offset_.append(0),
                              stride_.append(stride_.minor() * dim_.minor()));
  }
  // whole padded buffer: dims recovered from the strides, offset 0
  GPUArray<Upper, T> base_as_view() {
    return GPUArray<Upper, T>(mem_, stride_.packed_dim(dim_.minor()).append(batch_size_), Upper::Zero(),
                              stride_.append(stride_.minor() * dim_.minor()));
  }

  Dim dim() const { return dim_; }
  Dim offset() const { return offset_; }
  Dim stride() const { return stride_; }
  size_t batch_capacity() const { return batch_cap_; }
  size_t batch_size() const { return batch_size_; }
  size_t set_batch_size(size_t n) {
    assert(n <= batch_cap_);
    return batch_size_ = n;
  }
  uintptr_t dptr_addr() const { return mem_.dptr_addr(); }

  // dense host <-> device transfer of the first batch_size() items of a PACKED array
  void load_sync(const T *src, GPUConn &conn) {
    assert(offset_.is_zero() && dim_.is_packed(stride_));
    mem_.load_sync(src, 0, dim_.flat_size() * batch_size_, conn);
  }
  void store_sync(T *dst, GPUConn &conn) {
    assert(offset_.is_zero() && dim_.is_packed(stride_));
    mem_.store_sync(dst, 0, dim_.flat_size() * batch_size_, conn);
  }
  // the whole padded buffer (halo included), for tests
  void store_base_sync(T *dst, GPUConn &conn) { mem_.store_sync(dst, 0, stride_.minor() * dim_.minor() * batch_size_, conn); }
  void load_base_sync(const T *src, GPUConn &conn) { mem_.load_sync(src, 0, stride_.minor() * dim_.minor() * batch_size_, conn); }

private:
  Dim dim_, offset_, stride_;
  size_t batch_cap_, batch_size_;
  GPUMemory<T> mem_;
};

template <typename T> using GPUArray1D = GPUArray<Shape1D, T>;
template <typename T> using GPUArray4D = GPUArray<Shape4D, T>;
template <typename T> using GPUBatchArray0D = GPUBatchArray<Shape0D, T>;
template <typename T> using GPUBatchArray1D = GPUBatchArray<Shape1D, T>;
template <typename T> using GPUBatchArray3D = GPUBatchArray<Shape3D, T>;

}  // namespace arraydiff

#endif
