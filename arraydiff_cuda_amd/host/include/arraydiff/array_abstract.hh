// Index algebra of the spatial path: shapes with the FASTEST dimension first.
//
// Mirrors the interface of the reference's Shape0D..Shape4D
// (include/arraydiff/array_abstract.hh:18-341: major/minor/flat_size/append/packed_stride/
// packed_dim/is_packed/is_zero/to_index, public member `shape`), written once as a template
// over the rank instead of five hand-expanded classes.  Shape3D(d0,d1,d2) = (W,H,C); the batch
// dimension is appended as the slowest one, which makes memory cuDNN-NCHW.
#ifndef ARRAYDIFF_ARRAY_ABSTRACT_HH
#define ARRAYDIFF_ARRAY_ABSTRACT_HH

#include <array>
#include <cstddef>
#include <ostream>

namespace arraydiff {

template <size_t D>
class ShapeND {
public:
  typedef ShapeND<D + 1> Upper;

  static ShapeND Zero() { return ShapeND(); }

  ShapeND() { shape.fill(0); }
  template <typename... Ts, typename = typename std::enable_if<sizeof...(Ts) == D && (D > 0)>::type>
  ShapeND(Ts... dims) : shape{{static_cast<size_t>(dims)...}} {}

  // fastest / slowest extent (1 for rank 0 so that products stay neutral)
  size_t major() const { return D ? shape[0] : 1; }
  size_t minor() const { return D ? shape[D - 1] : 1; }

  size_t flat_size() const {
    size_t n = 1;
    for (size_t i = 0; i < D; ++i) n *= shape[i];
    return n;
  }

  Upper append(size_t slowest) const {
    Upper up;
    for (size_t i = 0; i < D; ++i) up.shape[i] = shape[i];
    up.shape[D] = slowest;
    return up;
  }

  // strides of a dense array of these extents: stride[0] = 1, stride[i] = stride[i-1]*dim[i-1]
  ShapeND packed_stride() const {
    ShapeND s;
    size_t acc = 1;
    for (size_t i = 0; i < D; ++i) {
      s.shape[i] = acc;
      acc *= shape[i];
    }
    return s;
  }

  // inverse of packed_stride for `*this` used AS a stride: the extents of the dense buffer that
  // has these strides, given its slowest extent
  ShapeND packed_dim(size_t slowest) const {
    ShapeND d;
    for (size_t i = 0; i + 1 < D; ++i) d.shape[i] = shape[i + 1] / shape[i];
    if (D) d.shape[D - 1] = slowest;
    return d;
  }

  bool is_packed(const ShapeND &stride) const { return packed_stride().shape == stride.shape; }

  bool is_zero() const {
    for (size_t i = 0; i < D; ++i)
      if (shape[i]) return false;
    return true;
  }

  // dot product with a stride: the linear index of coordinate *this
  size_t to_index(const ShapeND &stride) const {
    size_t idx = 0;
    for (size_t i = 0; i < D; ++i) idx += stride.shape[i] * shape[i];
    return idx;
  }

  bool operator==(const ShapeND &o) const { return shape == o.shape; }
  bool operator!=(const ShapeND &o) const { return !(*this == o); }

  std::array<size_t, D> shape;
};

template <size_t D>
std::ostream &operator<<(std::ostream &os, const ShapeND<D> &s) {
  os << "Shape" << D << "D(";
  for (size_t i = 0; i < D; ++i) os << (i ? ", " : "") << s.shape[i];
  return os << ")";
}

typedef ShapeND<0> Shape0D;
typedef ShapeND<1> Shape1D;
typedef ShapeND<2> Shape2D;
typedef ShapeND<3> Shape3D;
typedef ShapeND<4> Shape4D;

}  // namespace arraydiff

#endif
