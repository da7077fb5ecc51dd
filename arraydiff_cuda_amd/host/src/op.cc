// _forward / _backward of the spatial-path ops for float tiles: argument checks as in the
// reference's src/op.cc (cited per op), arithmetic behind the C ABI.
#include "arraydiff/op.hh"

#include "adh_capi.h"

namespace arraydiff {

uint64_t next_raw_id(int kind) {
  static thread_local uint64_t counters[4] = {0, 0, 0, 0};
  return ++counters[kind & 3];
}

typedef GPUBatchArray3D<float> V3;
typedef GPUArray4D<float> A4;

namespace {

struct TileDims {
  uint32_t W, H, C, N;
};
TileDims dims_of(V3 &a) {
  auto d = a.dim();
  return TileDims{(uint32_t)d.shape[0], (uint32_t)d.shape[1], (uint32_t)d.shape[2], (uint32_t)a.batch_size()};
}

// offset == (p,p,0) and stride == packed stride of the padded extents (op.cc:2587-2609)
void check_padded(V3 &a, size_t p, const char *who) {
  auto d = a.dim();
  auto want = Shape3D(d.shape[0] + 2 * p, d.shape[1] + 2 * p, d.shape[2]).packed_stride();
  if (a.offset() != Shape3D(p, p, 0) || a.stride() != want)
    throw std::invalid_argument(std::string(who) + ": array is not halo-padded by the expected width");
}
void check_packed(V3 &a, const char *who) {
  if (!a.offset().is_zero() || !a.dim().is_packed(a.stride()))
    throw std::invalid_argument(std::string(who) + ": array is not packed");
}

}  // namespace

// ---- flat-vector plumbing (op.cc:148-212) ----
namespace {
enum FlatKind { kLoadVal, kLoadGrad, kStoreVal, kStoreGrad };

// Visits every node once on the way back out of the graph (the order of the reference's walk),
// collects the arrays of `vars`, then moves them with one batched copy.
size_t flat_walk(Op *root, FlatKind kind, TxnId txn, VarIdSet &vars, size_t offset, GPUMemory<float> *mem) {
  const bool is_load = kind == kLoadVal || kind == kLoadGrad;
  if (is_load && !mem) throw std::invalid_argument("load from a flat vector needs the vector");
  FlatBatch batch;
  FlatBatch *b = mem ? &batch : nullptr;
  size_t end = offset;
  vars.lock();
  try {
    EpochId e;
    root->_push(e, [](Op *) {});
    root->_pop(e, [&](Op *op) {
      switch (kind) {
        case kLoadVal: end = op->_load_val(txn, vars, end, b); break;
        case kLoadGrad: end = op->_load_grad(txn, vars, end, b); break;
        case kStoreVal: end = op->_store_val(txn, vars, end, b); break;
        case kStoreGrad: end = op->_store_grad(txn, vars, end, b); break;
      }
    });
  } catch (...) {
    vars.unlock();
    throw;
  }
  vars.unlock();
  if (!mem || batch.arrays.empty()) return end;
  if (end > mem->size()) throw std::invalid_argument("flat vector shorter than the variables it should hold");
  if (is_load)
    adh_check(adh_flat_load_f32((uint32_t)batch.arrays.size(), batch.arrays.data(), batch.lens.data(), offset, mem->dptr(),
                                batch.stream),
              "Op::load_val");
  else
    adh_check(adh_flat_store_f32((uint32_t)batch.arrays.size(), batch.arrays.data(), batch.lens.data(), offset,
                                 mem->dptr(), batch.stream),
              "Op::store_val");
  return end;
}
}  // namespace

size_t Op::load_val(TxnId txn, VarIdSet &vars, size_t offset, GPUMemory<float> *reader) {
  return flat_walk(this, kLoadVal, txn, vars, offset, reader);
}
size_t Op::load_grad(TxnId txn, VarIdSet &vars, size_t offset, GPUMemory<float> *reader) {
  return flat_walk(this, kLoadGrad, txn, vars, offset, reader);
}
size_t Op::store_val(TxnId txn, VarIdSet &vars, size_t offset, GPUMemory<float> *writer) {
  return flat_walk(this, kStoreVal, txn, vars, offset, writer);
}
size_t Op::store_grad(TxnId txn, VarIdSet &vars, size_t offset, GPUMemory<float> *writer) {
  return flat_walk(this, kStoreGrad, txn, vars, offset, writer);
}
void Op::persist(TxnId txn, VarIdSet &vars) {
  EpochId e;
  _push(e, [txn, &vars](Op *op) { op->_persist(txn, vars); });
  _pop(e, [](Op *) {});
}
void Op::init(TxnId txn, std::mt19937_64 *rng) {
  EpochId e;
  _push(e, [txn, rng](Op *op) { op->_init(txn, rng); });
  _pop(e, [](Op *) {});
}

// ---- SpatialScatter2DOp (op.cc:2396-2468) ----
template <>
void SpatialScatter2DOp<V3>::_forward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &x = x_.val().get(txn, id());
  const TileDims xd = dims_of(x);
  if (y_.val().overwrite(txn, id(), ctx)) {
    GPUConn conn = ctx->conn();
    V3 &y = y_.val().get_excl(txn, id());
    y.set_batch_size(xd.N);
    check_packed(x, "SpatialScatter2DOp");
    const uint32_t Ht = xd.H / (uint32_t)num_ranks_;
    slice2d_copy_hw_nchw_packed<float>(xd.W, Ht, xd.W, xd.H, xd.W, Ht, xd.C, xd.N, x.as_view().dptr(), 0,
                                       (uint32_t)rank_ * Ht, y.as_view().dptr(), 0, 0, conn.stream());
  }
}
template <>
void SpatialScatter2DOp<V3>::_backward(TxnId txn) {
  if (!_requires_grad()) return;  // nothing below needs this gradient, and nobody produced ours
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &dy = y_.grad().get(txn, id());
  const TileDims yd = dims_of(dy);
  const size_t batch = yd.N;
  if (x_.grad().accumulate(txn, id(), ctx, [ctx, batch](V3 *g) {
        GPUConn conn = ctx->conn();
        g->set_batch_size(batch);
        g->as_view().set_constant(0.0f, conn);
      })) {
    GPUConn conn = ctx->conn();
    V3 &dx = x_.grad().get_mut(txn, id());
    const TileDims xd = dims_of(dx);
    slice2d_add_hw_nchw_packed<float>(xd.W, yd.H, xd.W, yd.H, xd.W, xd.H, xd.C, xd.N, dy.as_view().dptr(), 0, 0,
                                      dx.as_view().dptr(), 0, (uint32_t)rank_ * yd.H, conn.stream());
  }
}

// ---- SpatialGather2DOp (op.cc:2480-2553) ----
template <>
void SpatialGather2DOp<V3>::_forward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &x = x_.val().get(txn, id());
  const TileDims xd = dims_of(x);
  const size_t batch = xd.N;
  if (y_.val().accumulate(txn, id(), ctx, [ctx, batch](V3 *v) {
        GPUConn conn = ctx->conn();
        v->set_batch_size(batch);
        v->as_view().set_constant(0.0f, conn);
      })) {
    GPUConn conn = ctx->conn();
    V3 &y = y_.val().get_mut(txn, id());
    const TileDims yd = dims_of(y);
    slice2d_copy_hw_nchw_packed<float>(xd.W, xd.H, xd.W, xd.H, yd.W, yd.H, xd.C, xd.N, x.as_view().dptr(), 0, 0,
                                       y.as_view().dptr(), 0, (uint32_t)rank_ * xd.H, conn.stream());
  }
}
template <>
void SpatialGather2DOp<V3>::_backward(TxnId txn) {
  if (!_requires_grad()) return;  // nothing below needs this gradient, and nobody produced ours
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &dy = y_.grad().get(txn, id());
  const TileDims yd = dims_of(dy);
  const size_t batch = yd.N;
  if (x_.grad().accumulate(txn, id(), ctx, [ctx, batch](V3 *g) {
        GPUConn conn = ctx->conn();
        g->set_batch_size(batch);
        g->as_view().set_constant(0.0f, conn);
      })) {
    GPUConn conn = ctx->conn();
    V3 &dx = x_.grad().get_mut(txn, id());
    const TileDims xd = dims_of(dx);
    slice2d_add_hw_nchw_packed<float>(xd.W, xd.H, yd.W, yd.H, xd.W, xd.H, xd.C, xd.N, dy.as_view().dptr(), 0,
                                      (uint32_t)rank_ * xd.H, dx.as_view().dptr(), 0, 0, conn.stream());
  }
}

// ---- SpatialJoinedGather2DOp: gather of src/zoo.cc:1841-1842 without the zero-fill + allreduce ----
template <>
void SpatialJoinedGather2DOp<V3>::_forward(TxnId txn) {
  MultiGPUContext *ctx = mgpu_ctx_of(ctx_);
  GPUContext *dc = ctx->device_context(0).get();
  if (y_.val().overwrite(txn, id(), dc)) {
    const void *tiles[ADH_MAX_TILES];
    TileDims d{};
    for (size_t r = 0; r < xs_.size(); ++r) {
      V3 &x = xs_[r].val().get(txn, id());
      check_packed(x, "SpatialJoinedGather2DOp");
      d = dims_of(x);
      tiles[r] = x.as_view().dptr();
    }
    V3 &y = y_.val().get_excl(txn, id());
    y.set_batch_size(d.N);
    GPUConn conn = dc->conn();
    adh_check(adh_tiles_unpack_nchw(ADH_F32, (uint32_t)xs_.size(), 0, d.W, d.H * (uint32_t)xs_.size(), d.C, d.N, tiles,
                                    y.as_view().dptr(), conn.stream()),
              "SpatialJoinedGather2DOp::_forward");
  }
}
template <>
void SpatialJoinedGather2DOp<V3>::_backward(TxnId txn) {
  MultiGPUContext *ctx = mgpu_ctx_of(ctx_);
  V3 &dy = y_.grad().get(txn, id());
  const TileDims yd = dims_of(dy);
  const size_t batch = yd.N;
  for (size_t r = 0; r < xs_.size(); ++r) {
    GPUContext *dc = ctx->device_context(r).get();
    // the first toucher of a tile's gradient copies its rows, later ones add (the reference zeroes, then adds)
    bool first = false;
    if (xs_[r].grad().accumulate(txn, id(), dc, [batch, &first](V3 *g) {
          g->set_batch_size(batch);
          first = true;
        })) {
      GPUConn conn = dc->conn();
      V3 &dx = xs_[r].grad().get_mut(txn, id());
      const TileDims xd = dims_of(dx);
      if (first)
        slice2d_copy_hw_nchw_packed<float>(xd.W, xd.H, yd.W, yd.H, xd.W, xd.H, xd.C, xd.N, dy.as_view().dptr(), 0,
                                           (uint32_t)r * xd.H, dx.as_view().dptr(), 0, 0, conn.stream());
      else
        slice2d_add_hw_nchw_packed<float>(xd.W, xd.H, yd.W, yd.H, xd.W, xd.H, xd.C, xd.N, dy.as_view().dptr(), 0,
                                          (uint32_t)r * xd.H, dx.as_view().dptr(), 0, 0, conn.stream());
    }
  }
}

// ---- HaloPad2DOp (op.cc:2574-2712) ----
template <>
void HaloPad2DOp<V3>::_forward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &x = x_.val().get(txn, id());
  const TileDims xd = dims_of(x);
  const size_t batch = xd.N;
  // the pad kernel writes border and interior in one pass, so the first-touch step only has
  // to size the batch (the reference zero-fills here and then copies, op.cc:2581-2585,2634)
  if (y_.val().accumulate(txn, id(), ctx, [batch](V3 *v) { v->set_batch_size(batch); })) {
    GPUConn conn = ctx->conn();
    V3 &y = y_.val().get_mut(txn, id());
    check_packed(x, "HaloPad2DOp");
    check_padded(y, halo_pad_, "HaloPad2DOp");
    if (y.dim() != x.dim() || y.batch_size() != batch) throw std::invalid_argument("HaloPad2DOp: shape mismatch");
    adh_check(adh_halo_pad_nchw(ADH_F32, (uint32_t)halo_pad_, xd.W, xd.H, xd.C, xd.N, x.as_view().dptr(),
                                y.base_as_view().dptr(), conn.stream()),
              "HaloPad2DOp::_forward");
  }
}
template <>
void HaloPad2DOp<V3>::_backward(TxnId txn) {
  if (!_requires_grad()) return;  // nothing below needs this gradient, and nobody produced ours
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &dy = y_.grad().get(txn, id());
  const TileDims d = dims_of(dy);
  const size_t batch = d.N;
  // the first toucher of the input gradient overwrites it with the interior, later ones add
  bool first = false;
  if (x_.grad().accumulate(txn, id(), ctx, [batch, &first](V3 *g) {
        g->set_batch_size(batch);
        first = true;
      })) {
    GPUConn conn = ctx->conn();
    V3 &dx = x_.grad().get_mut(txn, id());
    check_padded(dy, halo_pad_, "HaloPad2DOp");
    adh_check(first ? adh_halo_unpad_nchw(ADH_F32, (uint32_t)halo_pad_, d.W, d.H, d.C, d.N, dy.base_as_view().dptr(),
                                          dx.as_view().dptr(), conn.stream())
                    : adh_halo_unpad_add_nchw(ADH_F32, (uint32_t)halo_pad_, d.W, d.H, d.C, d.N, dy.base_as_view().dptr(),
                                              dx.as_view().dptr(), conn.stream()),
              "HaloPad2DOp::_backward");
  }
}

// ---- HaloUnpad2DOp (op.cc:2715-2870) ----
template <>
void HaloUnpad2DOp<V3>::_forward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &x = x_.val().get(txn, id());
  const TileDims d = dims_of(x);
  if (y_.val().overwrite(txn, id(), ctx)) {
    GPUConn conn = ctx->conn();
    V3 &y = y_.val().get_excl(txn, id());
    y.set_batch_size(d.N);
    check_padded(x, halo_pad_, "HaloUnpad2DOp");  // op.cc:2746-2748
    adh_check(adh_halo_unpad_nchw(ADH_F32, (uint32_t)halo_pad_, d.W, d.H, d.C, d.N, x.base_as_view().dptr(),
                                  y.as_view().dptr(), conn.stream()),
              "HaloUnpad2DOp::_forward");
  }
}
template <>
void HaloUnpad2DOp<V3>::_backward(TxnId txn) {
  if (!_requires_grad()) return;  // nothing below needs this gradient, and nobody produced ours
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &dy = y_.grad().get(txn, id());
  const TileDims d = dims_of(dy);
  const size_t batch = d.N;
  if (x_.grad().accumulate(txn, id(), ctx, [ctx, batch](V3 *g) {
        GPUConn conn = ctx->conn();
        g->set_batch_size(batch);
        g->base_as_view().set_constant(0.0f, conn);
      })) {
    GPUConn conn = ctx->conn();
    V3 &dx = x_.grad().get_mut(txn, id());
    check_padded(dx, halo_pad_, "HaloUnpad2DOp");
    adh_check(adh_halo_pad_add_nchw(ADH_F32, (uint32_t)halo_pad_, d.W, d.H, d.C, d.N, dy.as_view().dptr(),
                                    dx.base_as_view().dptr(), conn.stream()),
              "HaloUnpad2DOp::_backward");
  }
}

// ---- HaloRepad2DOp (op.cc:2873-2960) ----
template <>
void HaloRepad2DOp<V3>::_forward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &x = x_.val().get(txn, id());
  const TileDims d = dims_of(x);
  const size_t batch = d.N;
  if (y_.val().accumulate(txn, id(), ctx, [batch](V3 *v) { v->set_batch_size(batch); })) {
    GPUConn conn = ctx->conn();
    V3 &y = y_.val().get_mut(txn, id());
    check_padded(x, src_pad_, "HaloRepad2DOp");
    check_padded(y, dst_pad_, "HaloRepad2DOp");
    adh_check(adh_halo_repad_nchw(ADH_F32, (uint32_t)src_pad_, (uint32_t)dst_pad_, d.W, d.H, d.C, d.N,
                                  x.base_as_view().dptr(), y.base_as_view().dptr(), conn.stream()),
              "HaloRepad2DOp::_forward");
  }
}

// ---- HaloExch2DOp (op.cc:2963-3052) ----
// All ranks or none take part (op.cc:2973,3021).  The reference brackets the exchange with two
// host-side syncs of every device (op.cc:2976,3001); with all tiles on one in-order stream the
// producers' kernels are already ordered before it, so there is nothing to wait for.
template <>
void HaloExch2DOp<V3>::_forward(TxnId txn) {
  MultiGPUContext *ctx = mgpu_ctx_of(ctx_);
  size_t num_writes = 0;
  for (size_t r = 0; r < ctx->num_ranks(); ++r)
    if (xs_.at(r).val().accumulate(txn, id(), ctx->device_context(r).get(), [](V3 *) {})) ++num_writes;
  if (num_writes != 0 && num_writes != ctx->num_ranks()) throw HazardError("HaloExch2DOp: some ranks already exchanged");
  if (num_writes == 0) return;
  if (forward_by_consumer_) return;  // the consuming convolution reads the neighbours' rows itself
  for (size_t r = 0; r < ctx->num_ranks(); ++r) {
    V3 &x = xs_.at(r).val().get_mut(txn, id());
    check_padded(x, halo_pad_, "HaloExch2DOp");  // op.cc:2981-2982
    const TileDims d = dims_of(x);
    ctx->spatial_comm(r)->group_start();
    ctx->spatial_comm(r)->halo_exchange(x.base_as_view().dptr(), (uint32_t)halo_pad_, d.W, d.H, d.C, d.N,
                                        SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
  }
  GPUConn conn = ctx->device_context(0)->conn();
  adh_check(Spatial2DComm::group_end_all(ctx->spatial_comm(0), conn), "HaloExch2DOp::_forward");
}
template <>
void HaloExch2DOp<V3>::_backward(TxnId txn) {
  if (!_requires_grad()) return;  // nothing below needs this gradient, and nobody produced ours
  MultiGPUContext *ctx = mgpu_ctx_of(ctx_);
  size_t num_writes = 0;
  for (size_t r = 0; r < ctx->num_ranks(); ++r) {
    GPUContext *dc = ctx->device_context(r).get();
    const size_t batch = xs_.at(r).val().get(txn, id()).batch_size();
    if (xs_.at(r).grad().accumulate(txn, id(), dc, [dc, batch](V3 *g) {
          GPUConn conn = dc->conn();
          g->set_batch_size(batch);
          g->base_as_view().set_constant(0.0f, conn);
        }))
      ++num_writes;
  }
  if (num_writes != 0 && num_writes != ctx->num_ranks()) throw HazardError("HaloExch2DOp: some ranks already reduced");
  if (num_writes == 0) return;
  if (forward_by_consumer_) return;  // the consuming convolution's input gradient arrives reduced
  for (size_t r = 0; r < ctx->num_ranks(); ++r) {
    V3 &g = xs_.at(r).grad().get_mut(txn, id());
    check_padded(g, halo_pad_, "HaloExch2DOp");
    const TileDims d = dims_of(g);
    ctx->spatial_comm(r)->group_start();
    ctx->spatial_comm(r)->halo_reduce(g.base_as_view().dptr(), (uint32_t)halo_pad_, d.W, d.H, d.C, d.N,
                                      SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
  }
  GPUConn conn = ctx->device_context(0)->conn();
  adh_check(Spatial2DComm::group_end_all(ctx->spatial_comm(0), conn), "HaloExch2DOp::_backward");
}

// ---- SlabConv2DOp (op.cc:1547-1727) ----
namespace {
GPUContext *rank_ctx(const shared_ptr<Context> &ctx, size_t r) {
  if (MultiGPUContext *m = dynamic_cast<MultiGPUContext *>(ctx.get())) return m->device_context(r).get();
  return gpu_ctx_of(ctx);
}
void check_filter(A4 &w, const Conv2DShape &cs, size_t cin) {
  if (w.dim() != Shape4D(cs.kernel[0], cs.kernel[1], cin, cs.filters) || !w.is_packed())
    throw std::invalid_argument("SlabConv2DOp: filter must be a packed Shape4D(kw,kh,Cin,Cout)");
}
void check_conv_input(V3 &x, const Conv2DShape &cs) {
  if (cs.halo_padded_input) {
    if (cs.pad[0] != cs.pad[1]) throw std::invalid_argument("SlabConv2DOp: halo width must be one number");
    check_padded(x, cs.pad[0], "SlabConv2DOp");
  } else {
    check_packed(x, "SlabConv2DOp");
  }
}
// scratch of the rank's context, grown to what the general conv entry points ask for
// The 3x3 stride-1 kernels tile an image plane per workgroup; a tile of at most 64 pixels (the late layers of
// a net split over several ranks) leaves them mostly idle, and the general kernel, which puts several images
// into one workgroup, is 1.2 to 1.9 times faster there.
// The 3x3 entry points also have limits the general ones do not (images x tiles in one grid dimension,
// one image inside a 2 GiB buffer range): shapes past them go to the general kernel instead of failing.
inline bool fits_3x3_kernels(const TileDims &d, uint32_t n, size_t filters) {
  const uint64_t cmax = d.C > filters ? d.C : filters;
  return (uint64_t)d.N * n <= 65535u && cmax * (d.H + 2ull) * (d.W + 2ull) * 4u < (1ull << 31);
}
template <typename Op>
bool use_3x3_kernels(const Op &op, const TileDims &d, uint32_t n, size_t filters) {
  return op.is_3x3_unit() && (uint64_t)d.H * d.W > 64u && fits_3x3_kernels(d, n, filters);
}
// The 3x3 backward-filter kernel streams an image's rows through a ring and pays the ring's fill once per image
// plane; its workgroups walk several planes, so with many planes (images x tiles) it is the faster one down to
// tiles of 64 pixels (4x16 tiles, 128 planes, 512 channels: 0.48 ms against 0.57; 2x8: 0.21 against 0.17).  With
// few planes the general kernel's units of 64 pixels win on tiles of at most 256 pixels.
template <typename Op>
bool use_3x3_filter_kernel(const Op &op, const TileDims &d, uint32_t n, size_t filters) {
  const uint64_t pixels = (uint64_t)d.H * d.W;
  return op.is_3x3_unit() && (pixels > 256u || (pixels >= 64u && (uint64_t)d.N * n >= 64u)) && fits_3x3_kernels(d, n, filters);
}

// With unexchanged rows the forward kernel and the filter-gradient kernel must both be the 3x3 ones, which can
// read a halo row from the neighbouring tile; any other shape exchanges first and runs as usual.
template <typename Op>
bool reads_neighbour_rows(const Op &op, const Conv2DShape &cs, const TileDims &d, uint32_t n) {
  return cs.unexchanged_rows && use_3x3_kernels(op, d, n, cs.filters) && use_3x3_filter_kernel(op, d, n, cs.filters);
}

// Tiles without halo: the 3x3 kernels where they are the faster ones (as over padded tiles), else the general ones
template <typename Op>
bool unpadded_3x3_kernels(const Op &op, const TileDims &d, uint32_t n, size_t filters) {
  return op.is_3x3_unit_unpadded() && (uint64_t)d.H * d.W > 64u && fits_3x3_kernels(d, n, filters);
}
template <typename Op>
bool unpadded_3x3_filter_kernel(const Op &op, const TileDims &d, uint32_t n, size_t filters) {
  const uint64_t pixels = (uint64_t)d.H * d.W;
  return op.is_3x3_unit_unpadded() && (pixels > 256u || (pixels >= 64u && (uint64_t)d.N * n >= 64u)) &&
         fits_3x3_kernels(d, n, filters);
}
#define ADH_UNPADDED_GEOMETRY(d, cs)                                                                                \
  (d).H, (d).W, (uint32_t)(cs).kernel[1], (uint32_t)(cs).kernel[0], (uint32_t)(cs).stride[1], (uint32_t)(cs).stride[0], \
      (uint32_t)(cs).dilate[1], (uint32_t)(cs).dilate[0], (uint32_t)(cs).pad[1], (uint32_t)(cs).pad[0]
void *unpadded_conv_scratch(GPUContext *dc, int which, uint32_t n, const TileDims &d, const Conv2DShape &cs, size_t *bytes) {
  *bytes = adh_conv2d_unpadded_workspace_bytes(which, ADH_F32, n, d.N, d.C, (uint32_t)cs.filters, ADH_UNPADDED_GEOMETRY(d, cs));
  dc->reserve_scratch(*bytes);
  auto scratch = dc->get_scratch();
  *bytes = scratch->size();
  return scratch->dptr();
}

void *conv_scratch(GPUContext *dc, int which, uint32_t n, const TileDims &d, const Conv2DShape &cs, size_t *bytes) {
  *bytes = adh_conv2d_workspace_bytes(which, ADH_F32, n, d.N, d.C, (uint32_t)cs.filters, d.H + 2 * (uint32_t)cs.pad[1],
                                      d.W + 2 * (uint32_t)cs.pad[0], (uint32_t)cs.kernel[1], (uint32_t)cs.kernel[0],
                                      (uint32_t)cs.stride[1], (uint32_t)cs.stride[0], (uint32_t)cs.dilate[1],
                                      (uint32_t)cs.dilate[0]);
  dc->reserve_scratch(*bytes);
  auto scratch = dc->get_scratch();
  *bytes = scratch->size();
  return scratch->dptr();
}
#define ADH_CONV_GEOMETRY(d, cs)                                                                                    \
  (d).H + 2 * (uint32_t)(cs).pad[1], (d).W + 2 * (uint32_t)(cs).pad[0], (uint32_t)(cs).kernel[1],                      \
      (uint32_t)(cs).kernel[0], (uint32_t)(cs).stride[1], (uint32_t)(cs).stride[0], (uint32_t)(cs).dilate[1],          \
      (uint32_t)(cs).dilate[0]
}  // namespace

template <>
void SlabConv2DOp<V3, A4>::_forward(TxnId txn) {
  const size_t K = xs_.size();
  vector<size_t> todo;
  for (size_t r = 0; r < K; ++r)
    if (ys_[r].val().overwrite(txn, id(), rank_ctx(ctx_, r))) todo.push_back(r);
  // group the ranks by filter buffer: one launch per distinct filter (one in all when the filters
  // are promised equal)
  const bool replicated = shape_.replicated_filters;
  bool exchanged = false;
  while (!todo.empty()) {
    const float *w0 = kernels_[replicated ? 0 : todo[0]].val().get(txn, id()).dptr();
    const void *xt[ADH_MAX_TILES];
    void *yt[ADH_MAX_TILES];
    const void *rt[ADH_MAX_TILES];
    const float *bt[ADH_MAX_TILES];
    uint32_t n = 0;
    TileDims d{}, yd{};
    vector<size_t> rest;
    for (size_t r : todo) {
      A4 &w = kernels_[r].val().get(txn, id());
      if (!replicated && w.dptr() != w0) {
        rest.push_back(r);
        continue;
      }
      V3 &x = xs_[r].val().get(txn, id());
      V3 &y = ys_[r].val().get_excl(txn, id());
      d = dims_of(x);
      y.set_batch_size(d.N);
      check_conv_input(x, shape_);
      check_filter(w, shape_, d.C);
      xt[n] = x.base_as_view().dptr();
      yt[n] = y.as_view().dptr();
      yd = dims_of(y);
      if (!res_.empty()) {
        V3 &res = res_[r].val().get(txn, id());
        check_packed(res, "SlabConv2DOp (residual)");
        if (dims_of(res).N != d.N) throw HazardError("SlabConv2DOp: the residual's batch differs from the input's");
        rt[n] = res.as_view().dptr();
      }
      if (!biases_.empty()) bt[n] = biases_[replicated ? 0 : r].val().get(txn, id()).dptr();
      ++n;
    }
    GPUContext *dc = rank_ctx(ctx_, todo[0]);
    GPUConn conn = dc->conn();
    // y += bias once the convolution of this group is enqueued (cudnnAddTensor, op.cc:1602-1610)
    auto add_bias = [&]() {
      if (biases_.empty()) return;
      adh_check(adh_conv_bias_add_tiles(ADH_F32, n, yd.N, yd.C, yd.H, yd.W, bt, yt, conn.stream()), "SlabConv2DOp::_forward (bias)");
    };
    if (shape_.unpadded_tiles) {
      if (n != K) throw HazardError("SlabConv2DOp: tiles without halo need every rank in one pass");
      if (unpadded_3x3_kernels(*this, d, n, shape_.filters)) {
        if (!res_.empty())
          adh_check(adh_conv3x3_unpadded_fwd_residual_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, d.H, d.W, xt, w0, rt,
                                                            yt, conn.stream()),
                    "SlabConv2DOp::_forward (tiles without halo, residual)");
        else
          adh_check(adh_conv3x3_unpadded_fwd_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, d.H, d.W, xt, w0, yt, 0.0f,
                                                   nullptr, 0, conn.stream()),
                    "SlabConv2DOp::_forward (tiles without halo)");
      } else {
        size_t ws_bytes;
        void *ws = unpadded_conv_scratch(dc, ADH_CONV_FWD, n, d, shape_, &ws_bytes);
        adh_check(adh_conv2d_unpadded_fwd_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, ADH_UNPADDED_GEOMETRY(d, shape_),
                                                xt, w0, yt, 0.0f, ws, ws_bytes, conn.stream()),
                  "SlabConv2DOp::_forward (tiles without halo, general)");
        if (!res_.empty()) {
          for (uint32_t t = 0; t < n; ++t)
            adh_check(adh_add_f32((uint64_t)yd.W * yd.H * yd.C * yd.N, (const float *)rt[t], (float *)yt[t], conn.stream()),
                      "SlabConv2DOp::_forward (residual)");
        }
      }
      add_bias();
      todo.swap(rest);
      continue;
    }
    const bool in_kernel_rows = n == K && reads_neighbour_rows(*this, shape_, d, n);
    if (shape_.unexchanged_rows && !in_kernel_rows && !exchanged) {
      // no kernel for this shape reads across tiles (or this launch does not hold every tile): exchange over
      // all ranks once, then the ordinary path
      void *all[ADH_MAX_TILES];
      for (size_t r = 0; r < K; ++r) all[r] = xs_[r].val().get(txn, id()).base_as_view().dptr();
      adh_check(adh_halo_exchange_nchw(ADH_F32, 1, (uint32_t)K, 1, d.W, d.H, d.C, d.N, all, conn.stream()),
                "SlabConv2DOp::_forward (exchange)");
      exchanged = true;
    }
    if (in_kernel_rows) {
      adh_check(adh_conv3x3_slab_fwd_tiles_unexchanged(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, d.H, d.W, xt, w0, yt,
                                                       0.0f, nullptr, 0, conn.stream()),
                "SlabConv2DOp::_forward (unexchanged)");
    } else if (use_3x3_kernels(*this, d, n, shape_.filters)) {
      adh_check(adh_conv3x3_slab_fwd_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, d.H, d.W, xt, w0, yt, 0.0f,
                                           nullptr, 0, conn.stream()),
                "SlabConv2DOp::_forward");
    } else {
      size_t ws_bytes;
      void *ws = conv_scratch(dc, ADH_CONV_FWD, n, d, shape_, &ws_bytes);
      if (!biases_.empty()) {
        // the bias in the convolution's stores where its kernel can (the stem), else added after it by the library
        adh_check(adh_conv2d_slab_fwd_bias_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, ADH_CONV_GEOMETRY(d, shape_),
                                                 xt, w0, bt, yt, 0.0f, ws, ws_bytes, conn.stream()),
                  "SlabConv2DOp::_forward (general, bias)");
        todo.swap(rest);
        continue;
      }
      adh_check(adh_conv2d_slab_fwd_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, ADH_CONV_GEOMETRY(d, shape_),
                                          xt, w0, yt, 0.0f, ws, ws_bytes, conn.stream()),
                "SlabConv2DOp::_forward (general)");
    }
    add_bias();
    todo.swap(rest);
  }
}

// db += sum of dy over images and pixels (cudnnConvolutionBackwardBias, op.cc:1632-1648; zeroed on first touch and
// accumulated with beta = 1 there, overwritten by the first toucher here).  Like the filter gradient: ranks that
// share a gradient buffer are summed in one launch; with replicated parameters rank 0's variable receives every
// tile's share and the other ranks' stay zero.
template <>
void SlabConv2DOp<V3, A4>::backward_bias(TxnId txn) {
  const size_t K = xs_.size();
  const bool replicated = shape_.replicated_filters;
  vector<size_t> todo;
  bool fresh[ADH_MAX_TILES] = {};
  for (size_t r = 0; r < K; ++r) {
    GPUContext *dc = rank_ctx(ctx_, r);
    bool *fresh_r = &fresh[r];
    const bool clear = replicated && r > 0 && !biases_[r].grad().known_zero();
    if (biases_[r].grad().accumulate(txn, id(), dc, [dc, fresh_r, clear](Bias *g) {
          *fresh_r = true;
          if (clear) {
            GPUConn conn = dc->conn();
            g->set_constant(0.0f, conn);
          }
        })) {
      todo.push_back(r);
      if (replicated && r > 0 && fresh[r]) biases_[r].grad().declare_zero(txn, id());
    }
  }
  for (size_t r = 0; r < K; ++r) {  // ranks whose variable was counted through a shared VarData still contribute
    bool listed = false;
    for (size_t q : todo) listed = listed || q == r;
    if (!listed)
      for (size_t q : todo)
        if (biases_[q].grad().var() == biases_[r].grad().var()) {
          todo.push_back(r);
          break;
        }
  }
  if (replicated && !todo.empty()) {
    todo.clear();
    for (size_t r = 0; r < K; ++r) todo.push_back(r);
  }
  while (!todo.empty()) {
    float *db = biases_[replicated ? 0 : todo[0]].grad().get_mut(txn, id()).dptr();
    const float beta = fresh[replicated ? 0 : todo[0]] ? 0.0f : 1.0f;
    const void *dyt[ADH_MAX_TILES];
    uint32_t n = 0;
    TileDims yd{};
    vector<size_t> rest;
    for (size_t r : todo) {
      if (!replicated && biases_[r].grad().get(txn, id()).dptr() != db) {
        rest.push_back(r);
        continue;
      }
      V3 &dy = ys_[r].grad().get(txn, id());
      yd = dims_of(dy);
      dyt[n++] = dy.as_view().dptr();
    }
    GPUContext *dc = rank_ctx(ctx_, todo[0]);
    GPUConn conn = dc->conn();
    dc->reserve_scratch(adh_conv_bwd_bias_workspace_bytes(n, yd.N, yd.C));
    auto scratch = dc->get_scratch();
    adh_check(adh_conv_bwd_bias_tiles(ADH_F32, n, yd.N, yd.C, yd.H, yd.W, dyt, db, beta, scratch->dptr(), scratch->size(),
                                      conn.stream()),
              "SlabConv2DOp::_backward (bias)");
    todo.swap(rest);
  }
}

template <>
void SlabConv2DOp<V3, A4>::_backward(TxnId txn) {
  const size_t K = xs_.size();
  if (!biases_.empty()) backward_bias(txn);
  // filter gradient: dw += sum over the tiles that share the filter (zeroed on first touch,
  // op.cc:1651-1654; beta = 1, op.cc:1660-1671)
  // (the first toucher of a filter gradient overwrites it, beta = 0, instead of clearing it and adding; with
  // replicated filters rank 0's variable receives every tile's share and the other ranks' are cleared)
  vector<size_t> todo;
  bool wfresh[ADH_MAX_TILES] = {};
  const bool replicated_w = shape_.replicated_filters;
  for (size_t r = 0; r < K; ++r) {
    GPUContext *dc = rank_ctx(ctx_, r);
    bool *fresh_r = &wfresh[r];
    // (a gradient that is still all zeros from the last time - nobody writes the other ranks' - is not cleared again)
    const bool clear = replicated_w && r > 0 && !kernels_[r].grad().known_zero();
    if (kernels_[r].grad().accumulate(txn, id(), dc, [dc, fresh_r, clear](A4 *g) {
          *fresh_r = true;
          if (clear) {
            GPUConn conn = dc->conn();
            g->set_constant(0.0f, conn);
          }
        })) {
      todo.push_back(r);
      if (replicated_w && r > 0 && wfresh[r]) kernels_[r].grad().declare_zero(txn, id());
    }
  }
  // ranks whose kernel variable was already counted through a shared VarData still contribute
  for (size_t r = 0; r < K; ++r) {
    bool listed = false;
    for (size_t q : todo) listed = listed || q == r;
    if (!listed) {
      for (size_t q : todo)
        if (kernels_[q].grad().var() == kernels_[r].grad().var()) {
          todo.push_back(r);
          break;
        }
    }
  }
  const bool replicated = shape_.replicated_filters;
  if (replicated && !todo.empty()) {
    // every rank's gradient was cleared above; all tiles now add into rank 0's
    todo.clear();
    for (size_t r = 0; r < K; ++r) todo.push_back(r);
  }
  while (!todo.empty()) {
    float *dw = kernels_[replicated ? 0 : todo[0]].grad().get_mut(txn, id()).dptr();
    const float wbeta = wfresh[replicated ? 0 : todo[0]] ? 0.0f : 1.0f;
    const void *xt[ADH_MAX_TILES];
    const void *dyt[ADH_MAX_TILES];
    uint32_t n = 0;
    TileDims d{};
    vector<size_t> rest;
    for (size_t r : todo) {
      if (!replicated && kernels_[r].grad().get(txn, id()).dptr() != dw) {
        rest.push_back(r);
        continue;
      }
      V3 &x = xs_[r].val().get(txn, id());
      V3 &dy = ys_[r].grad().get(txn, id());
      d = dims_of(x);
      xt[n] = x.base_as_view().dptr();
      dyt[n] = dy.as_view().dptr();
      ++n;
    }
    GPUContext *dc = rank_ctx(ctx_, todo[0]);
    GPUConn conn = dc->conn();
    if (shape_.unpadded_tiles) {
      if (n != K) throw HazardError("SlabConv2DOp: tiles without halo need every rank in one pass");
      if (unpadded_3x3_filter_kernel(*this, d, n, shape_.filters)) {
        const size_t ws = adh_conv3x3_workspace_bytes(ADH_CONV_BWD_FILTER, ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters,
                                                      d.H, d.W);
        dc->reserve_scratch(ws);
        auto scratch = dc->get_scratch();
        adh_check(adh_conv3x3_unpadded_bwd_filter_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, d.H, d.W, xt, dyt, dw,
                                                        wbeta, scratch->dptr(), scratch->size(), conn.stream()),
                  "SlabConv2DOp::_backward (filter, tiles without halo)");
      } else {
        size_t ws_bytes;
        void *ws = unpadded_conv_scratch(dc, ADH_CONV_BWD_FILTER, n, d, shape_, &ws_bytes);
        adh_check(adh_conv2d_unpadded_bwd_filter_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters,
                                                       ADH_UNPADDED_GEOMETRY(d, shape_), xt, dyt, dw, wbeta, ws, ws_bytes,
                                                       conn.stream()),
                  "SlabConv2DOp::_backward (filter, tiles without halo, general)");
      }
    } else if (use_3x3_filter_kernel(*this, d, n, shape_.filters)) {
      const size_t ws = adh_conv3x3_workspace_bytes(ADH_CONV_BWD_FILTER, ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters,
                                                    d.H, d.W);
      dc->reserve_scratch(ws);
      auto scratch = dc->get_scratch();
      // rows the forward pass read from the neighbours were never copied: read them there again
      auto entry = n == K && reads_neighbour_rows(*this, shape_, d, n) ? adh_conv3x3_slab_bwd_filter_tiles_unexchanged
                                                                       : adh_conv3x3_slab_bwd_filter_tiles;
      adh_check(entry(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, d.H, d.W, xt, dyt, dw, wbeta, scratch->dptr(),
                      scratch->size(), conn.stream()),
                "SlabConv2DOp::_backward (filter)");
    } else {
      size_t ws_bytes;
      void *ws = conv_scratch(dc, ADH_CONV_BWD_FILTER, n, d, shape_, &ws_bytes);
      adh_check(adh_conv2d_slab_bwd_filter_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters,
                                                 ADH_CONV_GEOMETRY(d, shape_), xt, dyt, dw, wbeta, ws, ws_bytes,
                                                 conn.stream()),
                "SlabConv2DOp::_backward (filter, general)");
    }
    todo.swap(rest);
  }
  // Input gradient over the WHOLE padded slab.  The reference zeroes it on first touch and always
  // accumulates (beta = 1, op.cc:1687-1712); the kernel writes every element, so the first toucher of
  // a transaction overwrites (beta = 0) instead: same values, one pass over the buffer instead of three.
  todo.clear();
  bool fresh[ADH_MAX_TILES] = {};
  bool reduce_after = false;  // unexchanged rows, but a kernel that cannot read across tiles: reduce once at the end
  void *all_dx[ADH_MAX_TILES] = {};
  size_t written = 0;
  TileDims dx_dims{};
  for (size_t r = 0; r < K; ++r) {
    if (!x_vars_[r]->_requires_grad()) continue;  // e.g. the first layer: nobody wants the image's gradient
    GPUContext *dc = rank_ctx(ctx_, r);
    const size_t batch = xs_[r].val().get(txn, id()).batch_size();
    bool *first = &fresh[r];
    if (xs_[r].grad().accumulate(txn, id(), dc, [batch, first](V3 *g) {
          g->set_batch_size(batch);
          *first = true;
        }))
      todo.push_back(r);
  }
  while (!todo.empty()) {
    const float *w0 = kernels_[replicated ? 0 : todo[0]].val().get(txn, id()).dptr();
    const bool first = fresh[todo[0]];
    const void *dyt[ADH_MAX_TILES];
    void *dxt[ADH_MAX_TILES];
    uint32_t n = 0;
    TileDims d{};
    vector<size_t> rest;
    for (size_t r : todo) {
      if ((!replicated && kernels_[r].val().get(txn, id()).dptr() != w0) || fresh[r] != first) {
        rest.push_back(r);
        continue;
      }
      V3 &dx = xs_[r].grad().get_mut(txn, id());
      V3 &dy = ys_[r].grad().get(txn, id());
      check_conv_input(dx, shape_);
      d = dims_of(dx);
      dyt[n] = dy.as_view().dptr();
      dxt[n] = dx.base_as_view().dptr();
      all_dx[r] = dxt[n];
      dx_dims = d;
      ++written;
      ++n;
    }
    GPUContext *dc = rank_ctx(ctx_, todo[0]);
    GPUConn conn = dc->conn();
    const float beta = first ? 0.0f : 1.0f;
    if (shape_.unpadded_tiles) {
      if (n != K) throw HazardError("SlabConv2DOp: tiles without halo need every rank in one pass");
      if (unpadded_3x3_kernels(*this, d, n, shape_.filters)) {
        adh_check(adh_conv3x3_unpadded_bwd_data_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, d.H, d.W, w0, dyt, dxt,
                                                      beta, nullptr, 0, conn.stream()),
                  "SlabConv2DOp::_backward (data, tiles without halo)");
      } else {
        size_t ws_bytes;
        void *ws = unpadded_conv_scratch(dc, ADH_CONV_BWD_DATA, n, d, shape_, &ws_bytes);
        adh_check(adh_conv2d_unpadded_bwd_data_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters,
                                                     ADH_UNPADDED_GEOMETRY(d, shape_), w0, dyt, dxt, beta, ws, ws_bytes,
                                                     conn.stream()),
                  "SlabConv2DOp::_backward (data, tiles without halo, general)");
      }
      todo.swap(rest);
      continue;
    }
    const bool in_kernel_rows = n == K && reads_neighbour_rows(*this, shape_, d, n);
    if (shape_.unexchanged_rows && !in_kernel_rows) {
      // a halo reduce after this pass would add what the halo rows held before it a second time
      if (!first) throw HazardError("SlabConv2DOp: unexchanged rows need the input gradient to themselves");
      reduce_after = true;
    }
    if (in_kernel_rows) {
      // the neighbours' edge rows of dy are multiplied here: the interior comes out as after a halo reduce
      adh_check(adh_conv3x3_slab_bwd_data_tiles_reduced(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, d.H, d.W, w0, dyt,
                                                        dxt, beta, nullptr, 0, conn.stream()),
                "SlabConv2DOp::_backward (data, reduced)");
    } else if (use_3x3_kernels(*this, d, n, shape_.filters)) {
      adh_check(adh_conv3x3_slab_bwd_data_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters, d.H, d.W, w0, dyt, dxt,
                                                beta, nullptr, 0, conn.stream()),
                "SlabConv2DOp::_backward (data)");
    } else {
      size_t ws_bytes;
      void *ws = conv_scratch(dc, ADH_CONV_BWD_DATA, n, d, shape_, &ws_bytes);
      adh_check(adh_conv2d_slab_bwd_data_tiles(ADH_F32, n, d.N, d.C, (uint32_t)shape_.filters,
                                               ADH_CONV_GEOMETRY(d, shape_), w0, dyt, dxt, beta, ws, ws_bytes,
                                               conn.stream()),
                "SlabConv2DOp::_backward (data, general)");
    }
    todo.swap(rest);
  }
  if (reduce_after) {
    // the mirror of the forward's single exchange: one reduce over all ranks' tiles once every group of ranks
    // (one per distinct filter) has written its gradient tiles
    if (written != K) throw HazardError("SlabConv2DOp: unexchanged rows need every rank's input gradient in one pass");
    GPUConn conn = rank_ctx(ctx_, 0)->conn();
    adh_check(adh_halo_reduce_nchw(ADH_F32, 1, (uint32_t)K, 1, dx_dims.W, dx_dims.H, dx_dims.C, dx_dims.N, all_dx,
                                   conn.stream()),
              "SlabConv2DOp::_backward (reduce)");
  }
}

// ---- SlabBatchNorm2DOp (op.cc:3907-4100) ----
typedef GPUArray1D<float> B1;

template <>
void SlabBatchNorm2DOp<bool, V3, B1>::_forward(TxnId txn) {
  const size_t K = xs_.size();
  const bool fixed = *switch_var_;
  const void *xt[ADH_MAX_TILES];
  void *yt[ADH_MAX_TILES];
  const float *sc[ADH_MAX_TILES], *sh[ADH_MAX_TILES], *fm[ADH_MAX_TILES], *fv[ADH_MAX_TILES];
  float *rm[ADH_MAX_TILES], *rv[ADH_MAX_TILES], *tm[ADH_MAX_TILES], *tv[ADH_MAX_TILES];
  uint32_t n = 0;
  TileDims d{};
  for (size_t r = 0; r < K; ++r) {
    GPUContext *dc = rank_ctx(ctx_, r);
    if (!ys_[r].val().overwrite(txn, id(), dc)) continue;
    V3 &x = xs_[r].val().get(txn, id());
    V3 &y = ys_[r].val().get_excl(txn, id());
    d = dims_of(x);
    y.set_batch_size(d.N);
    check_packed(x, "SlabBatchNorm2DOp");
    xt[n] = x.as_view().dptr();
    yt[n] = out_halo_ ? y.base_as_view().dptr() : y.as_view().dptr();
    sc[n] = scale_[r].val().get(txn, id()).dptr();
    sh[n] = shift_[r].val().get(txn, id()).dptr();
    if (fixed) {
      fm[n] = fixed_mean_[r].val().get(txn, id()).dptr();
      fv[n] = fixed_variance_[r].val().get(txn, id()).dptr();
    } else {
      // the reference asserts that it is the only writer of the four statistics (op.cc:3992-3995)
      if (!batch_mean_[r].val().overwrite(txn, id(), dc) || !batch_variance_[r].val().overwrite(txn, id(), dc) ||
          !tmp_mean_[r].overwrite(txn, id(), dc) || !tmp_variance_[r].overwrite(txn, id(), dc))
        throw HazardError("SlabBatchNorm2DOp: batch statistics already written in this transaction");
      rm[n] = batch_mean_[r].val().get_excl(txn, id()).dptr();
      rv[n] = batch_variance_[r].val().get_excl(txn, id()).dptr();
      tm[n] = tmp_mean_[r].get_excl(txn, id()).dptr();
      tv[n] = tmp_variance_[r].get_excl(txn, id()).dptr();
    }
    ++n;
  }
  if (n == 0) return;
  GPUContext *dc = rank_ctx(ctx_, 0);
  const size_t ws = adh_batchnorm2d_workspace_bytes(n, d.N, d.C);
  dc->reserve_scratch(ws);
  auto scratch = dc->get_scratch();
  GPUConn conn = dc->conn();
  adh_check(adh_batchnorm2d_fwd_tiles(ADH_F32, fixed ? 0 : 1, n, d.N, d.C, d.H, d.W, 1.0e-5f, relu_ ? 1 : 0, (uint32_t)out_halo_, xt, sc, sh,
                                      fixed ? fm : nullptr, fixed ? fv : nullptr, yt, fixed ? nullptr : rm,
                                      fixed ? nullptr : rv, fixed ? nullptr : tm, fixed ? nullptr : tv, scratch->dptr(),
                                      scratch->size(), conn.stream()),
            "SlabBatchNorm2DOp::_forward");
}

template <>
void SlabBatchNorm2DOp<bool, V3, B1>::_backward(TxnId txn) {
  const size_t K = xs_.size();
  // The first toucher of an input gradient overwrites it (the reference zeroes, then adds with beta = 1,
  // op.cc:4026-4031, 4059-4060); parameter gradients are small and keep the zero-then-add form.
  bool mine[ADH_MAX_TILES] = {}, fresh[ADH_MAX_TILES] = {}, pfresh[ADH_MAX_TILES] = {};
  for (size_t r = 0; r < K; ++r) {
    GPUContext *dc = rank_ctx(ctx_, r);
    const size_t batch = xs_[r].val().get(txn, id()).batch_size();
    bool *first = &fresh[r];
    mine[r] = xs_[r].grad().accumulate(txn, id(), dc, [batch, first](V3 *g) {
      g->set_batch_size(batch);
      *first = true;
    });
    if (!mine[r]) continue;
    if (*switch_var_) throw std::logic_error("SlabBatchNorm2DOp: backward with fixed statistics is unimplemented");
    // parameter gradients likewise: overwritten when this node is the first toucher of both
    bool fresh_scale = false, fresh_shift = false;
    if (!scale_[r].grad().accumulate(txn, id(), dc, [&fresh_scale](B1 *) { fresh_scale = true; }) ||
        !shift_[r].grad().accumulate(txn, id(), dc, [&fresh_shift](B1 *) { fresh_shift = true; }))
      throw HazardError("SlabBatchNorm2DOp: parameter gradients already written by this node");
    pfresh[r] = fresh_scale && fresh_shift;
    if (fresh_scale != fresh_shift) {  // one was begun by another node: clear the other and add to both
      GPUConn conn = dc->conn();
      (fresh_scale ? scale_[r] : shift_[r]).grad().get_mut(txn, id()).set_constant(0.0f, conn);
    }
  }
  for (int pass = 0; pass < 4; ++pass) {
    const bool first = (pass & 1) == 0, pfirst = (pass & 2) == 0;
    const void *xt[ADH_MAX_TILES], *dyt[ADH_MAX_TILES];
    void *dxt[ADH_MAX_TILES];
    const float *sc[ADH_MAX_TILES], *sh[ADH_MAX_TILES], *tm[ADH_MAX_TILES], *tv[ADH_MAX_TILES];
    float *dsc[ADH_MAX_TILES], *dsh[ADH_MAX_TILES];
    uint32_t n = 0;
    TileDims d{};
    for (size_t r = 0; r < K; ++r) {
      if (!mine[r] || fresh[r] != first || pfresh[r] != pfirst) continue;
      V3 &x = xs_[r].val().get(txn, id());
      d = dims_of(x);
      xt[n] = x.as_view().dptr();
      V3 &dy = ys_[r].grad().get(txn, id());
      dyt[n] = out_halo_ ? dy.base_as_view().dptr() : dy.as_view().dptr();
      dxt[n] = xs_[r].grad().get_mut(txn, id()).as_view().dptr();
      sc[n] = scale_[r].val().get(txn, id()).dptr();
      sh[n] = shift_[r].val().get(txn, id()).dptr();
      tm[n] = tmp_mean_[r].get(txn, id()).dptr();
      tv[n] = tmp_variance_[r].get(txn, id()).dptr();
      dsc[n] = scale_[r].grad().get_mut(txn, id()).dptr();
      dsh[n] = shift_[r].grad().get_mut(txn, id()).dptr();
      ++n;
    }
    if (n == 0) continue;
    GPUContext *dc = rank_ctx(ctx_, 0);
    const size_t ws = adh_batchnorm2d_workspace_bytes(n, d.N, d.C);
    dc->reserve_scratch(ws);
    auto scratch = dc->get_scratch();
    GPUConn conn = dc->conn();
    adh_check(adh_batchnorm2d_bwd_tiles(ADH_F32, n, d.N, d.C, d.H, d.W, relu_ ? 1 : 0, (uint32_t)out_halo_, xt, dyt, sc, sh,
                                        tm, tv, dxt, dsc, dsh, first ? 0.0f : 1.0f, pfirst ? 0.0f : 1.0f, scratch->dptr(),
                                        scratch->size(), conn.stream()),
              "SlabBatchNorm2DOp::_backward");
  }
}

// ---- CudnnActivationOp, kReluAct (op.cc:3189-3324) ----
template <>
void CudnnActivationOp<V3>::_forward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &x = x_.val().get(txn, id());
  if (y_.val().overwrite(txn, id(), ctx)) {
    GPUConn conn = ctx->conn();
    V3 &y = y_.val().get_excl(txn, id());
    const TileDims d = dims_of(x);
    y.set_batch_size(d.N);
    check_packed(x, "CudnnActivationOp");
    adh_check(adh_relu_fwd(ADH_F32, (uint64_t)d.W * d.H * d.C * d.N, x.as_view().dptr(), y.as_view().dptr(), conn.stream()),
              "CudnnActivationOp::_forward");
  }
}
template <>
void CudnnActivationOp<V3>::_backward(TxnId txn) {
  if (!_requires_grad()) return;  // nothing below needs this gradient, and nobody produced ours
  GPUContext *ctx = gpu_ctx_of(ctx_);
  const size_t batch = x_.val().get(txn, id()).batch_size();
  // the first toucher of the input gradient overwrites it (the reference zeroes, then adds with beta = 1)
  bool first = false;
  if (x_.grad().accumulate(txn, id(), ctx, [batch, &first](V3 *g) {
        g->set_batch_size(batch);
        first = true;
      })) {
    GPUConn conn = ctx->conn();
    V3 &y = y_.val().get(txn, id());
    const TileDims d = dims_of(y);
    adh_check(adh_relu_bwd(ADH_F32, (uint64_t)d.W * d.H * d.C * d.N, y.as_view().dptr(),
                           y_.grad().get(txn, id()).as_view().dptr(), x_.grad().get_mut(txn, id()).as_view().dptr(),
                           first ? 0.0f : 1.0f, conn.stream()),
              "CudnnActivationOp::_backward");
  }
}

// ---- ScaleOp (op.cc:1221-1290) ----
template <>
void ScaleOp<float, V3>::_forward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &x = x_.val().get(txn, id());
  if (y_.val().overwrite(txn, id(), ctx)) {
    GPUConn conn = ctx->conn();
    V3 &y = y_.val().get_excl(txn, id());
    const TileDims d = dims_of(x);
    y.set_batch_size(d.N);
    check_packed(x, "ScaleOp");
    const uint64_t n = (uint64_t)d.W * d.H * d.C * d.N;
    // y = scale * x + 0 * y needs a finite y: clear it first
    adh_check(adh_fill_f32(n, 0.0f, y.as_view().dptr(), conn.stream()), "ScaleOp::_forward");
    adh_check(adh_scale_add_f32(n, scale_, x.as_view().dptr(), 0.0f, y.as_view().dptr(), conn.stream()), "ScaleOp::_forward");
  }
}
template <>
void ScaleOp<float, V3>::_backward(TxnId txn) {
  if (!_requires_grad()) return;  // nothing below needs this gradient, and nobody produced ours
  GPUContext *ctx = gpu_ctx_of(ctx_);
  const size_t batch = x_.val().get(txn, id()).batch_size();
  if (x_.grad().accumulate(txn, id(), ctx, [ctx, batch](V3 *g) {
        GPUConn conn = ctx->conn();
        g->set_batch_size(batch);
        g->as_view().set_constant(0.0f, conn);
      })) {
    GPUConn conn = ctx->conn();
    V3 &dy = y_.grad().get(txn, id());
    const TileDims d = dims_of(dy);
    adh_check(adh_scale_add_f32((uint64_t)d.W * d.H * d.C * d.N, scale_, dy.as_view().dptr(), 1.0f,
                                x_.grad().get_mut(txn, id()).as_view().dptr(), conn.stream()),
              "ScaleOp::_backward");
  }
}

// ---- JoinOp<V, SumJoin> (op.cc:744-867) ----
template <>
void JoinOp<V3, SumJoin>::_forward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  if (y_.val().overwrite(txn, id(), ctx)) {
    GPUConn conn = ctx->conn();
    const void *xt[ADH_MAX_TILES];
    TileDims d{};
    for (size_t j = 0; j < xs_.size(); ++j) {
      V3 &x = xs_[j].val().get(txn, id());
      check_packed(x, "JoinOp");
      d = dims_of(x);
      xt[j] = x.as_view().dptr();
    }
    V3 &y = y_.val().get_excl(txn, id());
    y.set_batch_size(d.N);
    adh_check(adh_sum_fwd(ADH_F32, (uint32_t)xs_.size(), (uint64_t)d.W * d.H * d.C * d.N, xt, y.as_view().dptr(),
                          conn.stream()),
              "JoinOp::_forward");
  }
}
template <>
void JoinOp<V3, SumJoin>::_backward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &dy = y_.grad().get(txn, id());
  const TileDims d = dims_of(dy);
  const size_t batch = d.N;
  for (size_t j = 0; j < xs_.size(); ++j) {
    if (grad_shared_[j]) continue;  // the input's gradient IS dy (one buffer): nothing to copy
    // the first toucher of an input's gradient copies dy into it, later ones add
    bool first = false;
    if (xs_[j].grad().accumulate(txn, id(), ctx, [batch, &first](V3 *g) {
          g->set_batch_size(batch);
          first = true;
        })) {
      GPUConn conn = ctx->conn();
      V3 &dx = xs_[j].grad().get_mut(txn, id());
      check_packed(dx, "JoinOp");
      const uint64_t n = (uint64_t)d.W * d.H * d.C * d.N;
      if (first)
        gpu_copy_d2d(dx.as_view().dptr(), dy.as_view().dptr(), n * sizeof(float), conn.stream());
      else
        adh_check(adh_add_f32(n, dy.as_view().dptr(), dx.as_view().dptr(), conn.stream()), "JoinOp::_backward");
    }
  }
}

// ---- SlabPool2DOp (op.cc:3405-3530 forward, 3532-3660 backward) ----
template <>
void SlabPool2DOp<V3>::_forward(TxnId txn) {
  const size_t K = xs_.size();
  const void *xt[ADH_MAX_TILES];
  void *yt[ADH_MAX_TILES];
  uint32_t n = 0;
  TileDims d{};
  for (size_t r = 0; r < K; ++r) {
    if (!ys_[r].val().overwrite(txn, id(), rank_ctx(ctx_, r))) continue;
    V3 &x = xs_[r].val().get(txn, id());
    V3 &y = ys_[r].val().get_excl(txn, id());
    d = dims_of(x);
    y.set_batch_size(d.N);
    if (shape_.halo_padded_input) {
      if (shape_.pad[0] != shape_.pad[1]) throw std::invalid_argument("SlabPool2DOp: halo width must be one number");
      check_padded(x, shape_.pad[0], "SlabPool2DOp");
    } else {
      check_packed(x, "SlabPool2DOp");
    }
    xt[n] = x.base_as_view().dptr();
    yt[n] = y.as_view().dptr();
    ++n;
  }
  if (n == 0) return;
  GPUConn conn = rank_ctx(ctx_, 0)->conn();
  if (shape_.unpadded_tiles) {
    if (n != K) throw HazardError("SlabPool2DOp: tiles without halo need every rank in one pass");
    adh_check(adh_pool2d_unpadded_fwd_tiles(ADH_F32, shape_.pooling == kMaxPool ? ADH_POOL_MAX : ADH_POOL_AVG, n, d.N, d.C, d.H,
                                            d.W, (uint32_t)shape_.window[1], (uint32_t)shape_.window[0],
                                            (uint32_t)shape_.stride[1], (uint32_t)shape_.stride[0], (uint32_t)shape_.pad[1],
                                            (uint32_t)shape_.pad[0], xt, yt, conn.stream()),
              "SlabPool2DOp::_forward (tiles without halo)");
    return;
  }
  adh_check(adh_pool2d_slab_fwd_tiles(ADH_F32, shape_.pooling == kMaxPool ? ADH_POOL_MAX : ADH_POOL_AVG, n, d.N, d.C,
                                      d.H + 2 * (uint32_t)shape_.pad[1], d.W + 2 * (uint32_t)shape_.pad[0],
                                      (uint32_t)shape_.window[1], (uint32_t)shape_.window[0], (uint32_t)shape_.stride[1],
                                      (uint32_t)shape_.stride[0], xt, yt, conn.stream()),
            "SlabPool2DOp::_forward");
}

template <>
void SlabPool2DOp<V3>::_backward(TxnId txn) {
  const size_t K = xs_.size();
  // Input gradient over the WHOLE padded tile.  The reference zeroes it on first touch and accumulates
  // (beta = 1, op.cc:3540-3550, 3610-3619); the kernel writes every element, so the first toucher of a
  // transaction overwrites instead.
  bool mine[ADH_MAX_TILES] = {}, fresh[ADH_MAX_TILES] = {};
  for (size_t r = 0; r < K; ++r) {
    GPUContext *dc = rank_ctx(ctx_, r);
    const size_t batch = xs_[r].val().get(txn, id()).batch_size();
    bool *first = &fresh[r];
    mine[r] = xs_[r].grad().accumulate(txn, id(), dc, [batch, first](V3 *g) {
      g->set_batch_size(batch);
      *first = true;
    });
  }
  for (int pass = 0; pass < 2; ++pass) {
    const bool first = pass == 0;
    const void *xt[ADH_MAX_TILES];
    const void *yt[ADH_MAX_TILES];
    const void *dyt[ADH_MAX_TILES];
    void *dxt[ADH_MAX_TILES];
    uint32_t n = 0;
    TileDims d{};
    for (size_t r = 0; r < K; ++r) {
      if (!mine[r] || fresh[r] != first) continue;
      V3 &x = xs_[r].val().get(txn, id());
      V3 &dx = xs_[r].grad().get_mut(txn, id());
      d = dims_of(x);
      if (shape_.halo_padded_input) check_padded(dx, shape_.pad[0], "SlabPool2DOp");
      else check_packed(dx, "SlabPool2DOp");
      xt[n] = x.base_as_view().dptr();
      yt[n] = ys_[r].val().get(txn, id()).as_view().dptr();
      dyt[n] = ys_[r].grad().get(txn, id()).as_view().dptr();
      dxt[n] = dx.base_as_view().dptr();
      ++n;
    }
    if (n == 0) continue;
    GPUConn conn = rank_ctx(ctx_, 0)->conn();
    if (shape_.unpadded_tiles) {
      if (n != K) throw HazardError("SlabPool2DOp: tiles without halo need every rank in one pass");
      adh_check(adh_pool2d_unpadded_bwd_tiles(ADH_F32, shape_.pooling == kMaxPool ? ADH_POOL_MAX : ADH_POOL_AVG, n, d.N, d.C,
                                              d.H, d.W, (uint32_t)shape_.window[1], (uint32_t)shape_.window[0],
                                              (uint32_t)shape_.stride[1], (uint32_t)shape_.stride[0], (uint32_t)shape_.pad[1],
                                              (uint32_t)shape_.pad[0], xt, yt, dyt, dxt, first ? 0.0f : 1.0f, conn.stream()),
                "SlabPool2DOp::_backward (tiles without halo)");
      continue;
    }
    adh_check(adh_pool2d_slab_bwd_tiles(ADH_F32, shape_.pooling == kMaxPool ? ADH_POOL_MAX : ADH_POOL_AVG, n, d.N, d.C,
                                        d.H + 2 * (uint32_t)shape_.pad[1], d.W + 2 * (uint32_t)shape_.pad[0],
                                        (uint32_t)shape_.window[1], (uint32_t)shape_.window[0], (uint32_t)shape_.stride[1],
                                        (uint32_t)shape_.stride[0], xt, yt, dyt, dxt, first ? 0.0f : 1.0f, conn.stream()),
              "SlabPool2DOp::_backward");
  }
}

// ---- SoftmaxNLLLossOp, 1-D logits (op.cc:4118-4188) ----
typedef GPUBatchArray1D<float> V1;
typedef GPUBatchArray0D<uint32_t> L0;
typedef GPUBatchArray0D<float> F0;

// ---- FlattenNCHWOp (src/zoo.cc:1861) ----
template <>
void FlattenNCHWOp<V3, V1>::_forward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V3 &x = x_.val().get(txn, id());
  if (y_.val().overwrite(txn, id(), ctx)) {
    GPUConn conn = ctx->conn();
    V1 &y = y_.val().get_excl(txn, id());
    check_packed(x, "FlattenNCHWOp");
    y.set_batch_size(x.batch_size());
    gpu_copy_d2d(y.as_view().dptr(), x.as_view().dptr(), x.dim().flat_size() * x.batch_size() * sizeof(float), conn.stream());
  }
}
template <>
void FlattenNCHWOp<V3, V1>::_backward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  const size_t batch = x_.val().get(txn, id()).batch_size();
  bool first = false;
  if (x_.grad().accumulate(txn, id(), ctx, [batch, &first](V3 *g) {
        g->set_batch_size(batch);
        first = true;
      })) {
    GPUConn conn = ctx->conn();
    V3 &dx = x_.grad().get_mut(txn, id());
    V1 &dy = y_.grad().get(txn, id());
    const size_t n = dx.dim().flat_size() * batch;
    if (first)
      gpu_copy_d2d(dx.as_view().dptr(), dy.as_view().dptr(), n * sizeof(float), conn.stream());
    else
      array_add_packed<float>((uint32_t)n, dy.as_view().dptr(), dx.as_view().dptr(), conn.stream());
  }
}

template <>
void SoftmaxNLLLossOp<V1, L0, F0>::_forward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V1 &x = x_.val().get(txn, id());
  const uint32_t C = (uint32_t)x.dim().shape[0], N = (uint32_t)x.batch_size();
  const bool wy = y_.val().overwrite(txn, id(), ctx);
  const bool wl = loss_.val().overwrite(txn, id(), ctx);
  if (wy || wl) {
    GPUConn conn = ctx->conn();
    V1 &y = y_.val().get_excl(txn, id());
    F0 &loss = loss_.val().get_excl(txn, id());
    L0 &label = label_.val().get(txn, id());
    y.set_batch_size(N);
    loss.set_batch_size(N);
    if (label.batch_size() != N) throw std::invalid_argument("SoftmaxNLLLossOp: one label per example");
    // softmax and loss in one launch (the reference: a cuDNN call, then its own kernel, op.cc:4129-4163)
    adh_check(adh_softmax_xent_fwd(C, N, x.as_view().dptr(), label.as_view().dptr(), y.as_view().dptr(),
                                   loss.as_view().dptr(), conn.stream()),
              "SoftmaxNLLLossOp::_forward");
  }
}
template <>
void SoftmaxNLLLossOp<V1, L0, F0>::_backward(TxnId txn) {
  GPUContext *ctx = gpu_ctx_of(ctx_);
  V1 &y = y_.val().get(txn, id());
  const uint32_t C = (uint32_t)y.dim().shape[0], N = (uint32_t)y.batch_size();
  const size_t batch = N;
  // the first toucher overwrites (beta = 0) where the reference clears the gradient and then adds
  // (op.cc:4171-4176): the same values in one launch
  bool first = false;
  if (x_.grad().accumulate(txn, id(), ctx, [batch, &first](V1 *g) {
        g->set_batch_size(batch);
        first = true;
      })) {
    GPUConn conn = ctx->conn();
    adh_check(adh_softmax_nll_loss_bwd_scaled(C, N, y.as_view().dptr(), label_.val().get(txn, id()).as_view().dptr(),
                                              loss_.grad().get(txn, id()).as_view().dptr(), 0.0f, first ? 0.0f : 1.0f,
                                              x_.grad().get_mut(txn, id()).as_view().dptr(), conn.stream()),
              "SoftmaxNLLLossOp::_backward");
  }
}

}  // namespace arraydiff
