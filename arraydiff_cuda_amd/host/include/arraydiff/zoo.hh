// Builders of the spatially-parallel residual nets, by the reference's names
// (include/arraydiff/zoo.hh:19-183, src/zoo.cc:133-161, 577-741, 1475-1909): parallel_conv2d,
// spatial_parallel_residual_v2_conv2d, spatial_parallel_proj_residual_v2_conv2d and
// ResNet<float>::MakeParallelResNet18.  Ranks are row-tiles of one GPU; every rank owns its copy
// of every parameter, as in the reference, and ParallelSGDOptimizer keeps the copies equal.
//
// What differs from the reference's MakeParallelResNet18, all in the replicated tail after the
// spatial part: the input arrives as NCHW floats (no transpose / scale ops); the tiles are
// gathered once (SpatialJoinedGather2DOp replaces gather + all-reduce); every rank then pools the
// gathered activation and applies its own copy of the classifier, as in the reference, and the
// logits are summed over ranks and divided by the rank count before ONE loss node (the reference
// runs the loss per rank); the classifier is the 1x1 convolution over the pooled 1x1 image that a
// bias-free linear layer is; the mean over the minibatch is the loss's sink gradient.
#ifndef ARRAYDIFF_ZOO_HH
#define ARRAYDIFF_ZOO_HH

#include "arraydiff/op.hh"

#include <memory>
#include <vector>

namespace arraydiff {

template <typename V>
class ParallelParamOp {
public:
  vector<shared_ptr<Var<V>>> ops;
  vector<VarIdSet> params;
  vector<VarIdSet> grads;
};

template <typename V>
class ParallelBatchNormParamOp {
public:
  vector<shared_ptr<Var<V>>> ops;
  vector<VarIdSet> params;
  vector<VarIdSet> grads;
  vector<VarIdSet> batch_stats;
  vector<VarIdSet> fixed_stats;
};

inline void parallel_vars_insert_all(vector<VarIdSet> &dst, const vector<VarIdSet> &src) {
  if (dst.size() != src.size()) throw std::invalid_argument("parallel_vars_insert_all: rank counts differ");
  for (size_t rank = 0; rank < dst.size(); ++rank) dst[rank].insert_all(src[rank]);
}

// One filter variable per rank, one node for all of them (src/zoo.cc:133-161).  enable_bias adds one bias
// vector per rank, initialised to zeros, listed after the rank's filter in its parameter and gradient sets
// (src/zoo.cc:111-120; the spatial nets enable it on their stem, src/zoo.cc:1548).  The node is
// told that the copies are equal (Conv2DShape::replicated_filters), and they are from the start:
// Op::init draws rank 0's values and hands every other rank a copy of them (the reference draws
// each rank's own and the optimizer's first broadcast overwrites them, optimize.hh:283-300).
// ParallelSGDOptimizer keeps them equal; whoever loads values by hand must load the same ones
// into every rank.
template <typename V, typename A = GPUArray4D<float>>
ParallelParamOp<V> parallel_conv2d(Conv2DShape shape, vector<shared_ptr<Var<V>>> inputs,
                                   typename ParamOp<A>::InitFn kernel_init, bool enable_bias, shared_ptr<Context> ctx,
                                   vector<shared_ptr<Var<V>>> residuals = {}) {
  // every rank's copy starts from rank 0's values (ParallelSGDOptimizer::reset) and receives the
  // same update: one launch serves all tiles
  shape.replicated_filters = true;
  MultiGPUContext *mgpu_ctx = mgpu_ctx_of(ctx);
  if (inputs.size() != mgpu_ctx->num_ranks()) throw std::invalid_argument("parallel_conv2d: one input per rank");
  const size_t cin = inputs.at(0)->shape().shape[2];
  typedef GPUArray1D<float> B;
  ParallelParamOp<V> out;
  vector<shared_ptr<Var<A>>> kernels;
  vector<shared_ptr<Var<B>>> biases;
  // the conv node visits rank 0's filter before the others (SlabConv2DOp::_push), so its values exist
  // when the copies are made
  auto drawn = make_shared<std::unique_ptr<A>>();
  typename ParamOp<A>::InitFn draw = [kernel_init, drawn](A *a, std::mt19937_64 *rng, shared_ptr<Context> c) {
    kernel_init(a, rng, c);
    drawn->reset(new A(*a));  // a view of the same memory
  };
  typename ParamOp<A>::InitFn copy = [drawn](A *a, std::mt19937_64 *, shared_ptr<Context> c) {
    if (!*drawn) throw std::logic_error("parallel_conv2d: rank 0's filter was not initialised before the others");
    if (!a->is_packed() || !(*drawn)->is_packed() || a->dim() != (*drawn)->dim())
      throw std::logic_error("parallel_conv2d: filter copies differ in shape");
    GPUConn conn = gpu_ctx_of(c)->conn();
    gpu_copy_d2d(a->dptr(), (*drawn)->dptr(), a->dim().flat_size() * sizeof(float), conn.stream());
  };
  for (size_t rank = 0; rank < inputs.size(); ++rank) {
    auto kernel = ParamOp<A>::Make(Shape4D(shape.kernel[0], shape.kernel[1], cin, shape.filters), rank == 0 ? draw : copy,
                                   mgpu_ctx->device_context(rank));
    kernels.push_back(kernel);
    out.params.push_back(VarIdSet::Singleton(kernel->vars().at(0)));
    out.grads.push_back(VarIdSet::Singleton(kernel->vars().at(1)));
    if (enable_bias) {
      // zeros on every rank: equal from the start, and the optimizer keeps them so
      auto bias = ParamOp<B>::Make(Shape1D(shape.filters), zeros_init_gen<B>(), mgpu_ctx->device_context(rank));
      biases.push_back(bias);
      out.params.back().insert(bias->vars().at(0));
      out.grads.back().insert(bias->vars().at(1));
    }
  }
  out.ops = CudnnConv2DOp<V, A, B>::MakeParallel(shape, inputs, kernels, ctx, residuals, biases);
  return out;
}

namespace detail {
template <typename V>
void add_batch_norm(ParallelBatchNormParamOp<V> &block, const ParallelBatchNormOutput<V, GPUArray1D<float>> &bn) {
  parallel_vars_insert_all(block.params, bn.params);
  parallel_vars_insert_all(block.grads, bn.grads);
  parallel_vars_insert_all(block.batch_stats, bn.batch_stats);
  parallel_vars_insert_all(block.fixed_stats, bn.fixed_stats);
}
template <typename V>
ParallelBatchNormParamOp<V> empty_block(size_t num_ranks) {
  ParallelBatchNormParamOp<V> b;
  b.params.resize(num_ranks);
  b.grads.resize(num_ranks);
  b.batch_stats.resize(num_ranks);
  b.fixed_stats.resize(num_ranks);
  return b;
}
// halo exchange -> 3x3 conv with the given stride, over tiles that already carry a halo of 1
template <typename V>
vector<shared_ptr<Var<V>>> exchanged_conv3x3(ParallelBatchNormParamOp<V> &block, Conv2DShape shape, size_t stride,
                                             vector<shared_ptr<Var<V>>> padded, shared_ptr<Context> ctx) {
  typedef GPUArray4D<float> A;
  Conv2DShape cs = shape;
  cs.stride = {stride, stride};
  cs.halo_padded_input = true;
  // over row tiles the convolution reads its neighbours' rows itself and the exchange copies nothing
  cs.unexchanged_rows = mgpu_ctx_of(ctx)->spatial_comm(0)->num_w_ranks == 1 && padded.size() > 1;
  auto exch = HaloExch2DOp<V>::MakeParallel(1, padded, ctx, cs.unexchanged_rows);
  const size_t cin = padded.at(0)->shape().shape[2];
  auto conv = parallel_conv2d<V, A>(cs, exch, kaiming_init_gen<A>(cin * shape.kernel[0] * shape.kernel[1], shape.filters),
                                    false, ctx);
  parallel_vars_insert_all(block.params, conv.params);
  parallel_vars_insert_all(block.grads, conv.grads);
  return conv.ops;
}
// A conv over row tiles WITHOUT halo (Conv2DShape::unpadded_tiles): no pad and no exchange node, the conv node reads
// zero padding and its neighbours' rows itself and leaves an unpadded, complete input gradient.  Row tiles only,
// and a tile height the row stride divides.
template <typename V>
bool halo_free_conv(const Conv2DShape &shape, size_t stride, const vector<shared_ptr<Var<V>>> &inputs, shared_ptr<Context> ctx) {
  const auto tile = inputs.at(0)->shape();
  const size_t span = (shape.kernel[1] - 1) * shape.dilate[1] + 1;
  return mgpu_ctx_of(ctx)->spatial_comm(0)->num_w_ranks == 1 && tile.shape[1] % stride == 0 && 2 * shape.pad[1] < span &&
         span - 2 * shape.pad[1] <= stride && shape.pad[1] <= tile.shape[1] && span - 1 - shape.pad[1] <= tile.shape[1];
}
template <typename V>
vector<shared_ptr<Var<V>>> unpadded_conv(ParallelBatchNormParamOp<V> &block, Conv2DShape shape, size_t stride,
                                         vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx,
                                         vector<shared_ptr<Var<V>>> residuals = {}) {
  typedef GPUArray4D<float> A;
  Conv2DShape cs = shape;
  cs.stride = {stride, stride};
  cs.halo_padded_input = false;
  cs.unpadded_tiles = true;
  const size_t cin = inputs.at(0)->shape().shape[2];
  auto conv = parallel_conv2d<V, A>(cs, inputs, kaiming_init_gen<A>(cin * shape.kernel[0] * shape.kernel[1], shape.filters),
                                    false, ctx, residuals);
  parallel_vars_insert_all(block.params, conv.params);
  parallel_vars_insert_all(block.grads, conv.grads);
  return conv.ops;
}
// batch norm -> rectifier -> halo pad as ONE node (the reference has three, src/zoo.cc:596-604),
// then halo exchange -> 3x3 conv; over row tiles the batch norm does not pad and the conv runs over tiles
// without halo
template <typename V>
vector<shared_ptr<Var<V>>> bn_relu_pad_conv3x3(ParallelBatchNormParamOp<V> &block, Conv2DShape shape, size_t stride,
                                               shared_ptr<bool> switch_var, vector<shared_ptr<Var<V>>> inputs,
                                               shared_ptr<Context> ctx, vector<shared_ptr<Var<V>>> residuals = {}) {
  const size_t cin = inputs.at(0)->shape().shape[2];
  if (halo_free_conv(shape, stride, inputs, ctx)) {
    auto bnorm = CudnnBatchNorm2DOp<bool, V, GPUArray1D<float>>::MakeParallel(cin, switch_var, inputs, ctx, true, 0);
    add_batch_norm(block, bnorm);
    return unpadded_conv(block, shape, stride, bnorm.ops, ctx, residuals);
  }
  auto bnorm = CudnnBatchNorm2DOp<bool, V, GPUArray1D<float>>::MakeParallel(cin, switch_var, inputs, ctx, true, 1);
  add_batch_norm(block, bnorm);
  auto conv = exchanged_conv3x3(block, shape, stride, bnorm.ops, ctx);
  if (residuals.empty()) return conv;
  // the conv over exchanged tiles takes no residual: a sum node closes the block.  The conv feeds the sum only, and
  // the residual's other consumers lie upstream of the conv: both gradients are the sum's output gradient, one
  // buffer that the upstream nodes add to in place
  vector<vector<shared_ptr<Var<V>>>> join_inputs{residuals, conv};
  return parallel_sum<V>(join_inputs, ctx, 1, 0);
}
}  // namespace detail

// x + conv(relu(bn(conv(relu(bn(x)))))) on every rank's tile (src/zoo.cc:577-652)
template <typename V>
ParallelBatchNormParamOp<V> spatial_parallel_residual_v2_conv2d(Conv2DShape shape, shared_ptr<bool> switch_var,
                                                                vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx) {
  const size_t cin = inputs.at(0)->shape().shape[2];
  if (shape.filters != cin) throw std::invalid_argument("spatial_parallel_residual_v2_conv2d: the block keeps the channel count");
  auto block = detail::empty_block<V>(inputs.size());
  auto conv1 = detail::bn_relu_pad_conv3x3(block, shape, 1, switch_var, inputs, ctx);
  // the second conv adds the block input to its result.  The block input's other consumer (the first batch norm)
  // lies upstream of that conv: the input's gradient is the output's gradient, one buffer that the batch norm's
  // backward pass adds to in place
  block.ops = detail::bn_relu_pad_conv3x3(block, shape, 1, switch_var, conv1, ctx, inputs);
  return block;
}

// proj(a) + conv(relu(bn(conv_s(a)))) with a = relu(bn(x)), proj a strided 1x1 conv and conv_s the
// strided 3x3 (src/zoo.cc:654-741): the block that changes extents and channel count
template <typename V>
ParallelBatchNormParamOp<V> spatial_parallel_proj_residual_v2_conv2d(Conv2DShape shape, size_t stride,
                                                                     shared_ptr<bool> switch_var,
                                                                     vector<shared_ptr<Var<V>>> inputs,
                                                                     shared_ptr<Context> ctx) {
  typedef GPUArray1D<float> B;
  typedef GPUArray4D<float> A;
  const size_t cin = inputs.at(0)->shape().shape[2];
  auto block = detail::empty_block<V>(inputs.size());
  // a = relu(bn(x)) feeds the unpadded projection and the padded 3x3: batch norm and rectifier fused, pad separate
  auto bnorm0 = CudnnBatchNorm2DOp<bool, V, B>::MakeParallel(cin, switch_var, inputs, ctx, true, 0);
  detail::add_batch_norm(block, bnorm0);
  auto relu0 = bnorm0.ops;
  Conv2DShape proj_shape = shape;
  proj_shape.kernel = {1, 1};
  proj_shape.stride = {stride, stride};
  proj_shape.pad = {0, 0};
  proj_shape.halo_padded_input = false;
  auto proj = parallel_conv2d<V, A>(proj_shape, relu0, kaiming_init_gen<A>(cin, shape.filters), false, ctx);
  parallel_vars_insert_all(block.params, proj.params);
  parallel_vars_insert_all(block.grads, proj.grads);
  auto conv1 = detail::halo_free_conv(shape, stride, relu0, ctx)
                   ? detail::unpadded_conv(block, shape, stride, relu0, ctx)
                   : detail::exchanged_conv3x3(block, shape, stride, HaloPad2DOp<V>::MakeParallel(1, relu0, ctx), ctx);
  // the second conv adds the projection to its result; the projection feeds nothing else, so its gradient is the
  // output's gradient, one buffer
  block.ops = detail::bn_relu_pad_conv3x3(block, shape, 1, switch_var, conv1, ctx, proj.ops);
  return block;
}

// include/arraydiff/zoo.hh:166-173
class ConvNetConfig {
public:
  size_t input_w;
  size_t input_h;
  size_t batch_size;
  size_t minibatch_size;
};

// include/arraydiff/zoo.hh:128-146, plus the two sources (the reference feeds them through
// load_val on `inputs` / `labels`; here SrcOp::load does it)
template <typename V, typename L>
class ParallelCategoricalNLLBatchNormLoss {
public:
  shared_ptr<bool> batch_norm_use_fixed;
  shared_ptr<Var<V>> op;                                   // logits
  shared_ptr<SoftmaxNLLLossOp<V, GPUBatchArray0D<uint32_t>, L>> loss;  // per-example losses
  shared_ptr<Op> sum_loss;                                 // what the optimizer differentiates
  shared_ptr<SrcOp<GPUBatchArray3D<float>>> input;         // (W, H, 3) x batch, NCHW floats
  shared_ptr<SrcOp<GPUBatchArray0D<uint32_t>>> label;
  vector<VarIdSet> dev_params;
  vector<VarIdSet> dev_grads;
  vector<VarIdSet> dev_batch_stats;
  vector<VarIdSet> dev_fixed_stats;
};

template <typename T>
class ResNet {
public:
  // The reference's spatially-parallel 18-layer variant (src/zoo.cc:1475-1909): a 7x7 stem at
  // stride 1 over halo 3, 3x3 max pooling at stride 2 over halo 1, then
  // res2 x2 (64), res3 proj + plain (128), res4 proj + plain (256), res5 proj (512), res6 proj (512),
  // batch norm, rectifier, global average pooling, a 1000-way classifier, softmax loss.
  // Input extents must leave every stage's tile height even down to the last stride.
  static ParallelCategoricalNLLBatchNormLoss<GPUBatchArray1D<T>, GPUBatchArray0D<T>> MakeParallelResNet18(
      const ConvNetConfig &cfg, shared_ptr<Context> parallel_ctx, size_t num_classes = 1000);
};

}  // namespace arraydiff

#endif
