// ResNet<float>::MakeParallelResNet18 (src/zoo.cc:1475-1909 in the reference).
#include "arraydiff/zoo.hh"

namespace arraydiff {

typedef GPUBatchArray3D<float> V3;
typedef GPUBatchArray1D<float> V1;
typedef GPUBatchArray0D<float> F0;
typedef GPUBatchArray0D<uint32_t> L0;
typedef GPUArray4D<float> A4;
typedef GPUArray1D<float> B1;

template <>
ParallelCategoricalNLLBatchNormLoss<V1, F0> ResNet<float>::MakeParallelResNet18(const ConvNetConfig &cfg,
                                                                                 shared_ptr<Context> parallel_ctx,
                                                                                 size_t num_classes) {
  MultiGPUContext *mgpu_ctx = mgpu_ctx_of(parallel_ctx);
  const size_t num_ranks = mgpu_ctx->num_ranks();
  shared_ptr<Context> root = mgpu_ctx->device_context(0);
  // five halvings of the height; the last stage must still leave every rank two rows, since a halo
  // reduction over halo 1 needs two rows per tile
  if (cfg.input_h % (num_ranks * 64) != 0 || cfg.input_w % 32 != 0)
    throw std::invalid_argument("MakeParallelResNet18: input height must be a multiple of 64 x ranks, width of 32");

  ParallelCategoricalNLLBatchNormLoss<V1, F0> net;
  net.dev_params.resize(num_ranks);
  net.dev_grads.resize(num_ranks);
  net.dev_batch_stats.resize(num_ranks);
  net.dev_fixed_stats.resize(num_ranks);
  net.batch_norm_use_fixed = std::make_shared<bool>(false);
  auto add = [&net](const ParallelBatchNormParamOp<V3> &block) {
    parallel_vars_insert_all(net.dev_params, block.params);
    parallel_vars_insert_all(net.dev_grads, block.grads);
    parallel_vars_insert_all(net.dev_batch_stats, block.batch_stats);
    parallel_vars_insert_all(net.dev_fixed_stats, block.fixed_stats);
  };

  net.input = SrcOp<V3>::Make(Shape3D(cfg.input_w, cfg.input_h, 3), cfg.batch_size, root);
  net.label = SrcOp<L0>::Make(Shape0D(), cfg.batch_size, root);
  net.input->set_requires_grad(false);  // the image's gradient is of no use to a trainer

  vector<shared_ptr<Var<V3>>> par_ys(num_ranks, net.input);
  par_ys = SpatialScatter2DOp<V3>::MakeParallel(par_ys, parallel_ctx);

  // conv1: 7x7 over halo 3 (stride 1 in the reference's parallel variant, src/zoo.cc:1525-1538).  The image has three
  // channels, so padding and exchanging it costs nothing, and no input gradient is wanted: the padded form stays
  // (over tiles without halo the filter gradient is a tenth slower, 0.66 ms against 0.60).
  par_ys = HaloExch2DOp<V3>::MakeParallel(3, HaloPad2DOp<V3>::MakeParallel(3, par_ys, parallel_ctx), parallel_ctx);
  Conv2DShape conv1_shape;
  conv1_shape.filters = 64; conv1_shape.axes = {0, 1}; conv1_shape.kernel = {7, 7}; conv1_shape.dilate = {1, 1};
  conv1_shape.stride = {1, 1}; conv1_shape.pad = {3, 3}; conv1_shape.halo_padded_input = true; conv1_shape.enable_hmma = false;
  auto conv1 = parallel_conv2d<V3, A4>(conv1_shape, par_ys, xavier_init_gen<A4>(3 * 7 * 7, 64), true, parallel_ctx);  // with a bias, src/zoo.cc:1548
  parallel_vars_insert_all(net.dev_params, conv1.params);
  parallel_vars_insert_all(net.dev_grads, conv1.grads);
  par_ys = conv1.ops;

  // pool1: 3x3 max at stride 2 over halo 1 (src/zoo.cc:1562-1574)
  Pool2DShape pool1_shape;
  pool1_shape.pooling = kMaxPool; pool1_shape.axes = {0, 1}; pool1_shape.window = {3, 3}; pool1_shape.stride = {2, 2};
  pool1_shape.pad = {1, 1}; pool1_shape.halo_padded_input = true;
  const auto stem_tile = par_ys.at(0)->shape();
  // (very wide images: a band of window rows no longer fits LDS and the kernels over tiles without halo decline;
  // the padded form below has direct kernels for such rows)
  if (mgpu_ctx->spatial_comm(0)->num_w_ranks == 1 && stem_tile.shape[1] % 2 == 0 &&
      adh_pool2d_unpadded_supported(ADH_F32, ADH_POOL_MAX, (uint32_t)num_ranks, (uint32_t)cfg.batch_size, (uint32_t)stem_tile.shape[2],
                                    (uint32_t)stem_tile.shape[1], (uint32_t)stem_tile.shape[0], 3, 3, 2, 2, 1, 1) == ADH_OK) {
    // over row tiles the pooling reads its zero padding and its neighbours' rows itself: no pad, no exchange, and
    // the stem's output gradient comes out unpadded (two passes over the largest activation of the net fewer)
    pool1_shape.halo_padded_input = false;
    pool1_shape.unpadded_tiles = true;
  } else {
    par_ys = HaloExch2DOp<V3>::MakeParallel(1, HaloPad2DOp<V3>::MakeParallel(1, par_ys, parallel_ctx), parallel_ctx);
  }
  par_ys = CudnnPool2DOp<V3>::MakeParallel(pool1_shape, par_ys, parallel_ctx);

  auto res_shape = [](size_t filters) {
    Conv2DShape s;
    s.filters = filters; s.axes = {0, 1}; s.kernel = {3, 3}; s.dilate = {1, 1}; s.stride = {1, 1}; s.pad = {1, 1};
    s.halo_padded_input = true; s.enable_hmma = false;
    return s;
  };
  auto plain = [&](size_t filters) {
    auto block = spatial_parallel_residual_v2_conv2d<V3>(res_shape(filters), net.batch_norm_use_fixed, par_ys, parallel_ctx);
    add(block);
    par_ys = block.ops;
  };
  auto proj = [&](size_t filters) {
    auto block = spatial_parallel_proj_residual_v2_conv2d<V3>(res_shape(filters), 2, net.batch_norm_use_fixed, par_ys, parallel_ctx);
    add(block);
    par_ys = block.ops;
  };
  plain(64);   // res2_1
  plain(64);   // res2_2
  proj(128);   // res3_1
  plain(128);  // res3_2
  proj(256);   // res4_1
  plain(256);  // res4_2
  proj(512);   // res5_1   (res5_2 is switched off in the reference, src/zoo.cc:1760)
  proj(512);   // res6_1   (res6_2 likewise, :1801)

  auto bnorm_final = CudnnBatchNorm2DOp<bool, V3, B1>::MakeParallel(512, net.batch_norm_use_fixed, par_ys, parallel_ctx, true, 0);
  parallel_vars_insert_all(net.dev_params, bnorm_final.params);
  parallel_vars_insert_all(net.dev_grads, bnorm_final.grads);
  parallel_vars_insert_all(net.dev_batch_stats, bnorm_final.batch_stats);
  parallel_vars_insert_all(net.dev_fixed_stats, bnorm_final.fixed_stats);
  par_ys = bnorm_final.ops;  // batch norm and rectifier in one node

  // The replicated tail (src/zoo.cc:1841-1873): every rank pools the gathered activation and applies
  // ITS copy of the classifier; the logits are summed over ranks and divided by the rank count.  With
  // equal copies that is the classifier applied once; each copy receives 1/num_ranks of the gradient
  // and the optimizer's rank sum restores the whole.
  shared_ptr<Var<V3>> gathered = SpatialJoinedGather2DOp<V3>::Make(par_ys, parallel_ctx);
  Pool2DShape global_pool_shape;
  global_pool_shape.pooling = kAveragePool; global_pool_shape.axes = {0, 1};
  global_pool_shape.window = {gathered->shape().shape[0], gathered->shape().shape[1]};
  global_pool_shape.stride = global_pool_shape.window;
  global_pool_shape.pad = {0, 0}; global_pool_shape.halo_padded_input = false;
  Conv2DShape fc_shape;
  fc_shape.filters = num_classes; fc_shape.axes = {0, 1}; fc_shape.kernel = {1, 1}; fc_shape.dilate = {1, 1};
  fc_shape.stride = {1, 1}; fc_shape.pad = {0, 0}; fc_shape.halo_padded_input = false; fc_shape.enable_hmma = false;
  vector<shared_ptr<Var<V3>>> rank_pooled;
  for (size_t rank = 0; rank < num_ranks; ++rank)
    rank_pooled.push_back(CudnnPool2DOp<V3>::Make(global_pool_shape, gathered, mgpu_ctx->device_context(rank)));
  // one node (and, the copies being equal, one launch per pass) applies every rank's classifier
  auto fc = parallel_conv2d<V3, A4>(fc_shape, rank_pooled, xavier_init_gen<A4>(512, num_classes), false, parallel_ctx);
  parallel_vars_insert_all(net.dev_params, fc.params);
  parallel_vars_insert_all(net.dev_grads, fc.grads);
  vector<shared_ptr<Var<V3>>> rank_logits = fc.ops;
  shared_ptr<Var<V3>> y = sum<V3>(rank_logits, root);
  y = ScaleOp<float, V3>::Make(1.0f / static_cast<float>(num_ranks), y, root);
  net.op = FlattenNCHWOp<V3, V1>::Make(y, root);
  net.loss = softmax_nll_loss<V1, L0, F0>(net.op, net.label, root);
  net.loss->set_sink_grad(1.0f / static_cast<float>(cfg.minibatch_size));
  net.sum_loss = net.loss;
  return net;
}

}  // namespace arraydiff
