// Tests of the C++ host layer (arraydiff_cuda_amd/host) written the way a user of the
// reference's op API would write them.  `test_host cpu` runs the parts that need no GPU
// (shape algebra, Spatial2DComm protocol and error codes); `test_host gpu` builds the
// spatially-parallel conv graph with the reference's factories and checks values, input
// gradient and filter gradient against the CPU oracle's UNSPLIT convolution.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "arraydiff/op.hh"
#include "arraydiff/optimize.hh"
#include "arraydiff/zoo.hh"

extern "C" {
// CPU oracle (oracle/adh_oracle.c): the checker
void orc_conv_slab_fwd(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W, uint32_t k, const float *x_pad,
                       const float *wt, float beta, float *y);
void orc_conv_slab_bwd_data(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W, uint32_t k,
                            const float *wt, const float *dy, float beta, float *dx_pad);
void orc_conv_slab_bwd_filter(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t H, uint32_t W, uint32_t k,
                              const float *x_pad, const float *dy, float beta, float *dw);
void orc_conv2d_slab_fwd(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t kh, uint32_t kw,
                         uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, const float *x_pad, const float *wt,
                         float beta, float *y);
void orc_conv2d_slab_bwd_data(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t kh,
                              uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, const float *wt,
                              const float *dy, float beta, float *dx_pad);
void orc_conv2d_slab_bwd_filter(uint32_t N, uint32_t Cin, uint32_t Cout, uint32_t HP, uint32_t WP, uint32_t kh,
                                uint32_t kw, uint32_t sh, uint32_t sw, uint32_t dh, uint32_t dw, const float *x_pad,
                                const float *dy, float beta, float *dwt);
void orc_halo_pad(int dtype, uint32_t p, uint32_t W, uint32_t H, uint32_t C, uint32_t N, const void *x, void *y);
void orc_halo_unpad(int dtype, uint32_t p, uint32_t W, uint32_t H, uint32_t C, uint32_t N, const void *x, void *y);
int orc_halo_op(int which, int dtype, uint32_t gw, uint32_t gh, uint32_t p, uint32_t W, uint32_t H, uint32_t C,
                uint32_t N, void *const *tiles);
void orc_pool_slab_fwd(int mode, uint32_t N, uint32_t C, uint32_t HP, uint32_t WP, uint32_t wh, uint32_t ww, uint32_t sh,
                       uint32_t sw, const float *x, float *y);
void orc_pool_slab_bwd(int mode, uint32_t N, uint32_t C, uint32_t HP, uint32_t WP, uint32_t wh, uint32_t ww, uint32_t sh,
                       uint32_t sw, const float *x, const float *dy, float beta, float *dx);
void orc_batchnorm2d_fwd_train(uint32_t N, uint32_t C, uint32_t H, uint32_t W, float eps, int relu, uint32_t p,
                               const float *x, const float *scale, const float *shift, float *y, float *run_mean,
                               float *run_var, float *save_mean, float *save_invstd);
void orc_batchnorm2d_bwd(uint32_t N, uint32_t C, uint32_t H, uint32_t W, int relu, uint32_t p, const float *x,
                         const float *dy, const float *scale, const float *shift, const float *save_mean,
                         const float *save_invstd, float beta_data, float beta_param, float *dx, float *dscale,
                         float *dshift);
void orc_softmax_fwd(uint32_t C, uint32_t N, const float *x, float *y);
void orc_softmax_nll_loss_fwd(uint32_t C, uint32_t N, const float *y, const uint32_t *label, float *loss);
void orc_softmax_nll_loss_bwd(uint32_t C, uint32_t N, const float *y, const uint32_t *label, const float *dloss,
                              float *dx);
void orc_sgd_step(uint64_t n, uint32_t num_grads, const float *const *grads, float l2_reg, float mu, float alpha,
                  float next_alpha, int nesterov, float *param, float *momentum_grad, float *lagged, float *sum_grad);
void orc_stat_step(uint64_t n, float rate, const float *avg_stat, float *running_stat, float *stat);
}

using namespace arraydiff;

static int failures = 0;
#define CHECK(cond)                                                       \
  do {                                                                    \
    if (!(cond)) {                                                        \
      std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);         \
      ++failures;                                                         \
    }                                                                     \
  } while (0)

static double rel_err(const std::vector<float> &a, const std::vector<float> &b) {
  double num = 0, den = 0;
  for (size_t i = 0; i < a.size(); ++i) {
    num = std::fmax(num, std::fabs((double)a[i] - b[i]));
    den = std::fmax(den, std::fabs((double)b[i]));
  }
  return num / (den > 0 ? den : 1);
}

static void test_shapes() {
  Shape3D padded(58, 16, 64);
  CHECK(padded.packed_stride().shape[2] == 928);
  Shape3D dim(56, 14, 64), off(1, 1, 0), stride = padded.packed_stride();
  CHECK(stride.packed_dim(dim.minor()) == padded);
  CHECK(!dim.is_packed(stride) && dim.is_packed(dim.packed_stride()));
  CHECK(off.to_index(stride) == 59);
  CHECK(dim.append(32) == Shape4D(56, 14, 64, 32));
  CHECK(Shape3D::Zero().is_zero() && dim.flat_size() == 56u * 14 * 64);
  // brute force: to_index of (w,h,c,n) against nested loops over a padded buffer
  size_t p = 2, W = 5, H = 4, C = 3, N = 2, lin = 0;
  Shape4D st = Shape3D(W + 2 * p, H + 2 * p, C).packed_stride().append((W + 2 * p) * (H + 2 * p) * C);
  for (size_t n = 0; n < N; ++n)
    for (size_t c = 0; c < C; ++c)
      for (size_t h = 0; h < H + 2 * p; ++h)
        for (size_t w = 0; w < W + 2 * p; ++w, ++lin) CHECK(Shape4D(w, h, c, n).to_index(st) == lin);
  CHECK(Shape0D().flat_size() == 1 && Shape0D().append(7) == Shape1D(7));
}

static void test_comm_protocol() {
  Spatial2DComm comms[4];
  CHECK(Spatial2DComm::InitAll(comms, 2, 2) == ADH_OK);
  // rank = r_w + num_w * r_h
  CHECK(comms[3].rank == 3 && comms[3].rank_w == 1 && comms[3].rank_h == 1 && comms[2].rank_w == 0);
  CHECK(Spatial2DComm::InitAll(comms, 0, 2) == ADH_EINVAL);
  CHECK(Spatial2DComm::InitAll(nullptr, 1, 2) == ADH_ENULL);
  GPUConn conn(0, nullptr);
  float dummy[4];
  // 2x2 grid: every rank recorded, but the combination is unimplemented
  CHECK(Spatial2DComm::InitAll(comms, 2, 2) == ADH_OK);
  for (int r = 0; r < 4; ++r) {
    comms[r].group_start();
    comms[r].halo_exchange(dummy, 1, 2, 2, 1, 1, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
  }
  CHECK(comms[0].group_end(conn) == ADH_EUNIMPL);
  // 1x4: a peer that has not recorded for this epoch -> protocol error instead of a hang
  CHECK(Spatial2DComm::InitAll(comms, 1, 4) == ADH_OK);
  for (int r = 0; r < 3; ++r) {
    comms[r].group_start();
    comms[r].halo_exchange(dummy, 1, 2, 2, 1, 1, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
  }
  CHECK(comms[0].group_end(conn) == ADH_EPROTOCOL);
  comms[3].group_start();
  comms[3].halo_exchange(nullptr, 1, 2, 2, 1, 1, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
  CHECK(comms[0].group_end(conn) == ADH_ENULL);  // NULL buffer (src/spatial.cc:71-73)
  // unsupported format / type
  for (int r = 0; r < 4; ++r) {
    comms[r].group_start();
    comms[r].halo_exchange(dummy, 1, 2, 2, 1, 1, SPATIAL2D_TENSOR_NHWC, SPATIAL2D_DATA_FLOAT);
  }
  CHECK(comms[1].group_end(conn) == ADH_EUNIMPL);
  for (int r = 0; r < 4; ++r) {
    comms[r].group_start();
    comms[r].halo_reduce(dummy, 1, 2, 2, 1, 1, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_DOUBLE);
  }
  CHECK(comms[1].group_end(conn) == ADH_EUNIMPL);
  CHECK(Spatial2DComm::group_end_all(comms, conn) == ADH_EUNIMPL);
  // mismatched arguments between ranks
  for (int r = 0; r < 4; ++r) {
    comms[r].group_start();
    comms[r].halo_exchange(dummy, 1, 2 + (r == 2), 2, 1, 1, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
  }
  CHECK(Spatial2DComm::group_end_all(comms, conn) == ADH_EINVAL);
  // reduce with H < 2*halo: rejected by the C ABI before any launch
  for (int r = 0; r < 4; ++r) {
    comms[r].group_start();
    comms[r].halo_reduce(dummy, 2, 4, 3, 1, 1, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
  }
  CHECK(comms[2].group_end(conn) == ADH_EINVAL);
  // 1x1: nothing to do
  Spatial2DComm one[1];
  CHECK(Spatial2DComm::InitAll(one, 1, 1) == ADH_OK);
  one[0].group_start();
  one[0].halo_exchange(dummy, 1, 2, 2, 1, 1, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
  CHECK(one[0].group_end(conn) == ADH_OK);
  CHECK(comms[0].epoch == comms[1].epoch);
}

static std::vector<float> uniform(std::mt19937 &g, size_t n, float lo, float hi) {
  std::uniform_real_distribution<float> d(lo, hi);
  std::vector<float> v(n);
  for (auto &x : v) x = d(g);
  return v;
}
static std::vector<float> normal(std::mt19937 &g, size_t n, float s) {
  std::normal_distribution<float> d(0.f, s);
  std::vector<float> v(n);
  for (auto &x : v) x = d(g);
  return v;
}

// Broadcast(X) -> Scatter -> HaloPad -> HaloExch -> Conv(halo_padded_input) -> gather, the block
// of src/zoo.cc:577-652 and :1522-1526, on K row-tiles of one GPU.
// unexchanged: the exchange node copies nothing in the forward pass and the convolution reads its neighbours'
// rows itself (tiles of more than 256 pixels) or exchanges first (smaller ones)
// halo_free: no pad and no exchange node at all: the conv node takes the scattered tiles as they are
static void test_spatial_conv_graph(size_t K, size_t N, size_t C, size_t Co, size_t H, size_t W, bool unexchanged = false,
                                    bool halo_free = false) {
  std::mt19937 gen(1234 + (unsigned)K);
  auto ctx = MultiGPUContext::Make(K);
  std::vector<float> X = uniform(gen, N * C * H * W, -1, 1);
  std::vector<float> Wt = normal(gen, Co * C * 9, std::sqrt(2.0f / (C * 9)));
  std::vector<float> dY = normal(gen, N * Co * H * W, 1.0f);

  typedef GPUBatchArray3D<float> V;
  typedef GPUArray4D<float> A;
  auto x_src = SrcOp<V>::Make(Shape3D(W, H, C), N, ctx->device_context(0));
  auto w_src = ParamOp<A>::Make(Shape4D(3, 3, C, Co), ctx->device_context(0));
  vector<shared_ptr<Var<V>>> xs(K, x_src);
  vector<shared_ptr<Var<A>>> ws(K, w_src);
  auto tiles = SpatialScatter2DOp<V>::MakeParallel(xs, ctx);
  auto padded = HaloPad2DOp<V>::MakeParallel(1, tiles, ctx);
  auto exch = HaloExch2DOp<V>::MakeParallel(1, padded, ctx, unexchanged);
  Conv2DShape cs;
  cs.filters = Co;
  cs.axes = {0, 1};
  cs.kernel = {3, 3};
  cs.dilate = {1, 1};
  cs.stride = {1, 1};
  cs.pad = {1, 1};
  cs.halo_padded_input = !halo_free;
  cs.enable_hmma = false;
  cs.unexchanged_rows = unexchanged;
  cs.unpadded_tiles = halo_free;
  auto ys = CudnnConv2DOp<V, A, A>::MakeParallel(cs, halo_free ? tiles : exch, ws, ctx);
  auto y_full = SpatialJoinedGather2DOp<V>::Make(ys, ctx);
  auto sink = HostGradSinkOp<V>::Make(y_full, ctx->device_context(0));
  sink->set_host_grad(dY.data());

  CHECK(padded[0]->offset() == Shape3D(1, 1, 0));
  CHECK(padded[0]->stride() == Shape3D(W + 2, H / K + 2, C).packed_stride());
  CHECK(ys[0]->shape() == Shape3D(W, H / K, Co));

  for (int rep = 0; rep < 2; ++rep) {  // two transactions: buffers are reused, first touch re-zeroes
    TxnId txn;
    x_src->load(txn, X.data());
    w_src->load(txn, Wt.data());
    sink->gradient(txn);
    ctx->sync();
    std::vector<float> Y(N * Co * H * W), dX(X.size()), dW(Wt.size());
    sink->store_val(txn, Y.data());
    x_src->store_grad(txn, dX.data());
    w_src->store_grad(txn, dW.data());

    // oracle: the UNSPLIT convolution over the zero-padded full tensor
    std::vector<float> Xp(N * C * (H + 2) * (W + 2));
    orc_halo_pad(0, 1, W, H, C, N, X.data(), Xp.data());
    std::vector<float> Yr(Y.size()), dXp(Xp.size()), dXr(X.size()), dWr(Wt.size());
    orc_conv_slab_fwd(N, C, Co, H, W, 3, Xp.data(), Wt.data(), 0.f, Yr.data());
    orc_conv_slab_bwd_data(N, C, Co, H, W, 3, Wt.data(), dY.data(), 0.f, dXp.data());
    orc_halo_unpad(0, 1, W, H, C, N, dXp.data(), dXr.data());
    orc_conv_slab_bwd_filter(N, C, Co, H, W, 3, Xp.data(), dY.data(), 0.f, dWr.data());
    const double ey = rel_err(Y, Yr), ex = rel_err(dX, dXr), ew = rel_err(dW, dWr);
    std::printf("graph K=%zu N=%zu C=%zu->%zu %zux%zu%s rep %d: rel-err y %.2e dx %.2e dw %.2e\n", K, N, C, Co, H, W,
                halo_free ? " tiles without halo" : unexchanged ? " unexchanged" : "", rep, ey, ex, ew);
    CHECK(ey <= 1e-5 && ex <= 1e-5 && ew <= 1e-5);
  }
}

// rows [r*Ht, (r+1)*Ht) of an unsplit NCHW tensor <-> a packed tile
static std::vector<float> tile_of(const std::vector<float> &full, size_t N, size_t C, size_t H, size_t W, size_t K, size_t r) {
  const size_t Ht = H / K;
  std::vector<float> t(N * C * Ht * W);
  for (size_t nc = 0; nc < N * C; ++nc)
    std::memcpy(&t[nc * Ht * W], &full[(nc * H + r * Ht) * W], Ht * W * sizeof(float));
  return t;
}
static void put_tile(std::vector<float> &full, const std::vector<float> &t, size_t N, size_t C, size_t H, size_t W, size_t K,
                     size_t r) {
  const size_t Ht = H / K;
  for (size_t nc = 0; nc < N * C; ++nc)
    std::memcpy(&full[(nc * H + r * Ht) * W], &t[nc * Ht * W], Ht * W * sizeof(float));
}

// spatial_parallel_residual_v2_conv2d (src/zoo.cc:577-652) built with the reference's factories on K
// row-tiles of one GPU:  x -> BN -> ReLU -> HaloPad -> HaloExch -> conv -> BN -> ReLU -> HaloPad ->
// HaloExch -> conv -> (+ x).  Every rank's batch norm uses its own tile's statistics.  Oracle: the
// same chain with per-tile batch norms and UNSPLIT convolutions.
// fused: batch norm + rectifier + halo pad as one node (SlabBatchNorm2DOp with relu and out_halo) instead of three
// shared_grad: the sum's output gradient, the second conv's output gradient (JoinOp's sole_consumer_of) and the block
// input's gradient (trunk_input: the first batch norm adds to it in place) are one buffer: the sum's backward pass copies nothing
// sum_in_conv: both convs run over tiles without halo and the second adds the block input to its result (no pad,
// exchange or sum node; the block input's gradient is the second conv's output gradient)
static void test_spatial_residual_block(size_t K, size_t N, size_t C, size_t H, size_t W, bool fused = false,
                                        bool shared_grad = false, bool sum_in_conv = false) {
  std::mt19937 gen(31337 + (unsigned)K);
  auto ctx = MultiGPUContext::Make(K);
  typedef GPUBatchArray3D<float> V;
  typedef GPUArray4D<float> A;
  typedef GPUArray1D<float> B;
  const size_t Ht = H / K, full = N * C * H * W;
  std::vector<float> X = uniform(gen, full, -1, 1), dY = normal(gen, full, 1.0f);
  std::vector<float> W1 = normal(gen, C * C * 9, std::sqrt(2.0f / (C * 9))), W2 = normal(gen, C * C * 9, std::sqrt(2.0f / (C * 9)));
  std::vector<std::vector<float>> sc0(K), sh0(K), sc1(K), sh1(K);
  for (size_t r = 0; r < K; ++r) {
    sc0[r] = uniform(gen, C, 0.5f, 1.5f); sh0[r] = uniform(gen, C, -0.5f, 0.5f);
    sc1[r] = uniform(gen, C, 0.5f, 1.5f); sh1[r] = uniform(gen, C, -0.5f, 0.5f);
  }
  auto x_src = SrcOp<V>::Make(Shape3D(W, H, C), N, ctx->device_context(0));
  auto w1_src = ParamOp<A>::Make(Shape4D(3, 3, C, C), ctx->device_context(0));
  auto w2_src = ParamOp<A>::Make(Shape4D(3, 3, C, C), ctx->device_context(0));
  vector<shared_ptr<Var<V>>> xs(K, x_src);
  auto inputs = SpatialScatter2DOp<V>::MakeParallel(xs, ctx);
  auto switch_var = std::make_shared<bool>(false);
  Conv2DShape cs;
  cs.filters = C; cs.axes = {0, 1}; cs.kernel = {3, 3}; cs.dilate = {1, 1}; cs.stride = {1, 1}; cs.pad = {1, 1};
  cs.halo_padded_input = true; cs.enable_hmma = false;
  if (sum_in_conv) {
    cs.halo_padded_input = false;
    cs.unpadded_tiles = true;
  }
  const size_t halo = sum_in_conv ? 0 : 1;
  auto bnorm0 = CudnnBatchNorm2DOp<bool, V, B>::MakeParallel(C, switch_var, inputs, ctx, fused, fused ? halo : 0);
  auto pad1 = fused ? bnorm0.ops : HaloPad2DOp<V>::MakeParallel(1, parallel_relu<V>(bnorm0.ops, ctx), ctx);
  auto exch1 = sum_in_conv ? pad1 : HaloExch2DOp<V>::MakeParallel(1, pad1, ctx);
  auto conv1 = CudnnConv2DOp<V, A, A>::MakeParallel(cs, exch1, vector<shared_ptr<Var<A>>>(K, w1_src), ctx);
  auto bnorm1 = CudnnBatchNorm2DOp<bool, V, B>::MakeParallel(C, switch_var, conv1, ctx, fused, fused ? halo : 0);
  auto pad2 = fused ? bnorm1.ops : HaloPad2DOp<V>::MakeParallel(1, parallel_relu<V>(bnorm1.ops, ctx), ctx);
  auto exch2 = sum_in_conv ? pad2 : HaloExch2DOp<V>::MakeParallel(1, pad2, ctx);
  auto conv2 = CudnnConv2DOp<V, A, A>::MakeParallel(cs, exch2, vector<shared_ptr<Var<A>>>(K, w2_src), ctx,
                                                    sum_in_conv ? inputs : vector<shared_ptr<Var<V>>>());
  vector<vector<shared_ptr<Var<V>>>> join_inputs{inputs, conv2};
  auto join = sum_in_conv ? conv2 : parallel_sum<V>(join_inputs, ctx, shared_grad ? 1 : -1, shared_grad ? 0 : -1);
  auto y_full = SpatialJoinedGather2DOp<V>::Make(join, ctx);
  auto sink = HostGradSinkOp<V>::Make(y_full, ctx->device_context(0));
  sink->set_host_grad(dY.data());
  CHECK(bnorm0.params.at(0).size() == 2 && bnorm0.grads.at(0).size() == 2);

  for (int rep = 0; rep < 2; ++rep) {
    TxnId txn;
    x_src->load(txn, X.data());
    w1_src->load(txn, W1.data());
    w2_src->load(txn, W2.data());
    for (size_t r = 0; r < K; ++r) {
      bnorm0.scales[r]->load(txn, sc0[r].data()); bnorm0.shifts[r]->load(txn, sh0[r].data());
      bnorm1.scales[r]->load(txn, sc1[r].data()); bnorm1.shifts[r]->load(txn, sh1[r].data());
    }
    sink->gradient(txn);
    ctx->sync();
    std::vector<float> Y(full), dX(full), dW1(W1.size()), dW2(W2.size());
    sink->store_val(txn, Y.data());
    x_src->store_grad(txn, dX.data());
    w1_src->store_grad(txn, dW1.data());
    w2_src->store_grad(txn, dW2.data());

    // oracle forward
    const float eps = 1.0e-5f;
    std::vector<std::vector<float>> m0(K, std::vector<float>(C)), i0(K, std::vector<float>(C)), m1 = m0, i1 = i0;
    std::vector<float> A0(full), C1(full), A1(full), C2(full), Yr(full);
    for (size_t r = 0; r < K; ++r) {
      auto xt = tile_of(X, N, C, H, W, K, r);
      std::vector<float> yt(xt.size());
      orc_batchnorm2d_fwd_train(N, C, Ht, W, eps, 1, 0, xt.data(), sc0[r].data(), sh0[r].data(), yt.data(), nullptr, nullptr,
                                m0[r].data(), i0[r].data());
      put_tile(A0, yt, N, C, H, W, K, r);
    }
    std::vector<float> A0p(N * C * (H + 2) * (W + 2)), A1p(A0p.size());
    orc_halo_pad(0, 1, W, H, C, N, A0.data(), A0p.data());
    orc_conv_slab_fwd(N, C, C, H, W, 3, A0p.data(), W1.data(), 0.f, C1.data());
    for (size_t r = 0; r < K; ++r) {
      auto xt = tile_of(C1, N, C, H, W, K, r);
      std::vector<float> yt(xt.size());
      orc_batchnorm2d_fwd_train(N, C, Ht, W, eps, 1, 0, xt.data(), sc1[r].data(), sh1[r].data(), yt.data(), nullptr, nullptr,
                                m1[r].data(), i1[r].data());
      put_tile(A1, yt, N, C, H, W, K, r);
    }
    orc_halo_pad(0, 1, W, H, C, N, A1.data(), A1p.data());
    orc_conv_slab_fwd(N, C, C, H, W, 3, A1p.data(), W2.data(), 0.f, C2.data());
    for (size_t i = 0; i < full; ++i) Yr[i] = X[i] + C2[i];
    // oracle backward
    std::vector<float> dA1p(A1p.size()), dA1(full), dC1(full), dA0p(A0p.size()), dA0(full), dXr(full), dW1r(W1.size()),
        dW2r(W2.size());
    orc_conv_slab_bwd_data(N, C, C, H, W, 3, W2.data(), dY.data(), 0.f, dA1p.data());
    orc_conv_slab_bwd_filter(N, C, C, H, W, 3, A1p.data(), dY.data(), 0.f, dW2r.data());
    orc_halo_unpad(0, 1, W, H, C, N, dA1p.data(), dA1.data());
    double e_param = 0;
    for (size_t r = 0; r < K; ++r) {
      auto xt = tile_of(C1, N, C, H, W, K, r), dyt = tile_of(dA1, N, C, H, W, K, r);
      std::vector<float> dxt(xt.size()), ds(C), db(C), got_ds(C), got_db(C);
      orc_batchnorm2d_bwd(N, C, Ht, W, 1, 0, xt.data(), dyt.data(), sc1[r].data(), sh1[r].data(), m1[r].data(), i1[r].data(),
                          0.f, 0.f, dxt.data(), ds.data(), db.data());
      put_tile(dC1, dxt, N, C, H, W, K, r);
      bnorm1.scales[r]->store_grad(txn, got_ds.data());
      bnorm1.shifts[r]->store_grad(txn, got_db.data());
      e_param = std::fmax(e_param, std::fmax(rel_err(got_ds, ds), rel_err(got_db, db)));
    }
    orc_conv_slab_bwd_data(N, C, C, H, W, 3, W1.data(), dC1.data(), 0.f, dA0p.data());
    orc_conv_slab_bwd_filter(N, C, C, H, W, 3, A0p.data(), dC1.data(), 0.f, dW1r.data());
    orc_halo_unpad(0, 1, W, H, C, N, dA0p.data(), dA0.data());
    for (size_t r = 0; r < K; ++r) {
      auto xt = tile_of(X, N, C, H, W, K, r), dyt = tile_of(dA0, N, C, H, W, K, r);
      std::vector<float> dxt(xt.size()), ds(C), db(C), got_ds(C), got_db(C);
      orc_batchnorm2d_bwd(N, C, Ht, W, 1, 0, xt.data(), dyt.data(), sc0[r].data(), sh0[r].data(), m0[r].data(), i0[r].data(),
                          0.f, 0.f, dxt.data(), ds.data(), db.data());
      put_tile(dXr, dxt, N, C, H, W, K, r);
      bnorm0.scales[r]->store_grad(txn, got_ds.data());
      bnorm0.shifts[r]->store_grad(txn, got_db.data());
      e_param = std::fmax(e_param, std::fmax(rel_err(got_ds, ds), rel_err(got_db, db)));
    }
    for (size_t i = 0; i < full; ++i) dXr[i] += dY[i];
    const double ey = rel_err(Y, Yr), ex = rel_err(dX, dXr), ew1 = rel_err(dW1, dW1r), ew2 = rel_err(dW2, dW2r);
    std::printf("residual block%s K=%zu N=%zu C=%zu %zux%zu rep %d: rel-err y %.2e dx %.2e dw1 %.2e dw2 %.2e bn params %.2e\n",
                sum_in_conv ? " (sum in the second conv)" : fused ? " (fused bn+relu+pad)" : "", K, N, C, H, W, rep, ey, ex, ew1,
                ew2, e_param);
    CHECK(ey <= 1e-5 && ex <= 2e-5 && ew1 <= 2e-5 && ew2 <= 1e-5 && e_param <= 1e-4);
  }
}

// The same graph with any window k, stride s, dilation d and halo p = d * (k - 1) / 2: the 7x7 stem
// over halo 3 (src/zoo.cc:1525-1538), the stride-2 3x3 (src/zoo.cc:692-697) and the dilated 3x3 of
// tools/microbench_spatial_conv.cc:25-32, against the oracle's UNSPLIT convolution.
// halo_free: no pad and no exchange node: the conv node takes the scattered tiles as they are
static void test_spatial_general_conv_graph(size_t K, size_t N, size_t C, size_t Co, size_t H, size_t W, size_t k,
                                            size_t st, size_t dil, bool halo_free = false) {
  std::mt19937 gen(777 + (unsigned)(k * 10 + st));
  const size_t p = dil * (k - 1) / 2;
  const size_t OH = (H + 2 * p - (dil * (k - 1) + 1)) / st + 1, OW = (W + 2 * p - (dil * (k - 1) + 1)) / st + 1;
  auto ctx = MultiGPUContext::Make(K);
  std::vector<float> X = uniform(gen, N * C * H * W, -1, 1);
  std::vector<float> Wt = normal(gen, Co * C * k * k, std::sqrt(2.0f / (C * k * k)));
  std::vector<float> dY = normal(gen, N * Co * OH * OW, 1.0f);
  typedef GPUBatchArray3D<float> V;
  typedef GPUArray4D<float> A;
  auto x_src = SrcOp<V>::Make(Shape3D(W, H, C), N, ctx->device_context(0));
  auto w_src = ParamOp<A>::Make(Shape4D(k, k, C, Co), ctx->device_context(0));
  vector<shared_ptr<Var<V>>> xs(K, x_src);
  vector<shared_ptr<Var<A>>> ws(K, w_src);
  auto tiles = SpatialScatter2DOp<V>::MakeParallel(xs, ctx);
  auto padded = HaloPad2DOp<V>::MakeParallel(p, tiles, ctx);
  auto exch = HaloExch2DOp<V>::MakeParallel(p, padded, ctx);
  Conv2DShape cs;
  cs.filters = Co;
  cs.axes = {0, 1};
  cs.kernel = {k, k};
  cs.dilate = {dil, dil};
  cs.stride = {st, st};
  cs.pad = {p, p};
  cs.halo_padded_input = !halo_free;
  cs.unpadded_tiles = halo_free;
  cs.enable_hmma = false;
  auto ys = CudnnConv2DOp<V, A, A>::MakeParallel(cs, halo_free ? tiles : exch, ws, ctx);
  CHECK(ys[0]->shape() == Shape3D(OW, OH / K, Co));
  auto y_full = SpatialJoinedGather2DOp<V>::Make(ys, ctx);
  auto sink = HostGradSinkOp<V>::Make(y_full, ctx->device_context(0));
  sink->set_host_grad(dY.data());
  for (int rep = 0; rep < 2; ++rep) {
    TxnId txn;
    x_src->load(txn, X.data());
    w_src->load(txn, Wt.data());
    sink->gradient(txn);
    ctx->sync();
    std::vector<float> Y(dY.size()), dX(X.size()), dW(Wt.size());
    sink->store_val(txn, Y.data());
    x_src->store_grad(txn, dX.data());
    w_src->store_grad(txn, dW.data());
    const uint32_t HP = (uint32_t)(H + 2 * p), WP = (uint32_t)(W + 2 * p);
    std::vector<float> Xp(N * C * HP * WP), Yr(Y.size()), dXp(Xp.size()), dXr(X.size()), dWr(Wt.size());
    orc_halo_pad(0, (uint32_t)p, W, H, C, N, X.data(), Xp.data());
    orc_conv2d_slab_fwd(N, C, Co, HP, WP, k, k, st, st, dil, dil, Xp.data(), Wt.data(), 0.f, Yr.data());
    orc_conv2d_slab_bwd_data(N, C, Co, HP, WP, k, k, st, st, dil, dil, Wt.data(), dY.data(), 0.f, dXp.data());
    orc_halo_unpad(0, (uint32_t)p, W, H, C, N, dXp.data(), dXr.data());
    orc_conv2d_slab_bwd_filter(N, C, Co, HP, WP, k, k, st, st, dil, dil, Xp.data(), dY.data(), 0.f, dWr.data());
    const double ey = rel_err(Y, Yr), ex = rel_err(dX, dXr), ew = rel_err(dW, dWr);
    std::printf("general conv graph k=%zu s=%zu d=%zu K=%zu N=%zu C=%zu->%zu %zux%zu%s rep %d: rel-err y %.2e dx %.2e dw %.2e\n",
                k, st, dil, K, N, C, Co, H, W, halo_free ? " tiles without halo" : "", rep, ey, ex, ew);
    CHECK(ey <= 1e-5 && ex <= 1e-5 && ew <= 1e-5);
  }
}

// The conv graph with what every rank of the reference owns for itself: a bias vector per rank (CudnnConv2DOp built
// with a bias, src/op.cc:1602-1610, 1632-1648; distinct values per rank so that a tile given its neighbour's vector
// shows) and, with rank_filters, a filter variable per rank (equal values, distinct buffers: one launch per rank, the
// ranks' filter gradients add up to the unsplit one).  shared_bias: one bias variable for all ranks, whose gradient
// is the sum over all tiles.  unexchanged: HaloExch2DOp copies nothing forward and the conv node exchanges (or reads
// across tiles) itself; with rank_filters no single launch holds every tile, so it exchanges once before and reduces
// once after the per-rank launches.
static void test_spatial_conv_bias_graph(size_t K, size_t N, size_t C, size_t Co, size_t H, size_t W, size_t k, bool shared_bias,
                                         bool rank_filters, bool unexchanged = false, bool halo_free = false) {
  std::mt19937 gen(4321 + (unsigned)(K * 7 + k));
  const size_t p = (k - 1) / 2, Ht = H / K;
  auto ctx = MultiGPUContext::Make(K);
  std::vector<float> X = uniform(gen, N * C * H * W, -1, 1);
  std::vector<float> Wt = normal(gen, Co * C * k * k, std::sqrt(2.0f / (C * k * k)));
  std::vector<float> dY = normal(gen, N * Co * H * W, 1.0f);
  std::vector<std::vector<float>> Bv;
  for (size_t r = 0; r < (shared_bias ? 1 : K); ++r) Bv.push_back(uniform(gen, Co, -1, 1));
  typedef GPUBatchArray3D<float> V;
  typedef GPUArray4D<float> A;
  typedef GPUArray1D<float> B;
  auto x_src = SrcOp<V>::Make(Shape3D(W, H, C), N, ctx->device_context(0));
  vector<shared_ptr<ParamOp<A>>> w_srcs;
  vector<shared_ptr<ParamOp<B>>> b_srcs;
  vector<shared_ptr<Var<A>>> ws;
  vector<shared_ptr<Var<B>>> bs;
  for (size_t r = 0; r < K; ++r) {
    if (r == 0 || rank_filters) w_srcs.push_back(ParamOp<A>::Make(Shape4D(k, k, C, Co), ctx->device_context(r)));
    if (r == 0 || !shared_bias) b_srcs.push_back(ParamOp<B>::Make(Shape1D(Co), ctx->device_context(r)));
    ws.push_back(w_srcs.back());
    bs.push_back(b_srcs.back());
  }
  vector<shared_ptr<Var<V>>> xs(K, x_src);
  auto tiles = SpatialScatter2DOp<V>::MakeParallel(xs, ctx);
  vector<shared_ptr<Var<V>>> conv_in = tiles;
  if (!halo_free) conv_in = HaloExch2DOp<V>::MakeParallel(p, HaloPad2DOp<V>::MakeParallel(p, tiles, ctx), ctx, unexchanged);
  Conv2DShape cs;
  cs.filters = Co;
  cs.axes = {0, 1};
  cs.kernel = {k, k};
  cs.dilate = {1, 1};
  cs.stride = {1, 1};
  cs.pad = {p, p};
  cs.halo_padded_input = !halo_free;
  cs.unpadded_tiles = halo_free;
  cs.unexchanged_rows = unexchanged;
  cs.enable_hmma = false;
  auto ys = CudnnConv2DOp<V, A, B>::MakeParallel(cs, conv_in, ws, ctx, {}, bs);
  auto y_full = SpatialJoinedGather2DOp<V>::Make(ys, ctx);
  auto sink = HostGradSinkOp<V>::Make(y_full, ctx->device_context(0));
  sink->set_host_grad(dY.data());
  for (int rep = 0; rep < 2; ++rep) {
    TxnId txn;
    x_src->load(txn, X.data());
    for (auto &w : w_srcs) w->load(txn, Wt.data());
    for (size_t r = 0; r < b_srcs.size(); ++r) b_srcs[r]->load(txn, Bv[r].data());
    sink->gradient(txn);
    ctx->sync();
    std::vector<float> Y(dY.size()), dX(X.size()), dW(Wt.size(), 0.f), dWr_rank(Wt.size());
    sink->store_val(txn, Y.data());
    x_src->store_grad(txn, dX.data());
    for (auto &w : w_srcs) {
      w->store_grad(txn, dWr_rank.data());
      for (size_t i = 0; i < dW.size(); ++i) dW[i] += dWr_rank[i];
    }
    const uint32_t HP = (uint32_t)(H + 2 * p), WP = (uint32_t)(W + 2 * p);
    std::vector<float> Xp(N * C * HP * WP), Yr(Y.size()), dXp(Xp.size()), dXr(X.size()), dWr(Wt.size());
    orc_halo_pad(0, (uint32_t)p, W, H, C, N, X.data(), Xp.data());
    orc_conv2d_slab_fwd(N, C, Co, HP, WP, k, k, 1, 1, 1, 1, Xp.data(), Wt.data(), 0.f, Yr.data());
    for (size_t n = 0; n < N; ++n)  // rows of tile r take rank r's bias
      for (size_t c = 0; c < Co; ++c)
        for (size_t h = 0; h < H; ++h)
          for (size_t w = 0; w < W; ++w) Yr[((n * Co + c) * H + h) * W + w] += Bv[shared_bias ? 0 : h / Ht][c];
    orc_conv2d_slab_bwd_data(N, C, Co, HP, WP, k, k, 1, 1, 1, 1, Wt.data(), dY.data(), 0.f, dXp.data());
    orc_halo_unpad(0, (uint32_t)p, W, H, C, N, dXp.data(), dXr.data());
    orc_conv2d_slab_bwd_filter(N, C, Co, HP, WP, k, k, 1, 1, 1, 1, Xp.data(), dY.data(), 0.f, dWr.data());
    double eb = 0;
    for (size_t r = 0; r < b_srcs.size(); ++r) {
      std::vector<float> dB(Co), dBr(Co);
      b_srcs[r]->store_grad(txn, dB.data());
      for (size_t c = 0; c < Co; ++c) {
        double a = 0;
        for (size_t n = 0; n < N; ++n)
          for (size_t h = shared_bias ? 0 : r * Ht; h < (shared_bias ? H : (r + 1) * Ht); ++h)
            for (size_t w = 0; w < W; ++w) a += dY[((n * Co + c) * H + h) * W + w];
        dBr[c] = (float)a;
      }
      eb = std::fmax(eb, rel_err(dB, dBr));
    }
    const double ey = rel_err(Y, Yr), ex = rel_err(dX, dXr), ew = rel_err(dW, dWr);
    std::printf("conv + bias graph k=%zu K=%zu N=%zu C=%zu->%zu %zux%zu%s%s%s%s rep %d: rel-err y %.2e dx %.2e dw %.2e db %.2e\n", k,
                K, N, C, Co, H, W, shared_bias ? " shared bias" : " bias per rank", rank_filters ? ", filter per rank" : "",
                unexchanged ? ", unexchanged" : "", halo_free ? ", tiles without halo" : "", rep, ey, ex, ew, eb);
    CHECK(ey <= 1e-5 && ex <= 1e-5 && ew <= 1e-5 && eb <= 1e-5);
  }
}

// Scatter -> HaloPad(1) -> HaloExch(1) -> Pool(3x3, stride 2, pad 1, halo_padded_input) -> gather:
// the stem pooling of src/zoo.cc:1562-1573 on K row-tiles of one GPU, against the oracle's pooling
// of the zero-padded UNSPLIT tensor.
// halo_free: no pad and no exchange node: the pooling node takes the scattered tiles as they are
static void test_spatial_pool_graph(Pooling pooling, size_t K, size_t N, size_t C, size_t H, size_t W, bool halo_free = false) {
  std::mt19937 gen(4321 + (unsigned)K);
  auto ctx = MultiGPUContext::Make(K);
  const size_t OH = (H + 2 - 3) / 2 + 1, OW = (W + 2 - 3) / 2 + 1;
  std::vector<float> X = uniform(gen, N * C * H * W, -1, 1);
  std::vector<float> dY = normal(gen, N * C * OH * OW, 1.0f);
  typedef GPUBatchArray3D<float> V;
  auto x_src = SrcOp<V>::Make(Shape3D(W, H, C), N, ctx->device_context(0));
  vector<shared_ptr<Var<V>>> xs(K, x_src);
  auto tiles = SpatialScatter2DOp<V>::MakeParallel(xs, ctx);
  auto padded = HaloPad2DOp<V>::MakeParallel(1, tiles, ctx);
  auto exch = HaloExch2DOp<V>::MakeParallel(1, padded, ctx);
  Pool2DShape ps;
  ps.pooling = pooling;
  ps.axes = {0, 1};
  ps.window = {3, 3};
  ps.stride = {2, 2};
  ps.pad = {1, 1};
  ps.halo_padded_input = !halo_free;
  ps.unpadded_tiles = halo_free;
  auto ys = CudnnPool2DOp<V>::MakeParallel(ps, halo_free ? tiles : exch, ctx);
  auto y_full = SpatialJoinedGather2DOp<V>::Make(ys, ctx);
  auto sink = HostGradSinkOp<V>::Make(y_full, ctx->device_context(0));
  sink->set_host_grad(dY.data());
  CHECK(ys[0]->shape() == Shape3D(OW, OH / K, C));
  for (int rep = 0; rep < 2; ++rep) {
    TxnId txn;
    x_src->load(txn, X.data());
    sink->gradient(txn);
    ctx->sync();
    std::vector<float> Y(dY.size()), dX(X.size());
    sink->store_val(txn, Y.data());
    x_src->store_grad(txn, dX.data());
    std::vector<float> Xp(N * C * (H + 2) * (W + 2)), Yr(Y.size()), dXp(Xp.size()), dXr(X.size());
    orc_halo_pad(0, 1, W, H, C, N, X.data(), Xp.data());
    const int mode = pooling == kMaxPool ? 1 : 0;
    orc_pool_slab_fwd(mode, N, C, H + 2, W + 2, 3, 3, 2, 2, Xp.data(), Yr.data());
    orc_pool_slab_bwd(mode, N, C, H + 2, W + 2, 3, 3, 2, 2, Xp.data(), dY.data(), 0.f, dXp.data());
    orc_halo_unpad(0, 1, W, H, C, N, dXp.data(), dXr.data());
    const double ey = rel_err(Y, Yr), ex = rel_err(dX, dXr);
    std::printf("pool graph %s K=%zu N=%zu C=%zu %zux%zu%s rep %d: rel-err y %.2e dx %.2e\n", mode ? "max" : "avg", K, N, C, H,
                W, halo_free ? " tiles without halo" : "", rep, ey, ex);
    CHECK(ey <= 1e-5 && ex <= 1e-5);
  }
}

// The call sequence of tools/microbench_spatial_conv.cc:227-263: raw buffers, per-rank
// group_start / halo_exchange / group_end, no Op machinery.
static void test_microbench_sequence() {
  const uint32_t K = 4, p = 1, W = 9, H = 5, C = 3, N = 2;
  auto ctx = MultiGPUContext::Make(K);
  std::mt19937 gen(7);
  const size_t elems = (size_t)(W + 2 * p) * (H + 2 * p) * C * N;
  std::vector<std::vector<float>> host(K);
  std::vector<GPUMemory<float>> dev;
  void *want_ptrs[K];
  std::vector<std::vector<float>> want(K);
  for (uint32_t r = 0; r < K; ++r) {
    host[r] = uniform(gen, elems, -1, 1);
    want[r] = host[r];
    want_ptrs[r] = want[r].data();
    dev.emplace_back(elems, ctx->device_context(r).get());
    GPUConn conn = ctx->device_context(r)->conn();
    dev[r].load_sync(host[r].data(), 0, elems, conn);
  }
  for (int which = 0; which < 2; ++which) {
    CHECK(orc_halo_op(which, 0, 1, K, p, W, H, C, N, want_ptrs) == 0);
    for (uint32_t r = 0; r < K; ++r) {
      ctx->spatial_comm(r)->group_start();
      if (which == 0)
        ctx->spatial_comm(r)->halo_exchange(dev[r].dptr(), p, W, H, C, N, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
      else
        ctx->spatial_comm(r)->halo_reduce(dev[r].dptr(), p, W, H, C, N, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
    }
    for (uint32_t r = 0; r < K; ++r) {
      GPUConn conn = ctx->device_context(r)->conn();
      CHECK(ctx->spatial_comm(r)->group_end(conn) == ADH_OK);
    }
    ctx->sync();
    for (uint32_t r = 0; r < K; ++r) {
      std::vector<float> got(elems);
      GPUConn conn = ctx->device_context(r)->conn();
      dev[r].store_sync(got.data(), 0, elems, conn);
      CHECK(std::memcmp(got.data(), want[r].data(), elems * 4) == 0);
    }
  }
  // the reference's launcher names work on the same buffers
  float *b[4] = {dev[0].dptr(), dev[1].dptr(), dev[2].dptr(), dev[3].dptr()};
  CHECK(orc_halo_op(0, 0, 1, K, p, W, H, C, N, want_ptrs) == 0);
  for (uint32_t r = 0; r < K; ++r)
    spatial2d_1x4_halo_exch_nchw<float>(r, p, W, H, C, N, b[0], b[1], b[2], b[3], ctx->stream());
  ctx->sync();
  for (uint32_t r = 0; r < K; ++r) {
    std::vector<float> got(elems);
    GPUConn conn = ctx->device_context(r)->conn();
    dev[r].store_sync(got.data(), 0, elems, conn);
    CHECK(std::memcmp(got.data(), want[r].data(), elems * 4) == 0);
  }
}

static void test_softmax_loss_op() {
  const size_t N = 64, C = 1000;
  auto ctx = GPUContext::Make(0);
  std::mt19937 gen(99);
  std::vector<float> x = normal(gen, N * C, 2.0f);
  std::vector<uint32_t> label(N);
  for (size_t i = 0; i < N; ++i) label[i] = gen() % C;
  typedef GPUBatchArray1D<float> V1;
  typedef GPUBatchArray0D<uint32_t> L0;
  typedef GPUBatchArray0D<float> F0;
  auto x_src = SrcOp<V1>::Make(Shape1D(C), N, ctx);
  auto l_src = SrcOp<L0>::Make(Shape0D(), N, ctx);
  auto loss = softmax_nll_loss<V1, L0, F0>(x_src, l_src, ctx);
  TxnId txn;
  x_src->load(txn, x.data());
  l_src->load(txn, label.data());
  loss->gradient(txn);
  ctx->sync();
  std::vector<float> got_loss(N), got_dx(N * C), got_y(N * C);
  loss->store_loss(txn, got_loss.data());
  loss->store_prob(txn, got_y.data());
  x_src->store_grad(txn, got_dx.data());
  std::vector<float> y(N * C), l(N), dx(N * C, 0.f), ones(N, 1.0f);
  orc_softmax_fwd(C, N, x.data(), y.data());
  orc_softmax_nll_loss_fwd(C, N, y.data(), label.data(), l.data());
  orc_softmax_nll_loss_bwd(C, N, y.data(), label.data(), ones.data(), dx.data());
  const double ey = rel_err(got_y, y), el = rel_err(got_loss, l), ed = rel_err(got_dx, dx);
  std::printf("softmax-nll op: rel-err y %.2e loss %.2e dx %.2e\n", ey, el, ed);
  CHECK(ey <= 1e-5 && el <= 1e-5 && ed <= 1e-5);
}

static void test_txn_hazards() {
  auto ctx = GPUContext::Make(0);
  typedef GPUBatchArray3D<float> V;
  auto src = SrcOp<V>::Make(Shape3D(4, 4, 2), 1, ctx);
  auto pad = HaloPad2DOp<V>::Make(1, src, ctx);
  TxnId txn;
  bool threw = false;
  try {
    pad->eval(txn);  // the source was never loaded in this transaction
  } catch (const HazardError &) {
    threw = true;
  }
  CHECK(threw);
  // pad -> unpad round trip through the ops, and HaloRepad forward
  std::vector<float> x(32), y(32);
  for (size_t i = 0; i < x.size(); ++i) x[i] = (float)i + 1;
  auto unpad = HaloUnpad2DOp<V>::Make(1, pad, ctx);
  auto sink = HostGradSinkOp<V>::Make(unpad, ctx);
  std::vector<float> g(32, 2.0f), dx(32);
  sink->set_host_grad(g.data());
  TxnId t2;
  src->load(t2, x.data());
  sink->gradient(t2);
  sink->store_val(t2, y.data());
  src->store_grad(t2, dx.data());
  CHECK(x == y && dx == g);
  bool bad = false;
  try {
    Conv2DShape cs{};
    cs.filters = 2; cs.kernel = {5, 5}; cs.stride = {1, 1}; cs.dilate = {1, 1}; cs.pad = {2, 2}; cs.halo_padded_input = true;
    auto w = ParamOp<GPUArray4D<float>>::Make(Shape4D(5, 5, 2, 2), ctx);
    auto c = CudnnConv2DOp<V, GPUArray4D<float>>::Make(cs, pad, w, ctx);
  } catch (const std::invalid_argument &) {
    bad = true;
  }
  CHECK(bad);
  bad = false;
  try {
    Pool2DShape ps{};
    ps.pooling = kMaxPool; ps.window = {3, 3}; ps.stride = {2, 2}; ps.pad = {1, 1}; ps.halo_padded_input = false;
    auto q = CudnnPool2DOp<V>::Make(ps, src, ctx);  // implicit zero padding is not on this path
  } catch (const std::invalid_argument &) {
    bad = true;
  }
  CHECK(bad);
  // pooling a packed input without padding: the global average before the classifier
  Pool2DShape gp{};
  gp.pooling = kAveragePool; gp.window = {4, 4}; gp.stride = {4, 4}; gp.pad = {0, 0}; gp.halo_padded_input = false;
  auto pooled = CudnnPool2DOp<V>::Make(gp, src, ctx);
  CHECK(pooled->shape() == Shape3D(1, 1, 2));
  auto psink = HostGradSinkOp<V>::Make(pooled, ctx);
  std::vector<float> pg(2, 1.0f), py(2), pdx(32);
  psink->set_host_grad(pg.data());
  TxnId t3;
  src->load(t3, x.data());
  psink->gradient(t3);
  ctx->sync();
  psink->store_val(t3, py.data());
  src->store_grad(t3, pdx.data());
  CHECK(py[0] == 8.5f && py[1] == 24.5f);
  for (float v : pdx) CHECK(v == 1.0f / 16);
}


// ---------------------------------------------------------------------------------------------
// ParallelSGDOptimizer over the residual block: every rank owns its copies of the two filters and of
// the batch-norm parameters, as in the reference's parallel nets; the optimizer sums the ranks'
// gradients, updates and hands the result back to every rank.  The CPU side trains ONE set of
// parameters on the unsplit convolution with the oracle's update and must stay in step.
// ---------------------------------------------------------------------------------------------
struct BlockParams {
  std::vector<float> w1, w2, sc0, sh0, sc1, sh1;
  std::vector<std::vector<float> *> all() { return {&w1, &w2, &sc0, &sh0, &sc1, &sh1}; }
};

// gradients of <dY, y> for y = x + conv2(relu(bn1(conv1(relu(bn0(x)))))) with tile-local batch-norm statistics;
// the batch-norm parameter gradients are summed over the tiles.  stats[r] receives tile r's
// (mean0, var0, mean1, var1) as the forward pass reports them.
static BlockParams block_oracle_grads(size_t K, size_t N, size_t C, size_t H, size_t W, const std::vector<float> &X,
                                      const std::vector<float> &dY, BlockParams &P,
                                      std::vector<std::vector<std::vector<float>>> *stats) {
  const size_t Ht = H / K, full = N * C * H * W;
  const float eps = 1.0e-5f;
  std::vector<std::vector<float>> m0(K, std::vector<float>(C)), i0 = m0, m1 = m0, i1 = m0;
  std::vector<float> A0(full), C1(full), A1(full);
  stats->assign(K, std::vector<std::vector<float>>(4, std::vector<float>(C)));
  for (size_t r = 0; r < K; ++r) {
    auto xt = tile_of(X, N, C, H, W, K, r);
    std::vector<float> yt(xt.size());
    orc_batchnorm2d_fwd_train(N, C, Ht, W, eps, 1, 0, xt.data(), P.sc0.data(), P.sh0.data(), yt.data(), (*stats)[r][0].data(),
                              (*stats)[r][1].data(), m0[r].data(), i0[r].data());
    put_tile(A0, yt, N, C, H, W, K, r);
  }
  std::vector<float> A0p(N * C * (H + 2) * (W + 2)), A1p(A0p.size());
  orc_halo_pad(0, 1, W, H, C, N, A0.data(), A0p.data());
  orc_conv_slab_fwd(N, C, C, H, W, 3, A0p.data(), P.w1.data(), 0.f, C1.data());
  for (size_t r = 0; r < K; ++r) {
    auto xt = tile_of(C1, N, C, H, W, K, r);
    std::vector<float> yt(xt.size());
    orc_batchnorm2d_fwd_train(N, C, Ht, W, eps, 1, 0, xt.data(), P.sc1.data(), P.sh1.data(), yt.data(), (*stats)[r][2].data(),
                              (*stats)[r][3].data(), m1[r].data(), i1[r].data());
    put_tile(A1, yt, N, C, H, W, K, r);
  }
  orc_halo_pad(0, 1, W, H, C, N, A1.data(), A1p.data());
  BlockParams G;
  G.w1.assign(P.w1.size(), 0.f); G.w2.assign(P.w2.size(), 0.f);
  G.sc0.assign(C, 0.f); G.sh0.assign(C, 0.f); G.sc1.assign(C, 0.f); G.sh1.assign(C, 0.f);
  std::vector<float> dA1p(A1p.size()), dA1(full), dC1(full), dA0p(A0p.size()), dA0(full);
  orc_conv_slab_bwd_data(N, C, C, H, W, 3, P.w2.data(), dY.data(), 0.f, dA1p.data());
  orc_conv_slab_bwd_filter(N, C, C, H, W, 3, A1p.data(), dY.data(), 0.f, G.w2.data());
  orc_halo_unpad(0, 1, W, H, C, N, dA1p.data(), dA1.data());
  for (size_t r = 0; r < K; ++r) {
    auto xt = tile_of(C1, N, C, H, W, K, r), dyt = tile_of(dA1, N, C, H, W, K, r);
    std::vector<float> dxt(xt.size()), ds(C), db(C);
    orc_batchnorm2d_bwd(N, C, Ht, W, 1, 0, xt.data(), dyt.data(), P.sc1.data(), P.sh1.data(), m1[r].data(), i1[r].data(), 0.f,
                        0.f, dxt.data(), ds.data(), db.data());
    put_tile(dC1, dxt, N, C, H, W, K, r);
    for (size_t c = 0; c < C; ++c) { G.sc1[c] += ds[c]; G.sh1[c] += db[c]; }
  }
  orc_conv_slab_bwd_data(N, C, C, H, W, 3, P.w1.data(), dC1.data(), 0.f, dA0p.data());
  orc_conv_slab_bwd_filter(N, C, C, H, W, 3, A0p.data(), dC1.data(), 0.f, G.w1.data());
  orc_halo_unpad(0, 1, W, H, C, N, dA0p.data(), dA0.data());
  for (size_t r = 0; r < K; ++r) {
    auto xt = tile_of(X, N, C, H, W, K, r), dyt = tile_of(dA0, N, C, H, W, K, r);
    std::vector<float> dxt(xt.size()), ds(C), db(C);
    orc_batchnorm2d_bwd(N, C, Ht, W, 1, 0, xt.data(), dyt.data(), P.sc0.data(), P.sh0.data(), m0[r].data(), i0[r].data(), 0.f,
                        0.f, dxt.data(), ds.data(), db.data());
    for (size_t c = 0; c < C; ++c) { G.sc0[c] += ds[c]; G.sh0[c] += db[c]; }
  }
  return G;
}

static void test_parallel_sgd(size_t K, size_t N, size_t C, size_t H, size_t W, bool nesterov, size_t num_batches) {
  std::mt19937 gen(4242 + (unsigned)K + (nesterov ? 100 : 0));
  auto ctx = MultiGPUContext::Make(K);
  typedef GPUBatchArray3D<float> V;
  typedef GPUArray4D<float> A;
  typedef GPUArray1D<float> B;
  const size_t full = N * C * H * W, steps = 3;
  BlockParams P;
  P.w1 = normal(gen, C * C * 9, std::sqrt(2.0f / (C * 9))); P.w2 = normal(gen, C * C * 9, std::sqrt(2.0f / (C * 9)));
  P.sc0 = uniform(gen, C, 0.5f, 1.5f); P.sh0 = uniform(gen, C, -0.5f, 0.5f);
  P.sc1 = uniform(gen, C, 0.5f, 1.5f); P.sh1 = uniform(gen, C, -0.5f, 0.5f);
  std::vector<float> dY = normal(gen, full, 0.05f);

  auto x_src = SrcOp<V>::Make(Shape3D(W, H, C), N, ctx->device_context(0));
  vector<shared_ptr<ParamOp<A>>> w1(K), w2(K);
  vector<shared_ptr<Var<A>>> w1v(K), w2v(K);
  for (size_t r = 0; r < K; ++r) {
    w1v[r] = w1[r] = ParamOp<A>::Make(Shape4D(3, 3, C, C), ctx->device_context(r));
    w2v[r] = w2[r] = ParamOp<A>::Make(Shape4D(3, 3, C, C), ctx->device_context(r));
  }
  vector<shared_ptr<Var<V>>> xs(K, x_src);
  auto inputs = SpatialScatter2DOp<V>::MakeParallel(xs, ctx);
  auto switch_var = std::make_shared<bool>(false);
  Conv2DShape cs;
  cs.filters = C; cs.axes = {0, 1}; cs.kernel = {3, 3}; cs.dilate = {1, 1}; cs.stride = {1, 1}; cs.pad = {1, 1};
  cs.halo_padded_input = true; cs.enable_hmma = false;
  auto bnorm0 = CudnnBatchNorm2DOp<bool, V, B>::MakeParallel(C, switch_var, inputs, ctx);
  auto relu0 = parallel_relu<V>(bnorm0.ops, ctx);
  auto exch1 = HaloExch2DOp<V>::MakeParallel(1, HaloPad2DOp<V>::MakeParallel(1, relu0, ctx), ctx);
  auto conv1 = CudnnConv2DOp<V, A, A>::MakeParallel(cs, exch1, w1v, ctx);
  auto bnorm1 = CudnnBatchNorm2DOp<bool, V, B>::MakeParallel(C, switch_var, conv1, ctx);
  auto relu1 = parallel_relu<V>(bnorm1.ops, ctx);
  auto exch2 = HaloExch2DOp<V>::MakeParallel(1, HaloPad2DOp<V>::MakeParallel(1, relu1, ctx), ctx);
  auto conv2 = CudnnConv2DOp<V, A, A>::MakeParallel(cs, exch2, w2v, ctx);
  vector<vector<shared_ptr<Var<V>>>> join_inputs{inputs, conv2};
  auto y_full = SpatialJoinedGather2DOp<V>::Make(parallel_sum<V>(join_inputs, ctx), ctx);
  auto sink = HostGradSinkOp<V>::Make(y_full, ctx->device_context(0));
  sink->set_host_grad(dY.data());

  vector<VarIdSet> params(K), grads(K), batch_stats(K), fixed_stats(K);
  for (size_t r = 0; r < K; ++r) {
    params[r].insert_all(bnorm0.params[r]); params[r].insert_all(bnorm1.params[r]);
    grads[r].insert_all(bnorm0.grads[r]); grads[r].insert_all(bnorm1.grads[r]);
    params[r].insert(w1[r]->vars().at(0)); params[r].insert(w2[r]->vars().at(0));
    grads[r].insert(w1[r]->vars().at(1)); grads[r].insert(w2[r]->vars().at(1));
    batch_stats[r].insert_all(bnorm0.batch_stats[r]); batch_stats[r].insert_all(bnorm1.batch_stats[r]);
    fixed_stats[r].insert_all(bnorm0.fixed_stats[r]); fixed_stats[r].insert_all(bnorm1.fixed_stats[r]);
  }
  {  // initial values: rank 0 holds the real ones, the others something else that reset() must replace
    TxnId init;
    std::vector<float> zeros(C, 0.f);
    for (size_t r = 0; r < K; ++r) {
      const float f = r == 0 ? 1.0f : -3.0f;
      auto scaled = [f](std::vector<float> v) { for (float &e : v) e *= f; return v; };
      w1[r]->load(init, scaled(P.w1).data()); w2[r]->load(init, scaled(P.w2).data());
      bnorm0.scales[r]->load(init, scaled(P.sc0).data()); bnorm0.shifts[r]->load(init, scaled(P.sh0).data());
      bnorm1.scales[r]->load(init, scaled(P.sc1).data()); bnorm1.shifts[r]->load(init, scaled(P.sh1).data());
      bnorm0.fixed_means[r]->load(init, zeros.data()); bnorm0.fixed_variances[r]->load(init, zeros.data());
      bnorm1.fixed_means[r]->load(init, zeros.data()); bnorm1.fixed_variances[r]->load(init, zeros.data());
    }
  }
  SGDConfig cfg;
  cfg.minibatch_size = N * num_batches;
  cfg.compute_batch_size = N;
  cfg.step_size = std::make_shared<PiecewiseStepSchedule<double>>(0.05, 1, 0.03, 2, 0.02);
  cfg.momentum = std::make_shared<ConstantSchedule<double>>(0.9);
  cfg.nesterov = nesterov;
  cfg.l2_reg = 1.0e-3;
  cfg.batch_norm_rate = 0.25;
  ParallelSGDOptimizer<float> opt(cfg, sink, params, grads, batch_stats, fixed_stats);
  opt.reset(ctx);
  CHECK(opt.param_dim() == 2 * C * C * 9 + 4 * C && opt.stat_dim() == 4 * C);

  std::vector<std::vector<float>> batches;
  size_t next_batch = 0;
  function<void(TxnId, size_t, shared_ptr<Op>)> compute = [&](TxnId txn, size_t batch_size, shared_ptr<Op> loss) {
    CHECK(batch_size == N);
    for (size_t r = 0; r < K; ++r) {
      loss->persist(txn, params[r]);
      loss->persist(txn, fixed_stats[r]);
    }
    x_src->load(txn, batches.at(next_batch++).data());
    loss->gradient(txn);
  };

  BlockParams M;  // momentum, per array
  for (auto *v : {&M.w1, &M.w2}) v->assign(C * C * 9, 0.f);
  for (auto *v : {&M.sc0, &M.sh0, &M.sc1, &M.sh1}) v->assign(C, 0.f);
  BlockParams Lag = P;
  const BlockParams P0 = P;
  std::vector<std::vector<std::vector<float>>> running(K, std::vector<std::vector<float>>(4, std::vector<float>(C, 0.f)));
  for (size_t t = 0; t < steps; ++t) {
    batches.clear();
    next_batch = 0;
    for (size_t b = 0; b < num_batches; ++b) batches.push_back(uniform(gen, full, -1, 1));
    opt.step(compute, ctx);
    CHECK(next_batch == num_batches && opt.iter_count() == t + 1);

    // CPU: gradients summed over the compute batches, statistics averaged online over them
    BlockParams G;
    std::vector<std::vector<std::vector<float>>> avg;
    for (size_t b = 0; b < num_batches; ++b) {
      std::vector<std::vector<std::vector<float>>> st;
      BlockParams Gb = block_oracle_grads(K, N, C, H, W, batches[b], dY, P, &st);
      if (b == 0) {
        G = Gb;
        avg = st;
      } else {
        auto ga = G.all(), gb = Gb.all();
        for (size_t i = 0; i < ga.size(); ++i)
          for (size_t j = 0; j < ga[i]->size(); ++j) (*ga[i])[j] += (*gb[i])[j];
        const float a = 1.0f / (float)(b + 1);
        for (size_t r = 0; r < K; ++r)
          for (int q = 0; q < 4; ++q)
            for (size_t c = 0; c < C; ++c) avg[r][q][c] += a * (st[r][q][c] - avg[r][q][c]);
      }
    }
    const double steps_at[] = {0.05, 0.03, 0.02, 0.02};
    auto pa = P.all(), ga = G.all(), ma = M.all(), la = Lag.all();
    for (size_t i = 0; i < pa.size(); ++i) {
      std::vector<float> sg(pa[i]->size());
      const float *gl[1] = {ga[i]->data()};
      orc_sgd_step(pa[i]->size(), 1, gl, 1.0e-3f, 0.9f, (float)steps_at[t], (float)steps_at[t + 1], nesterov ? 1 : 0,
                   pa[i]->data(), ma[i]->data(), la[i]->data(), sg.data());
    }
    for (size_t r = 0; r < K; ++r)
      for (int q = 0; q < 4; ++q) {
        std::vector<float> stat(C);
        orc_stat_step(C, 0.25f, avg[r][q].data(), running[r][q].data(), stat.data());
      }

    // every rank now holds the updated parameters; the fixed statistics hold the running ones
    TxnId peek;
    for (size_t r = 0; r < K; ++r) {
      sink->persist(peek, params[r]);
      sink->persist(peek, fixed_stats[r]);
    }
    ctx->sync();
    double e_w = 0, e_bn = 0, e_stat = 0;
    for (size_t r = 0; r < K; ++r) {
      std::vector<float> g1(P.w1.size()), g2(P.w2.size()), a(C), b(C), c(C), d(C);
      w1[r]->store(peek, g1.data()); w2[r]->store(peek, g2.data());
      bnorm0.scales[r]->store(peek, a.data()); bnorm0.shifts[r]->store(peek, b.data());
      bnorm1.scales[r]->store(peek, c.data()); bnorm1.shifts[r]->store(peek, d.data());
      e_w = std::fmax(e_w, std::fmax(rel_err(g1, P.w1), rel_err(g2, P.w2)));
      e_bn = std::fmax(e_bn, std::fmax(std::fmax(rel_err(a, P.sc0), rel_err(b, P.sh0)), std::fmax(rel_err(c, P.sc1), rel_err(d, P.sh1))));
      std::vector<float> s(C);
      bnorm0.fixed_means[r]->store(peek, s.data()); e_stat = std::fmax(e_stat, rel_err(s, running[r][0]));
      bnorm0.fixed_variances[r]->store(peek, s.data()); e_stat = std::fmax(e_stat, rel_err(s, running[r][1]));
      bnorm1.fixed_means[r]->store(peek, s.data()); e_stat = std::fmax(e_stat, rel_err(s, running[r][2]));
      bnorm1.fixed_variances[r]->store(peek, s.data()); e_stat = std::fmax(e_stat, rel_err(s, running[r][3]));
    }
    std::printf("parallel sgd K=%zu N=%zu C=%zu %zux%zu nesterov=%d batches=%zu step %zu: rel-err filters %.2e bn %.2e stats %.2e\n",
                K, N, C, H, W, (int)nesterov, num_batches, t, e_w, e_bn, e_stat);
    CHECK(e_w <= 2e-5 && e_bn <= 2e-5 && e_stat <= 2e-5);
  }
  CHECK(rel_err(P.w1, P0.w1) > 1e-3 && rel_err(P.sc1, P0.sc1) > 1e-4);  // the steps did move the parameters
  // the lagged parameters (before the look-ahead) come back on request
  opt.reload_lagged_param(ctx);
  {
    TxnId peek;
    sink->persist(peek, params[K - 1]);
    std::vector<float> g1(P.w1.size());
    w1[K - 1]->store(peek, g1.data());
    CHECK(rel_err(g1, Lag.w1) <= 2e-5);
    if (nesterov) CHECK(rel_err(g1, P.w1) > 1e-4);
  }
  opt.reload_param(ctx);
}

static void test_schedules() {
  ConstantSchedule<double> c(0.1);
  CHECK(c.at(0) == 0.1 && c.at(1000000) == 0.1);
  PiecewiseStepSchedule<double> s(1.0, 10, 0.5, 20, 0.25);
  CHECK(s.at(0) == 1.0 && s.at(9) == 1.0 && s.at(10) == 0.5 && s.at(19) == 0.5 && s.at(20) == 0.25 && s.at(99) == 0.25);
  PiecewiseStepSchedule<double> s0(2.0);
  CHECK(s0.at(5) == 2.0);
  PiecewiseLinearSchedule<double> l(0.0, 10, 1.0);
  CHECK(l.at(0) == 0.0 && std::fabs(l.at(5) - 0.5) < 1e-12 && l.at(10) == 1.0 && l.at(50) == 1.0);
  PiecewiseLinearSchedule<double> l2(1.0, {{10, 2.0}, {30, 0.0}});
  CHECK(std::fabs(l2.at(5) - 1.5) < 1e-12 && std::fabs(l2.at(20) - 1.0) < 1e-12 && l2.at(30) == 0.0);
  VarIdSet set;
  VarId a, b;
  set.insert(a);
  bool threw = false;
  try { set.mask(a); } catch (const HazardError &) { threw = true; }
  CHECK(threw);
  set.lock();
  CHECK(set.mask(a) && !set.mask(a) && !set.mask(b));
  set.unlock();
  set.lock();
  CHECK(set.mask(a));
  set.unlock();
}


// The whole spatially-parallel ResNet-18 variant in evaluation mode (fixed batch-norm statistics, so that
// nothing depends on how the rows are dealt to ranks): the logits for 2 and 4 row-tiles must equal those of
// the unsplit net with the same parameters.  This exercises every halo exchange, the strided convolutions and
// the pooling over tile borders, and the gather, end to end.
// Op::init alone (no optimizer reset, no hand-loaded values) must leave every rank's copy of a
// parallel_conv2d filter equal to rank 0's: the node convolves all tiles with rank 0's filter.
static void test_parallel_conv2d_init_gives_equal_copies() {
  const size_t K = 4, N = 2, C = 8, Co = 16, H = 8, W = 12, Ht = H / K;
  typedef GPUBatchArray3D<float> V3;
  auto ctx = MultiGPUContext::Make(K);
  std::vector<std::shared_ptr<Var<V3>>> xs;
  std::vector<std::shared_ptr<SrcOp<V3>>> srcs;
  for (size_t r = 0; r < K; ++r) {
    auto src = SrcOp<V3>::Make(Shape3D(W, Ht, C), N, ctx->device_context(r));
    srcs.push_back(src);
    xs.push_back(src);
  }
  auto pad = HaloPad2DOp<V3>::MakeParallel(1, xs, ctx);
  auto exch = HaloExch2DOp<V3>::MakeParallel(1, pad, ctx);
  Conv2DShape cs;
  cs.filters = Co; cs.axes = {0, 1}; cs.kernel = {3, 3}; cs.stride = {1, 1}; cs.dilate = {1, 1}; cs.pad = {1, 1};
  cs.halo_padded_input = true; cs.enable_hmma = false;
  auto conv = parallel_conv2d<V3>(cs, exch, kaiming_init_gen<GPUArray4D<float>>(C * 9, Co), false, ctx);
  std::mt19937_64 rng(99);
  TxnId init_txn;
  for (size_t r = 0; r < K; ++r) conv.ops[r]->init(init_txn, &rng);
  ctx->sync();
  // read every rank's filter back through the flat-vector plumbing
  const size_t wdim = Co * C * 9;
  std::vector<std::vector<float>> w(K, std::vector<float>(wdim));
  GPUContext *root = ctx->device_context(0).get();
  for (size_t r = 0; r < K; ++r) {
    GPUMemory<float> flat = GPUMemory<float>::Zeros(wdim, root);
    CHECK(conv.ops[r]->store_val(init_txn, conv.params[r], 0, &flat) == wdim);
    GPUConn conn = root->conn();
    flat.store_sync(w[r].data(), 0, wdim, conn);
  }
  double norm = 0;
  for (float v : w[0]) norm += (double)v * v;
  CHECK(norm > 0.1);
  for (size_t r = 1; r < K; ++r) CHECK(w[r] == w[0]);
}

static void test_resnet18_tiling_invariance() {
  const size_t N = 2, H = 256, W = 32, classes = 10;
  ConvNetConfig cfg;
  cfg.input_w = W; cfg.input_h = H; cfg.batch_size = N; cfg.minibatch_size = N;
  std::mt19937 gen(77);
  std::vector<float> X = uniform(gen, N * 3 * H * W, 0.f, 1.f);
  std::vector<uint32_t> labels = {3, 7};
  std::vector<float> ref_logits, flat_host;
  size_t param_dim = 0;
  for (size_t K : {1, 2, 4}) {
    auto ctx = MultiGPUContext::Make(K);
    auto net = ResNet<float>::MakeParallelResNet18(cfg, ctx, classes);
    std::mt19937_64 rng(1234);
    {
      TxnId init_txn;
      net.sum_loss->init(init_txn, &rng);
    }
    TxnId txn;
    for (size_t r = 0; r < K; ++r) {
      net.sum_loss->persist(txn, net.dev_params[r]);
      net.sum_loss->persist(txn, net.dev_fixed_stats[r]);
    }
    GPUContext *root = ctx->device_context(0).get();
    if (K == 1) {
      param_dim = net.sum_loss->store_val(txn, net.dev_params[0], 0, nullptr);
      GPUMemory<float> flat = GPUMemory<float>::Zeros(param_dim, root);
      CHECK(net.sum_loss->store_val(txn, net.dev_params[0], 0, &flat) == param_dim);
      flat_host.resize(param_dim);
      GPUConn conn = root->conn();
      flat.store_sync(flat_host.data(), 0, param_dim, conn);
    } else {
      // every rank takes the unsplit net's parameters: a rank's variables come in the same order whatever K is
      GPUMemory<float> flat(param_dim, root);
      GPUConn conn = root->conn();
      flat.load_sync(flat_host.data(), 0, param_dim, conn);
      for (size_t r = 0; r < K; ++r) CHECK(net.sum_loss->load_val(txn, net.dev_params[r], 0, &flat) == param_dim);
    }
    *net.batch_norm_use_fixed = true;
    net.input->load(txn, X.data());
    net.label->load(txn, labels.data());
    net.sum_loss->eval(txn);
    ctx->sync();
    std::vector<float> prob(N * classes), loss(N);
    net.loss->store_prob(txn, prob.data());
    net.loss->store_loss(txn, loss.data());
    if (K == 1) {
      ref_logits = prob;
      bool spread = false;  // the net must not have collapsed to a constant output
      for (size_t i = 1; i < classes; ++i) spread = spread || std::fabs(prob[i] - prob[0]) > 1e-4f;
      CHECK(spread);
      CHECK(param_dim > 11000000);
    } else {
      const double e = rel_err(prob, ref_logits);
      std::printf("resnet18 eval, %zu row-tiles vs unsplit: rel-err of the class probabilities %.2e (loss %.5f %.5f)\n", K, e,
                  loss[0], loss[1]);
      CHECK(e <= 2e-5);
    }
  }
}

int main(int argc, char **argv) {
  const std::string mode = argc > 1 ? argv[1] : "cpu";
  test_shapes();
  test_comm_protocol();
  test_schedules();
  if (mode == "gpu") {
    test_txn_hazards();
    test_microbench_sequence();
    test_spatial_conv_graph(4, 2, 8, 16, 8, 12);
    test_spatial_conv_graph(2, 3, 5, 7, 6, 9);
    test_spatial_conv_graph(1, 1, 16, 16, 5, 5);
    test_spatial_conv_graph(4, 4, 64, 64, 56, 56);
    test_spatial_conv_graph(4, 4, 64, 64, 56, 56, true);
    test_spatial_conv_graph(2, 3, 5, 7, 40, 30, true);
    test_spatial_conv_graph(4, 2, 8, 16, 8, 12, true);
    test_spatial_conv_graph(4, 4, 64, 64, 56, 56, false, true);
    test_spatial_conv_graph(2, 3, 5, 7, 40, 30, false, true);
    test_spatial_conv_graph(4, 2, 8, 16, 8, 12, false, true);
    test_spatial_conv_graph(1, 1, 16, 16, 5, 5, false, true);
    test_spatial_general_conv_graph(4, 2, 3, 16, 32, 24, 7, 2, 1);   // the stem
    test_spatial_general_conv_graph(2, 2, 8, 12, 16, 20, 3, 2, 1);   // stride-2 3x3
    test_spatial_general_conv_graph(2, 1, 8, 8, 12, 14, 3, 1, 3);    // dilation 3 over halo 3
    test_spatial_general_conv_graph(2, 2, 6, 10, 8, 9, 1, 1, 1);     // 1x1 over packed tiles (halo 0)
    test_spatial_general_conv_graph(4, 2, 3, 16, 32, 24, 7, 2, 1, true);   // the same four over tiles without halo
    test_spatial_general_conv_graph(2, 2, 8, 12, 16, 20, 3, 2, 1, true);
    test_spatial_general_conv_graph(2, 1, 8, 8, 12, 14, 3, 1, 3, true);
    test_spatial_general_conv_graph(4, 3, 3, 16, 32, 24, 7, 1, 1, true);   // the stem as the spatial net builds it (stride 1)
    test_spatial_general_conv_graph(4, 4, 24, 24, 16, 16, 3, 1, 1, true);  // 4x16 tiles: stride-1 3x3 through the general kernels
    test_spatial_general_conv_graph(4, 4, 16, 24, 8, 8, 3, 2, 1, true);    // 2x8 tiles at stride 2
    test_spatial_conv_bias_graph(4, 3, 3, 16, 32, 24, 7, false, false);         // the stem's shape, a bias per rank
    test_spatial_conv_bias_graph(4, 3, 3, 16, 32, 24, 7, true, false);          // one bias variable for all ranks
    test_spatial_conv_bias_graph(2, 2, 8, 12, 40, 30, 3, false, true);          // 3x3, filter and bias per rank
    test_spatial_conv_bias_graph(2, 2, 8, 12, 40, 30, 3, false, true, true);    // unexchanged rows + a filter per rank
    test_spatial_conv_bias_graph(4, 2, 8, 16, 8, 12, 3, true, true, true);      // the same on small tiles (general kernels)
    test_spatial_conv_bias_graph(4, 4, 64, 64, 56, 56, 3, true, false, true);   // one launch reads across tiles, then the bias
    test_spatial_conv_bias_graph(4, 2, 8, 16, 32, 24, 3, false, false, false, true);  // tiles without halo
    test_spatial_residual_block(4, 2, 8, 16, 12);
    test_spatial_residual_block(2, 4, 64, 28, 28);
    test_spatial_residual_block(4, 2, 8, 16, 12, true);
    test_spatial_residual_block(2, 4, 64, 28, 28, true);
    test_spatial_residual_block(4, 2, 8, 16, 12, true, true);
    test_spatial_residual_block(2, 4, 64, 28, 28, false, true);
    test_spatial_residual_block(4, 2, 8, 16, 12, true, false, true);   // small tiles: the general kernel, then the sum
    test_spatial_residual_block(2, 4, 64, 28, 28, true, false, true);  // the 3x3 kernel adds the block input itself
    test_spatial_pool_graph(kMaxPool, 4, 2, 8, 16, 12);
    test_spatial_pool_graph(kAveragePool, 2, 3, 5, 8, 10);
    test_spatial_pool_graph(kMaxPool, 4, 8, 64, 112, 112);
    test_spatial_pool_graph(kMaxPool, 4, 2, 8, 16, 12, true);
    test_spatial_pool_graph(kAveragePool, 2, 3, 5, 8, 10, true);
    test_spatial_pool_graph(kMaxPool, 4, 8, 64, 112, 112, true);
    test_softmax_loss_op();
    test_parallel_conv2d_init_gives_equal_copies();
    test_resnet18_tiling_invariance();
    test_parallel_sgd(4, 2, 8, 16, 12, false, 1);
    test_parallel_sgd(2, 2, 8, 8, 10, true, 1);
    test_parallel_sgd(2, 2, 4, 8, 6, true, 2);
    test_parallel_sgd(1, 3, 4, 6, 6, false, 2);
  }
  std::printf("%s: %d failure(s)\n", mode.c_str(), failures);
  return failures ? 1 : 0;
}
