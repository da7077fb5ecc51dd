// Trains the spatially-parallel ResNet-18 variant on synthetic data: the role of the reference's
// tools/train_imagenet.cc:120-330 (config, optimizer, per-minibatch callback, step loop) without
// its data pipeline.  One fixed batch is fed every step, so the loss must fall; the last line
// printed is one JSON object with the step time.
//
//   train_resnet18 [--ranks K] [--batch N] [--size S] [--steps T] [--warmup W] [--classes C]
//                  [--lr a] [--nesterov 0|1] [--graph 0|1]
// --graph 1: after the warm-up steps one step (forward, backward, optimizer) is recorded as a HIP graph and
// the timed steps replay it; the step size and momentum are kernel arguments, fixed when the step is recorded,
// and the optimizer's iteration counter does not advance during replays: this is right only because both
// schedules are constant here (a varying schedule needs eager steps, or a new recording per value).
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "arraydiff/optimize.hh"
#include "arraydiff/zoo.hh"

using namespace arraydiff;

int main(int argc, char **argv) {
  size_t ranks = 4, batch = 32, size = 128, steps = 10, warmup = 2, classes = 1000;
  double lr = 0.05;
  int nesterov = 1, use_graph = 0;
  for (int i = 1; i + 1 < argc; i += 2) {
    const std::string k = argv[i];
    const char *v = argv[i + 1];
    if (k == "--ranks") ranks = std::strtoul(v, nullptr, 10);
    else if (k == "--batch") batch = std::strtoul(v, nullptr, 10);
    else if (k == "--size") size = std::strtoul(v, nullptr, 10);
    else if (k == "--steps") steps = std::strtoul(v, nullptr, 10);
    else if (k == "--warmup") warmup = std::strtoul(v, nullptr, 10);
    else if (k == "--classes") classes = std::strtoul(v, nullptr, 10);
    else if (k == "--lr") lr = std::strtod(v, nullptr);
    else if (k == "--nesterov") nesterov = std::atoi(v);
    else if (k == "--graph") use_graph = std::atoi(v);
    else {
      std::fprintf(stderr, "unknown option %s\n", k.c_str());
      return 2;
    }
  }
  try {
    auto parallel_ctx = MultiGPUContext::Make(ranks);
    ConvNetConfig net_cfg;
    net_cfg.input_w = size;
    net_cfg.input_h = size;
    net_cfg.batch_size = batch;
    net_cfg.minibatch_size = batch;
    auto net = ResNet<float>::MakeParallelResNet18(net_cfg, parallel_ctx, classes);

    std::mt19937_64 rng(20171231);
    {
      TxnId init_txn;
      net.sum_loss->init(init_txn, &rng);
    }
    SGDConfig sgd_cfg;
    sgd_cfg.minibatch_size = batch;
    sgd_cfg.compute_batch_size = batch;
    sgd_cfg.step_size = std::make_shared<ConstantSchedule<double>>(lr);
    sgd_cfg.momentum = std::make_shared<ConstantSchedule<double>>(0.9);
    sgd_cfg.nesterov = nesterov != 0;
    sgd_cfg.l2_reg = 1.0e-4;
    sgd_cfg.batch_norm_rate = 0.003;
    ParallelSGDOptimizer<float> sgd(sgd_cfg, net.sum_loss, net.dev_params, net.dev_grads, net.dev_batch_stats,
                                    net.dev_fixed_stats);
    sgd.reset(parallel_ctx);

    const size_t image_size = size * size * 3;
    std::vector<float> batch_input(image_size * batch);
    std::vector<uint32_t> batch_label(batch);
    std::vector<float> batch_loss(batch);
    std::uniform_real_distribution<float> pixel(0.0f, 1.0f);
    for (float &v : batch_input) v = pixel(rng);
    for (size_t i = 0; i < batch; ++i) batch_label[i] = (uint32_t)(rng() % classes);

    bool read_loss = true, recording = false;
    double last_loss = 0;
    TxnId recorded_txn;
    function<void(TxnId, size_t, shared_ptr<Op>)> batch_fn = [&](TxnId batch_txn, size_t batch_size, shared_ptr<Op> loss) {
      (void)batch_size;
      *net.batch_norm_use_fixed = false;
      for (size_t rank = 0; rank < ranks; ++rank) {
        loss->persist(batch_txn, net.dev_params.at(rank));
        loss->persist(batch_txn, net.dev_fixed_stats.at(rank));
      }
      if (recording) {
        // the batch is already in the sources' buffers (a host-to-device copy cannot be recorded): carry it over
        VarIdSet feed;
        feed.insert(net.input->vars().at(0));
        feed.insert(net.label->vars().at(0));
        loss->persist(batch_txn, feed);
        recorded_txn = batch_txn;
      } else {
        net.input->load(batch_txn, batch_input.data());
        net.label->load(batch_txn, batch_label.data());
      }
      loss->gradient(batch_txn);
      if (read_loss) {
        parallel_ctx->sync();
        net.loss->store_loss(batch_txn, batch_loss.data());
        double s = 0;
        for (float v : batch_loss) s += v;
        last_loss = s / (double)batch;
      }
    };

    std::vector<double> losses;
    for (size_t t = 0; t < warmup; ++t) {
      sgd.step(batch_fn, parallel_ctx);
      losses.push_back(last_loss);
      std::printf("warmup %zu: loss %.5f\n", t, last_loss);
      std::fflush(stdout);
    }
    // timed steps: the loss is read back only after the last one
    parallel_ctx->sync();
    read_loss = false;
    StreamCapture capture(dynamic_cast<MultiGPUContext *>(parallel_ctx.get())->stream());
    if (use_graph && warmup < 1) {
      // the first step allocates every buffer and sizes the scratch: that cannot happen inside a stream capture
      std::fprintf(stderr, "train_resnet18: --graph 1 needs at least one warm-up step\n");
      return 2;
    }
    if (use_graph) {
      recording = true;
      capture.begin();
      sgd.step(batch_fn, parallel_ctx);  // recorded, not run
      capture.end();
      recording = false;
      std::printf("recorded one step: %zu graph nodes\n", capture.num_nodes());
    }
    const auto start = std::chrono::steady_clock::now();
    for (size_t t = 0; t < steps; ++t) {
      if (use_graph) {
        // a data loader would copy the next batch into the sources' buffers here; the synthetic batch is fixed
        capture.replay();
      } else {
        if (t + 1 == steps) read_loss = true;
        sgd.step(batch_fn, parallel_ctx);
      }
    }
    parallel_ctx->sync();
    const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
    if (use_graph) {  // the losses of the last replay's forward pass
      net.loss->store_loss(recorded_txn, batch_loss.data());
      double s = 0;
      for (float v : batch_loss) s += v;
      last_loss = s / (double)batch;
    }
    losses.push_back(last_loss);
    const bool finite = std::isfinite(last_loss);
    std::printf("{\"workload\": \"spatially-parallel ResNet-18 variant, %zux%zu, batch %zu, %zu row-tiles, fp32, synthetic\", "
                "\"param_dim\": %zu, \"steps\": %zu, \"ms_per_step\": %.4f, \"img_per_s\": %.2f, \"loss_first\": %.5f, "
                "\"loss_last\": %.5f, \"graph\": %s, \"finite\": %s}\n",
                size, size, batch, ranks, sgd.param_dim(), steps, sec / (double)steps * 1e3, (double)(batch * steps) / sec,
                losses.front(), last_loss, use_graph ? "true" : "false", finite ? "true" : "false");
    return finite ? 0 : 1;
  } catch (const std::exception &e) {
    std::fprintf(stderr, "train_resnet18: %s\n", e.what());
    return 1;
  }
}
