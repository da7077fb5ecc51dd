// The reference's two spatial microbenchmarks, run through this library's Spatial2DComm and C ABI with the
// reference's own loops and figures of merit:
//
//   --which spatial       tools/microbench_spatial.cc:16-106: halo exchange on raw buffers, fp32 N=32, C=64,
//                         W=256, H=256/ranks, halo 1; per rank group_start(); halo_exchange(...); then per rank
//                         group_end(conn); then per rank sync; prints the average wall-clock time per trial and
//                         halo*W*C*N*4 bytes / time (:98-103)
//   --which spatial_conv  tools/microbench_spatial_conv.cc:18-480: N=32, C=64, a 512x512 image in `ranks` row
//                         tiles, 3x3 convolution with dilation 3 over halo 3: the halo exchange loop (:227-269),
//                         the halo reduce loop (:271-313), "spatial conv (fwd)" = exchange sequence, sync, one
//                         forward convolution per rank, sync (:316-392), "spatial conv (bwd)" = one
//                         backward-filter and one backward-data convolution per rank, sync, reduce sequence, sync
//                         (:394-477); average wall-clock milliseconds per trial, as printed there
//
//   --which conv          tools/microbench_conv.cc:16-241: one device, N=32, 64 -> 64 channels, a 3x3 convolution
//                         forward over a 64(+2) x 128(+2) halo-padded source, 1000 trials of (launch, stream
//                         synchronise), average wall clock and "est flops" 2*N*Co*Ci*H*W*9 (:53, :180-240).  The
//                         reference writes the result into the interior of a halo-padded destination through a
//                         strided descriptor (:41-44); here it lands in a packed tensor.
//
// The reference's first two loops pass src_width = W + 2*halo as base_width (:246, :291), which indexes past
// buf_size (:43); every loop here passes the interior width.  cuDNN's three convolution calls become the C ABI's
// adh_conv2d_slab_{fwd,bwd_filter,bwd_data}_tiles with one tile per call.
//
// Beside each per-rank sequence the same work is timed as this library is meant to be driven on one GPU: one
// launch for all ranks' tiles (Spatial2DComm::group_end_all, the *_tiles entry points over `ranks` tiles) and no
// synchronisation between exchange and convolution (one in-order stream is the barrier).  Each line printed is
// one JSON object; the last line is the summary bench.py reads.
//
//   microbench_spatial --which spatial|spatial_conv|conv [--ranks K] [--trials T] [--batch N]
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "adh_capi.h"
#include "arraydiff/array_gpu.hh"
#include "arraydiff/context.hh"
#include "arraydiff/spatial.hh"

using namespace arraydiff;

namespace {

struct Stat {
  double avg_ms = 0.0, std_ms = 0.0;
};

// The reference's timing loop (microbench_spatial_conv.cc:324-389): every rank is synchronised before the clock
// starts, trial 0 is not counted, mean and variance are updated online.
Stat time_trials(MultiGPUContext *ctx, int trials, const std::function<void()> &body) {
  Stat s;
  double sum_sq = 0.0;
  for (int t = 0; t < trials + 1; ++t) {
    for (size_t r = 0; r < ctx->num_ranks(); ++r) ctx->device_context(r)->sync();
    const auto start = std::chrono::steady_clock::now();
    body();
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - start).count();
    if (t >= 1) {
      const double prev = s.avg_ms;
      s.avg_ms += (ms - s.avg_ms) / (double)t;
      sum_sq += (ms - s.avg_ms) * (ms - prev);
    }
  }
  s.std_ms = trials > 1 ? std::sqrt(sum_sq / (double)(trials - 1)) : 0.0;
  return s;
}

void check(int code, const char *what) { adh_check(code, what); }

struct Halo {
  Spatial2DComm *comms;
  MultiGPUContext *ctx;
  uint32_t K, p, W, H, C, N;
  // per rank group_start + record, then per rank group_end on that rank's connection
  // (microbench_spatial.cc:74-88); sync_after: the per-rank sync that closes the reference's sequence
  void per_rank(bool reduce, float *const *bufs, bool sync_after) const {
    for (uint32_t r = 0; r < K; ++r) {
      comms[r].group_start();
      if (reduce)
        comms[r].halo_reduce(bufs[r], p, W, H, C, N, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
      else
        comms[r].halo_exchange(bufs[r], p, W, H, C, N, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
    }
    for (uint32_t r = 0; r < K; ++r) {
      GPUConn conn = ctx->device_context(r)->conn();
      check(comms[r].group_end(conn), "group_end");
    }
    if (sync_after)
      for (uint32_t r = 0; r < K; ++r) ctx->device_context(r)->sync();
  }
  // the same records, ended by ONE launch for all ranks
  void all_ranks(bool reduce, float *const *bufs) const {
    for (uint32_t r = 0; r < K; ++r) {
      comms[r].group_start();
      if (reduce)
        comms[r].halo_reduce(bufs[r], p, W, H, C, N, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
      else
        comms[r].halo_exchange(bufs[r], p, W, H, C, N, SPATIAL2D_TENSOR_NCHW, SPATIAL2D_DATA_FLOAT);
    }
    GPUConn conn = ctx->device_context(0)->conn();
    check(Spatial2DComm::group_end_all(comms, conn), "group_end_all");
  }
};

void print_entry(const char *which, const char *name, const Stat &seq, const Stat &one, double ref_bytes, double flops) {
  std::printf("{\"which\": \"%s\", \"name\": \"%s\", \"per_rank_sequence_ms\": %.5f, \"per_rank_sequence_std_ms\": %.5f, "
              "\"one_launch_ms\": %.5f, \"one_launch_std_ms\": %.5f",
              which, name, seq.avg_ms, seq.std_ms, one.avg_ms, one.std_ms);
  if (ref_bytes > 0)
    std::printf(", \"reference_figure_GBs_per_rank_sequence\": %.3f, \"reference_figure_GBs_one_launch\": %.3f",
                ref_bytes * 1e-9 / (seq.avg_ms * 1e-3), ref_bytes * 1e-9 / (one.avg_ms * 1e-3));
  if (flops > 0)
    std::printf(", \"tflops_per_rank_sequence\": %.2f, \"tflops_one_launch\": %.2f", flops * 1e-12 / (seq.avg_ms * 1e-3),
                flops * 1e-12 / (one.avg_ms * 1e-3));
  std::printf("}\n");
  std::fflush(stdout);
}

void fill_uniform(std::vector<float> &v, uint32_t seed) {
  uint64_t s = 0x9E3779B97F4A7C15ull * (seed + 1);
  for (auto &x : v) {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    x = (float)((double)(s >> 40) / (double)(1ull << 24)) * 2.0f - 1.0f;
  }
}

}  // namespace

int main(int argc, char **argv) {
  std::string which = "spatial";
  size_t ranks = 4, batch = 32;
  int trials = -1;
  for (int i = 1; i + 1 < argc; i += 2) {
    const std::string k = argv[i];
    const char *v = argv[i + 1];
    if (k == "--which") which = v;
    else if (k == "--ranks") ranks = std::strtoul(v, nullptr, 10);
    else if (k == "--trials") trials = std::atoi(v);
    else if (k == "--batch") batch = std::strtoul(v, nullptr, 10);
    else {
      std::fprintf(stderr, "unknown option %s\n", k.c_str());
      return 2;
    }
  }
  if ((which != "spatial" && which != "spatial_conv" && which != "conv") || ranks == 0 || ranks > ADH_MAX_TILES || batch == 0 ||
      argc % 2 == 0) {
    std::fprintf(stderr, "usage: microbench_spatial --which spatial|spatial_conv|conv [--ranks K] [--trials T] [--batch N]\n");
    return 2;
  }
  try {
    const uint32_t K = which == "conv" ? 1u : (uint32_t)ranks, N = (uint32_t)batch, C = 64;  // microbench_conv.cc:20: one device
    auto ctx = MultiGPUContext::Make(K);
    std::vector<Spatial2DComm> comms(K);
    check(Spatial2DComm::InitAll(comms.data(), 1, K), "InitAll");

    if (which == "spatial") {
      // microbench_spatial.cc:23-28
      const uint32_t p = 1, W = 256, H = 256 / K;
      if (trials < 0) trials = 1000;  // :68
      const size_t buf = (size_t)(W + 2 * p) * (H + 2 * p) * C * N;
      std::vector<float> host(buf);
      std::vector<GPUMemory<float>> x;
      std::vector<float *> xp;
      for (uint32_t r = 0; r < K; ++r) {
        x.emplace_back(buf, ctx->device_context(r).get());
        fill_uniform(host, r);
        GPUConn conn = ctx->device_context(r)->conn();
        x[r].load_sync(host.data(), 0, buf, conn);
        xp.push_back(x[r].dptr());
      }
      const Halo halo{comms.data(), ctx.get(), K, p, W, H, C, N};
      const Stat seq = time_trials(ctx.get(), trials, [&] { halo.per_rank(false, xp.data(), true); });
      const Stat one = time_trials(ctx.get(), trials, [&] {
        halo.all_ranks(false, xp.data());
        ctx->sync();
      });
      print_entry("spatial", "halo exchange", seq, one, (double)p * W * C * N * 4.0, 0.0);
      std::printf("{\"which\": \"spatial\", \"ranks\": %u, \"trials\": %d, \"halo\": %u, \"n\": %u, \"c\": %u, \"h\": %u, \"w\": %u, "
                  "\"exchange_per_rank_sequence_ms\": %.5f, \"exchange_one_launch_ms\": %.5f}\n",
                  K, trials, p, N, C, H, W, seq.avg_ms, one.avg_ms);
      return 0;
    }

    if (which == "conv") {
      // microbench_conv.cc:22-53
      const uint32_t W = 128, H = 128 / 2;
      if (trials < 0) trials = 1000;  // :180
      const size_t src = (size_t)(W + 2) * (H + 2) * C * N, dst = (size_t)W * H * C * N, wsz = (size_t)9 * C * C;
      GPUContext *dc = ctx->device_context(0).get();
      GPUConn conn = dc->conn();
      GPUMemory<float> x(src, dc), y(dst, dc), w(wsz, dc);
      {
        std::vector<float> host(src);
        fill_uniform(host, 1);
        x.load_sync(host.data(), 0, src, conn);
        host.resize(wsz);
        fill_uniform(host, 7);
        const float scale = std::sqrt(2.0f / (C * 9));
        for (auto &v : host) v *= scale;
        w.load_sync(host.data(), 0, wsz, conn);
      }
      ctx->sync();
      const double flops = 2.0 * N * C * C * (double)H * W * 9.0;  // :53
      const Stat one = time_trials(ctx.get(), trials, [&] {
        check(adh_conv3x3_slab_fwd(ADH_F32, N, C, C, H, W, x.dptr(), w.dptr(), y.dptr(), 0.0f, nullptr, 0, conn.stream()), "conv fwd");
        dc->sync();  // :227-230
      });
      std::printf("{\"which\": \"conv\", \"name\": \"conv forward over a halo-padded source\", \"trials\": %d, \"n\": %u, \"c\": %u, "
                  "\"h\": %u, \"w\": %u, \"avg_wallclock_ms\": %.5f, \"std_ms\": %.5f, \"est_gflop\": %.3f, \"tflops\": %.2f}\n",
                  trials, N, C, H, W, one.avg_ms, one.std_ms, flops * 1e-9, flops * 1e-12 / (one.avg_ms * 1e-3));
      return 0;
    }

    // microbench_spatial_conv.cc:25-48
    const uint32_t ksz = 3, dil = 3, p = 3, W = 512, H = 512 / K;
    const uint32_t HP = H + 2 * p, WP = W + 2 * p;
    const int halo_trials = trials < 0 ? 10000 : trials * 10;  // :228, :272
    const int conv_trials = trials < 0 ? 1000 : trials;        // :318, :395
    const size_t buf = (size_t)WP * HP * C * N, out = (size_t)W * H * C * N, wsz = (size_t)ksz * ksz * C * C;
    std::vector<GPUMemory<float>> x, y, dx, dy;
    std::vector<float *> xp, dxp;
    const void *x_tiles[ADH_MAX_TILES], *dy_tiles[ADH_MAX_TILES];
    void *y_tiles[ADH_MAX_TILES], *dx_tiles[ADH_MAX_TILES];
    {
      std::vector<float> host(buf);
      for (uint32_t r = 0; r < K; ++r) {
        GPUContext *dc = ctx->device_context(r).get();
        GPUConn conn = dc->conn();
        x.emplace_back(buf, dc);
        y.emplace_back(out, dc);
        dx.emplace_back(buf, dc);
        dy.emplace_back(out, dc);
        fill_uniform(host, r);
        x[r].load_sync(host.data(), 0, buf, conn);
        fill_uniform(host, 100 + r);
        dy[r].load_sync(host.data(), 0, out, conn);
        dx[r].set_constant(0.0f, conn);
        xp.push_back(x[r].dptr());
        dxp.push_back(dx[r].dptr());
        x_tiles[r] = x[r].dptr();
        y_tiles[r] = y[r].dptr();
        dx_tiles[r] = dx[r].dptr();
        dy_tiles[r] = dy[r].dptr();
      }
    }
    GPUContext *dc0 = ctx->device_context(0).get();
    GPUMemory<float> w(wsz, dc0), dw(wsz, dc0);
    {
      std::vector<float> host(wsz);
      fill_uniform(host, 7);
      const float scale = std::sqrt(2.0f / (C * ksz * ksz));
      for (auto &v : host) v *= scale;
      GPUConn conn = dc0->conn();
      w.load_sync(host.data(), 0, wsz, conn);
    }
    size_t ws_bytes = 0;
    for (int pass = 0; pass < 3; ++pass)
      for (uint32_t tiles : {1u, K})
        ws_bytes = std::max(ws_bytes, adh_conv2d_workspace_bytes(pass, ADH_F32, tiles, N, C, C, HP, WP, ksz, ksz, 1, 1, dil, dil));
    dc0->reserve_scratch(std::max<size_t>(4096, ws_bytes));  // :202
    auto scratch = dc0->get_scratch();
    ctx->sync();

    const Halo halo{comms.data(), ctx.get(), K, p, W, H, C, N};
    const double strip = (double)p * W * C * N * 4.0;  // :262
    const double flops = 2.0 * K * N * C * C * ksz * ksz * (double)H * W;

    // "spatial halo exchange (fwd)" :227-269, "spatial halo reduce (bwd)" :271-313
    Stat seq = time_trials(ctx.get(), halo_trials, [&] { halo.per_rank(false, xp.data(), true); });
    Stat one = time_trials(ctx.get(), halo_trials, [&] {
      halo.all_ranks(false, xp.data());
      ctx->sync();
    });
    print_entry("spatial_conv", "halo exchange", seq, one, strip, 0.0);
    const Stat exch_seq = seq, exch_one = one;
    seq = time_trials(ctx.get(), halo_trials, [&] { halo.per_rank(true, dxp.data(), true); });
    one = time_trials(ctx.get(), halo_trials, [&] {
      halo.all_ranks(true, dxp.data());
      ctx->sync();
    });
    print_entry("spatial_conv", "halo reduce", seq, one, strip, 0.0);
    const Stat red_seq = seq, red_one = one;

    // "spatial conv (fwd)" :316-392
    seq = time_trials(ctx.get(), conv_trials, [&] {
      halo.per_rank(false, xp.data(), true);
      for (uint32_t r = 0; r < K; ++r) {
        GPUConn conn = ctx->device_context(r)->conn();
        check(adh_conv2d_slab_fwd_tiles(ADH_F32, 1, N, C, C, HP, WP, ksz, ksz, 1, 1, dil, dil, &x_tiles[r], w.dptr(), &y_tiles[r],
                                        0.0f, scratch->dptr(), scratch->size(), conn.stream()),
              "conv fwd");
      }
      for (uint32_t r = 0; r < K; ++r) ctx->device_context(r)->sync();
    });
    one = time_trials(ctx.get(), conv_trials, [&] {
      halo.all_ranks(false, xp.data());
      GPUConn conn = dc0->conn();
      check(adh_conv2d_slab_fwd_tiles(ADH_F32, K, N, C, C, HP, WP, ksz, ksz, 1, 1, dil, dil, x_tiles, w.dptr(), y_tiles, 0.0f,
                                      scratch->dptr(), scratch->size(), conn.stream()),
            "conv fwd (all tiles)");
      ctx->sync();
    });
    print_entry("spatial_conv", "spatial conv (fwd): exchange + conv forward", seq, one, 0.0, flops);
    const Stat fwd_seq = seq, fwd_one = one;

    // "spatial conv (bwd)" :394-477: backward-filter per rank, backward-data per rank, sync, reduce, sync.  The
    // reference's ranks each overwrite their own dw (beta = 0); on one GPU the ranks' shares add up in one dw.
    seq = time_trials(ctx.get(), conv_trials, [&] {
      for (uint32_t r = 0; r < K; ++r) {
        GPUConn conn = ctx->device_context(r)->conn();
        check(adh_conv2d_slab_bwd_filter_tiles(ADH_F32, 1, N, C, C, HP, WP, ksz, ksz, 1, 1, dil, dil, &x_tiles[r], &dy_tiles[r],
                                               dw.dptr(), r ? 1.0f : 0.0f, scratch->dptr(), scratch->size(), conn.stream()),
              "conv bwd-filter");
      }
      for (uint32_t r = 0; r < K; ++r) {
        GPUConn conn = ctx->device_context(r)->conn();
        check(adh_conv2d_slab_bwd_data_tiles(ADH_F32, 1, N, C, C, HP, WP, ksz, ksz, 1, 1, dil, dil, w.dptr(), &dy_tiles[r],
                                             &dx_tiles[r], 0.0f, scratch->dptr(), scratch->size(), conn.stream()),
              "conv bwd-data");
      }
      for (uint32_t r = 0; r < K; ++r) ctx->device_context(r)->sync();
      halo.per_rank(true, dxp.data(), true);
    });
    one = time_trials(ctx.get(), conv_trials, [&] {
      GPUConn conn = dc0->conn();
      check(adh_conv2d_slab_bwd_filter_tiles(ADH_F32, K, N, C, C, HP, WP, ksz, ksz, 1, 1, dil, dil, x_tiles, dy_tiles, dw.dptr(),
                                             0.0f, scratch->dptr(), scratch->size(), conn.stream()),
            "conv bwd-filter (all tiles)");
      check(adh_conv2d_slab_bwd_data_tiles(ADH_F32, K, N, C, C, HP, WP, ksz, ksz, 1, 1, dil, dil, w.dptr(), dy_tiles, dx_tiles,
                                           0.0f, scratch->dptr(), scratch->size(), conn.stream()),
            "conv bwd-data (all tiles)");
      halo.all_ranks(true, dxp.data());
      ctx->sync();
    });
    print_entry("spatial_conv", "spatial conv (bwd): conv backward-filter + backward-data + reduce", seq, one, 0.0, 2.0 * flops);

    std::printf("{\"which\": \"spatial_conv\", \"ranks\": %u, \"halo_trials\": %d, \"conv_trials\": %d, \"conv\": %u, \"dilate\": %u, "
                "\"halo\": %u, \"n\": %u, \"c\": %u, \"h\": %u, \"w\": %u, "
                "\"exchange_per_rank_sequence_ms\": %.5f, \"exchange_one_launch_ms\": %.5f, "
                "\"reduce_per_rank_sequence_ms\": %.5f, \"reduce_one_launch_ms\": %.5f, "
                "\"fwd_per_rank_sequence_ms\": %.5f, \"fwd_one_launch_ms\": %.5f, "
                "\"bwd_per_rank_sequence_ms\": %.5f, \"bwd_one_launch_ms\": %.5f}\n",
                K, halo_trials, conv_trials, ksz, dil, p, N, C, H, W, exch_seq.avg_ms, exch_one.avg_ms, red_seq.avg_ms,
                red_one.avg_ms, fwd_seq.avg_ms, fwd_one.avg_ms, seq.avg_ms, one.avg_ms);
    return 0;
  } catch (const std::exception &e) {
    std::fprintf(stderr, "microbench_spatial: %s\n", e.what());
    return 1;
  }
}
