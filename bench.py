#!/usr/bin/env python3
"""Benchmark of the spatially-parallel convolution path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the hot path's dominant stage over one batch of synthetic input: the 3x3
slab convolution forward of the largest configuration that fits one GPU, the high-resolution one
(bf16 in HBM, fp32 accumulate, NCHW N=2, Cin=Cout=64, a 1024x2048 image in 8 row-tiles of 128(+2)
x 2048(+2)), one call through the C ABI over all tiles, inputs resident in HBM.  Before the
warm-up the same call is repeated, untimed, for at least 150 ms (`clock_ramp_ms`): the clocks of an
idle GPU need tens of milliseconds to come up and, under this kernel, settle at what the power
limit allows, so that 20 timed steps measure what 2000 would.  One JSON line is printed: `value`
is the conv throughput in TFLOP/s (algorithmic flops 2*N*Cout*Cin*H*W*9 per tile), `roofline` is
that kernel against the bf16 MFMA peak, `cpu_baseline` is the scalar CPU port timed on this host
(one thread, and one thread per tile), and `secondary` carries every other kernel of the path with
its own roofline figure: the fp32 conv of the ResNet-sized configurations, halo pack / unpack /
exchange / reduce, channel slice, softmax-NLL, the backward convolutions, and the three shapes the
reference's own microbenchmarks time.  Everything is timed with device events on the stream the
kernels are launched on.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# HBM bytes per launch of a kernel instance, measured with rocprofv3 PMC (FETCH_SIZE and WRITE_SIZE, each scaled
# by what the same counter reads for a 1 GiB plain copy).  Not re-measured by this script: the figures are read
# from the committed summaries under profiles/ (lines `traffic_bytes_per_launch[<kernel instance>] = <bytes>`),
# each belongs to the kernel instance named in its brackets, and an instance without such a line (the library
# routes the shape elsewhere, or the kernel changed its name) reports null.
def measured_traffic():
    import glob
    import re
    found = {}
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*_hbm_traffic.txt"))):
        with open(path) as f:
            for line in f:
                m = re.match(r"traffic_bytes_per_launch\[(.+)\] = ([0-9.eE+]+)", line.strip())
                if m:
                    found[m.group(1)] = (float(m.group(2)), os.path.relpath(path, ROOT))
    return found


CLOCK_RAMP_MS = 150.0
HBM_PEAK_GBS = 8000.0
MFMA_F32_PEAK_TFLOPS = 157.3
MFMA_BF16_PEAK_TFLOPS = 2500.0
METRIC = "halo pack/unpack GB/s (% HBM peak); 3x3 slab-conv TFLOP/s (% MFMA peak)"


def time_gpu(fn, reps, warmup):
    """Average milliseconds per call of fn(), device events on the current stream."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def time_gpu_flushed(fn, reps, scratch):
    """Average milliseconds per call of fn() when every call is preceded by a read of `scratch` (512 MB, twice
    the on-package cache), so that fn's operands come from HBM and the cache holds clean lines: the time of a
    (read, fn) loop minus the time of the read loop alone, best of three.  (Flushing by WRITING the buffer
    leaves the cache full of dirty lines whose write-back is then charged to fn: about a fifth slower.)"""
    import torch
    both, alone = [], []
    flush = lambda: torch.amax(scratch)
    for i in range(3):
        alone.append(time_gpu(flush, reps, 3))
        both.append(time_gpu(lambda: (flush(), fn()), reps, 3))
    return max(min(both) - min(alone), 1e-6)


def time_gpu_graph(fn, per_graph=50, replays=10):
    """Average milliseconds per call of fn() when `per_graph` calls are captured into one HIP graph and the
    graph is replayed: the device-side time of a launch-bound loop, without the host's launch cost."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(per_graph):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (replays * per_graph)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20,
                    help="untimed steps after the fixed clock-ramp phase")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-secondary", action="store_true", help="time only the headline kernel")
    ap.add_argument("--no-end-to-end", action="store_true",
                    help="skip the end-to-end trainer leg (a child process; leave it out under a profiler)")
    ap.add_argument("--only", default=None,
                    help="time only the secondary entries whose name contains this text (for profiling one kernel)")
    ap.add_argument("--lib", default=None,
                    help="another build of libadh.so to load (A/B measurements of a kernel variant)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain copy of known size (1 GiB read + 1 GiB written) 10 times: the kernel "
                         "whose FETCH_SIZE / WRITE_SIZE readings calibrate the HBM traffic counters")
    args = ap.parse_args()
    if args.lib:
        os.environ["ADH_LIB"] = os.path.abspath(args.lib)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU (the K row-tiles live in one HBM, there are no "
              "inter-GPU collectives); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    # End-to-end leg, run first as a child process (before this process touches the GPU): the synthetic-data trainer
    # of the spatially-parallel ResNet-18 variant, every op of the path plus the optimizer, 4 row-tiles.
    import torch
    if torch.cuda.device_count() == 0:  # counting devices does not initialise the GPU
        print("bench.py: no GPU visible; there is no CPU fallback", file=sys.stderr)
        sys.exit(3)
    end_to_end = None
    trainer = os.path.join(os.path.dirname(os.path.abspath(__file__)), "arraydiff_cuda_amd", "train_resnet18")
    if not args.no_secondary and not args.no_end_to_end and args.only is None:
        import subprocess
        if not os.path.exists(trainer):
            print("bench.py: %s is not built (run __graft_entry__.build())" % trainer, file=sys.stderr)
            sys.exit(3)
        r = subprocess.run([trainer, "--ranks", "4", "--batch", "32", "--size", "256", "--steps", "10", "--warmup", "3"],
                           capture_output=True, text=True, timeout=600)
        if r.returncode != 0:
            print("bench.py: the end-to-end trainer failed:\n" + r.stdout[-2000:] + r.stderr[-2000:], file=sys.stderr)
            sys.exit(4)
        end_to_end = json.loads(r.stdout.strip().splitlines()[-1])
        # the same steps replayed from one recorded HIP graph (forward, backward, optimizer): reported beside the eager figure
        g = subprocess.run([trainer, "--ranks", "4", "--batch", "32", "--size", "256", "--steps", "10", "--warmup", "3",
                            "--graph", "1"], capture_output=True, text=True, timeout=600)
        if g.returncode == 0:
            replay = json.loads(g.stdout.strip().splitlines()[-1])
            end_to_end["ms_per_step_graph_replay"] = replay["ms_per_step"]
            end_to_end["graph_replay_same_loss"] = replay["loss_last"] == end_to_end["loss_last"]
        else:
            print("bench.py: the graph-replay run of the trainer failed:\n" + g.stdout[-1000:] + g.stderr[-1000:], file=sys.stderr)

    # The reference's own microbenchmarks (tools/microbench_spatial.cc, tools/microbench_spatial_conv.cc, tools/microbench_conv.cc) as a C++
    # binary over this library's Spatial2DComm and C ABI, also a child process: per rank group_start / halo_* /
    # group_end with the reference's synchronisations, beside one launch for all ranks' tiles; wall-clock averages.
    reference_microbench = None
    micro = os.path.join(ROOT, "arraydiff_cuda_amd", "microbench_spatial")
    if not args.no_secondary and not args.no_end_to_end and args.only is None:
        import subprocess
        if not os.path.exists(micro):
            print("bench.py: %s is not built (run __graft_entry__.build())" % micro, file=sys.stderr)
            sys.exit(3)
        reference_microbench = []
        for which, trials in (("spatial", "1000"), ("spatial_conv", "100"), ("conv", "1000")):
            r = subprocess.run([micro, "--which", which, "--ranks", "4", "--trials", trials], capture_output=True, text=True,
                               timeout=600)
            if r.returncode != 0:
                print("bench.py: microbench_spatial --which %s failed:\n" % which + r.stdout[-2000:] + r.stderr[-2000:],
                      file=sys.stderr)
                sys.exit(4)
            lines = [json.loads(l) for l in r.stdout.strip().splitlines()]
            reference_microbench += [l for l in lines if "name" in l]

    import numpy as np
    import torch
    from arraydiff_cuda_amd import capi

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; there is no CPU fallback", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    lib = capi.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    g = torch.Generator(device="cuda").manual_seed(0x5EED)

    # ---- workload: the 3x3 slab conv forward of the high-resolution configuration on the bf16 matrix cores ----
    C = 64
    K5, N5, H5, W5 = 8, 2, 1024, 2048
    Ht5 = H5 // K5
    X5 = (torch.rand((N5, C, H5, W5), device="cuda", generator=g) * 2 - 1).to(torch.bfloat16)
    t5 = [torch.empty((N5, C, Ht5 + 2, W5 + 2), device="cuda", dtype=torch.bfloat16) for _ in range(K5)]
    t5_tbl, _k5 = capi.ptr_table([t.data_ptr() for t in t5])
    capi.check(lib.adh_tiles_pack_nchw(1, K5, 1, W5, H5, C, N5, X5.data_ptr(), t5_tbl, stream), "pack cfg5")
    w5 = (torch.randn((C, C, 3, 3), device="cuda", generator=g) * (2.0 / (C * 9)) ** 0.5).to(torch.bfloat16)
    y5 = [torch.empty((N5, C, Ht5, W5), device="cuda", dtype=torch.bfloat16) for _ in range(K5)]
    y5_tbl, _ky = capi.ptr_table([t.data_ptr() for t in y5])
    ws5_bytes = max(lib.adh_conv3x3_workspace_bytes(wh, 1, K5, N5, C, C, Ht5, W5) for wh in (0, 1, 2))
    ws5 = torch.empty(ws5_bytes // 4 + 64, device="cuda")
    flops5 = 2.0 * K5 * N5 * C * C * 9 * Ht5 * W5

    def conv_fwd5():
        return lib.adh_conv3x3_slab_fwd_tiles(1, K5, N5, C, C, Ht5, W5, t5_tbl, w5.data_ptr(), y5_tbl, 0.0,
                                              ws5.data_ptr(), ws5_bytes, stream)

    capi.check(conv_fwd5(), "conv fwd cfg5")

    # ---- clock ramp: the same launch, untimed, until the clocks have settled ----
    torch.cuda.synchronize()
    t_ramp = time.perf_counter()
    while (time.perf_counter() - t_ramp) * 1e3 < CLOCK_RAMP_MS:
        for _ in range(20):
            conv_fwd5()
        torch.cuda.synchronize()
    clock_ramp_ms = (time.perf_counter() - t_ramp) * 1e3

    # ---- the timed region: W warmup steps, then exactly K steps between two synchronisations ----
    for _ in range(args.warmup):
        conv_fwd5()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        conv_fwd5()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    kernel_ms = e0.elapsed_time(e1) / args.steps
    value = flops5 / (ms_per_step * 1e-3) / 1e12
    achieved = flops5 / (kernel_ms * 1e-3) / 1e12
    name5 = capi.conv_kernel_name(capi.ADH_CONV_FWD, capi.ADH_BF16, K5, N5, C, C, Ht5, W5)
    traffic = measured_traffic()
    in5_b = K5 * N5 * C * (Ht5 + 2) * (W5 + 2) * 2
    out5_b = N5 * C * H5 * W5 * 2
    ai5 = flops5 / (in5_b + out5_b + C * C * 9 * 2)

    out = {
        "metric": METRIC, "value": round(value, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic", "clock_ramp_ms": round(clock_ramp_ms, 1),
        "config": {"workload": "configs[4]: 3x3 slab conv fwd, bf16 in / fp32 accumulate, NCHW N=2 Cin=Cout=64, "
                               "1024x2048 image in 8 row-tiles of 128(+2)x2048(+2), one call over all tiles",
                   "flops_per_step": flops5, "tiles": K5, "halo": 1},
        "roofline": {"kernel": name5 + " (fwd; the only kernel of the call: it reads the filter as the caller holds it)", "bound": "mfma",
                     "achieved": round(achieved, 3), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": traffic.get(name5, (None, None))[0], "traffic_source": traffic.get(name5, (None, None))[1],
                     "launch_ms": round(kernel_ms, 5),
                     "compulsory_bytes": in5_b + out5_b + C * C * 9 * 2,
                     "min_mfma_hbm_bound_TFLOPs": round(min(MFMA_BF16_PEAK_TFLOPS, HBM_PEAK_GBS * ai5 / 1e3), 1)},
    }

    # ---- the tensors of the ResNet-sized configurations (cfg1-cfg3): fp32 N=32, C=64, 56x56 in 4 row-tiles of 14 rows ----
    K, p, N, H, W = 4, 1, 32, 56, 56
    Ht = H // K
    X = torch.rand((N, C, H, W), device="cuda", generator=g) * 2 - 1
    wt = torch.randn((C, C, 3, 3), device="cuda", generator=g) * (2.0 / (C * 9)) ** 0.5
    dY = torch.randn((N, C, H, W), device="cuda", generator=g)
    tiles = [torch.empty((N, C, Ht + 2, W + 2), device="cuda") for _ in range(K)]
    ys = [torch.empty((N, C, Ht, W), device="cuda") for _ in range(K)]
    dys = [dY[:, :, r * Ht:(r + 1) * Ht].contiguous() for r in range(K)]
    gs = [torch.zeros((N, C, Ht + 2, W + 2), device="cuda") for _ in range(K)]
    gw = torch.zeros_like(wt)
    Y = torch.empty_like(X)
    capi.check(capi.tiles_pack(K, p, W, H, C, N, X, tiles), "pack")

    tile_tbl, _k1 = capi.ptr_table([t.data_ptr() for t in tiles])
    y_tbl, _k2 = capi.ptr_table([t.data_ptr() for t in ys])
    dy_tbl, _k3 = capi.ptr_table([t.data_ptr() for t in dys])
    g_tbl, _k4 = capi.ptr_table([t.data_ptr() for t in gs])
    ws_bytes = capi.conv_workspace_bytes(capi.ADH_CONV_BWD_FILTER, capi.ADH_F32, K, N, C, C, Ht, W)
    ws = torch.empty(max(ws_bytes // 4, 1), device="cuda")
    flops_step = 2.0 * N * C * C * Ht * W * 9 * K
    capi.check(lib.adh_conv3x3_slab_fwd_tiles(capi.ADH_F32, K, N, C, C, Ht, W, tile_tbl, wt.data_ptr(), y_tbl, 0.0,
                                              None, 0, stream), "conv fwd")

    if args.copy_calibration:
        cw, chh, cc, cn = 1024, 1024, 64, 4  # 2^28 floats = 1 GiB each way, rows contiguous
        src = torch.ones((cn, cc, chh, cw), device="cuda")
        dst = torch.empty_like(src)
        for _ in range(10):
            capi.check(lib.adh_slice_copy_nchw(0, cw, chh, cc, cn, src.data_ptr(), cw, chh, cc, 0, 0, 0, dst.data_ptr(),
                                               cw, chh, cc, 0, 0, 0, stream), "copy calibration")
        torch.cuda.synchronize()
        out["copy_calibration_bytes_each_way"] = cw * chh * cc * cn * 4
        del src, dst

    # ---- secondary kernels of the path ----
    if not args.no_secondary:
        es = 4
        strip = p * W * C * N * es
        reps, wu = 200, 20
        sec = []

        flush_scratch = torch.empty(128 * 1024 * 1024, device="cuda")  # 512 MB

        def add(name, fn, bound, work, peak, unit, note=None, flushed=False, graph=False, extra=None):
            nonlocal stream
            if args.only is not None and args.only not in name:
                return
            ms = time_gpu(fn, reps, wu)
            ach = work / (ms * 1e-3) / (1e9 if unit == "GB/s" else 1e12)
            e = {"name": name, "ms": round(ms, 5), "bound": bound, "achieved": round(ach, 3), "peak": peak,
                 "unit": unit, "frac": round(ach / peak, 4), "work": work}
            if flushed:
                # the warm figure above has its operands resident in the 256 MB on-package cache;
                # this one reads 512 MB of something else before every call
                msf = time_gpu_flushed(fn, 30, flush_scratch)
                achf = work / (msf * 1e-3) / (1e9 if unit == "GB/s" else 1e12)
                e["ms_flushed"] = round(msf, 5)
                e["achieved_flushed"] = round(achf, 3)
                e["frac_flushed"] = round(achf / peak, 4)
            if graph:
                # launch-sized kernels: 50 launches captured into one HIP graph, replayed (the launches then come from
                # the device's queue, not from this interpreter)
                saved = stream

                def fn_on_current_stream():
                    nonlocal stream
                    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                    fn()

                msg = time_gpu_graph(fn_on_current_stream)
                stream = saved
                achg = work / (msg * 1e-3) / (1e9 if unit == "GB/s" else 1e12)
                e["ms_in_graph"] = round(msg, 5)
                e["achieved_in_graph"] = round(achg, 3)
                e["frac_in_graph"] = round(achg / peak, 4)
            if note:
                e["note"] = note
            if extra:
                e.update(extra(ms) if callable(extra) else extra)
            sec.append(e)

        unsplit_b = N * C * H * W * es
        padded_b = K * N * C * (Ht + 2 * p) * (W + 2 * p) * es
        name2 = capi.conv_kernel_name(capi.ADH_CONV_FWD, capi.ADH_F32, K, N, C, C, Ht, W)
        reps, wu = 500, 300
        add("conv fwd cfg2 (fp32, 4 tiles of 14(+2)x56(+2), one launch)",
            lambda: lib.adh_conv3x3_slab_fwd_tiles(capi.ADH_F32, K, N, C, C, Ht, W, tile_tbl, wt.data_ptr(), y_tbl, 0.0,
                                                   None, 0, stream),
            "mfma", flops_step, MFMA_F32_PEAK_TFLOPS, "TFLOP/s",
            extra={"kernel": name2, "traffic": traffic.get(name2, (None, None))[0]})
        reps, wu = 200, 20
        add("halo pack cfg1 (unsplit -> 4 padded tiles)",
            lambda: lib.adh_tiles_pack_nchw(0, K, p, W, H, C, N, X.data_ptr(), tile_tbl, stream),
            "hbm", unsplit_b + padded_b, HBM_PEAK_GBS, "GB/s", flushed=True, graph=True)
        add("halo unpack cfg1 (4 padded tiles -> unsplit)",
            lambda: lib.adh_tiles_unpack_nchw(0, K, p, W, H, C, N, tile_tbl, Y.data_ptr(), stream),
            "hbm", 2 * unsplit_b, HBM_PEAK_GBS, "GB/s", flushed=True, graph=True)
        add("halo exchange cfg1 (6 strips)",
            lambda: lib.adh_halo_exchange_nchw(0, 1, K, p, W, Ht, C, N, tile_tbl, stream),
            "hbm", 2 * 2 * (K - 1) * strip, HBM_PEAK_GBS, "GB/s",
            graph=True, extra=lambda ms: {"reference_figure_GBs": round(strip / (ms * 1e-3) / 1e9, 3),
                                          "reference_figure": "p*W*C*N*4 / t (tools/microbench_spatial.cc:100-101)"})
        add("halo reduce cfg1 (6 strips)",
            lambda: lib.adh_halo_reduce_nchw(0, 1, K, p, W, Ht, C, N, g_tbl, stream),
            "hbm", 3 * 2 * (K - 1) * strip, HBM_PEAK_GBS, "GB/s", graph=True)
        sl = torch.empty((N, 32, H, W), device="cuda")
        add("channel slice [16,48) cfg4",
            lambda: lib.adh_slice_copy_nchw(0, W, H, 32, N, X.data_ptr(), W, H, C, 0, 0, 16, sl.data_ptr(), W, H, 32,
                                            0, 0, 0, stream),
            "hbm", 2 * N * 32 * H * W * es, HBM_PEAK_GBS, "GB/s", flushed=True)
        Ns, Cs = 256, 1000
        logits = torch.randn((Ns, Cs), device="cuda", generator=g) * 2
        labels = torch.randint(0, Cs, (Ns,), device="cuda", dtype=torch.int32)
        sy = torch.empty_like(logits)
        sloss = torch.empty(Ns, device="cuda")
        sdx = torch.zeros_like(logits)
        dl = torch.full((Ns,), 1.0 / Ns, device="cuda")
        add("softmax + nll fwd cfg4 (256x1000)",
            lambda: lib.adh_softmax_xent_fwd(Cs, Ns, logits.data_ptr(), labels.data_ptr(), sy.data_ptr(),
                                             sloss.data_ptr(), stream),
            "hbm", 2 * Ns * Cs * 4 + 8 * Ns, HBM_PEAK_GBS, "GB/s", flushed=True, graph=True)
        add("softmax-nll bwd cfg4 (256x1000)",
            lambda: lib.adh_softmax_nll_loss_bwd(Cs, Ns, sy.data_ptr(), labels.data_ptr(), dl.data_ptr(),
                                                 sdx.data_ptr(), stream),
            "hbm", 3 * Ns * Cs * 4 + 8 * Ns, HBM_PEAK_GBS, "GB/s", graph=True)
        add("softmax + nll fwd and bwd in one kernel cfg4 (256x1000)",
            lambda: lib.adh_softmax_xent_fwd_bwd(Cs, Ns, logits.data_ptr(), labels.data_ptr(), dl.data_ptr(), 0.0,
                                                 sy.data_ptr(), sloss.data_ptr(), 0.0, sdx.data_ptr(), stream),
            "hbm", 3 * Ns * Cs * 4 + 12 * Ns, HBM_PEAK_GBS, "GB/s", graph=True)
        add("conv fwd cfg3 over unexchanged tiles (4 tiles, exchange + conv in one launch)",
            lambda: lib.adh_conv3x3_slab_fwd_tiles_unexchanged(0, K, N, C, C, Ht, W, tile_tbl, wt.data_ptr(), y_tbl, 0.0,
                                                               None, 0, stream),
            "mfma", flops_step, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
        add("halo exchange + conv fwd cfg3 (4 tiles, two launches: what the one above replaces)",
            lambda: (lib.adh_halo_exchange_nchw(0, 1, K, p, W, Ht, C, N, tile_tbl, stream),
                     lib.adh_conv3x3_slab_fwd_tiles(0, K, N, C, C, Ht, W, tile_tbl, wt.data_ptr(), y_tbl, 0.0, None, 0,
                                                    stream))[1],
            "mfma", flops_step, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
        add("conv bwd-data cfg3 (4 tiles)",
            lambda: lib.adh_conv3x3_slab_bwd_data_tiles(0, K, N, C, C, Ht, W, wt.data_ptr(), dy_tbl, g_tbl, 0.0, None,
                                                        0, stream),
            "mfma", flops_step, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
        add("conv bwd-data cfg3 with the halo reduce folded in (4 tiles, one launch)",
            lambda: lib.adh_conv3x3_slab_bwd_data_tiles_reduced(0, K, N, C, C, Ht, W, wt.data_ptr(), dy_tbl, g_tbl, 0.0,
                                                                None, 0, stream),
            "mfma", flops_step, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
        add("conv bwd-data cfg3 + halo reduce (two launches: what the one above replaces)",
            lambda: (lib.adh_conv3x3_slab_bwd_data_tiles(0, K, N, C, C, Ht, W, wt.data_ptr(), dy_tbl, g_tbl, 0.0, None, 0,
                                                         stream),
                     lib.adh_halo_reduce_nchw(0, 1, K, p, W, Ht, C, N, g_tbl, stream))[1],
            "mfma", flops_step, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
        add("conv bwd-filter cfg3 (4 tiles, two kernels)",
            lambda: lib.adh_conv3x3_slab_bwd_filter_tiles(0, K, N, C, C, Ht, W, tile_tbl, dy_tbl, gw.data_ptr(), 0.0,
                                                          ws.data_ptr(), ws_bytes, stream),
            "mfma", flops_step, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")

        # config 5 sized pack / unpack: 0.5 GB, larger than the on-package cache
        Y5 = torch.empty_like(X5)
        b5 = N5 * C * H5 * W5 * 2
        reps, wu = 50, 5
        add("halo pack cfg5 (bf16, 8 tiles of 128 rows)",
            lambda: lib.adh_tiles_pack_nchw(1, K5, 1, W5, H5, C, N5, X5.data_ptr(), t5_tbl, stream),
            "hbm", b5 + K5 * N5 * C * (H5 // K5 + 2) * (W5 + 2) * 2, HBM_PEAK_GBS, "GB/s")
        add("halo unpack cfg5 (bf16)",
            lambda: lib.adh_tiles_unpack_nchw(1, K5, 1, W5, H5, C, N5, t5_tbl, Y5.data_ptr(), stream),
            "hbm", 2 * b5, HBM_PEAK_GBS, "GB/s")
        # config 5 slab conv on the bf16 matrix cores: bwd-data (beta = 0, what the host op issues for the first
        # toucher of a gradient, and beta = 1, as the reference accumulates input gradients), bwd-filter; the
        # forward pass is the headline above
        gw5 = torch.zeros((C, C, 3, 3), device="cuda")
        reps, wu = 50, 10
        add("conv fwd cfg5 (bf16, 8 tiles)",
            lambda: lib.adh_conv3x3_slab_fwd_tiles(1, K5, N5, C, C, Ht5, W5, t5_tbl, w5.data_ptr(), y5_tbl, 0.0,
                                                   ws5.data_ptr(), ws5_bytes, stream),
            "mfma", flops5, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
        add("conv bwd-data cfg5 (bf16, beta=0: first toucher of the gradient, what the host op issues)",
            lambda: lib.adh_conv3x3_slab_bwd_data_tiles(1, K5, N5, C, C, Ht5, W5, w5.data_ptr(), y5_tbl, t5_tbl, 0.0,
                                                        ws5.data_ptr(), ws5_bytes, stream),
            "mfma", flops5, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
        add("conv bwd-data cfg5 (bf16, beta=1)",
            lambda: lib.adh_conv3x3_slab_bwd_data_tiles(1, K5, N5, C, C, Ht5, W5, w5.data_ptr(), y5_tbl, t5_tbl, 1.0,
                                                        ws5.data_ptr(), ws5_bytes, stream),
            "mfma", flops5, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
        add("conv bwd-filter cfg5 (bf16 in, fp32 filter gradient, two kernels)",
            lambda: lib.adh_conv3x3_slab_bwd_filter_tiles(1, K5, N5, C, C, Ht5, W5, t5_tbl, y5_tbl, gw5.data_ptr(), 0.0,
                                                          ws5.data_ptr(), ws5_bytes, stream),
            "mfma", flops5, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
        # the same convolution over tiles WITHOUT halo: one launch does what pack (pad + exchange) + conv, and conv
        # backward-data + halo reduce + unpack, do in two and three
        xu = [X5[:, :, r * Ht5:(r + 1) * Ht5, :].contiguous() for r in range(K5)]
        yu = [torch.empty((N5, C, Ht5, W5), device="cuda", dtype=torch.bfloat16) for _ in range(K5)]
        xu_tbl, _ku1 = capi.ptr_table([t.data_ptr() for t in xu])
        yu_tbl, _ku2 = capi.ptr_table([t.data_ptr() for t in yu])
        add("conv fwd cfg5 over tiles without halo (bf16; pad, exchange and conv in one launch)",
            lambda: lib.adh_conv3x3_unpadded_fwd_tiles(1, K5, N5, C, C, Ht5, W5, xu_tbl, w5.data_ptr(), yu_tbl, 0.0,
                                                       ws5.data_ptr(), ws5_bytes, stream),
            "mfma", flops5, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s",
            note="replaces halo pack cfg5 + conv fwd cfg5 above (their times add)")
        add("conv bwd-data cfg5 into tiles without halo (bf16, beta=0; conv, halo reduce and unpad in one launch)",
            lambda: lib.adh_conv3x3_unpadded_bwd_data_tiles(1, K5, N5, C, C, Ht5, W5, w5.data_ptr(), y5_tbl, xu_tbl, 0.0,
                                                            ws5.data_ptr(), ws5_bytes, stream),
            "mfma", flops5, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s",
            note="replaces conv bwd-data cfg5 + halo reduce + halo unpack cfg5 above (their times add)")
        gu = [torch.zeros((N5, C, Ht5, W5), device="cuda", dtype=torch.bfloat16) for _ in range(K5)]
        gu_tbl, _ku3 = capi.ptr_table([t.data_ptr() for t in gu])
        add("conv bwd-data cfg5 into tiles without halo (bf16, beta=1: accumulates into the gradient tiles)",
            lambda: lib.adh_conv3x3_unpadded_bwd_data_tiles(1, K5, N5, C, C, Ht5, W5, w5.data_ptr(), y5_tbl, gu_tbl, 1.0,
                                                            ws5.data_ptr(), ws5_bytes, stream),
            "mfma", flops5, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
        del gu
        add("conv bwd-filter cfg5 over tiles without halo (bf16 in, fp32 filter gradient, two kernels)",
            lambda: lib.adh_conv3x3_unpadded_bwd_filter_tiles(1, K5, N5, C, C, Ht5, W5, xu_tbl, y5_tbl, gw5.data_ptr(), 0.0,
                                                              ws5.data_ptr(), ws5_bytes, stream),
            "mfma", flops5, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
        del Y5, xu, yu
        # more than 64 channels on the bf16 matrix cores: 128 reduction channels per launch with the sums in registers
        # (256: two launches with fp32 sums between them); the filter gradient as 64 x 64 channel pairs.  The
        # high-resolution tiles at half (128 channels) and a quarter (256 channels) of the width.
        for Cw, Ww, how in ((128, W5 // 2, "one launch"), (256, W5 // 4, "two launches of 128 reduction channels")):
            xw = [torch.rand((N5, Cw, Ht5 + 2, Ww + 2), device="cuda", generator=g).to(torch.bfloat16) for _ in range(K5)]
            yw = [torch.rand((N5, Cw, Ht5, Ww), device="cuda", generator=g).to(torch.bfloat16) for _ in range(K5)]
            ww = (torch.randn((Cw, Cw, 3, 3), device="cuda", generator=g) * (2.0 / (Cw * 9)) ** 0.5).to(torch.bfloat16)
            gww = torch.zeros((Cw, Cw, 3, 3), device="cuda")
            xw_tbl, _kw1 = capi.ptr_table([t.data_ptr() for t in xw])
            yw_tbl, _kw2 = capi.ptr_table([t.data_ptr() for t in yw])
            wsw_bytes = max(capi.conv_workspace_bytes(wh, capi.ADH_BF16, K5, N5, Cw, Cw, Ht5, Ww)
                            for wh in (capi.ADH_CONV_FWD, capi.ADH_CONV_BWD_DATA, capi.ADH_CONV_BWD_FILTER))
            wsw = torch.empty(wsw_bytes // 4 + 64, device="cuda")
            flopsw = 2.0 * K5 * N5 * Cw * Cw * 9 * Ht5 * Ww
            shape_w = "%d->%d channels, 8 tiles of 128(+2)x%d(+2)" % (Cw, Cw, Ww)
            kname = capi.conv_kernel_name(capi.ADH_CONV_FWD, capi.ADH_BF16, K5, N5, Cw, Cw, Ht5, Ww)
            add("conv fwd bf16 %s (%s)" % (shape_w, how),
                lambda: lib.adh_conv3x3_slab_fwd_tiles(1, K5, N5, Cw, Cw, Ht5, Ww, xw_tbl, ww.data_ptr(), yw_tbl, 0.0,
                                                       wsw.data_ptr(), wsw_bytes, stream),
                "mfma", flopsw, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s",
                extra={"kernel": kname, "traffic": traffic.get(kname, (None, None))[0]})
            add("conv bwd-data bf16 %s (%s)" % (shape_w, how),
                lambda: lib.adh_conv3x3_slab_bwd_data_tiles(1, K5, N5, Cw, Cw, Ht5, Ww, ww.data_ptr(), yw_tbl, xw_tbl, 0.0,
                                                            wsw.data_ptr(), wsw_bytes, stream),
                "mfma", flopsw, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
            add("conv bwd-filter bf16 %s (channel pairs of 64 x 64 in one launch + reduction)" % shape_w,
                lambda: lib.adh_conv3x3_slab_bwd_filter_tiles(1, K5, N5, Cw, Cw, Ht5, Ww, xw_tbl, yw_tbl, gww.data_ptr(),
                                                              0.0, wsw.data_ptr(), wsw_bytes, stream),
                "mfma", flopsw, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
            if Cw == 128:
                xwu = [torch.rand((N5, Cw, Ht5, Ww), device="cuda", generator=g).to(torch.bfloat16) for _ in range(K5)]
                xwu_tbl, _kw3 = capi.ptr_table([t.data_ptr() for t in xwu])
                add("conv fwd bf16 %d->%d channels over tiles without halo, 8 tiles of 128x%d (one launch)" % (Cw, Cw, Ww),
                    lambda: lib.adh_conv3x3_unpadded_fwd_tiles(1, K5, N5, Cw, Cw, Ht5, Ww, xwu_tbl, ww.data_ptr(), yw_tbl,
                                                               0.0, wsw.data_ptr(), wsw_bytes, stream),
                    "mfma", flopsw, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
                add("conv bwd-data bf16 %d->%d channels into tiles without halo (beta=0, one launch)" % (Cw, Cw),
                    lambda: lib.adh_conv3x3_unpadded_bwd_data_tiles(1, K5, N5, Cw, Cw, Ht5, Ww, ww.data_ptr(), yw_tbl, xwu_tbl,
                                                                    0.0, wsw.data_ptr(), wsw_bytes, stream),
                    "mfma", flopsw, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s")
                del xwu
            del xw, yw, wsw
        # ---- the shapes the reference's own microbenchmarks time, with its own figures of merit ----
        # tools/microbench_spatial.cc:23-28: halo exchange, fp32 N=32, C=64, W=256, H=256/ndev, p=1 (ndev = 4 tiles);
        # it prints p*W*C*N*4 / t (:100-103)
        Km, Nm, Wm, Hm, pm = 4, 32, 256, 256 // 4, 1
        tm = [torch.rand((Nm, C, Hm + 2 * pm, Wm + 2 * pm), device="cuda", generator=g) for _ in range(Km)]
        tm_tbl, _km = capi.ptr_table([t.data_ptr() for t in tm])
        strip_m = pm * Wm * C * Nm * 4
        reps, wu = 200, 20
        add("reference microbench_spatial: halo exchange, N=32 C=64 W=256 H=64 per tile, p=1, 4 tiles",
            lambda: lib.adh_halo_exchange_nchw(0, 1, Km, pm, Wm, Hm, C, Nm, tm_tbl, stream),
            "hbm", 2 * 2 * (Km - 1) * strip_m, HBM_PEAK_GBS, "GB/s", graph=True,
            extra=lambda ms: {"reference_figure_GBs": round(strip_m / (ms * 1e-3) / 1e9, 3),
                              "reference_figure": "p*W*C*N*4 / t (tools/microbench_spatial.cc:100-101)"})
        del tm
        # tools/microbench_spatial_conv.cc:25-41: N=32, C=64, a 512x512 image in ndev row-tiles (4 tiles of 128 rows),
        # 3x3 convolution with dilation 3 over halo 3: halo exchange, halo reduce (:227-269), conv forward and
        # backward (:384-387, 473-476; it prints average milliseconds)
        Kd, Nd, Wd, Hd, pd = 4, 32, 512, 512 // 4, 3
        geo_d = (3, 3, 1, 1, 3, 3)
        HPd, WPd = Hd + 2 * pd, Wd + 2 * pd
        xd = [torch.rand((Nd, C, HPd, WPd), device="cuda", generator=g) * 2 - 1 for _ in range(Kd)]
        yd = [torch.empty((Nd, C, Hd, Wd), device="cuda") for _ in range(Kd)]
        gd = [torch.zeros((Nd, C, HPd, WPd), device="cuda") for _ in range(Kd)]
        wd = torch.randn((C, C, 3, 3), device="cuda", generator=g) * (2.0 / (C * 9)) ** 0.5
        gwd = torch.empty_like(wd)
        xd_tbl, _kd1 = capi.ptr_table([t.data_ptr() for t in xd])
        yd_tbl, _kd2 = capi.ptr_table([t.data_ptr() for t in yd])
        gd_tbl, _kd3 = capi.ptr_table([t.data_ptr() for t in gd])
        wsd_bytes = max(lib.adh_conv2d_workspace_bytes(wh, 0, Kd, Nd, C, C, HPd, WPd, *geo_d) for wh in (0, 1, 2))
        wsd = torch.empty(wsd_bytes // 4 + 64, device="cuda")
        strip_d = pd * Wd * C * Nd * 4
        fl_d = 2.0 * Kd * Nd * C * C * 9 * Hd * Wd
        reps, wu = 100, 10
        add("reference microbench_spatial_conv: halo exchange, N=32 C=64 512x128 per tile, p=3, 4 tiles",
            lambda: lib.adh_halo_exchange_nchw(0, 1, Kd, pd, Wd, Hd, C, Nd, xd_tbl, stream),
            "hbm", 2 * 2 * (Kd - 1) * strip_d, HBM_PEAK_GBS, "GB/s",
            extra=lambda ms: {"reference_figure_GBs": round(strip_d / (ms * 1e-3) / 1e9, 3)})
        add("reference microbench_spatial_conv: halo reduce, same tiles",
            lambda: lib.adh_halo_reduce_nchw(0, 1, Kd, pd, Wd, Hd, C, Nd, gd_tbl, stream),
            "hbm", 3 * 2 * (Kd - 1) * strip_d, HBM_PEAK_GBS, "GB/s",
            extra=lambda ms: {"reference_figure_GBs": round(strip_d / (ms * 1e-3) / 1e9, 3)})
        reps, wu = 10, 3
        add("reference microbench_spatial_conv: conv fwd 3x3 dilation 3 over halo 3 (fp32, 4 tiles; the 3x3 kernel with its taps three apart)",
            lambda: lib.adh_conv2d_slab_fwd_tiles(0, Kd, Nd, C, C, HPd, WPd, *geo_d, xd_tbl, wd.data_ptr(), yd_tbl, 0.0,
                                                  wsd.data_ptr(), wsd_bytes, stream),
            "mfma", fl_d, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
        add("reference microbench_spatial_conv: conv bwd-filter, same shape",
            lambda: lib.adh_conv2d_slab_bwd_filter_tiles(0, Kd, Nd, C, C, HPd, WPd, *geo_d, xd_tbl, yd_tbl, gwd.data_ptr(),
                                                         0.0, wsd.data_ptr(), wsd_bytes, stream),
            "mfma", fl_d, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
        add("reference microbench_spatial_conv: conv bwd-data, same shape",
            lambda: lib.adh_conv2d_slab_bwd_data_tiles(0, Kd, Nd, C, C, HPd, WPd, *geo_d, wd.data_ptr(), yd_tbl, gd_tbl,
                                                       0.0, wsd.data_ptr(), wsd_bytes, stream),
            "mfma", fl_d, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
        del xd, yd, gd, wsd
        # tools/microbench_conv.cc:30-54: one device, N=32, 64 -> 64 channels, 3x3 over a 64(+2) x 128(+2) slab,
        # "est flops" 2*N*Co*Ci*H*W*9 = 9.66 GF (:53)
        Nc, Hc, Wc = 32, 64, 128
        xc = torch.rand((Nc, C, Hc + 2, Wc + 2), device="cuda", generator=g) * 2 - 1
        yc_ = torch.empty((Nc, C, Hc, Wc), device="cuda")
        fl_c = 2.0 * Nc * C * C * 9 * Hc * Wc
        reps, wu = 100, 20
        add("reference microbench_conv: conv fwd 3x3, N=32 64->64, 64(+2)x128(+2) slab (fp32, one tile)",
            lambda: lib.adh_conv3x3_slab_fwd(0, Nc, C, C, Hc, Wc, xc.data_ptr(), wd.data_ptr(), yc_.data_ptr(), 0.0,
                                             None, 0, stream),
            "mfma", fl_c, MFMA_F32_PEAK_TFLOPS, "TFLOP/s",
            extra={"kernel": capi.conv_kernel_name(capi.ADH_CONV_FWD, capi.ADH_F32, 1, Nc, C, C, Hc, Wc)})
        del xc, yc_
        # column halos (a K x 1 grid, src/kernels/spatial.cu:654-731): cfg1's tensor split into 4 column-tiles
        # of 14 columns; a strip is p*H*C*N elements at row pitch
        Wk, Hk = W // K, H
        tk = [torch.rand((N, C, Hk + 2 * p, Wk + 2 * p), device="cuda", generator=g) for _ in range(K)]
        tk_tbl, _kk = capi.ptr_table([t.data_ptr() for t in tk])
        strip_k = p * Hk * C * N * es
        reps, wu = 200, 20
        add("column halo exchange (4 x 1 grid of 14-column tiles of cfg1's tensor, 6 strips)",
            lambda: lib.adh_halo_exchange_nchw(0, K, 1, p, Wk, Hk, C, N, tk_tbl, stream),
            "hbm", 2 * 2 * (K - 1) * strip_k, HBM_PEAK_GBS, "GB/s", graph=True)
        add("column halo reduce (same tiles)",
            lambda: lib.adh_halo_reduce_nchw(0, K, 1, p, Wk, Hk, C, N, tk_tbl, stream),
            "hbm", 3 * 2 * (K - 1) * strip_k, HBM_PEAK_GBS, "GB/s", graph=True)
        del tk
        # pooling over the padded slab: the 3x3 stride-2 max pooling of a residual network's stem,
        # 112x112 in 4 row-tiles of 28 rows with halo 1 -> 14x56 per tile
        Hq, Wq = 28 + 2, 112 + 2
        OHq, OWq = (Hq - 3) // 2 + 1, (Wq - 3) // 2 + 1
        xq = [torch.rand((N, C, Hq, Wq), device="cuda", generator=g) for _ in range(K)]
        yq = [torch.empty((N, C, OHq, OWq), device="cuda") for _ in range(K)]
        dq = [torch.randn((N, C, OHq, OWq), device="cuda", generator=g) for _ in range(K)]
        gq = [torch.empty((N, C, Hq, Wq), device="cuda") for _ in range(K)]
        xq_tbl, _kq1 = capi.ptr_table([t.data_ptr() for t in xq])
        yq_tbl, _kq2 = capi.ptr_table([t.data_ptr() for t in yq])
        dq_tbl, _kq3 = capi.ptr_table([t.data_ptr() for t in dq])
        gq_tbl, _kq4 = capi.ptr_table([t.data_ptr() for t in gq])
        in_b, out_b = K * N * C * Hq * Wq * 4, K * N * C * OHq * OWq * 4
        reps, wu = 100, 10
        add("max pool 3x3 s2 fwd over padded tiles (fp32, 4 tiles of 30x114)",
            lambda: lib.adh_pool2d_slab_fwd_tiles(0, 1, K, N, C, Hq, Wq, 3, 3, 2, 2, xq_tbl, yq_tbl, stream),
            "hbm", in_b + out_b, HBM_PEAK_GBS, "GB/s")
        add("max pool 3x3 s2 bwd over padded tiles (fp32)",
            lambda: lib.adh_pool2d_slab_bwd_tiles(0, 1, K, N, C, Hq, Wq, 3, 3, 2, 2, xq_tbl, yq_tbl, dq_tbl, gq_tbl,
                                                  0.0, stream),
            "hbm", 2 * in_b + out_b, HBM_PEAK_GBS, "GB/s", note="reads x and dy, writes dx; y is not read")
        # the same pooling over tiles without halo (no pad, exchange, reduce or unpad pass around it)
        xqu = [torch.rand((N, C, 28, 112), device="cuda", generator=g) for _ in range(K)]
        gqu = [torch.empty((N, C, 28, 112), device="cuda") for _ in range(K)]
        xqu_tbl, _kq5 = capi.ptr_table([t.data_ptr() for t in xqu])
        gqu_tbl, _kq6 = capi.ptr_table([t.data_ptr() for t in gqu])
        in_u = K * N * C * 28 * 112 * 4
        add("max pool 3x3 s2 fwd over tiles without halo (fp32, 4 tiles of 28x112; pad, exchange and pooling in one launch)",
            lambda: lib.adh_pool2d_unpadded_fwd_tiles(0, 1, K, N, C, 28, 112, 3, 3, 2, 2, 1, 1, xqu_tbl, yq_tbl, stream),
            "hbm", in_u + out_b, HBM_PEAK_GBS, "GB/s")
        add("max pool 3x3 s2 bwd into tiles without halo (fp32; pooling backward, halo reduce and unpad in one launch)",
            lambda: lib.adh_pool2d_unpadded_bwd_tiles(0, 1, K, N, C, 28, 112, 3, 3, 2, 2, 1, 1, xqu_tbl, yq_tbl, dq_tbl, gqu_tbl,
                                                      0.0, stream),
            "hbm", 2 * in_u + out_b, HBM_PEAK_GBS, "GB/s")
        del xq, yq, dq, gq, xqu, gqu
        # the 3x3 kernels and the general kernels over tiles without halo, at the shapes of the spatially-parallel
        # ResNet-18 (batch 32, 4 row tiles): a 64-channel 3x3 on 32x128 tiles, the stride-2 3x3 64 -> 128 on the same
        # tiles and 256 -> 512 on 8x32 tiles (kernels of their own for backward-data, backward-filter and, from 256 input
        # channels on, forward), and a 512-channel 3x3 on 4x16 tiles (the general kernels; padded tiles of 6x18 hold 1.7 times the pixels)
        for (nm, Ci, Co, Hu, Wu, su) in (("3x3 64->64 on 32x128 tiles", 64, 64, 32, 128, 1), ("3x3 stride 2 64->128 on 32x128 tiles", 64, 128, 32, 128, 2),
                                         ("3x3 stride 2 256->512 on 8x32 tiles", 256, 512, 8, 32, 2), ("3x3 512->512 on 4x16 tiles", 512, 512, 4, 16, 1)):
            OHu, OWu = Hu // su, (Wu + 2 - 3) // su + 1
            xu = [torch.randn((N, Ci, Hu, Wu), device="cuda", generator=g) for _ in range(K)]
            yu = [torch.randn((N, Co, OHu, OWu), device="cuda", generator=g) for _ in range(K)]
            wu_ = torch.randn((Co, Ci, 3, 3), device="cuda", generator=g) * (2.0 / (Ci * 9)) ** 0.5
            gwu = torch.empty((Co, Ci, 3, 3), device="cuda")
            xu_tbl, _ku1 = capi.ptr_table([t.data_ptr() for t in xu])
            yu_tbl, _ku2 = capi.ptr_table([t.data_ptr() for t in yu])
            small = su == 1 and Hu * Wu > 64  # the 3x3 kernels serve it; else the general ones
            wsb = max([lib.adh_conv2d_unpadded_workspace_bytes(wh, 0, K, N, Ci, Co, Hu, Wu, 3, 3, su, su, 1, 1, 1, 1) for wh in (0, 1, 2)] +
                      [lib.adh_conv3x3_workspace_bytes(2, 0, K, N, Ci, Co, Hu, Wu)])
            wsu = torch.empty(wsb // 4 + 64, device="cuda")
            flop = 2.0 * K * N * Ci * Co * 9 * OHu * OWu
            reps, wu = 50, 10
            if small:
                f = lambda: lib.adh_conv3x3_unpadded_fwd_tiles(0, K, N, Ci, Co, Hu, Wu, xu_tbl, wu_.data_ptr(), yu_tbl, 0.0, None, 0, stream)
                b = lambda: lib.adh_conv3x3_unpadded_bwd_data_tiles(0, K, N, Ci, Co, Hu, Wu, wu_.data_ptr(), yu_tbl, xu_tbl, 0.0, None, 0, stream)
            else:
                f = lambda: lib.adh_conv2d_unpadded_fwd_tiles(0, K, N, Ci, Co, Hu, Wu, 3, 3, su, su, 1, 1, 1, 1, xu_tbl, wu_.data_ptr(), yu_tbl,
                                                              0.0, wsu.data_ptr(), wsb, stream)
                b = lambda: lib.adh_conv2d_unpadded_bwd_data_tiles(0, K, N, Ci, Co, Hu, Wu, 3, 3, su, su, 1, 1, 1, 1, wu_.data_ptr(), yu_tbl,
                                                                   xu_tbl, 0.0, wsu.data_ptr(), wsb, stream)
            if su == 1:
                wgf = lambda: lib.adh_conv3x3_unpadded_bwd_filter_tiles(0, K, N, Ci, Co, Hu, Wu, xu_tbl, yu_tbl, gwu.data_ptr(), 0.0,
                                                                        wsu.data_ptr(), wsb, stream)
            else:
                wgf = lambda: lib.adh_conv2d_unpadded_bwd_filter_tiles(0, K, N, Ci, Co, Hu, Wu, 3, 3, su, su, 1, 1, 1, 1, xu_tbl, yu_tbl,
                                                                       gwu.data_ptr(), 0.0, wsu.data_ptr(), wsb, stream)
            add("conv fwd over tiles without halo, fp32, N=32, 4 tiles: " + nm, f, "mfma", flop, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
            add("conv bwd-data into tiles without halo, fp32: " + nm, b, "mfma", flop, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
            add("conv bwd-filter over tiles without halo, fp32: " + nm, wgf, "mfma", flop, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
            del xu, yu, wu_, gwu, wsu
        # the 1x1 stride-2 projection shortcuts of the same net (matrix-product kernels of their own): the first is
        # sized by memory (priced by the bytes of the pixels it uses and writes), the third by the matrix cores
        for (Ci, Co, Hu, Wu, bound) in ((64, 128, 32, 128, "hbm"), (256, 512, 8, 32, "mfma")):
            OHu, OWu = Hu // 2, Wu // 2
            xu = [torch.randn((N, Ci, Hu, Wu), device="cuda", generator=g) for _ in range(K)]
            yu = [torch.randn((N, Co, OHu, OWu), device="cuda", generator=g) for _ in range(K)]
            wu_ = torch.randn((Co, Ci, 1, 1), device="cuda", generator=g) * (2.0 / Ci) ** 0.5
            gwu = torch.empty((Co, Ci, 1, 1), device="cuda")
            xu_tbl, _ku1 = capi.ptr_table([t.data_ptr() for t in xu])
            yu_tbl, _ku2 = capi.ptr_table([t.data_ptr() for t in yu])
            geo1 = (1, 1, 2, 2, 1, 1)
            wsb = max(lib.adh_conv2d_workspace_bytes(wh, 0, K, N, Ci, Co, Hu, Wu, *geo1) for wh in (0, 1, 2))
            wsu = torch.empty(wsb // 4 + 64, device="cuda")
            flop = 2.0 * K * N * Ci * Co * OHu * OWu
            used = 4.0 * K * N * (Ci + Co) * OHu * OWu               # sampled pixels of x + y
            grad = 4.0 * K * N * (Ci * Hu * Wu + Co * OHu * OWu)     # dy read, the whole of dx written
            reps, wu = 50, 10
            nm = "1x1 stride 2 %d->%d on %dx%d tiles, fp32, N=32, 4 tiles" % (Ci, Co, Hu, Wu)
            price = (lambda b: (b, HBM_PEAK_GBS, "GB/s")) if bound == "hbm" else (lambda b: (flop, MFMA_F32_PEAK_TFLOPS, "TFLOP/s"))
            add("conv fwd " + nm,
                lambda: lib.adh_conv2d_slab_fwd_tiles(0, K, N, Ci, Co, Hu, Wu, *geo1, xu_tbl, wu_.data_ptr(), yu_tbl, 0.0,
                                                      wsu.data_ptr(), wsb, stream), bound, *price(used))
            add("conv bwd-data " + nm,
                lambda: lib.adh_conv2d_slab_bwd_data_tiles(0, K, N, Ci, Co, Hu, Wu, *geo1, wu_.data_ptr(), yu_tbl, xu_tbl, 0.0,
                                                           wsu.data_ptr(), wsb, stream), bound, *price(grad))
            add("conv bwd-filter " + nm + " (2 kernels)",
                lambda: lib.adh_conv2d_slab_bwd_filter_tiles(0, K, N, Ci, Co, Hu, Wu, *geo1, xu_tbl, yu_tbl, gwu.data_ptr(), 0.0,
                                                             wsu.data_ptr(), wsb, stream), bound, *price(used))
            del xu, yu, wu_, gwu, wsu
        # batch norm with tile-local statistics + rectifier + halo pad in one call (the BN -> ReLU -> HaloPad
        # prefix of the spatially-parallel residual block) on cfg1's 4 tiles, and its backward
        xb = [torch.randn((N, C, Ht, W), device="cuda", generator=g) + 0.5 for _ in range(K)]
        sc = [torch.rand(C, device="cuda", generator=g) + 0.5 for _ in range(K)]
        sh = [torch.rand(C, device="cuda", generator=g) - 0.5 for _ in range(K)]
        sm = [torch.empty(C, device="cuda") for _ in range(K)]
        si = [torch.empty(C, device="cuda") for _ in range(K)]
        dsc = [torch.empty(C, device="cuda") for _ in range(K)]
        dsh = [torch.empty(C, device="cuda") for _ in range(K)]
        dxb = [torch.empty((N, C, Ht, W), device="cuda") for _ in range(K)]
        tabs = {k: capi.ptr_table([t.data_ptr() for t in v]) for k, v in
                (("x", xb), ("sc", sc), ("sh", sh), ("sm", sm), ("si", si), ("dsc", dsc), ("dsh", dsh), ("dx", dxb))}
        bn_ws_bytes = lib.adh_batchnorm2d_workspace_bytes(K, N, C)
        bn_ws = torch.empty(bn_ws_bytes // 4, device="cuda")
        packed_b = K * N * C * Ht * W * 4
        reps, wu = 100, 10
        add("batch norm (training) + relu + halo pad fwd, cfg1 tiles (2 kernels)",
            lambda: lib.adh_batchnorm2d_fwd_tiles(0, 1, K, N, C, Ht, W, 1e-5, 1, 1, tabs["x"][0], tabs["sc"][0], tabs["sh"][0],
                                                  None, None, tile_tbl, None, None, tabs["sm"][0], tabs["si"][0],
                                                  bn_ws.data_ptr(), bn_ws_bytes, stream),
            "hbm", 2 * packed_b + padded_b, HBM_PEAK_GBS, "GB/s", note="x read for the statistics and again to normalise")
        add("batch norm + relu + halo unpad bwd, cfg1 tiles (2 kernels)",
            lambda: lib.adh_batchnorm2d_bwd_tiles(0, K, N, C, Ht, W, 1, 1, tabs["x"][0], g_tbl, tabs["sc"][0], tabs["sh"][0],
                                                  tabs["sm"][0], tabs["si"][0], tabs["dx"][0], tabs["dsc"][0], tabs["dsh"][0],
                                                  0.0, 0.0, bn_ws.data_ptr(), bn_ws_bytes, stream),
            "hbm", 2 * (packed_b + packed_b) + packed_b, HBM_PEAK_GBS, "GB/s",
            note="x and the interior of dy read twice (sums, then gradient), dx written")
        del xb, dxb
        # slab conv of any window (fp32 matrix cores): the 7x7 stride-2 stem over halo 3 (3 -> 64 channels, 224x224 in 4
        # row-tiles), the stride-1 stem of the spatially-parallel net (256x256 in 4 row-tiles; forward and backward-filter
        # of both by the kernels for at most three input channels) and a stride-2 3x3 (64 -> 128 channels) over cfg1's tiles
        for label, Ci, Co, Hs, Ws, ph, geo in (("7x7 s2 stem 3->64, 4 tiles of 62x230", 3, 64, 56, 224, 3, (7, 7, 2, 2, 1, 1)),
                                               ("7x7 s1 stem 3->64, 4 tiles of 70x262 (the parallel net's)", 3, 64, 64, 256, 3, (7, 7, 1, 1, 1, 1)),
                                               ("3x3 s2 64->128, 4 tiles of 16x58", 64, 128, 14, 56, 1, (3, 3, 2, 2, 1, 1))):
            HPs, WPs = Hs + 2 * ph, Ws + 2 * ph
            OHs = (HPs - ((geo[0] - 1) * geo[4] + 1)) // geo[2] + 1
            OWs = (WPs - ((geo[1] - 1) * geo[5] + 1)) // geo[3] + 1
            xg = [torch.rand((N, Ci, HPs, WPs), device="cuda", generator=g) * 2 - 1 for _ in range(K)]
            wg = torch.randn((Co, Ci, geo[0], geo[1]), device="cuda", generator=g) * (2.0 / (Ci * geo[0] * geo[1])) ** 0.5
            yg = [torch.empty((N, Co, OHs, OWs), device="cuda") for _ in range(K)]
            gg = [torch.empty((N, Ci, HPs, WPs), device="cuda") for _ in range(K)]
            gwg = torch.empty_like(wg)
            xg_tbl, _kg1 = capi.ptr_table([t.data_ptr() for t in xg])
            yg_tbl, _kg2 = capi.ptr_table([t.data_ptr() for t in yg])
            gg_tbl, _kg3 = capi.ptr_table([t.data_ptr() for t in gg])
            wsg_bytes = max(lib.adh_conv2d_workspace_bytes(wh, 0, K, N, Ci, Co, HPs, WPs, *geo) for wh in (0, 1, 2))
            wsg = torch.empty(wsg_bytes // 4 + 64, device="cuda")
            fl = 2.0 * K * N * Co * Ci * geo[0] * geo[1] * OHs * OWs
            reps, wu = 30, 5
            add("general conv fwd " + label,
                lambda: lib.adh_conv2d_slab_fwd_tiles(0, K, N, Ci, Co, HPs, WPs, *geo, xg_tbl, wg.data_ptr(), yg_tbl, 0.0,
                                                      wsg.data_ptr(), wsg_bytes, stream),
                "mfma", fl, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
            add("general conv bwd-data " + label,
                lambda: lib.adh_conv2d_slab_bwd_data_tiles(0, K, N, Ci, Co, HPs, WPs, *geo, wg.data_ptr(), yg_tbl, gg_tbl,
                                                           0.0, wsg.data_ptr(), wsg_bytes, stream),
                "mfma", fl, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
            add("general conv bwd-filter " + label,
                lambda: lib.adh_conv2d_slab_bwd_filter_tiles(0, K, N, Ci, Co, HPs, WPs, *geo, xg_tbl, yg_tbl, gwg.data_ptr(),
                                                             0.0, wsg.data_ptr(), wsg_bytes, stream),
                "mfma", fl, MFMA_F32_PEAK_TFLOPS, "TFLOP/s")
            del xg, yg, gg, wsg

        # the optimizer's flat vectors at ResNet-18's parameter count (11.69 M floats), gradients of 4 ranks
        res18 = [(64, 3, 7, 7)]
        for cin, cout, first in ((64, 64, False), (64, 128, True), (128, 256, True), (256, 512, True)):
            for blk in range(2):
                ci = cin if blk == 0 else cout
                res18 += [(ci,), (ci,), (cout, ci, 3, 3), (cout,), (cout,), (cout, cout, 3, 3)]
                if blk == 0 and first:
                    res18 += [(cout, ci, 1, 1)]
        res18 += [(512,), (512,), (1000, 512), (1000,)]
        p_arrays = [torch.randn(sh, device="cuda", generator=g) * 0.05 for sh in res18]
        pdim = sum(a.numel() for a in p_arrays)
        flat_p = torch.empty(pdim, device="cuda")
        flat_m = torch.zeros(pdim, device="cuda")
        flat_lag = torch.empty(pdim, device="cuda")
        flat_g = [torch.randn(pdim, device="cuda", generator=g) * 1e-3 for _ in range(K)]
        pa_tbl, _kp1 = capi.ptr_table([a.data_ptr() for a in p_arrays])
        pa_len = (ctypes.c_uint64 * len(p_arrays))(*[a.numel() for a in p_arrays])
        fg_tbl, _kp2 = capi.ptr_table([t.data_ptr() for t in flat_g])
        reps, wu = 50, 10
        add("flat store: %d parameter arrays -> one vector of %d floats" % (len(p_arrays), pdim),
            lambda: lib.adh_flat_store_f32(len(p_arrays), pa_tbl, pa_len, 0, flat_p.data_ptr(), stream),
            "hbm", 2.0 * pdim * 4, HBM_PEAK_GBS, "GB/s", flushed=True, graph=True)
        add("flat load: one vector -> %d parameter arrays" % len(p_arrays),
            lambda: lib.adh_flat_load_f32(len(p_arrays), pa_tbl, pa_len, 0, flat_p.data_ptr(), stream),
            "hbm", 2.0 * pdim * 4, HBM_PEAK_GBS, "GB/s", flushed=True, graph=True)
        add("sgd step (4 rank gradients summed + l2 + Nesterov momentum + lagged copy, one pass)",
            lambda: lib.adh_sgd_step_f32(pdim, K, fg_tbl, 1e-4, 0.9, 0.1, 0.1, 1, flat_p.data_ptr(), flat_m.data_ptr(),
                                         flat_lag.data_ptr(), None, stream),
            "hbm", (K + 2 + 3) * pdim * 4.0, HBM_PEAK_GBS, "GB/s", flushed=True,
            note="reads 4 gradient vectors + parameters + momentum, writes momentum + parameters + lagged copy")
        del p_arrays, flat_g, flush_scratch
        if reference_microbench is not None:
            # wall-clock milliseconds per trial of the reference's call sequence (synchronisations included), beside
            # the same work as one launch for all tiles; the device-event figures of the one-launch forms are the
            # "reference microbench_*" entries above
            for m in reference_microbench:
                m = dict(m)
                which = m.pop("which")
                if which == "conv":
                    m["name"] = "reference microbench_conv (C++ binary, one device, wall clock of launch + synchronise): %s" % m["name"]
                else:
                    m["name"] = "reference microbench_%s through Spatial2DComm (C++ binary, 4 ranks, wall clock): %s" % (which, m["name"])
                sec.append(m)
        out["secondary"] = sec
        # The halo half of the metric inside `roofline`: pack / unpack at the headline configuration (1.08 GB per
        # launch, four times the on-package cache: the sustained HBM rate) and at cfg1 (56 MB: `warm` has its operands
        # resident in the on-package cache, `flushed` reads 512 MB of something else before every launch).
        by_name = {e["name"]: e for e in sec}

        def halo_entry(name):
            e = by_name.get(name)
            if e is None:
                return None
            h = {"ms": e["ms"], "GBs": e["achieved"], "frac": e["frac"], "bytes": e["work"]}
            if "ms_flushed" in e:
                h = {"warm": h, "flushed": {"ms": e["ms_flushed"], "GBs": e["achieved_flushed"], "frac": e["frac_flushed"],
                                            "bytes": e["work"]}}
            return h

        out["roofline"]["halo"] = {
            "bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "pack_cfg5": halo_entry("halo pack cfg5 (bf16, 8 tiles of 128 rows)"),
            "unpack_cfg5": halo_entry("halo unpack cfg5 (bf16)"),
            "pack_cfg1": halo_entry("halo pack cfg1 (unsplit -> 4 padded tiles)"),
            "unpack_cfg1": halo_entry("halo unpack cfg1 (4 padded tiles -> unsplit)")}
    if end_to_end is not None:
        out["end_to_end"] = end_to_end

    # ---- CPU baseline: the scalar port on this host, one thread and one thread per tile, on a bounded sample ----
    if not args.no_cpu:
        import oracle
        cores_on_box = oracle.hardware_threads()
        # The sample: the first 48 output rows of image 0 of every one of the 8 tiles of the headline workload (same
        # filter, same bf16 values widened to fp32: exact products, fp32 sums, the arithmetic the kernel does):
        # 8 tiles x 64 x 64 x 9 x 48 x 2048 x 2 = 58 GFLOP per pass, 10-15 s on one host thread.  The secondary entries above have written into
        # the tiles: pack and convolve once more so that the CPU and the GPU work on the same input.
        capi.check(lib.adh_tiles_pack_nchw(1, K5, 1, W5, H5, C, N5, X5.data_ptr(), t5_tbl, stream), "pack cfg5")
        capi.check(conv_fwd5(), "conv fwd cfg5")
        torch.cuda.synchronize()
        rows = 48
        wn5 = w5.float().cpu().numpy()
        host_x5 = [np.ascontiguousarray(t[0:1, :, 0:rows + 2, :].float().cpu().numpy()) for t in t5]
        host_y5 = [np.empty((1, C, rows, W5), np.float32) for _ in range(K5)]
        sample_flops = 2.0 * K5 * C * C * 9 * rows * W5
        t0 = time.perf_counter()
        for r in range(K5):
            oracle.conv_slab_fwd_f32(host_x5[r], wn5, host_y5[r])
        dt1 = time.perf_counter() - t0
        err = max(float(np.abs(host_y5[r] - y5[r][0:1, :, 0:rows].float().cpu().numpy()).max() / np.abs(host_y5[r]).max())
                  for r in range(K5))
        t0 = time.perf_counter()
        oracle.conv_slab_fwd_f32_threaded(host_x5, wn5, host_y5)
        dtk = time.perf_counter() - t0
        out["cpu_baseline"] = {
            "value": round(sample_flops / dt1 / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "cores_on_box": cores_on_box,
            "value_thread_per_tile": round(sample_flops / dtk / 1e12, 6), "threads_thread_per_tile": K5,
            "sample": "rows 0-%d of image 0 of each of the 8 tiles of the headline workload (%.1f GFLOP): scalar fp32 "
                      "direct conv of the widened bf16 values, gcc -O2, %.2f s on one thread, %.2f s with one thread "
                      "per tile; GPU result (bf16) agrees to rel-err %.1e" % (rows - 1, sample_flops / 1e9, dt1, dtk, err)}
        # the reference kernels' own loop structure (idx -> (w,c,n) by div/mod) on cfg1: halo exchange, halo pack
        # (scatter + pad + exchange) and unpack (unpad + gather), one thread and one thread per rank
        capi.check(capi.tiles_pack(K, p, W, H, C, N, X, tiles), "pack")
        torch.cuda.synchronize()
        host_tiles = [t.cpu().numpy() for t in tiles]
        host_X = X.cpu().numpy()
        host_Y = np.empty_like(host_X)
        unsplit_b = N * C * H * W * 4
        padded_b = K * N * C * (Ht + 2 * p) * (W + 2 * p) * 4

        def cpu_time(fn, reps_cpu):
            t0 = time.perf_counter()
            for _ in range(reps_cpu):
                fn()
            return (time.perf_counter() - t0) / reps_cpu

        exch_b = 2 * 2 * (K - 1) * p * W * C * N * 4
        cb = out["cpu_baseline"]
        cb["halo_exchange_GBs"] = round(exch_b / cpu_time(lambda: oracle.halo_op(oracle.EXCH, 1, K, p, W, Ht, C, N, host_tiles), 20) / 1e9, 3)
        cb["halo_exchange_GBs_thread_per_rank"] = round(
            exch_b / cpu_time(lambda: oracle.halo_op_threaded(oracle.EXCH, 1, K, p, W, Ht, C, N, host_tiles), 20) / 1e9, 3)
        cb["halo_pack_GBs"] = round((unsplit_b + padded_b) / cpu_time(lambda: oracle.tiles_pack(K, p, W, H, C, N, host_X, host_tiles), 3) / 1e9, 3)
        cb["halo_pack_GBs_thread_per_rank"] = round(
            (unsplit_b + padded_b) / cpu_time(lambda: oracle.tiles_pack_threaded(K, p, W, H, C, N, host_X, host_tiles), 3) / 1e9, 3)
        cb["halo_unpack_GBs"] = round(2 * unsplit_b / cpu_time(lambda: oracle.tiles_unpack(K, p, W, H, C, N, host_tiles, host_Y), 3) / 1e9, 3)
        assert np.array_equal(host_Y, host_X)
        cb["halo_unpack_GBs_thread_per_rank"] = round(
            2 * unsplit_b / cpu_time(lambda: oracle.tiles_unpack_threaded(K, p, W, H, C, N, host_tiles, host_Y), 3) / 1e9, 3)
        assert np.array_equal(host_Y, host_X)
        cb["threads_thread_per_rank"] = K

    print(json.dumps(out))


if __name__ == "__main__":
    main()
