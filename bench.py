#!/usr/bin/env python3
"""Benchmark of the lowered-operator hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--ops]

A step is one forward pass of the ResNet-18 launch plan (fp32, batch 64, [64,3,224,224] input,
seeded synthetic weights/input already resident in HBM) enqueued on one stream through the C ABI.
Prints ONE JSON line: whole-job throughput (img/s), the roofline position of the dominant kernel
(the 3x3/1 convolution of layer1 -- the Winograd kernel the plan runs, with the implicit-GEMM kernel beside it --
timed with events on the launch stream), per-layer and
per-operator figures, and the single-core CPU baseline (the CPU checker in oracle/, timed on a
bounded sample: one image).
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def _event_time_ms(torch, fn, iters, warmup):
    """Average duration of fn() in ms, HIP events recorded on the stream fn launches on."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def _graph_time_ms(torch, fn, launches=20, replays=10):
    """Average duration of fn() in ms for kernels shorter than the host can enqueue them (a few microseconds):
    `launches` calls are captured into one HIP graph, and replays of that graph are timed with HIP events."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        fn()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(launches):
                fn()
        graph.replay()
        stream.synchronize()
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(replays):
            graph.replay()
        stop.record(stream)
        stream.synchronize()
    return start.elapsed_time(stop) / (launches * replays)


def _profiled_traffic_bytes(name):
    """HBM bytes per launch of the dominant kernel, as measured with the rocprofv3 FETCH_SIZE and
    WRITE_SIZE passes whose summary is kept beside this file (counters cannot be read from inside a run)."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", name)
    try:
        for line in open(path):
            if line.startswith("TRAFFIC_BYTES_PER_LAUNCH="):
                return int(line.split("=", 1)[1])
    except OSError:
        pass
    return None


def bench_generated(torch, pkg, hostapi, synth, dev, np, batch, steps, warmup):
    """ResNet-18 fp32 through kernels generated from the lowered loop nests only (CompileConfig::hip_use_handwritten =
    false, no fusion: 70 launches), with the per-launch times of one run grouped by the generator's schedule.  These
    kernels keep the CPU back end's order of additions; the hand-written plan's logits serve as the check."""
    consts = [dev(c) for c in synth.resnet18_consts(4)]
    x = dev(synth.resnet18_input(4, batch))
    out = torch.empty((batch, 1000), device="cuda")
    module = hostapi.CompiledResNet18(batch, 224, "hip", use_handwritten=False, fuse=False, sync_after_run=False)
    packed = module.packed([x] + consts + [out])
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(max(1, warmup)):
        module.run_packed(packed, stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        module.run_packed(packed, stream)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    by_schedule = {}
    for name, us in module.run_timed(packed, stream):
        schedule = name.rsplit("[generated:", 1)[1].rstrip("]") if "[generated:" in name else "other"
        op = name.split()[0]
        key = "%s/%s" % (op, schedule)
        e = by_schedule.setdefault(key, {"launches": 0, "us": 0.0})
        e["launches"] += 1
        e["us"] = round(e["us"] + us, 1)
    ref = torch.empty((batch, 1000), device="cuda")
    hand = hostapi.CompiledResNet18(batch, 224, "hip", sync_after_run=True)
    hand.run_packed(hand.packed([x] + consts + [ref]), stream)
    torch.cuda.synchronize()
    got, want = out.cpu().numpy(), ref.cpu().numpy()
    err = float(np.max(np.abs(got - want) / np.maximum(1.0, np.abs(want))))
    return {"metric": "resnet18_fp32_generated_kernels_img_per_s", "value": round(batch / ms * 1e3, 1), "unit": "img/s",
            "batch": batch, "ms_per_step": round(ms, 4), "steps": steps, "warmup": warmup, "launches_per_step": len(module.launches()),
            "tile_min_units": os.environ.get("KXC_HIPGEN_TILE_MIN_UNITS", "default (65536)"),
            "by_operator_and_schedule": by_schedule,
            "max_scaled_difference_from_the_hand_written_plan": err}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--eager", action="store_true", help="time only eager plan runs (no HIP graph replay)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-layers", action="store_true", help="skip the per-layer / per-operator timings")
    ap.add_argument("--int8-only", action="store_true",
                    help="run only the quantised ResNet-18 leg (for profiling its kernels) and print its JSON")
    ap.add_argument("--generated-only", action="store_true",
                    help="run only the ResNet-18 compiled to kernels generated from its TIR (no hand-written kernel) and print its JSON")
    ap.add_argument("--cpu-full", action="store_true",
                    help="also time the CPU path on the whole batch once (minutes on one core) -> cpu_baseline.batch_seconds")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    pkg = importlib.import_module("hdkx-aicompiler_amd")
    r18 = importlib.import_module("hdkx-aicompiler_amd.resnet18")
    hostapi = importlib.import_module("hdkx-aicompiler_amd.hostapi")
    synth = pkg.synth
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    attrs = pkg.device_attributes(0)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()

    batch = args.batch
    if args.int8_only:
        print(json.dumps(bench_int8(torch, pkg, synth, dev, np, batch)))
        return
    if args.generated_only:
        print(json.dumps(bench_generated(torch, pkg, hostapi, synth, dev, np, batch, args.steps, args.warmup)))
        return
    consts_h = synth.resnet18_consts(4)
    x_h = synth.resnet18_input(4, batch)
    consts = [dev(c) for c in consts_h]
    x = dev(x_h)
    out = torch.empty((batch, 1000), device="cuda")
    # The ResNet-18 Relay graph, compiled by the C++ host layer's Compiler::Compile for the "hip" target.
    module = hostapi.CompiledResNet18(batch, 224, "hip", sync_after_run=False)
    info = {"launches": module.launches(), "workspace_bytes": module.workspace_bytes()}
    # shares of the batch the plan runs side by side on streams of their own (launches of share k end in " @share<k>")
    shares = 1 + max([int(l.rsplit("@share", 1)[1]) for l in info["launches"] if "@share" in l], default=0)
    tensors = [x] + consts + [out]
    packed = module.packed(tensors)
    stream = torch.cuda.current_stream().cuda_stream

    def timed(run_step):
        for _ in range(args.warmup):
            run_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            run_step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    # Three modes, all named in `config`:
    #  * default: what a caller who only switched the target gets -- every run re-transforms the Winograd filters
    #    from the weight pointers it is given (one extra launch), launches enqueued one by one;
    #  * frozen (the mode `value` is quoted on): the caller declares the weights fixed (FreezeConstants), the filters
    #    are transformed once, in the warm-up; timed eagerly and as one captured HIP graph per step (needs a stream
    #    other than the null stream; the first run on it is eager, the second is captured), the faster one counts;
    #  * one stream: the frozen plan compiled with hip_batch_lanes = 1, i.e. without the second share's stream.
    unfrozen_ms = timed(lambda: module.run_packed(packed, stream))
    logits_default_mode = out.detach().cpu().numpy().copy()
    module.freeze_constants(True)
    eager_ms = timed(lambda: module.run_packed(packed, stream))
    graph_ms = None
    if not args.eager:
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            module.enable_graph_replay(True)
            for _ in range(3):
                module.run_packed(packed, side.cuda_stream)
            graph_ms = timed(lambda: module.run_packed(packed, side.cuda_stream))
        torch.cuda.synchronize()
        module.enable_graph_replay(False)
    ms_per_step = min(eager_ms, graph_ms) if graph_ms is not None else eager_ms
    timed_mode = "graph" if graph_ms is not None and graph_ms < eager_ms else "eager"
    img_s = batch / (ms_per_step * 1e-3)
    flop_step = r18.flops_per_image() * batch
    logits_ok = bool(torch.isfinite(out).all().item())
    logits_timed_plan = out.detach().cpu().numpy().copy()        # what the timed plan computed (checked below)
    default_equals_timed = bool(np.array_equal(logits_default_mode.view(np.uint32), logits_timed_plan.view(np.uint32)))
    one_stream_ms = None
    if shares > 1:
        prev = os.environ.get("KXC_HIP_BATCH_LANES")
        os.environ["KXC_HIP_BATCH_LANES"] = "1"
        try:
            single = hostapi.CompiledResNet18(batch, 224, "hip", sync_after_run=False)
        finally:
            if prev is None:
                del os.environ["KXC_HIP_BATCH_LANES"]
            else:
                os.environ["KXC_HIP_BATCH_LANES"] = prev
        out1 = torch.empty_like(out)
        packed1 = single.packed([x] + consts + [out1])
        single.freeze_constants(True)
        one_stream_ms = timed(lambda: single.run_packed(packed1, stream))
        if not args.eager:
            side1 = torch.cuda.Stream()
            with torch.cuda.stream(side1):
                single.enable_graph_replay(True)
                for _ in range(3):
                    single.run_packed(packed1, side1.cuda_stream)
                one_stream_ms = min(one_stream_ms, timed(lambda: single.run_packed(packed1, side1.cuda_stream)))
            torch.cuda.synchronize()
        single.close()
        del out1
    # per-launch durations inside the network (HIP events between consecutive launches, average of 5 passes)
    in_network = None
    if not args.no_layers:
        passes = []
        for _ in range(5):
            module.run_packed(packed, stream)        # keeps the GPU busy until the timed pass starts (no idle ramp)
            passes.append(module.run_timed(packed, stream))
        in_network = [{"launch": passes[0][i][0], "us": round(sum(p[i][1] for p in passes) / len(passes), 1)}
                      for i in range(len(passes[0]))]

    # ---- dominant kernel: layer1 3x3/1 conv, [64,64,56,56] * [64,64,3,3], fused bias + ReLU
    lx = dev(synth.uniform((batch, 64, 56, 56), 4100))
    lw = dev(synth.normal((64, 64, 3, 3), 4101, float(np.sqrt(2.0 / 576))))
    lb = dev(synth.uniform((64,), 4103, -0.1, 0.1))
    ly = torch.empty((batch, 64, 56, 56), device="cuda")
    conv_flop = 2.0 * batch * 64 * 56 * 56 * 64 * 9          # multiply-adds of the direct definition, x2
    gemm_ms = _event_time_ms(torch, lambda: pkg.conv2d(lx, lw, lb, None, 1, 1, 1, True, out=ly), 30, 5)
    gemm_tflops = conv_flop / (gemm_ms * 1e-3) / 1e12
    gemm_row = {"kernel": "conv_mfma_kernel<3,3> (implicit GEMM)", "variant": pkg.conv2d_variant((batch, 64, 56, 56), (64, 64, 3, 3), 1, 1),
                "avg_launch_ms": round(gemm_ms, 4), "achieved": round(gemm_tflops, 3), "frac": round(gemm_tflops / PEAK_FP32_MFMA_TFLOPS, 4),
                "traffic": _profiled_traffic_bytes("conv3x3_layer1_bs64_counters.md") if batch == 64 else None}
    algorithmic_bytes = 4 * (2 * batch * 64 * 56 * 56 + 64 * 64 * 9 + 64)
    if pkg.conv2d_winograd_preferred((batch, 64, 56, 56), (64, 64, 3, 3)) and os.environ.get("KXC_HIP_WINOGRAD", "1") != "0":
        # the launch plan runs this layer as Winograd F(2x2,3x3): 16 multiplies per 2x2 outputs instead of 36.
        # `achieved` is the ALGORITHMIC rate (direct-definition FLOP / time); `matrix_core_*` is what the matrix
        # cores actually execute (4/9 of it), i.e. how busy the MFMA pipe is.
        lu = pkg.conv2d_winograd_transform_weights(lx.shape, lw, 1)
        conv_ms = _event_time_ms(torch, lambda: pkg.conv2d_winograd(lx, lu, lw.shape, lb, None, 1, True, out=ly), 30, 5)
        conv_tflops = conv_flop / (conv_ms * 1e-3) / 1e12
        executed = conv_flop * 16.0 / 36.0
        roofline = {"bound": "mfma", "kernel": "wino_kernel (layer1: [%d,64,56,56]x[64,64,3,3] s1 p1 +bias+relu, Winograd F(2x2,3x3))" % batch,
                    "variant": pkg.conv2d_winograd_variant(lx.shape, lw.shape),
                    "achieved": round(conv_tflops, 3), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(conv_tflops / PEAK_FP32_MFMA_TFLOPS, 4), "avg_launch_ms": round(conv_ms, 4),
                    "flop_per_launch": conv_flop,
                    "matrix_core_flop_per_launch": executed,
                    "matrix_core_tflops": round(executed / (conv_ms * 1e-3) / 1e12, 3),
                    "matrix_core_frac": round(executed / (conv_ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                    "traffic": _profiled_traffic_bytes("winograd_layer1_bs64_counters.md") if batch == 64 else None,
                    "traffic_unit": "bytes per launch (FETCH_SIZE + WRITE_SIZE, calibrated on a copy; from profiles/)",
                    "algorithmic_bytes_per_launch": algorithmic_bytes, "same_layer_implicit_gemm": gemm_row,
                    "accounting": "achieved and frac divide the OPERATOR's FLOP (2*N*O*OH*OW*C*9, every output computed) by the measured "
                                  "time; Winograd F(2x2,3x3) executes 16/36 of those multiplies, so frac can reach or pass 1 while the "
                                  "matrix cores run at matrix_core_frac of their peak"}
        if shares > 1 and batch % shares == 0:
            # what the plan does with this layer: one launch per share of the batch, side by side on streams of
            # their own between a fork and a join on the timed stream (variants chosen for `shares` equal launches)
            part = batch // shares
            side = [torch.cuda.Stream() for _ in range(shares - 1)]
            fork = torch.cuda.Event()
            done = [torch.cuda.Event() for _ in side]
            prev = pkg.set_select_lanes(shares)
            try:
                def pair():
                    cur = torch.cuda.current_stream()
                    fork.record(cur)
                    pkg.conv2d_winograd(lx[:part], lu, lw.shape, lb, None, 1, True, out=ly[:part])
                    for k, st in enumerate(side):
                        st.wait_event(fork)
                        with torch.cuda.stream(st):
                            lo = (k + 1) * part
                            pkg.conv2d_winograd(lx[lo:lo + part], lu, lw.shape, lb, None, 1, True, out=ly[lo:lo + part])
                        done[k].record(st)
                        cur.wait_event(done[k])
                pair_ms = _event_time_ms(torch, pair, 30, 5)
                part_variant = pkg.conv2d_winograd_variant(lx[:part].shape, lw.shape)
            finally:
                pkg.set_select_lanes(prev)
            roofline["side_by_side"] = {
                "what": "%d launches of [%d,64,56,56] on %d streams, fork to join: the layer as the timed plan runs it" % (shares, part, shares),
                "variant": part_variant, "ms": round(pair_ms, 4), "achieved": round(conv_flop / (pair_ms * 1e-3) / 1e12, 3),
                "frac": round(conv_flop / (pair_ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                "matrix_core_frac": round(executed / (pair_ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)}
    else:
        roofline = {"bound": "mfma", "kernel": "conv_mfma_kernel<3,3> (layer1: [%d,64,56,56]x[64,64,3,3] s1 p1 +bias+relu)" % batch,
                    "variant": gemm_row["variant"], "achieved": gemm_row["achieved"], "peak": PEAK_FP32_MFMA_TFLOPS,
                    "unit": "TFLOP/s", "frac": gemm_row["frac"], "avg_launch_ms": gemm_row["avg_launch_ms"],
                    "flop_per_launch": conv_flop, "traffic": gemm_row["traffic"],
                    "traffic_unit": "bytes per launch (FETCH_SIZE + WRITE_SIZE, calibrated on a copy; from profiles/)",
                    "algorithmic_bytes_per_launch": algorithmic_bytes}

    result = {
        "metric": "resnet18_fp32_bs%d_img_per_s" % batch, "value": round(img_s, 2), "unit": "img/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "ResNet-18 fp32 inference, batch %d, input [%d,3,224,224], BN folded, seeded Kaiming weights "
                               "(benchmark configuration %d)" % (batch, batch, 4 if batch == 64 else 3),
                   "compiled_by": "C++ host layer, Compiler::Compile(Relay graph, target hip)",
                   "constants": "frozen (serving mode: Winograd filter transforms run once, in the warm-up); "
                                "default_mode_ms_per_step is what an unchanged caller gets",
                   "timed_mode": timed_mode,
                   "default_mode_ms_per_step": round(unfrozen_ms, 4),
                   "default_mode": "constants re-read (filters re-transformed) in every run, eager launches, %d share(s) of the batch" % shares,
                   "default_mode_logits_equal_timed_bit_for_bit": default_equals_timed,
                   "one_stream_ms_per_step": round(one_stream_ms, 4) if one_stream_ms is not None else round(ms_per_step, 4),
                   "one_stream": "hip_batch_lanes = 1 (no second stream inside the plan), frozen constants, faster of eager and graph",
                   "batch_shares": shares, "launches_per_step": len(info["launches"]), "workspace_bytes": info["workspace_bytes"]},
        "end_to_end_tflops": round(flop_step / (ms_per_step * 1e-3) / 1e12, 3),
        "end_to_end_frac_of_fp32_mfma_peak": round(flop_step / (ms_per_step * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
        "logits_finite": logits_ok,
        "eager_ms_per_step": round(eager_ms, 4), "hip_graph_replay_ms_per_step": round(graph_ms, 4) if graph_ms is not None else None,
        "eager_unfrozen_ms_per_step": round(unfrozen_ms, 4),
        "device": {"name": attrs.device_name.decode(), "arch": attrs.arch.decode(), "cus": int(attrs.multi_processor_count),
                   "clock_khz": int(attrs.max_clock_rate_khz)},
        "roofline": roofline,
    }

    if in_network is not None:
        result["launches_in_network"] = in_network
    if not args.no_layers:
        result["conv_layers"] = bench_conv_layers(torch, pkg, synth, dev, batch)
        result["ops"] = bench_ops(torch, pkg, synth, dev)
        result["resnet18_bs1_img_per_s"] = bench_batch1(torch, pkg, hostapi, synth, dev)
        result["int8"] = bench_int8(torch, pkg, synth, dev, np, batch)

    if not args.no_cpu:
        result["cpu_baseline"], want_head = cpu_baseline(np, synth, x_h, consts_h)
        result["gpu_over_cpu"] = round(img_s / result["cpu_baseline"]["value"], 1)
        result["gpu_over_cpu_note"] = ("GPU batch-%d throughput over the CPU path's rate on the first %d images of the same batch "
                                       "(one scalar thread, no batch effect; --cpu-full times all %d)" % (batch, want_head.shape[0], batch))
        if args.cpu_full:
            from oracle_lib import Oracle as _Oracle
            t0 = time.perf_counter()
            full = _Oracle(fast=True).resnet18(x_h, consts_h)
            secs = time.perf_counter() - t0
            result["cpu_baseline"]["batch_seconds"] = round(secs, 2)
            result["cpu_baseline"]["batch_img_per_s"] = round(batch / secs, 4)
            result["gpu_over_cpu_same_batch"] = round(img_s / (batch / secs), 1)
            g, w = logits_timed_plan.astype(np.float64), full.astype(np.float64)
            result["parity_whole_batch_max_scaled_err"] = float(np.max(np.abs(g - w) / np.maximum(1.0, np.abs(w))))
        # parity of the TIMED plan at its real size: its logits for the first and the last image of the batch against
        # the CPU path on those images (the reference's acceptance metric, max |a-r| / max(1,|r|), and the plain
        # relative error over logits above 1 % of the largest)
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        from oracle_lib import Oracle
        checks = [(n, want_head[n:n + 1]) for n in range(want_head.shape[0])]
        if batch > want_head.shape[0]:
            checks.append((batch - 1, Oracle(fast=True).resnet18(x_h[batch - 1:batch], consts_h)))
        scaled = rel = 0.0
        for n, want in checks:
            got = logits_timed_plan[n:n + 1].astype(np.float64); want = want.astype(np.float64)
            scaled = max(scaled, float(np.max(np.abs(got - want) / np.maximum(1.0, np.abs(want)))))
            m = np.abs(want) > 1e-2 * np.max(np.abs(want))
            rel = max(rel, float(np.max(np.abs(got[m] - want[m]) / np.abs(want[m]))))
        result["parity_max_scaled_err"] = scaled
        result["parity_max_rel_err"] = rel
        result["parity_images_checked"] = [n for n, _ in checks]
        result["parity_tolerance"] = 1e-3
        result["parity_ok"] = bool(scaled <= 1e-3 and rel <= 1e-3)
    print(json.dumps(result))


CONV_LAYERS = [  # name, C, H, O, k, s, p, count per network, residual
    ("conv1", 3, 224, 64, 7, 2, 3, 1, False),
    ("layer1.3x3", 64, 56, 64, 3, 1, 1, 4, False),
    ("layer2.0.conv1", 64, 56, 128, 3, 2, 1, 1, False),
    ("layer2.3x3", 128, 28, 128, 3, 1, 1, 3, True),
    ("layer2.0.down", 64, 56, 128, 1, 2, 0, 1, False),
    ("layer3.0.conv1", 128, 28, 256, 3, 2, 1, 1, False),
    ("layer3.3x3", 256, 14, 256, 3, 1, 1, 3, True),
    ("layer3.0.down", 128, 28, 256, 1, 2, 0, 1, False),
    ("layer4.0.conv1", 256, 14, 512, 3, 2, 1, 1, False),
    ("layer4.3x3", 512, 7, 512, 3, 1, 1, 3, True),
    ("layer4.0.down", 256, 14, 512, 1, 2, 0, 1, False),
]


def bench_conv_layers(torch, pkg, synth, dev, batch):
    rows = []
    for i, (name, c, h, o, k, s, p, count, res) in enumerate(CONV_LAYERS):
        x = dev(synth.uniform((batch, c, h, h), 4200 + i))
        w = dev(synth.normal((o, c, k, k), 4300 + i, float((2.0 / (c * k * k)) ** 0.5)))
        b = dev(synth.uniform((o,), 4400 + i, -0.1, 0.1))
        oh = (h + 2 * p - k) // s + 1
        y = torch.empty((batch, o, oh, oh), device="cuda")
        skip = torch.zeros_like(y) if res else None
        ms = _event_time_ms(torch, lambda: pkg.conv2d(x, w, b, skip, s, p, 1, True, out=y), 20, 3)
        flop = 2.0 * batch * o * oh * oh * c * k * k
        row = {"layer": name, "variant": pkg.conv2d_variant((batch, c, h, h), (o, c, k, k), s, p), "count": count,
               "ms": round(ms, 4), "tflops": round(flop / (ms * 1e-3) / 1e12, 2),
               "frac_fp32_mfma_peak": round(flop / (ms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)}
        if k == 3 and s == 1 and pkg.conv2d_winograd_preferred((batch, c, h, h), (o, c, k, k), s, p):
            # what the launch plan uses for this layer; tflops = direct-definition FLOP / time
            u = pkg.conv2d_winograd_transform_weights(x.shape, w, p)
            wms = _event_time_ms(torch, lambda: pkg.conv2d_winograd(x, u, w.shape, b, skip, p, True, out=y), 20, 3)
            row["winograd"] = {"variant": pkg.conv2d_winograd_variant(x.shape, w.shape, s, p), "ms": round(wms, 4),
                               "tflops": round(flop / (wms * 1e-3) / 1e12, 2),
                               "frac_fp32_mfma_peak": round(flop / (wms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                               "matrix_core_frac": round(flop * 16.0 / 36.0 / (wms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)}
        if name == "conv1":
            row["note"] = ("launched back to back: the 205 MB of output of one launch compete with the write-back of the "
                           "launch before; inside the network the same launch takes about 0.18 ms (launches_in_network)")
        rows.append(row)
    return rows


def bench_ops(torch, pkg, synth, dev):
    """Benchmark configuration 2: the bandwidth-bound operators at ResNet-18 shapes, algorithmic bytes / time."""
    rows = []
    x = dev(synth.uniform((64, 64, 112, 112), 2000))
    y = torch.empty((64, 64, 56, 56), device="cuda")
    ms = _event_time_ms(torch, lambda: pkg.pool2d(x, 3, 2, 1, out=y), 30, 5)
    rows.append(_bw_row("maxpool3x3s2 [64,64,112,112]", 256901120, ms))
    del x, y
    a = dev(synth.uniform((64, 128, 28, 28), 2010)); b = dev(synth.uniform((64, 128, 28, 28), 2011))
    ab = torch.empty_like(a)
    ms = _graph_time_ms(torch, lambda: pkg.binary(0, a, b, relu=True, out=ab))
    row = _bw_row("add+relu [64,128,28,28], operands resident in the last-level cache", 77070336, ms)
    row["frac_of"] = "8 TB/s, but this is a LAST-LEVEL-CACHE figure: 20 launches on the same 77 MB captured in one HIP graph"
    rows.append(row)
    # HBM-cold: ten operand sets (770 MB, three times the 256 MB last-level cache) used in rotation, so every launch
    # reads its operands from HBM; 20 launches captured in one graph (the kernel is shorter than a host enqueue)
    sets = [(torch.empty_like(a).copy_(a), torch.empty_like(b).copy_(b), torch.empty_like(a)) for _ in range(10)]
    turn = [0]

    def cold():
        sa, sb, sy = sets[turn[0] % len(sets)]
        turn[0] += 1
        pkg.binary(0, sa, sb, relu=True, out=sy)
    ms = _graph_time_ms(torch, cold)
    rows.append(_bw_row("add+relu [64,128,28,28], HBM-cold (10 operand sets in rotation)", 77070336, ms))
    del sets
    g = dev(synth.uniform((64, 512, 7, 7), 2020))
    gy = torch.empty((64, 512, 1, 1), device="cuda")
    ms = _graph_time_ms(torch, lambda: pkg.global_avg_pool2d(g, out=gy))
    rows.append(_bw_row("global_avg_pool [64,512,7,7]", 6553600, ms))
    rows[-1]["timing"] = "20 launches captured in one HIP graph (the kernel is shorter than a host enqueue)"
    fa = dev(synth.uniform((64, 512), 2030)); fw = dev(synth.uniform((1000, 512), 2031)); fb = dev(synth.uniform((1000,), 2032))
    fy = torch.empty((64, 1000), device="cuda")
    ms = _graph_time_ms(torch, lambda: pkg.gemm(fa, fw, fb, out=fy))
    rows.append({"op": "dense [64,512]x[1000,512]T+bias", "timing": "20 launches captured in one HIP graph", "ms": round(ms, 4), "gflops": round(65536000 / (ms * 1e-3) / 1e9, 1),
                 "gbs": round(2439072 / (ms * 1e-3) / 1e9, 1)})
    # a plain device-to-device copy of the max-pool input size, as the achievable-bandwidth yardstick
    src = torch.empty(205520896 // 4, device="cuda"); dst = torch.empty_like(src)
    ms = _event_time_ms(torch, lambda: dst.copy_(src), 20, 3)
    rows.append(_bw_row("copy 205.5 MB (yardstick, read+write)", 2 * 205520896, ms))
    return rows


def _bw_row(name, nbytes, ms):
    gbs = nbytes / (ms * 1e-3) / 1e9
    return {"op": name, "ms": round(ms, 4), "gbs": round(gbs, 1), "frac_hbm_peak": round(gbs / PEAK_HBM_GBS, 4)}


def bench_batch1(torch, pkg, hostapi, synth, dev):
    consts = [dev(c) for c in synth.resnet18_consts(3)]
    x = dev(synth.resnet18_input(3, 1))
    out = torch.empty((1, 1000), device="cuda")
    module = hostapi.CompiledResNet18(1, 224, "hip", sync_after_run=False)
    module.freeze_constants(True)          # serving mode, as for the batch-64 figure
    packed = module.packed([x] + consts + [out])
    stream = torch.cuda.current_stream().cuda_stream
    ms = _event_time_ms(torch, lambda: module.run_packed(packed, stream), 50, 10)
    # the same plan replayed as one captured HIP graph per image (needs a stream other than the null stream)
    side = torch.cuda.Stream()
    graph_ms = None
    with torch.cuda.stream(side):
        module.enable_graph_replay(True)
        graph_ms = _event_time_ms(torch, lambda: module.run_packed(packed, side.cuda_stream), 50, 10)
    torch.cuda.synchronize()
    module.close()
    best = min(ms, graph_ms)
    return {"value": round(1e3 / best, 1), "ms_per_image": round(best, 4), "eager_ms": round(ms, 4),
            "hip_graph_replay_ms": round(graph_ms, 4)}


def bench_int8(torch, pkg, synth, dev, np, batch):
    """Benchmark configuration 5: quantised ResNet-18, batch 64, int8 matrix cores (calibrated on the same batch).
    The network is the quantised Relay graph compiled by Compiler::Compile for the hip target."""
    qr = importlib.import_module("hdkx-aicompiler_amd.qresnet18")
    hostapi = importlib.import_module("hdkx-aicompiler_amd.hostapi")
    consts = synth.resnet18_consts(5)
    x = dev(synth.resnet18_input(5, batch))
    amax = qr.calibrate(x, [dev(c) for c in consts])
    model = qr.prepare(consts, amax)
    module = hostapi.CompiledQResNet18(model, batch, 224, "hip", sync_after_run=False)
    qconsts = [dev(c) for c in module.constants(model)]
    out = torch.empty((batch, 1000), device="cuda")
    packed = module.packed([x] + qconsts + [out])
    stream = torch.cuda.current_stream().cuda_stream
    # default mode: every run packs the int8 weights again from the pointers it is given (one extra launch)
    unfrozen_ms = _event_time_ms(torch, lambda: module.run_packed(packed, stream), 50, 10)
    module.freeze_constants(True)
    eager_ms = _event_time_ms(torch, lambda: module.run_packed(packed, stream), 50, 10)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        module.enable_graph_replay(True)
        graph_ms = _event_time_ms(torch, lambda: module.run_packed(packed, side.cuda_stream), 50, 10)
    torch.cuda.synchronize()
    ms = min(eager_ms, graph_ms)
    r18 = importlib.import_module("hdkx-aicompiler_amd.resnet18")
    ops = float(r18.flops_per_image()) * batch          # 2 integer operations per multiply-accumulate
    launches = module.launches()
    result = {"metric": "resnet18_int8_bs%d_img_per_s" % batch, "value": round(batch / (ms * 1e-3), 1), "ms_per_step": round(ms, 4),
              "compiled_by": "C++ host layer, Compiler::Compile(quantised Relay graph, target hip)",
              "timed_mode": "frozen constants, " + ("graph replay" if graph_ms < eager_ms else "eager"),
              "eager_ms_per_step": round(eager_ms, 4), "hip_graph_replay_ms_per_step": round(graph_ms, 4),
              "default_mode_ms_per_step": round(unfrozen_ms, 4),
              "int8_tops": round(ops / (ms * 1e-3) / 1e12, 1), "frac_int8_mfma_peak": round(ops / (ms * 1e-3) / 1e12 / 5000.0, 4),
              "launches_per_step": len(launches), "matrix_core_launches": sum(("qmfma" in l or "qrows" in l or "kxc_qdense" in l) for l in launches),
              "workspace_bytes": module.workspace_bytes(),
              "logits_finite": bool(torch.isfinite(out).all().item()),
              "parity": "bit-exact against the CPU int8 chain (tests/test_gpu_int8.py); definition is this build's own"}
    module.close()
    return result


CPU_SAMPLE_IMAGES = 16


def cpu_baseline(np, synth, x, consts):
    """The CPU checker (oracle/, -O3, strict fp32) on one core: one ResNet-18 forward pass of the first 16 images of
    the timed batch (about 15 s), whose logits also check the timed plan."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from oracle_lib import Oracle
    orc = Oracle(fast=True)
    n = min(CPU_SAMPLE_IMAGES, x.shape[0])
    t0 = time.perf_counter()
    logits = orc.resnet18(x[:n], consts)
    t = time.perf_counter() - t0
    return {"value": round(n / t, 4), "unit": "img/s", "cores": 1, "kind": "port",
            "sample": "one ResNet-18 fp32 forward pass of the first %d images of the timed batch, "
                      "gcc -O3 -march=native -ffp-contract=off" % n,
            "sample_images": n, "sample_seconds": round(t, 2), "seconds_per_image": round(t / n, 3),
            "host_cpus": os.cpu_count()}, logits


if __name__ == "__main__":
    main()
