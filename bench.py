#!/usr/bin/env python3
"""Benchmark of the int8 convolution hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2] [--layers all|none|C1,C3a,...]

A step is one pass of the hot path (one elx_conv-equivalent execute) over one batch of synthetic,
device-resident tensors of the named layer.  The headline workload is C2 (int8 3x3 direct conv,
ResNet-50 res3 shape, N=32).  Prints ONE JSON line: effective INT8 TOPS (2 x direct-conv MACs /
time, the reference's accounting), the roofline of the dominant kernel (from the same interval as
ms_per_step, with the HIP-event figure of the same steps beside it), the host-CPU baseline of the
same layer, and -- under "layers" -- the other configured layers, each with its own CPU baseline.
"""
import argparse
import ctypes
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
PKG = "deep-learning-math-kernel-research_amd"


PREHEAT_S = 0.1


class _HipEvents:
    """hipEvent_t pairs through the HIP runtime itself.  The two records sit inside the timed region; made for timing
    only (hipEventDisableSystemFence) and recorded without torch's wrapper they cost it 7 us, torch.cuda.Event 12 us
    (C2, 20 steps: 147 against 155 us; 143 us with no events at all)."""

    def __init__(self):
        self.lib = ctypes.CDLL("libamdhip64.so")
        self.lib.hipEventCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
        self.lib.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.lib.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.lib.hipEventDestroy.argtypes = [ctypes.c_void_p]
        self.free = []
        e0, e1 = self.pair()   # fails here if the runtime will not have it
        self.free += [e0, e1]

    def pair(self):
        while len(self.free) < 2:
            e = ctypes.c_void_p()
            if self.lib.hipEventCreateWithFlags(ctypes.byref(e), 0x20000000) != 0:   # hipEventDisableSystemFence
                raise RuntimeError("hipEventCreateWithFlags")
            self.free.append(e)
        return self.free.pop(), self.free.pop()

    def record(self, e, stream):
        if self.lib.hipEventRecord(e, stream) != 0:
            raise RuntimeError("hipEventRecord")

    def elapsed_ms(self, e0, e1):
        ms = ctypes.c_float()
        if self.lib.hipEventElapsedTime(ctypes.byref(ms), e0, e1) != 0:
            raise RuntimeError("hipEventElapsedTime")
        self.free += [e0, e1]
        return ms.value


_HIP_EVENTS = []


def _hip_events():
    """the process's _HipEvents, or None where the runtime library cannot be reached (then torch.cuda.Event)"""
    if not _HIP_EVENTS:
        try:
            _HIP_EVENTS.append(_HipEvents())
        except (OSError, AttributeError, RuntimeError):
            _HIP_EVENTS.append(None)
    return _HIP_EVENTS[0]


def chained_network(layers, batches):
    """The layers of a network in order, `count` executes of each, as one sequence per batch on one stream: timed as
    `batches` sequences enqueued launch by launch, and as the same number of replays of a HIP graph that holds one
    sequence.  Every kernel then follows a different kernel with different tensors, as in a model run.  The graph's
    last replay must leave the same bytes in every layer's output as the last eager sequence."""
    import torch
    s = torch.cuda.Stream()
    def sequence(stream):
        for count, l in layers:
            l.conv.execute_repeat(l.out, l.x, count, bias=l.bias, stream=stream)
    def timed(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(batches):
            fn()
        torch.cuda.synchronize()   # (a replay runs on the current stream, the sequences on s)
        return (time.perf_counter() - t0) / batches
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < max(PREHEAT_S, 0.02):   # also the first execute of every handle: its launch plans
        sequence(s.cuda_stream)
        s.synchronize()
    eager = timed(lambda: sequence(s.cuda_stream))
    # outputs of layers with the in-place sum change with every execute: compare from a common state
    def snapshot():
        return [l.out.clone() for _, l in layers]
    def restore(state):
        for (_, l), o in zip(layers, state):
            l.out.copy_(o)
    start = snapshot()
    sequence(s.cuda_stream)
    s.synchronize()
    want = snapshot()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        sequence(torch.cuda.current_stream().cuda_stream)
    restore(start)
    torch.cuda.synchronize()
    g.replay()
    torch.cuda.synchronize()
    same = all(torch.equal(a.view(torch.uint8), b.view(torch.uint8)) for a, b in zip(snapshot(), want))
    graph = timed(g.replay)
    return {"batches": batches, "eager_ms_per_batch": round(eager * 1e3, 4), "graph_ms_per_batch": round(graph * 1e3, 4),
            "graph_images_per_s": round(64 / graph, 1), "graph_replay_matches_eager": bool(same)}


def measure(layer, steps, warmup):
    """(wall seconds per step, HIP-event seconds per step).  Both regions hold exactly `steps`
    executions enqueued back to back on the stream the kernels run on (the default stream).
    Before the warmup steps the layer runs untimed for PREHEAT_S seconds: an idle GPU takes tens of
    milliseconds to reach its running clocks, far longer than `warmup` launches of a 10 us kernel
    (the same layer reads 12 % slower when timed straight from idle)."""
    import torch
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < PREHEAT_S:
        layer.run(200)
        torch.cuda.synchronize()
    hip = _hip_events()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)   # the stream the layer's kernels run on

    def region(count):
        # exactly `count` steps between two synchronisations, on the host clock and on HIP events
        torch.cuda.synchronize()
        if hip is None:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            e0.record()
            layer.run(count)
            e1.record()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            return (t1 - t0) / count, e0.elapsed_time(e1) * 1e-3 / count
        e0, e1 = hip.pair()
        t0 = time.perf_counter()
        hip.record(e0, stream)
        layer.run(count)
        hip.record(e1, stream)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return (t1 - t0) / count, hip.elapsed_ms(e0, e1) * 1e-3 / count

    # the warmup steps take the same path as the timed ones (event creation and recording included): what a
    # first call costs the host once -- lazy initialisation behind the first event, cold code -- stays out
    if warmup > 0:
        region(warmup)
    return region(steps)


def winograd_stage_rooflines(layer, wl, steps):
    """The stages of a Winograd layer, each timed on its own (ehip_conv_execute_stages, `steps` back-to-back
    launches between two synchronisations, HIP events on the launch stream): the transforms against the HBM
    peak with the bytes they read and write, the A x A GEMMs against the int8 MFMA peak with the multiplies they
    really do (A^2 / (A - 2)^2 / 9 of the direct algorithm's), as the reference splits the layer
    (src/elx_int8_conv_wino_xopt.hpp:70-121).  In the fused schedule the GEMM stage contains the output transform."""
    import torch
    from importlib import import_module
    W = import_module(PKG + ".workloads")
    E = import_module(PKG)
    hip = _hip_events()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    A = wl.tile or 6
    m = A - 2
    tiles = wl.n * ((wl.oh + m - 1) // m) ** 2
    icp, ocp = W.up16(wl.ic), W.up16(wl.oc)
    esz = {E.U8: 1, E.S8: 1, E.F32: 4}
    in_bytes = wl.n * icp * wl.hw * wl.hw * esz[wl.in_type]
    out_bytes = wl.n * ocp * wl.oh * wl.oh * esz[wl.out_type]
    tin_bytes = A * A * icp * tiles
    tout_bytes = A * A * ocp * tiles * 4
    w_bytes = A * A * icp * ocp
    fused = "k_wino_gemm_output" in layer.conv.kernel_name

    def timed(stages):
        layer.conv.execute_stages(layer.out, layer.x, stages, 3, bias=layer.bias)
        torch.cuda.synchronize()
        if hip is None:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            layer.conv.execute_stages(layer.out, layer.x, stages, steps, bias=layer.bias)
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e-3 / steps
        e0, e1 = hip.pair()
        hip.record(e0, stream)
        layer.conv.execute_stages(layer.out, layer.x, stages, steps, bias=layer.bias)
        hip.record(e1, stream)
        torch.cuda.synchronize()
        return hip.elapsed_ms(e0, e1) * 1e-3 / steps

    def hbm(nbytes, sec):
        return {"bound": "hbm", "bytes": float(nbytes), "us": round(sec * 1e6, 2), "achieved": round(nbytes / sec / 1e9, 1),
                "peak": W.PEAK_HBM_GBS, "unit": "GB/s", "frac": round(nbytes / sec / 1e9 / W.PEAK_HBM_GBS, 4)}

    stages = {}
    t_in = timed(1)
    stages["trans_input"] = hbm(in_bytes + tin_bytes, t_in)
    t_g = timed(2)
    gemm_ops = 2.0 * A * A * tiles * icp * ocp
    g = {"bound": "mfma", "ops": gemm_ops, "us": round(t_g * 1e6, 2), "achieved": round(gemm_ops / t_g / 1e12, 1),
         "peak": W.PEAK_INT8_TOPS, "unit": "TFLOP/s", "frac": round(gemm_ops / t_g / 1e12 / W.PEAK_INT8_TOPS, 4),
         "bytes": float(tin_bytes + w_bytes + (out_bytes if fused else tout_bytes)),
         "contains": "A x A GEMMs + output transform (fused)" if fused else "A x A GEMMs"}
    g["frac_hbm"] = round(g["bytes"] / t_g / 1e9 / W.PEAK_HBM_GBS, 4)
    stages["gemm"] = g
    if not fused:
        t_o = timed(4)
        stages["trans_output"] = hbm(tout_bytes + out_bytes, t_o)
    layer.run(1)   # leave the buffers as a whole execute leaves them
    torch.cuda.synchronize()
    return stages


def single_launch_latency(layer, reps=20):
    import torch
    best = 1e9
    for _ in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        layer.run(1)
        torch.cuda.synchronize()
        best = min(best, time.perf_counter() - t0)
    return best


def roofline_of(wl, sec_per_step, sec_per_step_events, traffic):
    """`achieved` and `frac` come from the same interval as ms_per_step (host clock around the timed
    steps, synchronised on both sides); `frac_event` is the same figure from the HIP events recorded
    on the kernels' stream around the same steps, which leaves out the host's share of the first
    enqueue and of the final synchronisation."""
    from importlib import import_module
    W = import_module(PKG + ".workloads")
    kind, _ = wl.bound()
    if kind == "mfma":
        work, scale = wl.ops(), 1e12
        peak, unit = W.PEAK_INT8_TOPS, "TFLOP/s"
    else:
        work, scale = wl.algorithmic_bytes(), 1e9
        peak, unit = W.PEAK_HBM_GBS, "GB/s"
    achieved = work / sec_per_step / scale
    return {"bound": kind, "achieved": round(achieved, 3), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 5), "traffic": traffic,
            "achieved_event": round(work / sec_per_step_events / scale, 3),
            "frac_event": round(work / sec_per_step_events / scale / peak, 5)}


def host_cpus():
    """(model name, logical CPUs visible, physical cores, threads per core) from /proc/cpuinfo"""
    model, cores, logical = "unknown", set(), 0
    phys = core = None
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                key, _, val = line.partition(":")
                key, val = key.strip(), val.strip()
                if key == "model name":
                    model = val
                elif key == "processor":
                    logical += 1
                elif key == "physical id":
                    phys = val
                elif key == "core id":
                    core = val
                    cores.add((phys, core))
    except OSError:
        pass
    physical = len(cores) or logical
    return model, logical, physical, (logical // physical if physical else 1)


def reference_iterations(ops):
    """the repeat count of the reference's benchmark loop (tests/elt_conv_utils.cpp:661-664)"""
    return min(1024, max(int(5e12 / ops), 64))


def cpu_baseline(wl, budget_s=12.0):
    """The CPU oracle (a port of the reference's loop nests; AVX-512-VNNI inner loops when the host
    has them) timed on this host's cores on the same layer: the direct 1x1 / k x k nest, the depthwise
    nest or the three Winograd stages (input transform, u8 x s8 GEMM, output transform), steady state
    (weight preparation excluded).  The reference's benchmark repeats a layer
    clamp(5e12 / ops, 64, 1024) times (tests/elt_conv_utils.cpp:661-664); here the same count is the
    upper limit and `budget_s` seconds end the loop earlier, and a layer whose single pass would not fit
    the budget runs on a slice of its batch (every image is independent, so the rate carries over)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import numpy as np
    import oracle_lib as ol
    E = importlib.import_module(PKG)
    rng = np.random.default_rng(7)
    lib = ol.oracle()
    vnni = bool(lib.orc_has_vnni())
    threads = int(lib.orc_num_threads())
    model, logical, physical, smt = host_cpus()
    wino = wl.algorithm == E.CONV_WINOGRAD
    first = wl.in_z != 0.0 or (wl.nhwc_in and wl.ic <= 4)
    # a first guess of one pass: ~1 TOPS per 8 VNNI threads for the direct nests, far less for the others
    n = wl.n
    rate = (0.12 if vnni else 0.004) * threads * (0.05 if wl.depthwise else (0.3 if wino else 1.0)) * 1e12
    while n > 1 and wl.ops() * n / wl.n / rate > budget_s / 4:
        n = (n + 1) // 2
    ic2, oc2 = ol.up16(wl.ic) // 16, ol.up16(wl.oc) // 16
    g = wl.ic if wl.depthwise else 1
    relu_hi = 255.0 if wl.relu6 else ol.FLT_MAX
    p = ol.make_params(n, wl.ic, wl.oc, wl.hw, wl.hw, wl.k, wl.k, wl.pad, wl.stride, g=g, out_type=wl.out_type,
                       with_sum=wl.with_sum, out_scale=0.02, sum_scale=0.7 if wl.with_sum else 0.0, relu_hi=relu_hi,
                       T=wl.T, out_hw=(wl.oh, wl.oh), pad_tl=wl.pad, wino_tile=wl.tile if wino else 0,
                       in_scale=1.0 if wl.in_type == E.F32 else 1.0 / 255.0, in_z=wl.in_z)
    b = rng.normal(0, 0.01, ol.up16(wl.oc)).astype(np.float32)
    out = np.zeros((n, oc2, wl.oh, wl.oh, 16), ol.NP_OF[wl.out_type])
    if wl.with_sum:
        out[...] = rng.integers(-127, 128, out.shape)
    if wino:
        x = rng.random((n, ic2, wl.hw, wl.hw, 16), dtype=np.float32)   # u8 input enters dequantized
        w = rng.normal(0, wl.w_sigma, (wl.oc, wl.ic, 3, 3)).astype(np.float32)
        mn, mx = ol.wino_tinput_range(p, x)
        p.tin_scale = (mx - mn + 1e-6) / 255.0
        p.tin_z = -mn * 255.0 / (mx - mn + 1e-6)
        twq, tscale, tshift = ol.wino_prepare(p, ol.weights_to_blocked(w))
        t, pos = ol.wino_tiles(p), ol.wino_positions(p)
        tin = np.zeros((pos, ic2, t, 16), np.uint8)
        tout = np.zeros((pos, oc2, t, 16), np.float32)
        pp = ctypes.byref(p)

        def one_pass():
            lib.orc_wino_trans_input(pp, ol.ptr(x), ol.ptr(tin))
            lib.orc_wino_gemm(pp, ol.ptr(tin), ol.ptr(twq), ol.ptr(tscale), ol.ptr(tshift), ol.ptr(tout), None)
            lib.orc_wino_trans_output(pp, ol.ptr(tout), ol.ptr(b), ol.ptr(out))
        nest = "Winograd input transform + u8 x s8 GEMM + output transform"
    elif first:
        # A first layer as the reference's tuned runs feed it (scripts/best_configs/resnetv1_5-n64-clx-1s-int8.sh:12):
        # three channels, input zero point 128, so the shift of a pixel depends on which taps fall inside the image.
        # The oracle runs it as the same k x k nest over one 16-channel unit (the image's channels padded to 16 --
        # the reference pads three to four, a quarter of these multiplies) with a shift row per pixel.
        x = rng.integers(0, 256, (n, ic2, wl.hw, wl.hw, 16)).astype(np.uint8)
        x[..., wl.ic:] = 0
        w = rng.normal(0, wl.w_sigma, (wl.oc, wl.ic, wl.k, wl.k)).astype(np.float32)
        wb = ol.weights_to_blocked(w)
        wq, scale, shift, _ = ol.direct_prepare(p, wb, b)
        smap = np.zeros((wl.oh, wl.oh, ol.up16(wl.oc)), np.float32)
        assert lib.orc_direct_border_shifts(ctypes.byref(p), ol.ptr(wb), ol.ptr(b), ol.ptr(smap)) == 0
        args = (ctypes.byref(p), ol.ptr(x), ol.ptr(wq), ol.ptr(scale), ol.ptr(smap), ol.ptr(out), None)

        def one_pass():
            assert lib.orc_direct_execute_border(*args) == 0
        nest = "direct %dx%d nest over the image's channels padded to 16, a shift row per pixel," % (wl.k, wl.k)
    elif wl.depthwise:
        x = rng.integers(0, 256, (n, ic2, wl.hw, wl.hw, 16)).astype(np.uint8)
        w = rng.normal(0, wl.w_sigma, (wl.ic, 1, 3, 3)).astype(np.float32)
        wq, scale, shift, _ = ol.depthwise_prepare(p, w, b)
        args = (ctypes.byref(p), ol.ptr(x), ol.ptr(wq), ol.ptr(scale), ol.ptr(shift), ol.ptr(out), None)

        def one_pass():
            lib.orc_depthwise_execute(*args)
        nest = "depthwise nest"
    else:
        x = rng.integers(0, 256, (n, ic2, wl.hw, wl.hw, 16)).astype(np.uint8)
        w = rng.normal(0, wl.w_sigma, (wl.oc, wl.ic, wl.k, wl.k)).astype(np.float32)
        wq, scale, shift, _ = ol.direct_prepare(p, ol.weights_to_blocked(w), b)
        args = (ctypes.byref(p), ol.ptr(x), ol.ptr(wq), ol.ptr(scale), ol.ptr(shift), ol.ptr(out), None)

        def one_pass():
            lib.orc_direct_execute(*args)
        nest = "direct %dx%d nest" % (wl.k, wl.k)
    one_pass()  # warm-up
    limit = reference_iterations(wl.ops())
    passes, t0 = 0, time.perf_counter()
    while True:
        one_pass()
        passes += 1
        el = time.perf_counter() - t0
        if el > budget_s or passes >= limit:
            break
    sec = el / passes
    ops = wl.ops() * n / wl.n
    return {"value": round(ops / sec / 1e12, 4), "unit": "TOPS", "cores": threads, "kind": "port",
            "isa": "avx512-vnni" if vnni else "scalar/auto-vectorised",
            "sample": "%d passes (the reference's loop would run %d) of the %s of %s with N=%d of %d in %.1f s on %d "
                      "OpenMP threads; weight preparation excluded" % (passes, limit, nest, wl.key, n, wl.n, el, threads),
            "ms_per_pass": round(sec * 1e3, 3), "images_per_s": round(n / sec, 1), "cpu_model": model,
            "host_logical_cpus": logical, "host_physical_cores": physical, "host_threads_per_core": smt}


def load_traffic():
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(path):
        with open(path) as f:
            return json.load(f)
    return {}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="C2")
    ap.add_argument("--layers", default="all", help="other layers to report: all, none or a comma list")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baselines")
    ap.add_argument("--cpu-budget", type=float, default=12.0, help="seconds of CPU work for the headline layer's baseline")
    ap.add_argument("--cpu-budget-layer", type=float, default=2.5,
                    help="seconds of CPU work for the baseline of each layer under \"layers\"")
    ap.add_argument("--batch", type=int, default=0, help="override the workload's batch size N (scaling studies; "
                                                         "the headline figure uses the configured N)")
    ap.add_argument("--network", default="", help="instead of one layer: every convolution layer of one of the reference's "
                                                  "tuned int8 model runs (resnet50_v1_5_int8, mobilenet_v1_int8, "
                                                  "vgg19_int8), each timed on its own synthetic tensors; prints the "
                                                  "per-layer table and the images/s of the sum")
    ap.add_argument("--direct3x3", action="store_true",
                    help="with --network: run the 3x3 stride-1 layers with CONV_DIRECT instead of the Winograd "
                         "algorithm the reference's scripts ask for (on this GPU the direct kernel is the faster one; "
                         "its results are the reference's DIRECT results, not its Winograd results)")
    ap.add_argument("--chained", action="store_true",
                    help="with --network: besides the sum of the layers' own times, run the whole list of layers in order "
                         "as ONE sequence per batch -- enqueued launch by launch on a stream, and replayed from a HIP "
                         "graph of the same launches -- so that every kernel follows a different one (cold caches, "
                         "launch gaps between unlike kernels); all layers' tensors stay resident")
    ap.add_argument("--preheat-ms", type=float, default=100.0,
                    help="untimed run of the layer before the warmup steps, so that the GPU is at its running clocks "
                         "(profiler runs pass a small value to keep their traces short)")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="rate of v_mfma_i32_32x32x32_i8 from registers, nothing else in the way")
    ap.add_argument("--hbm-probe", action="store_true",
                    help="instead of a layer, time plain device copy / fill / read of 1 GiB (the HBM rates a "
                         "trivial kernel reaches on this box)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="instead of a layer, run 20 plain device copies of MIB MiB (known traffic, used to "
                         "scale the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU: every layer is a single-device kernel and nothing here "
              "shards across devices (the layers would shard by batch: every image is independent); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    global PREHEAT_S
    PREHEAT_S = args.preheat_ms * 1e-3
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    E = importlib.import_module(PKG)
    W = importlib.import_module(PKG + ".workloads")
    rc = E.lib.ehip_init(0)
    if rc != 0:
        print("bench.py: " + E.lib.ehip_last_error().decode(), file=sys.stderr)
        sys.exit(1)
    traffic = load_traffic()

    if args.calibrate_copy:
        n = args.calibrate_copy << 20
        src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(20):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes": n, "launches": 20}))
        return

    if args.hbm_probe:
        n = 1 << 30
        a = torch.empty(n, dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        af = a.view(torch.float32)

        def rate(fn, nbytes, reps=20):
            fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return round(nbytes / (e0.elapsed_time(e1) * 1e-3 / reps) / 1e9, 1)
        print(json.dumps({"hbm_probe_bytes": n, "copy_read_plus_write_GBs": rate(lambda: b.copy_(a), 2 * n),
                          "fill_write_GBs": rate(lambda: a.zero_(), n), "sum_read_GBs": rate(lambda: af.sum(), n)}))
        return

    if args.mfma_probe:
        probe = ctypes.CDLL(os.path.join(ROOT, PKG, "build", "libehip_probe.so"))
        probe.ehip_bench_probe_mfma_i8.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                                   ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]

        def probe_mfma_i8(workgroups, iters, out, stream):
            ops = ctypes.c_double()
            rc = probe.ehip_bench_probe_mfma_i8(workgroups, iters, ctypes.c_void_p(out.data_ptr()), ctypes.byref(ops),
                                                ctypes.c_void_p(stream))
            assert rc == 0
            return ops.value
        out = torch.empty(4096 * 256, dtype=torch.int32, device="cuda")
        res = {}
        stream = torch.cuda.current_stream().cuda_stream
        for wgs in (256, 512, 1024, 2048, 4096):   # 1, 2, 4, 8, 16 waves per SIMD's worth of workgroups
            ops = probe_mfma_i8(wgs, 2000, out, stream)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(5):
                probe_mfma_i8(wgs, 2000, out, stream)
            e1.record()
            torch.cuda.synchronize()
            res["wgs_%d" % wgs] = round(ops / (e0.elapsed_time(e1) * 1e-3 / 5) / 1e12, 1)
        print(json.dumps({"mfma_i8_probe_TOPS": res, "instruction": "v_mfma_i32_32x32x32_i8", "published_peak_TOPS": 5000.0}))
        return

    if args.network:
        net = W.NETWORKS[args.network]
        rows, total_s, total_ops = [], 0.0, 0.0
        kept = []
        for count, w2 in net:
            if args.direct3x3 and w2.algorithm == E.CONV_WINOGRAD:
                w2 = W.Workload(w2.key, "3x3 direct %d->%d @%d u8->s8" % (w2.ic, w2.oc, w2.hw), w2.n, w2.ic, w2.oc, w2.hw, k=3,
                                pad=1, out_type=w2.out_type, T=14 if w2.hw % 14 == 0 else (7 if w2.hw % 7 == 0 else 0))
            l2 = W.DeviceLayer(w2)
            wall2, ev2 = measure(l2, 50 if w2.ops() > 5e10 else 200, 5)
            rows.append({"layer": w2.key, "title": w2.title, "count": count, "n": w2.n, "us": round(wall2 * 1e6, 2),
                         "tops": round(w2.ops() / wall2 / 1e12, 1), "kernel": l2.conv.kernel_name})
            # the FC layers are configured with n = 1 over 8 x 8 "pixels" = one row per image of the batch
            total_s += count * wall2
            total_ops += count * w2.ops()
            if args.chained:
                kept.append((count, l2))
                continue
            del l2
            torch.cuda.empty_cache()
        chained = None
        if args.chained:
            chained = chained_network(kept, 20 if total_s > 1e-3 else 50)
        print(json.dumps({"metric": "network_conv_layers_images_per_s", "network": args.network,
                          "three_by_three": "direct" if args.direct3x3 else "as configured by the reference's script",
                          "value": round(64 / total_s, 1), "unit": "images/s", "batch": 64,
                          "layers_total": sum(c for c, _ in net), "ms_per_batch": round(total_s * 1e3, 4),
                          "effective_tops": round(total_ops / total_s / 1e12, 1), "data": "synthetic",
                          "note": "sum over the network's convolution layers of count x time of one execute, each "
                                  "layer timed back to back on its own device-resident tensors; pooling, residual "
                                  "adds and softmax are not part of the library", "chained": chained, "layers": rows}))
        return

    wl = W.WORKLOADS[args.workload]
    if args.batch:
        import copy
        wl = copy.copy(wl)
        wl.n = args.batch
        wl.key = "%s@N=%d" % (wl.key, wl.n)
    layer = W.DeviceLayer(wl)
    wall, ev = measure(layer, args.steps, args.warmup)
    lat = single_launch_latency(layer)
    tops = wl.ops() / wall / 1e12
    result = {
        "metric": "effective_int8_tops", "value": round(tops, 3), "unit": "TOPS",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall * 1e3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "%s: %s" % (wl.key, wl.title), "ops_per_step": wl.ops(),
                   "algorithmic_bytes_per_step": wl.algorithmic_bytes(), "kernel": layer.conv.kernel_name,
                   "untimed_preheat_ms": PREHEAT_S * 1e3, "seed": W.seed_of(wl.key), "calibration": layer.calibration},
        "images_per_s": round(wl.n / wall, 1),
        "single_launch_latency_us": round(lat * 1e6, 2),
        "event_ms_per_step": round(ev * 1e3, 6),
        "roofline": roofline_of(wl, wall, ev, traffic.get(wl.key)),
    }
    if wl.algorithm == E.CONV_WINOGRAD:
        result["roofline"]["stages"] = winograd_stage_rooflines(layer, wl, 50)
    del layer
    torch.cuda.empty_cache()

    layers = {}
    keys = [] if args.layers == "none" else (
        [k for k in W.WORKLOADS if k != wl.key] if args.layers == "all" else args.layers.split(","))
    for k in keys:
        w2 = W.WORKLOADS[k]
        l2 = W.DeviceLayer(w2)
        steps = 200
        wall2, ev2 = measure(l2, steps, 10)
        layers[k] = {"title": w2.title, "tops": round(w2.ops() / wall2 / 1e12, 3),
                     "images_per_s": round(w2.n / wall2, 1), "ms_per_step": round(wall2 * 1e3, 5),
                     "event_ms_per_step": round(ev2 * 1e3, 5), "kernel": l2.conv.kernel_name,
                     "roofline": roofline_of(w2, wall2, ev2, traffic.get(k))}
        if w2.algorithm == E.CONV_WINOGRAD:
            layers[k]["roofline"]["stages"] = winograd_stage_rooflines(l2, w2, 50)
        del l2
        torch.cuda.empty_cache()
    if layers:
        result["layers"] = layers

    if not args.no_cpu:
        def baseline(w2, budget_s):
            try:
                return cpu_baseline(w2, budget_s)
            except Exception as exc:  # the baseline is a report, never a reason to lose the GPU number
                return {"value": None, "unit": "TOPS", "cores": 0, "kind": "port", "sample": "failed: %r" % (exc,)}
        result["cpu_baseline"] = baseline(wl, args.cpu_budget)
        for k in layers:
            layers[k]["cpu_baseline"] = baseline(W.WORKLOADS[k], args.cpu_budget_layer)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
