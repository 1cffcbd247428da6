#!/usr/bin/env python3
"""Benchmark of the int8 conv2d hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload = BASELINE config 2: x fp32 32x256x28x28 ~ N(0,1) quantized per tensor
(127/max|x|, one equal scale per image), weights 256x256x3x3 ~ N(0,0.05) int8 per output
channel, stride 1, pad 1, int32 accumulation, fp32 dequant + bias + ReLU output.
One "step" = one pass of the path over the batch: quantize+stage kernel, then the i8-MFMA
implicit-GEMM kernel with the fused epilogue, inputs resident in HBM.

Prints ONE JSON line.  `value` is the whole step's throughput in TOPS (2*MAC / step time);
`roofline` is the MFMA kernel alone (HIP events around back-to-back launches) against the
int8 dense MFMA peak; `cpu_baseline` times the same layer on the host cores with the
compiled TenniS reference (kind "reference") or, where that is absent, the CPU oracle
(kind "port").
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, 5.0 POP/s
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, 8 TB/s
PEAK_FP32_TFLOPS = 157.3  # MI355X dense fp32 MFMA

CFG = dict(n=32, c=256, h=28, w=28, cout=256, k=3, pad=1)

# HBM bytes per launch of the two kernels on this workload, from rocprofv3 FETCH_SIZE / WRITE_SIZE scaled by a
# known-size copy (profiles/conv2d_i8_config2_hbm_traffic.txt); a profiler figure, not measured by this script.
TRAFFIC_CONV_BYTES = 43.02e6
TRAFFIC_STAGE_BYTES = 32.54e6


def make_inputs(cfg, seed=1234):
    rng = np.random.default_rng(seed)
    n, c, h, w, cout, k = cfg["n"], cfg["c"], cfg["h"], cfg["w"], cfg["cout"], cfg["k"]
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, c, k, k)) * 0.05).astype(np.float32)
    bias = (rng.standard_normal(cout) * 0.1).astype(np.float32)
    s_x = np.float32(127.0) / np.abs(x).max().astype(np.float32)
    x_scales = np.full(n, s_x, np.float32)
    wmax = np.abs(wt.reshape(cout, -1)).max(axis=1).astype(np.float32)
    s_w = (np.float32(127.0) / wmax).astype(np.float32)
    q = wt * s_w[:, None, None, None]
    wq = np.clip(np.sign(q) * np.floor(np.abs(q) + 0.5), -127, 127).astype(np.int8)
    dq = (np.float32(1.0) / (s_x * s_w)).astype(np.float32)
    return x, x_scales, wq, dq, bias


def cpu_baseline(x, x_scales, wq, dq, bias, pad, images):
    """The reference's own operator chain on the host: quantize -> conv2d_quantized -> add_bias -> relu."""
    xs = np.ascontiguousarray(x[:images])
    sc = x_scales[:images]
    pads = (pad, pad, pad, pad)
    macs = images * wq.shape[0] * x.shape[2] * x.shape[3] * wq.shape[1] * wq.shape[2] * wq.shape[3]
    try:
        from oracle import ref
        have_ref = ref.available()
    except Exception:
        have_ref = False
    if have_ref:
        t0 = time.perf_counter()
        xq = ref.quantize(xs, sc, threads=1)
        y = ref.conv2d_quantized(xq, wq, dq, pads=pads, threads=1)
        y = ref.add_bias(y, bias, threads=1)
        y = ref.relu(y, threads=1)
        dt = time.perf_counter() - t0
        kind, cores = "reference", 1
        note = ("compiled TenniS CPU library (OpenMP+AVX2/FMA build), computing_thread_number=1: its int8 GEMM is "
                "single-threaded scalar and its dequant loop is only correct at one thread")
    else:
        from oracle import port
        port.set_threads(1)
        t0 = time.perf_counter()
        xq = port.quantize(xs, sc)
        port.conv2d_i8_fused(xq, wq, dq, bias, "relu", pads=pads)
        dt = time.perf_counter() - t0
        kind, cores = "port", 1
        note = "CPU oracle restatement, 1 thread"
    return {"value": 2.0 * macs / dt / 1e12, "unit": "TOPS", "cores": cores, "kind": kind,
            "sample": "%d of %d images of the same layer, %.2f s; %s" % (images, x.shape[0], dt, note),
            "host_cpus": os.cpu_count()}


def cpu_baseline_all_cores(x, x_scales, wq, dq, bias, pad):
    """The same operator chain with OpenMP on every loop, on all host cores: the CPU restatement (oracle/,
    checked bit for bit against the compiled reference), whose int8 GEMM and dequantize loops are parallel --
    the reference's own are single-threaded / racy above one thread.  A second baseline beside the faithful one."""
    from oracle import port
    threads = min(port.max_threads(), os.cpu_count() or 1, 16)
    port.set_threads(threads)
    pads = (pad, pad, pad, pad)
    port.conv2d_i8_fused(port.quantize(x[:2], x_scales[:2]), wq, dq, bias, "relu", pads=pads)     # warm-up
    t0 = time.perf_counter()
    xq = port.quantize(x, x_scales)
    port.conv2d_i8_fused(xq, wq, dq, bias, "relu", pads=pads)
    dt = time.perf_counter() - t0
    macs = x.shape[0] * wq.shape[0] * x.shape[2] * x.shape[3] * wq.shape[1] * wq.shape[2] * wq.shape[3]
    return {"value": 2.0 * macs / dt / 1e12, "unit": "TOPS", "cores": threads, "kind": "port",
            "sample": "all %d images of the layer, %.2f s; CPU restatement built -O3 -fopenmp -mavx2 -mfma, OpenMP on "
                      "every loop" % (x.shape[0], dt), "host_cpus": os.cpu_count()}


def _fp32_conv_rows(shape_x, shape_w, reps, seed):
    """conv2d_f32 (implicit im2col GEMM on the fp32 MFMA), both Winograd modes in their bit-exact form and F(6,3) as
    one MFMA launch on one 3x3 / stride 1 / pad 1 layer with bias + ReLU, all credited the direct convolution's
    flops; seconds per launch = median of 5 batches of `reps` back-to-back launches between events."""
    import torch
    from tennis_amd import capi
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cuda").manual_seed(seed)
    n, c, h, w = shape_x
    cout = shape_w[0]
    x = torch.rand(shape_x, device=dev, generator=g) * 2 - 1
    wt = torch.randn(shape_w, device=dev, generator=g) * (2.0 / (9 * c)) ** 0.5
    b = torch.randn(cout, device=dev, generator=g) * 0.01
    flops = 2.0 * n * cout * h * w * c * 9
    w63, w23 = capi.WinogradF63(wt, (1, 1, 1, 1)), capi.WinogradF23(wt, (1, 1, 1, 1))
    rows = {}
    direct, _ = capi.conv2d_f32_prepared(x, wt, (1, 1, 1, 1), bias=b, act="relu")
    for name, fn in (("im2col_gemm", direct),
                     ("winograd_f63", lambda: w63(x, bias=b, act="relu")), ("winograd_f23", lambda: w23(x, bias=b, act="relu")),
                     ("winograd_f63_fast", lambda: w63(x, bias=b, act="relu", fast=True))):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        per = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            per.append(e0.elapsed_time(e1) * 1e-3 / reps)
        t = float(np.median(per))
        rows[name] = {"us": t * 1e6, "GFLOPS": flops / t / 1e9, "frac_of_fp32_mfma_peak": flops / t / 1e12 / PEAK_FP32_TFLOPS}
    return flops, rows


def config1_leg(reps=50):
    """BASELINE config 1: fp32 conv2d 1x64x56x56 * 64x64x3x3, stride 1, pad 1, bias + ReLU."""
    flops, rows = _fp32_conv_rows((1, 64, 56, 56), (64, 64, 3, 3), reps, 5)
    return {"workload": "BASELINE config 1: fp32 conv2d 1x64x56x56 * 64x64x3x3 s1 p1 + bias + ReLU; %.1f MFLOP per launch "
                        "(Winograd credited the same), 49 tiles of 64x64: a batch of one cannot fill 256 CUs" % (flops / 1e6),
            "reps": reps, "peak_TFLOPS": PEAK_FP32_TFLOPS, **rows}


def winograd_shape_leg(reps=20):
    """A layer the reference's own selector gives to Winograd F(6,3) (winograd_mode_select_on_arm,
    src/kernels/common/function.cpp:154-173: Cin * Cout >= 65536 and a map larger than 16 x 16): 8x256x28x28 *
    256x256x3x3, stride 1, pad 1, bias + ReLU -- the same four kernels as on config 1."""
    flops, rows = _fp32_conv_rows((8, 256, 28, 28), (256, 256, 3, 3), reps, 6)
    return {"workload": "fp32 conv2d 8x256x28x28 * 256x256x3x3 s1 p1 + bias + ReLU (a shape the reference routes to Winograd "
                        "F(6,3)); %.2f GFLOP per launch by the direct convolution's count" % (flops / 1e9),
            "reps": reps, "peak_TFLOPS": PEAK_FP32_TFLOPS, **rows}


def ceiling_evidence(A, conv_launch, event_time, conv_ops, dev, stream, frags):
    """What bounds the config-2 MFMA kernel, measured on the measurement build of the library (A; `python -m
    tennis_amd.build --aids`): (1) the rate of a register-only MFMA loop against the number of busy CUs and the
    operand data (the clock the part grants falls with both), (2) where one launch of the weight-stationary kernel
    spends its time, per wavefront, from wall-clock and shader-clock stamps that build's kernel writes.
    `python bench.py --ceiling`; under rocprofv3 --pmc GRBM_GUI_ACTIVE the same run gives cycles / duration for the
    probe and the kernel from the counters' side."""
    import torch
    from tennis_amd import capi
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    iters = 20000
    probe = []
    for data in ("random int8", "zeros"):
        if data == "zeros":
            operands = torch.zeros(32768, dtype=torch.int8, device=dev)
        else:
            operands = torch.randint(-128, 128, (32768,), dtype=torch.int8, device=dev)
        for blocks in (64, 128, 224, 256, 512, 1024):
            t = event_time(lambda: capi.check(A.tsx_probe_mfma_i8(capi._ptr(operands), iters, blocks, capi._ptr(sink), stream)), 3)
            rate = blocks * 4 * iters * 8 * 65536.0 / t
            simds = min(blocks * 4, 1024)      # a workgroup of 4 wavefronts fills one CU's SIMDs; beyond 256 they queue up
            probe.append({"operands": data, "workgroups": blocks, "POP_per_s": rate / 1e15,
                          "GHz_equivalent_per_busy_simd": rate / simds / 2048 / 1e9})
    t_conv = event_time(conv_launch, 50)
    slots = 256 * 8 * 24 * 2                         # [workgroup][wavefront][24 stamps][wall clock, shader clock]
    stamps = torch.zeros(slots, dtype=torch.int64, device=dev)
    capi.check(A.tsx_debug_phase_stamps(capi._ptr(stamps), slots * 8))
    try:
        t_stamped = event_time(conv_launch, 20)      # the stamps of the last launch remain
    finally:
        capi.check(A.tsx_debug_phase_stamps(None, 0))
    st = stamps.cpu().numpy().reshape(-1, 8, 24, 2)
    st = st[st[:, 0, 0, 0] != 0]                     # workgroups beyond the last tile leave at once
    wall, clk = st[..., 0].astype(np.float64) * 10.0, st[..., 1].astype(np.float64)   # ns (100 MHz), cycles
    t_first = wall[:, :, 0].min()

    def stats(v):
        return {"mean": float(v.mean()), "min": float(v.min()), "max": float(v.max())}

    # wavefronts 0-3 multiply: stamps = entry, weights in registers + first rows in LDS, last fragment done;
    # wavefronts 4-7 serve (rows in, results out): entry, ring filled, last round done, stores issued, stores left
    mul, srv = wall[:, :4], wall[:, 4:]
    loop_ns = mul[:, :, 2] - mul[:, :, 1]
    phases = {
        "entry_after_first_wavefront_ns": stats(wall[:, :, 0] - t_first),
        "multiplying": {
            "weights_to_registers_and_first_rows_ns": stats(mul[:, :, 1] - mul[:, :, 0]),
            "all_fragments_ns": stats(loop_ns),
            "ns_per_fragment_full_tiles": float(np.median(loop_ns)) / frags,
            "shader_clock_GHz_in_the_loop": float(((clk[:, :4, 2] - clk[:, :4, 1]) / loop_ns).mean())},
        "serving": {
            "ring_prologue_ns": stats(srv[:, :, 1] - srv[:, :, 0]),
            "all_rounds_ns": stats(srv[:, :, 2] - srv[:, :, 1]),
            "last_sums_to_stores_issued_ns": stats(srv[:, :, 3] - srv[:, :, 2]),
            "stores_issued_to_stores_left_ns": stats(srv[:, :, 4] - srv[:, :, 3])},
        "end_after_first_wavefront_ns": stats(srv[:, :, 4] - t_first),
    }
    return {"workload": "BASELINE config 2 MFMA kernel (conv_i8_rs_kernel, %d fragments per tile): ceiling evidence" % frags,
            "mfma_probe": probe,
            "kernel_us": t_conv * 1e6, "kernel_us_with_stamps": t_stamped * 1e6,
            "kernel_TOP_per_s": conv_ops / t_conv / 1e12,
            "workgroups_with_stamps": int(st.shape[0]),
            "phases": phases,
            "fragment_mfma_cycles_per_simd": 36 * 32,
            "note": "wall clock = s_memrealtime (10 ns ticks), shader clock = s_memtime; the last position tile holds "
                    "fewer fragments than the others (it sets the minima); fragment_mfma_cycles_per_simd is what one "
                    "fragment's MFMAs alone occupy a SIMD's pipe for (36 v_mfma_i32_32x32x32_i8 x 32 cycles)"}


def tennis_runtime_leg(reps=5):
    """The ResNet-50-shaped network (BASELINE config 4) as a `.tsm` module through TenniS's own loader, graph compiler
    and Workbench on ComputingDevice("hip") -- the operator boundary as a TenniS user meets it (TenniS built with this
    repository's backend inside, tennis_amd/intree.py; absent where that library was not built)."""
    import tempfile
    from tennis_amd import intree, module_file as mf, resnet50
    if not intree.available():
        return None
    n = 32
    desc, params = resnet50.make_parameters(seed=0)
    module = resnet50.to_module(desc, params, batch=n)
    x = np.random.default_rng(1).random((n, 3, 224, 224), dtype=np.float32)
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "resnet50_int8_bs32.tsm")
        mf.write_module(path, module)
        fused0, hand0, host0 = intree.fused_chain_count(), intree.handover_counts(), intree.host_delegate_count()
        ms, logits = intree.time_module("hip", path, [x], warmup=2, reps=reps, resident=True)
        fused = intree.fused_chain_count() - fused0
        hand = tuple(a - b for a, b in zip(intree.handover_counts(), hand0))
        ms_upload, _ = intree.time_module("hip", path, [x], warmup=2, reps=reps, resident=False)
        host_runs = intree.host_delegate_count() - host0
    return {"workload": "BASELINE config 4 network as a .tsm module (every activation quantized with one fixed multiplier) "
                        "in TenniS's Workbench on device hip: quantize+conv+bias+relu chains (and residual joins) fused by "
                        "the backend's zipper option, int8 hand-over between fused nodes, fp32 inner_prod classifier; input "
                        "bound from device memory, each run ends with the logits on the host",
            "img_per_s": n / (ms * 1e-3), "ms_per_batch": ms, "reps": reps, "chains_fused_by_the_graph_compiler": fused,
            "int8_hand_overs": hand[0], "dual_output_nodes": hand[1],
            "operator_runs_handed_to_host_operators": host_runs,
            "ms_per_batch_input_uploaded_every_run": ms_upload,
            "logits_finite": bool(np.isfinite(logits).all())}


def resnet_leg(steps=20):
    """ResNet-50-shaped int8 network, batch 32 at 3x224x224 (BASELINE config 4): img/s of the whole forward pass,
    replayed from a captured HIP graph (the pass is 58 short kernels; capture removes the host launch cost)."""
    import torch
    from tennis_amd import resnet50
    n, size = 32, 224
    desc, params = resnet50.make_parameters(seed=0)
    net = resnet50.ResNet50Int8(desc, params)
    x = torch.rand((n, 3, size, size), device="cuda")
    net.set_scales(net.calibrate(x), n)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        net.forward(x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        logits = net.forward(x)
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    macs = resnet50.total_macs(desc, n, size)
    return {"workload": "BASELINE config 4: ResNet-50-shaped int8 network, batch 32, 3x224x224, random-init weights, "
                        "per-channel int8 weights, per-tensor int8 activations calibrated on the batch",
            "img_per_s": n / dt, "ms_per_batch": dt * 1e3, "TOPS": 2.0 * macs / dt / 1e12,
            "pct_of_int8_mfma_peak": 100.0 * 2.0 * macs / dt / 1e12 / PEAK_INT8_TOPS, "gmac_per_image": macs / n / 1e9,
            "steps": steps, "logits_finite": bool(torch.isfinite(logits).all().item())}


def yolo_leg(steps=5, mish="exact"):
    """YOLOv4-shaped int8 network, batch 8 at 3x608x608 (BASELINE config 5): img/s of the whole forward pass
    (three head tensors), replayed from a captured HIP graph.  mish = "exact": the Mish layers give the operator
    chain's values bit for bit (the default of the library); "fast": the opt-in one-exponential form."""
    import torch
    from tennis_amd import yolov4
    n, size = 8, 608
    L, heads = yolov4.layers()
    net = yolov4.YoloV4Int8(L, heads, yolov4.make_parameters(L, seed=0), mish=mish)
    x = torch.rand((n, 3, size, size), device="cuda")
    net.calibrate(x)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        net.forward(x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = net.forward(x)
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    macs = yolov4.total_macs(L, n, size)
    return {"workload": "BASELINE config 5: YOLOv4-shaped int8 network (CSPDarknet53 + SPP + PANet, Mish / LeakyReLU), "
                        "batch 8, 3x608x608, random-init weights, per-channel int8 weights, per-tensor int8 activations; "
                        "Mish in its %s form" % mish,
            "img_per_s": n / dt, "ms_per_batch": dt * 1e3, "TOPS": 2.0 * macs / dt / 1e12, "gmac_per_image": macs / n / 1e9,
            "steps": steps, "outputs_finite": bool(all(torch.isfinite(o).all().item() for o in outs))}


def gemm_leg(reps=20):
    """int8 GEMM sweep (BASELINE config 3): M in {1, 32, 256, 4096}, K = N in {1024, 2048, 4096}; one launch of
    tsx_gemm_i8 with per-row and per-output-channel dequantize scales and bias, fp32 output; GPU time per launch
    from a HIP-graph replay of `reps` launches."""
    import torch
    from tennis_amd import capi
    rows = []
    for k in (1024, 2048, 4096):
        n = k
        gemm = capi.GemmI8(torch.randint(-128, 128, (k, n), dtype=torch.int8, device="cuda"))
        dq = torch.rand(n, device="cuda") * 1e-2
        bias = torch.randn(n, device="cuda")
        for m in (1, 32, 256, 4096):
            a = torch.randint(-128, 128, (m, k), dtype=torch.int8, device="cuda")
            rs = torch.rand(m, device="cuda") * 1e-2
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                gemm(a, dq=dq, row_scale=rs, bias=bias)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(reps):
                    gemm(a, dq=dq, row_scale=rs, bias=bias)
            graph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(3):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e-3 / (3 * reps)
            ops = 2.0 * m * n * k
            nbytes = m * k + k * n + 4.0 * m * n + 4.0 * n
            # M <= 32 streams the weights once: HBM-bound; larger M is MFMA-bound
            rows.append({"m": m, "k": k, "n": n, "us": t * 1e6, "TOPS": ops / t / 1e12, "GBps": nbytes / t / 1e9,
                         "bound": "hbm" if m <= 32 else "mfma",
                         "frac": (nbytes / t / 1e9 / PEAK_HBM_GBS) if m <= 32 else (ops / t / 1e12 / PEAK_INT8_TOPS)})
    return {"workload": "BASELINE config 3: int8 GEMM sweep, per-row x per-output-channel dequantize + bias, fp32 out",
            "launches_per_figure": 3 * reps, "shapes": rows}



def kernels_leg(reps=20):
    """Every other kernel of the path on its own (for per-kernel counters under rocprofv3 and the figures next
    to BASELINE config 2): each is launched `reps` times back to back after 3 warm-up launches and timed with
    events on the launch stream.  `work` is algorithmic: ops for the MFMA-bound kernels, bytes for the HBM-bound."""
    import torch
    from tennis_amd import capi
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cuda").manual_seed(7)
    rnd = lambda *s: torch.randn(s, device=dev, generator=g)
    ri8 = lambda *s: torch.randint(-128, 128, s, dtype=torch.int8, device=dev, generator=g)
    rows = []

    def timed(name, bound, work, fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) * 1e-3 / reps
        peak = {"hbm": PEAK_HBM_GBS * 1e9, "mfma_i8": PEAK_INT8_TOPS * 1e12, "mfma_f32": PEAK_FP32_TFLOPS * 1e12}[bound]
        rows.append({"kernel": name, "bound": bound, "us": t * 1e6, "work": work, "achieved": work / t,
                     "unit": "B/s" if bound == "hbm" else "op/s", "frac": work / t / peak})

    # fp32 BASELINE config 1 (1x64x56x56 * 64x64x3x3, bias + ReLU): implicit GEMM and both Winograd modes
    x1, w1, b1 = torch.rand((1, 64, 56, 56), device=dev) * 2 - 1, rnd(64, 64, 3, 3) * 0.06, rnd(64) * 0.01
    flops1 = 2.0 * 64 * 56 * 56 * 64 * 9
    c1_launch, _ = capi.conv2d_f32_prepared(x1, w1, (1, 1, 1, 1), bias=b1, act="relu")
    timed("conv2d_f32 config 1 (conv3x3_f32_small_kernel)", "mfma_f32", flops1, c1_launch)
    w63, w23 = capi.WinogradF63(w1, (1, 1, 1, 1)), capi.WinogradF23(w1, (1, 1, 1, 1))
    timed("winograd F(6,3) config 1 (direct-conv flops)", "mfma_f32", flops1, lambda: w63(x1, bias=b1, act="relu"))
    timed("winograd F(2,3) config 1 (direct-conv flops)", "mfma_f32", flops1, lambda: w23(x1, bias=b1, act="relu"))
    # fp32 on a shape the reference's selector routes to Winograd F(6,3): 8x256x28x28 * 256x256x3x3
    x8, w8, b8 = torch.rand((8, 256, 28, 28), device=dev) * 2 - 1, rnd(256, 256, 3, 3) * 0.03, rnd(256) * 0.01
    flops8 = 2.0 * 8 * 256 * 28 * 28 * 256 * 9
    timed("conv2d_f32 8x256x28x28 (gemm_f32_kernel)", "mfma_f32", flops8, lambda: capi.conv2d_f32(x8, w8, (1, 1, 1, 1), bias=b8, act="relu"))
    w63b = capi.WinogradF63(w8, (1, 1, 1, 1))
    timed("winograd F(6,3) 8x256x28x28, bit-exact form (direct-conv flops)", "mfma_f32", flops8, lambda: w63b(x8, bias=b8, act="relu"))
    timed("winograd F(6,3) 8x256x28x28, one MFMA launch (direct-conv flops)", "mfma_f32", flops8,
          lambda: w63b(x8, bias=b8, act="relu", fast=True))
    # int8 GEMM: largest and a mid shape of BASELINE config 3, and the weight-streaming single row
    k = n = 4096
    gemm = capi.GemmI8(ri8(k, n))
    dq, bias = torch.rand(n, device=dev) * 1e-2, rnd(n)
    for m in (4096, 256, 1):
        a, rs = ri8(m, k), torch.rand(m, device=dev) * 1e-2
        if m > 32:
            timed("gemm_i8 M=%d K=N=4096 (%s)" % (m, "gemm_i8_ksplit_lds_kernel" if m <= 512 else "conv_i8_ws_kernel, row-major"),
                  "mfma_i8", 2.0 * m * n * k,
                  lambda a=a, rs=rs: gemm(a, dq=dq, row_scale=rs, bias=bias))
        else:
            timed("gemm_i8 M=%d K=N=4096 (gemm_i8_skinny_kernel)" % m, "hbm", m * k + k * n + 4.0 * m * n + 4.0 * n,
                  lambda a=a, rs=rs: gemm(a, dq=dq, row_scale=rs, bias=bias))
    # memory-bound 1x1 int8 layer (ResNet stage 1 expansion, 64 -> 256 channels at 56x56, batch 32), staged int8 in, fp32 out
    xq = ri8(32, 64, 56, 56)
    c11 = capi.Conv2dI8(ri8(256, 64, 1, 1))
    dq11, b11 = torch.rand(256, device=dev) * 1e-3, rnd(256)
    st = capi.StagedInput(c11, xq.shape)
    c11.stage(xq, st)
    ws_bytes = c11._plan(tuple(xq.shape))[2]
    timed("conv2d_i8 1x1 64->256 @56x56 bs32, fp32 out (conv_i8_ws_kernel)", "hbm", float(ws_bytes) + 4.0 * 32 * 256 * 56 * 56,
          lambda: c11.run_staged(st, dq11, b11, "relu"))
    # HBM-bound glue on a 32x256x56x56 fp32 tensor (103 MB)
    x = rnd(32, 256, 56, 56)
    nb = 4.0 * x.numel()
    wd = rnd(1, 256, 3, 3)
    timed("depthwise_conv2d 3x3 s1 p1", "hbm", 2 * nb, lambda: capi.depthwise_conv2d(x, wd, (1, 1, 1, 1)))
    timed("relu", "hbm", 2 * nb, lambda: capi.relu(x))
    bb = rnd(256)
    timed("add_bias", "hbm", 2 * nb, lambda: capi.add_bias(x, bb))
    x2 = rnd(32, 256, 56, 56)
    timed("add + relu (residual join)", "hbm", 3 * nb, lambda: capi.add(x, x2, act="relu"))
    qs = torch.full((32,), 20.0, device=dev)
    timed("quantize", "hbm", 1.25 * nb, lambda: capi.quantize(x, qs))
    timed("pooling2d max 3x3 s2 p1", "hbm", 1.25 * nb, lambda: capi.pooling2d(x, "max", (3, 3), (2, 2), (1, 1, 1, 1)))
    return {"workload": "kernels of the path one by one; time per launch includes the wrapper's output allocation from "
                        "torch's caching allocator (no device allocation in steady state)", "reps": reps, "kernels": rows}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-images", type=int, default=32, help="images of the batch timed on the CPU (0 = skip)")
    ap.add_argument("--no-resnet", action="store_true", help="skip the ResNet-50-shaped network leg")
    ap.add_argument("--no-yolo", action="store_true", help="skip the YOLOv4-shaped network leg")
    ap.add_argument("--no-gemm", action="store_true", help="skip the int8 GEMM sweep leg")
    ap.add_argument("--ceiling", action="store_true",
                    help="only the ceiling evidence of the config-2 MFMA kernel: MFMA probe rates and per-phase stamps")
    ap.add_argument("--profile", action="store_true",
                    help="for runs under a profiler: skip the int8-output variant (same kernel name as the roofline "
                         "kernel), the MFMA-rate probe and the CPU baseline, so per-kernel statistics cover the timed "
                         "kernels only")
    ap.add_argument("--network", choices=("resnet", "yolo", "yolo_fast_mish", "tennis"),
                    help="run only that network leg and print its figures (for per-kernel profiles of a network); "
                         "tennis = the ResNet-50-shaped module through TenniS's own runtime on device hip")
    ap.add_argument("--kernels", action="store_true",
                    help="run only the one-by-one kernel leg (GEMM, fp32, Winograd, 1x1, depthwise, elementwise, pooling) "
                         "and print its figures (for per-kernel counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    from tennis_amd import capi
    import ctypes

    if not torch.cuda.is_available():
        print("bench.py needs the MI355X (no CPU fallback)", file=sys.stderr)
        sys.exit(3)
    L = capi.lib()
    dev = torch.device("cuda:0")
    if args.network:
        leg = {"resnet": resnet_leg, "yolo": yolo_leg, "yolo_fast_mish": lambda: yolo_leg(mish="fast"),
               "tennis": tennis_runtime_leg}[args.network]
        print(json.dumps(leg()))
        return
    if args.kernels:
        print(json.dumps(kernels_leg()))
        return
    cfg = CFG
    x, x_scales, wq, dq, bias = make_inputs(cfg)
    pad = cfg["pad"]

    xd = torch.from_numpy(x).to(dev)
    xsd = torch.from_numpy(x_scales).to(dev)
    conv = capi.Conv2dI8(torch.from_numpy(wq).to(dev), (pad,) * 4)
    ep = capi._EpilogueArgs(torch.from_numpy(dq).to(dev), torch.from_numpy(bias).to(dev), "relu")
    geom, packed, ws_bytes = conv._plan(tuple(xd.shape))
    ho, wo = capi.conv_out_size(geom)
    out = torch.empty((cfg["n"], cfg["cout"], ho, wo), dtype=torch.float32, device=dev)
    ws = conv._workspace
    stream = capi._stream()
    g = ctypes.byref(geom)
    epp = ctypes.byref(ep.c)

    def step():
        capi.check(L.tsx_quantize_conv2d_i8_nchw(g, capi._ptr(xd), capi._ptr(xsd), xsd.numel(), capi._ptr(packed), 0.0,
                                                 epp, capi._ptr(out), None, None, capi._ptr(ws), ws_bytes, stream))

    def stage_only():
        capi.check(L.tsx_conv2d_i8_stage(g, capi._ptr(xd), 1, capi._ptr(xsd), xsd.numel(), 0.0, capi._ptr(ws), ws_bytes,
                                         stream))

    def mfma_only():
        capi.check(L.tsx_conv2d_i8_staged(g, capi._ptr(ws), capi._ptr(packed), epp, capi._ptr(out), None, None, stream))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    launch_mode = "direct C-ABI calls on one stream"

    # The same step captured once in a HIP graph and replayed: what a serving loop that fixes its shapes does.
    # Reported beside the direct-call time, which is the step time `value` is computed from.
    ms_direct, ms_graph = ms_per_step, None
    if not args.profile:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            capi.check(L.tsx_quantize_conv2d_i8_nchw(g, capi._ptr(xd), capi._ptr(xsd), xsd.numel(), capi._ptr(packed), 0.0, epp,
                                                     capi._ptr(out), None, None, capi._ptr(ws), ws_bytes, capi._stream()))
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            capi.check(L.tsx_quantize_conv2d_i8_nchw(g, capi._ptr(xd), capi._ptr(xsd), xsd.numel(), capi._ptr(packed), 0.0, epp,
                                                     capi._ptr(out), None, None, capi._ptr(ws), ws_bytes, capi._stream()))
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        ms_graph = (time.perf_counter() - t0) / args.steps * 1e3

    def event_time(fn, reps):
        """Seconds per launch: the median over 5 batches of `reps` back-to-back launches, each batch bracketed by
        events on the launch stream."""
        fn()
        torch.cuda.synchronize()
        per = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            per.append(e0.elapsed_time(e1) / reps * 1e-3)
        return float(np.median(per))

    if args.ceiling:
        A = capi.aids_lib()
        if A is None:
            print("bench.py --ceiling needs the measurement build: python -m tennis_amd.build --aids", file=sys.stderr)
            sys.exit(4)
        info = capi.conv2d_i8_plan_info(geom)
        if info["fp32_kernel"] != "weight_stationary":
            print("bench.py --ceiling reads the weight-stationary kernel's stamps; the plan is %r" % (info,), file=sys.stderr)
            sys.exit(4)

        def mfma_only_aids():
            capi.check(A.tsx_conv2d_i8_staged(g, capi._ptr(ws), capi._ptr(packed), epp, capi._ptr(out), None, None, stream))

        conv_ops = 2.0 * cfg["n"] * cfg["cout"] * ho * wo * cfg["c"] * cfg["k"] * cfg["k"]
        print(json.dumps(ceiling_evidence(A, mfma_only_aids, event_time, conv_ops, dev, stream, int(info["fragments_per_tile"]))))
        return

    reps = max(args.steps, 100)
    t_mfma = event_time(mfma_only, reps)
    t_stage = event_time(stage_only, reps)

    # Same MFMA kernel with the requantized int8 output a following quantized layer would consume
    # (quarter of the output bytes): reported beside the fp32-output figure, not instead of it.
    qs = torch.full((cfg["n"],), 20.0, dtype=torch.float32, device=dev)
    ep_q = capi._EpilogueArgs(torch.from_numpy(dq).to(dev), torch.from_numpy(bias).to(dev), "relu", q_scales=qs)
    out_q = torch.empty((cfg["n"], cfg["cout"], ho, wo), dtype=torch.int8, device=dev)

    def mfma_int8_out():
        capi.check(L.tsx_conv2d_i8_staged(g, capi._ptr(ws), capi._ptr(packed), ctypes.byref(ep_q.c), None, capi._ptr(out_q),
                                          None, stream))

    t_mfma_q = None if args.profile else event_time(mfma_int8_out, reps)

    # The int8 MFMA rate this part sustains with operands of the same statistics (register-only loop):
    # the practical ceiling below the nominal 5.0 POP/s.
    operands = torch.randint(-128, 128, (32768,), dtype=torch.int8, device=dev)
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    probe_iters, probe_blocks = 20000, 512

    A = None if args.profile else capi.aids_lib()      # the measurement build holds the probe kernel

    def probe():
        capi.check(A.tsx_probe_mfma_i8(capi._ptr(operands), probe_iters, probe_blocks, capi._ptr(sink), stream))

    t_probe = event_time(probe, 3) if A is not None else None
    sustained_tops = probe_blocks * 4 * probe_iters * 8 * 65536.0 / t_probe / 1e12 if A is not None else None

    # One device copy of known size: the dispatch the HBM counters of a profiler run are scaled by.
    calib_src = torch.empty(64 << 20, dtype=torch.uint8, device=dev).fill_(1)
    calib_dst = torch.empty_like(calib_src)
    for _ in range(3):
        calib_dst.copy_(calib_src)
    torch.cuda.synchronize()

    stage_bytes = 4.0 * x.size + float(ws_bytes)
    # What the device's own copy reaches on a transfer of the staging kernel's size (half read, half written): the
    # practical HBM rate for a single launch this small, launch and ramp included -- the figure to hold the staging
    # kernel's rate against, next to the 8 TB/s peak.
    half = int(stage_bytes) // 2
    copy_src = torch.empty(half, dtype=torch.uint8, device=dev).fill_(3)
    copy_dst = torch.empty_like(copy_src)
    t_copy = event_time(lambda: copy_dst.copy_(copy_src), reps)

    macs = cfg["n"] * cfg["cout"] * ho * wo * cfg["c"] * cfg["k"] * cfg["k"]
    ops = 2.0 * macs
    mfma_kernel = {"weight_stationary": "conv_i8_rs_kernel", "flat_tile": "conv_i8_fl_kernel",
                   "window_stationary": "conv_i8_ws_kernel", "igemm": "igemm_i8_kernel"}[capi.conv2d_i8_plan_info(geom)["fp32_kernel"]]
    tops = ops / (ms_per_step * 1e-3) / 1e12
    kernel_tops = ops / t_mfma / 1e12

    result = {
        "metric": "int8 conv2d TOPS & % MFMA peak; ResNet-50-shape img/s at bs=32, 1 MI355X",
        "value": tops,
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 x int8 -> int32 (fp32 epilogue)",
        "data": "synthetic",
        "config": {"workload": "BASELINE config 2: int8 conv2d 32x256x28x28 * 256x256x3x3 s1 p1, fp32 dequant+bias+ReLU "
                               "out; step = quantize+stage kernel + i8-MFMA implicit-GEMM kernel",
                   "algorithmic_ops_per_step": ops, "pct_of_int8_mfma_peak_whole_step": 100.0 * tops / PEAK_INT8_TOPS,
                   "launch": launch_mode, "ms_per_step_direct_calls": ms_direct, "ms_per_step_graph_replay": ms_graph},
        "roofline": {"bound": "mfma", "kernel": mfma_kernel, "achieved": kernel_tops, "peak": PEAK_INT8_TOPS,
                     "unit": "TOP/s", "frac": kernel_tops / PEAK_INT8_TOPS, "traffic": TRAFFIC_CONV_BYTES,
                     "traffic_unit": "HBM bytes per launch, a constant taken from rocprofv3 FETCH_SIZE / WRITE_SIZE of this "
                                     "kernel on this workload (profiles/conv2d_i8_config2_hbm_traffic.txt), not measured "
                                     "by this run; algorithmic 33.65e6",
                     "note": "int8 multiply-accumulate ops (TOP/s); 2*N*Cout*Ho*Wo*Cin*9 = %.4g ops per launch, "
                             "launch %.2f us = median of 5 batches of %d back-to-back launches" % (ops, t_mfma * 1e6, reps)},
        "sustained_mfma": None if sustained_tops is None else {
            "value": sustained_tops, "unit": "TOPS", "frac_of_it": kernel_tops / sustained_tops,
            "note": "register-only v_mfma_i32_32x32x32_i8 loop on random int8 operands, measured in this "
                    "run: the rate the part sustains under load (clocks drop with operand activity)"},
        "int8_output_variant": None if args.profile else {
            "achieved": ops / t_mfma_q / 1e12, "unit": "TOPS", "us": t_mfma_q * 1e6,
            "note": "same kernel, epilogue requantizes to int8 for a following quantized layer"},
        "stage_kernel": {"bound": "hbm", "kernel": "stage_rows_kernel<quantize>", "achieved": stage_bytes / t_stage / 1e9,
                         "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": stage_bytes / t_stage / 1e9 / PEAK_HBM_GBS,
                         "us": t_stage * 1e6, "bytes": stage_bytes, "traffic": TRAFFIC_STAGE_BYTES,
                         "device_copy_of_the_same_bytes": {"us": t_copy * 1e6, "GB_per_s": 2.0 * half / t_copy / 1e9,
                                                           "note": "torch copy_ of %d bytes device to device (read + "
                                                                   "written = the staging kernel's bytes), timed the "
                                                                   "same way" % half}},
    }
    if not args.no_resnet and not args.profile:
        result["resnet50_int8_bs32"] = resnet_leg()
    if not args.no_yolo and not args.profile:
        result["yolov4_int8_bs8"] = yolo_leg(mish="exact")
        result["yolov4_int8_bs8_fast_mish"] = yolo_leg(mish="fast")
    if not args.no_gemm and not args.profile:
        result["gemm_i8_sweep"] = gemm_leg()
    if not args.profile:
        result["conv2d_f32_config1"] = config1_leg()
        result["conv2d_f32_winograd_shape"] = winograd_shape_leg()
    if not args.no_resnet and not args.profile:
        result["resnet50_int8_bs32_tennis_runtime"] = tennis_runtime_leg()
    if args.cpu_images > 0 and not args.profile:
        result["cpu_baseline"] = cpu_baseline(x, x_scales, wq, dq, bias, pad, min(args.cpu_images, cfg["n"]))
        result["cpu_baseline_openmp_all"] = cpu_baseline_all_cores(x, x_scales, wq, dq, bias, pad)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
