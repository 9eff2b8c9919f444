#!/usr/bin/env python3
"""Benchmark of the Winograd F(2x2,3x3) forward convolution on one MI355X.

A "step" is one call of the reference's entry point ``convolutionForward`` (filter
transform + fused kernel, the quantity the reference times at
src/openCNN_winograd.cu:426-444) on one seeded synthetic layer resident in HBM.

Prints ONE JSON line: effective TFLOP/s (direct-convolution FLOPs 2*N*K*C*H*W*9 per
step), ms per layer, the roofline of the dominant kernel (fp32 MFMA, algorithmic
flops 32*N*T*C*K per launch) and a CPU baseline (the fp64 direct convolution of the
oracle on the host cores).  ``layers`` repeats the figures for every fp32 layer of the
benchmark set, in the sustained state and (``from_idle_*``) under the reference's own protocol of
one warm-up call and 100 timed calls from an idle device; only ``config.workload`` is the timed
K-step region.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3  # MI355X dense fp32 matrix peak
PEAK_F16_MFMA_TFLOPS = 2500.0  # dense fp16 / bf16 matrix peak
PEAK_HBM_GBS = 8000.0

# name -> (N, C, H=W, K, input range, filter distribution)
LAYERS = {
    "plumbing_n32_c8_h8_k64": (32, 8, 8, 64, (-1.0, 1.0), "uniform"),
    "resnet_n64_c64_h56_k64": (64, 64, 56, 64, (-1.0, 1.0), "he"),
    "resnet_n128_c128_h28_k128": (128, 128, 28, 128, (-1.0, 1.0), "he"),
    "deep_n128_c256_h14_k256": (128, 256, 14, 256, (0.0, 1.0), "he"),
    "deep_n128_c512_h7_k512": (128, 512, 7, 512, (0.0, 1.0), "he"),
    # reduced-precision configuration: fp16 / bf16 GEMM operands, fp32 transforms and accumulation
    "reduced_n128_c256_h14_k256": (128, 256, 14, 256, (-1.0, 1.0), "he"),
}
FP32_LAYERS = [k for k in LAYERS if not k.startswith("reduced")]
DEFAULT_WORKLOAD = "resnet_n64_c64_h56_k64"

# HBM bytes per launch of the fused kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs:
# profiles/traffic.json, written when the profiles are refreshed, with the commit the kernels
# were measured at (a later change of a kernel makes its entry stale: compare with HEAD).
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def measured_traffic(key):
    """(bytes per launch, commit they were measured at), or (None, None)."""
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None, None
    row = table.get("workloads", {}).get(key)
    return (row["traffic_bytes"], table.get("commit")) if row else (None, None)


def custom_layer(spec):
    """--shape N,C,H,K -> a workload of that shape (uniform[-1,1] input, He-init filters)."""
    n, c, h, k = (int(v) for v in spec.split(","))
    name = f"custom_n{n}_c{c}_h{h}_k{k}"
    LAYERS[name] = (n, c, h, k, (-1.0, 1.0), "he")
    return name


def work(N, C, H, K):
    T = ((H + 1) // 2) ** 2
    flops_direct = 2.0 * N * K * C * H * H * 9
    flops_mfma = 32.0 * N * T * C * K
    bytes_min = 4.0 * (N * C * H * H + 9 * K * C + 2 * 16 * K * C + N * K * H * H)
    return flops_direct, flops_mfma, bytes_min


class Layer:
    def __init__(self, ocn, torch, name):
        self.name = name
        self.N, self.C, self.H, self.K, xr, filt = LAYERS[name]
        self.x_host = ocn.synth_input(self.N, self.C, self.H, self.H, seed=0x0C99, p0=xr[0], p1=xr[1])
        if filt == "he":
            self.w_host = ocn.synth_filter(self.K, self.C, seed=0xF117)
        else:
            self.w_host = ocn.synth_filter(self.K, self.C, seed=0xF117, dist=ocn.DIST_UNIFORM,
                                           p0=-1.0, p1=1.0)
        dev = torch.device("cuda:0")
        self.x = torch.from_numpy(self.x_host).to(dev)
        self.w = torch.from_numpy(self.w_host).to(dev)
        self.y = torch.empty((self.K, self.H, self.H, self.N), device=dev)
        self.ws = torch.empty(ocn.workspace_bytes(self.C, self.K) // 4, device=dev)
        self.ocn = ocn
        self.td = ocn.tiles_dim(self.H)

    def step(self):
        o = self
        self.ocn.convolutionForward(o.x, o.H, o.H, o.w, o.H, o.H, o.N, o.K, o.y, o.ws,
                                    o.K * o.N * o.H * o.H, o.td, o.N, 4, o.td * 4, o.C, o.K,
                                    o.C, 3, 3, 4, 2)

    def kernel_times(self, warmup, iters, parts=("total", "main", "fx")):
        """HIP-event mean ms per call on the library's stream: (fx+main, main, fx)."""
        return self.ocn.time_forward(self.x, self.w, self.y, self.ws, self.N, self.C, self.H,
                                     self.H, self.K, warmup=warmup, iters=iters, parts=parts)


def from_idle(torch, lay, flops_mfma, peak, idle_s=0.5):
    """The reference's own protocol (src/openCNN_winograd.cu:426-444): one warm-up call, then 100
    back-to-back calls between two events, starting from an idle device - no settle phase.  Once
    for the whole call (filter transform + fused kernel) and, after another idle period, once
    for the fused kernel alone."""
    torch.cuda.synchronize()
    time.sleep(idle_s)
    total, _, _ = lay.kernel_times(1, 100, parts=("total",))
    time.sleep(idle_s)
    _, main, _ = lay.kernel_times(1, 100, parts=("main",))
    return {"protocol": "0.5 s idle, 1 warm-up call, 100 timed calls (HIP events), as the reference's bench",
            "ms_per_step": total, "ms_fused_kernel": main,
            "frac": flops_mfma / (main * 1e-3) / 1e12 / peak}


def settle(torch, lay, ms):
    """Untimed: run the step back to back for `ms` of wall time.  After an idle period (tensor
    set-up, the CPU leg) the device needs some tens of milliseconds of continuous work before
    its clocks and its launch path are in their sustained state; a layer of a network runs in
    that state, so every timed region here starts from it."""
    t_end = time.perf_counter() + ms * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(200):
            lay.step()
        torch.cuda.synchronize()


def shim_rows(ocn, torch, lay, iters=200):
    """The layout shims (NCHW -> CHWN, KHWN -> NKHW, KCRS -> CRSK; they replace the reference's
    data_cpy, src/openCNN_winograd.cu:147-153) and the filter transform on this layer: HBM-bound
    kernels, algorithmic bytes = one read + one write of every element (filter transform: 36 B
    read + 64 B written per (c, k)).  Timed with events on the null stream, which is the stream the
    library launches on unless opencnn_set_stream says otherwise."""
    o = lay
    dev = o.x.device
    nchw = torch.rand((o.N, o.C, o.H, o.H), device=dev)
    nkhw = torch.empty((o.N, o.K, o.H, o.H), device=dev)
    kcrs = torch.rand((o.K, o.C, 3, 3), device=dev)
    crsk = torch.empty((o.C, 3, 3, o.K), device=dev)
    chwn = torch.empty_like(o.x)
    cases = [
        ("nchw_to_chwn", lambda: ocn.nchw_to_chwn(nchw, chwn, o.N, o.C, o.H, o.H), 8.0 * nchw.numel()),
        ("khwn_to_nkhw", lambda: ocn.khwn_to_nkhw(o.y, nkhw, o.N, o.K, o.H, o.H), 8.0 * nkhw.numel()),
        ("kcrs_to_crsk", lambda: ocn.kcrs_to_crsk(kcrs, crsk, o.K, o.C), 8.0 * kcrs.numel()),
        ("filter_transform", lambda: ocn.filter_transform(o.w, o.ws, o.K, o.C, ocn.FILTER_CRSK, ocn.WW_MFMA),
         100.0 * o.K * o.C),
    ]
    rows = []
    for name, fn, nbytes in cases:
        for _ in range(iters):  # also the settle phase of this kernel
            fn()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        ev[0].record()
        for _ in range(iters):
            fn()
        ev[1].record()
        torch.cuda.synchronize()
        ms = ev[0].elapsed_time(ev[1]) / iters
        rows.append({"workload": o.name, "kernel": name, "us": ms * 1e3, "bytes": nbytes,
                     "gbs": nbytes / (ms * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS})
    return rows


def miopen_column(torch, lay, warmup=10, iters=200, settle_ms=150.0):
    """Informational only, never an oracle: ms per call of torch.nn.functional.conv2d (MIOpen's
    own choice of fp32 algorithm) on the same layer in NCHW / KCRS, the analogue of the
    reference bench's cuDNN column (src/openCNN_winograd.cu:449-464)."""
    x = lay.x.permute(3, 0, 1, 2).contiguous()
    w = lay.w.permute(3, 0, 1, 2).contiguous()
    torch.backends.cudnn.benchmark = True  # let MIOpen search instead of taking its first guess
    for _ in range(warmup):
        y = torch.nn.functional.conv2d(x, w, padding=1)
    torch.cuda.synchronize()
    t_end = time.perf_counter() + settle_ms * 1e-3  # same sustained state as the library's column
    while time.perf_counter() < t_end:
        for _ in range(100):
            y = torch.nn.functional.conv2d(x, w, padding=1)
        torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    ev[0].record()
    for _ in range(iters):
        y = torch.nn.functional.conv2d(x, w, padding=1)
    ev[1].record()
    torch.cuda.synchronize()
    del y
    return ev[0].elapsed_time(ev[1]) / iters


# (C, K, H = W, how many) of the 3x3 stride-1 layers of two networks
NETWORKS = {
    "resnet34": [(64, 64, 56, 6), (128, 128, 28, 7), (256, 256, 14, 11), (512, 512, 7, 5)],
    "vgg16": [(3, 64, 224, 1), (64, 64, 224, 1), (64, 128, 112, 1), (128, 128, 112, 1), (128, 256, 56, 1),
              (256, 256, 56, 2), (256, 512, 28, 1), (512, 512, 28, 2), (512, 512, 14, 3)],
}
NETWORK_BATCHES = (("resnet34", 128), ("resnet34", 32), ("resnet34", 8), ("vgg16", 64), ("vgg16", 16))


def network_rows(ocn, torch):
    """Informational: every 3x3 stride-1 layer of a network timed on its own in the sustained
    state (this library with fp32 and with fp16 GEMM operands; torch conv2d = MIOpen on fp32 and
    on half tensors), ms summed with the layer counts.  Never an oracle."""
    import numpy as np

    def ours(N, C, H, K, prec):
        x = torch.rand(C, H, H, N, device="cuda") * 2 - 1
        w = torch.randn(C, 3, 3, K, device="cuda") * float(np.sqrt(2 / (9 * C)))
        y = torch.empty(K, H, H, N, device="cuda")
        ws = torch.empty(ocn.workspace_bytes(C, K) // 4, device="cuda")
        iters = int(max(30, min(1000, 0.15 / (2.0 * N * K * C * H * H * 9 / 200e12))))
        try:
            ocn.set_operand_precision(prec)
            ocn.time_forward(x, w, y, ws, N, C, H, H, K, warmup=3, iters=iters)  # settles the device
            total, _, _ = ocn.time_forward(x, w, y, ws, N, C, H, H, K, warmup=3, iters=iters)
        finally:
            ocn.set_operand_precision(ocn.F32)
        return total, ocn.last_kernel()

    def miopen(N, C, H, K, dtype):
        x = (torch.rand(N, C, H, H, device="cuda") * 2 - 1).to(dtype)
        w = (torch.randn(K, C, 3, 3, device="cuda") * float(np.sqrt(2 / (9 * C)))).to(dtype)
        torch.backends.cudnn.benchmark = True
        iters = int(max(30, min(1000, 0.15 / (2.0 * N * K * C * H * H * 9 / 100e12))))
        for _ in range(10):
            torch.nn.functional.conv2d(x, w, padding=1)
        torch.cuda.synchronize()
        for _ in range(2):  # the first pass settles the device
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
            ev[0].record()
            for _ in range(iters):
                torch.nn.functional.conv2d(x, w, padding=1)
            ev[1].record()
            torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / iters

    rows = []
    for net, N in NETWORK_BATCHES:
        row = {"network": net, "N": N, "ms_fp32": 0.0, "ms_fp16_operands": 0.0, "ms_miopen_fp32": 0.0,
               "ms_miopen_fp16_tensors": 0.0, "layers": []}
        for C, K, H, count in NETWORKS[net]:
            a, ka = ours(N, C, H, K, ocn.F32)
            b, kb = ours(N, C, H, K, ocn.F16)
            m32, m16 = miopen(N, C, H, K, torch.float32), miopen(N, C, H, K, torch.float16)
            row["layers"].append({"C": C, "K": K, "H": H, "count": count, "ms_fp32": a, "ms_fp16_operands": b,
                                  "ms_miopen_fp32": m32, "ms_miopen_fp16_tensors": m16,
                                  "kernel_fp32": ka, "kernel_fp16_operands": kb})
            row["ms_fp32"] += a * count
            row["ms_fp16_operands"] += b * count
            row["ms_miopen_fp32"] += m32 * count
            row["ms_miopen_fp16_tensors"] += m16 * count
            print(f"bench.py --networks: {net} N={N} {C}->{K} {H}x{H}: {a:.4f} / {b:.4f} ms, "
                  f"MIOpen {m32:.4f} / {m16:.4f} ms", file=sys.stderr, flush=True)  # a long run stays audible
        rows.append(row)
    return rows


def timeline_summary(ocn, torch, lay, launches=20, operands="f32", settle_ms=150.0):
    """Where a launch of the assembly kernels spends its time: per-workgroup stamps (kernel start,
    end of the prologue, before / after every output transform) of the last of `launches`
    back-to-back launches with pre-transformed filters that follow `settle_ms` of untimed ones,
    summarised in microseconds."""
    import numpy as np

    o = lay
    buf = torch.zeros(1024 * 64, dtype=torch.int64, device=o.x.device)
    try:
        ocn.set_operand_precision({"f32": ocn.F32, "f16": ocn.F16, "bf16": ocn.BF16}[operands])
        ocn.filter_transform(o.w, o.ws, o.K, o.C, ocn.FILTER_CRSK, ocn.WW_MFMA)
        t_end = time.perf_counter() + settle_ms * 1e-3  # the sustained state, as for every timed region
        while time.perf_counter() < t_end:
            for _ in range(200):
                ocn.conv_forward_pretransformed(o.x, o.ws, o.y, o.N, o.C, o.H, o.H, o.K)
            torch.cuda.synchronize()
        ocn.set_timeline_buffer(buf)
        for _ in range(launches):
            ocn.conv_forward_pretransformed(o.x, o.ws, o.y, o.N, o.C, o.H, o.H, o.K)
        torch.cuda.synchronize()
    finally:
        ocn.set_timeline_buffer(None)
        ocn.set_operand_precision(ocn.F32)
    nwg = int((buf.cpu().numpy().reshape(-1, 64)[:, 0] > 0).sum())
    if nwg == 0:
        return {"workload": o.name, "recorded_workgroups": 0}
    t = [np.array(v) for v in ocn.read_timeline(buf, nwg)]
    ends = np.array([v[-1] for v in t])
    segs, epis = [], []
    for v in t:
        d = np.diff(v)          # prologue, then (segment, output transform) pairs
        segs += d[1::2].tolist()
        epis += d[2::2].tolist()
    segs, epis = np.array(segs), np.array(epis)
    chunks = o.C // (8 if operands == "f32" else 16)
    return {
        "workload": o.name, "recorded_workgroups": nwg,
        "kernel_span_us": float(ends.max()),
        "workgroup_end_us": {"min": float(ends.min()), "mean": float(ends.mean()), "max": float(ends.max())},
        "prologue_us_mean": float(np.mean([v[1] - v[0] for v in t])),
        "whole_tile_us_median": float(np.median(segs[segs > 0.75 * segs.max()])),
        "chunks_per_tile": chunks,
        "output_transform_us_median": float(np.median(epis)),
        "segments_per_workgroup_mean": float(np.mean([(len(v) - 2) // 2 for v in t])),
    }


def cpu_baseline(layer):
    """The oracle's fp64 direct convolution on the host cores: one warm pass, then whole-layer
    passes for about three seconds."""
    from oracle import oracle

    # bounded sample: the layer itself when it is small enough, else its first images
    n = layer.N
    x = layer.x_host[..., :n]
    oracle.direct_conv_f64(x[..., :32], layer.w_host)  # warm (threads, pages)
    passes, t0 = 0, time.perf_counter()
    while passes < 3 or time.perf_counter() - t0 < 3.0:  # a few seconds of CPU work
        y = oracle.direct_conv_f64(x, layer.w_host)
        passes += 1
    dt = (time.perf_counter() - t0) / passes
    flops = 2.0 * n * layer.K * layer.C * layer.H * layer.H * 9
    return y, {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": oracle.num_threads(),
        "kind": "port",
        "sample": f"fp64 direct convolution of the whole {layer.name} layer ({n} images), "
                  f"1 warm-up + {passes} timed passes, {dt * 1e3:.0f} ms each",
        "ms_per_layer": dt * 1e3,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(LAYERS))
    ap.add_argument("--shape", default=None, metavar="N,C,H,K",
                    help="time a layer of this shape instead of a named workload (for profiles of "
                         "shapes outside the benchmark set)")
    ap.add_argument("--operands", default="f32", choices=["f32", "f16", "bf16"],
                    help="GEMM operand precision of the timed workload (fp32 transforms and "
                         "accumulation in every case); the default is the reference's fp32")
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="untimed back-to-back run before every measurement (0: measure from idle)")
    ap.add_argument("--tile-order", type=int, default=None, metavar="BITS",
                    help="opencnn_set_tile_order for this run (measurements of the tile order; default: "
                         "the library's)")
    ap.add_argument("--range-weight", type=int, default=None, metavar="HALF_UNITS",
                    help="opencnn_set_range_weight for this run (weight of a tile end on the line the "
                         "balanced split cuts its ranges from; default: the library's choice)")
    ap.add_argument("--library", default=None, metavar="PATH",
                    help="time another build of the library (make -C opencnn_amd/csrc diagnostic: "
                         "kernels with parts of their work removed, WRONG RESULTS); the line says so")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-layers", action="store_true", help="skip the per-layer table")
    ap.add_argument("--timeline", action="store_true",
                    help="add the assembly kernels' per-workgroup timeline of the workload (and of every "
                         "fp32 layer of the table) to the output")
    ap.add_argument("--shims", action="store_true",
                    help="add the layout shims and the filter transform (HBM-bound kernels) of every "
                         "fp32 layer to the output")
    ap.add_argument("--networks", action="store_true",
                    help="add the summed 3x3 layers of ResNet-34 and VGG-16 at several batch sizes, with "
                         "informational MIOpen columns (takes about a minute)")
    ap.add_argument("--miopen", action="store_true",
                    help="add an informational MIOpen (torch conv2d, fp32) column to the per-layer table")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on ONE GPU (a single layer on one device, no "
                 "collectives); run it with --gpus 1")

    import torch

    import opencnn_amd as ocn

    ocn.load_library()  # raises if the HIP library is not built: there is no other path
    if args.library:
        ocn.use_library(args.library)
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    ocn.init()
    if args.tile_order is not None:
        ocn.set_tile_order(args.tile_order)
    if args.range_weight is not None:
        ocn.set_range_weight(args.range_weight)

    if args.shape:
        args.workload = custom_layer(args.shape)
    layer = Layer(ocn, torch, args.workload)
    fd, fm, bmin = work(layer.N, layer.C, layer.H, layer.K)
    reduced = args.operands != "f32"
    if reduced:
        ocn.set_operand_precision(ocn.F16 if args.operands == "f16" else ocn.BF16)
    peak = PEAK_F16_MFMA_TFLOPS if reduced else PEAK_FP32_MFMA_TFLOPS

    idle = from_idle(torch, layer, fm, peak)  # first: nothing has run on the device yet
    settle(torch, layer, args.settle_ms)
    for _ in range(args.warmup):
        layer.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        layer.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_step = dt * 1e3 / args.steps

    # dominant kernel, HIP events on the launch stream, same number of launches
    _, ms_main, ms_fx = layer.kernel_times(args.warmup, args.steps)
    achieved = fm / (ms_main * 1e-3) / 1e12
    traffic, traffic_commit = measured_traffic(layer.name + ("_" + args.operands if reduced else ""))
    kernel_name = ocn.last_kernel()
    grid, flag_set = ocn.last_launch()
    ocn.set_operand_precision(ocn.F32)
    ocn.check_status()  # raises if any launch so far gave up a hand-over between workgroups

    out = {
        "metric": "effective TFLOP/s (direct-conv FLOPs 2*N*K*C*H*W*9) of one 3x3 layer, "
                  "filter transform + fused Winograd kernel per call",
        "value": fd / (ms_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": args.settle_ms,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.operands,
        "data": "synthetic",
        "config": {"workload": layer.name, "N": layer.N, "C": layer.C, "H": layer.H,
                   "W": layer.H, "K": layer.K, "pad": 1, "stride": 1,
                   "layout": "CHWN in, CRSK filters, KHWN out",
                   **({"tile_order": args.tile_order} if args.tile_order is not None else {}),
                   **({"range_weight": args.range_weight} if args.range_weight is not None else {})},
        "roofline": {
            "kernel": kernel_name + " (fused Winograd kernel), %d workgroups, flag set %d" % (grid, flag_set),
            "bound": "mfma",
            "achieved": achieved,
            "peak": peak,
            "unit": "TFLOP/s",
            "frac": achieved / peak,
            "traffic": traffic,
            "traffic_commit": traffic_commit,
            "flops_per_launch": fm,
            "ms_per_launch": ms_main,
            "hbm_min_bytes": bmin,
            "hbm_gbs_at_min_bytes": bmin / (ms_step * 1e-3) / 1e9,
            "hbm_frac_of_peak_at_min_bytes": bmin / (ms_step * 1e-3) / 1e9 / PEAK_HBM_GBS,
            # measured traffic of the fused kernel (rocprof counters) over its measured duration
            "hbm_frac_of_peak_measured_traffic": (traffic / (ms_main * 1e-3) / 1e9 / PEAK_HBM_GBS) if traffic else None,
            "fx_ms_per_launch": ms_fx,
        },
        "from_idle": idle,
    }
    if reduced:
        # The fp16 / bf16 matrix pipe is not what bounds this kernel: a 16-channel unit needs 512
        # MFMA cycles but 96 KB of operands per workgroup (64 KB of transformed filters, 32 KB of
        # fp32 patches) through the compute unit's 64 B/clk vector-memory path: 1536 cycles.
        units = ((layer.H + 1) // 2) ** 2 * ((layer.N + 31) // 32) * ((layer.K + 127) // 128) * ((layer.C + 15) // 16)
        roof_ms = units * 1536 / 256 / 2.4e9 * 1e3
        out["roofline"]["operand_delivery_roof"] = {
            "what": "vector-memory path of a compute unit, 64 B/clk: 96 KB per (workgroup tile, 16-channel unit) "
                    "= 1536 cycles against 512 cycles of MFMA",
            "ms_at_roof": roof_ms, "frac": roof_ms / ms_main,
            "mfma_frac_at_this_roof": fm / (roof_ms * 1e-3) / 1e12 / peak}

    if args.library:
        out["library"] = args.library + " (a diagnostic build: timing only, results are wrong)"
    if not args.no_cpu:
        from oracle import oracle

        y_ref, base = cpu_baseline(layer)
        out["cpu_baseline"] = base
        rel, max_abs, max_ref = oracle.compare(layer.y.cpu().numpy(), y_ref)
        out["check"] = {"rel_l2_vs_fp64_direct": rel, "max_abs": max_abs, "max_ref": max_ref}
        if not rel <= (1.5e-2 if reduced else 1e-3):
            sys.exit(f"bench.py: GPU result differs from the fp64 direct convolution (rel-L2 {rel})")

    if args.timeline:
        out["timeline"] = [timeline_summary(ocn, torch, layer, operands=args.operands)]

    if not args.no_layers:
        rows = []
        for name in LAYERS:
            lay = layer if name == layer.name else Layer(ocn, torch, name)
            d, m, b = work(lay.N, lay.C, lay.H, lay.K)
            precisions = [("f32", ocn.F32, PEAK_FP32_MFMA_TFLOPS)]
            if name.startswith("reduced"):
                precisions = [("f16", ocn.F16, PEAK_F16_MFMA_TFLOPS), ("bf16", ocn.BF16, PEAK_F16_MFMA_TFLOPS)]
            for label, prec, peak in precisions:
                try:
                    ocn.set_operand_precision(prec)
                    settle(torch, lay, args.settle_ms / 2)
                    tot, mn, fx = lay.kernel_times(20, 200)
                    # the reference's own protocol on this layer, after the sustained figures: the
                    # idle period it starts with puts the device back into its idle state
                    idle_row = from_idle(torch, lay, m, peak)
                finally:
                    ocn.set_operand_precision(ocn.F32)
                extra = {}
                if args.miopen and label == "f32":
                    extra["ms_miopen_conv2d_fp32"] = miopen_column(torch, lay, settle_ms=args.settle_ms / 2)
                rows.append({
                    **extra,
                    "workload": name, "gemm_operands": label, "ms_per_layer": tot, "ms_fused_kernel": mn,
                    "ms_filter_transform": fx,
                    "effective_tflops": d / (tot * 1e-3) / 1e12,
                    "mfma_tflops": m / (mn * 1e-3) / 1e12,
                    "mfma_frac_of_peak": m / (mn * 1e-3) / 1e12 / peak,
                    "from_idle_ms_per_layer": idle_row["ms_per_step"],
                    "from_idle_ms_fused_kernel": idle_row["ms_fused_kernel"],
                    "from_idle_frac": idle_row["frac"],
                    "hbm_gbs_at_min_bytes": b / (tot * 1e-3) / 1e9,
                    "hbm_frac_of_peak_at_min_bytes": b / (tot * 1e-3) / 1e9 / PEAK_HBM_GBS,
                })
            if args.shims and not name.startswith("reduced"):
                out.setdefault("shims", []).extend(shim_rows(ocn, torch, lay))
            if args.timeline and name != layer.name and not name.startswith("reduced"):
                out["timeline"].append(timeline_summary(ocn, torch, lay))
            del lay
        out["layers"] = rows

    if args.networks:
        out["networks"] = network_rows(ocn, torch)

    print(json.dumps(out))


if __name__ == "__main__":
    main()
