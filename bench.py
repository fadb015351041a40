#!/usr/bin/env python3
"""Benchmark of the depthwise conv2d hot path on one MI355X.

Workload: the 12 depthwise layers of EfficientNet-B0,
fp32 NCHW, batch 128, padding k//2.  One "step" = forward of layers 1..12, then
grad-input and grad-weight of layers 12..1 (training order): 24 calls into the
C ABI of libdwconv_hip (12 forward, 12 combined backward; --separate-backward
makes it 36), all tensors resident in HBM before the clock starts.

Prints one JSON line.  `value` is achieved HBM GB/s = algorithmic bytes of the
step (every tensor of every pass touched exactly once: 12(|x|+|y|+|w|) bytes per
layer, 6 per element with --dtype f16/bf16) / step time; `ms_per_step` carries the fwd+bwd time itself.
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "depthwise-conv-pytorch_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
COLD_RING_BYTES = 512 * 1000 * 1000  # tensor sets a cache-sized workload rotates over (twice the Infinity Cache)
FP32_VECTOR_PEAK_TFLOPS = 157.3  # MI355X fp32 vector peak (packed); the kernels use unpacked FMAs (half of it)

# (C, H_in, k, stride), batch 128, padding k//2
EFFNET_B0 = [
    (32, 112, 3, 1), (96, 112, 3, 2), (144, 56, 3, 1), (144, 56, 5, 2),
    (240, 28, 5, 1), (240, 28, 3, 2), (480, 14, 3, 1), (480, 14, 5, 1),
    (672, 14, 5, 1), (672, 14, 5, 2), (1152, 7, 5, 1), (1152, 7, 3, 1),
]


def effnet_at(batch, res):
    """The same 12 layers for a res x res network input (224 gives EFFNET_B0's maps: 112, 56, 28, 14, 7)."""
    shapes, h = [], res // 2
    for (c, _, k, s) in EFFNET_B0:
        shapes.append((batch, c, h, h, k, s, k // 2))
        h = (h + 2 * (k // 2) - k) // s + 1
    return shapes


WORKLOADS = {
    "effnet_b0": lambda batch: [(batch, c, h, h, k, s, k // 2) for (c, h, k, s) in EFFNET_B0],
    # other input resolutions: 256 -> maps 128, 64, 32, 16, 8; 240 (EfficientNet-B1's) -> 120, 60, 30, 15, 8
    "effnet_b0_256": lambda batch: effnet_at(batch, 256),
    "effnet_b0_240": lambda batch: effnet_at(batch, 240),
    "effnet_b0_192": lambda batch: effnet_at(batch, 192),   # maps 96, 48, 24, 12, 6
    # EfficientNet-B3's resolution: maps 150, 75, 38, 19, 10, none of them whole groups of four elements wide
    "effnet_b0_300": lambda batch: effnet_at(batch, 300),
    # the options the reference's check_options refuses (a shape may carry dilation and depth multiplier as 8th and 9th
    # entries): the 3x3 stride-1 layers of the stack at dilation 2 (padding 2), a 5x5 one, and the first two layers
    # with two output channels per input channel
    "effnet_b0_dil2": lambda batch: [(batch, 32, 112, 112, 3, 1, 2, 2, 1), (batch, 144, 56, 56, 3, 1, 2, 2, 1),
                                     (batch, 240, 28, 28, 5, 1, 4, 2, 1), (batch, 480, 14, 14, 3, 1, 2, 2, 1),
                                     (batch, 1152, 7, 7, 3, 1, 2, 2, 1)],
    "effnet_b0_mult2": lambda batch: [(batch, 32, 112, 112, 3, 1, 1, 1, 2), (batch, 96, 112, 112, 3, 2, 1, 1, 2)],
    "cfg1": lambda batch: [(8, 32, 56, 56, 3, 1, 1)],
    "cfg2": lambda batch: [(16, 64, 256, 256, 5, 1, 2)],
    "cfg4": lambda batch: [(256, 1024, 7, 7, 7, 1, 3), (128, 512, 14, 14, 7, 1, 3)],
    "convnext_t": lambda batch: [(64, 96, 56, 56, 7, 1, 3), (64, 192, 28, 28, 7, 1, 3),
                                 (64, 384, 14, 14, 7, 1, 3), (64, 768, 7, 7, 7, 1, 3)],
    "stress": lambda batch: [(64, 256, 128, 96, 5, 2, 2)],
    # ConvNeXt-T's first three stages with the larger filters of its successors (9x9, 11x11, 13x13)
    # what only the kernels that loop over their taps serve: an even-sized filter, a 15x15 one, stride 3, and the
    # atrous 3x3 layers of a segmentation head at rates 6, 12 and 18 (general entry points)
    "any_geometry": lambda batch: [(16, 64, 128, 128, 4, 1, 2), (16, 64, 128, 128, 15, 1, 7), (16, 64, 128, 128, 3, 3, 1),
                                   (16, 256, 65, 65, 3, 1, 6, 6, 1), (16, 256, 65, 65, 3, 1, 12, 12, 1),
                                   (16, 256, 65, 65, 3, 1, 18, 18, 1)],
    "large_filters": lambda batch: [(64, 96, 56, 56, 9, 1, 4), (64, 192, 28, 28, 11, 1, 5), (64, 384, 14, 14, 13, 1, 6)],
}


class Layer:
    """Device tensors and the three C-ABI calls of one depthwise layer."""

    def __init__(self, shape, lib, torch, dev, gen, dtype="f32", layout="nchw"):
        n, c, h, w, k, s, p = shape[:7]
        dil, mult = (tuple(shape[7:9]) + (1, 1))[:2] if len(shape) > 7 else (1, 1)
        self.general = (dil, mult) if (dil, mult) != (1, 1) else None
        tdtype = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]
        es = 4 if dtype == "f32" else 2
        self.fn_fir = getattr(lib, "dwconv2d_" + dtype)
        self.fn_wgrad = getattr(lib, "dwconv2d_backward_kernel_" + dtype)
        self.fn_bwd = getattr(lib, "dwconv2d_backward_" + dtype)
        self.layout = layout
        if layout == "nhwc":
            self.fn_fir = self.fn_wgrad = None
            self.fn_fwd_nhwc = getattr(lib, "dwconv2d_nhwc_" + dtype)
            self.fn_bwd = getattr(lib, "dwconv2d_backward_nhwc_" + dtype)
        self.shape = shape
        self.lib = lib
        ke = dil * (k - 1) + 1
        oh, ow = (h + 2 * p - ke) // s + 1, (w + 2 * p - ke) // s + 1
        self.geom = (n, c, h, w, oh, ow, k, s, p)
        self.x = torch.randn(n, c, h, w, generator=gen).to(dev, tdtype)
        self.w = (torch.randn(c * mult, 1, k, k, generator=gen) / k).to(dev, tdtype)
        self.gy = torch.randn(n, c * mult, oh, ow, generator=gen).to(dev, tdtype)
        self.y = torch.empty(n, c * mult, oh, ow, device=dev, dtype=tdtype)
        self.gx = torch.empty_like(self.x)
        self.gw = torch.empty_like(self.w)
        # channels-last: the same element counts, stored (N,H,W,C); values are random either way
        if self.general:
            if layout != "nchw":
                raise SystemExit("dilation / depth multiplier workloads are NCHW")
            self.fn_gen = getattr(lib, "dwconv2d_general_" + dtype)
            self.fn_gen_bwd = getattr(lib, "dwconv2d_general_backward_" + dtype)
            self.ws_bytes = lib.dwconv2d_general_backward_workspace_bytes(n, c, h, w, mult, k, k, s, s, p, p, dil, dil, es)
        else:
            self.ws_bytes = (lib.dwconv2d_backward_nhwc_workspace_bytes(n, c, h, w, k, k, s, s, p, p, es) if layout == "nhwc"
                             else lib.dwconv2d_backward_kernel_workspace_bytes(n, c, h, w, oh, ow, k, k, s, s, p, p, es))
        self.ws = torch.empty(max(self.ws_bytes, 16), dtype=torch.uint8, device=dev)
        nx, ny, nw = n * c * h * w, n * c * mult * oh * ow, c * mult * k * k
        self.bytes = {"fwd": es * (nx + ny + nw), "gx": es * (ny + nx + nw), "gw": es * (nx + ny + nw)}
        # the combined backward call is credited with the bytes of the two passes it replaces
        self.bytes["bwd"] = self.bytes["gx"] + self.bytes["gw"]
        self.flops = 2 * ny * k * k
        # transposed-problem padding, torch_dwconv/dwconv.py:39-44
        self.g_pad = (k - p - 1, h - oh * s + p, k - p - 1, w - ow * s + p)
        self.name = f"C{c}_{h}x{w}_k{k}s{s}" + (f"d{dil}" if dil > 1 else "") + (f"m{mult}" if mult > 1 else "")

    def _check(self, rc):
        if rc != 0:
            raise RuntimeError(self.lib.dwconv_last_error().decode())

    def fwd(self, stream):
        n, c, h, w, oh, ow, k, s, p = self.geom
        if self.general:
            dil, mult = self.general
            self._check(self.fn_gen(self.x.data_ptr(), self.w.data_ptr(), self.y.data_ptr(), n, c, h, w, mult, k, k, s, s,
                                    p, p, dil, dil, stream))
            return
        if self.layout == "nhwc":
            self._check(self.fn_fwd_nhwc(self.x.data_ptr(), self.w.data_ptr(), self.y.data_ptr(), n, c, h, w, k, k,
                                         s, s, p, p, stream))
            return
        self._check(self.fn_fir(self.x.data_ptr(), self.w.data_ptr(), self.y.data_ptr(), n, c, h, w, k, k,
                                          1, 1, s, s, p, p, p, p, 1, stream))

    def bwd_input(self, stream):
        n, c, h, w, oh, ow, k, s, p = self.geom
        g = self.g_pad
        self._check(self.fn_fir(self.gy.data_ptr(), self.w.data_ptr(), self.gx.data_ptr(), n, c, oh, ow, k, k,
                                          s, s, 1, 1, g[0], g[1], g[2], g[3], 0, stream))

    def bwd_filter(self, stream):
        n, c, h, w, oh, ow, k, s, p = self.geom
        self._check(self.fn_wgrad(
            self.x.data_ptr(), self.gy.data_ptr(), self.gw.data_ptr(), self.ws.data_ptr(), self.ws_bytes,
            n, c, h, w, oh, ow, k, k, 1, 1, s, s, p, p, stream))


    def bwd(self, stream):
        n, c, h, w, oh, ow, k, s, p = self.geom
        if self.general:
            dil, mult = self.general
            self._check(self.fn_gen_bwd(self.x.data_ptr(), self.gy.data_ptr(), self.w.data_ptr(), self.gx.data_ptr(),
                                        self.gw.data_ptr(), self.ws.data_ptr(), self.ws_bytes, n, c, h, w, oh, ow, mult,
                                        k, k, s, s, p, p, dil, dil, stream))
            return
        self._check(self.fn_bwd(
            self.x.data_ptr(), self.gy.data_ptr(), self.w.data_ptr(), self.gx.data_ptr(), self.gw.data_ptr(),
            self.ws.data_ptr(), self.ws_bytes, n, c, h, w, oh, ow, k, k, s, s, p, p, stream))


def schedule(layers, separate_backward):
    """Training order: all forwards, then the backward passes last layer first."""
    calls = [(l, "fwd", l.fwd) for l in layers]
    for l in reversed(layers):
        if separate_backward:
            calls.append((l, "gx", l.bwd_input))
            calls.append((l, "gw", l.bwd_filter))
        else:
            calls.append((l, "bwd", l.bwd))
    return calls


def cpu_baseline(layers, torch, iters=5, budget_s=30.0):
    """fp32 F.conv2d(groups=C) forward + both gradients on the host cores, every layer of the workload at its full
    batch (the same tensors the GPU step runs on, copied to the host).  A step is the sum over the layers; the step is
    repeated `iters` times after one untimed pass and min / median / max are reported.  Layers are dropped from the
    end only if the time budget runs out (said in `sample`)."""
    from oracle import torch_cpu_fp32_step

    cores = os.cpu_count() or 1
    threads = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    t_start = time.perf_counter()
    per_layer, bytes_total, done = [], 0, 0
    for l in layers:
        n, c, h, w, oh, ow, k, s, p = l.geom
        x, wt, gy = l.x.float().cpu(), l.w.float().cpu(), l.gy.float().cpu()
        times, threads = torch_cpu_fp32_step(x, wt, gy, s, p, iters=iters, threads=threads, all_times=True)
        per_layer.append(times)
        bytes_total += 12 * (n * c * h * w + n * c * oh * ow + c * k * k)
        done += 1
        if time.perf_counter() - t_start > budget_s:
            break
    steps = sorted(sum(t[i] for t in per_layer) for i in range(iters))
    med = steps[len(steps) // 2]
    sample = (f"torch {torch.__version__} F.conv2d(groups=C) fp32 fwd + autograd.grad(x,w) at the full batch of "
              f"{layers[0].geom[0]} on {done} of {len(layers)} layers, {iters} timed steps after one warm-up; value = median")
    return {"value": round(bytes_total / med / 1e9, 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": sample, "ms_per_step": {"min": round(steps[0] * 1e3, 1), "median": round(med * 1e3, 1),
                                              "max": round(steps[-1] * 1e3, 1)}}


def miopen_native(layers, torch, iters=3):
    """The same layers through F.conv2d(groups=C) on the GPU (MIOpen's depthwise)."""
    import torch.nn.functional as F

    per_layer = []
    for l in layers:
        n, c, h, w, oh, ow, k, s, p = l.geom
        x = l.x.detach().requires_grad_(True)
        wt = l.w.detach().requires_grad_(True)
        ts = []
        for i in range(iters + 2):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            y = F.conv2d(x, wt, stride=s, padding=p, dilation=(l.general or (1, 1))[0], groups=c)
            torch.autograd.grad(y, (x, wt), l.gy)
            e1.record()
            torch.cuda.synchronize()
            if i >= 2:
                ts.append(e0.elapsed_time(e1))
        per_layer.append(statistics.median(ts))
    return per_layer


def epilogue_comparison(layers, lib, torch, stream, dtype, layout, iters=10):
    """Forward + folded batch-norm + SiLU over the workload: one fused C-ABI call per layer against the plain forward
    call followed by PyTorch's elementwise ops on its output, and the same block in training (forward + all four
    gradients through autograd).  Returns (fused ms, unfused ms, convolution-only ms, training fused ms, training
    composed ms) per pass over the layers."""
    import torch.nn.functional as F

    fn = getattr(lib, ("dwconv2d_fused_nhwc_" if layout == "nhwc" else "dwconv2d_fused_") + dtype)
    prepared = []
    for l in layers:
        n, c, h, w, oh, ow, k, s, p = l.geom
        scale = torch.rand(c, device=l.x.device) + 0.5
        shift = torch.randn(c, device=l.x.device)
        shape = (1, 1, 1, c) if layout == "nhwc" else (1, c, 1, 1)
        y = l.y.view(n, oh, ow, c) if layout == "nhwc" else l.y
        prepared.append((l, scale, shift, scale.view(shape).to(l.y.dtype), shift.view(shape).to(l.y.dtype), y))

    def call(l, scale, shift, act):
        n, c, h, w, oh, ow, k, s, p = l.geom
        l._check(fn(l.x.data_ptr(), l.w.data_ptr(), scale, shift, l.y.data_ptr(), n, c, h, w, k, k, s, s, p, p, act, stream))

    def fused():
        for l, scale, shift, _, _, _ in prepared:
            call(l, scale.data_ptr(), shift.data_ptr(), 3)

    def unfused():
        for l, _, _, scale_b, shift_b, y in prepared:
            call(l, None, None, 0)
            F.silu(y * scale_b + shift_b)

    def conv_only():
        for l, _, _, _, _, _ in prepared:
            call(l, None, None, 0)

    # the same block in training: forward + backward through the fused autograd Function (recompute, one
    # epilogue-backward sweep) against depthwise_conv2d followed by PyTorch's differentiable elementwise ops
    from torch_dwconv.dwconv import depthwise_conv2d, depthwise_conv2d_fused

    train = []
    for l, scale, shift, _, _, _ in prepared:
        n, c, h, w, oh, ow, k, s, p = l.geom
        fmt = torch.channels_last if layout == "nhwc" else torch.contiguous_format
        x = (l.x.view(n, h, w, c).permute(0, 3, 1, 2) if layout == "nhwc" else l.x).detach().requires_grad_(True)
        gy = l.gy.view(n, oh, ow, c).permute(0, 3, 1, 2) if layout == "nhwc" else l.gy
        assert x.is_contiguous(memory_format=fmt)
        train.append((x, l.w.detach().requires_grad_(True), scale.detach().requires_grad_(True),
                      shift.detach().requires_grad_(True), gy, s, p))

    def train_fused():
        for x, w, scale, shift, gy, s, p in train:
            y = depthwise_conv2d_fused(x, w, shift, scale, "silu", s, p)
            torch.autograd.grad(y, (x, w, scale, shift), gy)

    def train_composed():
        for x, w, scale, shift, gy, s, p in train:
            y = F.silu(depthwise_conv2d(x, w, stride=s, padding=p) * scale.view(1, -1, 1, 1) + shift.view(1, -1, 1, 1))
            torch.autograd.grad(y, (x, w, scale, shift), gy)

    out = []
    for run in (fused, unfused, conv_only, train_fused, train_composed):
        run()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            run()
        e1.record()
        torch.cuda.synchronize()
        out.append(e0.elapsed_time(e1) / iters)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="effnet_b0", choices=sorted(WORKLOADS))
    ap.add_argument("--batch", type=int, default=128)
    ap.add_argument("--dtype", default="f32", choices=["f32", "f16", "bf16"],
                    help="element type of the tensors (the headline metric is f32; 16-bit types accumulate in fp32)")
    ap.add_argument("--layout", default="nchw", choices=["nchw", "nhwc"],
                    help="memory layout of the activations (the headline metric is nchw, the reference's layout)")
    ap.add_argument("--only", default="", help="comma-separated layer indices of the workload to run (profiling aid)")
    ap.add_argument("--epilogue", action="store_true",
                    help="also time forward + folded batch-norm + SiLU, fused into the convolution against separate "
                         "elementwise passes (reported under 'fused_epilogue')")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-miopen", action="store_true")
    ap.add_argument("--separate-backward", action="store_true",
                    help="call grad-input and grad-weight as two entry points (36 calls per step) instead of the "
                         "combined backward entry point (24 calls)")
    ap.add_argument("--warm-only", action="store_true",
                    help="time a cache-sized workload on one tensor set only (no ring of cold sets)")
    ap.add_argument("--table", action="store_true", help="print a per-layer, per-pass table to stderr")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB first (a kernel of known traffic, "
                         "to scale rocprofv3 FETCH_SIZE/WRITE_SIZE readings)")
    ap.add_argument("--call-markers", action="store_true",
                    help="launch a one-element fill kernel after every C-ABI call, so that a profile's list of "
                         "dispatches can be split into calls (profiling aid; adds launches to the timed region)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: depthwise conv2d is a single-GPU kernel path; run with --gpus 1")

    import torch
    from torch_dwconv import _C

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (no HIP device visible)")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = _C._lib
    shapes = WORKLOADS[args.workload](args.batch)
    if args.only:
        shapes = [shapes[int(i)] for i in args.only.split(",")]
    gen = torch.Generator("cpu").manual_seed(0)
    if args.layout == "nhwc" and args.separate_backward:
        sys.exit("--separate-backward applies to the nchw entry points")
    layers = [Layer(s, lib, torch, dev, gen, args.dtype, args.layout) for s in shapes]
    # Cache policy.  A step whose activations (x, y, gy, gx of every layer) fit the 256 MB Infinity Cache would be
    # timed out of cache if it reused one set of tensors: such workloads rotate over a ring of distinct tensor
    # sets of >= 512 MB in total, so that every step finds its operands in HBM ("cold"); the same step on one set
    # is reported beside it as "warm".  Larger workloads (the headline one moves 2.8 GB of activations) evict
    # their own tensors between uses and run on one set.
    footprint = sum(t.numel() * t.element_size() for l in layers for t in (l.x, l.y, l.gy, l.gx))
    ring = 1 if footprint >= COLD_RING_BYTES or args.warm_only else min(128, -(-COLD_RING_BYTES // footprint))
    sets = [layers] + [[Layer(s, lib, torch, dev, gen, args.dtype, args.layout) for s in shapes] for _ in range(ring - 1)]
    call_sets = [schedule(ls, args.separate_backward) for ls in sets]
    calls = call_sets[0]
    stream_obj = torch.cuda.current_stream(dev)
    stream = ctypes.c_void_p(stream_obj.cuda_stream)
    step_bytes = sum(l.bytes["fwd"] + l.bytes["gx"] + l.bytes["gw"] for l in layers)
    turn = [0]

    marker = torch.zeros(1, device=dev) if args.call_markers else None

    def step():
        for _, _, fn in call_sets[turn[0] % ring]:
            fn(stream)
            if marker is not None:
                marker.zero_()
        turn[0] += 1

    def timed(n_steps):
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t = time.perf_counter()
        a.record(stream_obj)
        for _ in range(n_steps):
            step()
        b.record(stream_obj)
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n_steps, (time.perf_counter() - t) * 1e3 / n_steps

    if args.calibration_copy_mib:
        src = torch.ones(args.calibration_copy_mib * 1024 * 1024 // 4, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    ms_per_step, wall_ms = timed(args.steps)
    warm_ms = None
    if ring > 1:
        # the same step on one tensor set (operands left in the caches by the step before)
        saved, ring = ring, 1
        for _ in range(args.warmup):
            step()
        warm_ms, _ = timed(args.steps)
        ring = saved

    # Per-launch durations, same order and cache state, events on the launch stream.
    variants, durs = [], [[] for _ in calls]
    for it in range(max(3, min(args.steps, 20), ring)):
        evs = []
        for i, (l, kind, fn) in enumerate(call_sets[it % ring]):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream_obj)
            fn(stream)
            b.record(stream_obj)
            if it == 0:
                variants.append(lib.dwconv_last_variant().decode())
            evs.append((a, b))
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(evs):
            durs[i].append(a.elapsed_time(b))
    rows = []
    for i, (l, kind, fn) in enumerate(calls):
        ms = statistics.mean(durs[i])
        rows.append({"layer": l.name, "pass": kind, "variant": variants[i], "us": round(ms * 1e3, 1),
                     "GBs": round(l.bytes[kind] / ms / 1e6, 1), "bytes": l.bytes[kind]})
    # dominant kernel = the kernel function (template instance) with the largest share of the step
    by_kernel = {}
    for r in rows:
        key = r["variant"].split(">")[0] + (">" if ">" in r["variant"] else "")
        agg = by_kernel.setdefault(key, {"ms": 0.0, "bytes": 0, "launches": 0})
        agg["ms"] += r["us"] / 1e3
        agg["bytes"] += r["bytes"]
        agg["launches"] += 1
    # (instances within 5 % of the largest share count as tied, and the one with the most bytes per launch wins, so
    # that run-to-run jitter between two near-equal instances does not change which one is reported)
    top_ms = max(v["ms"] for v in by_kernel.values())
    dom_name, dom = max(((k, v) for k, v in by_kernel.items() if v["ms"] >= 0.95 * top_ms),
                        key=lambda kv: kv[1]["bytes"] / kv[1]["launches"])
    achieved = dom["bytes"] / dom["ms"] / 1e6
    # measured HBM bytes (rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE, scaled by a plain copy's readings) from the
    # committed summary of this very configuration: per launch of the dominant kernel, and per step (null where the
    # summary does not cover the configuration)
    traffic = measured_step = None
    if not args.only and not args.separate_backward:
        try:
            with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
                entry = json.load(f)["workloads"][f"{args.workload}/{args.dtype}/{args.layout}/b{shapes[0][0]}"]
            traffic = entry["bytes_per_launch"].get(dom_name)
            measured_step = entry["measured_bytes_per_step"]
        except (OSError, ValueError, KeyError):
            pass
    # the device function behind the variant name, as rocprofv3 lists it (backward calls end with a ~4.5 us
    # *_final_kernel that the per-call timing includes)
    family = dom_name.split("<")[0].rstrip("16")
    function = {"tile_down": "fir_down_kernel", "tile_up2": "fir_up2_kernel", "small_down": "small_down_kernel",
                "small_up2": "small_up2_kernel", "small_bwd": "small_bwd_kernel + wgrad_tile_final_kernel",
                "small_wgrad": "small_bwd_kernel + wgrad_tile_final_kernel",
                "bwd_tile": "wgrad_tile_kernel + wgrad_tile_final_kernel",
                "wgrad_tile": "wgrad_tile_kernel + wgrad_tile_final_kernel",
                "bwd_tile_s2": "bwd_s2_kernel + wgrad_tile_final_kernel",
                "tile_stack": "stack_kernel", "bwd_stack": "stack_kernel + wgrad_tile_final_kernel",
                "nhwc_bwd": "nhwc_bwd_fused_kernel + nhwc_wgrad_final_kernel"}.get(family, family)
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "kernel": dom_name, "kernel_function": function,
                "launches_per_step": dom["launches"], "avg_launch_us": round(dom["ms"] * 1e3 / dom["launches"], 1),
                "bytes_per_launch": dom["bytes"] // dom["launches"]}

    result = {
        "metric": "fwd+bwd achieved HBM GB/s, EfficientNet-B0 dw stack, 1 GPU" if args.workload == "effnet_b0"
        else f"fwd+bwd achieved HBM GB/s, {args.workload}, 1 GPU",
        "value": round(step_bytes / ms_per_step / 1e6, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: {len(layers)} depthwise layers, "
                               f"{'fp32' if args.dtype == 'f32' else args.dtype} {args.layout.upper()}, batch {shapes[0][0]}, "
                               "fwd + grad-input + grad-weight per layer, training order, "
                               f"{len(calls)} C-ABI calls per step",
                   "layers": [l.name for l in layers], "algorithmic_bytes_per_step": step_bytes},
        "frac_of_hbm_roofline": round(step_bytes / ms_per_step / 1e6 / HBM_PEAK_GBS, 4),
        # the same with the HBM bytes the counters saw in one step instead of the algorithmic ones: how busy the
        # memory system was, re-reads and write-backs included
        "measured_traffic_frac": round(measured_step / ms_per_step / 1e6 / HBM_PEAK_GBS, 4) if measured_step else None,
        "measured_over_algorithmic_bytes": round(measured_step / step_bytes, 3) if measured_step else None,
        # arithmetic side (matters for the 7x7-filter shapes): nominal FLOPs 2*|y|*k^2 per pass, three passes
        "tflops": round(3 * sum(l.flops for l in layers) / ms_per_step / 1e9, 2),
        "frac_of_fp32_vector_peak": round(3 * sum(l.flops for l in layers) / ms_per_step / 1e9 / FP32_VECTOR_PEAK_TFLOPS, 4),
        "host_wall_ms_per_step": round(wall_ms, 4),
        "sum_of_launch_us": round(sum(r["us"] for r in rows), 1),
        "roofline": roofline,
        "cache": {"activation_bytes_per_set": footprint, "tensor_sets": ring,
                  "state": ("cold: ring of %d tensor sets, %.0f MB in total" % (ring, ring * footprint / 1e6)) if ring > 1
                  else ("warm: one tensor set by request" if footprint < COLD_RING_BYTES
                        else "cold by size: one step streams %.0f MB of activations through the 256 MB cache" % (footprint / 1e6))},
    }
    if warm_ms is not None:
        result["cache"]["warm_ms_per_step"] = round(warm_ms, 4)
        result["cache"]["warm_value"] = round(step_bytes / warm_ms / 1e6, 1)
    if args.table:
        for r in rows:
            print(f"{r['layer']:>18} {r['pass']:>3} {r['us']:9.1f} us {r['GBs']:8.1f} GB/s  {r['variant']}", file=sys.stderr)
    result["per_pass_us"] = {k: round(sum(r["us"] for r in rows if r["pass"] == k), 1)
                             for k in ("fwd", "gx", "gw", "bwd") if any(r["pass"] == k for r in rows)}
    if not args.no_miopen and args.layout == "nchw":
        try:
            per_layer = miopen_native(layers, torch)
            result["miopen_native_ms_per_step"] = round(sum(per_layer), 3)
            result["speedup_vs_miopen_native"] = round(sum(per_layer) / ms_per_step, 2)
        except Exception as e:  # the comparison is informative only
            result["miopen_native_ms_per_step"] = f"failed: {type(e).__name__}"
    if args.epilogue:
        fused_ms, unfused_ms, conv_ms, train_fused_ms, train_composed_ms = epilogue_comparison(
            layers, lib, torch, stream, args.dtype, args.layout)
        result["fused_epilogue"] = {"what": "forward + per-channel scale/shift + SiLU over the workload's layers",
                                    "fused_ms": round(fused_ms, 4), "conv_then_torch_elementwise_ms": round(unfused_ms, 4),
                                    "conv_only_ms": round(conv_ms, 4),
                                    "training_fwd_bwd_fused_ms": round(train_fused_ms, 4),
                                    "training_fwd_bwd_conv_then_torch_elementwise_ms": round(train_composed_ms, 4)}
    if not args.no_cpu_baseline and args.dtype == "f32" and args.layout == "nchw" and not any(l.general for l in layers):
        result["cpu_baseline"] = cpu_baseline(layers, torch)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
