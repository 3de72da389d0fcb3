#!/usr/bin/env python3
"""Headline benchmark: images/s and achieved int8 TOPS of the ResNet-18-shaped int8 conv stack on one MI355X.

A step is one forward pass of the fused int8 network (excalibur_amd.resnet18) over a batch of N x 3 x 640 x 640
synthetic images already resident in HBM: input quantization, 20 convolutions on the int8 MFMA path with fused
dequant + bias + ReLU / shortcut add + requant epilogues, and the 3x3 max pool. Prints one JSON line.

`roofline` is for the dominant kernel, the implicit-GEMM convolution: algorithmic operations
(2 x N x OH x OW x K x C x kh x kw summed over the 20 layers, 947.5 GOP for N = 32) divided by the duration of its
20 consecutive launches, measured with one HIP event pair on the library's stream around them (the queue's hand-over
between launches included, as in the sum of a kernel trace's durations), against the 5.0 POP/s int8 MFMA peak.
`cpu_baseline` times the reference's own CPU path (compiled under oracle/_ref) or, where that is absent, this
repository's CPU restatement, on a bounded sample of the same workload on the host cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0  # MI355X dense int8 MFMA
PEAK_HBM_GBS = 8000.0
PEAK_F16_TFLOPS = 2500.0  # dense fp16 MFMA
PEAK_F32_TFLOPS = 157.3   # fp32 MFMA


def cpu_baseline(net, hw, budget_s=10.0):
    """The reference's CPU path on one image of the workload's own resolution, two legs of about `budget_s` seconds each:
    one core (the reference's default build: OpenMP off), and batch-parallel over the host cores with one pipeline and one
    image per worker thread (a pipeline instance is single-threaded). -> (one-core record, all-cores record or None)"""
    from oracle import ref
    x = np.random.default_rng(7).uniform(-1, 1, (1, 3, hw, hw)).astype(np.float32)
    gmac = net.gmac_per_image(hw, hw)
    if not ref.available():
        from tests import netref
        t0 = time.perf_counter()
        netref.oracle_forward(net, x)
        sec = time.perf_counter() - t0
        return {"value": round(1.0 / sec, 4), "unit": "images/s", "cores": 1, "kind": "port",
                "sample": f"one 3x{hw}x{hw} image through the same int8 topology, 1 timed forward, "
                          f"{sec * 1e3:.0f} ms = {2 * gmac / sec:.1f} GOP/s"}, None
    import tempfile
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    net.write_model(path)
    try:
        p = ref.Pipeline(net.topology(), path, "f32")
        t0 = time.perf_counter()
        p.forward(x)
        first = time.perf_counter() - t0
        iters = max(2, min(60, int(budget_s / max(first, 1e-3)) - 1))
        sec = p.time(x, 0, iters)
        p.close()
        one = {"value": round(1.0 / sec, 4), "unit": "images/s", "cores": 1, "kind": "reference",
               "sample": f"one 3x{hw}x{hw} image through the same int8 topology, {iters} timed forward(s), "
                         f"{sec * 1e3:.0f} ms each = {2 * gmac / sec:.1f} GOP/s"}
        # the GPU boxes give a job 16 cores, whatever the machine has
        workers = max(1, min(os.cpu_count() or 1, 16))
        each = max(1, int(budget_s / max(sec, 1e-3)))
        wall = ref.time_parallel(net.topology(), path, x, workers, 1, each)
        rate = workers * each / wall
        many = {"value": round(rate, 4), "unit": "images/s", "cores": workers, "kind": "reference",
                "sample": f"{workers} worker threads, each its own pipeline and one 3x{hw}x{hw} image, {each} timed forward(s) "
                          f"each in {wall:.1f} s = {2 * gmac * rate:.1f} GOP/s"}
    finally:
        os.unlink(path)
    return one, many


def csrc_digest():
    """A digest of the kernel sources: profiles taken under rocprofv3 carry it, so that a figure read back from a profile
    file is dropped once a kernel has changed."""
    import hashlib
    h = hashlib.sha256()
    d = os.path.join(ROOT, "excalibur_amd", "csrc")
    for name in sorted(os.listdir(d)):
        if name.endswith((".hip", ".h")):
            h.update(open(os.path.join(d, name), "rb").read())
    return h.hexdigest()[:16]


def measured_traffic(n, hw):
    """HBM bytes per conv launch from the committed rocprofv3 --pmc summary (FETCH_SIZE + WRITE_SIZE, scaled by a
    plain copy kernel). The counters cannot be read inside this process, so the figure comes from the profile file, which
    names the workload and the kernel sources it was taken with: None for another workload or other sources."""
    path = os.path.join(ROOT, "profiles", "int8_conv_resnet18_n32_640_hbm_traffic.txt")
    if (n, hw) != (32, 640) or not os.path.exists(path):
        return None
    text = open(path).read()
    if f"kernel sources {csrc_digest()}" not in text:
        return None
    for line in text.splitlines():
        if line.startswith("HBM traffic per forward"):
            return {"value": float(line.split("=")[-1].split("MB")[0]), "unit": "MB per launch (mean over the launches of a step)"}
    return None


def network_table(iters=10, only=None):
    """The generated topologies of the other configurations through pipeline<float> / pipeline<unsigned short> (float32 and
    fp16: layer by layer with the executor's joins; int8: the int8 graph plan where it takes the network, which the row's
    "executor" says), input resident on the device: wall time per forward over `iters` forwards, device drained before and
    after. Returns [{"network", "dtype", "executor", "ms", "images/s", ...}]."""
    import tempfile
    from excalibur_amd import pipeline as xp
    from excalibur_amd.mobilenet import CFG3, MobileFaceNetF32
    from excalibur_amd.yolo import YoloV5ShapedF32
    r = np.random.default_rng(0)
    rows = []

    def run(label, net, x, dtype, pipe_dtype):
        if only and only not in f"{label} {dtype}":   # --only: a substring of "<network label> <dtype>"
            return
        with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
            path = f.name
        net.write_model(path)
        p = xp.Pipeline(net.topology(), path, 0, pipe_dtype)
        os.unlink(path)
        p.set_input(x if pipe_dtype == "f32" else x.astype(np.float16).view(np.uint16))
        for _ in range(3):
            p.run()
        p.sync()
        t0 = time.perf_counter()
        for _ in range(iters):
            p.run()
        p.sync()
        ms = (time.perf_counter() - t0) / iters * 1e3
        executor = "int8 graph plan" if p.fused else "per-layer"
        p.close()
        from excalibur_amd import topologies
        gop = topologies.algorithmic_gop(net.topology(), x.shape[1:]) * x.shape[0]   # of the whole batch
        peak = {"f32": PEAK_F32_TFLOPS, "f16": PEAK_F16_TFLOPS, "int8": PEAK_INT8_TOPS}[dtype]
        rows.append({"network": label, "dtype": dtype, "layers": len(net.lines), "executor": executor, "ms": round(ms, 3),
                     "images/s": round(x.shape[0] / ms * 1e3, 1), "algorithmic_gop": round(gop, 1),
                     "achieved": round(gop / ms, 1), "peak": peak, "unit": "TOP/s" if dtype == "int8" else "TFLOP/s",
                     "frac": round(gop / ms / peak, 4)})
        print(f"{label:72s} {dtype:5s} {ms:7.2f} ms {x.shape[0] / ms * 1e3:9.0f} images/s", file=sys.stderr, flush=True)

    face = MobileFaceNetF32(hw=112, width=64, blocks=((2, 64, 2), (1, 64, 2), (1, 64, 2), (2, 128, 4), (1, 128, 2), (1, 128, 2),
                                                     (2, 128, 4), (1, 128, 2)), embed=128)
    x = r.uniform(0, 255, (64, 3, 112, 112)).astype(np.float32)
    for dt in ("f32", "f16"):
        run("MobileFaceNet-shaped (PReLU behind every convolution), 64x3x112x112", face, x, dt, dt)
    mobile = MobileFaceNetF32(**CFG3)
    x = r.uniform(0, 255, (64, 3, 224, 224)).astype(np.float32)
    for dt in ("f32", "f16"):
        run("3x3 s2 stem -> 32, dw3x3 + pw1x1 blocks 64..512, residual adds, 64x3x224x224", mobile, x, dt, dt)
    x = r.uniform(0, 255, (16, 3, 640, 640)).astype(np.float32)
    yolo = YoloV5ShapedF32(hw=640, width=32)
    for dt in ("f32", "f16"):
        run("YOLOv5s-shaped, 16x3x640x640", yolo, x, dt, dt)
    run("YOLOv5s-shaped, 16x3x640x640", YoloV5ShapedF32(hw=640, width=32, int8=True, outputs=8), x, "int8", "f32")

    # The detection configuration itself: the topology of the shipped yolov5s_simp (70 convolutions, 13 Concat, three
    # 255-channel heads), generated line for line, with seeded weights (int8: unit-range feature-map scales, which
    # decide values, not time).
    from excalibur_amd import modelfile as mf
    from excalibur_amd import topologies

    class Seeded:
        def __init__(self, text, seed):
            self.lines = [l for l in text.splitlines()[2:] if l.strip()]
            self._text = text
            self._model = mf.SeededModel(mf.parse_topology(text), seed, default_fs=0.25)

        def topology(self):
            return self._text

        def write_model(self, path):
            mf.write_model(path, self._model.blobs)

    for dt, int8 in (("f32", False), ("f16", False), ("int8", True)):
        text, _ = topologies.yolov5s_simp(640, int8=int8)
        run("yolov5s_simp topology (3 heads x 255 channels), 16x3x640x640", Seeded(text, 5), x, dt, "f32" if int8 else dt)
    # the int8 network Excalibur ships: a residual network with Eltwise sums, ReLU layers and a depthwise tail
    light = topologies.unicorn_light_int8()
    light = light[0] if isinstance(light, tuple) else light
    x = r.uniform(0, 255, (64, 3, 128, 128)).astype(np.float32)
    run("unicorn_light_int8 topology, 64x3x128x128", Seeded(light, 6), x, "int8", "f32")
    return rows


def layer_table(ctx, iters=30):
    """Single layers of the small configurations through the C ABI, NHWC operands resident: cfg1 (float32 3x3, one image)
    and cfg2 (int8 3x3 and 1x1 at 8 x 128 x 80 x 80, int8 NHWC result). HIP events around `iters` back-to-back launches."""
    from excalibur_amd import hip
    rng = np.random.default_rng(1)
    rows = []

    def timed(fn):
        for _ in range(5):
            fn()
        ctx.sync()
        e0, e1 = hip.Event(), hip.Event()
        e0.record(ctx)
        for _ in range(iters):
            fn()
        e1.record(ctx)
        ctx.sync()
        return e0.elapsed_ms(e1) / iters

    def row(label, dtype, gop, ms):
        peak = {"f32": PEAK_F32_TFLOPS, "f16": PEAK_F16_TFLOPS, "int8": PEAK_INT8_TOPS}[dtype]
        rows.append({"layer": label, "dtype": dtype, "us": round(ms * 1e3, 1), "algorithmic_gop": round(gop, 3),
                     "achieved": round(gop / ms, 1), "peak": peak, "unit": "TOP/s" if dtype == "int8" else "TFLOP/s",
                     "frac": round(gop / ms / peak, 4)})

    n, c, hw, k = 1, 64, 56, 64   # cfg1
    d = ctx.conv_desc(n, c, hw, hw, k, 3, 1, 1, 1, c, k)
    x = ctx.array(rng.uniform(-1, 1, (n, hw, hw, c)).astype(np.float32))
    wp = ctx.pack_conv_weights(d, hip.F32, rng.normal(0, 0.05, (k, c, 3, 3)).astype(np.float32))
    b = ctx.array(rng.normal(0, 0.01, k).astype(np.float32))
    y = ctx.empty((n, k, hw, hw), np.float32)
    row("cfg1 3x3 1x64x56x56 -> 64", "f32", 2.0 * n * hw * hw * c * k * 9 / 1e9, timed(lambda: ctx.conv2d_f32(d, x, wp, b, None, None, y)))
    n, c, hw = 8, 128, 80         # cfg2
    xq = ctx.array(rng.integers(-127, 128, (n, hw, hw, c)).astype(np.int8))
    for kernel, k in ((3, 128), (3, 256), (1, 128), (1, 256)):
        d = ctx.conv_desc(n, c, hw, hw, k, kernel, 1, kernel // 2, 1, c, k, 0, 16.0)
        wp = ctx.pack_conv_weights(d, hip.I8, rng.integers(-127, 128, (k, c, kernel, kernel)).astype(np.int8))
        scale = ctx.array(rng.uniform(1e-4, 1e-2, k).astype(np.float32))
        b = ctx.array(rng.normal(0, 1, k).astype(np.float32))
        yq = ctx.empty((n, hw, hw, k), np.int8)
        row(f"cfg2 {kernel}x{kernel} 8x128x80x80 -> {k}", "int8", 2.0 * n * hw * hw * c * k * kernel * kernel / 1e9,
            timed(lambda: ctx.conv2d_i8(d, xq, wp, scale, b, None, yq)))
    return rows


def bandwidth_table(iters=20, quiet=False, ctx=None):
    """The path's memory-bound kernels at the benchmark network's tensor sizes, through the C ABI with preallocated
    operands: HIP events around `iters` back-to-back launches, algorithmic bytes (every operand read once, every result
    written once) over the 8 TB/s HBM peak. Returns [{"kernel", "us", "GB/s", "frac"}]."""
    from excalibur_amd import hip
    own_ctx = ctx is None
    ctx = hip.Ctx(0) if own_ctx else ctx
    L = hip.lib()
    rng = np.random.default_rng(0)
    cf, sz = ctypes.c_float, ctypes.c_size_t
    rows = []

    def bw(label, nbytes, fn):
        for _ in range(3):
            rc = fn()
            assert rc == 0, (label, rc, L.exhip_last_error())
        ctx.sync()
        e0, e1 = hip.Event(), hip.Event()
        e0.record(ctx)
        for _ in range(iters):
            fn()
        e1.record(ctx)
        ctx.sync()
        ms = e0.elapsed_ms(e1) / iters
        rows.append({"kernel": label, "us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1),
                     "frac": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 3), "MB": round(nbytes / 1e6, 1)})
        # under 32 MB a launch is over in a few microseconds: the figure is then the rate at which this loop issues
        # launches, not the kernel's bandwidth
        if nbytes < (32 << 20):
            rows[-1]["launch_bound"] = True
        if not quiet:
            print(f"{label:66s} {ms * 1e3:8.1f} us {nbytes / ms / 1e6:8.1f} GB/s {100 * nbytes / ms / 1e6 / PEAK_HBM_GBS:5.1f} %", file=sys.stderr, flush=True)

    n, c, h, w = 32, 64, 160, 160          # the stage-1 tensors of the benchmark network
    cnt = n * c * h * w
    xf = ctx.array(rng.normal(0, 1, (n, c, h, w)).astype(np.float32))
    yf, zf = ctx.empty((n, c, h, w), np.float32).zero(), ctx.empty((n, c, h, w), np.float32)
    xh = ctx.array(rng.normal(0, 1, (n, c, h, w)).astype(np.float16).view(np.uint16))
    yh, zh = ctx.empty((n, c, h, w), np.uint16).zero(), ctx.empty((n, c, h, w), np.uint16)
    xin = ctx.array(rng.uniform(-1, 1, (n, 3, 640, 640)).astype(np.float32))
    q = ctx.empty((n, 640, 640, 4), np.int8)
    bw("first-layer quantizer, f32 NCHW 32x3x640x640 -> int8 NHWC4", xin.size * 4 + n * 640 * 640 * 4,
       lambda: L.exhip_quantize_nchw_f32_to_nhwc_i8(ctx.h, xin.ptr, n, 3, 640, 640, cf(20.0), None, 4, q.ptr))
    bw("layout NCHW f32 -> NHWC f32", cnt * 8, lambda: L.exhip_nchw_f32_to_nhwc_f32(ctx.h, xf.ptr, n, c, h, w, c, zf.ptr))
    bw("layout NHWC f32 -> NCHW f32", cnt * 8, lambda: L.exhip_nhwc_f32_to_nchw_f32(ctx.h, xf.ptr, n, c, h, w, c, zf.ptr))
    bw("layout NCHW f16 -> NHWC f16", cnt * 4, lambda: L.exhip_nchw_f16_to_nhwc_f16(ctx.h, xh.ptr, n, c, h, w, c, zh.ptr))
    bw("layout NHWC f16 -> NCHW f16", cnt * 4, lambda: L.exhip_nhwc_f16_to_nchw_f16(ctx.h, xh.ptr, n, c, h, w, c, zh.ptr))
    bw("f32 -> f16", cnt * 6, lambda: L.exhip_f32_to_f16(ctx.h, xf.ptr, zh.ptr, sz(cnt)))
    bw("f16 -> f32", cnt * 6, lambda: L.exhip_f16_to_f32(ctx.h, xh.ptr, zf.ptr, sz(cnt)))
    bw("eltwise add + ReLU f32", cnt * 12, lambda: L.exhip_add_f32(ctx.h, xf.ptr, yf.ptr, zf.ptr, sz(cnt), 1))
    bw("eltwise add + ReLU f16", cnt * 6, lambda: L.exhip_add_f16(ctx.h, xh.ptr, yh.ptr, zh.ptr, sz(cnt), 1))
    bw("ReLU f32", cnt * 8, lambda: L.exhip_relu_f32(ctx.h, xf.ptr, zf.ptr, sz(cnt)))
    ptrs, coef = (ctypes.c_void_p * 2)(xf.ptr, yf.ptr), (ctypes.c_float * 2)(1.0, 1.0)
    bw("Eltwise SUM f32, two inputs", cnt * 12, lambda: L.exhip_eltwise_f32(ctx.h, ptrs, 2, coef, 1, zf.ptr, sz(cnt)))
    bw("HardSwish f32", cnt * 8, lambda: L.exhip_unary_f32(ctx.h, 0, xf.ptr, zf.ptr, sz(cnt), cf(1 / 6), cf(0.5)))
    bw("HardSwish f16", cnt * 4, lambda: L.exhip_unary_f16(ctx.h, 0, xh.ptr, zh.ptr, sz(cnt), cf(1 / 6), cf(0.5)))
    p0, p1 = ctx.array(rng.normal(0, 1, c).astype(np.float32)), ctx.array(rng.normal(0, 1, c).astype(np.float32))
    bw("BatchNorm f32", cnt * 8, lambda: L.exhip_channelwise_f32(ctx.h, 1, xf.ptr, zf.ptr, n, c, h * w, p0.ptr, p1.ptr, 0))
    bw("BatchNorm f16", cnt * 4, lambda: L.exhip_channelwise_f16(ctx.h, 1, xh.ptr, zh.ptr, n, c, h * w, p0.ptr, p1.ptr, 0))
    bw("BatchNorm f16 NHWC", cnt * 4,
       lambda: L.exhip_channelwise_nhwc_f16(ctx.h, 1, xh.ptr, zh.ptr, ctypes.c_size_t(n * h * w), c, p0.ptr, p1.ptr, 0))
    big = ctx.empty((n, 2 * c, h, w), np.float32)
    chs = (ctypes.c_int * 2)(c, c)
    bw("Concat f32, 2 x 64 channels", cnt * 16, lambda: L.exhip_concat_channels_f32(ctx.h, ptrs, chs, 2, n, h * w, big.ptr))
    small = ctx.array(rng.normal(0, 1, (n, c, h // 2, w // 2)).astype(np.float32))
    bw("Interp nearest x2 f32", cnt * 5, lambda: L.exhip_interp_nearest_f32(ctx.h, small.ptr, zf.ptr, n, c, h // 2, w // 2, h, w))
    pf = ctx.empty((n, c, h // 2, w // 2), np.float32)
    bw("max pool 3x3 s2 p1 f32 NCHW", cnt * 5,
       lambda: L.exhip_pool2d_nchw_f32(ctx.h, xf.ptr, pf.ptr, n, c, h, w, h // 2, w // 2, 0, 3, 3, 2, 2, 1, 1, 1, 1, 0))
    pq = ctx.empty((n, h // 2, w // 2, c), np.int8)
    bw("max pool 3x3 s2 p1 f32 NHWC + int8 copy", cnt * 5 + cnt // 4,
       lambda: L.exhip_maxpool2d_nhwc_f32(ctx.h, xf.ptr, pf.ptr, pq.ptr, cf(20.0), n, c, h, w, c, h // 2, w // 2, 3, 3, 2, 2, 1, 1))
    ph = ctx.empty((n, h // 2, w // 2, c), np.uint16)
    bw("max pool 3x3 s2 p1 f16 NHWC", cnt * 2 + cnt // 2,
       lambda: L.exhip_pool2d_nhwc_f16(ctx.h, xh.ptr, ph.ptr, n, c, h, w, c, h // 2, w // 2, 0, 3, 3, 2, 2, 1, 1, 1, 1, 0))
    w9, b9 = ctx.array(rng.normal(0, 0.1, (128, 9)).astype(np.float32)), ctx.array(rng.normal(0, 0.1, 128).astype(np.float32))
    bw("depthwise 3x3 s1 f32 NCHW, 32x64x160x160", cnt * 8,
       lambda: L.exhip_dwconv3x3_nchw_f32(ctx.h, xf.ptr, w9.ptr, b9.ptr, zf.ptr, n, c, h, w, 1, 1, 1, 1, 1, 1))
    dn, dc, dh = 64, 128, 56               # the MobileNet-style stack's middle maps
    dx = ctx.array(rng.normal(0, 1, (dn, dh, dh, dc)).astype(np.float16).view(np.uint16))
    dy = ctx.empty((dn, dh, dh, dc), np.uint16)
    bw("depthwise 3x3 s1 f16 NHWC, 64x128x56x56", dx.size * 4,
       lambda: L.exhip_dwconv3x3_nhwc_f16(ctx.h, dx.ptr, w9.ptr, b9.ptr, dy.ptr, dn, dc, dh, dh, dc, 1, 1, 1, 1, 1, 1))
    bw("depthwise 3x3 s2 f16 NHWC, 64x128x56x56", dx.size * 2 + dx.size // 2,
       lambda: L.exhip_dwconv3x3_nhwc_f16(ctx.h, dx.ptr, w9.ptr, b9.ptr, dy.ptr, dn, dc, dh, dh, dc, 2, 1, 1, 1, 1, 1))
    # global average pooling, the last layer of the MobileNet-style stack (64 x 1024 x 7 x 7) and of a 20 x 20 backbone
    gx = ctx.array(rng.normal(0, 1, (64, 7, 7, 1024)).astype(np.float16).view(np.uint16))
    gy = ctx.empty((64, 1, 1, 1024), np.uint16)
    bw("global average pool f16 NHWC, 64x1024x7x7", gx.size * 2 + gy.size * 2,
       lambda: L.exhip_pool2d_nhwc_f16(ctx.h, gx.ptr, gy.ptr, 64, 1024, 7, 7, 1024, 1, 1, 1, 7, 7, 1, 1, 0, 0, 0, 0, 0))
    gf = ctx.array(rng.normal(0, 1, (32, 512, 20, 20)).astype(np.float32))
    gfy = ctx.empty((32, 512, 1, 1), np.float32)
    bw("global average pool f32 NCHW, 32x512x20x20", gf.size * 4 + gfy.size * 4,
       lambda: L.exhip_pool2d_nchw_f32(ctx.h, gf.ptr, gfy.ptr, 32, 512, 20, 20, 1, 1, 1, 20, 20, 1, 1, 0, 0, 0, 0, 0))
    # the detection topology's glue on halves, and the layers that so far had correctness-grade kernels only
    fx = ctx.array(rng.integers(0, 1 << 15, (16, 3, 640, 640)).astype(np.uint16))
    fy = ctx.empty((16, 12, 320, 320), np.uint16)
    bw("Focus f16, 16x3x640x640", fx.size * 4, lambda: L.exhip_focus_f16(ctx.h, fx.ptr, fy.ptr, 16, 3, 640, 640))
    ix = ctx.array(rng.integers(0, 1 << 15, (64, 3, 224, 224)).astype(np.uint16))
    iy = ctx.empty((64, 224, 224, 4), np.uint16)
    bw("layout NCHW f16 (3 channels) -> NHWC f16 pixels of 4, 64x3x224x224", ix.size * 2 + iy.size * 2,
       lambda: L.exhip_nchw_f16_to_nhwc_f16(ctx.h, ix.ptr, 64, 3, 224, 224, 4, iy.ptr))
    hptrs, hchs = (ctypes.c_void_p * 2)(xh.ptr, yh.ptr), (ctypes.c_int * 2)(c, c)
    bigh = ctx.empty((n, h, w, 2 * c), np.uint16)
    pa, pb = ctx.array(rng.normal(0, 1, 2 * c).astype(np.float32)), ctx.array(rng.uniform(0.5, 2, 2 * c).astype(np.float32))
    bw("Concat -> BatchNorm -> LeakyReLU f16 NHWC, 2 x 64 channels", cnt * 8,
       lambda: L.exhip_concat_batchnorm_unary_nhwc_f16(ctx.h, hptrs, hchs, 2, sz(n * h * w), pa.ptr, pb.ptr, 1, cf(0.1), cf(0.0), bigh.ptr))
    tp, th_, tw_ = 48, 85, 6400            # a detection head: 16 images x 3 anchors, 85 values x 80 x 80 positions
    tx = ctx.array(rng.normal(0, 1, (tp, th_, tw_)).astype(np.float32))
    ty = ctx.empty((tp, tw_, th_), np.float32)
    bw("Transpose rows / columns f32, 48 planes of 85 x 6400", tx.size * 8, lambda: L.exhip_transpose_hw_f32(ctx.h, tx.ptr, ty.ptr, tp, th_, tw_))
    txh = ctx.array(rng.integers(0, 1 << 15, (tp, th_, tw_)).astype(np.uint16))
    tyh = ctx.empty((tp, tw_, th_), np.uint16)
    bw("Transpose rows / columns f16, 48 planes of 85 x 6400", txh.size * 4, lambda: L.exhip_transpose_hw_f16(ctx.h, txh.ptr, tyh.ptr, tp, th_, tw_))
    sx = ctx.array(rng.normal(0, 1, (16, 21, 320, 320)).astype(np.float32))
    sy = ctx.empty((16, 21, 320, 320), np.float32)
    bw("Softmax over 21 channels f32, 16x21x320x320", sx.size * 8, lambda: L.exhip_softmax_channels_f32(ctx.h, sx.ptr, sy.ptr, 16, 21, 320 * 320))
    # the int8 graph plan's glue: the fused front, Concat -> BatchNorm -> LeakyReLU on float32 NHWC with the int8 copy, a head's regrouping
    gx = ctx.array(rng.uniform(0, 255, (16, 3, 640, 640)).astype(np.float32))
    gq = ctx.empty((16, 320, 320, 32), np.int8)
    gm, gs = (cf * 3)(0.0, 0.0, 0.0), (cf * 3)(0.0039215, 0.0039215, 0.0039215)
    bw("Input + Focus + int8 quantizer, 16x3x640x640 -> 16x320x320x32", gx.size * 4 + gq.size,
       lambda: L.exhip_input_focus_quantize_nchw_f32_to_nhwc_i8(ctx.h, gx.ptr, 16, 3, 640, 640, gm, gs, cf(60.0), 32, gq.ptr))
    fptrs, fchs = (ctypes.c_void_p * 2)(xf.ptr, yf.ptr), (ctypes.c_int * 2)(c, c)
    bigq = ctx.empty((n, h, w, 2 * c), np.int8)
    bw("Concat -> BatchNorm -> LeakyReLU f32 NHWC -> int8, 2 x 64 channels", cnt * 8 + cnt * 2,
       lambda: L.exhip_concat_batchnorm_unary_nhwc_f32(ctx.h, fptrs, fchs, fchs, 2, sz(n * h * w), pa.ptr, pb.ptr, 1, cf(0.1), cf(0.0), 2 * c,
                                                       None, bigq.ptr, cf(8.0)))
    hx = ctx.array(rng.normal(0, 1, (16, 80, 80, 256)).astype(np.float32))
    hy = ctx.empty((16, 3, 6400, 85), np.float32)
    bw("Head regrouping f32 NHWC 16x80x80x(3x85) -> 16x3x6400x85", hy.size * 8,
       lambda: L.exhip_nhwc_f32_to_grouped_f32(ctx.h, hx.ptr, 16, 6400, 3, 85, 256, hy.ptr))
    if own_ctx:
        ctx.close()
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--hw", type=int, default=640)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--in-flight", type=int, default=2,
                    help="forwards in flight: steps are dealt in turn to this many pipelines, each on a HIP stream of its own (1..8)")
    ap.add_argument("--shared-gpu-plans", action="store_true",
                    help="set the planner option share_gpu: one more group per CU wherever a single activation tile buffer allows "
                         "it (3 %% faster with two forwards in flight, 2 %% slower with one; off by default)")
    ap.add_argument("--no-memory-bound", action="store_true", help="skip the memory-bound kernels' block of the line")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the other configurations' block of the line")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="set a library option (exhip_set_option) before the network is planned; may be repeated")
    ap.add_argument("--exhip-lib", default=None, metavar="PATH",
                    help="load this build of libexhip.so instead of the one in the tree (comparing kernel builds in one session)")
    ap.add_argument("--per-layer", action="store_true", help="print per-launch timings to stderr")
    ap.add_argument("--networks", action="store_true",
                    help="time the other configurations' whole topologies (MobileNet- and YOLOv5s-shaped, f32 / f16 / int8) "
                         "through the pipeline (per-layer executor; int8 graph plan) instead of the headline benchmark")
    ap.add_argument("--only", default=None, metavar="TEXT",
                    help="with --networks: only the rows whose '<network label> <dtype>' contains TEXT (e.g. 'yolov5s_simp topology (3 heads x 255 channels), 16x3x640x640 int8')")
    ap.add_argument("--bandwidth", action="store_true",
                    help="instead of the network: time the memory-bound kernels of the path and print their GB/s")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; the batch shards trivially across GPUs but no multi-GPU path "
              "is part of it (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    if args.exhip_lib:
        from excalibur_amd import hip as _hip
        _hip.LIB_PATH = os.path.abspath(args.exhip_lib)

    if args.option:   # library options hold for every mode of this script
        from excalibur_amd import pipeline as _xp
        for item in args.option:
            name, _, value = item.partition("=")
            _xp.set_option(name, int(value))
    if args.bandwidth:
        print(json.dumps({"metric": "achieved HBM GB/s of the memory-bound kernels", "peak_GB/s": PEAK_HBM_GBS,
                          "kernels": bandwidth_table()}))
        return
    if args.networks:
        print(json.dumps({"metric": "forward time of the generated topologies through the pipeline (executor per row)",
                          "networks": network_table(only=args.only)}))
        return

    import tempfile

    from excalibur_amd import hip
    from excalibur_amd import pipeline as xp
    from excalibur_amd.resnet18 import FusedRunner, ResNet18Int8

    ctx = hip.Ctx(0)
    net = ResNet18Int8(seed=1234, calib_hw=64)
    n, hw = args.batch, args.hw
    x = np.random.default_rng(99).uniform(-1, 1, (n, 3, hw, hw)).astype(np.float32)

    # The timed path: the generated .phai / .racy loaded through the host-side pipeline<float>(lines, model, device 0),
    # which runs the int8 chain as one fused plan over the exhip C ABI. The input blob is uploaded before timing.
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        model_path = f.name
    net.write_model(model_path)
    # Steps are dealt in turn to `in_flight` pipelines of the same network, each in a stream slot of its own (its own HIP
    # stream, activation buffers and input copy): step i + 1 is queued while step i runs, so the second forward's groups
    # fill the CUs the first leaves idle in the tail of every launch and in the hand-over between launches. Every step is
    # a whole forward of the batch; all K of them finish inside the timed region.
    in_flight = max(1, min(args.in_flight, 8))
    if args.shared_gpu_plans:
        xp.set_option("share_gpu", 1)
    pipes = []
    for k in range(in_flight):
        xp.set_stream_slot(k)
        q = xp.Pipeline(net.topology(), model_path, 0, "f32", fusion=True)
        q.set_input(x)
        pipes.append(q)
    xp.set_stream_slot(0)
    os.unlink(model_path)
    pipe = pipes[0]

    def timed(group, steps, warmup):
        for i in range(warmup):
            group[i % len(group)].run()
        for q in group:
            q.sync()
        t0 = time.perf_counter()
        for i in range(steps):
            group[i % len(group)].run()
        for q in group:
            q.sync()
        return time.perf_counter() - t0

    # The timed pipeline brackets the convolution launches of every forward with a HIP event pair of its own (a ring of
    # 32 pairs, read after the loop's closing synchronisation): the roofline's launch durations are taken in the steps
    # that `value` counts, events' own cost included in both.
    pipe.time_fused_span(-2)
    one_elapsed = timed(pipes[:1], args.steps, args.warmup)
    spans = pipe.recent_spans(min(args.steps, 32))
    _, n_conv = pipe.last_span()
    pipe.time_fused_span(-1)
    assert pipe.fused, "the int8 ResNet-18 topology did not take the fused plan"
    # `value` is the rate with one forward in flight, the regime the roofline block and the profiles describe; the rate
    # with `in_flight` forwards queued on streams of their own is reported beside it (config.in_flight_N).
    many_elapsed = timed(pipes, args.steps, args.warmup) if in_flight > 1 else one_elapsed
    elapsed = one_elapsed
    ms_per_step = elapsed / args.steps * 1e3
    images_per_s = n * args.steps / elapsed
    # every pipeline was fed the same batch: after the timed loops their results must be the same bytes
    first_out = pipes[0].get(net.output)
    assert np.isfinite(first_out).all() and np.count_nonzero(first_out) > first_out.size // 8
    for q in pipes[1:]:
        assert np.array_equal(q.get(net.output), first_out), "pipelines in different stream slots disagree"

    # One plain copy-like kernel of known size (ReLU over 64 Mi floats: 256 MiB read + 256 MiB written), outside
    # the timed region: it calibrates the FETCH_SIZE / WRITE_SIZE counters when this command runs under rocprofv3 --pmc.
    cal = ctx.empty((64 << 20,), np.float32).zero()
    ctx.relu_f32(cal).free()
    cal.free()

    # The same launches issued one by one from Python, for per-kernel event timing.
    run = FusedRunner(ctx, net, n, hw, hw)
    run.set_input(x)
    for _ in range(2):
        run.forward()
    ctx.sync()

    # The dominant kernel's launches of one forward, timed with one HIP event pair on the library's stream: from in
    # front of the first convolution to behind the last (the launches follow each other without anything else between
    # them; an input quantizer in front of them, where the stem kernel does not quantize its own input, stays outside).
    # The interval holds the launches and the queue's hand-over between them, as the sum of a kernel trace's durations
    # does. The samples are those of the timed region's last steps (above).
    assert n_conv == len(run.conv_gop), f"the fused plan's span holds {n_conv} launches, expected {len(run.conv_gop)} convolutions"
    conv_ms = float(np.mean(spans))
    conv_gop = sum(run.conv_gop.values())
    achieved_tops = conv_gop / conv_ms  # GOP / ms = TOP/s

    if args.per_layer:
        # Per-launch intervals for diagnosis: an event pair around every launch, minus what a pair adds (the interval
        # around a launch that does next to nothing, median of 50, each behind a long kernel so that the queue is busy).
        tiny_in, tiny_out = ctx.empty((64,), np.float32).zero(), ctx.empty((64,), np.float32)
        big_in, big_out = ctx.empty((8 << 20,), np.float32).zero(), ctx.empty((8 << 20,), np.float32)
        lib = hip.lib()
        pairs = [(hip.Event(), hip.Event()) for _ in range(50)]
        for e0, e1 in pairs:
            lib.exhip_relu_f32(ctx.h, big_in.ptr, big_out.ptr, ctypes.c_size_t(8 << 20))
            lib.exhip_event_record(ctx.h, e0.h)
            lib.exhip_relu_f32(ctx.h, tiny_in.ptr, tiny_out.ptr, ctypes.c_size_t(64))
            lib.exhip_event_record(ctx.h, e1.h)
        ctx.sync()
        event_overhead_ms = float(np.median([e0.elapsed_ms(e1) for e0, e1 in pairs]))
        acc = {}
        reps = max(3, min(args.steps, 10))
        for _ in range(reps):
            for label, kind, ms in run.forward_timed():
                a = acc.setdefault(label, [kind, 0.0])
                a[1] += max(ms - event_overhead_ms, 0.0) / reps
        for label, (kind, ms) in acc.items():
            extra = f"{run.conv_gop[label] / ms:8.1f} TOP/s" if kind == "conv" else f"{run.bytes[label] / ms / 1e6:8.1f} GB/s"
            print(f"{label:16s} {kind:5s} {ms * 1e3:9.1f} us  {extra}", file=sys.stderr)
        print(f"sum of launches {sum(v[1] for v in acc.values()):.3f} ms (event overhead {event_overhead_ms * 1e3:.1f} us subtracted from each), "
              f"convolution span {conv_ms:.3f} ms, step {ms_per_step:.3f} ms", file=sys.stderr)

    line = {
        "metric": "images/sec + achieved int8 TOPS (% MFMA peak) for ResNet-18-shaped conv stack, 1 GPU",
        "value": round(images_per_s, 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": f"ResNet-18-shaped int8 backbone (7x7 s2 stem, 3x3 s2 maxpool, 4 stages of BasicBlocks "
                               f"64/128/256/512, add+ReLU, per-channel requant), input {n}x3x{hw}x{hw}",
                   "batch": n, "device": ctx.device_name().strip(), "forwards_in_flight": 1,
                   f"in_flight_{in_flight}": {"value": round(n * args.steps / many_elapsed, 1), "ms_per_step": round(many_elapsed / args.steps * 1e3, 4),
                                              "note": f"the same steps dealt to {in_flight} pipelines on HIP streams of their own: launches of "
                                                      f"different forwards overlap, none is shortened"},
                   "int8_tops_whole_step": round(conv_gop / ms_per_step, 1)},
        "roofline": {"bound": "mfma", "kernel": "the int8 convolution launches of a step (stem_conv_pool_kernel, conv3x3_i8_lean_kernel, "
                                                 f"conv_igemm_kernel: {n_conv} launches for the 20 convolutions)",
                     "achieved": round(achieved_tops, 1), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": round(achieved_tops / PEAK_INT8_TOPS, 4), "traffic": measured_traffic(n, hw),
                     "algorithmic_gop_per_step": round(conv_gop, 1), "launches_per_step": n_conv, "avg_launch_ms": round(conv_ms / n_conv, 4),
                     "timed_region": {"achieved": round(conv_gop / ms_per_step, 1), "frac": round(conv_gop / ms_per_step / PEAK_INT8_TOPS, 4),
                                      "note": "algorithmic GOP of a step over the wall time per step of the timed region (one forward in "
                                              "flight, host-side launch gaps included)"},
                     "timing": f"HIP events around the {n_conv} consecutive launches of a forward, recorded by the timed pipeline in "
                               f"the steps of the timed region (one forward in flight), mean of its last {len(spans)} steps"},
    }
    if not args.no_memory_bound:
        every = bandwidth_table(iters=10, quiet=True, ctx=ctx)
        rows = [r for r in every if not r.get("launch_bound")]
        fr = sorted(r["frac"] for r in rows)
        worst = min(rows, key=lambda r: r["frac"])
        line["memory_bound"] = {"bound": "hbm", "peak": PEAK_HBM_GBS, "unit": "GB/s", "kernels": len(rows),
                                "worst_frac": worst["frac"], "worst_kernel": worst["kernel"], "median_frac": fr[len(fr) // 2],
                                "below_0.60": [r["kernel"] for r in rows if r["frac"] < 0.60],
                                "launch_bound": [f'{r["kernel"]} ({r["MB"]} MB, {r["us"]} us per launch)' for r in every if r.get("launch_bound")],
                                "timing": "HIP events around 10 back-to-back launches of each memory-bound kernel of the path, "
                                          "algorithmic bytes over the 8 TB/s peak (python bench.py --bandwidth prints every row)"}
    if not args.no_other_configs:
        # the other configurations: single layers of cfg1 / cfg2 and the whole generated topologies of cfg3 / cfg5 through
        # the per-layer executor (python bench.py --networks prints the latter as a table)
        line["other_configs"] = {"layers": layer_table(ctx), "networks": network_table(iters=5),
                                 "note": "networks: wall time per forward of the executor the row names, algorithmic GOP of the batch "
                                         "(convolutions and inner products) over it, against the dense MFMA peak of the dtype"}
    if not args.no_cpu_baseline:
        one, many = cpu_baseline(net, hw)
        line["cpu_baseline"] = one
        if many:
            line["cpu_baseline_all_cores"] = many
    print(json.dumps(line))
    for q in pipes:
        q.close()
    ctx.close()


if __name__ == "__main__":
    main()
