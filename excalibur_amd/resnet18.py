"""ResNet-18-shaped int8 backbone in Excalibur's own terms: a `.phai` topology, a `.racy` weight blob with
per-output-channel weight scales and per-tensor activation scales, and the fused MI355X execution of it.

Shape (7x7 s2 stem, 3x3 s2 max pool, four stages of two BasicBlocks with 64/128/256/512 channels, 1x1 s2
projection shortcuts, BinaryOp add + ReLU) follows the way the reference's shipped ResNet-18 is written
(models/det_db_resnet18.phai:3-64: Convolution -> ReLU -> ... -> BinaryOp 0=0 -> ReLU -> Split).

Weights are random (He-normal) and quantized with ws_k = 127 / max|W_k|; activation scales come from a
synthetic calibration pass of the float network on a small random image, fs = 127 / max|x|. Everything is
seeded, so the GPU path and the CPU checker read identical bytes.
"""
import numpy as np

from . import modelfile as mf

STAGES = (64, 128, 256, 512)


def _np_conv(x, w, stride, pad):
    """float32 convolution by im2col (calibration only, tiny inputs)."""
    n, c, h, wd = x.shape
    k, _, kh, kw = w.shape
    xp = np.pad(x, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
    oh, ow = (h + 2 * pad - kh) // stride + 1, (wd + 2 * pad - kw) // stride + 1
    cols = np.empty((n, c, kh, kw, oh, ow), np.float32)
    for i in range(kh):
        for j in range(kw):
            cols[:, :, i, j] = xp[:, :, i:i + stride * oh:stride, j:j + stride * ow:stride]
    return np.einsum("kq,nqp->nkp", w.reshape(k, -1), cols.reshape(n, c * kh * kw, oh * ow)).reshape(n, k, oh, ow)


def _np_maxpool(x, k, s, p):
    n, c, h, w = x.shape
    xp = np.pad(x, ((0, 0), (0, 0), (p, p), (p, p)), constant_values=-np.inf)
    oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
    out = np.full((n, c, oh, ow), -np.inf, np.float32)
    for i in range(k):
        for j in range(k):
            out = np.maximum(out, xp[:, :, i:i + s * oh:s, j:j + s * ow:s])
    return out


class ConvLayer:
    def __init__(self, name, bottom, top, c, k, kernel, stride, pad, act):
        self.name, self.bottom, self.top = name, bottom, top
        self.c, self.k, self.kernel, self.stride, self.pad, self.act = c, k, kernel, stride, pad, act
        self.w_i8 = self.ws = self.bias = None
        self.fs = None

    def line(self):
        return mf.conv_line("Convolution", self.name, self.bottom, self.top, self.k, self.kernel, self.stride, self.pad,
                            True, self.k * self.c * self.kernel * self.kernel, 1, int8=True, act=self.act)

    def blob(self):
        return mf.conv_blob_i8(self.w_i8, self.bias, self.ws, self.fs)


class ResNet18Int8:
    """Builds the network description. `lines` is the topology, `convs` the weighted layers in file order."""

    def __init__(self, seed=1234, calib_hw=64):
        rng = np.random.default_rng(seed)
        self.convs = []
        self.lines = []
        self.blocks = []  # (conv1, conv2, downsample or None)
        x = rng.uniform(-1, 1, (1, 3, calib_hw, calib_hw)).astype(np.float32)

        def conv(name, bottom, top, c, k, kernel, stride, pad, act, xin):
            layer = ConvLayer(name, bottom, top, c, k, kernel, stride, pad, act)
            fan_in = c * kernel * kernel
            wf = rng.normal(0, np.sqrt(2.0 / fan_in), (k, c, kernel, kernel)).astype(np.float32)
            layer.ws = (np.float32(127.0) / np.abs(wf).reshape(k, -1).max(axis=1)).astype(np.float32)
            layer.w_i8 = np.clip(np.rint(wf * layer.ws[:, None, None, None]), -127, 127).astype(np.int8)
            layer.bias = rng.normal(0, 0.05, (k,)).astype(np.float32)
            layer.fs = np.float32(127.0 / max(float(np.abs(xin).max()), 1e-6))
            self.convs.append(layer)
            self.lines.append(layer.line())
            y = _np_conv(xin, layer.w_i8.astype(np.float32) / layer.ws[:, None, None, None], stride, pad)
            y = y + layer.bias[None, :, None, None]
            return layer, (np.maximum(y, 0) if act == 1 else y)

        self.stem, x = conv("conv1", "data", "conv1", 3, 64, 7, 2, 3, 1, x)
        self.lines.append(mf.pool_line("pool1", "conv1", "pool1", 0, 3, 2, 1))
        x = _np_maxpool(x, 3, 2, 1)
        cur, cin = "pool1", 64
        for si, k in enumerate(STAGES):
            for bi in range(2):
                stride = 2 if (si > 0 and bi == 0) else 1
                p = f"l{si + 1}b{bi + 1}"
                need_ds = stride != 1 or cin != k
                n_split = 2
                outs = [f"{cur}_s{i}" for i in range(n_split)]
                self.lines.append(f"Split {p}_split 1 {n_split} {cur} " + " ".join(outs))
                c1, y = conv(f"{p}_conv1", outs[0], f"{p}_c1", cin, k, 3, stride, 1, 1, x)
                c2, y = conv(f"{p}_conv2", f"{p}_c1", f"{p}_c2", k, k, 3, 1, 1, 0, y)
                ds = None
                short, short_name = x, outs[1]
                if need_ds:
                    ds, short = conv(f"{p}_down", outs[1], f"{p}_ds", cin, k, 1, stride, 0, 0, x)
                    short_name = f"{p}_ds"
                self.lines.append(f"BinaryOp {p}_add 2 1 {p}_c2 {short_name} {p}_sum 0=0")
                self.lines.append(f"ReLU {p}_relu 1 1 {p}_sum {p}_out")
                x = np.maximum(y + short, 0)
                self.blocks.append((c1, c2, ds))
                cur, cin = f"{p}_out", k
        self.output = cur

    def topology(self):
        return mf.topology(self.lines, "resnet18_int8")

    def write_model(self, path):
        mf.write_model(path, [c.blob() for c in self.convs])

    def gmac_per_image(self, h, w):
        """Algorithmic multiply-accumulates per image: N*OH*OW*K*C*kh*kw summed over the convolutions."""
        total = 0
        hh, ww = h, w
        oh, ow = (hh + 6 - 7) // 2 + 1, (ww + 6 - 7) // 2 + 1
        total += oh * ow * 64 * 3 * 49
        oh, ow = (oh + 2 - 3) // 2 + 1, (ow + 2 - 3) // 2 + 1
        for c1, c2, ds in self.blocks:
            ih, iw = oh, ow
            oh, ow = (ih + 2 - 3) // c1.stride + 1, (iw + 2 - 3) // c1.stride + 1
            total += oh * ow * c1.k * c1.c * 9 + oh * ow * c2.k * c2.c * 9
            if ds is not None:
                total += oh * ow * ds.k * ds.c
        return total / 1e9


class FusedRunner:
    """Executes the network on one GPU through the exhip C ABI with int8 NHWC tensors between layers.

    Every convolution's epilogue applies dequantization + bias (+ ReLU / shortcut add + ReLU) and writes what
    its consumers read: the next convolution's int8 input (quantized with that layer's fs) and, where the
    tensor feeds a shortcut, its float32 copy. The values are the reference's: each int8 input is
    float32_to_int8(x * fs) of the very float the CPU path would have produced.
    """

    def __init__(self, ctx, net, n, h, w, profile=False, fuse_pool=True, fuse_projection=True):
        from . import hip
        self.ctx, self.net, self.n, self.h, self.w = ctx, net, n, h, w
        self.fuse_pool = fuse_pool  # stem convolution and max pool as one launch
        self.fuse_projection = fuse_projection  # a block's projection shortcut inside its second convolution's launch
        self.hip = hip
        self.steps = []       # (label, kind, callable)
        self.conv_gop = {}    # label -> algorithmic GOP per launch
        self.bytes = {}       # label -> algorithmic bytes per launch
        self._build()

    def _conv(self, layer, x_i8, hin, win, cs_in, residual, post_relu, fs_out, want_f32_nhwc, want_nchw):
        ctx, hip = self.ctx, self.hip
        ks = hip.pad_to(layer.k, 32)
        d = ctx.conv_desc(self.n, layer.c, hin, win, layer.k, layer.kernel, layer.stride, layer.pad, layer.act, cs_in, ks,
                          post_relu, float(fs_out or 0.0))
        oh, ow = ctx.conv_out_hw(d)
        wp = ctx.pack_conv_weights(d, hip.I8, layer.w_i8)
        ws, fs = layer.ws, layer.fs
        with np.errstate(divide="ignore"):
            scale = np.where(np.abs(ws.astype(np.float64)) <= 1e-6, np.float32(0),
                             np.float32(1.0) / (ws * fs).astype(np.float32)).astype(np.float32)
        scale_d, bias_d = ctx.array(scale), ctx.array(layer.bias)
        y_i8 = ctx.empty((self.n, oh, ow, ks), np.int8) if fs_out is not None else None
        y_f32 = ctx.empty((self.n, oh, ow, ks), np.float32) if want_f32_nhwc else None
        y_nchw = ctx.empty((self.n, layer.k, oh, ow), np.float32) if want_nchw else None
        gop = 2.0 * self.n * oh * ow * layer.k * layer.c * layer.kernel * layer.kernel / 1e9
        self.conv_gop[layer.name] = gop
        self.steps.append((layer.name, "conv", lambda: ctx.conv2d_i8(d, x_i8, wp, scale_d, bias_d, residual, y_i8, y_f32,
                                                                      y_nchw, None)))
        return y_i8, y_f32, y_nchw, oh, ow, ks

    def _scales(self, layer):
        ws, fs = layer.ws, layer.fs
        with np.errstate(divide="ignore"):
            scale = np.where(np.abs(ws.astype(np.float64)) <= 1e-6, np.float32(0),
                             np.float32(1.0) / (ws * fs).astype(np.float32)).astype(np.float32)
        return self.ctx.array(scale), self.ctx.array(layer.bias)

    def _conv_projection(self, layer, x_i8, hin, win, cs_in, proj, xp_i8, hp, wp_, cs_p, fs_out):
        """A block's second convolution with the block's projection shortcut computed in the same launch (sum and ReLU
        included): int8 and float32 NHWC results, or None where the library leaves the pair to two launches."""
        ctx, hip = self.ctx, self.hip
        ks = hip.pad_to(layer.k, 32)
        d = ctx.conv_desc(self.n, layer.c, hin, win, layer.k, layer.kernel, layer.stride, layer.pad, layer.act, cs_in, ks, 1, float(fs_out))
        dp = ctx.conv_desc(self.n, proj.c, hp, wp_, proj.k, proj.kernel, proj.stride, proj.pad, proj.act, cs_p, ks, 0, 0.0)
        oh, ow = ctx.conv_out_hw(d)
        if ks != layer.k or cs_p != proj.c or ctx.conv_out_hw(dp) != (oh, ow):
            return None
        w_main, w_proj = ctx.pack_conv_weights(d, hip.I8, layer.w_i8), ctx.pack_conv_weights(dp, hip.I8, proj.w_i8)
        scale_d, bias_d = self._scales(layer)
        scale_p, bias_p = self._scales(proj)
        y_i8 = ctx.empty((self.n, oh, ow, ks), np.int8)
        y_f32 = ctx.empty((self.n, oh, ow, ks), np.float32)
        if not ctx.conv2d_i8_projection(d, x_i8, w_main, scale_d, bias_d, dp, xp_i8, w_proj, scale_p, bias_p, y_i8, y_f32):
            return None
        self.conv_gop[layer.name] = (2.0 * self.n * oh * ow * layer.k * layer.c * layer.kernel * layer.kernel +
                                     2.0 * self.n * oh * ow * proj.k * proj.c) / 1e9
        self.steps.append((layer.name, "conv", lambda: ctx.conv2d_i8_projection(d, x_i8, w_main, scale_d, bias_d, dp, xp_i8, w_proj,
                                                                                  scale_p, bias_p, y_i8, y_f32)))
        return y_i8, y_f32, None, oh, ow, ks

    def _conv_maxpool(self, layer, x_i8, hin, win, cs_in, fs_out):
        """Convolution and the 3x3 stride-2 pad-1 max pool behind it as one launch: pooled f32 and int8 NHWC."""
        ctx, hip = self.ctx, self.hip
        d = ctx.conv_desc(self.n, layer.c, hin, win, layer.k, layer.kernel, layer.stride, layer.pad, layer.act, cs_in, layer.k,
                          0, float(fs_out))
        oh, ow = ctx.conv_out_hw(d)
        ph, pw = (oh + 2 - 3) // 2 + 1, (ow + 2 - 3) // 2 + 1
        wp = ctx.pack_conv_weights(d, hip.I8, layer.w_i8)
        ws, fs = layer.ws, layer.fs
        with np.errstate(divide="ignore"):
            scale = np.where(np.abs(ws.astype(np.float64)) <= 1e-6, np.float32(0),
                             np.float32(1.0) / (ws * fs).astype(np.float32)).astype(np.float32)
        scale_d, bias_d = ctx.array(scale), ctx.array(layer.bias)
        y = ctx.empty((self.n, ph, pw, layer.k), np.float32)
        yq = ctx.empty((self.n, ph, pw, layer.k), np.int8)
        self.conv_gop[layer.name] = 2.0 * self.n * oh * ow * layer.k * layer.c * layer.kernel * layer.kernel / 1e9
        self.steps.append((layer.name, "conv", lambda: ctx.conv2d_i8_maxpool3x3s2(d, 1, ph, pw, x_i8, wp, scale_d, bias_d, yq, y)))
        return y, yq, ph, pw, layer.k

    def _stem(self, layer, x, fs_out):
        """Quantizer, stem convolution and max pool as one launch where the library offers it (None otherwise)."""
        ctx, hip = self.ctx, self.hip
        d = ctx.conv_desc(self.n, layer.c, self.h, self.w, layer.k, layer.kernel, layer.stride, layer.pad, layer.act, 4, layer.k,
                          0, float(fs_out))
        oh, ow = ctx.conv_out_hw(d)
        ph, pw = (oh + 2 - 3) // 2 + 1, (ow + 2 - 3) // 2 + 1
        wp = ctx.pack_conv_weights(d, hip.I8, layer.w_i8)
        ws, fs = layer.ws, layer.fs
        with np.errstate(divide="ignore"):
            scale = np.where(np.abs(ws.astype(np.float64)) <= 1e-6, np.float32(0),
                             np.float32(1.0) / (ws * fs).astype(np.float32)).astype(np.float32)
        nonneg = bool((scale >= 0).all())
        scale_d, bias_d = ctx.array(scale), ctx.array(layer.bias)
        y = ctx.empty((self.n, ph, pw, layer.k), np.float32)
        yq = ctx.empty((self.n, ph, pw, layer.k), np.int8)
        if not ctx.stem_f32_conv_i8_maxpool3x3s2(d, 1, ph, pw, x, float(fs), wp, scale_d, nonneg, bias_d, yq, y):
            return None
        self.conv_gop[layer.name] = 2.0 * self.n * oh * ow * layer.k * layer.c * layer.kernel * layer.kernel / 1e9
        self.steps.append((layer.name, "conv", lambda: ctx.stem_f32_conv_i8_maxpool3x3s2(d, 1, ph, pw, x, float(fs), wp, scale_d, nonneg,
                                                                                         bias_d, yq, y)))
        return y, yq, ph, pw, layer.k

    def _quantize_input(self, x, q, fs):
        import ctypes
        ctx, n, h, w = self.ctx, self.n, self.h, self.w
        lib, check = self.hip.lib(), self.hip._check
        fs = ctypes.c_float(float(fs))
        self.bytes["quantize_input"] = n * h * w * (3 * 4 + 4)
        self.steps.append(("quantize_input", "bw", lambda: check(
            lib.exhip_quantize_nchw_f32_to_nhwc_i8(ctx.h, x.ptr, n, 3, h, w, fs, None, 4, q.ptr))))

    def _maxpool(self, x_f32, c, h, w, cs, fs_out):
        """3x3 stride-2 pad-1 max pool on NHWC f32 that also emits the next convolution's int8 input."""
        import ctypes
        ctx, n = self.ctx, self.n
        lib, check = self.hip.lib(), self.hip._check
        ph, pw = (h + 2 - 3) // 2 + 1, (w + 2 - 3) // 2 + 1
        y = ctx.empty((n, ph, pw, cs), np.float32)
        yq = ctx.empty((n, ph, pw, cs), np.int8)
        fs = ctypes.c_float(float(fs_out))
        self.bytes["maxpool"] = n * (h * w * cs * 4 + ph * pw * cs * 5)
        self.steps.append(("maxpool", "bw", lambda: check(lib.exhip_maxpool2d_nhwc_f32(
            ctx.h, x_f32.ptr, y.ptr, yq.ptr, fs, n, c, h, w, cs, ph, pw, 3, 3, 2, 2, 1, 1))))
        return y, yq, ph, pw

    def _build(self):
        # Each launch is recorded by a helper that binds its own arguments: a closure made here would see the
        # loop variables' final values when it runs.
        ctx, net, n = self.ctx, self.net, self.n
        self.x = ctx.empty((n, 3, self.h, self.w), np.float32)
        self.q0 = ctx.empty((n, self.h, self.w, 4), np.int8)
        stem = self._stem(net.stem, self.x, net.blocks[0][0].fs) if self.fuse_pool else None
        if stem is not None:
            pool_f32, pool_i8, ph, pw, ks = stem
        elif self.fuse_pool:
            self._quantize_input(self.x, self.q0, net.stem.fs)
            pool_f32, pool_i8, ph, pw, ks = self._conv_maxpool(net.stem, self.q0, self.h, self.w, 4, net.blocks[0][0].fs)
        else:
            self._quantize_input(self.x, self.q0, net.stem.fs)
            _, stem_f32, _, oh, ow, ks = self._conv(net.stem, self.q0, self.h, self.w, 4, None, 0, None, True, False)
            pool_f32, pool_i8, ph, pw = self._maxpool(stem_f32, 64, oh, ow, ks, net.blocks[0][0].fs)
        cur_i8, cur_f32, hh, ww, cs = pool_i8, pool_f32, ph, pw, ks
        nb = len(net.blocks)
        for bi, (c1, c2, ds) in enumerate(net.blocks):
            last = bi == nb - 1
            nxt_fs = None if last else net.blocks[bi + 1][0].fs
            if ds is not None:
                assert ds.fs == c1.fs, "both consumers of a tensor share its activation scale"
            a_i8, _, _, oh, ow, ks = self._conv(c1, cur_i8, hh, ww, cs, None, 0, c2.fs, False, False)
            # the float32 copy is the next block's shortcut: not needed when that block has a downsample convolution
            want_f32 = not last and net.blocks[bi + 1][2] is None
            fused = None
            if ds is not None and want_f32 and self.fuse_projection:
                fused = self._conv_projection(c2, a_i8, oh, ow, ks, ds, cur_i8, hh, ww, cs, nxt_fs)
            if fused is not None:
                o_i8, o_f32, o_nchw, oh, ow, ks = fused
            else:
                if ds is not None:
                    _, short, _, _, _, _ = self._conv(ds, cur_i8, hh, ww, cs, None, 0, None, True, False)
                else:
                    short = cur_f32
                o_i8, o_f32, o_nchw, oh, ow, ks = self._conv(c2, a_i8, oh, ow, ks, short, 1, nxt_fs, want_f32, last)
            cur_i8, cur_f32, hh, ww, cs = o_i8, o_f32, oh, ow, ks
            if last:
                self.out = o_nchw

    def set_input(self, x_host):
        self.x.upload(x_host)

    def forward(self):
        for _, _, fn in self.steps:
            fn()

    def forward_conv_span(self):
        """One forward with one HIP event pair around its convolution launches (from in front of the first one to
        behind the last launch); returns (ms, convolution launches). Everything else in the span must be
        convolutions too, which holds when the stem's pool is fused."""
        kinds = [kind for _, kind, _ in self.steps]
        first = kinds.index("conv")
        assert all(k == "conv" for k in kinds[first:]), "a non-convolution launch inside the span"
        if not hasattr(self, "_span"):
            self._span = (self.hip.Event(), self.hip.Event())
        record, ctx_h = self.hip.lib().exhip_event_record, self.ctx.h
        e0, e1 = self._span
        for i, (_, _, fn) in enumerate(self.steps):
            if i == first:
                record(ctx_h, e0.h)
            fn()
        record(ctx_h, e1.h)
        self.ctx.sync()
        return e0.elapsed_ms(e1), len(kinds) - first

    def forward_timed(self):
        """One forward with a HIP event pair around every launch; returns [(label, kind, ms)].

        The events exist before the first launch and are recorded through the bare library entry point, so
        that the host stays ahead of the GPU and the intervals hold the kernels, not host-side gaps.
        """
        import ctypes
        if not hasattr(self, "_events"):
            self._events = [(self.hip.Event(), self.hip.Event()) for _ in self.steps]
        record, ctx_h = self.hip.lib().exhip_event_record, self.ctx.h
        for (label, kind, fn), (e0, e1) in zip(self.steps, self._events):
            record(ctx_h, e0.h)
            fn()
            record(ctx_h, e1.h)
        self.ctx.sync()
        return [(label, kind, e0.elapsed_ms(e1)) for (label, kind, fn), (e0, e1) in zip(self.steps, self._events)]
