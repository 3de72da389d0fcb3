"""A YOLOv5s-shaped detector (float, or with int8 convolutions) as `.phai` topology text + `.racy` weights, built from a seed.

The layer mix of the detection topology the library ships with (Input scaling, Focus, convolutions with HardSwish, a
cross-stage block with a residual BinaryOp sum, Concat + BatchNorm + LeakyRelu, a spatial pyramid of 5 / 9 / 13 max
pools, nearest upsampling into a Concat with an earlier stage, and two heads that end in Reshape + Transpose) at a size
a CPU evaluates in a second. One image per forward: the reference's Focus layer fills image 0 only.
"""
import numpy as np

from . import modelfile as mf


class YoloV5ShapedF32:
    def __init__(self, seed=11, hw=64, width=8, anchors=3, outputs=6, int8=False, fs=96.0):
        """int8: every convolution carries int8 weights with per-channel scales ws = 127 / max|w| and quantizes its
        input with the feature-map scale `fs` (activations of this network stay below 1.6, so a few saturate); the other layers stay
        float, as in the library's int8 topologies."""
        r = np.random.default_rng(seed)
        self.hw = hw
        self.int8 = int8
        self.lines, self.blobs, self.ops = [], [], []
        self.scale = 0.0039215
        self.lines.append(f"Input images 0 1 images 0={hw} 1={hw} 2=3 3=0,0,0 4={self.scale!r}")
        self.ops.append(("input", "images_input", "images"))
        self._r = r
        self._n = 0

        def name(prefix):
            self._n += 1
            return f"{prefix}_{self._n}"

        def conv(bottom, cin, k, kernel, stride, act=True, bias=True):
            pad = kernel // 2
            w = r.normal(0, np.sqrt(2.0 / (cin * kernel * kernel)), (k, cin, kernel, kernel)).astype(np.float32)
            b = r.normal(0, 0.05, (k,)).astype(np.float32) if bias else None
            top = name("conv")
            self.lines.append(mf.conv_line("Convolution", top + "_l", bottom, top, k, kernel, stride, pad, bias, w.size, 1, int8=int8, act=0))
            if int8:
                ws = (np.float32(127.0) / np.abs(w).reshape(k, -1).max(axis=1)).astype(np.float32)
                wq = np.clip(np.rint(w * ws[:, None, None, None]), -127, 127).astype(np.int8)
                self.blobs.append(mf.conv_blob_i8(wq, b, ws, np.float32(fs)))
                self.ops.append(("conv_i8", bottom, top, wq, b, kernel, stride, pad, ws, np.float32(fs)))
            else:
                self.blobs.append(mf.conv_blob_f32(w, b))
                self.ops.append(("conv", bottom, top, w, b, kernel, stride, pad))
            if not act:
                return top
            out = name("hs")
            self.lines.append(f"HardSwish {out}_l 1 1 {top} {out} 0=1.666667e-01 1=5.000000e-01")
            self.ops.append(("hardswish", top, out, np.float32(1.666667e-01), np.float32(0.5)))
            return out

        def split(bottom, n):
            tops = [f"{bottom}_s{i}" for i in range(n)]
            self.lines.append(f"Split {bottom}_split 1 {n} {bottom} " + " ".join(tops))
            self.ops.append(("split", bottom, tops))
            return tops

        def concat(bottoms):
            top = name("cat")
            self.lines.append(f"Concat {top}_l {len(bottoms)} 1 " + " ".join(bottoms) + f" {top} 0=-1")
            self.ops.append(("concat", bottoms, top))
            return top

        self.lines.append("YoloV5Focus focus 1 1 images focus")
        self.ops.append(("focus", "images", "focus"))
        x = conv("focus", 12, width, 3, 1)
        x = conv(x, width, 2 * width, 3, 2)                       # hw / 4
        # cross-stage block
        c, hdn = 2 * width, width
        a, b = split(x, 2)
        u = conv(b, c, hdn, 1, 1)
        u0, u1 = split(u, 2)
        v = conv(conv(u1, hdn, hdn, 1, 1), hdn, hdn, 3, 1)
        s = name("add")
        self.lines.append(f"BinaryOp {s}_l 2 1 {u0} {v} {s} 0=0")
        self.ops.append(("add", (u0, v), s))
        y1 = conv(s, hdn, hdn, 1, 1, act=False, bias=False)
        y2 = conv(a, c, hdn, 1, 1, act=False, bias=False)
        cat = concat([y1, y2])
        bn = name("bn")
        params = [r.uniform(0.5, 1.5, (c,)).astype(np.float32), r.normal(0, 0.3, (c,)).astype(np.float32),
                  r.uniform(0.3, 2.0, (c,)).astype(np.float32), r.normal(0, 0.2, (c,)).astype(np.float32)]
        self.lines.append(f"BatchNorm {bn}_l 1 1 {cat} {bn} 0={c}")
        self.blobs.append(mf.floats_blob(*params))
        self.ops.append(("batchnorm", cat, bn, *params))
        lk = name("leaky")
        self.lines.append(f"LeakyRelu {lk}_l 1 1 {bn} {lk} 0=1.000000e-01")
        self.ops.append(("leakyrelu", bn, lk, np.float32(1.0e-01)))
        p3 = conv(lk, c, c, 1, 1)
        p3_down, p3_skip = split(p3, 2)
        x = conv(p3_down, c, 4 * width, 3, 2)                     # hw / 8
        # spatial pyramid pooling
        x = conv(x, 4 * width, 2 * width, 1, 1)
        parts = split(x, 4)
        pooled = [parts[0]]
        for part, kernel in zip(parts[1:], (5, 9, 13)):
            top = name("pool")
            self.lines.append(mf.pool_line(top + "_l", part, top, 0, kernel, 1, kernel // 2))
            self.ops.append(("maxpool", part, top, kernel))
            pooled.append(top)
        p4 = conv(concat(pooled), 8 * width, 4 * width, 1, 1)
        p4_neck, p4_head = split(p4, 2)
        # neck: upsample and join the earlier stage
        n1 = conv(p4_neck, 4 * width, 2 * width, 1, 1)
        up = name("up")
        self.lines.append(f"Interp {up}_l 1 1 {n1} {up} 0=1 1=2.000000e+00 2=2.000000e+00 ")
        self.ops.append(("interp", n1, up, 2.0, 2.0))
        n2 = conv(concat([up, p3_skip]), 4 * width, 2 * width, 1, 1)
        self.outputs = []
        for feat, cin, cells in ((n2, 2 * width, (hw // 4) ** 2), (p4_head, 4 * width, (hw // 8) ** 2)):
            h = conv(feat, cin, anchors * outputs, 1, 1, act=False)
            rs, tr = name("reshape"), name("out")
            self.lines.append(f"Reshape {rs}_l 1 1 {h} {rs} 0={cells} 1={outputs} 2={anchors}")
            self.ops.append(("reshape", h, rs, (anchors, outputs, cells)))
            self.lines.append(f"Transpose {tr}_l 1 1 {rs} {tr} 0=1,0,2")
            self.ops.append(("transpose", rs, tr))
            self.outputs.append(tr)
        self.output = self.outputs[0]

    def topology(self):
        return mf.topology(self.lines, "yolov5_shaped_int8" if self.int8 else "yolov5_shaped_f32")

    def write_model(self, path):
        mf.write_model(path, self.blobs)
