"""A MobileFaceNet-shaped float network as `.phai` topology text + `.racy` weights, built from a seed.

The layer mix of the recognition models the library ships with (Input normalisation, 3x3 stride-2 stem, depthwise
3x3 + pointwise 1x1 bottlenecks with PReLU, Eltwise residual sums over Split blobs, global average pooling, one
InnerProduct) at a size a CPU evaluates in a second. It exists to run one realistic multi-layer topology through the
loader and the per-layer executor in float32 and float16.
"""
import numpy as np

from . import modelfile as mf


class MobileFaceNetF32:
    def __init__(self, seed=7, hw=64, width=16, blocks=((2, 32, 2), (1, 32, 1), (1, 32, 1), (2, 64, 2), (1, 64, 1)), embed=32):
        r = np.random.default_rng(seed)
        self.hw = hw
        self.lines, self.blobs = [], []
        self.means, self.scale = (127.5, 127.5, 127.5), 0.0078125
        self.lines.append(f"Input data 0 1 data 0={hw} 1={hw} 2=3 3=" + ",".join(repr(m) for m in self.means) + f" 4={self.scale!r}")
        self.ops = [("input",)]
        cur, c = "data", 3

        def conv(name, bottom, top, cin, k, kernel, stride, pad, dw=False):
            groups = cin if dw else 1
            w = r.normal(0, np.sqrt(2.0 / (cin // groups * kernel * kernel)), (k, cin // groups, kernel, kernel)).astype(np.float32)
            b = r.normal(0, 0.05, (k,)).astype(np.float32)
            typ = "ConvolutionDepthWise" if dw else "Convolution"
            self.lines.append(mf.conv_line(typ, name, bottom, top, k, kernel, stride, pad, True, w.size, groups, act=0))
            self.blobs.append(mf.conv_blob_f32(w, b))
            self.ops.append(("dw" if dw else "conv", bottom, top, w, b, kernel, stride, pad, groups))

        def prelu(name, bottom, top, ch):
            s = np.abs(r.normal(0.1, 0.1, (ch,))).astype(np.float32)
            self.lines.append(f"PReLU {name} 1 1 {bottom} {top} 0={ch}")
            self.blobs.append(mf.floats_blob(s))
            self.ops.append(("prelu", bottom, top, s))

        conv("conv1", cur, "conv1", c, width, 3, 2, 1)
        prelu("relu1", "conv1", "conv1_r", width)
        conv("conv1_dw", "conv1_r", "conv1_dw", width, width, 3, 1, 1, dw=True)
        prelu("relu1_dw", "conv1_dw", "conv1_dw_r", width)
        cur, c = "conv1_dw_r", width
        for i, (stride, k, expand) in enumerate(blocks):
            p = f"b{i}"
            residual = stride == 1 and k == c
            src = cur
            if residual:
                self.lines.append(f"Split {p}_split 1 2 {cur} {p}_s0 {p}_s1")
                self.ops.append(("split", cur, (f"{p}_s0", f"{p}_s1")))
                src = f"{p}_s0"
            e = c * expand
            conv(f"{p}_ex", src, f"{p}_ex", c, e, 1, 1, 0)
            prelu(f"{p}_ex_r", f"{p}_ex", f"{p}_ex_r", e)
            conv(f"{p}_dw", f"{p}_ex_r", f"{p}_dw", e, e, 3, stride, 1, dw=True)
            prelu(f"{p}_dw_r", f"{p}_dw", f"{p}_dw_r", e)
            conv(f"{p}_pr", f"{p}_dw_r", f"{p}_pr", e, k, 1, 1, 0)
            cur = f"{p}_pr"
            if residual:
                self.lines.append(f"Eltwise {p}_sum 2 1 {p}_s1 {p}_pr {p}_out 0=1")
                self.ops.append(("sum", (f"{p}_s1", f"{p}_pr"), f"{p}_out"))
                cur = f"{p}_out"
            c = k
        conv("conv_last", cur, "conv_last", c, 2 * c, 1, 1, 0)
        prelu("relu_last", "conv_last", "conv_last_r", 2 * c)
        self.lines.append(mf.pool_line("gap", "conv_last_r", "gap", 1, global_pool=True))
        self.ops.append(("gap", "conv_last_r", "gap"))
        wfc = r.normal(0, 0.1, (embed, 2 * c)).astype(np.float32)
        bfc = r.normal(0, 0.05, (embed,)).astype(np.float32)
        self.lines.append(f"InnerProduct fc 1 1 gap out 0={embed} 1=1 2={wfc.size}")
        self.blobs.append(mf.fc_blob_f32(wfc, bfc))
        self.ops.append(("fc", "gap", "out", wfc, bfc))
        self.output = "out"

    def topology(self):
        return mf.topology(self.lines, "mobilefacenet_f32")

    def write_model(self, path):
        mf.write_model(path, self.blobs)


# The MobileNet-style fp16 configuration of the benchmark set: 3x3 stride-2 stem to 32 channels, depthwise 3x3 (stride 1 / 2)
# + pointwise 1x1 blocks of 64 ... 512 channels with residual sums where the shapes match, global average pooling; 224 x 224.
CFG3 = dict(hw=224, width=32, blocks=((2, 64, 2), (1, 64, 2), (2, 128, 2), (1, 128, 2), (2, 256, 2), (1, 256, 2),
                                      (1, 256, 2), (2, 512, 2), (1, 512, 2)), embed=128)
