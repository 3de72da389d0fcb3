"""Generators of the `.phai` topology text of four networks the library ships under models/: the YOLOv5s detector
(`yolov5s_simp.phai`), the ResNet-18 DBNet text detector (`det_db_resnet18.phai`), the MobileNet-style face network
(`mobile_unicorn.phai`) and the int8 residual face network (`unicorn_light_..._int8.phai`).

Each generator builds the network from its architecture (stages, blocks, widths) and numbers layers and blobs the way the
converter that wrote the shipped files did (ONNX node / tensor indices for the first two, Caffe layer names for the face
networks), so that at the shipped input size the text equals the shipped file token for token; a test compares them
where the reference tree is present. The input size is a parameter: a detector accepts any multiple of 32.

Format of a line (src/Excalibur/pipeline.cpp:49-116): Type name n_in n_out bottoms... tops... key=value...
"""


class _Graph:
    """Collects layers with logical blob names, then inserts Split layers for blobs with several readers."""

    def __init__(self, node=0, blob=0):
        self.node, self.blob = node, blob   # next ONNX node index / tensor index (unused by the Caffe-named networks)
        self.layers = []                    # [type, name, [bottoms], [tops], params]
        self.origin = {}                    # top -> Caffe layer that made it (names the Caffe-style Split)

    def add(self, kind, name, bottoms, top, params="", origin=None):
        self.layers.append([kind, name, list(bottoms), [top], params])
        if origin:
            self.origin[top] = origin
        return top

    def onnx(self, kind, prefix, bottoms, params="", node_skip=0, blob_skip=0, top=None):
        """A layer named <prefix>_<node index> writing tensor <blob index>; *_skip: indices the exporter spent on
        nodes / tensors that the converter folded into this layer."""
        self.node += node_skip
        self.blob += blob_skip
        name = f"{prefix}_{self.node}"
        top = str(self.blob) if top is None else top
        self.node += 1
        self.blob += 1
        return self.add(kind, name, bottoms, top, params)

    def lines(self, split_style):
        readers = {}
        for li, (_, _, bottoms, _, _) in enumerate(self.layers):
            for b in bottoms:
                readers.setdefault(b, []).append(li)
        out, n_split = [], 0
        renamed = {}  # (reader layer index, blob) -> split output
        for li, (kind, name, bottoms, tops, params) in enumerate(self.layers):
            bottoms = [renamed.pop((li, b), b) for b in bottoms]
            out.append(" ".join([kind, name, str(len(bottoms)), str(len(tops))] + bottoms + tops + ([params] if params else [])))
            for t in tops:
                rd = readers.get(t, [])
                if len(rd) < 2:
                    continue
                if split_style == "onnx":   # splitexcalibur_<i>; the last reader takes output 0
                    sname = f"splitexcalibur_{n_split}"
                    outs = [f"{t}_splitexcalibur_{j}" for j in range(len(rd))]
                    for j, r in enumerate(reversed(rd)):
                        renamed[(r, t)] = outs[j]
                else:                       # Caffe's insert_splits: <blob>_<layer>_0_split; the first reader takes output 0
                    sname = f"{t}_{self.origin.get(t, t)}_0_split"
                    outs = [f"{sname}_{j}" for j in range(len(rd))]
                    for j, r in enumerate(rd):
                        renamed[(r, t)] = outs[j]
                n_split += 1
                out.append(" ".join(["Split", sname, "1", str(len(outs)), t] + outs))
        return out


def _text(header, counts, lines):
    return "\n".join([header, counts] + lines) + "\n"


def _conv_onnx(k, kernel, stride, pad, bias, cin):
    return (f"0={k} 1={kernel} 11={kernel} 2=1 12=1 3={stride} 13={stride} 4={pad} 14={pad} 15={pad} 16={pad} "
            f"5={int(bias)} 6={k * cin * kernel * kernel}")


# ----------------------------------------------------------------------------------------------- YOLOv5s
def yolov5s_simp(size=640, classes=80, anchors=3, int8=False):
    """YOLOv5s (Focus, cross-stage-partial blocks of depth 1 / 3 / 3 / 1 with HardSwish, spatial pyramid pooling 5 / 9 / 13,
    a feature pyramid with two nearest upsamplings and a path aggregation back down, three heads of
    anchors * (classes + 5) channels at strides 8 / 16 / 32, each reshaped to [anchors][outputs][cells] and transposed). int8: every
    convolution carries key 8=2 (int8 weights, quantized input), the detector's int8 configuration; not a shipped file."""
    assert size % 32 == 0
    g = _Graph(node=41, blob=208)
    outputs = classes + 5

    def conv(x, cin, k, kernel=1, stride=1, act=True, bias=True):
        y = g.onnx("Convolution", "Conv", [x], _conv_onnx(k, kernel, stride, kernel // 2, bias, cin) + (" 8=2" if int8 else ""))
        if act:  # x * clamp(x / 6 + 0.5, 0, 1): eight exporter nodes, the last one a Div
            y = g.onnx("HardSwish", "Div", [y], "0=1.666667e-01 1=5.000000e-01", node_skip=7, blob_skip=7)
        return y

    def csp(x, cin, cout, depth, shortcut=True):
        hidden = cout // 2
        y = conv(x, cin, hidden)
        for _ in range(depth):
            z = conv(conv(y, hidden, hidden), hidden, hidden, 3)
            y = g.onnx("BinaryOp", "Add", [y, z], "0=0") if shortcut else z
        y1 = conv(y, hidden, hidden, act=False, bias=False)
        y2 = conv(x, cin, hidden, act=False, bias=False)
        cat = g.onnx("Concat", "Concat", [y1, y2], "0=-1")
        bn = g.onnx("BatchNorm", "BatchNormalization", [cat], f"0={2 * hidden}")
        act = g.onnx("LeakyRelu", "LeakyRelu", [bn], "0=1.000000e-01")
        return conv(act, 2 * hidden, cout)

    def upsample(x):
        return g.onnx("Interp", "Resize", [x], "0=1 1=2.000000e+00 2=2.000000e+00", node_skip=1, blob_skip=4)

    g.add("Input", "images", [], "images", f"0={size} 1={size} 2=3 3=0,0,0 4=0.0039215")
    x = g.add("YoloV5Focus", "focus", ["images"], "207")
    x = conv(x, 12, 32, 3)
    x = csp(conv(x, 32, 64, 3, 2), 64, 64, 1)
    p3 = csp(conv(x, 64, 128, 3, 2), 128, 128, 3)
    p4 = csp(conv(p3, 128, 256, 3, 2), 256, 256, 3)
    x = conv(conv(p4, 256, 512, 3, 2), 512, 256)
    pools = [g.onnx("Pooling", "MaxPool", [x], f"0=0 1={k} 11={k} 2=1 12=1 3={k // 2} 13={k // 2} 14={k // 2} 15={k // 2} 5=1 4=0")
             for k in (5, 9, 13)]
    x = conv(g.onnx("Concat", "Concat", [x] + pools, "0=-1"), 1024, 512)
    x = csp(x, 512, 512, 1, shortcut=False)
    top5 = conv(x, 512, 256)
    x = csp(g.onnx("Concat", "Concat", [upsample(top5), p4], "0=-1"), 512, 256, 1, shortcut=False)
    top4 = conv(x, 256, 128)
    head3 = csp(g.onnx("Concat", "Concat", [upsample(top4), p3], "0=-1"), 256, 128, 1, shortcut=False)
    x = g.onnx("Concat", "Concat", [conv(head3, 128, 128, 3, 2), top4], "0=-1")
    head4 = csp(x, 256, 256, 1, shortcut=False)
    x = g.onnx("Concat", "Concat", [conv(head4, 256, 256, 3, 2), top5], "0=-1")
    head5 = csp(x, 512, 512, 1, shortcut=False)
    outs = []
    for i, (feat, cin, stride) in enumerate(((head3, 128, 8), (head4, 256, 16), (head5, 512, 32))):
        if i:  # the exporter's box decoding of the previous head, dropped by the converter
            g.node += 281
            g.blob += 289
        h = conv(feat, cin, anchors * outputs, act=False)
        r = g.onnx("Reshape", "Reshape", [h], f"0={(size // stride) ** 2} 1={outputs} 2={anchors}", node_skip=13, blob_skip=17)
        outs.append(g.onnx("Transpose", "Transpose", [r], "0=1,0,2"))
    return _text("glsv1", "286 319", g.lines("onnx")), outs


# ----------------------------------------------------------------------------------------------- DBNet on ResNet-18
def det_db_resnet18(size=800):
    """ResNet-18 (three 3x3 stem convolutions, max pooling, four stages of two basic blocks; a stage's first block
    downsamples its shortcut with a 2x2 average pooling and a 1x1 convolution), a feature pyramid (1x1 laterals to 256
    channels, nearest upsampling and sums, 3x3 smoothing to 64 channels, upsampling to stride 4, Concat) and the
    binarisation head (3x3 convolution, two 2x2 stride-2 transposed convolutions, Sigmoid)."""
    assert size % 32 == 0
    g = _Graph(node=0, blob=77)

    def conv(x, cin, k, kernel=3, stride=1, bias=True, relu=False):
        y = g.onnx("Convolution", "Conv", [x], _conv_onnx(k, kernel, stride, kernel // 2, bias, cin))
        return g.onnx("ReLU", "Relu", [y]) if relu else y

    def block(x, cin, k, stride):
        y = conv(conv(x, cin, k, 3, stride, relu=True), k, k)
        if stride != 1:    # the exporter pads, then pools: one node and one tensor more
            s = g.onnx("Pooling", "AveragePool", [x], "0=1 1=2 11=2 2=2 12=2 3=0 13=0 14=1 15=1 5=1 4=0", node_skip=1, blob_skip=1)
            s = conv(s, cin, k, 1)
        elif cin != k or x == pooled:
            s = conv(x, cin, k, 1)
        else:
            s = x
        operands = [y, s]
        return g.onnx("ReLU", "Relu", [g.onnx("BinaryOp", "Add", operands, "0=0")])

    def upsample(x, factor):
        return g.onnx("Interp", "Upsample", [x], f"0=1 1={factor:e} 2={factor:e}", blob_skip=3)

    g.add("Input", "input", [], "input", f"0={size} 1={size} 2=3 3=123.675,116.28,103.53 4=0.0171247,0.017507,0.0174292")
    x = conv(conv(conv("input", 3, 32, 3, 2, relu=True), 32, 32, relu=True), 32, 64, relu=True)
    pooled = g.onnx("Pooling", "MaxPool", [x], "0=0 1=3 11=3 2=2 12=2 3=1 13=1 14=1 15=1 5=1 4=0")
    c2 = block(block(pooled, 64, 64, 1), 64, 64, 1)
    c3 = block(block(c2, 64, 128, 2), 128, 128, 1)
    c4 = block(block(c3, 128, 256, 2), 256, 256, 1)
    c5 = block(block(c4, 256, 512, 2), 512, 512, 1)
    in5, in4, in3, in2 = (conv(c, cin, 256, 1, bias=False) for c, cin in ((c5, 512), (c4, 256), (c3, 128), (c2, 64)))
    out4 = g.onnx("BinaryOp", "Add", [upsample(in5, 2.0), in4], "0=0")
    out3 = g.onnx("BinaryOp", "Add", [upsample(out4, 2.0), in3], "0=0")
    out2 = g.onnx("BinaryOp", "Add", [upsample(out3, 2.0), in2], "0=0")
    p5, p4, p3, p2 = (conv(f, 256, 64, bias=False) for f in (in5, out4, out3, out2))
    u3, u4, u5 = upsample(p3, 2.0), upsample(p4, 4.0), upsample(p5, 8.0)
    fuse = g.onnx("Concat", "Concat", [u5, u4, u3, p2], "0=-1")
    x = conv(fuse, 256, 64, relu=True)
    deconv = "0={k} 1=2 11=2 2=1 12=1 3=2 13=2 4=0 14=0 15=0 16=0 5=1 6={count} 7=1"
    x = g.onnx("Deconvolution", "ConvTranspose", [x], deconv.format(k=64, count=64 * 64 * 4))
    x = g.onnx("ReLU", "Relu", [g.onnx("BatchNorm", "BatchNormalization", [x], "0=64")])
    x = g.onnx("Deconvolution", "ConvTranspose", [x], deconv.format(k=1, count=64 * 4))
    g.onnx("Sigmoid", "Sigmoid", [x], top="output")
    return _text("glsv1", "91 105", g.lines("onnx")), ["output"]


# ----------------------------------------------------------------------------------------------- face networks (Caffe names)
def _conv_caffe(k, kernel, stride, pad, cin, groups=1, int8=0):
    s = f"0={k} 1={kernel} 2=1 3={stride} 4={pad} 5=1 6={k * (cin // groups) * kernel * kernel}"
    if groups != 1:
        s += f" 7={groups}"
    if int8:
        s += f" 8={int8}"
    return s


def mobile_unicorn(size=128):
    """MobileNet-v2-style face network: a 3x3 stride-2 stem, inverted residual units (1x1 expansion, PReLU, 3x3 depthwise,
    PReLU, linear 1x1 projection, Eltwise sum) in stages of 4 / 6 / 2 units behind stride-2 transition units, a global
    8x8 depthwise convolution and a 128-way InnerProduct without bias. The input size is fixed by the last two layers."""
    g = _Graph()

    def unit(x, cin, name, expand, cout, stride, merged_scale=False):
        def cp(x, lname, rname, kind, params):
            y = g.add(kind, lname, [x], lname, params)
            return g.add("PReLU", rname, [y], f"{lname}_{rname}", f"0={params.split()[0][2:]}")
        y = cp(x, f"conv{name}_ex", f"relu{name}_ex", "Convolution", _conv_caffe(expand, 1, 1, 0, cin))
        y = cp(y, f"conv{name}_dw", f"relu{name}_dw", "ConvolutionDepthWise", _conv_caffe(expand, 3, stride, 1, expand, expand))
        lname = f"conv{name}_em"
        return g.add("Convolution", lname, [y], lname, _conv_caffe(cout, 1, 1, 0, expand), origin=f"{lname}/scale" if merged_scale else None)

    g.add("Input", "data", [], "data", f"0={size} 1={size} 2=3 3=123.0,117.0,104.0 4=0.0078125")
    x = g.add("Convolution", "conv1", ["data"], "conv1", _conv_caffe(64, 3, 2, 1, 3))
    x = g.add("PReLU", "relu1", [x], "conv1_relu1", "0=64")
    x = g.add("ConvolutionDepthWise", "conv1_dw", [x], "conv1_dw", _conv_caffe(64, 3, 1, 1, 64, 64))
    x = g.add("PReLU", "relu1_dw", [x], "conv1_dw_relu1_dw", "0=64")
    cin = 64
    for stage, (expand, cout, units, unit_expand) in zip((2, 3, 4), ((128, 64, 4, 128), (256, 128, 6, 256), (512, 128, 2, 256))):
        x = unit(x, cin, str(stage), expand, cout, 2, merged_scale=True)
        for i in range(1, units + 1):
            y = unit(x, cout, f"{stage}_{i}", unit_expand, cout, 1)
            res = f"res{stage}_{i}"
            x = g.add("Eltwise", res, [x, y], res, "0=1 -23301=0", origin=res)
        cin = cout
    x = g.add("Convolution", "conv5_ex", [x], "conv5_ex", _conv_caffe(512, 1, 1, 0, 128))
    x = g.add("PReLU", "relu5_ex", [x], "conv5_ex_relu5_ex", "0=512")
    x = g.add("ConvolutionDepthWise", "conv5_dw", [x], "conv5_dw", _conv_caffe(512, 8, 1, 0, 512, 512))
    g.add("InnerProduct", "fc5", [x], "fc5", f"0=128 1=0 2={128 * 512}")
    return _text("glsv1 Unicorn_Mobile_Net", "108 121", g.lines("caffe")), ["fc5"]


def unicorn_light_int8(size=128):
    """Residual face network with int8 convolutions (key 8=2): per stage an unpadded 3x3 convolution that widens, a 2x2 max
    pooling, then residual pairs of padded 3x3 convolutions with ReLU (1 / 2 / 5 / 3 pairs) summed with their input by
    Eltwise; a last unpadded convolution and a global 4x4 depthwise convolution with int8 weights (8=1)."""
    g = _Graph()

    def conv(x, name, relu, cin, k, pad):
        y = g.add("Convolution", name, [x], name, _conv_caffe(k, 3, 1, pad, cin, int8=2))
        return g.add("ReLU", relu, [y], f"{name}_{relu}")

    g.add("Input", "data", [], "data", f"0={size} 1={size} 2=3 3=104,117,123 4=0.0078125")
    x = conv("data", "conv1a", "relu1a", 3, 16, 0)
    x = conv(x, "conv1b", "relu1b", 16, 32, 0)
    width = 32
    for stage, pairs in ((1, 1), (2, 2), (3, 5), (4, 3)):
        pool = "pool1b" if stage == 1 else f"pool{stage}"
        x = g.add("Pooling", pool, [x], pool, "0=0 1=2 2=2 3=0 4=0")
        for i in range(1, pairs + 1):
            a, b = f"{stage + 1}_{2 * i - 1}", f"{stage + 1}_{2 * i}"
            y = conv(conv(x, f"conv{a}", f"relu{a}", width, width, 1), f"conv{b}", f"relu{b}", width, width, 1)
            x = g.add("Eltwise", f"res{b}", [x, y], f"res{b}", "0=1 -23301=0")
        name = f"conv{stage + 1}"
        wider = min(2 * width, 256)
        x = conv(x, name, f"relu{stage + 1}", width, wider, 0)
        width = wider
    g.add("ConvolutionDepthWise", "conv5_dw", [x], "conv5_dw", _conv_caffe(256, 4, 1, 0, 256, 256, int8=1))
    return _text("glsv1 unicorn_light_int8", "84 96", g.lines("onnx")), ["conv5_dw"]


SHIPPED = {
    "yolov5s_simp.phai": yolov5s_simp,
    "det_db_resnet18.phai": det_db_resnet18,
    "mobile_unicorn.phai": mobile_unicorn,
    "unicorn_light_806204_m1x3x2+120k_universial_noised_usefulpart_int8.phai": unicorn_light_int8,
}


def algorithmic_gop(text, input_chw):
    """2 x multiply-accumulates of the Convolution / ConvolutionDepthWise / Deconvolution / InnerProduct layers of a
    topology for one image of shape (c, h, w), in GOP: 2 * OH * OW * K * (C / groups) * kh * kw per convolution
    (src/Excalibur/operation_convolution.cpp:270-271 for the output size), 2 * K * C * H * W per InnerProduct. Shapes
    follow the layers' parameters; layers that keep their input's shape need no entry here."""
    shapes = {}
    gop = 0.0
    for line in text.splitlines()[2:]:
        t = line.split()
        if not t:
            continue
        typ, nb, nt = t[0], int(t[2]), int(t[3])
        bots, tops = t[4:4 + nb], t[4 + nb:4 + nb + nt]
        kv = dict(x.split("=", 1) for x in t[4 + nb + nt:] if "=" in x)
        geti = lambda k, d=0: int(float(kv.get(str(k), d)))
        if typ == "Input":
            shapes[tops[0]] = tuple(input_chw)
            continue
        if not bots or bots[0] not in shapes:
            for tp in tops:
                shapes[tp] = tuple(input_chw)   # a topology that starts at its first layer
            if typ not in ("Convolution", "ConvolutionDepthWise", "InnerProduct"):
                continue
            shapes.setdefault(bots[0] if bots else tops[0], tuple(input_chw))
        c, h, w = shapes[bots[0]]
        if typ in ("Convolution", "ConvolutionDepthWise"):
            k, kw, kh = geti(0), geti(1), geti(11, geti(1))
            sw, sh = geti(3, 1), geti(13, geti(3, 1))
            pl = geti(4)
            pr, pt, pb = geti(15, pl), geti(14, pl), geti(16, pl)
            groups = max(1, geti(7, 1))
            oh, ow = (h + pt + pb - kh) // sh + 1, (w + pl + pr - kw) // sw + 1
            gop += 2.0 * oh * ow * k * (c // groups) * kh * kw / 1e9
            shapes[tops[0]] = (k, oh, ow)
        elif typ == "InnerProduct":
            k = geti(0)
            gop += 2.0 * k * c * h * w / 1e9
            shapes[tops[0]] = (k, 1, 1)
        elif typ == "Pooling":
            if geti(4):
                shapes[tops[0]] = (c, 1, 1)
            else:
                kw, kh = geti(1), geti(11, geti(1))
                sw, sh = geti(2, 1), geti(12, geti(2, 1))
                pl = geti(3)
                pr, pt, pb = geti(14, pl), geti(13, pl), geti(15, pl)
                ceil_mode = geti(5, 1) == 0
                def size(n, k_, s_, a, b):
                    v = n + a + b - k_
                    return (-(-v // s_) if ceil_mode else v // s_) + 1
                shapes[tops[0]] = (c, size(h, kh, sh, pt, pb), size(w, kw, sw, pl, pr))
        elif typ == "YoloV5Focus":
            shapes[tops[0]] = (4 * c, h // 2, w // 2)
        elif typ == "Interp":
            ws_, hs_ = float(kv.get("1", 1.0)), float(kv.get("2", 1.0))
            ow, oh = geti(3), geti(4)
            shapes[tops[0]] = (c, oh if oh > 0 else int(h * hs_), ow if ow > 0 else int(w * ws_))
        elif typ == "Concat":
            shapes[tops[0]] = (sum(shapes[b][0] for b in bots), h, w)
        else:   # Split, activations, BatchNorm, Eltwise, BinaryOp, Reshape, Transpose ...: the input's shape (no MACs behind them)
            for tp in tops:
                shapes[tp] = (c, h, w)
    return gop
