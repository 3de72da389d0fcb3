"""Seeded single-layer cases shared by the fixture generator, the oracle tests and the GPU parity tests.

A case is a dict of plain numpy arrays and ints: the op kind, its hyper-parameters in the reference's
terms and its inputs. `reference_io(case)` turns it into the topology text and weight blob the
reference reads, `oracle_eval(case)` evaluates it with the CPU restatement.
"""
import numpy as np

from excalibur_amd import modelfile as mf
from oracle import port


def _rng(seed):
    return np.random.default_rng(seed)


def conv_f32_case(seed, n, c, h, w, k, kernel, stride=1, pad=0, act=1, groups=1, bias=True, dw=False):
    r = _rng(seed)
    kh, kw = (kernel, kernel) if np.isscalar(kernel) else kernel
    return dict(op="dw_f32" if dw else "conv_f32", n=n, c=c, h=h, w=w, k=k, kh=kh, kw=kw, stride=stride, pad=pad,
                act=act, groups=groups,
                x=r.uniform(-1, 1, (n, c, h, w)).astype(np.float32),
                wt=r.normal(0, 0.05, (k, c // groups, kh, kw)).astype(np.float32),
                bias=r.normal(0, 0.01, (k,)).astype(np.float32) if bias else None)


def conv_i8_case(seed, n, c, h, w, k, kernel, stride=1, pad=0, act=1, bias=True, integer_x=False, groups=1, out_scale=1.0):
    r = _rng(seed)
    kh, kw = (kernel, kernel) if np.isscalar(kernel) else kernel
    if integer_x:
        x = r.integers(-127, 128, (n, c, h, w)).astype(np.float32)
        fs = np.float32(1.0)
    else:
        x = r.uniform(-3, 3, (n, c, h, w)).astype(np.float32)
        fs = np.float32(127.0 / np.abs(x).max() * 1.1)  # a few values saturate
    wt = r.integers(-127, 128, (k, c // groups, kh, kw)).astype(np.int8)
    s = (r.uniform(1e-4, 1e-2, (k,)) * out_scale).astype(np.float32)  # wanted dequant scale (out_scale < 1: outputs of a few units, where sigmoid / mish bend)
    ws = (np.float32(1.0) / (s * fs)).astype(np.float32)     # stored weight scale
    ws[0] = np.float32(5e-7)                                  # |ws| <= 1e-6 -> scale forced to 0
    return dict(op="conv_i8", n=n, c=c, h=h, w=w, k=k, kh=kh, kw=kw, stride=stride, pad=pad, act=act, groups=groups,
                x=x, wt=wt, ws=ws, fs=fs,
                bias=(r.integers(-2 ** 15, 2 ** 15, (k,)).astype(np.float32) * s).astype(np.float32) if bias else None)


def dw_i8_case(seed, n, c, h, w, stride, pad=1, act=1):
    r = _rng(seed)
    ws = r.uniform(20, 200, (c,)).astype(np.float32)
    ws[1] = np.float32(-3.0)  # negative scale -> weights become 0 (no fabs in the reference)
    return dict(op="dw_i8", n=n, c=c, h=h, w=w, k=c, kh=3, kw=3, stride=stride, pad=pad, act=act, groups=c,
                x=r.uniform(-1, 1, (n, c, h, w)).astype(np.float32),
                wt=r.integers(-127, 128, (c, 1, 3, 3)).astype(np.int8), ws=ws, fs=np.float32(1.0),
                bias=r.normal(0, 0.01, (c,)).astype(np.float32))


def pool_case(seed, n, c, h, w, ptype, kernel=0, stride=1, pad=0, global_pool=False, pad_mode=1, count_include_pad=0):
    r = _rng(seed)
    return dict(op="pool", n=n, c=c, h=h, w=w, ptype=ptype, kernel=kernel, stride=stride, pad=pad,
                global_pool=global_pool, pad_mode=pad_mode, count_include_pad=count_include_pad,
                x=r.uniform(-1, 1, (n, c, h, w)).astype(np.float32))


def eltwise_case(seed, shape, etype, n_inputs=2, coeffs=None):
    r = _rng(seed)
    return dict(op="eltwise", etype=etype, coeffs=coeffs,
                xs=[r.uniform(-2, 2, shape).astype(np.float32) for _ in range(n_inputs)])


def binaryop_case(seed, shape):
    r = _rng(seed)
    return dict(op="binaryop_add", xs=[r.uniform(-2, 2, shape).astype(np.float32) for _ in range(2)])


def relu_case(seed, shape):
    return dict(op="relu", x=_rng(seed).uniform(-2, 2, shape).astype(np.float32))


def fc_case(seed, m, c, h, w, n_out, bias=True):
    r = _rng(seed)
    return dict(op="fc", n_out=n_out, x=r.uniform(-1, 1, (m, c, h, w)).astype(np.float32),
                wt=r.normal(0, 0.05, (n_out, c * h * w)).astype(np.float32),
                bias=r.normal(0, 0.01, (n_out,)).astype(np.float32) if bias else None)


def unary_case(seed, kind, shape, **params):
    """kind: hardswish / leakyrelu / sigmoid / hardsigmoid / focus / interp (params: the layer's keys)."""
    return dict(op=kind, x=_rng(seed).uniform(-4, 4, shape).astype(np.float32), **params)


def binaryop_bc_case(seed, shape, op_type, small, swap=False):
    """BinaryOp (0 ADD, 1 SUB, 2 MUL, 3 DIV) of a tensor with a smaller operand derived from it inside the topology, the
    way the shipped networks do (squeeze-and-excite gates): `small` = "equal" (the tensor clipped to [0.5, 3]), "channel"
    (global average, [n][c][1][1]), "pixel" (a 1x1 convolution to one channel, [n][1][h][w]) or "image" (the global
    average of that, [n][1][1][1]). swap: the smaller operand is written first in the layer line."""
    r = _rng(seed)
    x = r.uniform(0.5, 2.0, shape).astype(np.float32) * r.choice([-1.0, 1.0], shape).astype(np.float32)
    w = r.uniform(0.2, 1.0, (1, shape[1], 1, 1)).astype(np.float32)
    return dict(op="binaryop_bc", x=x, op_type=op_type, small=small, swap=swap, wt=w)


def binaryop_bc_small(case):
    """The smaller operand, evaluated by the oracle restatement."""
    x = case["x"]
    if case["small"] == "equal":
        return port.clip(x, 0.5, 3.0)
    if case["small"] == "channel":
        return port.pool2d(x, port.POOL_AVE, global_pool=True)
    plane = port.conv2d_f32(x, case["wt"], None, 0, port.geom(x.shape, 1, 1))
    return plane if case["small"] == "pixel" else port.pool2d(plane, port.POOL_AVE, global_pool=True)


def reshape_shape(case):
    """The layer's shape rule (src/Excalibur/operation_reshape.cpp:49-86): given dimensions replace the old ones, absent
    ones (or negative ones) follow from the element count, channels first, then height, then width."""
    shape = list(case["x"].shape)
    given = [None, case.get("new_c"), case.get("new_h"), case.get("new_w")]
    for axis in (1, 2, 3):
        if given[axis] is not None and given[axis] > 0:
            shape[axis] = given[axis]
    for axis in (1, 2, 3):
        if given[axis] is None or given[axis] < 0:
            others = int(np.prod([shape[i] for i in range(4) if i != axis]))
            shape[axis] = case["x"].size // others
    return tuple(shape)


def prelu_case(seed, shape, shared=False):
    r = _rng(seed)
    return dict(op="prelu", x=r.uniform(-2, 2, shape).astype(np.float32),
                slope=np.abs(r.normal(0, 0.3, (1 if shared else shape[1],))).astype(np.float32))


def batchnorm_case(seed, shape, eps=1e-5):
    r = _rng(seed)
    c = shape[1]
    return dict(op="batchnorm", x=r.uniform(-2, 2, shape).astype(np.float32), eps=eps,
                slope=r.uniform(0.5, 1.5, (c,)).astype(np.float32), mean=r.normal(0, 0.5, (c,)).astype(np.float32),
                var=r.uniform(0.2, 2.0, (c,)).astype(np.float32), bias=r.normal(0, 0.3, (c,)).astype(np.float32))


def input_case(seed, shape, means, scales):
    return dict(op="input", x=_rng(seed).uniform(0, 255, shape).astype(np.float32), means=list(means), scales=list(scales))


def concat_case(seed, n, channels, h, w):
    r = _rng(seed)
    return dict(op="concat", xs=[r.uniform(-2, 2, (n, c, h, w)).astype(np.float32) for c in channels])


def deconv_case(seed, n, c, h, w, k, kernel, stride, pad=0, bias=True):
    r = _rng(seed)
    return dict(op="deconv", k=k, kernel=kernel, stride=stride, pad=pad, x=r.uniform(-1, 1, (n, c, h, w)).astype(np.float32),
                wt=r.normal(0, 0.1, (c, k, kernel, kernel)).astype(np.float32),
                bias=r.normal(0, 0.1, (k,)).astype(np.float32) if bias else None)


def geom_of(case):
    return port.geom((case["n"], case["c"], case["h"], case["w"]), case["k"], case["kh"], case["kw"],
                     case["stride"], case["pad"], case["groups"])


def reference_io(case):
    """-> (topology text, weight blob bytes or b'', [input arrays], output blob name)."""
    op = case["op"]
    if op in ("conv_f32", "dw_f32", "conv_i8", "dw_i8"):
        typ = "ConvolutionDepthWise" if op.startswith("dw") else "Convolution"
        line = mf.conv_line(typ, "layer", "data", "out", case["k"], (case["kh"], case["kw"]), case["stride"],
                            case["pad"], case["bias"] is not None, case["wt"].size, case["groups"],
                            int8=op.endswith("i8"), act=case["act"])
        if op.endswith("i8"):
            blob = mf.conv_blob_i8(case["wt"], case["bias"], case["ws"], case["fs"])
        else:
            blob = mf.conv_blob_f32(case["wt"], case["bias"])
        return mf.topology([line]), blob, [case["x"]], "out"
    if op == "pool":
        line = mf.pool_line("layer", "data", "out", case["ptype"], case["kernel"], case["stride"], case["pad"],
                            case["global_pool"], case["pad_mode"], case["count_include_pad"])
        return mf.topology([line]), b"", [case["x"]], "out"
    if op == "relu":
        return mf.topology(["ReLU layer 1 1 data out"]), b"", [case["x"]], "out"
    if op == "fc":
        line = f"InnerProduct layer 1 1 data out 0={case['n_out']} 1={int(case['bias'] is not None)} 2={case['wt'].size}"
        return mf.topology([line]), mf.fc_blob_f32(case["wt"], case["bias"]), [case["x"]], "out"
    if op == "deconv":
        line = mf.conv_line("Deconvolution", "layer", "data", "out", case["k"], case["kernel"], case["stride"], case["pad"],
                            case["bias"] is not None, case["wt"].size, 1)
        return mf.topology([line]), mf.conv_blob_f32(case["wt"], case["bias"]), [case["x"]], "out"
    if op == "hardswish":
        return mf.topology([f"HardSwish layer 1 1 data out 0={case['alpha']!r} 1={case['beta']!r}"]), b"", [case["x"]], "out"
    if op == "leakyrelu":
        return mf.topology([f"LeakyRelu layer 1 1 data out 0={case['alpha']!r}"]), b"", [case["x"]], "out"
    if op == "sigmoid":
        return mf.topology(["Sigmoid layer 1 1 data out"]), b"", [case["x"]], "out"
    if op == "hardsigmoid":
        return mf.topology([f"HardSigmoid layer 1 1 data out 0={case['alpha']!r} 1={case['beta']!r}"]), b"", [case["x"]], "out"
    if op == "focus":
        return mf.topology(["Yolov5focus layer 1 1 data out"]), b"", [case["x"]], "out"
    if op == "interp":
        # key 1 is read into the width scale and key 2 into the height scale (src/Excalibur/operation_interp.cpp:196-201)
        return mf.topology([f"Interp layer 1 1 data out 0=1 1={case['width_scale']!r} 2={case['height_scale']!r}"]), b"", [case["x"]], "out"
    if op == "binaryop_bc":
        lines, blob = ["Split s 1 2 data a b"], b""
        if case["small"] == "equal":
            lines.append("Clip k 1 1 b small 0=0.5 1=3.0")
        elif case["small"] == "channel":
            lines.append(mf.pool_line("gap", "b", "small", 1, global_pool=True))
        else:
            lines.append(mf.conv_line("Convolution", "c1", "b", "plane" if case["small"] == "image" else "small", 1, 1, 1, 0, False,
                                      case["wt"].size, 1, act=0))
            blob = mf.conv_blob_f32(case["wt"], None)
            if case["small"] == "image":
                lines.append(mf.pool_line("gap", "plane", "small", 1, global_pool=True))
        operands = "small a" if case["swap"] else "a small"
        lines.append(f"BinaryOp e 2 1 {operands} out 0={case['op_type']}")
        return mf.topology(lines), blob, [case["x"]], "out"
    if op == "clip":
        return mf.topology([f"Clip layer 1 1 data out 0={case['lo']!r} 1={case['hi']!r}"]), b"", [case["x"]], "out"
    if op == "softmax":
        return mf.topology(["Softmax layer 1 1 data out 0=0"]), b"", [case["x"]], "out"
    if op == "transpose":
        return mf.topology(["Transpose layer 1 1 data out 0=" + ",".join(str(v) for v in case["order"])]), b"", [case["x"]], "out"
    if op == "reshape":
        keys = " ".join(f"{k}={case[name]}" for k, name in ((0, "new_w"), (1, "new_h"), (2, "new_c")) if case.get(name) is not None)
        return mf.topology([f"Reshape layer 1 1 data out {keys}"]), b"", [case["x"]], "out"
    if op == "flatten":
        return mf.topology([f"Flatten layer 1 1 data out 0={case['axis']}"]), b"", [case["x"]], "out"
    if op == "prelu":
        return mf.topology([f"PReLU layer 1 1 data out 0={case['slope'].size}"]), mf.floats_blob(case["slope"]), [case["x"]], "out"
    if op == "batchnorm":
        line = f"BatchNorm layer 1 1 data out 0={case['x'].shape[1]} 1={case['eps']!r}"
        return mf.topology([line]), mf.floats_blob(case["slope"], case["mean"], case["var"], case["bias"]), [case["x"]], "out"
    if op == "input":
        c_, h_, w_ = case["x"].shape[1:]
        line = (f"Input layer 1 1 data out 0={w_} 1={h_} 2={c_} 3=" + ",".join(repr(float(v)) for v in case["means"]) +
                " 4=" + ",".join(repr(float(v)) for v in case["scales"]))
        return mf.topology([line]), b"", [case["x"]], "out"
    raise ValueError(op)


def multi_input_topology(case):
    """Eltwise / BinaryOp take several producers but the reference feeds only one pipeline input
    (src/Excalibur/pipeline.cpp:242): the operands are channel slices of one input tensor, cut by a
    Split_Slice layer (src/Excalibur/operation_split_slice.cpp:12-36, axis key 1=0 is the channel axis).
    -> (topology text, the concatenated input)."""
    n = len(case["xs"])
    names = " ".join(f"x{i}" for i in range(n))
    lines = [f"Split_Slice cut 1 {n} data {names} 0={n}," + ",".join(str(a.shape[1]) for a in case["xs"]) + " 1=0"]
    if case["op"] == "concat":
        lines.append(f"Concat layer {n} 1 {names} out 0=-1")
    elif case["op"] == "eltwise":
        extra = f"0={case['etype']}"
        if case.get("coeffs") is not None:
            extra += " -23301=" + ",".join([str(n + 1)] + [repr(float(v)) for v in case["coeffs"]])
        lines.append(f"Eltwise layer {n} 1 {names} out {extra}")
    else:
        lines.append(f"BinaryOp layer 2 1 {names} out 0=0")
    return mf.topology(lines), np.concatenate(case["xs"], axis=1)


def oracle_eval(case):
    op = case["op"]
    if op == "conv_f32":
        return port.conv2d_f32(case["x"], case["wt"], case["bias"], case["act"], geom_of(case))
    if op == "dw_f32":
        return port.dwconv_f32(case["x"], case["wt"], case["bias"], case["act"], geom_of(case))
    if op == "dw_i8":
        wf = port.dw_dequant_weights(case["wt"], case["ws"])
        return port.dwconv_f32(case["x"], wf, case["bias"], case["act"], geom_of(case))
    if op == "conv_i8":
        return port.conv2d_i8(case["x"], case["wt"], case["bias"], case["ws"], case["fs"], case["act"], geom_of(case))
    if op == "pool":
        return port.pool2d(case["x"], case["ptype"], case["kernel"], case["stride"], case["pad"], case["global_pool"],
                           case["pad_mode"], case["count_include_pad"])
    if op == "eltwise":
        return port.eltwise(case["xs"], case["etype"], case.get("coeffs"))
    if op == "binaryop_add":
        return port.binaryop_add(*case["xs"])
    if op == "relu":
        return port.relu(case["x"])
    if op == "fc":
        return port.innerproduct(case["x"], case["wt"], case["bias"])
    if op == "deconv":
        return port.deconv2d_f32(case["x"], case["wt"], case["bias"], case["stride"], case["pad"])
    if op == "hardswish":
        return port.hardswish(case["x"], case["alpha"], case["beta"])
    if op == "leakyrelu":
        return port.leakyrelu(case["x"], case["alpha"])
    if op == "sigmoid":
        return port.sigmoid(case["x"])
    if op == "hardsigmoid":
        return port.hardsigmoid(case["x"], case["alpha"], case["beta"])
    if op == "focus":
        return port.focus(case["x"])
    if op == "interp":
        return port.interp_nearest(case["x"], case["height_scale"], case["width_scale"])
    if op == "binaryop_bc":
        small = binaryop_bc_small(case)
        return port.binaryop(small, case["x"], case["op_type"]) if case["swap"] else port.binaryop(case["x"], small, case["op_type"])
    if op == "clip":
        return port.clip(case["x"], case["lo"], case["hi"])
    if op == "softmax":
        return port.softmax_channels(case["x"])
    if op == "transpose":
        return port.transpose_hw(case["x"]) if tuple(case["order"]) == (1, 0, 2) else case["x"].copy()
    if op == "reshape":
        return case["x"].reshape(reshape_shape(case))
    if op == "flatten":
        n, c, h, w = case["x"].shape
        hw = {0: (c * h * w, 1), 1: (c * h, w), 2: (c, h * w)}.get(case["axis"], (1, c * h * w))
        return case["x"].reshape(n, 1, *hw)
    if op == "prelu":
        return port.prelu(case["x"], case["slope"])
    if op == "batchnorm":
        return port.batchnorm(case["x"], case["slope"], case["mean"], case["var"], case["bias"], case["eps"])
    if op == "input":
        return port.input_layer(case["x"], case["means"], case["scales"])
    if op == "concat":
        return port.concat_channels(case["xs"])
    raise ValueError(op)


def check_value(a, b, t):
    """The reference's only tolerance rule (src/Julius/julius_test.cpp:12-39):
    |a - b| <= max(t, t * max(|a|, |b|)). Returns the number of violations."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return int((np.abs(a - b) > np.maximum(t, t * np.maximum(np.abs(a), np.abs(b)))).sum())
