"""Evaluates a case from tests/cases.py on the GPU through the exhip C ABI (excalibur_amd.hip)."""
import numpy as np

from excalibur_amd import hip
from tests import cases


def dequant_scales(ws, fs, k):
    """Host-side scale exactly as src/Excalibur/operation_convolution.cpp:400-403 (float32 arithmetic)."""
    ws = np.broadcast_to(np.asarray(ws, np.float32).ravel(), (k,)) if np.size(ws) == 1 else np.asarray(ws, np.float32)
    fs = np.float32(fs)
    with np.errstate(divide="ignore", over="ignore"):
        s = np.float32(1.0) / (ws * fs).astype(np.float32)
    return np.where(np.abs(ws.astype(np.float64)) <= 1e-6, np.float32(0), s).astype(np.float32)


def in_stride(c, dtype, kw):
    es = {hip.I8: 1, hip.F16: 2, hip.F32: 4}[dtype]
    if c <= 4 and ((dtype == hip.I8 and kw <= 8) or (dtype == hip.F16 and kw <= 4)):
        return 4
    return hip.pad_to(c * es, 32) // es


def conv_i8(ctx, case, fs_out=None, residual=None, post_relu=0, want=("nchw", "acc"), post_op=None, post_alpha=0.0, post_beta=0.0,
            residual_last=0):
    n, c, h, w = case["x"].shape
    k = case["k"]
    cs = in_stride(c, hip.I8, case["kw"])
    ks = hip.pad_to(k, 32)
    d = ctx.conv_desc(n, c, h, w, k, (case["kh"], case["kw"]), case["stride"], case["pad"], case["act"], cs, ks,
                      post_relu, float(fs_out or 0.0), post_op, post_alpha, post_beta, residual_last)
    oh, ow = ctx.conv_out_hw(d)
    xq = ctx.quantize_nchw_to_nhwc_i8(ctx.array(case["x"]), case["fs"], cs)
    wp = ctx.pack_conv_weights(d, hip.I8, case["wt"])
    scale = ctx.array(dequant_scales(case["ws"], case["fs"], k))
    bias = ctx.array(case["bias"]) if case["bias"] is not None else None
    out = {}
    y_nchw = ctx.empty((n, k, oh, ow), np.float32) if "nchw" in want else None
    acc = ctx.empty((n, k, oh, ow), np.int32) if "acc" in want else None
    y_nhwc = ctx.empty((n, oh, ow, ks), np.float32) if "nhwc" in want else None
    y_i8 = ctx.empty((n, oh, ow, ks), np.int8) if fs_out is not None else None
    res = ctx.array(residual) if residual is not None else None
    ctx.conv2d_i8(d, xq, wp, scale, bias, res, y_i8, y_nhwc, y_nchw, acc)
    ctx.sync()
    for name, arr in (("nchw", y_nchw), ("acc", acc), ("nhwc", y_nhwc), ("i8", y_i8)):
        if arr is not None:
            out[name] = arr.download()
    out["xq"] = xq.download()
    return out


def conv_f32(ctx, case):
    n, c, h, w = case["x"].shape
    k = case["k"]
    cs = in_stride(c, hip.F32, case["kw"])
    d = ctx.conv_desc(n, c, h, w, k, (case["kh"], case["kw"]), case["stride"], case["pad"], case["act"], cs, hip.pad_to(k, 4))
    oh, ow = ctx.conv_out_hw(d)
    x = ctx.nchw_to_nhwc(ctx.array(case["x"]), cs, "f32")
    wp = ctx.pack_conv_weights(d, hip.F32, case["wt"])
    bias = ctx.array(case["bias"]) if case["bias"] is not None else None
    y = ctx.empty((n, k, oh, ow), np.float32)
    ctx.conv2d_f32(d, x, wp, bias, None, None, y)
    return y.download()


def conv_f16(ctx, case, x16):
    """fp16 layer: half NCHW in, half NCHW out, f32 accumulation; weights rounded to half (RNE) on the host."""
    n, c, h, w = x16.shape
    k = case["k"]
    cs = in_stride(c, hip.F16, case["kw"])
    d = ctx.conv_desc(n, c, h, w, k, (case["kh"], case["kw"]), case["stride"], case["pad"], case["act"], cs, hip.pad_to(k, 16))
    oh, ow = ctx.conv_out_hw(d)
    x = ctx.nchw_to_nhwc(ctx.array(x16, np.uint16), cs, "f16")
    wp = ctx.pack_conv_weights(d, hip.F16, case["wt"].astype(np.float16).view(np.uint16))
    bias = ctx.array(case["bias"]) if case["bias"] is not None else None
    y = ctx.empty((n, k, oh, ow), np.uint16)
    ctx.conv2d_f16(d, x, wp, bias, None, None, y, None)
    return y.download()


def gpu_eval(ctx, case):
    op = case["op"]
    if op == "conv_i8":
        if case["groups"] != 1:
            return conv_direct(ctx, case)
        return conv_i8(ctx, case, want=("nchw",))["nchw"]
    if op == "conv_f32":
        if case["groups"] != 1:
            return conv_direct(ctx, case)
        return conv_f32(ctx, case)
    if op in ("dw_f32", "dw_i8"):
        x = ctx.array(case["x"])
        if op == "dw_i8":
            wf = ctx.dw_dequant_weights(ctx.array(case["wt"]), ctx.array(case["ws"]))
        else:
            wf = ctx.array(case["wt"])
        bias = ctx.array(case["bias"]) if case["bias"] is not None else None
        return ctx.dwconv3x3_nchw_f32(x, wf, bias, case["stride"], case["pad"], case["act"]).download()
    if op == "pool":
        return ctx.pool2d_nchw_f32(ctx.array(case["x"]), case["ptype"], case["kernel"], case["stride"], case["pad"],
                                   case["global_pool"], case["pad_mode"], case["count_include_pad"]).download()
    if op == "eltwise":
        return ctx.eltwise_f32([ctx.array(a) for a in case["xs"]], case["etype"], case.get("coeffs")).download()
    if op == "binaryop_add":
        return ctx.add_f32(ctx.array(case["xs"][0]), ctx.array(case["xs"][1])).download()
    if op == "relu":
        return ctx.relu_f32(ctx.array(case["x"])).download()
    if op == "fc":
        return ctx.innerproduct_f32(ctx.array(case["x"]), ctx.array(case["wt"]),
                                    ctx.array(case["bias"]) if case["bias"] is not None else None).download()
    if op == "deconv":
        return ctx.deconv2d_f32(ctx.array(case["x"]), ctx.array(case["wt"]), ctx.array(case["bias"]) if case["bias"] is not None else None,
                                case["stride"], case["pad"]).download()
    if op in ("hardswish", "hardsigmoid"):
        return ctx.unary_f32(op, ctx.array(case["x"]), case["alpha"], case["beta"]).download()
    if op == "leakyrelu":
        return ctx.unary_f32(op, ctx.array(case["x"]), case["alpha"]).download()
    if op == "sigmoid":
        return ctx.unary_f32(op, ctx.array(case["x"])).download()
    if op == "binaryop_bc":
        x = ctx.array(case["x"])
        kind = case["small"]
        if kind == "equal":
            small, mode = ctx.unary_f32("clip", x, 0.5, 3.0), 0
        elif kind == "channel":
            small, mode = ctx.pool2d_nchw_f32(x, 1, global_pool=True), 2
        else:
            small, mode = ctx.array(cases.binaryop_bc_small(dict(case, small="pixel"))), 3  # the 1x1 convolution is not under test
            if kind == "image":
                small, mode = ctx.pool2d_nchw_f32(small, 1, global_pool=True), 1
        if kind == "equal" and case["swap"]:
            return ctx.binaryop_f32(case["op_type"], 0, small, x).download()
        return ctx.binaryop_f32(case["op_type"], mode, x, small).download()
    if op == "clip":
        return ctx.unary_f32("clip", ctx.array(case["x"]), case["lo"], case["hi"]).download()
    if op == "softmax":
        return ctx.softmax_channels_f32(ctx.array(case["x"])).download()
    if op == "transpose":
        return ctx.transpose_hw_f32(ctx.array(case["x"])).download() if tuple(case["order"]) == (1, 0, 2) else case["x"].copy()
    if op in ("reshape", "flatten"):  # no kernel of their own: a new shape over the same values (Flatten copies them)
        return cases.oracle_eval(case)
    if op == "prelu":
        return ctx.channelwise_f32("prelu", ctx.array(case["x"]), ctx.array(case["slope"]), shared=case["slope"].size == 1).download()
    if op == "batchnorm":
        # a and b as the layer computes them when it loads (src/Excalibur/operation_batchnorm.cpp:52-64)
        sqrt_var = np.sqrt((case["var"] + np.float32(case["eps"])).astype(np.float64)).astype(np.float32)
        a = (case["bias"] - case["slope"] * case["mean"] / sqrt_var).astype(np.float32)
        b = (case["slope"] / sqrt_var).astype(np.float32)
        return ctx.channelwise_f32("batchnorm", ctx.array(case["x"]), ctx.array(a), ctx.array(b)).download()
    if op == "input":
        return ctx.channelwise_f32("input", ctx.array(case["x"]), ctx.array(np.asarray(case["means"], np.float32)),
                                   ctx.array(np.asarray(case["scales"], np.float32))).download()
    if op == "concat":
        return ctx.concat_channels_f32([ctx.array(a) for a in case["xs"]]).download()
    if op == "interp":
        h, w = case["x"].shape[2:]
        oh, ow = int(np.float32(h) * np.float32(case["height_scale"])), int(np.float32(w) * np.float32(case["width_scale"]))
        return ctx.interp_nearest_f32(ctx.array(case["x"]), oh, ow).download()
    if op == "focus":
        return ctx.focus_f32(ctx.array(case["x"])).download()
    raise ValueError(op)


def conv_direct(ctx, case):
    n, c, h, w = case["x"].shape
    k = case["k"]
    d = ctx.conv_desc(n, c, h, w, k, (case["kh"], case["kw"]), case["stride"], case["pad"], case["act"])
    oh, ow = ctx.conv_out_hw(d)
    y = ctx.empty((n, k, oh, ow), np.float32)
    bias = ctx.array(case["bias"]) if case["bias"] is not None else None
    if case["op"] == "conv_i8":
        ctx.conv2d_direct(d, case["groups"], ctx.array(case["x"]), y, w_i8=ctx.array(case["wt"]), fs=case["fs"],
                          scale=ctx.array(dequant_scales(case["ws"], case["fs"], k)), bias=bias)
    else:
        ctx.conv2d_direct(d, case["groups"], ctx.array(case["x"]), y, w_f32=ctx.array(case["wt"]), bias=bias)
    return y.download()
