"""The pointwise (1x1 stride-1) fp16 kernel without staging (conv_pw.hip) against the general kernel, whose roundings
it repeats (same packed weights, same order of the float32 sums: bit for bit), and against the CPU oracle at 2e-3."""
import numpy as np
import pytest

from excalibur_amd import hip
from oracle import port
from tests import cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = hip.Ctx(0)
    yield c
    c.close()


@pytest.fixture
def options():
    changed = []

    def set_(name, value):
        hip.set_option(name, value)
        changed.append(name)
    yield set_
    defaults = dict(pw=1, force_splits=0, direct=1, lean=4, lean_f16=1, pw_tile=0)
    for name in changed:
        hip.set_option(name, defaults[name])


def operands(seed, n, c, h, w, k, c_stride, k_stride, shortcut):
    r = np.random.default_rng(seed)
    x = np.zeros((n, h, w, c_stride), np.float16)
    x[..., :c] = r.uniform(-1, 1, (n, h, w, c)).astype(np.float16)
    wt = r.normal(0, 0.08, (k, c, 1, 1)).astype(np.float16)
    bias = r.normal(0, 0.1, k).astype(np.float32)
    res = r.uniform(-1, 1, (n, h, w, k_stride)).astype(np.float16) if shortcut else None
    return x, wt, bias, res


def run(ctx, n, c, h, w, k, x, wt, bias, res, c_stride, k_stride, act=0, post_relu=0, post_op=None, alpha=0.0, beta=0.0, residual_last=0,
        kernel=1):
    d = ctx.conv_desc(n, c, h, w, k, kernel, 1, kernel // 2, act, c_stride, k_stride, post_relu, 0.0, post_op, alpha, beta, residual_last)
    xd = ctx.array(x.view(np.uint16))
    wp = ctx.pack_conv_weights(d, hip.F16, wt.view(np.uint16))
    bd = ctx.array(bias) if bias is not None else None
    rd = ctx.array(res.view(np.uint16)) if res is not None else None
    y = ctx.array(np.full((n, h, w, k_stride), 0x7e00, np.uint16))   # NaN bits: what the kernel leaves alone shows
    ctx.conv2d_f16(d, xd, wp, bd, rd, y, None, None)
    ctx.sync()
    return y.download()


SHAPES = [
    # seed, n, c, h, w, k, c_stride, k_stride, shortcut, act, post_relu, post_op
    (700, 2, 32, 56, 56, 64, 32, 64, False, 0, 0, None),            # MobileNet pointwise
    (701, 1, 128, 40, 40, 255, 128, 256, False, 0, 0, None),        # detection head: ragged channels, one pad channel
    (702, 1, 64, 33, 31, 64, 64, 64, True, 0, 1, None),             # 1023 pixels: a ragged last tile; shortcut + ReLU
    (703, 3, 16, 9, 7, 32, 16, 32, False, 1, 0, None),              # one k-step, one 32-channel block (128 pixels per wave)
    (704, 1, 48, 20, 20, 96, 48, 96, False, 0, 0, "hardswish"),     # three k-steps, three blocks in two slabs
    (705, 1, 512, 20, 20, 256, 512, 256, False, 0, 0, "hardswish"),  # 32 k-steps: the request ring turns four times
    (706, 1, 1024, 10, 10, 512, 1024, 512, False, 0, 0, "leakyrelu"),
    (707, 2, 32, 256, 256, 32, 32, 32, False, 0, 0, "hardswish"),    # 131 072 pixels
    (708, 2, 64, 200, 200, 64, 64, 64, True, 0, 0, None),            # 64 x 64 per wave, shortcut without ReLU
    (709, 1, 40, 12, 12, 24, 48, 32, False, 3, 0, None),             # channel strides beyond the channel counts
    (710, 1, 256, 40, 40, 128, 256, 128, False, 0, 0, "clip"),
    (711, 1, 64, 17, 5, 128, 64, 128, False, 4, 0, None),            # sigmoid: the out-of-line activation
]


@pytest.mark.parametrize("args", SHAPES, ids=[f"s{a[0]}" for a in SHAPES])
def test_pointwise_kernel_repeats_the_general_kernel_bit_for_bit(ctx, options, args):
    seed, n, c, h, w, k, cs, ks, shortcut, act, post_relu, post_op = args
    x, wt, bias, res = operands(seed, n, c, h, w, k, cs, ks, shortcut)
    alpha, beta = {"hardswish": (1 / 6, 0.5), "leakyrelu": (0.1, 0.0), "clip": (-0.25, 0.5), None: (0.0, 0.0)}[post_op]
    options("force_splits", 1)   # a small launch of the general kernel would split its sum, which changes its order
    options("pw", 0)
    want = run(ctx, n, c, h, w, k, x, wt, bias, res, cs, ks, act, post_relu, post_op, alpha, beta)
    options("pw", 2)             # every layer the kernel can take, not only those it is faster on
    got = run(ctx, n, c, h, w, k, x, wt, bias, res, cs, ks, act, post_relu, post_op, alpha, beta)
    assert not np.any(want[..., :k] == 0x7e00)
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} of {want.size} halves differ"


@pytest.mark.parametrize("args", [(720, 2, 32, 56, 56, 64), (721, 1, 128, 40, 40, 255), (722, 1, 512, 20, 20, 256), (723, 1, 64, 33, 31, 32)],
                         ids=["s720", "s721", "s722", "s723"])
def test_pointwise_kernel_within_2e3_of_the_oracle(ctx, options, args):
    seed, n, c, h, w, k = args
    options("pw", 2)
    case = cases.conv_f32_case(seed, n, c, h, w, k, 1, 1, 0)
    x16 = case["x"].astype(np.float16)
    want = port.float2half(cases.oracle_eval(dict(case, x=x16.astype(np.float32)))).view(np.float16).astype(np.float32)
    ks = hip.pad_to(k, 16)
    got = run(ctx, n, c, h, w, k, np.ascontiguousarray(x16.transpose(0, 2, 3, 1)), case["wt"].astype(np.float16), case["bias"], None, c, ks,
              act=case["act"])
    got = got[..., :k].view(np.float16).astype(np.float32).transpose(0, 3, 1, 2)
    assert cases.check_value(got, want, 2e-3) == 0


@pytest.mark.parametrize("kernel,pw", [(1, 0), (1, 2), (3, 0)], ids=["general-1x1", "pointwise", "general-3x3"])
def test_shortcut_behind_the_activation_equals_the_sum_layer(ctx, options, kernel, pw):
    """convolution -> HardSwish -> add in one launch (residual_last) == the launch without the shortcut, then the sum layer
    on the stored halves."""
    n, c, h, w, k = 2, 64, 20, 24, 64
    r = np.random.default_rng(730 + kernel)
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float16)
    wt = r.normal(0, 0.08, (k, c, kernel, kernel)).astype(np.float16)
    bias = r.normal(0, 0.1, k).astype(np.float32)
    res = r.uniform(-1, 1, (n, h, w, k)).astype(np.float16)
    options("pw", pw)
    plain = run(ctx, n, c, h, w, k, x, wt, bias, None, c, k, post_op="hardswish", alpha=1 / 6, beta=0.5, kernel=kernel)
    want = ctx.add_f16(ctx.array(plain), ctx.array(res.view(np.uint16))).download()
    assert np.array_equal(want, (plain.view(np.float16).astype(np.float32) + res.astype(np.float32)).astype(np.float16).view(np.uint16))
    got = run(ctx, n, c, h, w, k, x, wt, bias, res, c, k, post_op="hardswish", alpha=1 / 6, beta=0.5, residual_last=1, kernel=kernel)
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} of {want.size} halves differ"
    # in front of the activation (the default) the shortcut gives other values
    front = run(ctx, n, c, h, w, k, x, wt, bias, res, c, k, post_op="hardswish", alpha=1 / 6, beta=0.5, kernel=kernel)
    assert not np.array_equal(front, want)


I8_SHAPES = [
    # seed, n, c, h, w, k, shortcut (0 none, 1 in front of the activation, 2 behind it), act, post_relu, post_op
    (740, 2, 32, 56, 56, 64, 0, 0, 0, None),
    (741, 1, 128, 40, 40, 255, 0, 0, 0, None),              # ragged channels: the last block's stores are guarded
    (742, 1, 64, 33, 31, 64, 1, 0, 1, None),                # a ragged last tile; shortcut + ReLU
    (743, 3, 16, 9, 7, 32, 0, 1, 0, None),                  # one k-step (16 of its 32 bytes are pad), one 32-channel block
    (744, 1, 48, 20, 20, 96, 2, 0, 0, "hardswish"),         # the sum behind the activation layer
    (745, 1, 512, 20, 20, 256, 0, 0, 0, "hardswish"),       # 16 k-steps: the request ring turns twice
    (746, 2, 32, 128, 128, 32, 0, 0, 0, "leakyrelu"),       # 32 768 pixels, a lone 32-channel block
    (747, 2, 64, 100, 100, 64, 1, 0, 0, "clip"),
    (748, 1, 40, 12, 12, 24, 0, 3, 0, None),
    (749, 1, 64, 17, 5, 128, 0, 4, 0, "hardsigmoid"),       # sigmoid: the out-of-line activation
]
I8_PARAMS = {"hardswish": (1 / 6, 0.5), "leakyrelu": (0.1, 0.0), "clip": (-0.25, 0.5), "hardsigmoid": (0.2, 0.5), None: (0.0, 0.0)}


@pytest.mark.parametrize("outputs", ["both", "int8", "float32"])
@pytest.mark.parametrize("args", I8_SHAPES, ids=[f"s{a[0]}" for a in I8_SHAPES])
def test_int8_pointwise_kernel_repeats_the_general_kernel_bit_for_bit(ctx, options, args, outputs):
    """The int8 form of the kernel (same byte geometry, v_mfma_i32_32x32x32_i8, the general kernel's int8 epilogue) against
    the general kernel on the same packed weights: float32 NHWC and requantized int8 NHWC results. The general kernel's
    results are pinned against the oracle in tests/test_gpu_ops.py."""
    from tests import gpueval
    seed, n, c, h, w, k, shortcut, act, post_relu, post_op = args
    case = cases.conv_i8_case(seed, n, c, h, w, k, 1, 1, 0, act=act)
    ks = hip.pad_to(k, 32)
    res = np.random.default_rng(seed + 50).uniform(-2, 2, (n, h, w, ks)).astype(np.float32) if shortcut else None
    alpha, beta = I8_PARAMS[post_op]
    want_list = ("nhwc",) if outputs != "int8" else ()
    fs_out = None if outputs == "float32" else np.float32(9.7)
    kw = dict(fs_out=fs_out, residual=res, post_relu=post_relu, want=want_list, post_op=post_op, post_alpha=alpha, post_beta=beta,
              residual_last=1 if shortcut == 2 else 0)
    options("force_splits", 1)
    options("pw", 0)
    want = gpueval.conv_i8(ctx, case, **kw)
    options("pw", 2)
    got = gpueval.conv_i8(ctx, case, **kw)
    for name in ("nhwc", "i8"):
        if name in want:
            a, b = want[name][..., :k], got[name][..., :k]
            assert np.array_equal(a.view(np.uint32) if name == "nhwc" else a, b.view(np.uint32) if name == "nhwc" else b), \
                f"{name}: {np.count_nonzero(a != b)} of {a.size} differ"
            assert act == 3 or np.count_nonzero(b) > b.size // 8   # activation 3 zeroes what lies above 6
            if k < ks:
                assert not got[name][..., k:].any()     # pad channels are written as zeros


@pytest.mark.parametrize("args", [(760, 2, 32, 28, 28, 64), (761, 1, 128, 20, 20, 255), (762, 1, 256, 10, 10, 96)], ids=["s760", "s761", "s762"])
def test_int8_pointwise_kernel_equals_the_oracle(ctx, options, args):
    seed, n, c, h, w, k = args
    options("pw", 2)
    from tests import gpueval
    case = cases.conv_i8_case(seed, n, c, h, w, k, 1, 1, 0)
    want = port.conv2d_i8(case["x"], case["wt"], case["bias"], case["ws"], case["fs"], case["act"], cases.geom_of(case))
    fs_out = np.float32(7.3)
    got = gpueval.conv_i8(ctx, case, fs_out=fs_out, want=("nhwc",))
    assert np.array_equal(got["nhwc"][..., :k].view(np.uint32), want.transpose(0, 2, 3, 1).view(np.uint32))
    assert np.array_equal(got["i8"][..., :k], port.quantize(want, fs_out).transpose(0, 2, 3, 1))


@pytest.mark.parametrize("unary", [None, "leakyrelu", "hardswish"])
@pytest.mark.parametrize("splits", [(32, 64), (64, 32, 32), (96,)], ids=["32+64", "64+32+32", "96"])
def test_int8_pointwise_layers_write_their_slices_of_a_concat_with_its_batchnorm_and_activation(ctx, options, splits, unary):
    """Concat -> BatchNorm -> activation over 1x1 int8 layers, done by the layers themselves: each launch carries its slice
    of the BatchNorm coefficients (post_bn_a / post_bn_b), the activation (post_op), the Concat's channel count as output
    stride and exact_k = 1, and writes channels [offset, offset + k) of the int8 tensor only. Against the oracle's
    convolution and quantizer around the float32 layers' own BatchNorm and activation kernels; what a launch does not own
    (the other layers' slices, pad channels of the stride) keeps the fill value."""
    r = np.random.default_rng(905)
    n, c, h, w = 2, 64, 9, 11
    total = sum(splits)
    stride = total + 32            # a stride wider than the Concat: those channels belong to nobody
    pa = r.normal(0, 0.5, total).astype(np.float32)
    pb = r.uniform(0.5, 2, total).astype(np.float32)
    alpha, beta = I8_PARAMS[unary]
    fs_out = np.float32(11.5)
    bn = (ctx.array(pa), ctx.array(pb))
    y = ctx.array(np.full((n, h, w, stride), 77, np.int8))
    parts, offset = [], 0
    for i, k in enumerate(splits):
        case = cases.conv_i8_case(906 + i, n, c, h, w, k, 1, 1, 0, act=0, out_scale=0.02)
        parts.append(port.conv2d_i8(case["x"], case["wt"], case["bias"], case["ws"], case["fs"], 0, cases.geom_of(case)))
        d = ctx.conv_desc(n, c, h, w, k, 1, 1, 0, 0, 64, stride, 0, float(fs_out), unary, alpha, beta, 0,
                          (bn[0].at(4 * offset), bn[1].at(4 * offset)), 1)
        xq = ctx.quantize_nchw_to_nhwc_i8(ctx.array(case["x"]), case["fs"], 64)
        wp = ctx.pack_conv_weights(d, hip.I8, case["wt"])
        from tests.gpueval import dequant_scales
        ctx.conv2d_i8(d, xq, wp, ctx.array(dequant_scales(case["ws"], case["fs"], k)), ctx.array(case["bias"]), None, y.at(offset))
        ctx.sync()
        got = y.download()
        assert (got[..., offset + k:] == 77).all()      # nothing behind the slice is touched
        offset += k
    dev = ctx.channelwise_f32("batchnorm", ctx.array(np.ascontiguousarray(np.concatenate(parts, axis=1))), *bn)
    if unary:
        dev = ctx.unary_f32(unary, dev, alpha, beta)
    ctx.sync()
    want = port.quantize(dev.download(), fs_out).transpose(0, 2, 3, 1)
    assert np.array_equal(got[..., :total], want), f"{np.count_nonzero(got[..., :total] != want)} of {want.size} differ"
    assert np.count_nonzero(want) > want.size // 2


def test_batchnorm_and_exact_channels_are_refused_outside_the_int8_pointwise_kernel(ctx):
    """The two descriptor fields exist for 1x1 int8 layers only: every other layer answers EXHIP_ERR_UNSUPPORTED."""
    n, c, h, w, k = 1, 64, 8, 8, 64
    case = cases.conv_i8_case(930, n, c, h, w, k, 3, 1, 1, act=0)
    bn = (ctx.array(np.zeros(k, np.float32)), ctx.array(np.ones(k, np.float32)))
    xq = ctx.quantize_nchw_to_nhwc_i8(ctx.array(case["x"]), case["fs"], 64)
    from tests.gpueval import dequant_scales
    scale = ctx.array(dequant_scales(case["ws"], case["fs"], k))
    y = ctx.empty((n, h, w, k), np.int8)
    for kwargs in (dict(post_bn=bn), dict(exact_k=1)):
        d = ctx.conv_desc(n, c, h, w, k, 3, 1, 1, 0, 64, k, 0, 5.0, **kwargs)
        wp = ctx.pack_conv_weights(d, hip.I8, case["wt"])
        with pytest.raises(hip.ExhipError):
            ctx.conv2d_i8(d, xq, wp, scale, None, None, y)
    d = ctx.conv_desc(n, c, h, w, 48, 1, 1, 0, 0, 64, 64, 0, 5.0, exact_k=1)     # exact_k needs whole 32-channel blocks
    case1 = cases.conv_i8_case(931, n, c, h, w, 48, 1, 1, 0, act=0)
    wp = ctx.pack_conv_weights(d, hip.I8, case1["wt"])
    with pytest.raises(hip.ExhipError):
        ctx.conv2d_i8(d, xq, wp, ctx.array(dequant_scales(case1["ws"], case1["fs"], 48)), None, None, y)


TAP_SHAPES = [
    # seed, n, c, h, w, k, kernel, stride, pad, shortcut (0 none, 1 in front, 2 behind), act, post_relu, post_op
    (800, 2, 12, 40, 36, 32, 3, 1, 1, 0, 0, 0, "hardswish"),       # a first layer behind Focus: 12 channels in a 32-byte pixel
    (801, 2, 32, 41, 37, 64, 3, 2, 1, 0, 0, 0, "hardswish"),       # stride 2 on odd sizes
    (802, 1, 64, 20, 20, 128, 3, 2, 1, 0, 1, 0, None),
    (803, 2, 32, 17, 19, 32, 3, 1, 1, 2, 0, 0, "leakyrelu"),       # a bottleneck's 3x3 with the sum behind the activation
    (804, 1, 64, 14, 14, 96, 3, 1, 1, 1, 0, 1, None),              # shortcut + ReLU; 96 channels: a half-empty second group
    (805, 1, 16, 13, 11, 40, 5, 1, 2, 0, 1, 0, None),              # 25 taps, ragged channels
    (806, 3, 64, 16, 16, 64, 1, 2, 0, 0, 0, 0, None),              # a projection shortcut: 1x1 stride 2
    (807, 1, 32, 9, 30, 64, (3, 1), 1, (1, 1, 0, 0), 0, 1, 0, None),   # 3x1 filter
    (808, 1, 128, 12, 12, 64, 3, 1, 0, 0, 0, 0, "clip"),           # no padding: the output is smaller than the input
    (809, 2, 48, 10, 10, 32, 2, 2, 0, 0, 0, 0, None),              # 2x2 stride 2 (a 64-byte pixel with 16 pad bytes)
]


@pytest.mark.parametrize("outputs", ["both", "int8", "float32"])
@pytest.mark.parametrize("args", TAP_SHAPES, ids=[f"s{a[0]}" for a in TAP_SHAPES])
def test_int8_layers_with_a_filter_on_the_kernel_without_staging_repeat_the_general_kernel(ctx, options, args, outputs):
    """The tapped form of the kernel (pixel fragments fetched from the filter's taps around each output pixel, zeros
    outside the image) against the general and lean kernels on the same packed weights, bit for bit; those are pinned
    against the oracle in tests/test_gpu_ops.py."""
    from tests import gpueval
    seed, n, c, h, w, k, kernel, stride, pad, shortcut, act, post_relu, post_op = args
    case = cases.conv_i8_case(seed, n, c, h, w, k, kernel, stride, pad, act=act)
    ks = hip.pad_to(k, 32)
    oh, ow = port.out_hw(cases.geom_of(case))
    res = np.random.default_rng(seed + 50).uniform(-2, 2, (n, oh, ow, ks)).astype(np.float32) if shortcut else None
    alpha, beta = I8_PARAMS[post_op]
    want_list = ("nhwc",) if outputs != "int8" else ()
    fs_out = None if outputs == "float32" else np.float32(9.7)
    kw = dict(fs_out=fs_out, residual=res, post_relu=post_relu, want=want_list, post_op=post_op, post_alpha=alpha, post_beta=beta,
              residual_last=1 if shortcut == 2 else 0)
    options("force_splits", 1)
    options("direct", 0)
    want = gpueval.conv_i8(ctx, case, **kw)
    options("direct", 2)
    got = gpueval.conv_i8(ctx, case, **kw)
    for name in ("nhwc", "i8"):
        if name in want:
            a, b = want[name][..., :k], got[name][..., :k]
            assert a.shape == (n, oh, ow, k)
            assert np.array_equal(a.view(np.uint32) if name == "nhwc" else a, b.view(np.uint32) if name == "nhwc" else b), \
                f"{name}: {np.count_nonzero(a != b)} of {a.size} differ"
            assert np.count_nonzero(b) > b.size // 8
            if k < ks:
                assert not got[name][..., k:].any()


def test_int8_tapped_form_equals_the_oracle(ctx, options):
    from tests import gpueval
    options("direct", 2)
    for seed, n, c, h, w, k, kernel, stride, pad in [(820, 2, 12, 24, 20, 32, 3, 1, 1), (821, 1, 32, 23, 25, 64, 3, 2, 1), (822, 1, 64, 9, 9, 255, 3, 1, 1)]:
        case = cases.conv_i8_case(seed, n, c, h, w, k, kernel, stride, pad)
        want = port.conv2d_i8(case["x"], case["wt"], case["bias"], case["ws"], case["fs"], case["act"], cases.geom_of(case))
        fs_out = np.float32(7.3)
        got = gpueval.conv_i8(ctx, case, fs_out=fs_out, want=("nhwc",))
        assert np.array_equal(got["nhwc"][..., :k].view(np.uint32), want.transpose(0, 2, 3, 1).view(np.uint32))
        assert np.array_equal(got["i8"][..., :k], port.quantize(want, fs_out).transpose(0, 2, 3, 1))


F16_TAP_SHAPES = [
    # seed, n, c, h, w, k, kernel, stride, pad, shortcut, act, post_relu, post_op
    (840, 2, 12, 40, 36, 32, 3, 1, 1, False, 0, 0, "hardswish"),
    (841, 2, 32, 41, 37, 64, 3, 2, 1, False, 0, 0, "hardswish"),
    (842, 1, 64, 20, 20, 128, 3, 2, 1, False, 1, 0, None),
    (843, 2, 32, 17, 19, 32, 3, 1, 1, True, 0, 1, None),
    (844, 1, 16, 13, 11, 40, 5, 1, 2, False, 1, 0, None),
    (845, 3, 64, 16, 16, 64, 1, 2, 0, False, 0, 0, None),
]


@pytest.mark.parametrize("args", F16_TAP_SHAPES, ids=[f"s{a[0]}" for a in F16_TAP_SHAPES])
def test_fp16_layers_with_a_filter_on_the_kernel_without_staging(ctx, options, args):
    """fp16: against the general kernel (the k-steps run in the same order: bit for bit) and against the oracle on the
    half-rounded operands at 2e-3."""
    seed, n, c, h, w, k, kernel, stride, pad, shortcut, act, post_relu, post_op = args
    r = np.random.default_rng(seed)
    cs, ks = hip.pad_to(c, 16), hip.pad_to(k, 16)
    x = np.zeros((n, h, w, cs), np.float16)
    x[..., :c] = r.uniform(-1, 1, (n, h, w, c)).astype(np.float16)
    wt = r.normal(0, 0.08, (k, c, kernel, kernel)).astype(np.float16)
    bias = r.normal(0, 0.1, k).astype(np.float32)
    g = port.geom((n, c, h, w), k, kernel, kernel, stride, pad)
    oh, ow = port.out_hw(g)
    res = r.uniform(-1, 1, (n, oh, ow, ks)).astype(np.float16) if shortcut else None
    alpha, beta = I8_PARAMS[post_op]

    def launch():
        d = ctx.conv_desc(n, c, h, w, k, kernel, stride, pad, act, cs, ks, post_relu, 0.0, post_op, alpha, beta, 0)
        wp = ctx.pack_conv_weights(d, hip.F16, wt.view(np.uint16))
        y = ctx.array(np.full((n, oh, ow, ks), 0x7e00, np.uint16))
        ctx.conv2d_f16(d, ctx.array(x.view(np.uint16)), wp, ctx.array(bias), ctx.array(res.view(np.uint16)) if shortcut else None, y, None, None)
        ctx.sync()
        return y.download()

    options("force_splits", 1)
    options("lean_f16", 0)
    options("direct", 0)
    want = launch()
    options("direct", 2)
    got = launch()
    assert np.array_equal(want, got), f"{np.count_nonzero(want != got)} of {want.size} differ"
    ref = port.conv2d_f32(x[..., :c].astype(np.float32).transpose(0, 3, 1, 2), wt.astype(np.float32), bias, act, g)
    if shortcut:
        ref = ref + res[..., :k].astype(np.float32).transpose(0, 3, 1, 2)
    if post_relu:
        ref = np.maximum(ref, 0)
    if post_op:
        ref = port.hardswish(ref, alpha, beta)
    assert cases.check_value(got[..., :k].view(np.float16).astype(np.float32), ref.transpose(0, 2, 3, 1), 2e-3) == 0


def test_the_two_wave_tiles_give_the_same_results(ctx, options):
    """Layers of more than 32 output channels run on 32-pixel x 64-channel wave tiles; option pw_tile = 2 brings back the
    64 x 64 tile for launches of 2048 waves and more. Same k-step order, same epilogue: int8 and fp16 results bit for bit,
    pointwise and with a filter."""
    from tests import gpueval
    options("pw", 2)
    options("direct", 2)
    options("lean_f16", 0)
    options("force_splits", 1)
    for kernel, stride, pad, h in ((1, 1, 0, 128), (3, 2, 1, 256)):
        case = cases.conv_i8_case(950 + kernel, 2, 32, h, h, 256, kernel, stride, pad, act=0, out_scale=0.05)
        res = {}
        for tile in (0, 2):
            options("pw_tile", tile)
            res[tile] = gpueval.conv_i8(ctx, case, fs_out=np.float32(3.1), want=("nhwc",), post_op="hardswish", post_alpha=1 / 6, post_beta=0.5)
        assert np.array_equal(res[0]["nhwc"].view(np.uint32), res[2]["nhwc"].view(np.uint32))
        assert np.array_equal(res[0]["i8"], res[2]["i8"]) and np.count_nonzero(res[0]["i8"]) > res[0]["i8"].size // 4
    x, wt, bias, _ = operands(955, 2, 64, 128, 128, 256, 64, 256, False)
    out = {}
    for tile in (0, 2):
        options("pw_tile", tile)
        out[tile] = run(ctx, 2, 64, 128, 128, 256, x, wt, bias, None, 64, 256, post_op="hardswish", alpha=1 / 6, beta=0.5)
    assert np.array_equal(out[0], out[2]) and np.count_nonzero(out[0]) > out[0].size // 2
