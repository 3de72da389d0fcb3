"""GPU parity tests: every operator of the hot path through the exhip C ABI against
(1) the golden fixtures written by the compiled reference, (2) the CPU restatement on larger seeded
shapes, (3) size-independent properties at the benchmark sizes.

Bars: int32 accumulators, dequantized outputs of the int8 path, requantized int8 outputs, depthwise,
pooling and elementwise results bit-exact (== on floats, so +0.0 equals -0.0); fp32 convolution and
inner product within 1e-4 and fp16 within 2e-3 under the reference's check_value rule
(|a-b| <= max(t, t*max(|a|,|b|)), src/Julius/julius_test.cpp:12-39).
"""
import glob
import os

import numpy as np
import pytest

from oracle import port
from tests import cases, gpueval
from tests.golden.make_fixtures import load_case

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
NAMES = sorted(os.path.basename(f)[:-4] for f in glob.glob(os.path.join(GOLDEN, "*.npz")) if not os.path.basename(f).startswith("net_"))
TOLERANT = ("conv_f32", "fc_", "deconv", "softmax", "binaryop_pixel", "binaryop_image", "conv_i8_mish")


@pytest.fixture(scope="module")
def ctx():
    from excalibur_amd import hip
    c = hip.Ctx(0)
    yield c
    c.close()


@pytest.mark.parametrize("name", [n for n in NAMES if not n.startswith("f16_")])
def test_golden_fixture(ctx, name):
    case, expected = load_case(os.path.join(GOLDEN, name + ".npz"))
    got = gpueval.gpu_eval(ctx, case)
    assert got.shape == expected.shape
    if name.startswith(TOLERANT):
        assert cases.check_value(got, expected, 1e-4) == 0
    else:
        assert np.array_equal(got, expected)


@pytest.mark.parametrize("name", ["f16_conv_3x3s1", "f16_conv_tail75"])
def test_golden_fixture_fp16_conv(ctx, name):
    case, expected = load_case(os.path.join(GOLDEN, name + ".npz"))
    got = gpueval.conv_f16(ctx, case, case["x"])
    assert cases.check_value(got.view(np.float16).astype(np.float32), expected.view(np.float16).astype(np.float32), 2e-3) == 0


I8_SHAPES = [
    # seed, n, c, h, w, k, kernel, stride, pad
    (200, 2, 128, 80, 80, 128, 3, 1, 1),    # cfg2 3x3 (two of the eight images)
    (201, 2, 128, 80, 80, 256, 1, 1, 0),    # cfg2 1x1
    (202, 1, 64, 160, 160, 64, 3, 1, 1),    # ResNet-18 stage 1
    (203, 2, 64, 160, 160, 128, 3, 2, 1),   # stage 2 entry, stride 2
    (204, 2, 64, 160, 160, 128, 1, 2, 0),   # 1x1 stride-2 downsample
    (205, 1, 3, 256, 256, 64, 7, 2, 3),     # stem shape (packed first-layer form)
    (206, 3, 512, 20, 20, 512, 3, 1, 1),    # stage 4: patch wider than the image rows
    (207, 2, 48, 33, 31, 72, 3, 1, 1),      # channels not a multiple of 32, odd sizes
    (208, 1, 128, 40, 40, 255, 1, 1, 0),    # YOLO head: K = 255
    (209, 2, 32, 17, 17, 40, 5, 1, 2),      # 5x5
    (210, 1, 16, 30, 30, 24, 7, 2, 3),      # 7x7 with 16 channels (generic form)
    (211, 2, 96, 24, 24, 160, 3, 2, (0, 1, 0, 1)),  # asymmetric padding
    (212, 1, 32, 256, 8, 64, 1, 1, 0),      # 1x1 on a 256-row map: the planner's patch is one pixel wide
    (213, 1, 32, 40, 1, 64, 3, 1, 1),       # an image one pixel wide
]


@pytest.mark.parametrize("args", I8_SHAPES, ids=[f"s{a[0]}" for a in I8_SHAPES])
def test_conv_i8_acc_and_output_bit_exact(ctx, args):
    case = cases.conv_i8_case(*args)
    g = cases.geom_of(case)
    want_y, want_acc = port.conv2d_i8(case["x"], case["wt"], case["bias"], case["ws"], case["fs"], case["act"], g, want_acc=True)
    got = gpueval.conv_i8(ctx, case)
    # quantized input in NHWC equals the reference's quantizer
    q = port.quantize(case["x"], case["fs"])
    assert np.array_equal(got["xq"][..., :case["c"]], q.transpose(0, 2, 3, 1))
    assert not got["xq"][..., case["c"]:].any()
    assert np.array_equal(got["acc"], want_acc)
    assert np.array_equal(got["nchw"], want_y)


def test_conv_i8_fused_residual_relu_requant(ctx):
    """conv(act 0) -> + shortcut -> ReLU -> next layer's quantizer, in one epilogue."""
    case = cases.conv_i8_case(220, 2, 64, 40, 40, 64, 3, 1, 1, act=0)
    r = np.random.default_rng(221)
    res_nchw = r.uniform(-4, 4, (2, 64, 40, 40)).astype(np.float32)
    fs_out = np.float32(17.3)
    y = cases.oracle_eval(case)
    z = port.relu(port.binaryop_add(y, res_nchw))
    want_q = port.quantize(z, fs_out)
    got = gpueval.conv_i8(ctx, case, fs_out=fs_out, residual=np.ascontiguousarray(res_nchw.transpose(0, 2, 3, 1)),
                          post_relu=1, want=("nchw", "nhwc"))
    assert np.array_equal(got["nchw"], z)
    assert np.array_equal(got["nhwc"], z.transpose(0, 2, 3, 1))
    assert np.array_equal(got["i8"], want_q.transpose(0, 2, 3, 1))


ONE_BUFFER_SHAPES = [
    # seed, n, c, h, w, k, kernel, stride, pad
    (225, 2, 128, 40, 40, 128, 3, 1, 1),   # two 64-byte chunks, three groups per CU
    (226, 1, 256, 24, 20, 64, 3, 1, 1),    # four chunks
    (227, 2, 128, 41, 39, 256, 3, 2, 1),   # strided: the 512-thread variant in its 128-register form, four 32-byte chunks
    (228, 2, 128, 24, 24, 128, 1, 1, 0),   # 1x1
]


@pytest.fixture
def one_tile_buffer():
    from excalibur_amd import hip
    hip.set_option("force_abufs", 1)
    yield
    hip.set_option("force_abufs", 0)


@pytest.mark.parametrize("args", ONE_BUFFER_SHAPES, ids=[f"s{a[0]}" for a in ONE_BUFFER_SHAPES])
def test_conv_i8_single_tile_buffer_bit_exact(ctx, args, one_tile_buffer):
    """The planner trades the second activation tile buffer for one more workgroup per CU only on launches large enough
    to gain from it; the option force_abufs = 1 makes these small launches take that path: fused int8 and
    float32 outputs with a shortcut, and the plain NCHW output, all bit-exact."""
    case = cases.conv_i8_case(*args, act=0)
    g = cases.geom_of(case)
    want_y, want_acc = port.conv2d_i8(case["x"], case["wt"], case["bias"], case["ws"], case["fs"], case["act"], g, want_acc=True)
    got = gpueval.conv_i8(ctx, case)
    assert np.array_equal(got["acc"], want_acc)
    assert np.array_equal(got["nchw"], want_y)
    r = np.random.default_rng(args[0] + 1000)
    res_nchw = r.uniform(-4, 4, want_y.shape).astype(np.float32)
    fs_out = np.float32(11.7)
    z = port.relu(port.binaryop_add(want_y, res_nchw))
    fused = gpueval.conv_i8(ctx, case, fs_out=fs_out, residual=np.ascontiguousarray(res_nchw.transpose(0, 2, 3, 1)), post_relu=1,
                            want=("nhwc",))
    assert np.array_equal(fused["nhwc"], z.transpose(0, 2, 3, 1))
    assert np.array_equal(fused["i8"], port.quantize(z, fs_out).transpose(0, 2, 3, 1))
    q_only = gpueval.conv_i8(ctx, dict(case, act=1), fs_out=fs_out, want=())
    assert np.array_equal(q_only["i8"], port.quantize(port.relu(want_y), fs_out).transpose(0, 2, 3, 1))


def test_conv_i8_requant_pad_channels_are_zero(ctx):
    case = cases.conv_i8_case(222, 1, 32, 12, 12, 40, 3, 1, 1)
    fs_out = np.float32(9.0)
    got = gpueval.conv_i8(ctx, case, fs_out=fs_out, want=("nchw",))
    want_q = port.quantize(cases.oracle_eval(case), fs_out).transpose(0, 2, 3, 1)
    assert got["i8"].shape[-1] == 64
    assert np.array_equal(got["i8"][..., :40], want_q)
    assert not got["i8"][..., 40:].any()


CONV_POOL_SHAPES = [
    # seed, n, c, h, w, k, kernel, stride, pad, pool pad, pool pad_mode
    (240, 2, 3, 150, 134, 64, 7, 2, 3, 1, 1),   # stem + pool, sizes that leave ragged pooled tiles
    (241, 1, 3, 64, 64, 64, 7, 2, 3, 0, 0),     # no pool padding, the reference's "full" output size (clipped windows)
    (242, 2, 32, 37, 41, 64, 3, 1, 1, 1, 1),    # generic (unpacked) convolution in front of the pool
    (243, 1, 64, 9, 11, 64, 3, 1, 1, 1, 1),     # image smaller than one pooled tile
]


@pytest.mark.parametrize("act,negate", [(1, False), (0, False), (1, True), (0, True)], ids=["relu", "linear", "relu-negscale", "linear-negscale"])
@pytest.mark.parametrize("args", CONV_POOL_SHAPES, ids=[f"s{a[0]}" for a in CONV_POOL_SHAPES])
def test_conv_i8_maxpool_one_launch_bit_exact(ctx, args, act, negate):
    """Convolution (+ReLU) and the 3x3 stride-2 max pool behind it in one kernel == oracle conv then oracle pool. With
    scales >= 0 the kernel pools the int32 accumulators and dequantizes the pooled pixels; a negative weight scale in
    some channels makes it pool the dequantized floats instead."""
    seed, n, c, h, w, k, kernel, stride, pad, ppad, pad_mode = args
    case = cases.conv_i8_case(seed, n, c, h, w, k, kernel, stride, pad, act=act)
    if negate:
        case["ws"] = case["ws"].copy()
        case["ws"][::3] *= np.float32(-1)
    fs_out = np.float32(23.5)
    y = cases.oracle_eval(case)
    want = port.pool2d(y, port.POOL_MAX, 3, 2, ppad, pad_mode=pad_mode)
    poh, pow_ = want.shape[2:]
    cs = gpueval.in_stride(c, gpueval.hip.I8, kernel)
    d = ctx.conv_desc(n, c, h, w, k, kernel, stride, pad, act, cs, k, 0, float(fs_out))
    xq = ctx.quantize_nchw_to_nhwc_i8(ctx.array(case["x"]), case["fs"], cs)
    wp = ctx.pack_conv_weights(d, gpueval.hip.I8, case["wt"])
    scale = ctx.array(gpueval.dequant_scales(case["ws"], case["fs"], k))
    bias = ctx.array(case["bias"])
    yf = ctx.empty((n, poh, pow_, k), np.float32)
    yq = ctx.empty((n, poh, pow_, k), np.int8)
    ctx.conv2d_i8_maxpool3x3s2(d, ppad, poh, pow_, xq, wp, scale, bias, yq, yf)
    ctx.sync()
    assert np.array_equal(yf.download(), want.transpose(0, 2, 3, 1))
    assert np.array_equal(yq.download(), port.quantize(want, fs_out).transpose(0, 2, 3, 1))
    # the int8 copy alone
    yq2 = ctx.empty((n, poh, pow_, k), np.int8)
    ctx.conv2d_i8_maxpool3x3s2(d, ppad, poh, pow_, xq, wp, scale, bias, yq2, None)
    ctx.sync()
    assert np.array_equal(yq2.download(), yq.download())


@pytest.mark.parametrize("shape", [(2, 3, 5, 7), (2, 3, 8, 10), (1, 1, 4, 4), (1, 4, 3, 3)], ids=str)
def test_first_layer_quantizer_packs_four_channel_pixels(ctx, shape):
    """float NCHW -> int8 NHWC with 4-byte pixels, through both the one-pixel and the four-pixel kernel."""
    x = np.random.default_rng(250).uniform(-2, 2, shape).astype(np.float32)
    fs = np.float32(77.7)
    got = ctx.quantize_nchw_to_nhwc_i8(ctx.array(x), fs, 4).download()
    want = port.quantize(x, fs).transpose(0, 2, 3, 1)
    assert np.array_equal(got[..., :shape[1]], want)
    assert not got[..., shape[1]:].any()


F32_SHAPES = [
    (230, 1, 64, 56, 56, 64, 3, 1, 1),      # cfg1
    (231, 1, 64, 56, 56, 128, 3, 1, 1),
    (232, 2, 24, 31, 29, 40, 3, 2, 1),
    (233, 1, 3, 64, 64, 32, 7, 2, 3),
    (234, 2, 128, 14, 14, 256, 1, 1, 0),
]


@pytest.mark.parametrize("args", F32_SHAPES, ids=[f"s{a[0]}" for a in F32_SHAPES])
def test_conv_f32_within_1e4(ctx, args):
    case = cases.conv_f32_case(*args)
    assert cases.check_value(gpueval.conv_f32(ctx, case), cases.oracle_eval(case), 1e-4) == 0


F16_SHAPES = [
    (240, 2, 32, 56, 56, 64, 1, 1, 0),      # MobileNet pointwise
    (241, 1, 3, 112, 112, 32, 3, 2, 1),     # MobileNet stem (packed first-layer form)
    (242, 2, 64, 28, 28, 128, 3, 1, 1),
    (243, 1, 128, 40, 40, 255, 1, 1, 0),
]


@pytest.mark.parametrize("args", F16_SHAPES, ids=[f"s{a[0]}" for a in F16_SHAPES])
def test_conv_f16_within_2e3(ctx, args):
    case = cases.conv_f32_case(*args)
    x16 = case["x"].astype(np.float16).view(np.uint16)
    want = port.float2half(cases.oracle_eval(dict(case, x=port.half2float(x16))))
    got = gpueval.conv_f16(ctx, case, x16)
    assert cases.check_value(got.view(np.float16).astype(np.float32), want.view(np.float16).astype(np.float32), 2e-3) == 0


@pytest.mark.parametrize("groups", [2, 4])
def test_grouped_conv_definition_kernel(ctx, groups):
    case = cases.conv_f32_case(250 + groups, 2, 16, 13, 13, 24 if groups == 2 else 16, 3, 1, 1, groups=groups)
    assert cases.check_value(gpueval.gpu_eval(ctx, case), cases.oracle_eval(case), 1e-4) == 0
    ci = cases.conv_i8_case(260 + groups, 1, 16, 12, 12, 16, 3, 2, 1, groups=groups)
    assert np.array_equal(gpueval.gpu_eval(ctx, ci), cases.oracle_eval(ci))


@pytest.mark.parametrize("stride,h,w", [(1, 56, 56), (2, 57, 55), (1, 7, 9), (2, 112, 112)])
def test_depthwise_bit_exact(ctx, stride, h, w):
    case = cases.conv_f32_case(270 + h, 2, 32, h, w, 32, 3, stride, 1, groups=32, dw=True)
    assert np.array_equal(gpueval.gpu_eval(ctx, case), cases.oracle_eval(case))
    ci = cases.dw_i8_case(280 + h, 1, 16, h, w, stride)
    assert np.array_equal(gpueval.gpu_eval(ctx, ci), cases.oracle_eval(ci))


@pytest.mark.parametrize("stride,h,w,pad,act", [(1, 23, 36, 1, 1), (2, 41, 36, 1, 0), (1, 12, 8, 0, 3), (2, 13, 44, 0, 1),
                                               (1, 5, 4, 1, 1), (2, 6, 4, 1, 1), (1, 40, 40, 1, 4)])
def test_depthwise_rows_of_four_bit_exact(ctx, stride, h, w, pad, act):
    """Rows a multiple of four floats long take the four-outputs-per-thread kernel (activation 4 does not): halos on
    both sides, ragged output rows, several bands."""
    case = cases.conv_f32_case(275 + h, 3, 24, h, w, 24, 3, stride, pad, act=act, groups=24, dw=True)
    assert np.array_equal(gpueval.gpu_eval(ctx, case), cases.oracle_eval(case))


@pytest.mark.parametrize("stride,c,h,w,act", [(2, 40, 28, 30, 1), (1, 40, 28, 30, 1), (1, 128, 56, 56, 0), (2, 64, 57, 55, 3),
                                             (1, 8, 7, 9, 1), (2, 24, 6, 5, 1), (1, 40, 19, 23, 4)])
def test_depthwise_nhwc_f16(ctx, stride, c, h, w, act):
    """Half storage, float arithmetic in the reference's order: the halves must be the float results rounded to nearest.
    Strides 1 and 2 with the plain activations take the strip kernel (ragged strips, bands and channel padding are
    all in these shapes); activation 4 takes the one-pixel-per-thread kernel."""
    from excalibur_amd import hip
    case = cases.conv_f32_case(290 + h, 2, c, h, w, c, 3, stride, 1, act=act, groups=c, dw=True)
    x16 = case["x"].astype(np.float16).view(np.uint16)
    want32 = cases.oracle_eval(dict(case, x=port.half2float(x16)))
    want = port.float2half(want32)
    x = ctx.nchw_to_nhwc(ctx.array(x16), hip.pad_to(c, 16), "f16")
    y = ctx.dwconv3x3_nhwc_f16(x, c, ctx.array(case["wt"]), ctx.array(case["bias"]), stride, 1, case["act"])
    got = ctx.nhwc_to_nchw(y, c, "f16").download()
    assert cases.check_value(got.view(np.float16).astype(np.float32), want.view(np.float16).astype(np.float32), 2e-3) == 0
    if act != 4:  # same float results, rounded to nearest even by the hardware conversion
        assert np.array_equal(got, want32.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("stride,c,h,w,shared", [(1, 24, 28, 32, False), (2, 40, 41, 36, False), (1, 16, 9, 12, True)])
def test_depthwise_with_the_prelu_layer_behind_it(ctx, stride, c, h, w, shared):
    """exhip_dwconv3x3_*_prelu: the depthwise layer (no activation of its own) and the PReLU layer behind it in one
    kernel, against the two restated layers one after the other: float32 bit for bit; half storage with the PReLU on the
    rounded half, as the fp16 pipeline's two layers compute it."""
    from excalibur_amd import hip
    case = cases.conv_f32_case(310 + h, 2, c, h, w, c, 3, stride, 1, act=0, groups=c, dw=True)
    slope = np.random.default_rng(311).uniform(-0.5, 0.5, 1 if shared else c).astype(np.float32)
    want = port.prelu(cases.oracle_eval(case), slope)
    got = ctx.dwconv3x3_nchw_f32_prelu(ctx.array(case["x"]), ctx.array(case["wt"]), ctx.array(case["bias"]), ctx.array(slope), shared,
                                       stride, 1).download()
    assert np.array_equal(got, want)
    x16 = case["x"].astype(np.float16).view(np.uint16)
    # halves rounded to nearest even, as the hardware conversion of the two separate kernels does
    mid = cases.oracle_eval(dict(case, x=port.half2float(x16))).astype(np.float16)
    want16 = port.prelu(mid.astype(np.float32), slope).astype(np.float16).view(np.uint16)
    x = ctx.nchw_to_nhwc(ctx.array(x16), hip.pad_to(c, 16), "f16")
    y = ctx.dwconv3x3_nhwc_f16_prelu(x, c, ctx.array(case["wt"]), ctx.array(case["bias"]), ctx.array(slope), shared, stride, 1)
    assert np.array_equal(ctx.nhwc_to_nchw(y, c, "f16").download(), want16)


POOLS = [
    dict(ptype=0, kernel=3, stride=2, pad=1), dict(ptype=0, kernel=5, stride=1, pad=2),
    dict(ptype=0, kernel=9, stride=1, pad=4), dict(ptype=0, kernel=13, stride=1, pad=6),
    dict(ptype=1, kernel=2, stride=2, pad=0), dict(ptype=1, kernel=2, stride=2, pad=(0, 1, 0, 1)),
    dict(ptype=1, kernel=3, stride=2, pad=1, pad_mode=0), dict(ptype=1, kernel=3, stride=2, pad=1, count_include_pad=1),
    dict(ptype=1, global_pool=True), dict(ptype=0, global_pool=True),
]


@pytest.mark.parametrize("kw", POOLS, ids=[str(i) for i in range(len(POOLS))])
def test_pool_bit_exact(ctx, kw):
    case = cases.pool_case(300, 2, 6, 41, 38, **kw)
    got, want = gpueval.gpu_eval(ctx, case), cases.oracle_eval(case)
    if kw.get("global_pool") and kw["ptype"] == 1:
        # a plane of 64 values or more is summed in interleaved runs (same bits every launch), not in the reference's
        # element order: the float sum agrees to 1e-4, the tolerance of this layer
        assert cases.check_value(got, want, 1e-4) == 0
        assert np.array_equal(got, gpueval.gpu_eval(ctx, case))
        small = cases.pool_case(301, 2, 6, 7, 7, **kw)   # small planes keep the element order
        assert np.array_equal(gpueval.gpu_eval(ctx, small), cases.oracle_eval(small))
    else:
        assert np.array_equal(got, want)


def test_global_average_pool_half_storage(ctx):
    """The MobileNet-style stack's last pooling (N x 1024 x 7 x 7 on NHWC half blobs) and a ragged one: partial sums over
    interleaved pixels, 2e-3 of the float operator on the half-rounded input, the same bits on every launch."""
    r = np.random.default_rng(320)
    for (n, c, h, w) in [(3, 1024, 7, 7), (2, 24, 5, 9), (1, 8, 20, 20)]:
        x16 = r.uniform(-3, 3, (n, c, h, w)).astype(np.float16)
        xd = ctx.nchw_to_nhwc(ctx.array(x16.view(np.uint16)), c, "f16")
        got = ctx.nhwc_to_nchw(ctx.pool2d_nhwc_f16(xd, c, 1, global_pool=True), c, "f32").download()
        want = port.pool2d(x16.astype(np.float32), port.POOL_AVE, global_pool=True)
        assert got.shape == want.shape
        assert cases.check_value(got, want, 2e-3) == 0
        again = ctx.nhwc_to_nchw(ctx.pool2d_nhwc_f16(xd, c, 1, global_pool=True), c, "f32").download()
        assert np.array_equal(got, again)


S2_POOLS = [
    dict(ptype=0, kernel=3, stride=2, pad=1), dict(ptype=0, kernel=3, stride=2, pad=0), dict(ptype=0, kernel=3, stride=2, pad=0, pad_mode=0),
    dict(ptype=0, kernel=2, stride=2, pad=0), dict(ptype=0, kernel=2, stride=2, pad=(0, 1, 0, 1)), dict(ptype=0, kernel=2, stride=2, pad=1),
    dict(ptype=1, kernel=2, stride=2, pad=0), dict(ptype=1, kernel=2, stride=2, pad=(0, 1, 0, 1)),
    dict(ptype=1, kernel=3, stride=2, pad=1, pad_mode=0), dict(ptype=1, kernel=3, stride=2, pad=1, count_include_pad=1),
    dict(ptype=1, kernel=3, stride=2, pad=0, pad_mode=0), dict(ptype=1, kernel=3, stride=2, pad=(2, 1, 1, 0)),
]


@pytest.mark.parametrize("hw", [(41, 40), (40, 36), (17, 8), (6, 4), (9, 64)], ids=lambda v: "%dx%d" % v)
@pytest.mark.parametrize("kw", S2_POOLS, ids=[str(i) for i in range(len(S2_POOLS))])
def test_pool_stride2_rows_of_four_bit_exact(ctx, kw, hw):
    """Rows a multiple of four floats long take the four-outputs-per-thread kernel: same results as the oracle for
    both halo sides, ceil and floor output sizes, clipped windows and both average divisors."""
    case = cases.pool_case(305 + hw[0], 2, 5, hw[0], hw[1], **kw)
    assert np.array_equal(gpueval.gpu_eval(ctx, case), cases.oracle_eval(case))


def test_maxpool_nhwc_with_requant_commutes(ctx):
    """NHWC f32 max pooling that also emits the next layer's int8 input: max commutes with the quantizer."""
    r = np.random.default_rng(310)
    x = r.uniform(-3, 3, (2, 64, 30, 34)).astype(np.float32)
    fs = np.float32(40.0)
    want = port.pool2d(x, port.POOL_MAX, 3, 2, 1)
    xd = ctx.nchw_to_nhwc(ctx.array(x), 64, "f32")
    y, yq = ctx.maxpool2d_nhwc_f32(xd, 64, 3, 2, 1, fs_out=fs)
    assert np.array_equal(y.download(), want.transpose(0, 2, 3, 1))
    assert np.array_equal(yq.download(), port.quantize(want, fs).transpose(0, 2, 3, 1))


def test_pool_nhwc_f16(ctx):
    r = np.random.default_rng(311)
    x16 = r.uniform(-3, 3, (2, 24, 14, 14)).astype(np.float16)
    xd = ctx.nchw_to_nhwc(ctx.array(x16.view(np.uint16)), 24, "f16")
    got = ctx.nhwc_to_nchw(ctx.pool2d_nhwc_f16(xd, 24, 1, global_pool=True), 24, "f32").download()
    want = port.pool2d(x16.astype(np.float32), port.POOL_AVE, global_pool=True)
    assert cases.check_value(got, want, 2e-3) == 0
    got = ctx.nhwc_to_nchw(ctx.pool2d_nhwc_f16(xd, 24, 0, 3, 2, 1), 24, "f32").download()
    assert np.array_equal(got, port.pool2d(x16.astype(np.float32), port.POOL_MAX, 3, 2, 1))


@pytest.mark.parametrize("shape", [(2, 3, 64, 96), (1, 3, 10, 14), (2, 5, 7, 9), (1, 1, 32, 16)], ids=str)
def test_focus_and_transpose_on_half_storage_move_the_halves(ctx, shape):
    """The fp16 pipeline's Focus and Transpose layers only move values: the halves land where the float layers put the
    floats (rows of 16 take the vector kernel, others one element per thread; odd sizes drop their last row / column)."""
    x = np.random.default_rng(385).integers(0, 1 << 16, shape).astype(np.uint16)
    n, c, h, w = shape
    want = np.concatenate([x[:, :, (g % 2):(h // 2) * 2:2, (g // 2):(w // 2) * 2:2] for g in range(4)], axis=1)
    assert np.array_equal(ctx.focus_f16(ctx.array(x)).download(), want)
    xf = x.astype(np.float32)
    assert np.array_equal(ctx.focus_f32(ctx.array(xf)).download(), want.astype(np.float32))   # the float layer agrees on the order
    assert np.array_equal(ctx.transpose_hw_f16(ctx.array(x)).download(), x.transpose(0, 1, 3, 2))


@pytest.mark.parametrize("unary,alpha,beta", [("leakyrelu", 0.1, 0.0), ("hardswish", 1 / 6, 0.5), (None, 0.0, 0.0), ("clip", -0.5, 0.75)])
@pytest.mark.parametrize("channels,with_bn", [((32, 32), True), ((64, 8, 24), True), ((16,), True), ((40, 24), False)], ids=str)
def test_concat_batchnorm_activation_in_one_kernel_equals_the_separate_layers(ctx, channels, with_bn, unary, alpha, beta):
    """Concat -> BatchNorm -> activation of the fp16 pipeline in one kernel against the three layers' own entry points
    (each of which stores halves), on NHWC half blobs; one input = BatchNorm -> activation alone."""
    r = np.random.default_rng(386)
    n, h, w = 2, 9, 13
    blobs = [ctx.array(r.normal(0, 2, (n, h, w, c)).astype(np.float16).view(np.uint16)) for c in channels]
    total = sum(channels)
    a = ctx.array(r.normal(0, 0.5, total).astype(np.float32))
    b = ctx.array(r.uniform(0.5, 2, total).astype(np.float32))
    want = ctx.concat_nhwc_f16(blobs) if len(blobs) > 1 else blobs[0]
    if with_bn:
        want = ctx.channelwise_nhwc_f16("batchnorm", want, a, b)
    if unary:
        want = ctx.unary_f16(unary, want, alpha, beta)
    got = ctx.concat_nhwc_f16(blobs, (a, b) if with_bn else None, unary, alpha, beta)
    ctx.sync()
    assert np.array_equal(got.download(), want.download())


@pytest.mark.parametrize("shape", [(2, 3, 8, 16), (3, 1, 4, 6), (1, 4, 16, 16), (2, 2, 5, 7), (2, 3, 3, 8)], ids=str)
def test_half_planes_to_four_channel_pixels(ctx, shape):
    """Half NCHW -> NHWC with four-half pixels (the packed first-layer form of the fp16 convolution): planes of a multiple
    of eight pixels take the eight-pixels-per-thread kernel, the others the general one; absent channels are zero."""
    x = np.random.default_rng(387).integers(1, 1 << 16, shape).astype(np.uint16)
    got = ctx.nchw_to_nhwc(ctx.array(x), 4, "f16").download()
    assert np.array_equal(got[..., :shape[1]], x.transpose(0, 2, 3, 1))
    assert not got[..., shape[1]:].any()


def _half(a):
    """Round-to-nearest-even to half storage, widened again (what a tensor of the fp16 path holds)."""
    return a.astype(np.float16)


@pytest.mark.parametrize("shape", [(2, 16, 20, 24), (1, 3, 5, 7), (1, 1, 1, 1)])
@pytest.mark.parametrize("kind,params", [("hardswish", dict(alpha=1 / 6, beta=0.5)), ("leakyrelu", dict(alpha=0.1)), ("sigmoid", {}),
                                         ("hardsigmoid", dict(alpha=0.2, beta=0.5))])
def test_unary_half_storage_bit_exact(ctx, kind, params, shape):
    """The fp16 activation layers in one pass: half in, the float formula, one rounding to half out."""
    case = cases.unary_case(325, kind, shape, **params)
    x16 = _half(case["x"])
    want = _half(cases.oracle_eval(dict(case, x=x16.astype(np.float32))))
    got = ctx.unary_f16(kind, ctx.array(x16.view(np.uint16)), params.get("alpha", 0.0), params.get("beta", 0.0)).download()
    assert np.array_equal(got, want.view(np.uint16))


def test_clip_half_storage_bit_exact(ctx):
    x16 = _half(np.random.default_rng(326).uniform(-4, 4, (2, 5, 9, 11)).astype(np.float32))
    got = ctx.unary_f16("clip", ctx.array(x16.view(np.uint16)), 0.5, 3.0).download()
    assert np.array_equal(got, _half(port.clip(x16.astype(np.float32), 0.5, 3.0)).view(np.uint16))


@pytest.mark.parametrize("shape", [(2, 16, 20, 24), (2, 5, 7, 9), (1, 3, 1, 1)])
def test_channelwise_half_storage_bit_exact(ctx, shape):
    """PReLU (per-channel and shared slope), BatchNorm and Input on half storage with float parameters."""
    for shared in (False, True):
        case = cases.prelu_case(327, shape, shared)
        x16 = _half(case["x"])
        got = ctx.channelwise_f16("prelu", ctx.array(x16.view(np.uint16)), ctx.array(case["slope"]), shared=shared).download()
        assert np.array_equal(got, _half(cases.oracle_eval(dict(case, x=x16.astype(np.float32)))).view(np.uint16))
    case = cases.batchnorm_case(328, shape)
    x16 = _half(case["x"])
    sqrt_var = np.sqrt((case["var"] + np.float32(case["eps"])).astype(np.float64)).astype(np.float32)
    a = (case["bias"] - case["slope"] * case["mean"] / sqrt_var).astype(np.float32)
    b = (case["slope"] / sqrt_var).astype(np.float32)
    got = ctx.channelwise_f16("batchnorm", ctx.array(x16.view(np.uint16)), ctx.array(a), ctx.array(b)).download()
    assert np.array_equal(got, _half(cases.oracle_eval(dict(case, x=x16.astype(np.float32)))).view(np.uint16))
    case = cases.input_case(329, (shape[0], 3) + shape[2:], [127.5, 120.0, 110.25], [1 / 128.0, 0.017, 0.0175])
    x16 = _half(case["x"])
    got = ctx.channelwise_f16("input", ctx.array(x16.view(np.uint16)), ctx.array(np.asarray(case["means"], np.float32)),
                              ctx.array(np.asarray(case["scales"], np.float32))).download()
    assert np.array_equal(got, _half(cases.oracle_eval(dict(case, x=x16.astype(np.float32)))).view(np.uint16))


def test_channelwise_more_planes_than_one_launch_takes(ctx):
    """A per-channel layer over more than 65535 (image, channel) planes (a launch's limit on block rows) runs as several
    launches of whole images: 3 images x 30000 channels of PReLU, float32 and half storage, against the closed form."""
    r = np.random.default_rng(333)
    x = r.normal(0, 1, (3, 30000, 2, 4)).astype(np.float32)
    slope = r.uniform(-0.5, 0.5, 30000).astype(np.float32)
    want = np.where(x >= 0, x, slope[None, :, None, None] * x).astype(np.float32)
    assert np.array_equal(ctx.channelwise_f32("prelu", ctx.array(x), ctx.array(slope)).download(), want)
    x16 = _half(x)
    want16 = _half(np.where(x16 >= 0, x16.astype(np.float32), slope[None, :, None, None] * x16.astype(np.float32)).astype(np.float32))
    got16 = ctx.channelwise_f16("prelu", ctx.array(x16.view(np.uint16)), ctx.array(slope)).download()
    assert np.array_equal(got16, want16.view(np.uint16))


def test_channelwise_nhwc_half_storage_bit_exact(ctx):
    """PReLU and BatchNorm on the NHWC half tensors the fp16 pipeline keeps between layers == the NCHW layer transposed."""
    shape = (2, 16, 9, 11)
    for shared in (False, True):
        case = cases.prelu_case(331, shape, shared)
        x16 = _half(case["x"])
        want = _half(cases.oracle_eval(dict(case, x=x16.astype(np.float32)))).view(np.uint16).transpose(0, 2, 3, 1)
        xd = ctx.array(np.ascontiguousarray(x16.view(np.uint16).transpose(0, 2, 3, 1)))
        got = ctx.channelwise_nhwc_f16("prelu", xd, ctx.array(case["slope"]), shared=shared).download()
        assert np.array_equal(got, want)
    case = cases.batchnorm_case(332, shape)
    x16 = _half(case["x"])
    sqrt_var = np.sqrt((case["var"] + np.float32(case["eps"])).astype(np.float64)).astype(np.float32)
    a = (case["bias"] - case["slope"] * case["mean"] / sqrt_var).astype(np.float32)
    b = (case["slope"] / sqrt_var).astype(np.float32)
    want = _half(cases.oracle_eval(dict(case, x=x16.astype(np.float32)))).view(np.uint16).transpose(0, 2, 3, 1)
    xd = ctx.array(np.ascontiguousarray(x16.view(np.uint16).transpose(0, 2, 3, 1)))
    assert np.array_equal(ctx.channelwise_nhwc_f16("batchnorm", xd, ctx.array(a), ctx.array(b)).download(), want)


@pytest.mark.parametrize("etype,n,coeffs", [(1, 2, None), (1, 3, [0.5, -1.25, 2.0]), (2, 3, None), (0, 3, None)])
def test_eltwise_bit_exact(ctx, etype, n, coeffs):
    case = cases.eltwise_case(320 + etype, (2, 16, 21, 23), etype, n, coeffs)
    assert np.array_equal(gpueval.gpu_eval(ctx, case), cases.oracle_eval(case))


def test_add_relu_and_empty_and_ragged(ctx):
    from excalibur_amd import hip
    for shape in [(1, 1, 1, 1), (1, 3, 5, 7), (2, 64, 40, 40)]:
        case = cases.binaryop_case(330, shape)
        a, b = (ctx.array(v) for v in case["xs"])
        assert np.array_equal(ctx.add_f32(a, b).download(), port.binaryop_add(*case["xs"]))
        assert np.array_equal(ctx.add_f32(a, b, relu=True).download(), port.relu(port.binaryop_add(*case["xs"])))
        assert np.array_equal(ctx.relu_f32(a).download(), port.relu(case["xs"][0]))
    # empty tensors are a no-op, not an error
    e = ctx.empty((0,), np.float32)
    assert hip.lib().exhip_add_f32(ctx.h, e.ptr, e.ptr, e.ptr, 0, 0) == 0


def test_innerproduct_within_1e4(ctx):
    for args in [(340, 4, 512, 1, 1, 1000), (341, 32, 64, 7, 7, 100), (342, 3, 5, 3, 3, 7)]:
        case = cases.fc_case(*args)
        assert cases.check_value(gpueval.gpu_eval(ctx, case), cases.oracle_eval(case), 1e-4) == 0


def test_error_paths_return_codes_not_crashes(ctx):
    from excalibur_amd import hip
    d = ctx.conv_desc(1, 20, 8, 8, 8, 3, 1, 1, c_stride=20)  # 20-byte pixels: not a multiple of 32
    assert hip.lib().exhip_conv_packed_bytes(__import__("ctypes").byref(d), hip.I8) == 0
    assert b"multiple of 32" in hip.lib().exhip_last_error()
    with pytest.raises(hip.ExhipError):
        ctx.eltwise_f32([ctx.array(np.zeros(4, np.float32))], 1)  # fewer than two inputs
    assert hip.lib().exhip_pool2d_nchw_f32(ctx.h, None, None, 1, 1, 4, 4, 2, 2, 0, 2, 2, 2, 2, 0, 0, 0, 0, 0) == 10001


def _sampled_acc(case, q_nchw, samples, rng):
    """Brute-force int32 accumulators at random output positions (numpy, a few thousand dot products)."""
    n, c, h, w = q_nchw.shape
    k, kh, kw, s = case["k"], case["kh"], case["kw"], case["stride"]
    pt, pb, pl, pr = (case["pad"],) * 4 if np.isscalar(case["pad"]) else case["pad"]
    oh, ow = (h + pt + pb - kh) // s + 1, (w + pl + pr - kw) // s + 1
    qp = np.zeros((n, c, h + pt + pb, w + pl + pr), np.int32)
    qp[:, :, pt:pt + h, pl:pl + w] = q_nchw
    wt = case["wt"].astype(np.int32)
    idx = [(rng.integers(n), rng.integers(k), rng.integers(oh), rng.integers(ow)) for _ in range(samples)]
    idx += [(0, 0, 0, 0), (n - 1, k - 1, oh - 1, ow - 1), (n - 1, 0, 0, ow - 1), (0, k - 1, oh - 1, 0)]
    vals = [int((qp[a, :, y * s:y * s + kh, x * s:x * s + kw] * wt[b]).sum()) for a, b, y, x in idx]
    return idx, vals


FULL = [
    ("cfg2_3x3", (400, 8, 128, 80, 80, 128, 3, 1, 1)),
    ("cfg2_1x1_k256", (401, 8, 128, 80, 80, 256, 1, 1, 0)),
    ("cfg2_3x3_k256", (404, 8, 128, 80, 80, 256, 3, 1, 1)),
    ("cfg2_1x1_k128", (405, 8, 128, 80, 80, 128, 1, 1, 0)),
    ("resnet_stage1_n8", (402, 8, 64, 160, 160, 64, 3, 1, 1)),
    ("resnet_stem_n4", (403, 4, 3, 640, 640, 64, 7, 2, 3)),
]


@pytest.mark.parametrize("name,args", FULL, ids=[f[0] for f in FULL])
def test_full_size_sampled_and_linear(ctx, name, args):
    """At the benchmark sizes: (a) sampled accumulators against brute force, (b) linearity in the weights:
    acc(w1) + acc(w2) == acc(w1 + w2), (c) the dequantized output recomputed from the GPU's own
    accumulators with the closed form fmaf(acc, s, b) + ReLU."""
    case = cases.conv_i8_case(*args, integer_x=True)
    rng = np.random.default_rng(args[0])
    got = gpueval.conv_i8(ctx, case)
    q = case["x"].astype(np.int32)
    idx, vals = _sampled_acc(case, q, 1500, rng)
    assert [int(got["acc"][i]) for i in idx] == vals
    w1 = (case["wt"].astype(np.int32) // 2).astype(np.int8)
    w2 = (case["wt"].astype(np.int32) - w1).astype(np.int8)
    a1 = gpueval.conv_i8(ctx, dict(case, wt=w1), want=("acc",))["acc"]
    a2 = gpueval.conv_i8(ctx, dict(case, wt=w2), want=("acc",))["acc"]
    assert np.array_equal(a1 + a2, got["acc"])
    want = port.dequant(got["acc"], case["ws"], case["fs"], case["bias"])
    assert np.array_equal(got["nchw"], port.relu(want))


@pytest.mark.parametrize("k,kernel", [(128, 3), (256, 3), (128, 1), (256, 1)], ids=["3x3k128", "3x3k256", "1x1k128", "1x1k256"])
def test_cfg2_requantized_int8_output_at_full_size(ctx, k, kernel):
    """8 x 128 x 80 x 80 -> K with ReLU and the next layer's quantizer in the epilogue (the fused int8 output): the int8
    NHWC tensor recomputed from the GPU's own accumulators (checked against brute force by the test above) with the closed
    form q8(relu(fmaf(acc, s, b)) * fs_out), every element; and with a float32 shortcut added before the ReLU."""
    case = cases.conv_i8_case(410 + k + kernel, 8, 128, 80, 80, k, kernel, 1, kernel // 2, act=0)
    fs_out = np.float32(23.7)
    r = np.random.default_rng(k + kernel)
    res = r.uniform(-3, 3, (8, 80, 80, k)).astype(np.float32)
    base = gpueval.conv_i8(ctx, case, want=("acc",))
    y = port.dequant(base["acc"], case["ws"], case["fs"], case["bias"])
    got = gpueval.conv_i8(ctx, case, fs_out=fs_out, post_relu=1, want=())
    assert np.array_equal(got["i8"], port.quantize(port.relu(y), fs_out).transpose(0, 2, 3, 1))
    got = gpueval.conv_i8(ctx, case, fs_out=fs_out, residual=res, post_relu=1, want=("nhwc",))
    z = port.relu(port.binaryop_add(y, np.ascontiguousarray(res.transpose(0, 3, 1, 2))))
    assert np.array_equal(got["nhwc"], z.transpose(0, 2, 3, 1))
    assert np.array_equal(got["i8"], port.quantize(z, fs_out).transpose(0, 2, 3, 1))


@pytest.mark.parametrize("shape,cs", [((2, 5, 7, 9), 32), ((1, 3, 6, 6), 4), ((2, 40, 5, 4), 64)], ids=str)
def test_quantizer_with_per_input_channel_scales(ctx, shape, cs):
    """quantize_float32_to_int8's second branch (src/Excalibur/operation_general_conv.cpp:596): one scale per input
    channel. Values at +-0.5 ties and beyond saturation included; pad channels are zero."""
    r = np.random.default_rng(shape[1])
    fs = r.uniform(0.5, 60, (shape[1],)).astype(np.float32)
    x = r.uniform(-4, 4, shape).astype(np.float32)
    x[0, :, 0, 0] = (np.float32(2.5) / fs).astype(np.float32)    # ties after scaling, where they are representable
    x[0, :, 0, 1] = np.float32(1000.0)
    x[0, :, 0, 2] = np.float32(-1000.0)
    got = ctx.quantize_nchw_to_nhwc_i8(ctx.array(x), 0.0, cs, fs_per_channel=ctx.array(fs)).download()
    want = port.quantize(x, fs).transpose(0, 2, 3, 1)
    assert np.array_equal(got[..., :shape[1]], want)
    assert not got[..., shape[1]:].any()


@pytest.fixture(params=[1, 0, 3])
def splits(request):
    """The convolution's split reduction: never (1), the planner's choice (0), three groups per tile where the layer allows."""
    from excalibur_amd import hip
    hip.set_option("force_splits", request.param)
    yield request.param
    hip.set_option("force_splits", 0)


SPLIT_SHAPES = [
    # seed, n, c, h, w, k, kernel, stride, pad: launches of a few tiles with several channel chunks
    (600, 1, 256, 14, 14, 64, 3, 1, 1),
    (601, 1, 512, 7, 9, 128, 3, 1, 1),
    (602, 2, 384, 6, 6, 72, 1, 1, 0),      # 1x1: three chunks to a part; ragged channel count (general epilogue)
    (603, 1, 128, 20, 20, 256, 3, 2, 1),
]


@pytest.mark.parametrize("args", SPLIT_SHAPES, ids=[f"s{a[0]}" for a in SPLIT_SHAPES])
def test_conv_split_reduction_int8_bit_exact(ctx, args, splits):
    """Few tiles, deep reduction: the tile's channel chunks are reduced by several groups and the int32 parts added by
    the last one to arrive. Accumulators, float output and the fused shortcut / requantized outputs equal the oracle's
    whichever way the launch is split; run twice in a row (the arrival counters must be back at zero)."""
    case = cases.conv_i8_case(*args, act=0)
    g = cases.geom_of(case)
    want_y, want_acc = port.conv2d_i8(case["x"], case["wt"], case["bias"], case["ws"], case["fs"], 0, g, want_acc=True)
    for _ in range(2):
        got = gpueval.conv_i8(ctx, case)
        assert np.array_equal(got["acc"], want_acc)
        assert np.array_equal(got["nchw"], want_y)
    if args[5] % 64 == 0:
        r = np.random.default_rng(args[0] + 1)
        res = r.uniform(-4, 4, want_y.shape).astype(np.float32)
        fs_out = np.float32(13.1)
        z = port.relu(port.binaryop_add(want_y, res))
        fused = gpueval.conv_i8(ctx, case, fs_out=fs_out, residual=np.ascontiguousarray(res.transpose(0, 2, 3, 1)), post_relu=1, want=("nhwc",))
        assert np.array_equal(fused["nhwc"], z.transpose(0, 2, 3, 1))
        assert np.array_equal(fused["i8"], port.quantize(z, fs_out).transpose(0, 2, 3, 1))


def test_conv_split_reduction_many_tiles_equals_the_unsplit_launch(ctx):
    """128 tiles x 2 groups each (8 x 512 x 20 x 20 -> 512, eight chunks): every accumulator and every output of the split
    launch equals the unsplit launch's, which the tests above pin against the oracle. The forced split of three is clamped
    to what the fixed scratch holds."""
    from excalibur_amd import hip
    case = cases.conv_i8_case(620, 8, 512, 20, 20, 512, 3, 1, 1, act=0)
    hip.set_option("force_splits", 1)
    try:
        want = gpueval.conv_i8(ctx, case)
        hip.set_option("force_splits", 3)
        got = gpueval.conv_i8(ctx, case)
    finally:
        hip.set_option("force_splits", 0)
    for name in ("acc", "nchw"):
        bad = np.flatnonzero(got[name].ravel() != want[name].ravel())
        assert bad.size == 0, f"{name}: first of {bad.size} mismatches at flat index {bad[0]}"


def test_conv_split_reduction_float_within_tolerance(ctx, splits):
    """The benchmark set's single float32 layer (1 x 64 x 56 x 56 -> 64, 3x3, bias, ReLU: 13 tiles on 256 CUs) and a half
    layer: the parts are added in split order, so a launch gives the same bits every time, within 1e-4 / 2e-3 of the oracle."""
    case = cases.conv_f32_case(610, 1, 64, 56, 56, 64, 3, 1, 1)
    want = cases.oracle_eval(case)
    a = gpueval.conv_f32(ctx, case)
    assert cases.check_value(a, want, 1e-4) == 0
    assert np.array_equal(a, gpueval.conv_f32(ctx, case))
    case = cases.conv_f32_case(611, 1, 256, 14, 14, 128, 3, 1, 1)
    x16 = case["x"].astype(np.float16)
    want = cases.oracle_eval(dict(case, x=x16.astype(np.float32)))
    h = gpueval.conv_f16(ctx, case, x16.view(np.uint16))
    assert cases.check_value(h.view(np.float16).astype(np.float32), want, 2e-3) == 0
    assert np.array_equal(h, gpueval.conv_f16(ctx, case, x16.view(np.uint16)))


@pytest.mark.parametrize("channels,strides,out_stride,with_bn,unary,alpha,beta", [
    ((32, 32), (32, 32), 64, True, "leakyrelu", 0.1, 0.0),        # the detection block: Concat -> BatchNorm -> LeakyRelu
    ((64, 32, 32), (64, 64, 32), 128, True, None, 0.0, 0.0),      # an input whose stride holds pad channels
    ((24, 8), (32, 8), 32, False, "hardswish", 1 / 6, 0.5),
    ((20,), (32,), 32, False, None, 0.0, 0.0),                    # one input: the quantizer on an NHWC blob, pad channels zero
    ((16,), (16,), 32, True, "clip", -0.5, 1.5),
], ids=["cat-bn-leaky", "cat-bn", "cat-hardswish", "quantizer", "bn-clip"])
def test_concat_batchnorm_activation_float32_nhwc_with_int8_copy(ctx, channels, strides, out_stride, with_bn, unary, alpha, beta):
    """The int8 executor's glue kernel against the float32 layers' own kernels (Concat as a copy, BatchNorm and the
    activation on NCHW) and the oracle's quantizer: the float32 NHWC result and the int8 copy q8(v * fs), pad channels zero."""
    r = np.random.default_rng(390)
    n, h, w = 2, 7, 9
    arrays = []
    for c, st in zip(channels, strides):
        a = r.normal(0, 2, (n, h, w, st)).astype(np.float32)
        a[..., c:] = np.nan    # pad channels of an input are never read
        arrays.append(a)
    total = sum(channels)
    pa = r.normal(0, 0.5, total).astype(np.float32)
    pb = r.uniform(0.5, 2, total).astype(np.float32)
    want = np.ascontiguousarray(np.concatenate([a[..., :c] for a, c in zip(arrays, channels)], axis=3).transpose(0, 3, 1, 2))
    dev = ctx.array(want)
    if with_bn:
        dev = ctx.channelwise_f32("batchnorm", dev, ctx.array(pa), ctx.array(pb))
    if unary:
        dev = ctx.unary_f32(unary, dev, alpha, beta)
    ctx.sync()
    want = dev.download()
    fs = np.float32(9.3)
    for want_f32 in (True, False):
        y_f, y_q = ctx.concat_nhwc_f32([ctx.array(a) for a in arrays], channels, out_stride, (ctx.array(pa), ctx.array(pb)) if with_bn else None,
                                       unary, alpha, beta, want_f32=want_f32, fs_out=fs)
        ctx.sync()
        if want_f32:
            got = y_f.download()
            assert np.array_equal(got[..., :total].view(np.uint32), want.transpose(0, 2, 3, 1).view(np.uint32))
            assert not got[..., total:].any()
        q = y_q.download()
        assert np.array_equal(q[..., :total], port.quantize(want, fs).transpose(0, 2, 3, 1))
        assert not q[..., total:].any()


_POST_LAYERS = {
    "hardswish": (1 / 6, 0.5, lambda v: port.hardswish(v, 1 / 6, 0.5)),
    "leakyrelu": (0.1, 0.0, lambda v: port.leakyrelu(v, 0.1)),
    "hardsigmoid": (0.2, 0.5, lambda v: port.hardsigmoid(v, 0.2, 0.5)),
    "clip": (-0.75, 1.25, lambda v: port.clip(v, -0.75, 1.25)),
}


@pytest.mark.parametrize("shortcut", ["none", "front", "behind"])
@pytest.mark.parametrize("post_op", list(_POST_LAYERS))
@pytest.mark.parametrize("c,k,kernel", [(32, 64, 3), (32, 128, 1), (32, 48, 3), (64, 64, 3), (128, 128, 3), (32, 32, 3), (64, 96, 3), (16, 160, 3)],
                         ids=["k64-3x3", "k128-1x1", "k48-3x3", "c64-k64-3x3", "c128-k128-3x3", "k32-3x3", "k96-3x3", "k160-3x3"])
def test_conv_int8_activation_layer_and_sum_in_the_epilogue(ctx, c, k, kernel, post_op, shortcut):
    """int8 convolution -> activation layer [-> sum], or -> sum -> activation layer, in one launch against the oracle's
    layers one after the other: float32 NHWC / NCHW results and the requantized int8 copy, bit for bit. Output channel
    counts that are multiples of 32 take the epilogue with the per-wave tiles (32, 96 and 160: the last 64-channel slab is
    half empty), 48 the general one; with 64 / 128 input channels and without the NCHW result the 3x3 layers run in the lean
    kernel (checked in a second launch)."""
    case = cases.conv_i8_case(640 + k + c, 2, c, 11, 13, k, kernel, 1, kernel // 2, act=0)
    y = port.conv2d_i8(case["x"], case["wt"], case["bias"], case["ws"], case["fs"], 0, cases.geom_of(case))
    res = np.random.default_rng(641).uniform(-2, 2, y.shape).astype(np.float32)
    alpha, beta, layer = _POST_LAYERS[post_op]
    want = y
    if shortcut == "front":
        want = port.binaryop_add(want, res)
    want = layer(want)
    if shortcut == "behind":
        want = port.binaryop_add(want, res)
    fs_out = np.float32(11.7)
    ks = (k + 31) // 32 * 32
    res_nhwc = None
    if shortcut != "none":
        res_nhwc = np.zeros(y.shape[:1] + y.shape[2:] + (ks,), np.float32)
        res_nhwc[..., :k] = res.transpose(0, 2, 3, 1)
    got = gpueval.conv_i8(ctx, case, fs_out=fs_out, residual=res_nhwc, want=("nhwc", "nchw"), post_op=post_op, post_alpha=alpha,
                          post_beta=beta, residual_last=1 if shortcut == "behind" else 0)
    assert np.array_equal(got["nchw"].view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got["nhwc"][..., :k].view(np.uint32), want.transpose(0, 2, 3, 1).view(np.uint32))
    assert np.array_equal(got["i8"][..., :k], port.quantize(want, fs_out).transpose(0, 2, 3, 1))
    # the NHWC results alone (what a network's inner layers ask for): the lean and pointwise kernels take these launches
    got = gpueval.conv_i8(ctx, case, fs_out=fs_out, residual=res_nhwc, want=("nhwc",), post_op=post_op, post_alpha=alpha,
                          post_beta=beta, residual_last=1 if shortcut == "behind" else 0)
    assert np.array_equal(got["nhwc"][..., :k].view(np.uint32), want.transpose(0, 2, 3, 1).view(np.uint32))
    assert np.array_equal(got["i8"][..., :k], port.quantize(want, fs_out).transpose(0, 2, 3, 1))


@pytest.mark.parametrize("shape", [(2, 3, 16, 24), (1, 3, 6, 10), (3, 3, 32, 32)], ids=str)
def test_input_focus_quantizer_in_one_pass(ctx, shape):
    """The front of an int8 detection network (Input layer, YoloV5Focus, the first convolution's quantizer) in one kernel
    against the oracle's three layers; int8 NHWC pixels of 32 bytes, 12 of them channels."""
    r = np.random.default_rng(395)
    x = r.uniform(0, 255, shape).astype(np.float32)
    means, scales, fs = [10.0, 20.5, 30.25], [0.0039215, 0.004, 0.0038], np.float32(113.0)
    want = port.quantize(port.focus(port.input_layer(x, means, scales)), fs).transpose(0, 2, 3, 1)
    got = ctx.input_focus_quantize(ctx.array(x), means, scales, fs)
    assert got is not None
    got = got.download()
    assert np.array_equal(got[..., :12], want)
    assert not got[..., 12:].any()
    assert np.count_nonzero(want) > want.size // 2
    # shapes the kernel does not take are refused, not mangled
    assert ctx.input_focus_quantize(ctx.array(x[:, :, :-1]), means, scales, fs) is None
    assert ctx.input_focus_quantize(ctx.array(x), means, scales, fs, c_stride=64) is None


@pytest.mark.parametrize("n,h,w,groups,per_group,stride", [(2, 8, 8, 3, 85, 256), (1, 5, 3, 3, 7, 32), (3, 4, 4, 1, 16, 16)], ids=str)
def test_detection_head_regrouping(ctx, n, h, w, groups, per_group, stride):
    """Reshape [n, G * J, h, w] -> [n, G, J, h * w] and Transpose of the last two axes, from the float32 NHWC tensor: the
    oracle's transpose of the reshaped NCHW tensor."""
    r = np.random.default_rng(396)
    k = groups * per_group
    nhwc = r.normal(0, 1, (n, h, w, stride)).astype(np.float32)
    nchw = np.ascontiguousarray(nhwc[..., :k].transpose(0, 3, 1, 2))
    want = port.transpose_hw(nchw.reshape(n, groups, per_group, h * w))
    got = ctx.nhwc_to_grouped_f32(ctx.array(nhwc), k, groups).download()
    assert got.shape == want.shape
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("kernel,stride,pad,h,w", [(2, 2, 0, 12, 14), (3, 2, 1, 13, 9), (5, 1, 2, 10, 10), (13, 1, 6, 8, 7), (2, 2, 0, 7, 9)], ids=str)
def test_max_pooling_on_int8_nhwc(ctx, kernel, stride, pad, h, w):
    """MAX pooling on an int8 NHWC tensor against the oracle's pooling of the same values as floats (the quantizer is
    monotone: pooling the quantized tensor gives the quantized pooled tensor); clipped windows, ragged sizes, pad channels
    carried along."""
    r = np.random.default_rng(397)
    n, c, cs = 2, 24, 32
    x = r.integers(-128, 128, (n, h, w, cs)).astype(np.int8)
    want = port.pool2d(np.ascontiguousarray(x[..., :c].transpose(0, 3, 1, 2)).astype(np.float32), port.POOL_MAX, kernel, stride, pad)
    oh, ow = want.shape[2:]
    got = ctx.maxpool2d_nhwc_i8(ctx.array(x), c, kernel, stride, (pad, pad), oh, ow).download()
    assert np.array_equal(got[..., :c].astype(np.float32), want.transpose(0, 2, 3, 1))
    # and through the quantizer: q8(max(v) * fs) == max(q8(v * fs))
    v = r.normal(0, 3, (n, c, h, w)).astype(np.float32)
    fs = np.float32(21.0)
    q = np.zeros((n, h, w, cs), np.int8)
    q[..., :c] = port.quantize(v, fs).transpose(0, 2, 3, 1)
    got = ctx.maxpool2d_nhwc_i8(ctx.array(q), c, kernel, stride, (pad, pad), oh, ow).download()
    assert np.array_equal(got[..., :c], port.quantize(port.pool2d(v, port.POOL_MAX, kernel, stride, pad), fs).transpose(0, 2, 3, 1))


def test_quantizer_and_clamped_activations_at_the_edges_of_their_ranges(ctx):
    """float32_to_int8 and the activations that clamp (HardSwish, HardSigmoid) on the values where their selects turn:
    zeros of both signs, denormals, the halves around every rounding step near the saturation points, values beyond the
    int32 range and infinities -- against the oracle, bit for bit. (NaN is left out: the reference's conversion of it is
    undefined behaviour.)"""
    edge = [0.0, -0.0, 1e-45, -1e-45, 1e-39, -1e-39, 0.49999997, 0.5, 0.50000006, -0.49999997, -0.5, -0.50000006, 1.4999999, 1.5, -1.5,
            126.49999, 126.5, 127.0, 127.49999, 127.5, 128.0, 128.5, 1000.0, -127.5, -128.0, -128.49999, -128.5, -129.0, -1000.0,
            2147483520.0, 2147483648.0, -2147483648.0, 4294967296.0, 3e38, -3e38, np.inf, -np.inf,
            -3.0, -2.9999998, -3.0000002, 3.0, 2.9999998, 3.0000002, -2.5, 2.5, 6.0, -6.0]
    r = np.random.default_rng(77)
    x = np.concatenate([np.array(edge, np.float32), r.uniform(-140, 140, 4096).astype(np.float32),
                        (r.integers(-130, 131, 2048) + r.choice([-0.5, 0.5], 2048)).astype(np.float32)]).astype(np.float32)
    x = np.ascontiguousarray(x.reshape(1, 1, 1, -1))
    for fs in (1.0, 0.37, 3.0):
        q = ctx.quantize_nchw_to_nhwc_i8(ctx.array(x), fs, 32)
        ctx.sync()
        assert np.array_equal(q.download()[0, 0, :, 0], port.quantize(x, np.float32(fs))[0, 0, 0])
    for name, fn, a, b in (("hardswish", port.hardswish, 1 / 6, 0.5), ("hardsigmoid", port.hardsigmoid, 0.2, 0.5),
                           ("hardswish", port.hardswish, 0.5, -0.25)):
        y = ctx.unary_f32(name, ctx.array(x), a, b)
        ctx.sync()
        want = fn(x, a, b)
        got = y.download()
        ok = ~np.isnan(want)     # inf * 0 is NaN on both sides; payloads are not compared
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32)), name


@pytest.mark.parametrize("shape,k,levels", [((2, 20, 20, 64), 5, 3), ((1, 7, 11, 32), 5, 3), ((3, 30, 32, 16), 3, 2), ((1, 1, 9, 16), 5, 1),
                                            ((1, 40, 40, 32), 5, 3)],
                         ids=["spp-20x20", "ragged-7x11", "k3-two-levels", "one-row", "40x40-level-by-level"])
def test_int8_pooling_pyramid_in_one_launch(ctx, shape, k, levels):
    """y1 = pool_k(x), y2 = pool_k(y1), y3 = pool_k(y2) on an int8 NHWC tensor in one launch, against the oracle's MAX pooling
    of x with windows k, 2k - 1, 3k - 2 (stride 1, "same" padding): the SPP block's three Pooling layers. The 40 x 40 map does
    not fit a group's LDS and goes level by level through the window kernel."""
    n, h, w, c = shape
    x = np.random.default_rng(1200 + h).integers(-128, 128, shape).astype(np.int8)
    ys = ctx.maxpool_same_pyramid_nhwc_i8(ctx.array(x), c, k, levels)
    ctx.sync()
    xf = np.ascontiguousarray(x.astype(np.float32).transpose(0, 3, 1, 2))
    for level, y in enumerate(ys):
        win = (level + 1) * (k - 1) + 1
        want = port.pool2d(xf, 0, win, 1, win // 2).transpose(0, 2, 3, 1)
        assert np.array_equal(y.download().astype(np.float32), want), f"level {level + 1}"
