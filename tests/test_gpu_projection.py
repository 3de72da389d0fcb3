"""A residual block's closing layers in one kernel (exhip_conv2d_i8_projection: 3x3 convolution + 1x1 projection of the
block's input + sum + ReLU) against the CPU oracle's four layers and against the library's own two-call form."""
import numpy as np
import pytest

from excalibur_amd import hip
from oracle import port
from tests import cases, gpueval

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
    defaults = dict(lean=4, lean_cfg=0, lean_groups=0, force_splits=0, force_variant=-1)
    for name in changed:
        hip.set_option(name, defaults[name])


SHAPES = [
    # seed, n, k (channels of the 3x3 layer, in and out), h, w (output), c0 (projection's input channels), stride
    (960, 2, 128, 24, 24, 64, 2),     # two chunks + one projection chunk, border patches only
    (961, 1, 128, 40, 36, 64, 2),     # interior and ragged patches
    (962, 2, 256, 20, 20, 128, 2),    # four chunks + two, four slabs
    (963, 1, 512, 20, 20, 256, 2),    # eight chunks + four (three slice buffers, one tile buffer)
    (964, 3, 128, 9, 11, 64, 2),      # an image smaller than a patch
    (965, 2, 128, 24, 24, 64, 1),     # a projection without downsampling
    (966, 1, 64, 40, 40, 64, 2),      # one chunk of each: the streamed form where the resident filter would serve
    (967, 1, 128, 13, 17, 128, 2),    # odd sizes: the projection's input is 25 x 33
]


def block_case(seed, n, k, h, w, c0, stride):
    main = cases.conv_i8_case(seed, n, k, h, w, k, 3, 1, 1, act=0)
    ph, pw = (h - 1) * stride + 1, (w - 1) * stride + 1
    if seed != 967 and stride == 2:
        ph, pw = h * 2, w * 2   # the usual even size, whose last row and column the 1x1 layer never reads
    proj = cases.conv_i8_case(seed + 1000, n, c0, ph, pw, k, 1, stride, 0, act=0)
    return main, proj


def oracle_block(main, proj, fs_out):
    y2 = port.conv2d_i8(main["x"], main["wt"], main["bias"], main["ws"], main["fs"], 0, cases.geom_of(main))
    short = port.conv2d_i8(proj["x"], proj["wt"], proj["bias"], proj["ws"], proj["fs"], 0, cases.geom_of(proj))
    z = port.relu(port.binaryop_add(y2, short))
    return z.transpose(0, 2, 3, 1), port.quantize(z, fs_out).transpose(0, 2, 3, 1)


def device_operands(ctx, case, post_relu, fs_out):
    n, c, h, w = case["x"].shape
    k = case["k"]
    d = ctx.conv_desc(n, c, h, w, k, (case["kh"], case["kw"]), case["stride"], case["pad"], case["act"], c, k, post_relu, float(fs_out))
    xq = ctx.quantize_nchw_to_nhwc_i8(ctx.array(case["x"]), case["fs"], c)
    wp = ctx.pack_conv_weights(d, hip.I8, case["wt"])
    scale = ctx.array(gpueval.dequant_scales(case["ws"], case["fs"], k))
    bias = ctx.array(case["bias"]) if case["bias"] is not None else None
    return d, xq, wp, scale, bias


def run_block(ctx, main, proj, fs_out, fused):
    n, k, h, w = main["x"].shape
    d, x, wp, scale, bias = device_operands(ctx, main, 1, fs_out)
    dp, xp, wpp, scalep, biasp = device_operands(ctx, proj, 0, 0.0)
    y_i8 = ctx.empty((n, h, w, k), np.int8)
    y_f = ctx.empty((n, h, w, k), np.float32)
    if fused:
        if not ctx.conv2d_i8_projection(d, x, wp, scale, bias, dp, xp, wpp, scalep, biasp, y_i8, y_f):
            return None
    else:
        short = ctx.empty((n, h, w, k), np.float32)
        ctx.conv2d_i8(dp, xp, wpp, scalep, biasp, None, None, short, None, None)
        ctx.conv2d_i8(d, x, wp, scale, bias, short, y_i8, y_f, None, None)
    ctx.sync()
    return y_f.download(), y_i8.download()


@pytest.mark.parametrize("cfg,groups", [(0, 0), (1, 0), (2, 0), (1, 2), (2, 1)], ids=["auto", "a2w2", "a1w3", "walk2-a2w2", "walk1-a1w3"])
@pytest.mark.parametrize("args", SHAPES, ids=[f"s{a[0]}" for a in SHAPES])
def test_projection_kernel_bit_exact(ctx, options, args, cfg, groups):
    main, proj = block_case(*args)
    fs_out = np.float32(10.3)
    want_f, want_q = oracle_block(main, proj, fs_out)
    options("force_splits", 1)   # small launches would otherwise split their reduction, which this kernel does not do
    options("force_variant", 0)  # and would plan 128-channel slabs: the kernel reads the 64-channel packing of the large layers
    if cfg:
        options("lean", 1)
        options("lean_cfg", cfg)
    options("lean_groups", groups)
    got = run_block(ctx, main, proj, fs_out, fused=True)
    assert got is not None, "the library refused a shape the kernel is meant to take"
    assert np.array_equal(got[0], want_f), f"float32: {np.count_nonzero(got[0] != want_f)} of {want_f.size} values differ"
    assert np.array_equal(got[1], want_q), f"int8: {np.count_nonzero(got[1] != want_q)} of {want_q.size} values differ"


def test_projection_kernel_equals_the_two_calls_on_a_stage_sized_launch(ctx):
    """8 x 128 x 80 x 80 with a 64-channel 160 x 160 block input: persistent groups that walk several patches of both slabs."""
    main, proj = block_case(970, 8, 128, 80, 80, 64, 2)
    fs_out = np.float32(7.9)
    want = run_block(ctx, main, proj, fs_out, fused=False)
    got = run_block(ctx, main, proj, fs_out, fused=True)
    assert got is not None
    assert np.array_equal(got[0], want[0])
    assert np.array_equal(got[1], want[1])


def test_projection_entry_point_refuses_what_the_kernel_does_not_take(ctx, options):
    main, proj = block_case(971, 1, 128, 24, 24, 64, 2)
    fs_out = np.float32(5.0)
    options("force_splits", 1)
    options("force_variant", 0)
    n, k, h, w = main["x"].shape
    d, x, wp, scale, bias = device_operands(ctx, main, 1, fs_out)
    dp, xp, wpp, scalep, biasp = device_operands(ctx, proj, 0, 0.0)
    y_i8 = ctx.empty((n, h, w, k), np.int8)
    y_f = ctx.empty((n, h, w, k), np.float32)
    assert ctx.conv2d_i8_projection(d, x, wp, scale, bias, dp, xp, wpp, scalep, biasp, y_i8, y_f)
    # an activation on the projection, a 3x3 layer without the closing ReLU, the lean kernel switched off
    dp_relu = ctx.conv_desc(n, 64, 48, 48, k, 1, 2, 0, 1, 64, k, 0, 0.0)
    assert not ctx.conv2d_i8_projection(d, x, wp, scale, bias, dp_relu, xp, wpp, scalep, biasp, y_i8, y_f)
    d_plain = ctx.conv_desc(n, k, h, w, k, 3, 1, 1, 0, k, k, 0, float(fs_out))
    assert not ctx.conv2d_i8_projection(d_plain, x, wp, scale, bias, dp, xp, wpp, scalep, biasp, y_i8, y_f)
    options("lean", 0)
    assert not ctx.conv2d_i8_projection(d, x, wp, scale, bias, dp, xp, wpp, scalep, biasp, y_i8, y_f)
    ctx.sync()
