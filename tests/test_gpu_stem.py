"""The stem in one kernel (csrc/stem_i8.hip): quantizer + first convolution + 3x3 stride-2 max pooling, against the
oracle's three layers and against the library's own two-launch form."""
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


STEM_SHAPES = [
    # seed, n, c, h, w, k, kernel, pad, pool pad, pool pad_mode
    (950, 2, 3, 150, 134, 64, 7, 3, 1, 1),    # ragged pooled patches on the right and at the bottom
    (951, 1, 3, 64, 64, 64, 7, 3, 0, 0),      # no pool padding, clipped windows ("full" output size)
    (952, 3, 3, 30, 26, 128, 7, 3, 1, 1),     # image smaller than a patch, two slabs
    (953, 2, 4, 96, 120, 64, 5, 2, 1, 1),     # four channels, 5x5
    (954, 1, 3, 70, 58, 64, 3, 1, 1, 1),      # 3x3
    (955, 2, 3, 224, 224, 64, 7, 3, 1, 1),    # interior patches
]


@pytest.mark.parametrize("act", [1, 0], ids=["relu", "linear"])
@pytest.mark.parametrize("groups", [0, 1], ids=["resident", "walk"])
@pytest.mark.parametrize("args", STEM_SHAPES, ids=[f"s{a[0]}" for a in STEM_SHAPES])
def test_stem_one_kernel_bit_exact(ctx, args, act, groups):
    seed, n, c, h, w, k, kernel, pad, ppad, pad_mode = args
    case = cases.conv_i8_case(seed, n, c, h, w, k, kernel, 2, pad, act=act)
    case["ws"] = np.abs(case["ws"])
    fs_out = np.float32(23.5)
    y = cases.oracle_eval(case)
    want = port.pool2d(y, port.POOL_MAX, 3, 2, ppad, pad_mode=pad_mode)
    poh, pow_ = want.shape[2:]
    d = ctx.conv_desc(n, c, h, w, k, kernel, 2, pad, act, 4, k, 0, float(fs_out))
    wp = ctx.pack_conv_weights(d, hip.I8, case["wt"])
    scale = ctx.array(gpueval.dequant_scales(case["ws"], case["fs"], k))
    bias = ctx.array(case["bias"])
    x = ctx.array(case["x"])
    yf = ctx.empty((n, poh, pow_, k), np.float32)
    yq = ctx.empty((n, poh, pow_, k), np.int8)
    hip.set_option("lean_groups", groups)
    try:
        taken = ctx.stem_f32_conv_i8_maxpool3x3s2(d, ppad, poh, pow_, x, float(case["fs"]), wp, scale, True, bias, yq, yf)
        ctx.sync()
    finally:
        hip.set_option("lean_groups", 0)
    assert taken, "the one-kernel stem refused a shape it is meant for"
    got_f, got_q = yf.download(), yq.download()
    assert np.array_equal(got_f, want.transpose(0, 2, 3, 1)), f"{np.count_nonzero(got_f != want.transpose(0, 2, 3, 1))} float values differ"
    assert np.array_equal(got_q, port.quantize(want, fs_out).transpose(0, 2, 3, 1))
    # the library's two launches give the same bytes
    xq = ctx.quantize_nchw_to_nhwc_i8(x, case["fs"], 4)
    yf2 = ctx.empty((n, poh, pow_, k), np.float32)
    ctx.conv2d_i8_maxpool3x3s2(d, ppad, poh, pow_, xq, wp, scale, bias, None, yf2)
    ctx.sync()
    assert np.array_equal(yf2.download(), got_f)


def test_stem_one_kernel_refuses_what_it_cannot_do(ctx):
    case = cases.conv_i8_case(960, 1, 3, 40, 40, 64, 7, 2, 3, act=1)
    d = ctx.conv_desc(1, 3, 40, 40, 64, 7, 2, 3, 1, 4, 64, 0, 10.0)
    wp = ctx.pack_conv_weights(d, hip.I8, case["wt"])
    scale = ctx.array(gpueval.dequant_scales(case["ws"], case["fs"], 64))
    x = ctx.array(case["x"])
    yq = ctx.empty((1, 10, 10, 64), np.int8)
    # negative scales are not stated to be absent: the maximum on accumulators would be wrong
    assert ctx.stem_f32_conv_i8_maxpool3x3s2(d, 1, 10, 10, x, float(case["fs"]), wp, scale, False, None, yq, None) is False
    d1 = ctx.conv_desc(1, 3, 40, 40, 64, 7, 1, 3, 1, 4, 64, 0, 10.0)   # stride 1
    assert ctx.stem_f32_conv_i8_maxpool3x3s2(d1, 1, 20, 20, x, float(case["fs"]), wp, scale, True, None, yq, None) is False
