"""The fp16 3x3 stride-1 layers on the lean kernel (conv_i8_lean.hip, E_HALF) against the general kernel, whose fp16
epilogue it repeats on the same packed weights and in the same order of the float32 sums: bit for bit. (The general
kernel's fp16 results are checked against the CPU oracle in test_gpu_ops.py and on whole networks.)"""
import numpy as np
import pytest

from excalibur_amd import hip

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
    defaults = dict(lean_f16=1, lean_groups=0, force_splits=0, force_variant=-1, debug_plan=0)
    for name in changed:
        hip.set_option(name, defaults[name])


def run(ctx, n, c, h, w, k, x, wt, bias, res, act=0, post_relu=0, post_op=None, alpha=0.0, beta=0.0, residual_last=0):
    d = ctx.conv_desc(n, c, h, w, k, 3, 1, 1, act, c, k, post_relu, 0.0, post_op, alpha, beta, residual_last)
    xd = ctx.array(x.view(np.uint16))
    wp = ctx.pack_conv_weights(d, hip.F16, wt.view(np.uint16))
    bd = ctx.array(bias) if bias is not None else None
    rd = ctx.array(res.view(np.uint16)) if res is not None else None
    y = ctx.array(np.full((n, h, w, k), 0x7e00, np.uint16))   # NaN bits: what the kernel leaves alone shows
    ctx.conv2d_f16(d, xd, wp, bd, rd, y, None, None)
    ctx.sync()
    return y.download()


SHAPES = [
    # seed, n, c, h, w, k, shortcut (0 none, 1 in front of the activation, 2 behind it), act, post_relu, post_op
    (800, 2, 32, 40, 36, 64, 0, 0, 0, "hardswish"),     # one chunk: the resident filter; interior and ragged patches
    (801, 1, 64, 80, 80, 64, 2, 0, 0, "hardswish"),     # the detection topology's bottleneck: sum behind the activation
    (802, 2, 128, 24, 24, 128, 1, 0, 1, None),          # four chunks, two slabs; residual block: sum, then ReLU
    (803, 1, 256, 20, 20, 256, 0, 1, 0, None),          # eight chunks: persistent groups with three slice buffers
    (804, 3, 64, 9, 11, 128, 0, 0, 0, "leakyrelu"),     # images smaller than a patch
    (805, 1, 320, 13, 17, 64, 2, 0, 0, "clip"),         # ten chunks, odd sizes
    (806, 2, 96, 33, 31, 192, 0, 0, 0, None),           # three chunks, three slabs
]
PARAMS = {"hardswish": (1 / 6, 0.5), "leakyrelu": (0.1, 0.0), "clip": (-0.25, 0.5), None: (0.0, 0.0)}


@pytest.mark.parametrize("form,groups", [(1, 0), (2, 0), (3, 0), (4, 0), (4, 2), (3, 1)],
                         ids=["auto", "one-shot", "three-slices", "two-slices", "walk2-two-slices", "walk1-three-slices"])
@pytest.mark.parametrize("args", SHAPES, ids=[f"s{a[0]}" for a in SHAPES])
def test_lean_fp16_repeats_the_general_kernel_bit_for_bit(ctx, options, capfd, args, form, groups):
    seed, n, c, h, w, k, shortcut, act, post_relu, post_op = args
    r = np.random.default_rng(seed)
    x = r.uniform(-1, 1, (n, h, w, c)).astype(np.float16)
    wt = r.normal(0, 0.05, (k, c, 3, 3)).astype(np.float16)
    bias = r.normal(0, 0.1, k).astype(np.float32)
    res = r.uniform(-1, 1, (n, h, w, k)).astype(np.float16) if shortcut else None
    alpha, beta = PARAMS[post_op]
    options("force_splits", 1)    # a small launch of the general kernel would split its sum, which changes its order
    options("force_variant", 0)   # the 64-channel-slab packing both kernels read
    options("lean_f16", 0)
    want = run(ctx, n, c, h, w, k, x, wt, bias, res, act, post_relu, post_op, alpha, beta, 1 if shortcut == 2 else 0)
    assert not np.any(want == 0x7e00)
    options("lean_f16", form)
    options("lean_groups", groups)
    options("debug_plan", 1)
    capfd.readouterr()
    got = run(ctx, n, c, h, w, k, x, wt, bias, res, act, post_relu, post_op, alpha, beta, 1 if shortcut == 2 else 0)
    options("debug_plan", 0)
    assert "lean fp16:" in capfd.readouterr().err, "the layer did not take the lean kernel"
    assert np.array_equal(got, want), f"{np.count_nonzero(got != want)} of {want.size} halves differ"
