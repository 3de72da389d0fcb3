"""The lean 3x3 stride-1 int8 kernel (csrc/conv_i8_lean.hip) against the CPU oracle and against the general kernel:
every staging configuration, persistent groups that walk many patches, one group per patch, border and ragged
patches, several channel chunks and slabs, each epilogue it has."""
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
    """Sets library options for one test and restores the defaults afterwards."""
    changed = []

    def set_(name, value):
        hip.set_option(name, value)
        changed.append(name)
    yield set_
    defaults = dict(lean=4, lean_cfg=0, lean_groups=0)
    for name in changed:
        hip.set_option(name, defaults[name])


LEAN_SHAPES = [
    # seed, n, c, h, w, k
    (900, 2, 64, 40, 40, 64),     # resident filter, 3 x 3 patches per image, border patches only
    (901, 1, 64, 70, 52, 64),     # interior patches, ragged right and bottom patches
    (902, 2, 128, 24, 24, 128),   # two chunks, two slabs
    (903, 1, 256, 20, 20, 64),    # four chunks
    (904, 3, 128, 9, 11, 192),    # an image smaller than a patch, three slabs
    (905, 2, 512, 20, 20, 128),   # eight chunks, patch wider than tall
    (906, 2, 256, 40, 40, 64),    # patches as wide as the image (one per row band)
    (907, 3, 64, 12, 14, 64),     # one patch per image
]


def reference(case):
    g = cases.geom_of(case)
    return port.conv2d_i8(case["x"], case["wt"], case["bias"], case["ws"], case["fs"], case["act"], g)


def all_epilogues(ctx, case, want_y):
    """The epilogues of a ResNet block's two convolutions and of a network's last layer."""
    seed = int(case["x"].shape[1] * 7 + case["k"])
    r = np.random.default_rng(seed)
    res_nchw = r.uniform(-4, 4, want_y.shape).astype(np.float32)
    res = np.ascontiguousarray(res_nchw.transpose(0, 2, 3, 1))
    fs_out = np.float32(11.7)
    out = {}
    relu_y = port.relu(want_y) if case["act"] == 0 else want_y
    q_only = gpueval.conv_i8(ctx, dict(case, act=1), fs_out=fs_out, want=())
    out["q_only"] = (q_only["i8"], port.quantize(relu_y, fs_out).transpose(0, 2, 3, 1))
    if case["act"] == 0:
        z = port.relu(port.binaryop_add(want_y, res_nchw))
        fused = gpueval.conv_i8(ctx, case, fs_out=fs_out, residual=res, post_relu=1, want=("nhwc",))
        out["res_f"] = (fused["nhwc"], z.transpose(0, 2, 3, 1))
        out["res_q"] = (fused["i8"], port.quantize(z, fs_out).transpose(0, 2, 3, 1))
        last = gpueval.conv_i8(ctx, case, residual=res, post_relu=1, want=("nchw",))
        out["res_nchw"] = (last["nchw"], z)
        zz = port.binaryop_add(want_y, res_nchw)
        signed = gpueval.conv_i8(ctx, case, fs_out=fs_out, residual=res, post_relu=0, want=("nhwc", "nchw"))
        out["signed_f"] = (signed["nhwc"], zz.transpose(0, 2, 3, 1))
        out["signed_nchw"] = (signed["nchw"], zz)
        out["signed_q"] = (signed["i8"], port.quantize(zz, fs_out).transpose(0, 2, 3, 1))
    plain = gpueval.conv_i8(ctx, case, want=("nhwc",))
    out["f_only"] = (plain["nhwc"], want_y.transpose(0, 2, 3, 1))
    return out


@pytest.mark.parametrize("mode,cfg,groups", [(1, 0, 0), (1, 1, 0), (1, 2, 0), (2, 0, 0), (1, 0, 2), (1, 1, 3), (1, 2, 1), (3, 0, 0), (3, 0, 2), (3, 0, 1)],
                         ids=["persist-a1w2", "persist-a2w2", "persist-a1w3", "oneshot", "walk2-a1w2", "walk3-a2w2", "walk1-a1w3",
                              "roles", "roles-walk2", "roles-walk1"])
@pytest.mark.parametrize("args", LEAN_SHAPES, ids=[f"s{a[0]}" for a in LEAN_SHAPES])
def test_lean_kernel_bit_exact(ctx, options, args, mode, cfg, groups):
    seed, n, c, h, w, k = args
    case = cases.conv_i8_case(seed, n, c, h, w, k, 3, 1, 1, act=0)
    want_y = reference(case)
    options("lean", mode)
    options("lean_cfg", cfg)
    options("lean_groups", groups)
    for name, (got, want) in all_epilogues(ctx, case, want_y).items():
        assert got.shape == want.shape, name
        assert np.array_equal(got, want), f"{name}: {np.count_nonzero(got != want)} of {want.size} values differ"


def test_lean_and_general_kernel_agree_on_a_stage_sized_launch(ctx, options):
    """4 x 128 x 80 x 80 -> 128: persistent groups that walk several patches of both slabs; the general kernel is the
    reference here (it is pinned against the oracle by the other tests)."""
    case = cases.conv_i8_case(910, 4, 128, 80, 80, 128, 3, 1, 1, act=0)
    r = np.random.default_rng(911)
    res = r.uniform(-4, 4, (4, 80, 80, 128)).astype(np.float32)
    fs_out = np.float32(9.3)
    options("lean", 0)
    want = gpueval.conv_i8(ctx, case, fs_out=fs_out, residual=res, post_relu=1, want=("nhwc",))
    for mode, groups in ((1, 0), (1, 5), (3, 0), (3, 5)):
        options("lean", mode)
        options("lean_groups", groups)
        got = gpueval.conv_i8(ctx, case, fs_out=fs_out, residual=res, post_relu=1, want=("nhwc",))
        assert np.array_equal(got["nhwc"], want["nhwc"])
        assert np.array_equal(got["i8"], want["i8"])
