"""The CPU restatement against the compiled reference, live, on more shapes than the fixtures hold.
Runs only where oracle/_ref was built (marker `ref`)."""
import numpy as np
import pytest

from tests import cases

pytestmark = pytest.mark.ref


def _ref(case, dtype="f32"):
    from tests.refrun import run_reference
    return run_reference(case, dtype)


@pytest.mark.parametrize("args", [
    (100, 1, 64, 20, 20, 64, 3, 1, 1),      # cfg1-shaped, reduced
    (101, 2, 32, 17, 19, 40, 3, 1, 1),      # odd sizes: Winograd tile padding
    (102, 1, 32, 16, 16, 128, 3, 1, 1),     # K = 128 switches to im2col
    (103, 2, 24, 15, 15, 36, 3, 2, 1),
    (104, 1, 64, 8, 8, 256, 1, 1, 0),
    (105, 1, 16, 12, 12, 32, 1, 2, 0),      # 1x1 stride 2 (downsample branch)
    (106, 1, 3, 40, 40, 64, 7, 2, 3),
])
def test_conv_i8_bit_exact(args):
    case = cases.conv_i8_case(*args)
    assert np.array_equal(_ref(case), cases.oracle_eval(case))


@pytest.mark.parametrize("args", [
    (110, 1, 64, 28, 28, 64, 3, 1, 1),
    (111, 1, 32, 14, 14, 128, 3, 1, 1),
    (112, 2, 16, 15, 15, 24, 3, 2, 1),
    (113, 1, 3, 48, 48, 32, 7, 2, 3),
])
def test_conv_f32_within_1e4(args):
    case = cases.conv_f32_case(*args)
    assert cases.check_value(_ref(case), cases.oracle_eval(case), 1e-4) == 0


@pytest.mark.parametrize("stride,h", [(1, 14), (1, 15), (2, 14), (2, 15)])
def test_depthwise_bit_exact(stride, h):
    case = cases.conv_f32_case(120 + h + stride, 2, 16, h, h + 1, 16, 3, stride, 1, groups=16, dw=True)
    assert np.array_equal(_ref(case), cases.oracle_eval(case))


@pytest.mark.parametrize("kw", [
    dict(ptype=0, kernel=3, stride=2, pad=1), dict(ptype=0, kernel=5, stride=1, pad=2),
    dict(ptype=0, kernel=9, stride=1, pad=4), dict(ptype=0, kernel=13, stride=1, pad=6),
    dict(ptype=1, kernel=2, stride=2, pad=0), dict(ptype=1, kernel=2, stride=2, pad=(0, 1, 0, 1)),
    dict(ptype=1, global_pool=True), dict(ptype=0, global_pool=True),
])
def test_pool_bit_exact(kw):
    case = cases.pool_case(130, 2, 6, 21, 22, **kw)
    assert np.array_equal(_ref(case), cases.oracle_eval(case))


def test_fc_within_1e4():
    case = cases.fc_case(140, 4, 64, 7, 7, 100)
    assert cases.check_value(_ref(case), cases.oracle_eval(case), 1e-4) == 0
