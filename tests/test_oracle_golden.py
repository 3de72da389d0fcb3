"""The CPU restatement against the golden fixtures produced by the compiled reference
(tests/golden/make_fixtures.py). Bit-exact for int8 / pooling / elementwise / depthwise paths,
1e-4 (the reference's check_value rule) for f32 convolution and inner product, 2e-3 for fp16."""
import glob
import os

import numpy as np
import pytest

from oracle import port
from tests import cases
from tests.golden.make_fixtures import load_case

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FILES = sorted(f for f in glob.glob(os.path.join(GOLDEN, "*.npz")) if not os.path.basename(f).startswith("net_"))
NAMES = [os.path.basename(f)[:-4] for f in FILES]

# the float paths whose summation order the restatement does not reproduce (it sums in double)
TOLERANT = ("conv_f32", "fc_", "deconv", "softmax", "binaryop_pixel", "binaryop_image")


def test_fixture_inventory():
    assert len(FILES) >= 36


@pytest.mark.parametrize("name", [n for n in NAMES if not n.startswith("f16_")])
def test_oracle_matches_reference_fixture(name):
    case, expected = load_case(os.path.join(GOLDEN, name + ".npz"))
    got = cases.oracle_eval(case)
    assert got.shape == expected.shape
    if name.startswith(TOLERANT):
        assert cases.check_value(got, expected, 1e-4) == 0
    else:
        # == on floats: +0.0 and -0.0 compare equal (the reference's two int8 paths differ in the sign of zero)
        assert np.array_equal(got, expected)


@pytest.mark.parametrize("name", [n for n in NAMES if n.startswith("f16_")])
def test_oracle_fp16_layer(name):
    """fp16 layer = float2half(op_f32(half2float(x))), include/Excalibur/operation.hpp:234-260."""
    case, expected = load_case(os.path.join(GOLDEN, name + ".npz"))
    x16 = case["x"]
    case = dict(case, x=port.half2float(x16))
    got16 = port.float2half(cases.oracle_eval(case))
    # at most one half ulp apart (double vs float summation decides a truncation boundary)
    assert np.abs(got16.astype(np.int32) - expected.astype(np.int32)).max() <= 1
    assert cases.check_value(got16.view(np.float16).astype(np.float32),
                             expected.view(np.float16).astype(np.float32), 2e-3) == 0
    if not name.startswith("f16_conv"):
        assert np.array_equal(got16, expected)
