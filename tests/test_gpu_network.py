"""The fused int8 ResNet-18-shaped stack on the GPU against the reference-semantics CPU chain."""
import numpy as np
import pytest

from excalibur_amd.resnet18 import FusedRunner, ResNet18Int8
from tests import netref

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from excalibur_amd import hip
    c = hip.Ctx(0)
    yield c
    c.close()


@pytest.mark.parametrize("n,hw", [(2, 96), (1, 160), (3, 64)])
def test_fused_resnet18_int8_bit_exact(ctx, n, hw):
    net = ResNet18Int8(seed=11, calib_hw=32)
    x = np.random.default_rng(12 + hw).uniform(-1, 1, (n, 3, hw, hw)).astype(np.float32)
    want, blobs = netref.oracle_forward(net, x)
    run = FusedRunner(ctx, net, n, hw, hw)
    run.set_input(x)
    run.forward()
    ctx.sync()
    got = run.out.download()
    assert got.shape == want.shape
    assert np.array_equal(got, want)
    assert np.count_nonzero(want) > want.size // 8
    # a second forward on the same buffers gives the same bytes (no state carried between calls)
    run.forward()
    ctx.sync()
    assert np.array_equal(run.out.download(), want)
