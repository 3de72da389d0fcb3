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


def test_benchmark_batch_at_full_size():
    """The benchmark's own workload (32 x 3 x 640 x 640 through the host pipeline) checked by what does not need a CPU
    pass over 32 images: (a) images are independent, so a single image run alone (other tile plans, other groups per CU)
    gives the bytes of its row of the batch; (b) the per-layer executor (float NCHW blobs between layers, every kernel
    at its real size) agrees with the fused plan; (c) where the compiled reference is present, one 640 x 640 image through
    the reference's CPU path, bit for bit."""
    import os
    import tempfile

    from excalibur_amd import pipeline as xp
    from oracle import ref

    net = ResNet18Int8(seed=1234, calib_hw=64)
    n, hw = 32, 640
    x = np.random.default_rng(99).uniform(-1, 1, (n, 3, hw, hw)).astype(np.float32)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    try:
        net.write_model(path)
        p = xp.Pipeline(net.topology(), path, 0, "f32", fusion=True)
        p.forward(x)
        assert p.fused
        batch = p.get(net.output)
        assert batch.shape == (n, 512, 20, 20)
        assert np.count_nonzero(batch) > batch.size // 8
        for i in (0, 17, 31):
            p.forward(x[i:i + 1])
            assert np.array_equal(p.get(net.output)[0], batch[i]), f"image {i} alone differs from its row of the batch"
        p.close()
        layers = xp.Pipeline(net.topology(), path, 0, "f32", fusion=False)
        layers.forward(x[:2])
        assert not layers.fused
        assert np.array_equal(layers.get(net.output), batch[:2])
        layers.close()
        if ref.available():
            r = ref.Pipeline(net.topology(), path, "f32")
            r.forward(x[17:18])
            assert np.array_equal(r.get(net.output)[0], batch[17])
            r.close()
    finally:
        os.unlink(path)
