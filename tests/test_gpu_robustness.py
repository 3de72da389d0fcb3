"""Host-side corner cases of the device runtime and the fused executor: a recorded graph next to split-reduction launches
of another size, a failed allocation followed by a launch, packed weights a live plan points to while other geometries
come and go, and blobs asked for after the input tensor has been rewritten."""
import os
import tempfile

import numpy as np
import pytest

from excalibur_amd import hip
from excalibur_amd import pipeline as xp
from excalibur_amd.resnet18 import ResNet18Int8

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def model():
    net = ResNet18Int8(seed=21, calib_hw=32)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    net.write_model(path)
    yield net, path
    os.unlink(path)


def fresh_result(net, path, x, blob=None):
    p = xp.Pipeline(net.topology(), path, 0)
    p.forward(x)
    out = p.get(blob or net.output)
    p.close()
    return out


def test_graph_replays_survive_split_launches_of_another_size_on_the_same_stream(model):
    """One image of 64 x 64 splits the reduction of its deep layers over several groups (few tiles); so does a 2 x 128 x 96
    batch, with more tiles and splits. Both pipelines work in the same stream slot, hence with the same scratch: the
    recorded graph's launches must find it where it was when they were recorded."""
    net, path = model
    r = np.random.default_rng(22)
    small = [r.uniform(-1, 1, (1, 3, 64, 64)).astype(np.float32) for _ in range(4)]
    large = r.uniform(-1, 1, (2, 3, 128, 96)).astype(np.float32)
    graph = xp.Pipeline(net.topology(), path, 0)
    graph.set_graphs(True)
    other = xp.Pipeline(net.topology(), path, 0)
    want_large = fresh_result(net, path, large)
    for i, x in enumerate(small):
        graph.forward(x)        # the second forward records the graph, the later ones replay it
        assert graph.fused
        assert np.array_equal(graph.get(net.output), fresh_result(net, path, x)), i
        other.forward(large)    # eager launches with a larger split in between
        assert np.array_equal(other.get(net.output), want_large), i
    graph.close()
    other.close()


def test_a_failed_allocation_leaves_no_error_for_the_next_launch():
    ctx = hip.Ctx(0)
    with pytest.raises(hip.ExhipError):
        ctx.empty((1 << 45,), np.uint8)
    x = ctx.array(np.array([-1.5, 0.0, 2.5, -0.0], np.float32))
    y = ctx.relu_f32(x)
    ctx.sync()
    assert np.array_equal(y.download(), np.array([0.0, 0.0, 2.5, 0.0], np.float32))
    ctx.close()


def test_packed_weights_of_a_live_plan_stay_while_other_geometries_come_and_go(model):
    """The fused plan keeps pointers to its layers' packed weights; the per-layer executor packs for every new input
    geometry and keeps only a few copies per layer. After five other shapes the plan must still convolve with its own."""
    net, path = model
    r = np.random.default_rng(23)
    first = r.uniform(-1, 1, (2, 3, 64, 96)).astype(np.float32)
    want = fresh_result(net, path, first)
    p = xp.Pipeline(net.topology(), path, 0)
    p.forward(first)
    assert p.fused and np.array_equal(p.get(net.output), want)
    xp.lib().exc_pipeline_set_fusion(p.h, 0)
    for hw in ((64, 64), (96, 64), (32, 64), (64, 32), (96, 96), (32, 32)):
        p.forward(r.uniform(-1, 1, (1, 3) + hw).astype(np.float32))
        assert not p.fused
    xp.lib().exc_pipeline_set_fusion(p.h, 1)
    p.forward(first)
    assert p.fused and np.array_equal(p.get(net.output), want)
    p.close()


def test_a_blob_the_plan_did_not_store_is_refused_once_the_input_has_been_rewritten(model):
    net, path = model
    r = np.random.default_rng(24)
    a = r.uniform(-1, 1, (1, 3, 64, 64)).astype(np.float32)
    b = r.uniform(-1, 1, (1, 3, 64, 64)).astype(np.float32)
    p = xp.Pipeline(net.topology(), path, 0)
    p.forward(a)
    assert p.fused and not p.stored("pool1")
    p.set_input(b)              # the caller refills the input tensor without a forward
    with pytest.raises(KeyError):
        p.get("pool1")          # a per-layer rerun would now compute b's blob beside a's results: refused
    assert np.array_equal(p.get(net.output), fresh_result(net, path, a))   # what the last forward stored is still there
    p.run()
    p.sync()
    assert np.array_equal(p.get("pool1"), fresh_result(net, path, b, "pool1"))   # materialised by a rerun of the same input
    p.set_input(a)
    assert np.array_equal(p.get("pool1"), fresh_result(net, path, b, "pool1"))   # stored by that rerun: still b's
    p.close()
