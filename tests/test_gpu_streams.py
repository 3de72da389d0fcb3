"""Pipelines in different stream slots: forwards queued back to back on two HIP streams give the bytes of the same
forwards run alone, in the fused int8 plan and in the per-layer executor (whose blobs come from per-slot block caches)."""
import os
import tempfile
import threading

import numpy as np
import pytest

from excalibur_amd import pipeline as xp
from excalibur_amd.mobilenet import MobileFaceNetF32
from excalibur_amd.resnet18 import ResNet18Int8

pytestmark = pytest.mark.gpu


def _model_file(net):
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    net.write_model(path)
    return path


def _solo(net, path, dtype, xs, fusion=True):
    p = xp.Pipeline(net.topology(), path, 0, dtype, fusion=fusion)
    outs = []
    for x in xs:
        p.forward(x)
        outs.append(p.get(net.output).copy())
    p.close()
    return outs


def test_fused_plans_in_two_slots_interleaved():
    net = ResNet18Int8(seed=21, calib_hw=32)
    r = np.random.default_rng(22)
    xs = [r.uniform(-1, 1, (3, 3, 96, 96)).astype(np.float32) for _ in range(2)]
    path = _model_file(net)
    try:
        want = _solo(net, path, "f32", xs)
        assert not np.array_equal(want[0], want[1])
        pipes = []
        for slot in (0, 1):
            xp.set_stream_slot(slot)
            pipes.append(xp.Pipeline(net.topology(), path, 0, "f32", fusion=True))
        xp.set_stream_slot(0)
        assert [p.stream_slot for p in pipes] == [0, 1]
        for p, x in zip(pipes, xs):
            p.set_input(x)
        for _ in range(6):  # nothing waits between these: the two streams run side by side
            pipes[0].run()
            pipes[1].run()
        assert all(p.fused for p in pipes)
        for p, w in zip(pipes, want):
            assert np.array_equal(p.get(net.output), w)  # get waits for the pipeline's own stream
        # inputs swapped: each slot's buffers are rewritten, no state is shared
        for p, x in zip(pipes, xs[::-1]):
            p.set_input(x)
        for _ in range(2):
            pipes[1].run()
            pipes[0].run()
        for p, w in zip(pipes, want[::-1]):
            assert np.array_equal(p.get(net.output), w)
        for p in pipes:
            p.close()
    finally:
        xp.set_stream_slot(0)
        os.unlink(path)


def test_per_layer_executors_in_two_slots_interleaved():
    net = MobileFaceNetF32(seed=23, hw=64)
    r = np.random.default_rng(24)
    xs = [r.uniform(0, 255, (2, 3, 64, 64)).astype(np.float32) for _ in range(2)]
    path = _model_file(net)
    try:
        want32 = _solo(net, path, "f32", xs[:1])[0]
        want16 = _solo(net, path, "f16", [xs[1].astype(np.float16).view(np.uint16)])[0]
        xp.set_stream_slot(2)
        p16 = xp.Pipeline(net.topology(), path, 0, "f16")
        xp.set_stream_slot(0)
        p32 = xp.Pipeline(net.topology(), path, 0, "f32")
        p32.set_input(xs[0])
        p16.set_input(xs[1].astype(np.float16).view(np.uint16))
        for _ in range(4):  # every forward allocates and releases its blobs: each slot recycles its own blocks
            p32.run()
            p16.run()
        assert np.array_equal(p32.get(net.output), want32)
        assert np.array_equal(p16.get(net.output), want16)
        p32.close()
        p16.close()
    finally:
        xp.set_stream_slot(0)
        os.unlink(path)


def test_threads_with_a_slot_and_a_pipeline_each():
    net = ResNet18Int8(seed=25, calib_hw=32)
    r = np.random.default_rng(26)
    xs = [r.uniform(-1, 1, (2, 3, 64, 64)).astype(np.float32) for _ in range(3)]
    path = _model_file(net)
    try:
        want = _solo(net, path, "f32", xs)
        got, errors = [None] * 3, []

        def work(k):
            try:
                xp.set_stream_slot(k + 1)  # thread-local: the main thread stays in slot 0
                p = xp.Pipeline(net.topology(), path, 0, "f32", fusion=True)
                for _ in range(3):
                    p.forward(xs[k])
                got[k] = (p.stream_slot, p.get(net.output).copy())
                p.close()
            except Exception as e:  # surfaced in the main thread below
                errors.append(e)

        threads = [threading.Thread(target=work, args=(k,)) for k in range(3)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert not errors, errors
        for k in range(3):
            assert got[k][0] == k + 1
            assert np.array_equal(got[k][1], want[k])
        with pytest.raises(ValueError):
            xp.set_stream_slot(8)
    finally:
        os.unlink(path)
