"""A C++ application compiled against the mirrored headers (excalibur_amd/host/include) alone, shaped like the
reference's speed benchmark, run as a child process: its output blob equals what the C wrapper returns."""
import os
import subprocess
import tempfile

import numpy as np
import pytest

from excalibur_amd import pipeline as xp
from excalibur_amd.resnet18 import ResNet18Int8

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_caller_against_the_mirrored_headers_equals_the_c_wrapper():
    host = os.path.join(ROOT, "excalibur_amd", "host")
    net = ResNet18Int8(seed=41, calib_hw=32)
    x = np.random.default_rng(42).uniform(-1, 1, (2, 3, 96, 96)).astype(np.float32)
    with tempfile.TemporaryDirectory() as tmp:
        exe = os.path.join(tmp, "speed_caller")
        subprocess.check_call(["g++", "-std=gnu++17", "-O1", "-I", os.path.join(host, "include"), os.path.join(ROOT, "tests", "cpp", "speed_caller.cpp"),
                               "-o", exe, "-L", os.path.join(host, "lib"), "-lexcalibur_hip",
                               "-Wl,-rpath," + os.path.join(host, "lib"), "-Wl,-rpath," + os.path.join(ROOT, "excalibur_amd", "lib")])
        phai, racy, xin, yout = (os.path.join(tmp, n) for n in ("net.phai", "net.racy", "x.bin", "y.bin"))
        with open(phai, "w") as f:
            f.write(net.topology())
        net.write_model(racy)
        x.tofile(xin)
        out = subprocess.run([exe, phai, racy, "2", "3", "96", "96", xin, net.output, yout, "10"], capture_output=True, text=True, timeout=300)
        assert out.returncode == 0, out.stdout + out.stderr
        assert "Min" in out.stdout and net.output in out.stdout
        got = np.fromfile(yout, np.float32)
        p = xp.Pipeline(net.topology(), racy, 0, "f32", fusion=True)
        p.forward(x)
        want = p.get(net.output)
        p.close()
    assert got.size == want.size
    assert np.array_equal(got.reshape(want.shape), want)
