"""Runs a case from tests/cases.py through the compiled reference (oracle/_ref). Test infrastructure."""
import os
import tempfile

import numpy as np

from excalibur_amd import modelfile as mf
from oracle import ref
from tests import cases


def run_reference(case, dtype="f32"):
    op = case["op"]
    if op in ("eltwise", "binaryop_add", "concat"):
        topo, x = cases.multi_input_topology(case)
        return ref.run(topo, "", x, ["out"], dtype)["out"]
    topo, blob, xs, out = cases.reference_io(case)
    x = xs[0]
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        f.write(blob if blob else b"\0\0\0\0")
        path = f.name
    try:
        # the int8 im2col convolution of the reference computes image 0 only: drive it per image
        per_image = op == "conv_i8"
        if dtype == "f16":
            x = np.ascontiguousarray(x).view(np.uint16) if x.dtype == np.uint16 else x
        return ref.run(topo, path, x, [out], dtype, per_image=per_image)[out]
    finally:
        os.unlink(path)
