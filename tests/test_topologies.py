"""The generated topologies of excalibur_amd.topologies against the files the library ships under models/, token for
token, where the reference tree is present (the shipped text itself is not part of this repository)."""
import os

import pytest

from excalibur_amd import topologies

MODELS = "/root/reference/models"


@pytest.mark.parametrize("name", sorted(topologies.SHIPPED))
def test_generated_topology_equals_the_shipped_file(name):
    path = os.path.join(MODELS, name)
    if not os.path.exists(path):
        pytest.skip("the reference tree is not present")
    text, outputs = topologies.SHIPPED[name]()
    want = [line.split() for line in open(path).read().splitlines() if line.strip()]
    got = [line.split() for line in text.splitlines() if line.strip()]
    for i, (g, w) in enumerate(zip(got, want)):
        assert g == w, f"line {i}: {' '.join(g)!r} != {' '.join(w)!r}"
    assert len(got) == len(want)
    produced = {t for line in got[2:] for t in line[4 + int(line[2]):4 + int(line[2]) + int(line[3])]}
    assert set(outputs) <= produced


@pytest.mark.parametrize("size", [64, 320])
def test_detector_topologies_scale_with_the_input(size):
    text, outs = topologies.yolov5s_simp(size)
    reshapes = [line for line in text.splitlines() if line.startswith("Reshape")]
    assert [int(line.split()[6][2:]) for line in reshapes] == [(size // s) ** 2 for s in (8, 16, 32)]
    assert len(outs) == 3
    text, outs = topologies.det_db_resnet18(size)
    assert f"0={size} 1={size}" in text and outs == ["output"]
