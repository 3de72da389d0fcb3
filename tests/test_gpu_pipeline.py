"""The host-side mirror of the reference's operator / pipeline API on the GPU: single layers and whole topologies
loaded from `.phai` text + `.racy` blobs through pipeline<Dtype>(lines, model_file, device = 0), against the golden
fixtures of the compiled reference and the CPU restatement."""
import glob
import os
import tempfile

import numpy as np
import pytest

from excalibur_amd import pipeline as xp
from excalibur_amd.resnet18 import ResNet18Int8
from oracle import port
from tests import cases, netref
from tests.golden.make_fixtures import load_case

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
NAMES = sorted(os.path.basename(f)[:-4] for f in glob.glob(os.path.join(GOLDEN, "*.npz")) if not os.path.basename(f).startswith("net_"))
TOLERANT = ("conv_f32", "fc_", "deconv", "softmax", "binaryop_pixel", "binaryop_image", "conv_i8_mish")


def run_case(case, dtype="f32"):
    if case["op"] in ("eltwise", "binaryop_add"):
        topo, x = cases.multi_input_topology(case)
        blob = b""
    else:
        topo, blob, xs, _ = cases.reference_io(case)
        x = xs[0]
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        f.write(blob if blob else b"\0\0\0\0")
        path = f.name
    try:
        p = xp.Pipeline(topo, path, 0, dtype)
        p.forward(x)
        out = p.get("out")
        p.close()
        return out
    finally:
        os.unlink(path)


# the host layer registers Split_Slice only as far as the hot path needs it: multi-input cases use it to cut operands
MULTI = ("eltwise", "binaryop", "concat")


@pytest.mark.parametrize("name", [n for n in NAMES if not n.startswith("f16_") and not n.startswith(MULTI)])
def test_single_layer_topologies_match_reference_fixtures(name):
    case, expected = load_case(os.path.join(GOLDEN, name + ".npz"))
    got = run_case(case)
    assert got.shape == expected.shape
    if name.startswith(TOLERANT):
        assert cases.check_value(got, expected, 1e-4) == 0
    else:
        assert np.array_equal(got, expected)


@pytest.mark.parametrize("name", [n for n in NAMES if n.startswith("f16_")])
def test_fp16_pipeline_matches_reference_fixtures(name):
    case, expected = load_case(os.path.join(GOLDEN, name + ".npz"))
    got = run_case(case, "f16")
    assert got.shape == expected.shape
    assert cases.check_value(got.view(np.float16).astype(np.float32), expected.view(np.float16).astype(np.float32), 2e-3) == 0


@pytest.mark.parametrize("fusion", [False, True])
def test_resnet18_topology_through_the_pipeline(fusion):
    net = ResNet18Int8(seed=21, calib_hw=32)
    x = np.random.default_rng(22).uniform(-1, 1, (2, 3, 96, 96)).astype(np.float32)
    want, blobs = netref.oracle_forward(net, x)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    try:
        net.write_model(path)
        p = xp.Pipeline(net.topology(), path, 0, "f32", fusion=fusion)
        p.forward(x)
        assert p.fused == fusion
        got = p.get(net.output)
        assert np.array_equal(got, want)
        if not fusion:  # every intermediate blob exists as a float NCHW tensor, as in the reference
            assert np.array_equal(p.get("pool1"), blobs["pool1"])
            assert np.array_equal(p.get("l3b1_out"), blobs["l3b1_out"])
        # device time of the convolution launches of a fused forward (what the benchmark's roofline divides by)
        p.time_fused_span(-2)  # from the first convolution's launch on, whether or not an input quantizer stands in front of it
        p.forward(x)
        ms, launches = p.last_span()
        assert (launches, ms > 0) == ((20, True) if fusion else (0, False))
        assert np.array_equal(p.get(net.output), want)
        # forwards queued back to back are read after one synchronisation, oldest first, from a ring of 32 event pairs
        for _ in range(3):
            p.run()
        recent = p.recent_spans()
        assert len(recent) == (4 if fusion else 0) and all(v > 0 for v in recent)
        assert not fusion or recent[-1] == p.last_span()[0]
        assert len(p.recent_spans(2)) == (2 if fusion else 0)
        p.time_fused_span(-1)
        p.forward(x)
        assert p.last_span() == (0.0, 0)
        # a second input of another shape rebuilds the plan
        x2 = np.random.default_rng(23).uniform(-1, 1, (1, 3, 64, 64)).astype(np.float32)
        p.forward(x2)
        assert np.array_equal(p.get(net.output), netref.oracle_forward(net, x2)[0])
        p.close()
    finally:
        os.unlink(path)


def test_mixed_topology_plans_the_convolution_and_runs_the_rest_as_layers():
    """conv(int8) -> global average pool -> inner product: the int8 graph plan takes the convolution and runs the two
    layers behind it as layers on its NCHW result; with fusion off everything runs layer by layer. Same values."""
    from excalibur_amd import modelfile as mf
    r = np.random.default_rng(31)
    c = cases.conv_i8_case(32, 2, 16, 12, 12, 32, 3, 1, 1)
    wfc = r.normal(0, 0.1, (10, 32)).astype(np.float32)
    bfc = r.normal(0, 0.1, (10,)).astype(np.float32)
    lines = [mf.conv_line("Convolution", "c", "data", "a", 32, 3, 1, 1, True, c["wt"].size, 1, int8=True, act=1),
             mf.pool_line("gap", "a", "b", 1, global_pool=True),
             f"InnerProduct fc 1 1 b out 0=10 1=1 2={wfc.size}"]
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        f.write(mf.conv_blob_i8(c["wt"], c["bias"], c["ws"], c["fs"]) + mf.fc_blob_f32(wfc, bfc))
        path = f.name
    try:
        a = cases.oracle_eval(c)
        b = port.pool2d(a, port.POOL_AVE, global_pool=True)
        want = port.innerproduct(b, wfc, bfc)
        outs = {}
        for fusion in (True, False):
            p = xp.Pipeline(mf.topology(lines), path, 0, fusion=fusion)
            p.forward(c["x"])
            assert p.fused == fusion
            assert np.array_equal(p.get("a"), a)
            outs[fusion] = p.get("out")
            assert cases.check_value(outs[fusion], want, 1e-4) == 0
            p.close()
        assert np.array_equal(outs[True], outs[False])
    finally:
        os.unlink(path)


@pytest.mark.parametrize("k,pool", [(64, (3, 2, 1)), (32, (3, 2, 1)), (64, (2, 2, 0))],
                         ids=["one-kernel", "k32-two-kernels", "pool2x2-two-kernels"])
def test_fused_plan_conv_then_maxpool_as_network_output(k, pool):
    """conv(int8, ReLU) -> max pool -> conv(int8): the pool joins the convolution's node; its output is also fetched."""
    from excalibur_amd import modelfile as mf
    c1 = cases.conv_i8_case(41, 2, 32, 21, 23, k, 3, 1, 1)
    a = cases.oracle_eval(c1)
    pk, ps, pp = pool
    b = port.pool2d(a, port.POOL_MAX, pk, ps, pp)
    c2 = cases.conv_i8_case(42, 2, k, b.shape[2], b.shape[3], 64, 3, 1, 1)
    c2["x"] = b
    c2["fs"] = np.float32(127.0 / np.abs(b).max())
    want = cases.oracle_eval(c2)
    lines = [mf.conv_line("Convolution", "c1", "data", "a", k, 3, 1, 1, True, c1["wt"].size, 1, int8=True, act=1),
             mf.pool_line("p", "a", "b", 0, pk, ps, pp),
             "Split s 1 2 b b0 b1",
             mf.conv_line("Convolution", "c2", "b0", "out", 64, 3, 1, 1, True, c2["wt"].size, 1, int8=True, act=1)]
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        f.write(mf.conv_blob_i8(c1["wt"], c1["bias"], c1["ws"], c1["fs"]) + mf.conv_blob_i8(c2["wt"], c2["bias"], c2["ws"], c2["fs"]))
        path = f.name
    try:
        p = xp.Pipeline(mf.topology(lines), path, 0)
        p.forward(c1["x"])
        assert p.fused
        assert np.array_equal(p.get("out"), want)
        assert np.array_equal(p.get("b1"), b)
        p.close()
    finally:
        os.unlink(path)


@pytest.mark.parametrize("layer,evaluate", [
    ("Eltwise e 2 1 ra b out 0=1", lambda a, b: port.eltwise([a, b], port.ELT_SUM)),
    ("Eltwise e 2 1 ra b out 0=1 -23301=3,0.5,-1.25", lambda a, b: port.eltwise([a, b], port.ELT_SUM, [0.5, -1.25])),
    ("Eltwise e 2 1 ra b out 0=2", lambda a, b: port.eltwise([a, b], port.ELT_MAX)),
    ("Eltwise e 2 1 ra b out 0=0", lambda a, b: port.eltwise([a, b], port.ELT_PROD)),
    ("BinaryOp e 2 1 ra b out 0=0", lambda a, b: port.binaryop_add(a, b)),
    ("Concat e 2 1 ra b out 0=-1", lambda a, b: port.concat_channels([a, b])),
])
def test_two_input_layers_through_split_aliasing(layer, evaluate):
    """Split hands one blob to two consumers (aliasing, as in the reference); the operands are relu(x) and x."""
    from excalibur_amd import modelfile as mf
    x = np.random.default_rng(41).uniform(-2, 2, (2, 5, 9, 11)).astype(np.float32)
    lines = ["Split s 1 2 data a b", "ReLU r 1 1 a ra", layer]
    p = xp.Pipeline(mf.topology(lines), "", 0)
    p.forward(x)
    assert np.array_equal(p.get("out"), evaluate(port.relu(x), x))
    p.close()


def test_detection_head_reshape_then_transpose():
    """The YOLOv5 head of models/yolov5s_simp.phai:186-188: a 1x1 convolution to 3 x 6 channels, Reshape to
    [n][3][6][h*w] (a new shape over the same storage), Transpose 1,0,2 to [n][3][h*w][6]; float32 and fp16."""
    from excalibur_amd import modelfile as mf
    c = cases.conv_f32_case(61, 2, 8, 6, 10, 18, 1, 1, 0, act=0)
    lines = [mf.conv_line("Convolution", "c", "data", "a", 18, 1, 1, 0, True, c["wt"].size, 1, act=0),
             "Reshape r 1 1 a b 0=60 1=6 2=3", "Transpose t 1 1 b out 0=1,0,2"]
    conv = cases.oracle_eval(c)
    want = conv.reshape(2, 3, 6, 60).transpose(0, 1, 3, 2)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        f.write(mf.conv_blob_f32(c["wt"], c["bias"]))
        path = f.name
    try:
        p = xp.Pipeline(mf.topology(lines), path, 0)
        p.forward(c["x"])
        got = p.get("out")
        assert got.shape == (2, 3, 60, 6)
        assert cases.check_value(got, want, 1e-4) == 0
        p.close()
        p16 = xp.Pipeline(mf.topology(lines), path, 0, "f16")
        p16.forward(c["x"].astype(np.float16).view(np.uint16))
        got16 = p16.get("out").view(np.float16).astype(np.float32)
        assert got16.shape == (2, 3, 60, 6)
        assert cases.check_value(got16, want, 4e-3) == 0
        p16.close()
    finally:
        os.unlink(path)


def test_classifier_tail_flatten_innerproduct_softmax():
    """Flatten -> InnerProduct -> Softmax, the tail of models/FASMV2_merged.phai:110-113 (a [n][c][1][1] feature vector
    flattened to [n][1][c][1]); Clip in front bounds the features."""
    from excalibur_amd import modelfile as mf
    r = np.random.default_rng(62)
    x = r.uniform(-3, 3, (3, 120, 1, 1)).astype(np.float32)
    wfc = r.normal(0, 0.1, (7, 120)).astype(np.float32)
    bfc = r.normal(0, 0.1, (7,)).astype(np.float32)
    lines = ["Clip k 1 1 data a 0=-2.0 1=2.0", "Flatten f 1 1 a b 0=1", f"InnerProduct fc 1 1 b c 0=7 1=1 2={wfc.size}",
             "Softmax s 1 1 c out 0=0"]
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        f.write(mf.fc_blob_f32(wfc, bfc))
        path = f.name
    try:
        p = xp.Pipeline(mf.topology(lines), path, 0)
        p.forward(x)
        a = port.clip(x, -2.0, 2.0)
        logits = port.innerproduct(a, wfc, bfc)
        want = port.softmax_channels(logits.reshape(3, 7, 1, 1))
        assert np.array_equal(p.get("a"), a)
        assert p.get("b").shape == (3, 1, 120, 1)
        got = p.get("out")
        assert cases.check_value(got.reshape(want.shape), want, 1e-4) == 0
        assert np.allclose(got.reshape(3, 7).sum(1), 1.0, atol=1e-6)
        p.close()
    finally:
        os.unlink(path)


def test_squeeze_and_excite_gate():
    """The gate of models/angle_cool_best.phai:10-16: Split, global average, 1x1 convolution + ReLU, 1x1 convolution +
    HardSigmoid, BinaryOp MUL of the [n][c][h][w] tensor with the [n][c][1][1] gate; float32 and fp16."""
    from excalibur_amd import modelfile as mf
    r = np.random.default_rng(81)
    x = r.uniform(-2, 2, (2, 16, 7, 9)).astype(np.float32)
    c1 = cases.conv_f32_case(82, 2, 16, 1, 1, 4, 1, 1, 0, act=0)
    c2 = cases.conv_f32_case(83, 2, 4, 1, 1, 16, 1, 1, 0, act=0)
    lines = ["Split s 1 2 data a b", mf.pool_line("gap", "b", "g", 1, global_pool=True),
             mf.conv_line("Convolution", "c1", "g", "g1", 4, 1, 1, 0, True, c1["wt"].size, 1, act=0), "ReLU r 1 1 g1 g2",
             mf.conv_line("Convolution", "c2", "g2", "g3", 16, 1, 1, 0, True, c2["wt"].size, 1, act=0),
             "HardSigmoid h 1 1 g3 gate 0=1.666667e-01 1=5.000000e-01", "BinaryOp m 2 1 a gate out 0=2"]
    g = port.pool2d(x, port.POOL_AVE, global_pool=True)
    g = port.relu(cases.oracle_eval(dict(c1, x=g)))
    gate = port.hardsigmoid(cases.oracle_eval(dict(c2, x=g)), 1.666667e-01, 0.5)
    want = port.binaryop(x, gate, 2)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        f.write(mf.conv_blob_f32(c1["wt"], c1["bias"]) + mf.conv_blob_f32(c2["wt"], c2["bias"]))
        path = f.name
    try:
        p = xp.Pipeline(mf.topology(lines), path, 0)
        p.forward(x)
        assert cases.check_value(p.get("gate"), gate, 1e-4) == 0
        assert cases.check_value(p.get("out"), want, 1e-4) == 0
        p.close()
        p16 = xp.Pipeline(mf.topology(lines), path, 0, "f16")
        p16.forward(x.astype(np.float16).view(np.uint16))
        assert cases.check_value(p16.get("out").view(np.float16).astype(np.float32), want, 5e-3) == 0
        p16.close()
    finally:
        os.unlink(path)


@pytest.mark.parametrize("bias", [True, False])
def test_int8_innerproduct_is_the_int8_1x1_convolution_of_the_flattened_input(bias):
    """The reference reads the int8 InnerProduct blob but has no forward for it (include/Excalibur/operation.hpp:353-357).
    The layer is defined here by the int8 convolution's arithmetic, so the pinned int8 convolution restatement, run as a
    1x1 convolution over the [m][c*h*w][1][1] view of the input, is its oracle: bit-exact."""
    from excalibur_amd import modelfile as mf
    r = np.random.default_rng(71)
    x = r.uniform(-3, 3, (5, 6, 3, 4)).astype(np.float32)
    k, n_out = 72, 10
    wq = r.integers(-127, 128, (n_out, k)).astype(np.int8)
    fs = np.float32(127.0 / np.abs(x).max() * 1.05)
    ws = np.float32(1.0 / (3e-3 * fs))
    b = r.normal(0, 0.5, (n_out,)).astype(np.float32) if bias else None
    line = f"InnerProduct fc 1 1 data out 0={n_out} 1={int(bias)} 2={wq.size} 8=1"
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        f.write(mf.fc_blob_i8(wq, b, np.array([ws], np.float32), fs))
        path = f.name
    try:
        p = xp.Pipeline(mf.topology([line]), path, 0)
        p.forward(x)
        g = port.geom((5, k, 1, 1), n_out, 1)
        want = port.conv2d_i8(x.reshape(5, k, 1, 1), wq.reshape(n_out, k, 1, 1), b, np.full((n_out,), ws, np.float32), fs, 0, g)
        got = p.get("out")
        assert got.shape == (5, n_out, 1, 1)
        assert np.array_equal(got, want)
        p.close()
    finally:
        os.unlink(path)


def test_input_layer_without_bottoms_normalises_the_pipeline_input():
    """`Input name 0 1 blob ...` (no bottoms): the pipeline input is `<name>_input`, the layer subtracts the means and
    scales (one scale repeated over the channels), then a float convolution with PReLU behind it: fp32 and fp16."""
    from excalibur_amd import modelfile as mf
    r = np.random.default_rng(51)
    x = r.uniform(0, 255, (2, 3, 12, 14)).astype(np.float32)
    c = cases.conv_f32_case(52, 2, 3, 12, 14, 8, 3, 1, 1, act=0)
    slope = np.abs(r.normal(0, 0.3, (8,))).astype(np.float32)
    lines = ["Input data 0 1 data 0=14 1=12 2=3 3=123.0,117.0,104.0 4=0.0078125",
             mf.conv_line("Convolution", "c", "data", "a", 8, 3, 1, 1, True, c["wt"].size, 1, act=0),
             "PReLU p 1 1 a out 0=8"]
    xin = port.input_layer(x, [123.0, 117.0, 104.0], [0.0078125] * 3)
    c["x"] = xin
    want = port.prelu(cases.oracle_eval(c), slope)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        f.write(mf.conv_blob_f32(c["wt"], c["bias"]) + mf.floats_blob(slope))
        path = f.name
    try:
        p = xp.Pipeline(mf.topology(lines), path, 0)
        p.forward(x)
        assert np.array_equal(p.get("data"), xin)
        assert cases.check_value(p.get("out"), want, 1e-4) == 0
        p.close()
        p16 = xp.Pipeline(mf.topology(lines), path, 0, "f16")
        p16.forward(x.astype(np.float16).view(np.uint16))
        got = p16.get("out").view(np.float16).astype(np.float32)
        assert cases.check_value(got, want, 2e-2) == 0  # two half roundings of values up to 255 in front of the convolution
        p16.close()
    finally:
        os.unlink(path)


def test_mobilefacenet_shaped_float_topology_matches_the_reference_fixture():
    """Input -> conv/PReLU -> depthwise/pointwise bottlenecks with Eltwise residuals -> global average -> InnerProduct,
    loaded from generated `.phai` + `.racy`: float32 against the compiled reference's output, float16 alongside."""
    from excalibur_amd.mobilenet import MobileFaceNetF32
    net = MobileFaceNetF32()
    z = np.load(os.path.join(GOLDEN, "net_mobilefacenet_f32.npz"))
    x = np.random.default_rng(int(z["input_seed"])).uniform(0, 255, (2, 3, net.hw, net.hw)).astype(np.float32)
    expected = z["expected"]
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    try:
        net.write_model(path)
        p = xp.Pipeline(net.topology(), path, 0)
        p.forward(x)
        got = p.get(net.output)
        assert not p.fused
        assert got.shape == expected.shape
        assert cases.check_value(got, expected, 1e-4) == 0
        want, blobs = netref.oracle_forward_mobilenet(net, x)
        assert cases.check_value(p.get("b1_out"), blobs["b1_out"], 1e-4) == 0  # an intermediate blob by name
        p.close()
        p16 = xp.Pipeline(net.topology(), path, 0, "f16")
        p16.forward(x.astype(np.float16).view(np.uint16))
        got16 = p16.get(net.output).view(np.float16).astype(np.float32)
        assert cases.check_value(got16, expected, 3e-2) == 0  # every layer rounds to half: error grows with depth
        p16.close()
    finally:
        os.unlink(path)


def test_yolov5_shaped_float_topology_matches_the_reference_fixture():
    """Focus -> HardSwish convolutions -> cross-stage block (BinaryOp sum, Concat, BatchNorm, LeakyRelu) -> pyramid of
    5 / 9 / 13 max pools -> upsampling + Concat -> two heads ending in Reshape + Transpose, loaded from generated
    `.phai` + `.racy`: float32 against the compiled reference's outputs, float16 alongside."""
    from excalibur_amd.yolo import YoloV5ShapedF32
    net = YoloV5ShapedF32()
    z = np.load(os.path.join(GOLDEN, "net_yolov5_shaped_f32.npz"))
    x = np.random.default_rng(int(z["input_seed"])).uniform(0, 255, (1, 3, net.hw, net.hw)).astype(np.float32)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    try:
        net.write_model(path)
        p = xp.Pipeline(net.topology(), path, 0)
        p.forward(x)
        assert not p.fused
        for i, name in enumerate(net.outputs):
            got = p.get(name)
            assert got.shape == z[f"expected{i}"].shape
            assert cases.check_value(got, z[f"expected{i}"], 1e-4) == 0
        p.close()
        p16 = xp.Pipeline(net.topology(), path, 0, "f16")
        p16.forward(x.astype(np.float16).view(np.uint16))
        for i, name in enumerate(net.outputs):
            got16 = p16.get(name).view(np.float16).astype(np.float32)
            assert cases.check_value(got16, z[f"expected{i}"], 3e-2) == 0  # every layer rounds to half
        p16.close()
    finally:
        os.unlink(path)


@pytest.mark.parametrize("which", ["mobilefacenet", "yolov5"])
def test_fp16_pipeline_nhwc_resident_equals_nchw_blobs(which):
    """pipeline<unsigned short> keeps blobs NHWC between its convolution, depthwise, pooling, elementwise and per-channel
    layers; with that switched off every blob is NCHW as in the reference. Layer by layer the arithmetic is the same, so
    the two agree bit for bit: on the output and on blobs in the middle, which come out of the pipeline as NCHW."""
    if which == "mobilefacenet":
        from excalibur_amd.mobilenet import MobileFaceNetF32
        net = MobileFaceNetF32(seed=5, hw=32, width=16, blocks=((2, 16, 2), (1, 16, 2), (2, 32, 4)), embed=32)
        outputs, kinds = [net.output], ("PReLU", "Eltwise")  # convolution and depthwise blobs live inside their PReLU pair
    else:  # Focus, Concat, nearest Interp, the 5 / 9 / 13 pooling pyramid, heads whose channel count is no multiple of 8
        from excalibur_amd.yolo import YoloV5ShapedF32
        net = YoloV5ShapedF32(seed=7, hw=64, width=8)
        outputs, kinds = list(net.outputs), ("Concat", "Interp", "Pooling", "HardSwish")
    x = np.random.default_rng(6).uniform(0, 255, (3, 3, net.hw, net.hw)).astype(np.float32)
    x16 = x.astype(np.float16).view(np.uint16)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    try:
        net.write_model(path)
        names = outputs
        # the first output blob of a few layers in the middle (line: type name n_in n_out bottoms... tops... keys)
        middle = [l.split()[4 + int(l.split()[2])] for l in net.lines if l.split()[0] in kinds][:12]
        got = {}
        try:
            for flag in ("0", "1"):
                xp.set_option("f16_nchw_only", int(flag))
                p = xp.Pipeline(net.topology(), path, 0, "f16")
                p.forward(x16)
                got[flag] = {b: p.get(b) for b in names + middle}
                p.close()
        finally:
            xp.set_option("f16_nchw_only", 0)
        for b in names + middle:
            assert got["0"][b].shape == got["1"][b].shape
            assert np.array_equal(got["0"][b], got["1"][b]), b
        out = got["0"][names[0]].view(np.float16).astype(np.float32)
        assert np.isfinite(out).all() and np.count_nonzero(out) > out.size // 2
    finally:
        os.unlink(path)


def _activation_pairs_net(seed, int8):
    """Convolutions followed by every activation layer the convolution kernel can apply itself, plus the cases it must
    leave alone: a sigmoid, a blob with a second reader, a blob that is a result of the network, a grouped layer."""
    from excalibur_amd import modelfile as mf
    r = np.random.default_rng(seed)
    lines, blobs = ["Input data 0 1 data 0=20 1=20 2=3 3=0,0,0 4=1.0"], []

    def conv(bottom, top, cin, k, kernel, stride, groups=1):
        w = r.normal(0, np.sqrt(2.0 / (cin // groups * kernel * kernel)), (k, cin // groups, kernel, kernel)).astype(np.float32)
        b = r.normal(0, 0.5, (k,)).astype(np.float32)
        if int8 and groups == 1:
            ws = (np.float32(127.0) / np.abs(w).reshape(k, -1).max(axis=1)).astype(np.float32)
            wq = np.clip(np.rint(w * ws[:, None, None, None]), -127, 127).astype(np.int8)
            lines.append(mf.conv_line("Convolution", top + "_l", bottom, top, k, kernel, stride, kernel // 2, True, w.size, 1, int8=True))
            blobs.append(mf.conv_blob_i8(wq, b, ws, np.float32(40.0)))
        else:
            kind = "Convolution" if groups == 1 else "ConvolutionDepthWise"
            lines.append(mf.conv_line(kind, top + "_l", bottom, top, k, kernel, stride, kernel // 2, True, w.size, groups))
            blobs.append(mf.conv_blob_f32(w, b))

    conv("data", "c1", 3, 16, 3, 1)
    lines.append("HardSwish hs1 1 1 c1 a1 0=1.666667e-01 1=5.000000e-01")
    conv("a1", "c1b", 16, 16, 3, 1)
    lines.append("PReLU pr1b 1 1 c1b a1b 0=16")                          # one slope per channel
    blobs.append(mf.floats_blob(r.uniform(-0.5, 0.5, 16).astype(np.float32)))
    conv("a1b", "c1c", 16, 24, 1, 1)
    lines.append("PReLU pr1c 1 1 c1c a1c 0=1")                           # one slope for all
    blobs.append(mf.floats_blob(np.asarray([0.25], np.float32)))
    conv("a1c", "c2", 24, 32, 1, 1)
    lines.append("LeakyRelu lk2 1 1 c2 c2 0=1.000000e-01")              # writes over its input
    conv("c2", "c3", 32, 32, 3, 2)
    lines.append("ReLU r3 1 1 c3 a3")
    conv("a3", "c4", 32, 24, 1, 1)                                        # 24 channels: no multiple of 16
    lines.append("Clip cl4 1 1 c4 a4 0=-0.25 1=0.75")
    conv("a4", "c5", 24, 16, 3, 1)
    lines.append("HardSigmoid hg5 1 1 c5 a5 0=2.000000e-01 1=5.000000e-01")
    conv("a5", "c6", 16, 16, 1, 1)
    lines.append("Sigmoid sg6 1 1 c6 a6")                                 # stays a layer
    conv("a6", "c7", 16, 16, 3, 1)
    lines.append("HardSwish hs7 1 1 c7 a7 0=1.666667e-01 1=5.000000e-01")  # c7 has a second reader below
    lines.append("Eltwise sum7 2 1 c7 a7 s7 0=1")
    conv("s7", "c8", 16, 16, 3, 1, groups=16)                             # depthwise: its kernel has no such epilogue
    lines.append("HardSwish hs8 1 1 c8 a8 0=1.666667e-01 1=5.000000e-01")
    conv("a8", "c8b", 16, 16, 3, 2, groups=16)                           # depthwise 3x3 + PReLU: one kernel
    lines.append("PReLU pr8b 1 1 c8b a8b 0=16")
    blobs.append(mf.floats_blob(r.uniform(-0.5, 0.5, 16).astype(np.float32)))
    conv("a8b", "c8c", 16, 16, 1, 1)                                      # fp16: the sum behind it joins its epilogue
    lines.append("Eltwise sum8 2 1 c8c a8b s8 0=1")
    conv("s8", "c8d", 16, 16, 3, 1)
    lines.append("BinaryOp add8 2 1 s8 c8d s8d 0=0")                      # the convolution's blob as second operand
    conv("s8d", "c9", 16, 16, 1, 1)
    lines.append("Split sp9 1 2 c9 c9a c9b")
    lines.append("ReLU r9 1 1 c9a a9")                                    # c9b stays a result of the network
    return lines, blobs, ["a9", "c9b"], ["a1", "a1b", "a1c", "c2", "a3", "a4", "a5", "a6", "a7", "s7", "a8", "a8b", "s8", "s8d"]


@pytest.mark.parametrize("kind", ["f32", "f16", "int8"])
def test_activation_layer_in_the_convolution_epilogue_equals_two_layers(kind):
    """With fusion on, the per-layer executor hands a HardSwish / LeakyRelu / ReLU / Clip / HardSigmoid / PReLU layer that is the
    only reader of a convolution to that convolution's epilogue. The values are bit for bit those of the two layers run
    one after the other (fusion off), in float32, in float16 (where the layer between rounds to half) and behind the
    int8 convolution; the blob between the two is not kept."""
    from excalibur_amd import modelfile as mf
    lines, blobs, outputs, middle = _activation_pairs_net(21, kind == "int8")
    x = np.random.default_rng(22).normal(0, 1.5, (2, 3, 20, 20)).astype(np.float32)
    dtype = "f16" if kind == "f16" else "f32"
    xin = x.astype(np.float16).view(np.uint16) if kind == "f16" else x
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    try:
        mf.write_model(path, blobs)
        got = {}
        for fusion in (False, True):
            p = xp.Pipeline(mf.topology(lines, "pairs"), path, 0, dtype, fusion=fusion)
            p.forward(xin)
            assert not p.fused
            got[fusion] = {b: p.get(b) for b in outputs}
            if fusion:  # which blobs the forward itself stored (asked before get() materialises the others)
                for gone in ("c1", "c1b", "c1c", "c3", "c4", "c5", "c8b"):
                    assert not p.stored(gone), gone
                for summed in ("c8c", "c8d"):  # the residual adds: in the convolution only on NHWC half blobs
                    assert p.stored(summed) == (kind != "f16"), summed
                for kept in ("c6", "c7", "c8", "c9b"):
                    assert p.stored(kept), kept
                for b in middle:  # with int8 convolutions, a blob read by int8 convolutions alone has no float form
                    assert p.stored(b) or kind == "int8", b
            else:
                assert all(p.stored(b) for b in middle)
            for b in middle:
                got[fusion][b] = p.get(b)
            if fusion:  # a skipped blob comes from a per-layer rerun of the same input: the plain pipeline's bytes
                assert np.array_equal(p.get("c1"), plain_c1)
            else:
                plain_c1 = p.get("c1")
            p.close()
        assert len(got[True]) >= len(outputs) + 4
        for b in got[True]:
            assert got[False][b].shape == got[True][b].shape
            assert np.array_equal(got[False][b].view(np.uint32 if dtype == "f32" else np.uint16),
                                  got[True][b].view(np.uint32 if dtype == "f32" else np.uint16)), b
        last = got[True]["a9"]
        last = last.view(np.float16).astype(np.float32) if kind == "f16" else last
        assert np.isfinite(last).all() and np.count_nonzero(last) > last.size // 8
    finally:
        os.unlink(path)


@pytest.mark.parametrize("fusion", [False, True])
def test_yolov5_shaped_int8_topology_matches_the_reference_fixture(fusion):
    """The detector topology with int8 convolutions through pipeline<float>: each convolution quantizes its float input,
    accumulates in int32 and dequantizes with fmaf, every other layer is float, so the outputs equal the compiled
    reference's bit for bit, layer by layer and through the int8 graph plan (fusion: int8 / float32 NHWC tensors between
    the layers, activation layers and sums in the convolutions' epilogues, Concat -> BatchNorm -> LeakyRelu in one kernel)."""
    from excalibur_amd.yolo import YoloV5ShapedF32
    net = YoloV5ShapedF32(int8=True, outputs=8)
    z = np.load(os.path.join(GOLDEN, "net_yolov5_shaped_int8.npz"))
    x = np.random.default_rng(int(z["input_seed"])).uniform(0, 255, (1, 3, net.hw, net.hw)).astype(np.float32)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    try:
        net.write_model(path)
        p = xp.Pipeline(net.topology(), path, 0, fusion=fusion)
        p.forward(x)
        assert p.fused == fusion   # with fusion the int8 graph plan takes the network
        for i, name in enumerate(net.outputs):
            got = p.get(name)
            assert got.shape == z[f"expected{i}"].shape
            assert np.array_equal(got, z[f"expected{i}"])
        p.close()
    finally:
        os.unlink(path)


def test_int8_convolutions_hand_their_readers_int8_tensors():
    """With fusion on, an int8 convolution read by int8 convolutions (directly, through Split layers, behind its paired
    activation) writes their quantized input itself and they skip the quantizer; a blob all of whose readers are such
    convolutions is never stored as float. Same values as layer by layer, bit for bit: conv -> conv, conv -> HardSwish
    -> Split -> two convs, a convolution read by a float layer as well, one whose reader uses another scale, one with
    fewer output channels than the reader's channel stride."""
    from excalibur_amd import modelfile as mf
    r = np.random.default_rng(51)
    lines, blobs = ["Input data 0 1 data 0=24 1=24 2=3 3=0,0,0 4=1.0"], []

    def conv(bottom, top, cin, k, kernel, stride, fs):
        w = r.normal(0, np.sqrt(2.0 / (cin * kernel * kernel)), (k, cin, kernel, kernel)).astype(np.float32)
        b = r.normal(0, 0.3, (k,)).astype(np.float32)
        ws = (np.float32(127.0) / np.abs(w).reshape(k, -1).max(axis=1)).astype(np.float32)
        wq = np.clip(np.rint(w * ws[:, None, None, None]), -127, 127).astype(np.int8)
        lines.append(mf.conv_line("Convolution", top + "_l", bottom, top, k, kernel, stride, kernel // 2, True, w.size, 1, int8=True))
        blobs.append(mf.conv_blob_i8(wq, b, ws, np.float32(fs)))

    conv("data", "c1", 3, 64, 3, 1, 40.0)
    conv("c1", "c2", 64, 24, 3, 2, 30.0)                     # c1: one int8 reader, float never stored; 24 of 32 channels
    lines.append("HardSwish hs2 1 1 c2 a2 0=1.666667e-01 1=5.000000e-01")
    lines.append("Split sp2 1 2 a2 a2x a2y")
    conv("a2x", "c3", 24, 32, 1, 1, 50.0)                    # both readers of a2 quantize with 50
    conv("a2y", "c4", 24, 32, 3, 1, 50.0)
    lines.append("Split sp3 1 2 c3 c3x c3y")                 # c3: an int8 reader and a float reader
    conv("c3x", "c5", 32, 32, 1, 1, 20.0)
    lines.append("Split sp4 1 2 c4 c4a c4b")
    lines.append("Eltwise sum 2 1 c3y c4a s 0=1")            # c4: float readers only
    lines.append("Sigmoid sg4 1 1 c4b g4")                   # a sigmoid in the middle: no int8 plan takes this network,
    conv("g4", "c9", 32, 16, 1, 1, 90.0)                     # so the per-layer executor's own joins are what runs
    conv("s", "c6", 32, 64, 3, 1, 25.0)
    lines.append("Split sp6 1 2 c6 c6x c6y")                 # c6: two int8 readers with different scales
    conv("c6x", "c7", 64, 16, 1, 1, 35.0)
    conv("c6y", "c8", 64, 16, 1, 1, 45.0)
    outputs = ["c5", "c7", "c8", "c9"]
    x = np.random.default_rng(52).normal(0, 1.0, (2, 3, 24, 24)).astype(np.float32)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    try:
        mf.write_model(path, blobs)
        got = {}
        for fusion in (False, True):
            p = xp.Pipeline(mf.topology(lines, "links"), path, 0, fusion=fusion)
            p.forward(x)
            assert not p.fused
            got[fusion] = {b: p.get(b) for b in outputs + ["c3", "c4", "s"]}
            if fusion:
                for gone in ("c1", "c2", "a2"):         # int8 only, or inside the pair
                    assert not p.stored(gone), gone
                assert np.isfinite(p.get("c6")).all()    # its second reader quantizes the float form itself
                p.forward(x)                              # a second forward reuses the pooled blocks
                for b in outputs:
                    assert np.array_equal(p.get(b), got[True][b])
            else:
                for b in ("c1", "c2", "a2", "c6"):
                    assert np.isfinite(p.get(b)).all()
            p.close()
        for b in got[False]:
            assert np.array_equal(got[False][b].view(np.uint32), got[True][b].view(np.uint32)), b
        assert all(np.count_nonzero(got[True][b]) > got[True][b].size // 4 for b in outputs)
    finally:
        os.unlink(path)


def _fp16_joins_net(seed):
    """The joins of the fp16 executor beyond the activation pairs: Focus / Reshape / Transpose on halves, the sum behind
    convolution -> activation, Concat -> BatchNorm -> activation chains and their shorter forms, and the cases that
    must stay separate layers (a second reader in the middle of a chain, a sigmoid)."""
    from excalibur_amd import modelfile as mf
    r = np.random.default_rng(seed)
    lines, blobs = ["Input data 0 1 data 0=32 1=32 2=3 3=0,0,0 4=1.0", "YoloV5Focus focus 1 1 data f0"], []

    def conv(bottom, top, cin, k, kernel, stride=1):
        w = r.normal(0, np.sqrt(2.0 / (cin * kernel * kernel)), (k, cin, kernel, kernel)).astype(np.float32)
        b = r.normal(0, 0.5, (k,)).astype(np.float32)
        lines.append(mf.conv_line("Convolution", top + "_l", bottom, top, k, kernel, stride, kernel // 2, True, w.size, 1))
        blobs.append(mf.conv_blob_f32(w, b))

    def batchnorm(bottom, top, c):
        lines.append(f"BatchNorm {top}_l 1 1 {bottom} {top} 0={c}")
        blobs.append(mf.floats_blob(r.uniform(0.5, 1.5, c), r.normal(0, 0.3, c), r.uniform(0.3, 2.0, c), r.normal(0, 0.2, c)))

    hs = "0=1.666667e-01 1=5.000000e-01"
    conv("f0", "c1", 12, 32, 3)
    lines.append(f"HardSwish hs1 1 1 c1 a1 {hs}")
    lines.append("Split sp1 1 3 a1 a1a a1b a1c")
    conv("a1a", "c2", 32, 32, 1)                       # pointwise kernel, activation, then the sum behind the activation
    lines.append(f"HardSwish hs2 1 1 c2 a2 {hs}")
    conv("a2", "c3", 32, 32, 3)                        # 3x3: the lean kernel's fp16 form with the sum behind the activation
    lines.append(f"HardSwish hs3 1 1 c3 a3 {hs}")
    lines.append("BinaryOp add3 2 1 a1b a3 s3 0=0")
    conv("s3", "c4", 32, 32, 1)                        # no bias-less form needed: Concat -> BatchNorm -> LeakyRelu
    conv("a1c", "c5", 32, 32, 1)
    lines.append("Concat cat6 2 1 c4 c5 k6 0=-1")
    batchnorm("k6", "b6", 64)
    lines.append("LeakyRelu lk6 1 1 b6 a6 0=1.000000e-01")
    lines.append("Split sp6 1 3 a6 a6a a6b a6c")
    conv("a6a", "c7", 64, 32, 3, 2)
    lines.append("Interp up7 1 1 c7 u7 0=1 1=2.000000e+00 2=2.000000e+00")
    lines.append("Concat cat8 2 1 u7 a6b k8 0=-1")      # Concat -> BatchNorm, no activation behind it
    batchnorm("k8", "b8", 96)
    conv("b8", "c9", 96, 64, 1)
    batchnorm("c9", "b9", 64)                          # BatchNorm -> HardSwish without a Concat
    lines.append(f"HardSwish hs9 1 1 b9 a9 {hs}")
    lines.append("Concat cat10 2 1 a9 a6c k10 0=-1")    # Concat whose BatchNorm output has a second reader: the chain ends at the BatchNorm
    batchnorm("k10", "b10", 128)
    lines.append("Split sp10 1 2 b10 b10a b10b")
    lines.append("LeakyRelu lk10 1 1 b10a a10 0=1.000000e-01")
    lines.append("Eltwise sum11 2 1 a10 b10b s11 0=1")
    batchnorm("s11", "b11", 128)                       # BatchNorm -> Sigmoid: the sigmoid stays a layer
    lines.append("Sigmoid sg11 1 1 b11 a11")
    conv("a11", "c12", 128, 21, 1)                     # a detection head: 21 channels, Reshape and Transpose on halves
    lines.append("Reshape rs12 1 1 c12 r12 0=256 1=7 2=3")
    lines.append("Transpose tp12 1 1 r12 t12 0=1,0,2")
    middle = ["f0", "a1", "a2", "s3", "a6", "b8", "a9", "b10", "a10", "s11", "a11"]
    gone = ["c2", "c3", "a3", "k6", "b6", "k8", "b9", "k10"]
    return lines, blobs, ["t12"], middle, gone


def test_fp16_executor_joins_equal_the_separate_layers():
    """fusion on against fusion off in pipeline<unsigned short>, bit for bit, on a network with every join of the fp16
    executor; the blobs inside a join are not stored and come from a per-layer rerun when asked for."""
    from excalibur_amd import modelfile as mf
    lines, blobs, outputs, middle, gone = _fp16_joins_net(31)
    x = np.random.default_rng(32).normal(0, 1.0, (2, 3, 32, 32)).astype(np.float16).view(np.uint16)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    try:
        mf.write_model(path, blobs)
        got = {}
        for fusion in (False, True):
            p = xp.Pipeline(mf.topology(lines, "joins"), path, 0, "f16", fusion=fusion)
            p.forward(x)
            if fusion:
                for b in gone:
                    assert not p.stored(b), b
                for b in middle:
                    assert p.stored(b), b
            else:
                assert all(p.stored(b) for b in middle + gone)
            got[fusion] = {b: p.get(b) for b in outputs + middle + gone}
            p.close()
        for b in got[True]:
            assert got[False][b].shape == got[True][b].shape, b
            assert np.array_equal(got[False][b], got[True][b]), b
        out = got[True]["t12"].view(np.float16).astype(np.float32)
        assert out.shape == (2, 3, 256, 7)
        assert np.isfinite(out).all() and np.count_nonzero(out) > out.size // 2
    finally:
        os.unlink(path)


def _int8_graph_net(seed, head_channels=21):
    """An int8 detection-shaped network with every join of the int8 graph plan: Input + Focus in front; convolution ->
    HardSwish; the sum behind convolution -> HardSwish (a bottleneck) and convolution -> add -> ReLU; Concat -> BatchNorm
    -> LeakyRelu read by a convolution; a 5 / 9 pooling pyramid whose Concat is read by a convolution only (int8
    Concat); Interp -> Concat; a Concat that leaves the network; heads of 21 channels with Reshape and Transpose."""
    from excalibur_amd import modelfile as mf
    r = np.random.default_rng(seed)
    lines, blobs = ["Input data 0 1 data 0=64 1=64 2=3 3=10.0,20.0,30.0 4=0.0039215", "YoloV5Focus focus 1 1 data f0"], []

    def conv(bottom, top, cin, k, kernel, stride=1, scale=8.0, bias=True):
        w = r.normal(0, np.sqrt(2.0 / (cin * kernel * kernel)), (k, cin, kernel, kernel)).astype(np.float32)
        b = r.normal(0, 0.3, (k,)).astype(np.float32)
        ws = (np.float32(127.0) / np.abs(w).reshape(k, -1).max(axis=1)).astype(np.float32)
        wq = np.clip(np.rint(w * ws[:, None, None, None]), -127, 127).astype(np.int8)
        lines.append(mf.conv_line("Convolution", top + "_l", bottom, top, k, kernel, stride, kernel // 2, bias, w.size, 1, int8=True))
        blobs.append(mf.conv_blob_i8(wq, b if bias else None, ws, np.float32(scale)))

    def batchnorm(bottom, top, c):
        lines.append(f"BatchNorm {top}_l 1 1 {bottom} {top} 0={c}")
        blobs.append(mf.floats_blob(r.uniform(0.5, 1.5, c), r.normal(0, 0.3, c), r.uniform(0.3, 2.0, c), r.normal(0, 0.2, c)))

    hs = "0=1.666667e-01 1=5.000000e-01"
    conv("f0", "c1", 12, 32, 3, scale=60.0)
    lines.append(f"HardSwish hs1 1 1 c1 a1 {hs}")
    conv("a1", "c2", 32, 64, 3, 2, scale=20.0)
    lines.append(f"HardSwish hs2 1 1 c2 a2 {hs}")
    lines.append("Split sp2 1 2 a2 a2a a2b")
    conv("a2a", "c3", 64, 32, 1, scale=12.0)           # the block's first 1x1, read by the bottleneck and by its sum
    lines.append(f"HardSwish hs3 1 1 c3 a3 {hs}")
    lines.append("Split sp3 1 2 a3 a3a a3b")
    conv("a3a", "c4", 32, 32, 1, scale=14.0)
    lines.append(f"HardSwish hs4 1 1 c4 a4 {hs}")
    conv("a4", "c5", 32, 32, 3, scale=15.0)
    lines.append(f"HardSwish hs5 1 1 c5 a5 {hs}")
    lines.append("BinaryOp add5 2 1 a3b a5 s5 0=0")     # the sum behind the activation
    lines.append("Split sp5 1 2 s5 s5a s5b")
    conv("s5a", "c6", 32, 32, 3, scale=9.0)            # a second block in the ResNet order: convolution -> add -> ReLU
    lines.append("BinaryOp add6 2 1 c6 s5b s6 0=0")
    lines.append("ReLU relu6 1 1 s6 a6")
    conv("a6", "c7", 32, 32, 1, scale=11.0, bias=False)   # the two plain convolutions in front of Concat -> BatchNorm -> LeakyRelu
    conv("a2b", "c8", 64, 32, 1, scale=12.0, bias=False)
    lines.append("Concat cat9 2 1 c7 c8 k9 0=-1")
    batchnorm("k9", "b9", 64)
    lines.append("LeakyRelu lk9 1 1 b9 a9 0=1.000000e-01")
    conv("a9", "c10", 64, 64, 1, scale=10.0)
    lines.append(f"HardSwish hs10 1 1 c10 a10 {hs}")
    lines.append("Split sp10 1 2 a10 a10a a10b")
    conv("a10a", "c11", 64, 128, 3, 2, scale=10.0)
    lines.append(f"HardSwish hs11 1 1 c11 a11 {hs}")
    conv("a11", "c12", 128, 64, 1, scale=13.0)          # the pooling pyramid
    lines.append(f"HardSwish hs12 1 1 c12 a12 {hs}")
    lines.append("Split sp12 1 3 a12 a12a a12b a12c")
    lines.append(mf.pool_line("p5", "a12b", "q5", 0, kernel=5, stride=1, pad=2))
    lines.append(mf.pool_line("p9", "a12c", "q9", 0, kernel=9, stride=1, pad=4))
    lines.append("Concat cat13 3 1 a12a q5 q9 k13 0=-1")
    conv("k13", "c14", 192, 64, 1, scale=16.0)
    lines.append(f"HardSwish hs14 1 1 c14 a14 {hs}")
    lines.append("Split sp14 1 2 a14 a14a a14b")
    lines.append("Interp up15 1 1 a14a u15 0=1 1=2.000000e+00 2=2.000000e+00")
    lines.append("Concat cat16 2 1 u15 a10b k16 0=-1")  # Interp -> Concat read by two convolutions and kept as an output
    lines.append("Split sp16 1 3 k16 k16a k16b k16c")
    conv("k16a", "c17", 128, head_channels, 1, scale=18.0)
    lines.append(f"Reshape rs17 1 1 c17 r17 0=256 1={head_channels // 3} 2=3")
    lines.append("Transpose tp17 1 1 r17 t17 0=1,0,2")
    conv("k16b", "c18", 128, 32, 3, scale=18.0)
    lines.append(f"HardSwish hs18 1 1 c18 a18 {hs}")
    conv("a14b", "c19", 64, head_channels, 1, scale=17.0)
    lines.append(f"Reshape rs19 1 1 c19 r19 0=64 1={head_channels // 3} 2=3")
    lines.append("Transpose tp19 1 1 r19 t19 0=1,0,2")
    return lines, blobs, ["t17", "a18", "t19", "k16c"]


def test_int8_graph_plan_equals_the_per_layer_executor():
    """The int8 executor for networks beyond residual blocks (activation layers, sums behind them, Concat / BatchNorm /
    Interp / pooling pyramids, Focus in front, Reshape / Transpose behind) against the per-layer executor with fusion
    off: bit for bit on every output, on a second forward, and on an input of another size (the plan is rebuilt)."""
    from excalibur_amd import modelfile as mf
    lines, blobs, outputs = _int8_graph_net(61)
    with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
        path = f.name
    try:
        mf.write_model(path, blobs)
        plain = xp.Pipeline(mf.topology(lines, "graph"), path, 0, fusion=False)
        fused = xp.Pipeline(mf.topology(lines, "graph"), path, 0, fusion=True)
        for seed, n in ((62, 2), (63, 3), (62, 2)):
            x = np.random.default_rng(seed).uniform(0, 255, (n, 3, 64, 64)).astype(np.float32)
            plain.forward(x)
            assert not plain.fused
            fused.forward(x)
            assert fused.fused
            for b in outputs:
                want, got = plain.get(b), fused.get(b)
                assert want.shape == got.shape, b
                assert np.array_equal(want.view(np.uint32), got.view(np.uint32)), (b, seed)
                assert np.isfinite(got).all() and np.count_nonzero(got) > got.size // 4, b
            # a blob inside the plan comes from a per-layer rerun of the same input
            assert not fused.stored("a5")
            assert np.array_equal(fused.get("s5"), plain.get("s5"))
        # the plan's launches replayed as one HIP graph (the front kernel stays eager, the tail layers run behind the replay):
        # every replay against the eager results, with other work and synchronisations between the replays
        replay = xp.Pipeline(mf.topology(lines, "graph"), path, 0, fusion=True)
        replay.set_graphs(True)
        for seed in (62, 66, 62, 67):
            x = np.random.default_rng(seed).uniform(0, 255, (2, 3, 64, 64)).astype(np.float32)
            fused.forward(x)
            replay.forward(x)
            for b in outputs:
                assert np.array_equal(fused.get(b).view(np.uint32), replay.get(b).view(np.uint32)), (b, seed)
        replay.close()
        plain.close()
        fused.close()
    finally:
        os.unlink(path)


def test_int8_graph_plan_second_scale_and_refusal():
    """Two readers of one tensor with different feature-map scales: the plan makes the second int8 form from the float32
    form with a quantizer launch and still takes the network. A sigmoid layer (not an activation the epilogues apply) at
    the end of a branch runs as a layer behind the plan's launches; in the middle, where a convolution reads its result, it
    leaves the network to the per-layer executor. Same results as with fusion off in every case."""
    from excalibur_amd import modelfile as mf
    for change in ("scale", "sigmoid at the end", "sigmoid in the middle"):
        lines, blobs, outputs = _int8_graph_net(64)
        if change == "scale":
            # c8 is the 8th convolution: it reads a2 next to c3, whose scale stays 12
            at = [i for i, l in enumerate(lines) if l.startswith("Convolution c8_l ")][0]
            n_conv = sum(1 for l in lines[:at] if l.startswith("Convolution "))
            n_blob = sum(1 for l in lines[:at] if l.startswith(("Convolution ", "BatchNorm ")))
            assert n_conv == 7
            raw = bytearray(blobs[n_blob])
            raw[-4:] = np.float32(13.0).tobytes()     # the blob ends with the feature-map scale
            blobs[n_blob] = bytes(raw)
        elif change == "sigmoid at the end":
            at = [i for i, l in enumerate(lines) if l.startswith("HardSwish hs18 ")][0]
            lines[at] = "Sigmoid hs18 1 1 c18 a18"
        else:
            at = [i for i, l in enumerate(lines) if l.startswith("HardSwish hs10 ")][0]
            lines[at] = "Sigmoid hs10 1 1 c10 a10"
        with tempfile.NamedTemporaryFile(suffix=".racy", delete=False) as f:
            path = f.name
        try:
            mf.write_model(path, blobs)
            x = np.random.default_rng(65).uniform(0, 255, (2, 3, 64, 64)).astype(np.float32)
            got = {}
            for fusion in (False, True):
                p = xp.Pipeline(mf.topology(lines, "graph"), path, 0, fusion=fusion)
                p.forward(x)
                assert p.fused == (fusion and change != "sigmoid in the middle"), change
                got[fusion] = {b: p.get(b) for b in outputs}
                p.close()
            for b in outputs:
                assert np.array_equal(got[False][b].view(np.uint32), got[True][b].view(np.uint32)), (change, b)
        finally:
            os.unlink(path)
