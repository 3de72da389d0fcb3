"""Pins of the CPU restatement that do not need the reference: closed forms, brute force on tiny
inputs, invariants. Each is chosen so that a plausible slip (wrong rounding, sign, index, transposed
operand, dropped padding) fails."""
import numpy as np
import pytest

from oracle import port
from tests import cases


def test_float32_to_int8_ties_and_saturation():
    f = port.float32_to_int8
    assert [f(v) for v in (0.0, 0.49, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, -0.49)] == [0, 0, 1, 2, 3, -1, -2, -3, 0]
    # 0.49999997f + 0.5f rounds to 1.0f in float: the reference's add-then-truncate gives 1, rintf would give 0
    assert f(np.float32(0.49999997)) == 1
    assert [f(v) for v in (126.4, 126.5, 127.0, 127.49, 127.5, 300.0, 1e30)] == [126, 127, 127, 127, 127, 127, 127]
    assert [f(v) for v in (-127.5, -128.0, -128.4, -128.5, -129.0, -1e30)] == [-128, -128, -128, -128, -128, -128]


def test_quantize_dense_sweep_against_closed_form():
    x = np.linspace(-130, 130, 260001, dtype=np.float32).reshape(1, 1, 1, -1)
    q = port.quantize(x, np.float32(1.0)).ravel().astype(np.int64)
    xd = x.ravel().astype(np.float64)
    t = np.where(xd >= 0, (x.ravel() + np.float32(0.5)), (x.ravel() - np.float32(0.5))).astype(np.float64)
    want = np.clip(np.trunc(t), -128, 127).astype(np.int64)
    assert np.array_equal(q, want)
    # per-channel scales pick the input channel
    x2 = np.ones((1, 3, 2, 2), np.float32)
    q2 = port.quantize(x2, np.array([1, 2, 3], np.float32))
    assert [int(q2[0, c, 0, 0]) for c in range(3)] == [1, 2, 3]
    # ... for every image and position, against the closed form written per element
    r = np.random.default_rng(12)
    x3 = r.uniform(-5, 5, (2, 4, 3, 5)).astype(np.float32)
    fs = r.uniform(0.5, 40, 4).astype(np.float32)
    q3 = port.quantize(x3, fs)
    for idx in np.ndindex(x3.shape):
        v = np.float32(x3[idx] * fs[idx[1]])
        t = np.float32(v + np.float32(0.5)) if v >= 0 else np.float32(v - np.float32(0.5))
        assert int(q3[idx]) == int(np.clip(np.trunc(np.float64(t)), -128, 127)), idx


def _brute_conv(q, w, stride, pad, groups=1):
    n, c, h, wd = q.shape
    k, cg, kh, kw = w.shape
    pt, pb, pl, pr = pad
    oh = (h + pt + pb - kh) // stride + 1
    ow = (wd + pl + pr - kw) // stride + 1
    qp = np.zeros((n, c, h + pt + pb, wd + pl + pr), np.int64)
    qp[:, :, pt:pt + h, pl:pl + wd] = q
    out = np.zeros((n, k, oh, ow), np.int64)
    kg = k // groups
    for kk in range(k):
        g = kk // kg
        for y in range(oh):
            for x in range(ow):
                patch = qp[:, g * cg:(g + 1) * cg, y * stride:y * stride + kh, x * stride:x * stride + kw]
                out[:, kk, y, x] = (patch * w[kk].astype(np.int64)).sum(axis=(1, 2, 3))
    return out


@pytest.mark.parametrize("shape", [
    dict(n=2, c=3, h=7, w=6, k=4, kh=3, kw=3, stride=1, pad=(1, 1, 1, 1), groups=1),
    dict(n=1, c=4, h=9, w=8, k=6, kh=3, kw=3, stride=2, pad=(1, 1, 1, 1), groups=2),
    dict(n=1, c=2, h=11, w=11, k=3, kh=7, kw=7, stride=2, pad=(3, 3, 3, 3), groups=1),
    dict(n=1, c=5, h=4, w=5, k=2, kh=1, kw=1, stride=1, pad=(0, 0, 0, 0), groups=1),
    dict(n=1, c=2, h=6, w=7, k=2, kh=3, kw=2, stride=1, pad=(0, 2, 1, 0), groups=1),
])
def test_int_conv_matches_brute_force(shape):
    r = np.random.default_rng(7)
    q = r.integers(-128, 128, (shape["n"], shape["c"], shape["h"], shape["w"])).astype(np.int8)
    w = r.integers(-128, 128, (shape["k"], shape["c"] // shape["groups"], shape["kh"], shape["kw"])).astype(np.int8)
    g = port.geom(q.shape, shape["k"], shape["kh"], shape["kw"], shape["stride"], shape["pad"], shape["groups"])
    assert np.array_equal(port.conv2d_i8_acc(q, w, g).astype(np.int64),
                          _brute_conv(q, w, shape["stride"], shape["pad"], shape["groups"]))


def test_int_conv_invariants():
    r = np.random.default_rng(8)
    q = r.integers(-128, 128, (1, 8, 10, 10)).astype(np.int8)
    w1 = r.integers(-60, 60, (4, 8, 3, 3)).astype(np.int8)
    w2 = r.integers(-60, 60, (4, 8, 3, 3)).astype(np.int8)
    g = port.geom(q.shape, 4, 3, 3, 1, 1)
    a1, a2, a12 = (port.conv2d_i8_acc(q, w, g) for w in (w1, w2, (w1 + w2).astype(np.int8)))
    assert np.array_equal(a1 + a2, a12)                       # linear in the weights
    # 1x1 convolution is a GEMM over channels
    w = r.integers(-128, 128, (5, 8, 1, 1)).astype(np.int8)
    a = port.conv2d_i8_acc(q, w, port.geom(q.shape, 5, 1))
    want = np.einsum("kc,nchw->nkhw", w[:, :, 0, 0].astype(np.int64), q.astype(np.int64))
    assert np.array_equal(a.astype(np.int64), want)
    # translation: shifting the image right by one shifts interior outputs right by one
    qs = np.zeros_like(q)
    qs[..., 1:] = q[..., :-1]
    b = port.conv2d_i8_acc(qs, w1, g)
    assert np.array_equal(b[..., 2:-1], a1[..., 1:-2])
    # worst-case magnitude does not overflow: 127*128*Kd for Kd = 4608
    qbig = np.full((1, 512, 3, 3), -128, np.int8)
    wbig = np.full((1, 512, 3, 3), 127, np.int8)
    acc = port.conv2d_i8_acc(qbig, wbig, port.geom(qbig.shape, 1, 3, 3, 1, 1))
    assert int(acc[0, 0, 1, 1]) == -128 * 127 * 4608


def test_dequant_scale_and_fma():
    assert port.dequant_scale(np.float32(1e-6), np.float32(3.0)) == 0.0
    assert port.dequant_scale(np.float32(-5e-7), np.float32(3.0)) == 0.0
    ws, fs = np.float32(37.3), np.float32(2.7)
    assert port.dequant_scale(ws, fs) == np.float32(1.0) / np.float32(ws * fs)
    # one fused multiply-add: differs from round(acc*s)+b on this triple
    x = np.zeros((1, 1, 1, 1), np.float32) + 1
    c = dict(op="conv_i8", n=1, c=1, h=1, w=1, k=1, kh=1, kw=1, stride=1, pad=0, act=0, groups=1, x=x * 77,
             wt=np.array([[[[113]]]], np.int8), ws=np.array([0.37], np.float32), fs=np.float32(1.0),
             bias=np.array([0.123456], np.float32))
    y = cases.oracle_eval(c)[0, 0, 0, 0]
    s = np.float32(1.0) / np.float32(np.float32(0.37) * np.float32(1.0))
    fused = np.float32(np.float64(77 * 113) * np.float64(s) + np.float64(np.float32(0.123456)))
    assert y == fused


def test_relu6_zeroes_above_six_and_relu_keeps_values():
    y = port.activation(np.array([-1, 0, 3, 6, 6.0001, 50], np.float32), port.ACT_RELU6_ZEROING)
    assert y.tolist() == [0, 0, 3, 6, 0, 0]
    y = port.activation(np.array([-1, 0, 3, 50], np.float32), port.ACT_RELU)
    assert y.tolist() == [0, 0, 3, 50]
    s = port.activation(np.array([0.0, 2.0], np.float32), port.ACT_SIGMOID)
    assert s[0] == 0.5 and abs(float(s[1]) - 1 / (1 + np.exp(-2.0))) < 1e-7


def test_conv_f32_against_numpy_float64():
    c = cases.conv_f32_case(9, 2, 6, 9, 8, 5, (3, 2), 1, (1, 0, 2, 1), act=0)
    y = cases.oracle_eval(c)
    pt, pb, pl, pr = c["pad"]
    xp = np.pad(c["x"].astype(np.float64), ((0, 0), (0, 0), (pt, pb), (pl, pr)))
    oh, ow = y.shape[2:]
    want = np.zeros(y.shape)
    for i in range(3):
        for j in range(2):
            want += np.einsum("nchw,kc->nkhw", xp[:, :, i:i + oh, j:j + ow], c["wt"][:, :, i, j].astype(np.float64))
    want += c["bias"][None, :, None, None]
    assert np.abs(y - want).max() < 1e-6


def test_depthwise_equals_grouped_conv_within_rounding():
    c = cases.conv_f32_case(10, 2, 6, 9, 9, 6, 3, 2, 1, groups=6, dw=True)
    a = cases.oracle_eval(c)
    b = cases.oracle_eval(dict(c, op="conv_f32"))
    assert np.abs(a - b).max() < 1e-6


def test_pool_closed_forms():
    x = np.arange(2 * 3 * 6 * 6, dtype=np.float32).reshape(2, 3, 6, 6)
    m = port.pool2d(x, port.POOL_MAX, 2, 2, 0)
    assert np.array_equal(m, x.reshape(2, 3, 3, 2, 3, 2).max(axis=(3, 5)))
    a = port.pool2d(x, port.POOL_AVE, 2, 2, 0)
    assert np.allclose(a, x.reshape(2, 3, 3, 2, 3, 2).mean(axis=(3, 5)), rtol=1e-6)
    g = port.pool2d(x, port.POOL_AVE, global_pool=True)
    assert g.shape == (2, 3, 1, 1) and np.allclose(g[..., 0, 0], x.mean(axis=(2, 3)), rtol=1e-6)
    # floor vs ceil output size, and a corner window of an average pool divides by the valid count
    assert port.pool2d(x, port.POOL_MAX, 3, 2, 0, pad_mode=1).shape[2:] == (2, 2)
    assert port.pool2d(x, port.POOL_MAX, 3, 2, 0, pad_mode=0).shape[2:] == (3, 3)
    ones = np.ones((1, 1, 4, 4), np.float32)
    assert np.array_equal(port.pool2d(ones, port.POOL_AVE, 3, 1, 1), ones)
    inc = port.pool2d(ones, port.POOL_AVE, 3, 1, 1, count_include_pad=1)
    assert inc[0, 0, 0, 0] == np.float32(4.0) / np.float32(9.0) and inc[0, 0, 1, 1] == 1.0


def test_half_conversions():
    halfs = np.arange(65536, dtype=np.uint16)
    f = port.half2float(halfs)
    ref = halfs.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(f[~nan], ref[~nan]) and np.isnan(f[nan]).all()
    # truncating conversion is the identity on exactly representable values (arrays of length % 8 == 0)
    finite = halfs[~nan & ~np.isinf(ref)]
    finite = finite[: finite.size - finite.size % 8]
    assert np.array_equal(port.float2half(port.half2float(finite)), finite)
    # truncation toward zero vs round-to-nearest: 1 + 3/4 ulp stays at 1.0 when truncated
    v = np.full(8, 1.0 + 0.75 * 2 ** -10, np.float32)
    assert (port.float2half(v) == 0x3C00).all()
    # the first length % 8 elements are rounded to nearest even instead
    v = np.full(11, 1.0 + 0.75 * 2 ** -10, np.float32)
    out = port.float2half(v)
    assert (out[:3] == 0x3C01).all() and (out[3:] == 0x3C00).all()


def test_innerproduct_is_x_wT_plus_b():
    c = cases.fc_case(11, 4, 3, 2, 2, 5)
    y = cases.oracle_eval(c)[:, :, 0, 0]
    want = c["x"].reshape(4, -1).astype(np.float64) @ c["wt"].astype(np.float64).T + c["bias"]
    assert np.abs(y - want).max() < 1e-6
    # a transposed weight matrix would fail: W is [n_out][k_in]
    assert c["wt"].shape == (5, 12)
