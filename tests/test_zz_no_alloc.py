"""The entry point that allocates nothing (exhip_maxpool_same_nhwc_f16_static) against the entry point it is a variant
of (exhip_maxpool_same_nhwc_f16, caller-provided workspace) and against the CPU restatement: bit for bit, on two calls
in a row, the second on a smaller tensor, so that what the first call left in the static array would show."""
import numpy as np
import pytest

from oracle import port

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from excalibur_amd import hip
    c = hip.Ctx(0)
    yield c
    c.close()


def _nhwc_half(rng, n, h, w, c):
    return rng.uniform(-4, 4, (n, h, w, c)).astype(np.float16)


def _oracle(x16, k):
    want = port.pool2d(np.ascontiguousarray(x16.astype(np.float32).transpose(0, 3, 1, 2)), port.POOL_MAX, k, 1, k // 2)
    return np.ascontiguousarray(want.transpose(0, 2, 3, 1)).astype(np.float16)


def test_static_scratch_pooling_equals_workspace_pooling_twice(ctx):
    from excalibur_amd import hip
    rng = np.random.default_rng(77)
    assert hip.lib().exhip_static_scratch_bytes() == 8 << 20
    for (n, h, w, c, k) in [(3, 20, 24, 64, 5), (1, 9, 7, 16, 13)]:  # the second call is the smaller one
        x16 = _nhwc_half(rng, n, h, w, c)
        x = ctx.array(x16.view(np.uint16))
        y = ctx.empty(x16.shape, np.uint16).zero()
        got = ctx.maxpool_same_nhwc_f16_static(x, k, y).download()
        ref = ctx.maxpool_same_nhwc_f16(x, k).download()
        assert np.array_equal(got, ref), (n, h, w, c, k)
        assert np.array_equal(got.view(np.float16), _oracle(x16, k)), (n, h, w, c, k)


def test_static_scratch_pooling_refuses_more_than_its_array_holds(ctx):
    from excalibur_amd import hip
    n, h, w, c = 1, 64, 64, 1032  # 8.06 MiB of halves
    x = ctx.empty((n, h, w, c), np.uint16).zero()
    y = ctx.empty((n, h, w, c), np.uint16)
    with pytest.raises(hip.ExhipError, match="static scratch array holds"):
        ctx.maxpool_same_nhwc_f16_static(x, 5, y)
