"""No-GPU checks of the drop-in boundary: both shared libraries load and export every symbol their headers
declare, and the operator registry holds the reference's class names."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ex(?:hip|c)_[a-z0-9_]+)\s*\(", text)))


def test_exhip_exports_every_declared_symbol():
    from excalibur_amd import hip
    L = hip.lib()
    names = _declared("exhip.h")
    assert len(names) >= 40
    for n in names:
        assert hasattr(L, n), f"libexhip.so does not export {n}"


def test_capi_exports_every_declared_symbol():
    from excalibur_amd import pipeline
    L = pipeline.lib()
    names = _declared("excalibur_capi.h")
    assert len(names) >= 10
    for n in names:
        assert hasattr(L, n), f"libexcalibur_hip.so does not export {n}"


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_registry_holds_the_reference_class_names(dtype):
    from excalibur_amd import pipeline
    got = set(pipeline.registered_operations(dtype))
    want = {"operation_convolution", "operation_convolutiondepthwise", "operation_pooling", "operation_eltwise",
            "operation_binaryop", "operation_relu", "operation_innerproduct", "operation_split"}
    assert want <= got


def test_argument_errors_need_no_gpu():
    """Descriptor validation and output-size arithmetic run on the host."""
    from excalibur_amd import hip
    L = hip.lib()
    d = hip.Ctx.conv_desc(1, 64, 56, 56, 64, 3, 1, 1, c_stride=64)
    assert hip.Ctx.conv_out_hw(d) == (56, 56)
    assert L.exhip_conv_packed_bytes(ctypes.byref(d), hip.I8) == 9 * 64 * 64
    bad = hip.Ctx.conv_desc(1, 20, 8, 8, 8, 3, 1, 1, c_stride=20)
    assert L.exhip_conv_packed_bytes(ctypes.byref(bad), hip.I8) == 0
    assert b"multiple of 32" in L.exhip_last_error()
    assert hip.Ctx.pool_out_hw(20, 20, 3, 3, 2, 2, 1, 1, 1, 1, 1) == (10, 10)
    assert hip.Ctx.pool_out_hw(14, 14, 3, 3, 2, 2, 0, 0, 0, 0, 0) == (7, 7)
    assert hip.Ctx.pool_out_hw(14, 14, 3, 3, 2, 2, 0, 0, 0, 0, 1) == (6, 6)


def test_stream_slots_and_options_need_no_gpu():
    """The slot of a thread is thread-local state of the host library, and unknown option names are refused."""
    import threading

    from excalibur_amd import pipeline
    L = pipeline.lib()
    assert L.exc_set_stream_slot(3) == 0
    assert L.exc_set_stream_slot(8) == -1 and L.exc_set_stream_slot(-1) == -1
    seen = []

    def other():
        seen.append(L.exc_set_stream_slot(5))  # another thread's slot does not move this one's

    t = threading.Thread(target=other)
    t.start()
    t.join()
    assert seen == [0]
    assert L.exc_set_stream_slot(0) == 0
    with pytest.raises(ValueError):
        pipeline.set_option("no_such_option", 1)
    pipeline.set_option("share_gpu", 0)
