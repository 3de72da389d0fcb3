"""ctypes binding of the host-side pipeline (include/excalibur_capi.h): Excalibur's `pipeline<Dtype>` API on the MI355X
backend. Loads excalibur_amd/host/lib/libexcalibur_hip.so and fails loudly if it is missing."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "host", "lib", "libexcalibur_hip.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is not built; run `make -C excalibur_amd/csrc && make -C excalibur_amd/host`")
        from . import hip
        hip.lib()  # libexhip.so first: the host library links against it
        L = ctypes.CDLL(LIB_PATH)
        L.exc_pipeline_create.restype = ctypes.c_void_p
        L.exc_pipeline_create.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int]
        L.exc_pipeline_create_from_files.restype = ctypes.c_void_p
        L.exc_pipeline_create_from_files.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int]
        L.exc_pipeline_run_keeping.argtypes = [ctypes.c_void_p]
        L.exc_pipeline_get_kept.restype = ctypes.c_long
        L.exc_pipeline_get_kept.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_long,
                                            ctypes.POINTER(ctypes.c_int)]
        L.exc_pipeline_destroy.argtypes = [ctypes.c_void_p]
        L.exc_pipeline_set_fusion.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.exc_pipeline_last_fused.argtypes = [ctypes.c_void_p]
        L.exc_pipeline_set_graphs.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.exc_pipeline_blob_stored.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        L.exc_pipeline_set_input.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]
        L.exc_pipeline_run.argtypes = [ctypes.c_void_p]
        L.exc_pipeline_sync.argtypes = [ctypes.c_void_p]
        L.exc_set_stream_slot.argtypes = [ctypes.c_int]
        L.exc_pipeline_stream_slot.argtypes = [ctypes.c_void_p]
        L.exc_pipeline_forward.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]
        L.exc_pipeline_get.restype = ctypes.c_long
        L.exc_pipeline_get.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_long,
                                       ctypes.POINTER(ctypes.c_int)]
        L.exc_pipeline_time_fused_span.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.exc_pipeline_last_span.restype = ctypes.c_float
        L.exc_pipeline_last_span.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]
        L.exc_pipeline_recent_spans.restype = ctypes.c_int
        L.exc_pipeline_recent_spans.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_float), ctypes.c_int]
        L.exc_registered_operations.restype = ctypes.c_size_t
        L.exc_registered_operations.argtypes = [ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]
        _lib = L
    return _lib


def set_option(name, value):
    """Test / development switches of the backend (see include/excalibur_capi.h)."""
    rc = lib().exc_set_option(name.encode(), int(value))
    if rc:
        raise ValueError(f"unknown option {name}")


def set_stream_slot(slot):
    """Pipelines this thread creates from now on work on the HIP stream of `slot` (0..7; see include/excalibur_capi.h)."""
    if lib().exc_set_stream_slot(int(slot)):
        raise ValueError(f"stream slot {slot} out of range")


def registered_operations(dtype="f32"):
    buf = ctypes.create_string_buffer(4096)
    lib().exc_registered_operations({"f32": 0, "f16": 1, "f64": 2}[dtype], buf, 4096)
    return buf.value.decode().split()


class Pipeline:
    """pipeline<float> (dtype 'f32') or pipeline<unsigned short> (dtype 'f16') on HIP device `device`."""

    def __init__(self, topology, model_path="", device=0, dtype="f32", fusion=True, topology_file=None):
        """topology: the `.phai` text; topology_file: instead, the path of a `.phai` file (the reference's file-path
        constructors); model_path "" loads dummy weights."""
        self.dtype = np.float32 if dtype == "f32" else np.uint16
        code = 0 if dtype == "f32" else 1
        if topology_file is not None:
            self.h = lib().exc_pipeline_create_from_files(topology_file.encode(), (model_path or "").encode(), device, code)
        else:
            self.h = lib().exc_pipeline_create(topology.encode(), (model_path or "").encode(), device, code)
        lib().exc_pipeline_set_fusion(self.h, int(fusion))

    def close(self):
        if self.h:
            lib().exc_pipeline_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def set_input(self, x):
        x = np.ascontiguousarray(x, self.dtype)
        assert x.ndim == 4
        lib().exc_pipeline_set_input(self.h, x.ctypes.data, (ctypes.c_int * 4)(*x.shape))

    def run(self):
        lib().exc_pipeline_run(self.h)

    def set_graphs(self, on):
        """Fused int8 plans replay their launches as one HIP graph, or (default) issue them one by one."""
        lib().exc_pipeline_set_graphs(self.h, int(on))

    def run_keeping(self):
        """forward() while the results of the earlier forwards stay held; get_kept(back, name) reads them."""
        lib().exc_pipeline_run_keeping(self.h)

    def get_kept(self, back, name):
        shape = (ctypes.c_int * 4)()
        n = lib().exc_pipeline_get_kept(self.h, back, name.encode(), None, 0, shape)
        if n < 0:
            raise KeyError(name)
        out = np.empty(tuple(shape), self.dtype)
        lib().exc_pipeline_get_kept(self.h, back, name.encode(), out.ctypes.data, out.size, shape)
        return out

    @property
    def stream_slot(self):
        return lib().exc_pipeline_stream_slot(self.h)

    def sync(self):
        rc = lib().exc_pipeline_sync(self.h)
        if rc:
            raise RuntimeError(f"exhip_sync failed ({rc})")

    def forward(self, x):
        self.set_input(x)
        self.run()
        self.sync()

    def time_fused_span(self, first_launch):
        """Every later fused forward records device events around its launches first_launch .. last (0 = the input
        quantizer unless the stem kernel quantizes the input itself, -2 = the first convolution's launch); -1 switches
        that off."""
        lib().exc_pipeline_time_fused_span(self.h, int(first_launch))

    def last_span(self):
        """(milliseconds, launches) between the events of the last fused forward; waits for the device."""
        n = ctypes.c_int(0)
        ms = lib().exc_pipeline_last_span(self.h, ctypes.byref(n))
        return float(ms), n.value

    def recent_spans(self, capacity=32):
        """Milliseconds between the events of the latest fused forwards since time_fused_span (oldest first, at most 32);
        waits for the device once, so forwards queued back to back are read without a synchronisation between them."""
        buf = (ctypes.c_float * capacity)()
        n = lib().exc_pipeline_recent_spans(self.h, buf, capacity)
        return [float(buf[i]) for i in range(n)]

    @property
    def fused(self):
        return bool(lib().exc_pipeline_last_fused(self.h))

    def stored(self, name):
        """Whether the last forward itself stored this blob (get() materialises the others by a per-layer rerun)."""
        return bool(lib().exc_pipeline_blob_stored(self.h, name.encode()))

    def get(self, name):
        shape = (ctypes.c_int * 4)()
        n = lib().exc_pipeline_get(self.h, name.encode(), None, 0, shape)
        if n < 0:
            raise KeyError(name)
        out = np.empty(tuple(shape), self.dtype)
        lib().exc_pipeline_get(self.h, name.encode(), out.ctypes.data, out.size, shape)
        return out
