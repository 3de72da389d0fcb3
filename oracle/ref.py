"""Driver of the compiled reference (oracle/_ref/libexcalibur_ref.so). Test infrastructure only.

The library is built by `make -C oracle ref` from the reference's own sources; it exists only
where that build was made. `available()` says whether it can be loaded.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_ref", "libexcalibur_ref.so")
_lib = None


def available():
    return os.path.exists(_SO)


def lib():
    global _lib
    if _lib is None:
        L = ctypes.CDLL(_SO)
        L.exref_pipeline_create.restype = ctypes.c_void_p
        L.exref_pipeline_create.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int]
        L.exref_pipeline_destroy.argtypes = [ctypes.c_void_p]
        L.exref_pipeline_forward.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)]
        L.exref_pipeline_get.restype = ctypes.c_long
        L.exref_pipeline_get.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_long,
                                         ctypes.POINTER(ctypes.c_int)]
        L.exref_pipeline_time.restype = ctypes.c_double
        L.exref_pipeline_time.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int),
                                          ctypes.c_int, ctypes.c_int]
        L.exref_pipeline_time_parallel.restype = ctypes.c_double
        L.exref_pipeline_time_parallel.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_void_p,
                                                   ctypes.POINTER(ctypes.c_int), ctypes.c_int, ctypes.c_int, ctypes.c_int]
        _lib = L
    return _lib


def time_parallel(topology, model_path, image, workers, warmup, iters, dtype="f32"):
    """`workers` threads, each with its own pipeline<Dtype> and the same single image (shape 1 x C x H x W), run `iters`
    timed forwards each -> wall-clock seconds of the timed part."""
    image = np.ascontiguousarray(image, np.float32 if dtype == "f32" else np.uint16)
    shape = (ctypes.c_int * 4)(*image.shape)
    return lib().exref_pipeline_time_parallel(topology.encode(), (model_path or "").encode(), 0 if dtype == "f32" else 1,
                                              image.ctypes.data, shape, int(workers), int(warmup), int(iters))


class Pipeline:
    """pipeline<float> (dtype 'f32') or pipeline<unsigned short> (dtype 'f16') on the CPU path."""

    def __init__(self, topology, model_path="", dtype="f32"):
        self.dtype = np.float32 if dtype == "f32" else np.uint16
        self.h = lib().exref_pipeline_create(topology.encode(), (model_path or "").encode(),
                                             0 if dtype == "f32" else 1)

    def close(self):
        if self.h:
            lib().exref_pipeline_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def forward(self, x):
        x = np.ascontiguousarray(x, self.dtype)
        assert x.ndim == 4
        shape = (ctypes.c_int * 4)(*x.shape)
        lib().exref_pipeline_forward(self.h, x.ctypes.data, shape)

    def get(self, name):
        shape = (ctypes.c_int * 4)()
        n = lib().exref_pipeline_get(self.h, name.encode(), None, 0, shape)
        if n < 0:
            raise KeyError(name)
        out = np.empty(tuple(shape), self.dtype)
        lib().exref_pipeline_get(self.h, name.encode(), out.ctypes.data, out.size, shape)
        return out

    def time(self, x, warmup, iters):
        x = np.ascontiguousarray(x, self.dtype)
        shape = (ctypes.c_int * 4)(*x.shape)
        return lib().exref_pipeline_time(self.h, x.ctypes.data, shape, warmup, iters)


def run(topology, model_path, x, outputs, dtype="f32", per_image=False):
    """Runs a topology on x and returns {name: array}. per_image drives one image at a time, which the
    reference's int8 im2col convolution needs (it computes only image 0 of a batch,
    src/Excalibur/operation_convolution.cpp:2284-2300)."""
    p = Pipeline(topology, model_path, dtype)
    try:
        if not per_image:
            p.forward(x)
            return {o: p.get(o) for o in outputs}
        parts = {o: [] for o in outputs}
        for i in range(x.shape[0]):
            p.forward(x[i:i + 1])
            for o in outputs:
                parts[o].append(p.get(o))
        return {o: np.concatenate(parts[o], axis=0) for o in outputs}
    finally:
        p.close()
