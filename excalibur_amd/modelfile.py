"""Writers for Excalibur's model formats: `.phai` topology text and `.racy` weight blobs.

Formats as read by the reference: topology lines by src/Excalibur/pipeline.cpp:49-116, weight blobs by
src/Excalibur/operation_convolution.cpp:71-152 and src/Excalibur/operation_innerproduct.cpp:77-120
(little-endian, no header, one blob per weighted operation in topology order).
"""
import struct

import numpy as np

INT8_TAG = 871224


def conv_line(op_type, name, bottom, top, k, kernel, stride=1, pad=0, bias=True, weight_count=0, groups=1,
              int8=False, act=0):
    kh, kw = (kernel, kernel) if np.isscalar(kernel) else kernel
    sh, sw = (stride, stride) if np.isscalar(stride) else stride
    pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
    s = (f"{op_type} {name} 1 1 {bottom} {top} 0={k} 1={kw} 11={kh} 2=1 12=1 3={sw} 13={sh} "
         f"4={pl} 14={pt} 15={pr} 16={pb} 5={int(bias)} 6={weight_count} 7={groups} 9={act}")
    if int8:
        s += " 8=2"
    return s


def pool_line(name, bottom, top, ptype, kernel=0, stride=1, pad=0, global_pool=False, pad_mode=1, count_include_pad=0):
    kh, kw = (kernel, kernel) if np.isscalar(kernel) else kernel
    sh, sw = (stride, stride) if np.isscalar(stride) else stride
    pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
    return (f"Pooling {name} 1 1 {bottom} {top} 0={ptype} 1={kw} 11={kh} 2={sw} 12={sh} 3={pl} 13={pt} 14={pr} "
            f"15={pb} 4={int(global_pool)} 5={pad_mode} 6={count_include_pad}")


def topology(lines, name="net"):
    n_blobs = len(lines) + 1
    return "\n".join([f"glsv1 {name}", f"{len(lines)} {n_blobs}"] + list(lines)) + "\n"


def conv_blob_f32(w, bias=None):
    out = struct.pack("<i", 0) + np.ascontiguousarray(w, np.float32).tobytes()
    if bias is not None:
        out += np.ascontiguousarray(bias, np.float32).tobytes()
    return out


def conv_blob_i8(w, bias, ws, fs):
    w = np.ascontiguousarray(w, np.int8).tobytes()
    w += b"\0" * ((-len(w)) % 4)
    out = struct.pack("<i", INT8_TAG) + w
    if bias is not None:
        out += np.ascontiguousarray(bias, np.float32).tobytes()
    out += np.ascontiguousarray(ws, np.float32).tobytes()
    out += np.ascontiguousarray(np.atleast_1d(fs), np.float32).tobytes()
    return out


fc_blob_f32 = conv_blob_f32
fc_blob_i8 = conv_blob_i8  # one weight scale and one feature-map scale (src/Excalibur/operation_innerproduct.cpp:95-113)


def floats_blob(*arrays):
    """Untagged float arrays one after the other: PReLU slopes (src/Excalibur/operation_prelu.cpp:36-41), BatchNorm
    slope / mean / var / bias (src/Excalibur/operation_batchnorm.cpp:33-50)."""
    return b"".join(np.ascontiguousarray(a, np.float32).tobytes() for a in arrays)


def write_model(path, blobs):
    with open(path, "wb") as f:
        for b in blobs:
            f.write(b)
