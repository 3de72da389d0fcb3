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


# ---- reading a topology back, and seeded weights for any topology ----
class Layer:
    """One topology line: type, name, bottoms, tops and the key=value parameters (strings, in file order)."""

    def __init__(self, kind, name, bottoms, tops, params):
        self.kind, self.name, self.bottoms, self.tops, self.params = kind, name, bottoms, tops, params

    def get(self, key, default=None, cast=int):
        v = self.params.get(str(key))
        return default if v is None else cast(v)


def parse_topology(text):
    """-> [Layer] in file order, tokenised as src/Excalibur/pipeline.cpp:63-116 does: lines 0 and 1 are the header, a
    layer without inputs reads the synthetic blob <name>_input."""
    layers = []
    for line in text.splitlines()[2:]:
        tok = line.split()
        if not tok:
            continue
        n_in, n_out = int(tok[2]), int(tok[3])
        bottoms = tok[4:4 + n_in] if n_in else [tok[1] + "_input"]
        tops = tok[4 + n_in:4 + n_in + n_out]
        params = dict(t.split("=", 1) for t in tok[4 + n_in + n_out:])
        layers.append(Layer(tok[0], tok[1], bottoms, tops, params))
    return layers


WEIGHTED = ("Convolution", "ConvolutionDepthWise", "Deconvolution", "InnerProduct", "BatchNorm", "PReLU")


class SeededModel:
    """Random weights for every weighted layer of a topology, from a seed: `.blobs` is the `.racy` content in file
    order, `.weights[layer name]` the arrays behind it. Convolution weights are N(0, 2 / fan_in) so that activations keep
    their scale through deep stacks; layers with key 8 set carry int8 weights with per-channel scales
    ws = 127 / max|w| and the feature-map scale fs[layer name] (default `default_fs`)."""

    def __init__(self, layers, seed, fs=None, default_fs=16.0, gain=2.0):
        r = np.random.default_rng(seed)
        self.blobs, self.weights = [], {}
        fs = fs or {}
        for L in layers:
            if L.kind in ("Convolution", "ConvolutionDepthWise", "Deconvolution"):
                k, kw = L.get(0), L.get(1)
                kh = L.get(11, kw)
                count, groups, bias = L.get(6), L.get(7, 1), L.get(5, 0) != 0
                cin_g = count // (k * kh * kw)
                if L.kind == "Deconvolution":   # [c_in][k][kh][kw], fan-in per output value c_in * kh * kw / stride^2
                    shape, fan = (cin_g, k, kh, kw), cin_g * kh * kw / float(L.get(3, 1) * L.get(13, L.get(3, 1)))
                else:
                    shape, fan = (k, cin_g, kh, kw), cin_g * kh * kw
                w = r.normal(0, np.sqrt(gain / fan), shape).astype(np.float32)
                b = r.normal(0, 0.05, (k,)).astype(np.float32) if bias else None
                entry = {"w": w, "bias": b}
                if L.get(8, 0) != 0:
                    ws = (np.float32(127.0) / np.abs(w).reshape(k, -1).max(axis=1)).astype(np.float32)
                    wq = np.clip(np.rint(w * ws[:, None, None, None]), -127, 127).astype(np.int8)
                    f = np.float32(fs.get(L.name, default_fs))
                    entry.update(w_i8=wq, ws=ws, fs=f)
                    self.blobs.append(conv_blob_i8(wq, b, ws, f))
                else:
                    self.blobs.append(conv_blob_f32(w, b))
                self.weights[L.name] = entry
            elif L.kind == "InnerProduct":
                n_out, bias, count = L.get(0), L.get(1, 0) != 0, L.get(2)
                w = r.normal(0, np.sqrt(1.0 / (count // n_out)), (n_out, count // n_out)).astype(np.float32)
                b = r.normal(0, 0.05, (n_out,)).astype(np.float32) if bias else None
                self.weights[L.name] = {"w": w, "bias": b}
                self.blobs.append(fc_blob_f32(w, b))
            elif L.kind == "BatchNorm":
                c = L.get(0)
                p = [r.uniform(0.5, 1.5, (c,)), r.normal(0, 0.3, (c,)), r.uniform(0.3, 2.0, (c,)), r.normal(0, 0.2, (c,))]
                p = [a.astype(np.float32) for a in p]
                self.weights[L.name] = {"slope": p[0], "mean": p[1], "var": p[2], "bias": p[3]}
                self.blobs.append(floats_blob(*p))
            elif L.kind == "PReLU":
                s = r.uniform(0.05, 0.3, (L.get(0),)).astype(np.float32)
                self.weights[L.name] = {"slope": s}
                self.blobs.append(floats_blob(s))

    def write(self, path):
        write_model(path, self.blobs)
