"""ctypes binding of the CPU oracle (libzc_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py.  The product package never imports this.
"""
import ctypes as C
import os
import subprocess
import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libzc_oracle.so")


def build():
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)


class Linear(C.Structure):
    _fields_ = [("weight", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p),
                ("input", C.c_uint32), ("output", C.c_uint32), ("group", C.c_uint32), ("bits", C.c_uint32)]


class Config(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("hidden", "experts", "topk", "inter", "group", "bits_gate_up",
                                          "bits_down", "shared_bits_gate_up", "shared_bits_down")]


class Layer(C.Structure):
    _fields_ = [("router", C.c_void_p), ("router_offsets", C.c_void_p), ("shared_gate", C.c_void_p),
                ("shared_record", C.c_void_p), ("expert_records", C.c_void_p), ("record_stride", C.c_uint64)]


class Trace(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("logits", "ids", "weights", "expert_out", "shared", "gate")]


def _load():
    if not os.path.exists(_LIB):
        build()
    lib = C.CDLL(_LIB)
    f32, u16 = C.c_float, C.c_uint16
    lib.zco_bf.restype = f32; lib.zco_bf.argtypes = [f32]
    lib.zco_b16.restype = f32; lib.zco_b16.argtypes = [u16]
    lib.zco_expf.restype = f32; lib.zco_expf.argtypes = [f32]
    lib.zco_sigmoid_bf.restype = f32; lib.zco_sigmoid_bf.argtypes = [f32]
    lib.zco_affine_dot.restype = f32
    lib.zco_dispatch.restype = C.c_int
    lib.zco_moe_layer.restype = C.c_int
    lib.zco_projection_bytes.restype = C.c_uint64
    lib.zco_projection_bytes.argtypes = [C.c_uint32] * 4
    lib.zco_record_bytes.restype = C.c_uint64
    lib.zco_softplus_bf.restype = f32; lib.zco_softplus_bf.argtypes = [f32]
    lib.zco_unary.restype = f32; lib.zco_unary.argtypes = [f32, C.c_uint32]
    return lib


lib = _load()


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def bf(x):
    """Vectorised qwen.metal:17-21 (round-to-nearest-even to BF16, kept in fp32)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    r = ((u + np.uint32(0x7fff) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xffff0000)).view(np.float32)
    return np.where(np.isnan(x), np.float32(np.nan), r).astype(np.float32)


def bf_bits(x):
    return (bf(x).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def b16(h):
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def make_linear(weight, scales, biases, K, N, group=64, bits=4):
    """weight/scales/biases: contiguous numpy arrays that the caller keeps alive."""
    l = Linear(_p(weight), _p(scales), _p(biases), K, N, group, bits)
    l._keep = (weight, scales, biases)
    return l


def linear(l, x, tokens, float_output=False):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty((tokens, l.output), np.float32)
    lib.zco_linear(C.byref(l), _p(x), C.c_uint32(tokens), _p(out), C.c_int(int(float_output)))
    return out


def gated_linear(gate, up, x, tokens, rows=None):
    x = np.ascontiguousarray(x, dtype=np.float32)
    r = None if rows is None else np.ascontiguousarray(rows, dtype=np.int32)
    out = np.empty((tokens, gate.output), np.float32)
    lib.zco_gated_linear(C.byref(gate), C.byref(up), _p(x), C.c_uint32(tokens), _p(r), _p(out))
    return out


def plain_mm(w, x, K, N, tokens, dtype=0, float_output=False):
    w = np.ascontiguousarray(w); x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty((tokens, N), np.float32)
    lib.zco_plain_mm(_p(w), C.c_uint32(dtype), _p(x), C.c_uint32(K), C.c_uint32(N), C.c_uint32(tokens), _p(out),
                     C.c_int(int(float_output)))
    return out


def router_logits(w_bf16, x, tokens, K, E, offsets=None):
    w = np.ascontiguousarray(w_bf16, dtype=np.uint16); x = np.ascontiguousarray(x, dtype=np.float32)
    o = None if offsets is None else np.ascontiguousarray(offsets, dtype=np.float32)
    out = np.empty((tokens, E), np.float32)
    lib.zco_router_logits(_p(w), _p(x), C.c_uint32(tokens), C.c_uint32(K), C.c_uint32(E), _p(o), _p(out))
    return out


def exp32(x):
    """zco_expf elementwise: the fp32 exponential shared by the sigmoid and the routing softmax."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return np.array([lib.zco_expf(float(v)) for v in x.ravel()], dtype=np.float32).reshape(x.shape)


def route(logits, tokens, E, topk=10):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    ids = np.empty((tokens, topk), np.int32); w = np.empty((tokens, topk), np.float32)
    lib.zco_route(_p(logits), C.c_uint32(tokens), C.c_uint32(E), C.c_uint32(topk), _p(ids), _p(w))
    return ids, w


def dispatch(ids, tokens, topk, E):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    offsets = np.empty(E + 1, np.int32); slots = np.empty(tokens * topk, np.int32); sel = np.empty(E, np.int32)
    n = lib.zco_dispatch(_p(ids), C.c_uint32(tokens), C.c_uint32(topk), C.c_uint32(E), _p(offsets), _p(slots), _p(sel))
    if n < 0:
        raise RuntimeError("invalid router output")
    return offsets, slots, sel[:n].copy()


def scatter_experts(x, positions, H, out):
    x = np.ascontiguousarray(x, dtype=np.float32); p = np.ascontiguousarray(positions, dtype=np.int32)
    lib.zco_scatter_experts(_p(x), _p(p), C.c_uint32(len(p)), C.c_uint32(H), _p(out))


def moe_sum(experts, weights, shared, gate, tokens, H, topk=10):
    a = [np.ascontiguousarray(v, dtype=np.float32) for v in (experts, weights, shared, gate)]
    out = np.empty((tokens, H), np.float32)
    lib.zco_moe_sum(_p(a[0]), _p(a[1]), _p(a[2]), _p(a[3]), C.c_uint32(tokens), C.c_uint32(H), C.c_uint32(topk), _p(out))
    return out


def record_bytes(cfg, shared=False):
    return lib.zco_record_bytes(C.byref(cfg), C.c_int(int(shared)))


def expert_linear(cfg, record, projection, shared=False):
    """record: contiguous uint8 numpy array holding one record (kept alive by the result)."""
    l = Linear()
    lib.zco_expert_linear(C.byref(cfg), C.c_int(int(shared)), _p(record), C.c_int(projection), C.byref(l))
    l._keep = record
    return l


def moe_layer(cfg, router, shared_gate, shared_record, expert_records, record_stride, x, tokens,
              router_offsets=None, threads=1, trace=False):
    """Whole layer (model.cpp:431-557). Returns out[T,H] (and a dict of intermediates)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    keep = [np.ascontiguousarray(router, dtype=np.uint16), np.ascontiguousarray(shared_gate, dtype=np.uint16),
            np.ascontiguousarray(shared_record, dtype=np.uint8), np.ascontiguousarray(expert_records, dtype=np.uint8)]
    off = None if router_offsets is None else np.ascontiguousarray(router_offsets, dtype=np.float32)
    layer = Layer(_p(keep[0]), _p(off), _p(keep[1]), _p(keep[2]), _p(keep[3]), record_stride)
    out = np.empty((tokens, cfg.hidden), np.float32)
    tr, tp = None, None
    if trace:
        n = tokens * cfg.topk
        tr = dict(logits=np.empty((tokens, cfg.experts), np.float32), ids=np.empty((tokens, cfg.topk), np.int32),
                  weights=np.empty((tokens, cfg.topk), np.float32), expert_out=np.empty((n, cfg.hidden), np.float32),
                  shared=np.empty((tokens, cfg.hidden), np.float32), gate=np.empty(tokens, np.float32))
        tp = Trace(*[_p(tr[k]) for k in ("logits", "ids", "weights", "expert_out", "shared", "gate")])
    status = lib.zco_moe_layer(C.byref(cfg), C.byref(layer), _p(x), C.c_uint32(tokens), _p(out),
                               C.byref(tp) if tp else None, C.c_int(threads))
    if status:
        raise RuntimeError("invalid router output")
    return (out, tr) if trace else out


# ---- the callers' glue either side of the layer


def unary(x, op):
    x = np.ascontiguousarray(x, dtype=np.float32); y = np.empty_like(x)
    lib.zco_unary_n(_p(x), C.c_uint64(x.size), C.c_uint32(op), _p(y))
    return y


def binary(x, y, op):
    x = np.ascontiguousarray(x, dtype=np.float32); y = np.ascontiguousarray(y, dtype=np.float32); out = np.empty_like(x)
    lib.zco_binary_n(_p(x), _p(y), C.c_uint64(x.size), C.c_uint32(op), _p(out))
    return out


def hc_mix(x, w, tokens, hidden):
    x = np.ascontiguousarray(x, dtype=np.float32); w = np.ascontiguousarray(w, dtype=np.float32)
    out = np.empty((tokens, hidden), np.float32)
    lib.zco_hc_mix(_p(x), _p(w), C.c_uint32(tokens), C.c_uint32(hidden), _p(out))
    return out


def hc_add(hyper, x, inject, tokens, hidden):
    a = [np.ascontiguousarray(v, dtype=np.float32) for v in (hyper, x, inject)]
    out = np.empty((tokens, 4, hidden), np.float32)
    lib.zco_hc_add(_p(a[0]), _p(a[1]), _p(a[2]), C.c_uint32(tokens), C.c_uint32(hidden), _p(out))
    return out


def norm(x, w, group, width, tokens):
    """w: uint16 (BF16 bits) or float32 weights of length width."""
    x = np.ascontiguousarray(x, dtype=np.float32); w = np.ascontiguousarray(w)
    dtype = 1 if w.dtype == np.float32 else 0
    out = np.empty(tokens * width, np.float32)
    lib.zco_norm(_p(x), _p(w), C.c_uint32(dtype), C.c_uint32(group), C.c_uint32(width), C.c_uint32(tokens), _p(out))
    return out
