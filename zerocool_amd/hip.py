"""ctypes face of the C ABI in include/zc_hip.h.  Device memory is owned by the
context (`Context.alloc`), addressed by plain integers wrapped in `DevBuf`."""
import ctypes as C
import os
import numpy as np

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libzc_hip.so")
_lib = None


class ZcError(RuntimeError):
    """Raised for any non-zero zc_status; `.status` keeps the code (1 invalid argument,
    2 runtime error, 3 logic error, 4 out of range, 5 budget exceeded)."""

    def __init__(self, status, text):
        super().__init__(text)
        self.status = status


class Linear(C.Structure):
    _fields_ = [("weight", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p),
                ("input", C.c_uint32), ("output", C.c_uint32), ("group", C.c_uint32), ("dtype", C.c_uint32),
                ("quantized", C.c_uint32), ("bits", C.c_uint32)]


class Config(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("hidden", "experts", "topk", "inter", "group", "bits_gate_up",
                                          "bits_down", "shared_bits_gate_up", "shared_bits_down")]


class Layer(C.Structure):
    _fields_ = [("router", C.c_void_p), ("router_offsets", C.c_void_p), ("shared_gate", C.c_void_p),
                ("shared_record", C.c_void_p), ("expert_records", C.c_void_p), ("record_stride", C.c_uint64)]


class StackTrace(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("ids", "weights", "outputs", "clocks")]


class Trace(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("logits", "ids", "weights", "expert_out", "shared", "gate")]


def load_library():
    """Loads libzc_hip.so; there is no fallback path."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
    lib = C.CDLL(LIB_PATH)
    lib.zc_hip_last_error.restype = C.c_char_p
    lib.zc_hip_version.restype = C.c_char_p
    for name in ("zc_hip_allocated", "zc_hip_peak", "zc_hip_moe_workspace_bytes", "zc_hip_moe_prefill_workspace_bytes", "zc_hip_projection_bytes",
                 "zc_hip_record_bytes", "zc_hip_moe_static_scratch_bytes", "zc_hip_store_stride", "zc_hip_store_capacity", "zc_hip_store_occupancy",
                 "zc_hip_store_protected_entries"):
        getattr(lib, name).restype = C.c_uint64
    lib.zc_hip_store_policy.restype = C.c_char_p
    lib.zc_hip_store_policy.argtypes = [C.c_void_p]
    lib.zc_hip_store_protected_entries.argtypes = [C.c_void_p]
    lib.zc_hip_stream.restype = C.c_void_p
    lib.zc_hip_store_backing.restype = C.c_void_p
    for name in ("zc_hip_store_backing", "zc_hip_store_stride", "zc_hip_store_capacity", "zc_hip_store_occupancy"):
        getattr(lib, name).argtypes = [C.c_void_p] + ([C.c_uint32, C.c_uint32] if name.endswith("backing") else [])
    lib.zc_hip_projection_bytes.argtypes = [C.c_uint32] * 4
    _lib = lib
    return lib


class StoreStats(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("hits", "misses", "evictions", "bytes", "ready_hits", "loading_joins",
                                          "prefetches", "prefetch_claims", "prefetch_unclaimed")]


class StoreTableStats(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("reads", "slot_reads", "home_reads", "home_read_bytes", "switched", "joined", "not_admitted")]


class StoreLease(C.Structure):
    _fields_ = [("lease", C.c_uint64), ("record", C.c_void_p), ("acquisition", C.c_int32)]


class Store:
    """Expert store (zc_hip_store_*): records live in pinned host memory, `slots` HBM slots cache them.  ctx=None gives a
    store with host-memory slots whose fills can be held back, for tests of the policy without a GPU."""

    ACQUISITIONS = ("new_miss", "ready_hit", "loading_join")

    def __init__(self, ctx, layers, experts, record_bytes, slots, policy="clock", home_layers=None):
        self.lib = load_library()
        self.ctx, self.layers, self.experts, self.record_bytes = ctx, layers, experts, record_bytes
        self.handle = C.c_void_p()
        self._check(self.lib.zc_hip_store_create_shared_homes(ctx.handle if ctx else None, C.c_uint32(layers), C.c_uint32(experts),
                                                              C.c_uint64(record_bytes), C.c_uint64(slots), policy.encode(),
                                                              C.c_uint32(home_layers or layers), C.byref(self.handle)))

    def _check(self, status):
        if status:
            raise ZcError(status, self.lib.zc_hip_last_error().decode())

    def close(self):
        if self.handle:
            self.lib.zc_hip_store_destroy(self.handle)
            self.handle = C.c_void_p()

    def backing(self, layer, expert):
        """The record's home in (pinned) host memory as a writable numpy byte array."""
        p = self.lib.zc_hip_store_backing(self.handle, layer, expert)
        if not p:
            raise IndexError("invalid expert id")
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(self.record_bytes,))

    def acquire(self, layer, expert):
        lease = StoreLease()
        self._check(self.lib.zc_hip_store_acquire(self.handle, C.c_uint32(layer), C.c_uint32(expert), C.byref(lease)))
        return lease

    def wait(self, lease):
        self._check(self.lib.zc_hip_store_wait(self.handle, C.c_uint64(lease.lease)))
        return DevBuf(self.ctx, lease.record, self.record_bytes) if self.ctx else lease.record

    def release(self, lease):
        self._check(self.lib.zc_hip_store_release(self.handle, C.c_uint64(lease.lease)))

    def prefetch(self, layer, expert):
        issued = C.c_int(0)
        self._check(self.lib.zc_hip_store_prefetch(self.handle, C.c_uint32(layer), C.c_uint32(expert), C.byref(issued)))
        return bool(issued.value)

    def ready(self, layer, expert):
        return bool(self.lib.zc_hip_store_ready(self.handle, C.c_uint32(layer), C.c_uint32(expert)))

    def hold(self, layer, expert, hold=True):
        self._check(self.lib.zc_hip_store_hold(self.handle, C.c_uint32(layer), C.c_uint32(expert), C.c_int(int(hold))))

    def clear(self):
        self._check(self.lib.zc_hip_store_clear(self.handle))

    def resize(self, slots):
        self._check(self.lib.zc_hip_store_resize(self.handle, C.c_uint64(slots)))

    @property
    def capacity(self):
        return self.lib.zc_hip_store_capacity(self.handle)

    @property
    def policy(self):
        return self.lib.zc_hip_store_policy(self.handle).decode()

    @property
    def protected_entries(self):
        return self.lib.zc_hip_store_protected_entries(self.handle)

    @property
    def occupancy(self):
        return self.lib.zc_hip_store_occupancy(self.handle)

    @property
    def stride(self):
        return self.lib.zc_hip_store_stride(self.handle)

    def stats(self):
        st = StoreStats()
        self._check(self.lib.zc_hip_store_stats(self.handle, C.byref(st)))
        return st

    def layer_stats(self, layer):
        h, m = C.c_uint64(), C.c_uint64()
        self._check(self.lib.zc_hip_store_layer_stats(self.handle, C.c_uint32(layer), C.byref(h), C.byref(m)))
        return h.value, m.value

    # the device-side view: a table of record addresses that kernels read
    def table(self):
        """Address of the table (creates it; the store must still be empty)."""
        t = C.c_void_p()
        self._check(self.lib.zc_hip_store_table(self.handle, C.byref(t)))
        return t.value

    def table_entries(self):
        """Host-memory stores: the table as an array of addresses."""
        return np.ctypeslib.as_array(C.cast(self.table(), C.POINTER(C.c_uint64)), shape=(self.layers * self.experts,))

    def table_refresh(self):
        self._check(self.lib.zc_hip_store_table_refresh(self.handle))

    def table_refresh_joining(self):
        self._check(self.lib.zc_hip_store_table_refresh_joining(self.handle))

    def table_observe(self, layer, ids):
        ids = np.ascontiguousarray(ids, np.int32)
        self._check(self.lib.zc_hip_store_table_observe(self.handle, C.c_uint32(layer), ids.ctypes.data_as(C.c_void_p), C.c_uint32(ids.size)))

    def table_observe_layers(self, ids):
        """ids [layers][per_layer]: what one launch through all layers chose."""
        ids = np.ascontiguousarray(ids, np.int32).reshape(self.layers, -1)
        self._check(self.lib.zc_hip_store_table_observe_layers(self.handle, ids.ctypes.data_as(C.c_void_p), C.c_uint32(ids.shape[1])))

    def table_stats(self):
        st = StoreTableStats()
        self._check(self.lib.zc_hip_store_table_stats(self.handle, C.byref(st)))
        return st

    def slot_bytes(self, lease):
        """Host-memory stores: the slot's current bytes."""
        return np.ctypeslib.as_array(C.cast(lease.record, C.POINTER(C.c_uint8)), shape=(self.record_bytes,))


class DevBuf:
    """A device allocation (or a view into one)."""

    def __init__(self, ctx, ptr, nbytes, owner=None):
        self.ctx, self.ptr, self.nbytes, self.owner = ctx, ptr, nbytes, owner

    def view(self, offset, nbytes=None):
        nbytes = self.nbytes - offset if nbytes is None else nbytes
        assert 0 <= offset and offset + nbytes <= self.nbytes
        return DevBuf(self.ctx, self.ptr + offset, nbytes, self.owner or self)

    def numpy(self, dtype, count=None):
        dtype = np.dtype(dtype)
        count = self.nbytes // dtype.itemsize if count is None else count
        out = np.empty(count, dtype)
        self.ctx._call("zc_hip_download", out.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr), C.c_uint64(out.nbytes))
        return out


def _ptr(b):
    if b is None:
        return C.c_void_p(None)
    return C.c_void_p(b.ptr if isinstance(b, DevBuf) else int(b))


class Context:
    def __init__(self, device=0, budget=0):
        self.lib = load_library()
        self.handle = C.c_void_p()
        self._check(self.lib.zc_hip_create(C.c_int(device), C.c_uint64(budget), C.byref(self.handle)))

    def close(self):
        if self.handle:
            self.lib.zc_hip_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, status):
        if status:
            raise ZcError(status, self.lib.zc_hip_last_error().decode())

    def _call(self, name, *args):
        self._check(getattr(self.lib, name)(self.handle, *args))

    # memory --------------------------------------------------------------
    def alloc(self, nbytes):
        p = C.c_void_p()
        self._call("zc_hip_alloc", C.c_uint64(nbytes), C.byref(p))
        return DevBuf(self, p.value, nbytes)

    def free(self, buf):
        self._call("zc_hip_free", C.c_void_p(buf.ptr))

    def zeros(self, nbytes):
        b = self.alloc(nbytes)
        self._call("zc_hip_memset", _ptr(b), C.c_int(0), C.c_uint64(nbytes))
        return b

    def fill(self, buf, byte):
        self._call("zc_hip_memset", _ptr(buf), C.c_int(byte), C.c_uint64(buf.nbytes))

    def copy(self, dst, src, nbytes):
        """Device-to-device copy on the context's stream."""
        self._call("zc_hip_copy", _ptr(dst), _ptr(src), C.c_uint64(nbytes))

    def upload(self, array, into=None):
        a = np.ascontiguousarray(array)
        b = into or self.alloc(max(a.nbytes, 4))
        self._call("zc_hip_upload", _ptr(b), a.ctypes.data_as(C.c_void_p), C.c_uint64(a.nbytes))
        return b

    def timer_start(self):
        self._call("zc_hip_timer_start")

    def timer_stop(self):
        ms = C.c_float()
        self._call("zc_hip_timer_stop", C.byref(ms))
        return ms.value

    def configure(self, affine_policy):
        """0: literal lane kernels everywhere; 1 (default): exact-integer matrix-core kernels where the shape allows."""
        self._call("zc_hip_configure", C.c_uint32(affine_policy))

    def finish(self):
        self._call("zc_hip_finish")

    def submit(self):
        t = C.c_uint64()
        self._call("zc_hip_submit", C.byref(t))
        return t.value

    def wait(self, ticket):
        self._call("zc_hip_wait", C.c_uint64(ticket))

    @property
    def allocated(self):
        return self.lib.zc_hip_allocated(self.handle)

    @property
    def stream(self):
        return self.lib.zc_hip_stream(self.handle)

    # operators -----------------------------------------------------------
    def linear(self, l, x, tokens, float_output=False, out=None):
        out = out or self.alloc(tokens * l.output * 4)
        self._call("zc_hip_linear_into", C.byref(l), _ptr(x), C.c_uint32(tokens), _ptr(out), C.c_int(int(float_output)))
        return out

    def router_logits(self, w, x, tokens, hidden, experts, offsets=None, out=None):
        out = out or self.alloc(tokens * experts * 4)
        self._call("zc_hip_router_logits", _ptr(w), _ptr(x), C.c_uint32(tokens), C.c_uint32(hidden), C.c_uint32(experts),
                   _ptr(offsets), _ptr(out))
        return out

    def gated_linear(self, gate, up, x, x_rows, tokens, rows=None, out=None):
        out = out or self.alloc(tokens * gate.output * 4)
        self._call("zc_hip_gated_linear", C.byref(gate), C.byref(up), _ptr(x), C.c_uint32(x_rows), C.c_uint32(tokens),
                   _ptr(rows), _ptr(out))
        return out

    def route(self, logits, tokens, experts, topk=10):
        ids, w = self.alloc(tokens * topk * 4), self.alloc(tokens * topk * 4)
        self._call("zc_hip_route", _ptr(logits), C.c_uint32(tokens), C.c_uint32(experts), C.c_uint32(topk), _ptr(ids), _ptr(w))
        return ids, w

    def build_dispatch(self, ids, tokens, topk, experts):
        off, slots = self.alloc((experts + 1) * 4), self.zeros(tokens * topk * 4)
        sel, count, status = self.zeros(experts * 4), self.zeros(4), self.zeros(4)
        self._call("zc_hip_build_dispatch", _ptr(ids), C.c_uint32(tokens), C.c_uint32(topk), C.c_uint32(experts),
                   _ptr(off), _ptr(slots), _ptr(sel), _ptr(count), _ptr(status))
        return off, slots, sel, count, status

    def scatter_experts(self, x, positions, n, hidden, out):
        self._call("zc_hip_scatter_experts", _ptr(x), _ptr(positions), C.c_uint32(n), C.c_uint32(hidden), _ptr(out))

    def moe_sum(self, experts, weights, shared, gate, tokens, hidden, topk=10, out=None):
        out = out or self.alloc(tokens * hidden * 4)
        self._call("zc_hip_moe_sum", _ptr(experts), _ptr(weights), _ptr(shared), _ptr(gate), C.c_uint32(tokens),
                   C.c_uint32(hidden), C.c_uint32(topk), _ptr(out))
        return out

    # ---- the callers' glue either side of the layer
    def unary(self, x, n, op, out=None):
        out = out or self.alloc(n * 4)
        self._call("zc_hip_unary", _ptr(x), C.c_uint64(n), C.c_uint32(op), _ptr(out))
        return out

    def binary(self, x, y, n, op, out=None):
        out = out or self.alloc(n * 4)
        self._call("zc_hip_binary", _ptr(x), _ptr(y), C.c_uint64(n), C.c_uint32(op), _ptr(out))
        return out

    def hc_mix(self, x, w, tokens, hidden, out=None):
        out = out or self.alloc(tokens * hidden * 4)
        self._call("zc_hip_hc_mix", _ptr(x), _ptr(w), C.c_uint32(tokens), C.c_uint32(hidden), _ptr(out))
        return out

    def hc_add(self, hyper, x, inject, tokens, hidden, out=None):
        out = out or self.alloc(tokens * 4 * hidden * 4)
        self._call("zc_hip_hc_add", _ptr(hyper), _ptr(x), _ptr(inject), C.c_uint32(tokens), C.c_uint32(hidden), _ptr(out))
        return out

    def norm(self, x, w, dtype, group, width, tokens, out=None):
        out = out or self.alloc(tokens * width * 4)
        self._call("zc_hip_norm", _ptr(x), _ptr(w), C.c_uint32(dtype), C.c_uint32(group), C.c_uint32(width), C.c_uint32(tokens), _ptr(out))
        return out

    def grouped_experts(self, cfg, records, positions, x, out, scratch):
        n = len(records)
        recs = (C.c_void_p * max(n, 1))(*[r.ptr for r in records])
        pos = (C.c_uint32 * max(len(positions), 1))(*positions)
        self._call("zc_hip_grouped_experts", C.byref(cfg), recs, pos, C.c_uint32(n), _ptr(x), _ptr(out), _ptr(scratch))

    def expert_linear(self, cfg, record, projection, shared=False):
        l = Linear()
        self._check(self.lib.zc_hip_expert_linear(C.byref(cfg), C.c_int(int(shared)), _ptr(record), C.c_int(projection), C.byref(l)))
        return l

    def record_bytes(self, cfg, shared=False):
        return self.lib.zc_hip_record_bytes(C.byref(cfg), C.c_int(int(shared)))

    def moe_workspace_bytes(self, cfg, tokens):
        return self.lib.zc_hip_moe_workspace_bytes(C.byref(cfg), C.c_uint32(tokens))

    def moe_forward(self, cfg, layer, x, tokens, out, workspace, trace=None):
        self._call("zc_hip_moe_forward", C.byref(cfg), C.byref(layer), _ptr(x), C.c_uint32(tokens), _ptr(out),
                   _ptr(workspace), C.byref(trace) if trace is not None else None)

    def moe_forward_static(self, cfg, layer, x, tokens, out, trace=None):
        """zc_hip_moe_forward with its workspace in the library's static device array: allocates nothing."""
        self._call("zc_hip_moe_forward_static", C.byref(cfg), C.byref(layer), _ptr(x), C.c_uint32(tokens), _ptr(out),
                   C.byref(trace) if trace is not None else None)

    def moe_prefill_workspace_bytes(self, cfg, tokens):
        return self.lib.zc_hip_moe_prefill_workspace_bytes(C.byref(cfg), C.c_uint32(tokens))

    def moe_prefill(self, cfg, layer, x, tokens, out, workspace, trace=None):
        self._call("zc_hip_moe_prefill", C.byref(cfg), C.byref(layer), _ptr(x), C.c_uint32(tokens), _ptr(out),
                   _ptr(workspace), C.byref(trace) if trace is not None else None)

    def moe_check(self):
        self._call("zc_hip_moe_check")

    # statistics -----------------------------------------------------------
    def profile(self, on=True):
        self._call("zc_hip_profile", C.c_int(int(on)))

    def label(self, stage, layer=-1, tokens=0, offset=0):
        self._call("zc_hip_label", stage.encode(), C.c_int32(layer), C.c_uint32(tokens), C.c_uint32(offset))

    def stats(self, store=None):
        """The statistics object of zc_hip_stats (memory, profile rows, expert cache counters) as a dict."""
        import json
        needed = C.c_uint64(0)
        handle = store.handle if store is not None else None
        self.lib.zc_hip_stats(self.handle, handle, None, C.c_uint64(0), C.byref(needed))
        buf = C.create_string_buffer(needed.value)
        self._call("zc_hip_stats", handle, buf, C.c_uint64(needed.value), C.byref(needed))
        return json.loads(buf.value.decode())

    def stack_glue(self, y, tokens, hidden, out):
        self._call("zc_hip_stack_glue", _ptr(y), C.c_uint32(tokens), C.c_uint32(hidden), _ptr(out))

    def stack_create(self, cfg, layers, max_tokens):
        arr = (Layer * len(layers))(*layers)
        h = C.c_void_p()
        self._call("zc_hip_stack_create", C.byref(cfg), arr, C.c_uint32(len(layers)), C.c_uint32(max_tokens), C.byref(h))
        return h

    def stack_create_with_store(self, cfg, layers, max_tokens, store):
        arr = (Layer * len(layers))(*layers)
        h = C.c_void_p()
        self._call("zc_hip_stack_create_with_store", C.byref(cfg), arr, C.c_uint32(len(layers)), C.c_uint32(max_tokens), store.handle, C.byref(h))
        return h

    def stack_destroy(self, stack):
        self._call("zc_hip_stack_destroy", stack)

    def stack_decode(self, stack, x, tokens, out, trace=None, layered=False):
        self._call("zc_hip_stack_decode", stack, _ptr(x), C.c_uint32(tokens), _ptr(out),
                   C.byref(trace) if trace is not None else None, C.c_uint32(1 if layered else 0))

    def stack_set_speculation(self, stack, on):
        self._call("zc_hip_stack_set_speculation", stack, C.c_int(int(on)))

    def stack_settle(self, stack):
        self._call("zc_hip_stack_settle", stack)

    def stack_set_wait_limit(self, stack, polls):
        self._call("zc_hip_stack_set_wait_limit", stack, C.c_uint32(polls))

    def stack_is_persistent(self, stack, tokens):
        return bool(self.lib.zc_hip_stack_is_persistent(self.handle, stack, C.c_uint32(tokens)))

    # synthetic tensors ---------------------------------------------------
    def synth_words(self, dst, count, seed):
        self._call("zc_hip_synth_words", _ptr(dst), C.c_uint64(count), C.c_uint64(seed))

    def synth_scales(self, scales, biases, count, seed, lo, span, factor):
        self._call("zc_hip_synth_scales", _ptr(scales), _ptr(biases), C.c_uint64(count), C.c_uint64(seed),
                   C.c_float(lo), C.c_float(span), C.c_float(factor))

    def synth_normal_f32(self, dst, count, seed, sigma=1.0):
        self._call("zc_hip_synth_normal_f32", _ptr(dst), C.c_uint64(count), C.c_uint64(seed), C.c_float(sigma))

    def synth_normal_bf16(self, dst, count, seed, sigma=1.0):
        self._call("zc_hip_synth_normal_bf16", _ptr(dst), C.c_uint64(count), C.c_uint64(seed), C.c_float(sigma))

    def synth_records(self, cfg, records, stride, count, seed, shared=False):
        self._call("zc_hip_synth_records", C.byref(cfg), C.c_int(int(shared)), _ptr(records), C.c_uint64(stride),
                   C.c_uint32(count), C.c_uint64(seed))
