"""Synthetic MoE layers of the benchmark configurations, generated on the device.

Shapes: S = one layer (hidden 2048, 512 experts, top-10, intermediate 512, group 64);
F = one layer of the 48-layer stand-in stack (hidden 3072, intermediate 1024).
Routed records are affine Q4 (codes uniform 0..15, BF16 scale ~U(0.002,0.02), bias -8*scale);
the mixed artifact keeps gate/up Q4 and makes down + the shared expert affine Q8
(scale ~U(0.0002,0.002), bias -128*scale)."""
import ctypes as C
import math
import numpy as np
from . import synth
from .hip import Config, Layer

BASE_SEED = 0x5EED


def config(name):
    if name == "S":
        return Config(2048, 512, 10, 512, 64, 4, 4, 4, 4)
    if name == "S-mixed":
        return Config(2048, 512, 10, 512, 64, 4, 8, 8, 8)
    if name == "F":
        return Config(3072, 512, 10, 1024, 64, 4, 4, 4, 4)
    if name == "ref":   # the reference's own shape (storage.hpp:26-27)
        return Config(2560, 512, 10, 640, 64, 4, 4, 4, 4)
    raise KeyError(name)


def tiny_config(hidden=512, experts=32, topk=4, inter=128, group=64, bits=(4, 4, 4, 4)):
    return Config(hidden, experts, topk, inter, group, *bits)


def record_stride(ctx, cfg):
    return (ctx.record_bytes(cfg) + 255) // 256 * 256


class LayerWeights:
    """Device buffers of one layer plus the zc_moe_layer that points at them."""

    def __init__(self, ctx, cfg, seed, skew=None, records=None, keep_records=False):
        H, E = cfg.hidden, cfg.experts
        self.ctx, self.cfg, self.seed = ctx, cfg, seed
        self.stride = record_stride(ctx, cfg)
        self.router = ctx.alloc(E * H * 2)
        self.shared_gate = ctx.alloc(H * 2)
        self.shared_record = ctx.alloc(ctx.record_bytes(cfg, shared=True))
        self.records = records if records is not None else ctx.alloc(E * self.stride)
        sigma = 1.0 / math.sqrt(H)
        ctx.synth_normal_bf16(self.router, E * H, seed * 16 + 1, sigma)
        ctx.synth_normal_bf16(self.shared_gate, H, seed * 16 + 2, sigma)
        ctx.synth_records(cfg, self.shared_record, self.shared_record.nbytes, 1, seed * 16 + 3, shared=True)
        if not keep_records:   # (keep_records: the buffer already holds another layer's records, which this layer shares)
            ctx.synth_records(cfg, self.records, self.stride, E, (seed * 16 + 4) * 4096)
        self.offsets_host = None
        if skew is not None:
            kind, value = skew
            self.offsets_host = (synth.normal_offsets(E, seed * 16 + 5, value) if kind == "normal"
                                 else synth.zipf_offsets(E, seed * 16 + 5, value))
        self.offsets = ctx.upload(self.offsets_host) if self.offsets_host is not None else None
        self.layer = Layer(self.router.ptr, self.offsets.ptr if self.offsets else None, self.shared_gate.ptr,
                           self.shared_record.ptr, self.records.ptr, self.stride)

    def host(self):
        """Host copies for the CPU checker: router, shared_gate (uint16), records (uint8)."""
        return dict(router=self.router.numpy(np.uint16), shared_gate=self.shared_gate.numpy(np.uint16),
                    shared_record=self.shared_record.numpy(np.uint8), records=self.records.numpy(np.uint8),
                    offsets=self.offsets_host, stride=self.stride)


def hidden_rows(ctx, tokens, hidden, seed):
    x = ctx.alloc(tokens * hidden * 4)
    ctx.synth_normal_f32(x, tokens * hidden, seed, 1.0)
    return x


def layer_bytes(cfg, unique_experts, tokens, ctx):
    """Algorithmic bytes of one layer step: router + shared gate + U routed records +
    shared record + activations in/out + route ids/weights."""
    H, E, k = cfg.hidden, cfg.experts, cfg.topk
    return (2 * H * E + 2 * H + unique_experts * ctx.record_bytes(cfg) + ctx.record_bytes(cfg, shared=True)
            + tokens * 4 * H + tokens * k * 8)


class StoreBackedStack:
    """A stack of layers whose routed records live in an expert store: the home of every record is pinned host
    memory, `slots` HBM slots cache the records in use (the capped-HBM run of the 48-layer configuration).  The layer
    step is the reference's orchestration (src/engine/model.cpp:431-557): router, route, ONE readback of the ids,
    leases for the selected experts (fills on the store's side stream), per-expert gate/up + down into the expert's
    slots, shared expert, weighted combine; leases are released once the step's GPU work has finished."""

    def __init__(self, ctx, cfg, seeds, skew, slots, home_layers=None):
        """home_layers < len(seeds): layer l shares its records' home with layer l - home_layers (routers, shared experts
        and router offsets stay every layer's own), for hosts that cannot pin all records."""
        from .hip import Store, DevBuf
        self.ctx, self.cfg = ctx, cfg
        home_layers = home_layers or len(seeds)
        self.store = Store(ctx, len(seeds), cfg.experts, ctx.record_bytes(cfg), slots, home_layers=home_layers)
        assert self.store.stride == record_stride(ctx, cfg)
        self.layers = []
        for l, seed in enumerate(seeds):
            home = self.store.lib.zc_hip_store_backing(self.store.handle, l, 0)
            # the generator kernel writes the records straight into their pinned-host home (mapped into the GPU)
            records = DevBuf(ctx, home, cfg.experts * self.store.stride)
            self.layers.append(LayerWeights(ctx, cfg, seed, skew, records=records, keep_records=l >= home_layers))
        ctx.finish()

    def close(self):
        self.store.close()

    def decode_stack(self, max_tokens=8):
        """The single-launch decode stack over this store (zc_hip_stack_create_with_store)."""
        return self.ctx.stack_create_with_store(self.cfg, [w.layer for w in self.layers], max_tokens, self.store)

    def layer_forward(self, l, x, T):
        ctx, cfg, w = self.ctx, self.cfg, self.layers[l]
        H, E, k, I = cfg.hidden, cfg.experts, cfg.topk, cfg.inter
        logits = ctx.router_logits(w.router, x, T, H, E, w.offsets)
        ids, weights = ctx.route(logits, T, E, k)
        host_ids = ids.numpy(np.int32)                      # the one readback (model.cpp:446)
        if ((host_ids < 0) | (host_ids >= E)).any():
            raise RuntimeError("invalid router output")     # model.cpp:459
        order = np.argsort(host_ids, kind="stable")          # slots grouped by expert, ascending slot inside an expert
        selected, starts = np.unique(host_ids[order], return_index=True)
        expert_out = ctx.alloc(T * k * H * 4)
        temporaries = [logits, ids, weights, expert_out]
        bounds = list(starts) + [len(order)]
        group = max(1, min(int(self.store.capacity), 32))   # leases out at once (pipeline.cpp:71-220 works in such groups)
        for g0 in range(0, len(selected), group):
            batch = range(g0, min(g0 + group, len(selected)))
            leases = [self.store.acquire(l, int(selected[j])) for j in batch]   # fills start on the side stream
            for j, lease in zip(batch, leases):
                record = self.store.wait(lease)              # the compute stream waits for the slot's fill, the host does not
                slots = order[bounds[j]:bounds[j + 1]].astype(np.int32)
                rows = ctx.upload((slots // k).astype(np.int32))
                act = ctx.gated_linear(ctx.expert_linear(cfg, record, 0), ctx.expert_linear(cfg, record, 1), x, T, len(slots), rows)
                if len(slots) == 1:                          # direct rows (model.cpp:527-531)
                    ctx.linear(ctx.expert_linear(cfg, record, 2), act, 1, out=expert_out.view(int(slots[0]) * H * 4, H * 4))
                    temporaries += [rows, act]
                else:                                        # encode_expert_rows (pipeline.cpp:7-31)
                    y = ctx.linear(ctx.expert_linear(cfg, record, 2), act, len(slots))
                    positions = ctx.upload(slots)
                    ctx.scatter_experts(y, positions, len(slots), H, expert_out)
                    temporaries += [rows, act, y, positions]
            ctx.finish()                                     # GPU users of the slots are done: the leases may go
            for lease in leases:
                self.store.release(lease)
        sact = ctx.gated_linear(ctx.expert_linear(cfg, w.shared_record, 0, shared=True), ctx.expert_linear(cfg, w.shared_record, 1, shared=True), x, T, T)
        shared = ctx.linear(ctx.expert_linear(cfg, w.shared_record, 2, shared=True), sact, T)
        from .hip import Linear
        gate = ctx.linear(Linear(w.shared_gate.ptr, None, None, H, 1, 64, 0, 0, 4), x, T)
        out = ctx.moe_sum(expert_out, weights, shared, gate, T, H, k)
        ctx.finish()
        for b in temporaries + [sact, shared, gate]:
            ctx.free(b)
        return out, host_ids
