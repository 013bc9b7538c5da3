"""Expert store on the GPU: records travel from their pinned-host home into HBM slots on the side stream, and a layer
computed through a small number of slots equals the layer computed from HBM-resident records byte for byte."""
import numpy as np
import pytest
import zerocool_amd as z
from zerocool_amd import workload

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.fixture(scope="module")
def ctx():
    c = z.Context(0)
    yield c
    c.close()


def test_slots_hold_the_records_they_were_asked_for(ctx):
    record, experts = 4096 + 64, 40
    s = z.Store(ctx, 2, experts, record, 4)
    rng = np.random.default_rng(5)
    for l in range(2):
        for e in range(experts):
            s.backing(l, e)[:] = rng.integers(0, 256, record, dtype=np.uint8)
    for step in range(200):
        l, e = int(rng.integers(0, 2)), int(rng.integers(0, experts))
        lease = s.acquire(l, e)
        slot = s.wait(lease)
        got = slot.numpy(np.uint8)          # a download on the compute stream: ordered after the fill by the wait above
        assert got.tobytes() == s.backing(l, e).tobytes(), (step, l, e)
        s.release(lease)
    st = s.stats()
    assert st.hits + st.misses == 200 and st.evictions >= st.misses - 4 and st.bytes == st.misses * record
    assert sum(s.layer_stats(l)[1] for l in range(2)) == st.misses
    with pytest.raises(z.ZcError):
        s.hold(0, 0)                        # only stores without a context can hold fills back
    s.close()


def test_leases_pin_slots_on_the_gpu(ctx):
    s = z.Store(ctx, 1, 8, 1024, 2)
    for e in range(8):
        s.backing(0, e)[:] = e + 1
    a, b = s.acquire(0, 0), s.acquire(0, 1)
    with pytest.raises(z.ZcError) as err:
        s.acquire(0, 2)
    assert "exhausted by outstanding leases" in str(err.value)
    s.release(b)
    c = s.acquire(0, 2)
    assert s.wait(a).numpy(np.uint8)[0] == 1 and s.wait(c).numpy(np.uint8)[0] == 3
    s.release(a); s.release(c)
    assert s.prefetch(0, 5) is True
    ctx.finish()
    hit = s.acquire(0, 5)
    assert hit.acquisition in (1, 2) and s.stats().prefetch_claims == 1
    assert s.wait(hit).numpy(np.uint8)[0] == 6
    s.release(hit)
    s.resize(4)
    assert s.ready(0, 5) and s.wait(s.acquire(0, 5)).numpy(np.uint8)[0] == 6   # survivors keep their bytes across a resize
    s.close()


@pytest.mark.parametrize("tokens", [1, 5])
def test_layer_through_capped_slots_equals_resident_layer(ctx, tokens):
    cfg = workload.tiny_config(hidden=512, experts=32, topk=4, inter=128)
    seeds = [41, 42]
    capped = workload.StoreBackedStack(ctx, cfg, seeds, ("normal", 0.5), slots=6)   # 64 records, six slots
    for l, seed in enumerate(seeds):
        resident = workload.LayerWeights(ctx, cfg, seed, ("normal", 0.5))
        for step in range(3):
            x = workload.hidden_rows(ctx, tokens, cfg.hidden, 900 + 10 * l + step)
            want = ctx.alloc(tokens * cfg.hidden * 4)
            ws = ctx.alloc(ctx.moe_workspace_bytes(cfg, tokens))
            ids = ctx.alloc(tokens * cfg.topk * 4)
            ctx.moe_forward(cfg, resident.layer, x, tokens, want, ws, z.Trace(None, ids.ptr, None, None, None, None))
            ctx.moe_check()
            got, host_ids = capped.layer_forward(l, x, tokens)
            assert host_ids.tobytes() == ids.numpy(np.int32).tobytes()
            assert got.numpy(f32).tobytes() == want.numpy(f32).tobytes()
    st = capped.store.stats()
    assert st.misses > 6 and st.evictions > 0 and st.hits + st.misses > 0
    capped.close()


def test_capped_layer_at_the_stack_shape_against_the_oracle(ctx):
    # One layer of the 48-layer configuration (hidden 3072, intermediate 1024, 512 experts, top-10) whose 512 records live
    # in pinned host memory with 24 HBM slots in front of them, checked against the CPU oracle, which reads the records'
    # home directly: routing ids and output bytes.
    import ctypes as C
    import oracle
    cfg = workload.config("F")
    capped = workload.StoreBackedStack(ctx, cfg, [71], ("zipf", 1.1), slots=24)
    w = capped.layers[0]
    stride = capped.store.stride
    home = capped.store.lib.zc_hip_store_backing(capped.store.handle, 0, 0)
    records = np.ctypeslib.as_array(C.cast(home, C.POINTER(C.c_uint8)), shape=(cfg.experts * stride,))
    ocfg = oracle.Config(*[getattr(cfg, n) for n, _ in z.Config._fields_])
    for tokens, seed in ((1, 5), (3, 6), (1, 7)):
        x = workload.hidden_rows(ctx, tokens, cfg.hidden, 950 + seed)
        got, host_ids = capped.layer_forward(0, x, tokens)
        want, tr = oracle.moe_layer(ocfg, w.router.numpy(np.uint16), w.shared_gate.numpy(np.uint16), w.shared_record.numpy(np.uint8),
                                    records, stride, x.numpy(f32), tokens, router_offsets=w.offsets_host, threads=16, trace=True)
        assert host_ids.tobytes() == tr["ids"].tobytes(), "routing ids differ from the oracle"
        g = got.numpy(f32).reshape(tokens, cfg.hidden)
        assert float(np.max(np.abs(g - want)) / np.max(np.abs(want))) <= 2e-3
        assert g.tobytes() == want.tobytes()
    st = capped.store.stats()
    assert st.misses >= 10 and st.hits > 0      # the second and third steps find most of their experts in the slots
    capped.close()


def _stack_pair(ctx, cfg, seeds, skew, slots):
    """The same layers twice: records resident in HBM, and records behind an expert store with `slots` HBM slots."""
    resident = [workload.LayerWeights(ctx, cfg, seed, skew) for seed in seeds]
    capped = workload.StoreBackedStack(ctx, cfg, seeds, skew, slots)
    return resident, ctx.stack_create(cfg, [w.layer for w in resident], 24), capped, capped.decode_stack(24)


def test_decode_stack_behind_a_store_equals_the_resident_stack(ctx):
    # Three layers of 32 experts (96 records) behind ten HBM slots: every launch reads some records from their slots and
    # the others from their pinned-host homes, fills follow between the launches, slots are given away again and again.
    # The bytes must be those of the stack whose records all sit in HBM, at one token and at several, launch after launch.
    cfg = workload.tiny_config(hidden=512, experts=32, topk=4, inter=512)
    resident, full, capped, stack = _stack_pair(ctx, cfg, [51, 52, 53], ("normal", 0.5), slots=10)
    assert ctx.stack_is_persistent(stack, 1) and ctx.stack_is_persistent(stack, 8)
    n = 3 * 24 * cfg.topk
    ids_a, w_a, ids_b, w_b = (ctx.alloc(n * 4) for _ in range(4))
    for step, tokens in enumerate((1, 1, 3, 1, 8, 1, 1, 2, 1, 24, 1, 5, 1, 13, 1)):
        x = workload.hidden_rows(ctx, tokens, cfg.hidden, 7000 + step)
        want, got = ctx.alloc(tokens * cfg.hidden * 4), ctx.alloc(tokens * cfg.hidden * 4)
        traced = step % 2 == 0   # with the caller's trace buffers and with the stack's own
        ctx.stack_decode(full, x, tokens, want, z.StackTrace(ids_a.ptr, w_a.ptr, None, None))
        ctx.stack_decode(stack, x, tokens, got, z.StackTrace(ids_b.ptr, w_b.ptr, None, None) if traced else None)
        ctx.moe_check()
        assert got.numpy(f32).tobytes() == want.numpy(f32).tobytes(), f"step {step} ({tokens} tokens)"
        if traced:
            m = 3 * tokens * cfg.topk
            assert ids_b.numpy(np.int32, m).tobytes() == ids_a.numpy(np.int32, m).tobytes()
        for b in (x, want, got):
            ctx.free(b)
    ctx.stack_settle(stack)   # the last launch's routes, if the store has not seen them yet
    seen, st = capped.store.table_stats(), capped.store.stats()
    assert seen.reads == seen.slot_reads + seen.home_reads and seen.slot_reads > 0 and seen.home_reads > 10
    assert seen.home_read_bytes == seen.home_reads * ctx.record_bytes(cfg)
    assert seen.switched > 10 and st.evictions > 0 and st.misses + st.hits + seen.not_admitted == seen.reads
    with pytest.raises(z.ZcError):   # layer by layer would need every record resident
        x = workload.hidden_rows(ctx, 1, cfg.hidden, 1)
        ctx.stack_decode(stack, x, 1, ids_a, layered=True)
    ctx.stack_destroy(stack); ctx.stack_destroy(full)
    capped.close()


def test_stack_shape_behind_a_store(ctx):
    # Two layers of the 48-layer configuration behind 40 slots (1024 records of 5.3 MB): a cold launch that reads all of its
    # records over the host link, then launches that find them in HBM.
    cfg = workload.config("F")
    resident, full, capped, stack = _stack_pair(ctx, cfg, [81, 82], ("zipf", 1.1), slots=40)
    for step, tokens in enumerate((1, 1, 8, 1)):
        x = workload.hidden_rows(ctx, tokens, cfg.hidden, 7100 + step)
        want, got = ctx.alloc(tokens * cfg.hidden * 4), ctx.alloc(tokens * cfg.hidden * 4)
        ctx.stack_decode(full, x, tokens, want)
        ctx.stack_decode(stack, x, tokens, got)
        ctx.finish()   # the fills that the launch caused are given time to land
        ctx.moe_check()
        assert got.numpy(f32).tobytes() == want.numpy(f32).tobytes(), f"step {step} ({tokens} tokens)"
    ctx.stack_settle(stack)
    seen = capped.store.table_stats()
    assert seen.home_reads >= 20 and seen.slot_reads > 0 and seen.joined + seen.switched > 0
    ctx.stack_destroy(stack); ctx.stack_destroy(full)
    capped.close()
