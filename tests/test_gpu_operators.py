"""GPU parity of every operator of the path against the CPU oracle, through the C ABI.
Inputs restate the reference's own test cases (tests/test_qwen.cpp, cited per test).
The bar: byte equality with the oracle, for integer outputs and for floating point."""
import json
import math
import os
import numpy as np
import pytest
import oracle
import zerocool_amd as z
from zerocool_amd import synth, workload
from test_oracle_golden import route_stress_values, _router_case, G

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.fixture(scope="module")
def ctx():
    c = z.Context(0)
    yield c
    c.close()


def dev_linear(ctx, w, s, b, K, N, group=64, bits=4):
    bufs = (ctx.upload(w), ctx.upload(s), ctx.upload(b))
    l = z.Linear(bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, K, N, group, 0, 1, bits)
    l._keep = bufs
    return l


def same_bytes(a, b):
    return np.ascontiguousarray(a).tobytes() == np.ascontiguousarray(b).tobytes()


def test_device_generator_matches_host_statement(ctx):
    for count, seed in ((1, 1), (1001, 7), (65537, 0x5EED)):
        d = ctx.alloc(count * 4)
        ctx.synth_words(d, count, seed)
        assert same_bytes(d.numpy(np.uint32), synth.words(count, seed))
        ctx.synth_normal_f32(d, count, seed, 0.25)
        assert same_bytes(d.numpy(np.float32), synth.normal(count, seed, 0.25))
        h = ctx.alloc(count * 2)
        ctx.synth_normal_bf16(h, count, seed, 1.0)
        assert same_bytes(h.numpy(np.uint16), synth.bf_bits(synth.normal(count, seed, 1.0)))
        s, b = ctx.alloc(count * 2), ctx.alloc(count * 2)
        ctx.synth_scales(s, b, count, seed, 0.002, 0.018, -8.0)
        hs, hb = synth.scales(count, seed, 0.002, 0.018, -8.0)
        assert same_bytes(s.numpy(np.uint16), hs) and same_bytes(b.numpy(np.uint16), hb)


def test_q4_matmul_and_swiglu(ctx):  # :634-659
    K, N, T = 128, 7, 3
    w = np.array([(0x76543210 + (i % 8) * 0x11111111) & 0xffffffff for i in range(N * K // 8)], dtype=np.uint32)
    s = np.full(N * K // 64, 0x3d80, np.uint16); b = np.full(N * K // 64, 0xbe80, np.uint16)
    x = np.array([(i % 11 - 5) / 16 for i in range(T * K)], dtype=np.float32)
    ol = oracle.make_linear(w, s, b, K, N); dl = dev_linear(ctx, w, s, b, K, N); dx = ctx.upload(x)
    assert same_bytes(ctx.linear(dl, dx, T).numpy(f32), oracle.linear(ol, x, T))
    assert same_bytes(ctx.gated_linear(dl, dl, dx, T, T).numpy(f32), oracle.gated_linear(ol, ol, x, T))


def test_q4_bias_uses_bf16_sum_of_four(ctx):  # :863-874
    codes = np.zeros(16, np.uint32); sc = np.full(2, 0x3f80, np.uint16)
    x = np.zeros(128, f32); x[0::4] = 1; x[1::4] = 1.0 / 512; x[2::4] = -1
    out = ctx.linear(dev_linear(ctx, codes, sc, sc, 128, 1), ctx.upload(x), 1).numpy(f32)
    assert out[0] == 0.0


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("K,N,Gs", [(320, 7, 64), (640, 8, 32), (2560, 8, 64)])
def test_affine_shapes_tiles_and_gathered_rows(ctx, bits, K, N, Gs):  # :661-696 and :964-1010
    T = 9
    w = np.array([(i * 17 + 251) % 256 for i in range(K * N * bits // 8)], dtype=np.uint8)
    s = np.array([0xbb80 if i % 2 else 0x3b80 for i in range(K * N // Gs)], dtype=np.uint16)
    b = np.array([0xbf00 if i % 3 else 0x3e80 for i in range(K * N // Gs)], dtype=np.uint16)
    x = oracle.bf(np.array([(i % 29 - 14) / 128 for i in range(T * K)], dtype=f32))
    x[0], x[1], x[2] = 1, 1.0 / 512, -1          # BF16 input-sum ties
    rows = np.array([(T - i) % 4 for i in range(T)], dtype=np.int32)
    ol = oracle.make_linear(w, s, b, K, N, Gs, bits); dl = dev_linear(ctx, w, s, b, K, N, Gs, bits)
    dx = ctx.upload(x)
    assert same_bytes(ctx.linear(dl, dx, T).numpy(f32), oracle.linear(ol, x, T))
    assert same_bytes(ctx.linear(dl, dx, T, float_output=True).numpy(f32), oracle.linear(ol, x, T, float_output=True))
    assert same_bytes(ctx.gated_linear(dl, dl, dx, T, T).numpy(f32), oracle.gated_linear(ol, ol, x, T))
    assert same_bytes(ctx.gated_linear(dl, dl, dx, T, T, ctx.upload(rows)).numpy(f32), oracle.gated_linear(ol, ol, x, T, rows))
    if bits == 8:   # exact equality with the double-precision dot (:661-683)
        x3 = np.array([(i % 9 - 4) / 16 for i in range(3 * K)], dtype=f32)
        got = ctx.linear(dl, ctx.upload(x3), 3).numpy(f32).reshape(3, N)
        dec = (w.astype(f32).reshape(N, K) * np.repeat(oracle.b16(s).reshape(N, K // Gs), Gs, 1)
               + np.repeat(oracle.b16(b).reshape(N, K // Gs), Gs, 1)).astype(np.float64)
        assert same_bytes(got, oracle.bf((x3.astype(np.float64).reshape(3, K) @ dec.T).astype(f32)))
    # refusals (:688-694)
    bad = z.Linear(dl.weight, dl.scales, dl.biases, K, N, Gs, 0, 1, 3)
    with pytest.raises(z.ZcError):
        ctx.linear(bad, dx, T)
    with pytest.raises(z.ZcError):
        ctx.gated_linear(dl, dl, dx, T, 1, ctx.upload(np.array([T], np.int32)))
    ctx.finish()


@pytest.mark.parametrize("K,N", [(2560, 640), (640, 2560), (2560, 10240), (6144, 2560), (10240, 320), (320, 10240),
                                 (2560, 512), (512, 1024), (704, 2560), (2048, 512), (512, 2048), (3072, 1024), (1024, 3072)])
def test_single_token_rows(ctx, K, N):  # :1100-1125 shapes plus the benchmark shapes
    rng = np.random.default_rng(K * 31 + N)
    mk = lambda: (rng.integers(0, 2 ** 32, N * K // 8, dtype=np.uint64).astype(np.uint32),
                  oracle.bf_bits(0.01 * np.abs(rng.standard_normal(N * K // 64)) + 1e-4),
                  oracle.bf_bits(-0.08 * np.abs(rng.standard_normal(N * K // 64))))
    a, u = mk(), mk()
    x = oracle.bf(0.7 * rng.standard_normal(K))
    ol, ou = oracle.make_linear(*a, K, N), oracle.make_linear(*u, K, N)
    dl, du = dev_linear(ctx, *a, K, N), dev_linear(ctx, *u, K, N)
    dx = ctx.upload(x)
    assert same_bytes(ctx.linear(dl, dx, 1).numpy(f32), oracle.linear(ol, x, 1))
    assert same_bytes(ctx.linear(dl, dx, 1, float_output=True).numpy(f32), oracle.linear(ol, x, 1, float_output=True))
    assert same_bytes(ctx.gated_linear(dl, du, dx, 1, 1).numpy(f32), oracle.gated_linear(ol, ou, x, 1))
    for b in dl._keep + du._keep + (dx,):
        ctx.free(b)


# the last three: a row of sixteen-load and eight-load batches plus single steps, rows shorter than one batch, and an odd
# number of weights (their 16-bit words are then read one by one, not through aligned 32-bit words)
@pytest.mark.parametrize("K,N", [(10240, 4), (2560, 1), (2560, 48), (2048, 1), (3072, 1), (864, 5), (96, 2), (257, 3)])
def test_plain_rows(ctx, K, N):  # :1126-1135, the shared_expert_gate shape
    rng = np.random.default_rng(K + N)
    w = oracle.bf_bits(0.02 * rng.standard_normal(N * K)); x = oracle.bf(rng.standard_normal(2 * K))
    l = z.Linear(ctx.upload(w).ptr, None, None, K, N, 64, 0, 0, 4)
    got = ctx.linear(l, ctx.upload(x), 2).numpy(f32)
    assert same_bytes(got, oracle.plain_mm(w, x, K, N, 2))


def test_router_captured_words_and_chunks(ctx):  # :798-826
    r, T, K, N, w, x = _router_case()
    dw = ctx.upload(w)
    full = ctx.router_logits(dw, ctx.upload(x), T, K, N).numpy(f32)
    for i, e in zip(r["indices"], r["expected_bits"]):
        assert int(full[i:i + 1].view(np.uint32)[0]) == e
    assert same_bytes(full, oracle.router_logits(w, x, T, K, N))
    for offset, count in ((0, 1), (1, 7), (8, 3)):
        part = ctx.router_logits(dw, ctx.upload(x[offset:offset + count]), count, K, N).numpy(f32)
        assert same_bytes(part, full.reshape(T, N)[offset:offset + count])


# the last four reach the long-batch kernels: register-tiled (T >= 64) and LDS-staged (T >= 256, K % 512 == 0), with token and
# expert counts that do not fill the last tile
@pytest.mark.parametrize("H,E,T", [(2048, 512, 1), (2048, 512, 9), (3072, 512, 8), (512, 32, 5),
                                    (640, 40, 70), (2048, 512, 300), (512, 40, 257), (1024, 24, 1030)])
def test_router_random_with_offsets(ctx, H, E, T):
    w = synth.bf_bits(synth.normal(E * H, 3, 1 / math.sqrt(H))); x = synth.normal(T * H, 4)
    off = synth.normal_offsets(E, 5)
    got = ctx.router_logits(ctx.upload(w), ctx.upload(x), T, H, E, ctx.upload(off)).numpy(f32)
    assert same_bytes(got, oracle.router_logits(w, x, T, H, E, off))


def test_route_stress_rows(ctx):  # :744-797
    v = route_stress_values()
    T = v.shape[0]
    ids, w = ctx.route(ctx.upload(v), T, 512)
    oi, ow = oracle.route(v, T, 512)
    assert same_bytes(ids.numpy(np.int32), oi)
    assert same_bytes(w.numpy(f32), ow)            # NaN rows included: same NaN bits
    v1 = np.array([i % 41 - 100 for i in range(512)], dtype=f32)
    ids, w = ctx.route(ctx.upload(v1), 1, 512)
    assert same_bytes(ids.numpy(np.int32), oracle.route(v1, 1, 512)[0])
    assert float(np.sum(w.numpy(f32).astype(np.float64))) == pytest.approx(1, abs=1e-6)
    for bad_tokens in (0, 8193):
        with pytest.raises(z.ZcError):
            ctx.route(ctx.upload(v), bad_tokens, 512)


@pytest.mark.parametrize("T,E,k", [(1, 512, 10), (7, 512, 10), (64, 512, 10), (513, 512, 10), (2048, 512, 10), (5, 32, 4), (1000, 512, 10), (821, 64, 3), (2731, 130, 3)])
def test_dispatch_matches_counting_sort(ctx, T, E, k):  # model.cpp:449-479
    rng = np.random.default_rng(T)
    skew = rng.standard_normal(E) * 2
    ids = np.stack([np.argsort(-(rng.standard_normal(E) + skew), kind="stable")[:k] for _ in range(T)]).astype(np.int32)
    off, slots, sel, count, status = ctx.build_dispatch(ctx.upload(ids), T, k, E)
    o_off, o_slots, o_sel = oracle.dispatch(ids, T, k, E)
    assert same_bytes(off.numpy(np.int32), o_off) and same_bytes(slots.numpy(np.int32), o_slots)
    n = int(count.numpy(np.int32)[0])
    assert n == len(o_sel) and same_bytes(sel.numpy(np.int32)[:n], o_sel) and status.numpy(np.int32)[0] == 0
    if T * k > 1024:   # an id array that is only four-byte aligned (the long-batch kernels read sixteen bytes at a time when they can)
        shifted = ctx.upload(np.concatenate([np.zeros(1, np.int32), ids.reshape(-1)])).view(4)
        off2, slots2, _, _, _ = ctx.build_dispatch(shifted, T, k, E)
        assert same_bytes(off2.numpy(np.int32), o_off) and same_bytes(slots2.numpy(np.int32), o_slots)
    ids[T // 2, k - 1] = -1
    assert ctx.build_dispatch(ctx.upload(ids), T, k, E)[4].numpy(np.int32)[0] != 0
    ids[T // 2, k - 1] = E
    assert ctx.build_dispatch(ctx.upload(ids), T, k, E)[4].numpy(np.int32)[0] != 0


def test_moe_sum_midpoint_and_random(ctx):  # :827-842
    m = G["moe_sum"]; H = 2560
    e = np.zeros((10, H), f32); e[:, 0] = np.array(m["values"], dtype=f32)
    w = np.array(m["weight_bits"], dtype=np.uint32).view(f32)
    shared = np.zeros(H, f32); shared[0] = m["shared"]; gate = np.array([m["gate"]], f32)
    out = ctx.moe_sum(ctx.upload(e), ctx.upload(w), ctx.upload(shared), ctx.upload(gate), 1, H).numpy(f32)
    assert out[0] == m["expected"] and (out[1:] == 0).all()
    rng = np.random.default_rng(2)
    # widths that are and are not a multiple of four (four columns per thread or one), top-k at, below and above ten
    for T, Hh, k in ((5, 2048, 10), (3, 3072, 10), (4, 256, 4), (2, 250, 10), (2, 252, 12), (3, 1028, 10), (1, 17, 3)):
        e = oracle.bf(rng.standard_normal((T * k, Hh))); w = rng.random((T, k)).astype(f32)
        sh = oracle.bf(rng.standard_normal((T, Hh))); g = oracle.bf(rng.standard_normal(T) * 2)
        got = ctx.moe_sum(ctx.upload(e), ctx.upload(w), ctx.upload(sh), ctx.upload(g), T, Hh, k).numpy(f32)
        assert same_bytes(got, oracle.moe_sum(e, w, sh, g, T, Hh, k))


def expert_fixture(cfg, seed):
    """Closed-form record of tests/test_qwen.cpp:1074-1085 at a parameterised shape."""
    shapes = [(cfg.hidden, cfg.inter), (cfg.hidden, cfg.inter), (cfg.inter, cfg.hidden)]
    parts = []
    for p, (K, N) in enumerate(shapes):
        i = np.arange(K * N // 8, dtype=np.uint64)
        parts.append(((i * 2654435761 + (seed + p * 29) * 1234567) & 0xffffffff).astype(np.uint32).view(np.uint8))
        parts.append(np.full(K // 64 * N, 0x3b00 + p * 32, np.uint16).view(np.uint8))
        parts.append(np.full(K // 64 * N, 0xbc00 + p * 16, np.uint16).view(np.uint8))
    return np.concatenate(parts)


def test_direct_rows_preserve_other_destinations(ctx):  # :1087-1099
    cfg = workload.config("ref"); H, I, k = cfg.hidden, cfg.inter, cfg.topk
    rec = expert_fixture(cfg, 1); drec = ctx.upload(rec)
    x = np.array([(i % 23 - 11) / 32 for i in range(I)], dtype=f32); dx = ctx.upload(x)
    down = ctx.expert_linear(cfg, drec, 2)
    want = oracle.linear(oracle.expert_linear(cfg_o(cfg), rec, 2), x, 1)
    out = ctx.upload(np.full((k + 2) * H, -17, f32))
    for pos in range(k):
        ctx.linear(down, dx, 1, out=out.view((pos + 1) * H * 4, H * 4))
    got = out.numpy(f32).reshape(k + 2, H)
    for pos in range(k):
        assert same_bytes(got[pos + 1], want)
    assert (got[0] == -17).all() and (got[k + 1] == -17).all()
    with pytest.raises(z.ZcError):
        ctx.linear(down, dx, 1, out=out.view(1, H * 4))        # misaligned
    with pytest.raises(z.ZcError):
        ctx.linear(down, dx, 1, out=drec.view(2 * 921600, H * 4))   # aliases the weights
    ctx.finish()


def cfg_o(cfg):
    return oracle.Config(*[getattr(cfg, n) for n, _ in z.Config._fields_])


def test_grouped_experts_keep_router_positions(ctx):  # :1188-1208
    cfg = workload.config("ref"); H, I, k = cfg.hidden, cfg.inter, cfg.topk
    x = np.array([(i % 17 - 8) / 64 for i in range(H)], dtype=f32); dx = ctx.upload(x)
    recs = [expert_fixture(cfg, i + 1) for i in range(8)]; drecs = [ctx.upload(r) for r in recs]
    oc = cfg_o(cfg)
    ref = []
    for r in recs:
        act = oracle.gated_linear(oracle.expert_linear(oc, r, 0), oracle.expert_linear(oc, r, 1), x, 1)
        ref.append(oracle.linear(oracle.expert_linear(oc, r, 2), act, 1)[0])
    positions = [9, 1, 7, 3, 5, 0, 8, 4]
    for n in (1, 2, 3, 4, 7, 8):
        out = ctx.upload(np.full(k * H, -19, f32)); scratch = ctx.zeros(8 * I * 4)
        ctx.grouped_experts(cfg, drecs[:n], positions[:n], dx, out, scratch)
        got = out.numpy(f32).reshape(k, H)
        for i in range(n):
            assert same_bytes(got[positions[i]], ref[i])
        for p in range(k):
            if p not in positions[:n]:
                assert (got[p] == -19).all()
        with pytest.raises(z.ZcError):
            ctx.grouped_experts(cfg, drecs[:2], [1, 1], dx, out, scratch)
    ctx.finish()


def test_scatter_rows(ctx):  # qwen.metal:800-803
    H = 2048; x = np.arange(3 * H, dtype=f32); out = ctx.upload(np.full(12 * H, -17, f32))
    ctx.scatter_experts(ctx.upload(x), ctx.upload(np.array([9, 1, 7], np.int32)), 3, H, out)
    got = out.numpy(f32).reshape(12, H)
    want = np.full((12, H), -17, f32); oracle.scatter_experts(x, [9, 1, 7], H, want)
    assert same_bytes(got, want)


def test_stack_glue_is_max_normalised(ctx):
    y = synth.normal(3 * 3072, 9, 5.0).reshape(3, 3072)
    y[1, 7] = np.nan
    out = ctx.alloc(y.nbytes); ctx.stack_glue(ctx.upload(y), 3, 3072, out)
    got = out.numpy(f32).reshape(3, 3072)
    m = np.nanmax(np.abs(y), axis=1, keepdims=True).astype(f32)
    want = oracle.bf(y * (f32(1) / m))
    assert got.tobytes() == want.tobytes()
    assert np.nanmax(np.abs(got)) == 1.0


def test_profile_rows_carry_the_labels_and_statistics_are_json(ctx):
    # Metal::label + KernelConfig::profile (metal.mm:267-270) and Model::stats (model.cpp:706-732) through the C ABI.
    from zerocool_amd import workload
    cfg = workload.tiny_config(hidden=512, experts=32, topk=4, inter=512)
    layers = [workload.LayerWeights(ctx, cfg, 60 + l, ("normal", 0.5)) for l in range(2)]
    stack = ctx.stack_create(cfg, [w.layer for w in layers], 8)
    x = workload.hidden_rows(ctx, 2, cfg.hidden, 11)
    out, ws = ctx.alloc(2 * cfg.hidden * 4), ctx.alloc(ctx.moe_workspace_bytes(cfg, 2))
    ctx.label("ignored", 7, 1, 0)                     # no recording yet: a label is a no-op, as in the reference
    ctx.moe_forward(cfg, layers[0].layer, x, 2, out, ws)
    quiet = ctx.stats()
    assert quiet["profile"] == {"recording": False, "rows_recorded": 0, "rows_dropped": 0, "stages": [], "rows": []}
    assert quiet["memory"]["allocated_bytes"] == ctx.allocated and quiet["memory"]["peak_bytes"] >= ctx.allocated
    ctx.profile(True)
    ctx.moe_forward(cfg, layers[0].layer, x, 2, out, ws)   # before any label
    ctx.label("router", 3, 2, 5)
    logits = ctx.router_logits(layers[0].router, x, 2, cfg.hidden, cfg.experts, layers[0].offsets)
    ctx.label("experts", 3, 2, 5)
    ctx.moe_forward(cfg, layers[1].layer, x, 2, out, ws)
    ctx.moe_forward(cfg, layers[1].layer, x, 2, out, ws)
    ctx.label("decode", -1, 2, 6)
    ctx.stack_decode(stack, x, 2, out, layered=True)   # calls the layer operator twice inside: one row, its own
    ctx.stack_decode(stack, x, 2, out)
    ctx.profile(False)
    ctx.moe_forward(cfg, layers[0].layer, x, 2, out, ws)   # not recorded
    s = ctx.stats()
    rows = s["profile"]["rows"]
    assert [(r["stage"], r["operator"]) for r in rows] == [("unlabelled", "moe_forward"), ("router", "router_logits"), ("experts", "moe_forward"),
                                                          ("experts", "moe_forward"), ("decode", "stack_decode"), ("decode", "stack_decode")]
    assert rows[1]["layer"] == 3 and rows[1]["tokens"] == 2 and rows[1]["offset"] == 5 and rows[4]["layer"] == -1
    assert all(0 < r["gpu_us"] < 1e5 for r in rows)
    stages = {(e["stage"], e["operator"]): e for e in s["profile"]["stages"]}
    assert stages[("experts", "moe_forward")]["calls"] == 2 and stages[("decode", "stack_decode")]["calls"] == 2
    assert abs(stages[("experts", "moe_forward")]["gpu_us"] - rows[2]["gpu_us"] - rows[3]["gpu_us"]) < 1e-2
    assert s["profile"]["recording"] is False and s["profile"]["rows_recorded"] == 6
    ctx.profile(True)                                   # a new recording starts empty
    assert ctx.stats()["profile"]["rows"] == []
    ctx.profile(False)
    store = z.Store(ctx, 1, 8, 4096, 3)
    lease = store.acquire(0, 2); store.wait(lease); ctx.finish(); store.release(lease)
    cache = ctx.stats(store)["expert_cache"]
    assert (cache["capacity"], cache["occupancy"], cache["misses"], cache["hits"], cache["application_read_bytes"]) == (3, 1, 1, 0, 4096)
    assert cache["record_table"]["reads"] == 0
    store.close()
    ctx.stack_destroy(stack)
    for b in (x, out, ws, logits):
        ctx.free(b)
