"""Prefill path (BASELINE config 3 at reduced and full size): sorted tokens + grouped GEMM on the bf16 matrix cores.
Routing ids, softmax weights and the dispatch must equal the exact path bit for bit; expert outputs and the layer
output are checked against the exact path (itself byte-equal to the CPU oracle) within max relative error 2e-3."""
import numpy as np
import pytest
import oracle
import zerocool_amd as z
from zerocool_amd import workload

pytestmark = pytest.mark.gpu
f32 = np.float32
TOLERANCE = 2e-3   # max |got - want| / max |want|


@pytest.fixture(scope="module")
def ctx():
    c = z.Context(0)
    yield c
    c.close()


def run_both(ctx, cfg, weights, x, T):
    n = T * cfg.topk
    outs = []
    for prefill in (False, True):
        out = ctx.alloc(T * cfg.hidden * 4)
        size = ctx.moe_prefill_workspace_bytes(cfg, T) if prefill else ctx.moe_workspace_bytes(cfg, T)
        assert size > 0
        ws = ctx.alloc(size)
        ids, w = ctx.alloc(n * 4), ctx.alloc(n * 4)
        eo, sh = ctx.alloc(n * cfg.hidden * 4), ctx.alloc(T * cfg.hidden * 4)
        trace = z.Trace(None, ids.ptr, w.ptr, eo.ptr, sh.ptr, None)
        (ctx.moe_prefill if prefill else ctx.moe_forward)(cfg, weights.layer, x, T, out, ws, trace)
        ctx.moe_check()
        outs.append(dict(out=out.numpy(f32), ids=ids.numpy(np.int32), weights=w.numpy(f32), expert_out=eo.numpy(f32), shared=sh.numpy(f32)))
        for b in (out, ws, ids, w, eo, sh):
            ctx.free(b)
    return outs


def rel(got, want):
    return float(np.max(np.abs(got - want)) / np.max(np.abs(want)))


ONE_BF16_STEP = 2.0 ** -7   # the spacing of BF16 numbers relative to their magnitude, at most


@pytest.mark.parametrize("shape,tokens", [((512, 32, 4, 128), 1), ((512, 32, 4, 128), 37), ((512, 32, 4, 128), 300),
                                          ((1024, 64, 10, 256), 129), ((2048, 512, 10, 512), 96),
                                          ((3072, 16, 4, 1024), 70), ((4096, 8, 2, 128), 33)])   # 48 and 64 scale groups: the largest K
def test_prefill_matches_the_exact_path(ctx, shape, tokens):
    cfg = workload.tiny_config(*shape)
    weights = workload.LayerWeights(ctx, cfg, 61 + tokens, ("normal", 0.5))
    x = workload.hidden_rows(ctx, tokens, cfg.hidden, 700 + tokens)
    exact, fast = run_both(ctx, cfg, weights, x, tokens)
    assert fast["ids"].tobytes() == exact["ids"].tobytes()
    assert fast["weights"].tobytes() == exact["weights"].tobytes()
    # The two paths differ only by the order of fp32 additions, so a BF16-rounded value could at most tip over to the
    # neighbouring BF16 number where its fp32 sum sits on a rounding boundary; the prefill path recomputes exactly the
    # sums that land near such a boundary.  Intermediates: no error larger than one such step of the largest value;
    # layer output: within the stated tolerance, and all but a sliver of the values identical.
    assert rel(fast["shared"], exact["shared"]) <= ONE_BF16_STEP
    assert rel(fast["expert_out"], exact["expert_out"]) <= ONE_BF16_STEP
    print(f"T={tokens} {shape}: layer output max rel err {rel(fast['out'], exact['out']):.3g}, "
          f"identical {np.mean(fast['out'].view(np.uint32) == exact['out'].view(np.uint32)):.5f}, "
          f"expert outputs identical {np.mean(fast['expert_out'].view(np.uint32) == exact['expert_out'].view(np.uint32)):.5f}")
    assert rel(fast["out"], exact["out"]) <= TOLERANCE
    same = np.mean(fast["out"].view(np.uint32) == exact["out"].view(np.uint32))
    assert same > 0.9999, same
    # a call that asks for no intermediates hands the slots' outputs to the combine as bf16: the same values, the same output
    out, ws = ctx.alloc(tokens * cfg.hidden * 4), ctx.alloc(ctx.moe_prefill_workspace_bytes(cfg, tokens))
    ctx.moe_prefill(cfg, weights.layer, x, tokens, out, ws)
    ctx.moe_check()
    assert out.numpy(f32).tobytes() == fast["out"].tobytes()
    for b in (weights.router, weights.shared_gate, weights.shared_record, weights.records, x, out, ws):
        ctx.free(b)


@pytest.mark.parametrize("shape,bits,tokens", [((512, 32, 4, 128), (4, 8, 8, 8), 37),      # the mixed artifact: Q4 gate/up, Q8 down and shared expert
                                               ((512, 32, 4, 128), (8, 8, 8, 8), 150),     # every projection Q8, narrow lanes (K not a multiple of 512 for the down rows)
                                               ((1024, 64, 10, 512), (4, 8, 8, 8), 129),   # wide lanes on both sides
                                               ((1024, 64, 10, 512), (8, 4, 4, 8), 70),
                                               ((2048, 512, 10, 512), (4, 8, 8, 8), 96)])  # BASELINE config 4's shape
def test_prefill_with_affine_q8_projections(ctx, shape, bits, tokens):
    # Affine Q8 records through the same grouped product: byte codes are exact in bf16, the fold uses the Q8 lanes' plain
    # input sums (qwen.metal:112-125), and the sums near a BF16 rounding boundary are recomputed on the Q8 lanes themselves.
    cfg = workload.tiny_config(*shape, bits=bits)
    weights = workload.LayerWeights(ctx, cfg, 161 + tokens, ("normal", 0.5))
    x = workload.hidden_rows(ctx, tokens, cfg.hidden, 800 + tokens)
    exact, fast = run_both(ctx, cfg, weights, x, tokens)
    assert fast["ids"].tobytes() == exact["ids"].tobytes()
    assert fast["weights"].tobytes() == exact["weights"].tobytes()
    assert rel(fast["shared"], exact["shared"]) <= ONE_BF16_STEP
    assert rel(fast["expert_out"], exact["expert_out"]) <= ONE_BF16_STEP
    same = np.mean(fast["out"].view(np.uint32) == exact["out"].view(np.uint32))
    print(f"T={tokens} {shape} bits {bits}: layer output max rel err {rel(fast['out'], exact['out']):.3g}, identical {same:.5f}, "
          f"expert outputs identical {np.mean(fast['expert_out'].view(np.uint32) == exact['expert_out'].view(np.uint32)):.5f}")
    assert rel(fast["out"], exact["out"]) <= TOLERANCE
    assert same > 0.9999, same
    # and against the CPU oracle directly on a few token rows
    sample = np.arange(0, tokens, max(1, tokens // 8))[:8]
    h = weights.host()
    ocfg = oracle.Config(*[getattr(cfg, n) for n, _ in z.Config._fields_])
    xs = x.numpy(f32).reshape(tokens, cfg.hidden)[sample]
    want, tr = oracle.moe_layer(ocfg, h["router"], h["shared_gate"], h["shared_record"], h["records"], h["stride"],
                                xs, len(sample), router_offsets=h["offsets"], threads=8, trace=True)
    assert fast["ids"].reshape(tokens, cfg.topk)[sample].tobytes() == tr["ids"].tobytes()
    assert rel(fast["out"].reshape(tokens, cfg.hidden)[sample], want) <= TOLERANCE
    for b in (weights.router, weights.shared_gate, weights.shared_record, weights.records, x):
        ctx.free(b)


def test_prefill_against_the_cpu_oracle(ctx):
    cfg = workload.tiny_config(512, 32, 4, 128)
    T = 70
    weights = workload.LayerWeights(ctx, cfg, 91, ("zipf", 1.1))
    x = workload.hidden_rows(ctx, T, cfg.hidden, 92)
    h = weights.host()
    ocfg = oracle.Config(*[getattr(cfg, n) for n, _ in z.Config._fields_])
    want, tr = oracle.moe_layer(ocfg, h["router"], h["shared_gate"], h["shared_record"], h["records"], h["stride"],
                                x.numpy(f32), T, router_offsets=h["offsets"], threads=8, trace=True)
    _, fast = run_both(ctx, cfg, weights, x, T)
    assert fast["ids"].tobytes() == tr["ids"].tobytes()
    assert rel(fast["out"].reshape(T, cfg.hidden), want) <= TOLERANCE


def test_prefill_full_size_unskewed(ctx):
    # BASELINE config 3 as written: 2048 tokens through the single-layer shape, no router skew (every expert gets rows,
    # about forty each, so an expert's rows span several 32-row tiles).  Checked on ALL tokens against the exact path
    # (itself byte-equal to the oracle at every smaller size) and on a sample of token rows against the CPU oracle
    # directly: tokens are independent of each other, so the oracle can run on the sample alone.
    cfg = workload.config("S")
    T = 2048
    weights = workload.LayerWeights(ctx, cfg, 301, None)
    x = workload.hidden_rows(ctx, T, cfg.hidden, 302)
    exact, fast = run_both(ctx, cfg, weights, x, T)
    assert fast["ids"].tobytes() == exact["ids"].tobytes()
    assert fast["weights"].tobytes() == exact["weights"].tobytes()
    counts = np.bincount(exact["ids"].ravel(), minlength=cfg.experts)
    assert counts.min() > 0 and counts.max() > 32, "the unskewed batch should touch every expert and need several tiles for some"
    assert rel(fast["expert_out"], exact["expert_out"]) <= ONE_BF16_STEP
    assert rel(fast["out"], exact["out"]) <= TOLERANCE
    same = np.mean(fast["out"].view(np.uint32) == exact["out"].view(np.uint32))
    print(f"T={T} unskewed: {int((counts > 0).sum())} experts used, {counts.max()} rows at most; layer output max rel err "
          f"{rel(fast['out'], exact['out']):.3g}, identical {same:.6f}")
    assert same > 0.9999, same
    sample = np.random.default_rng(5).choice(T, 256, replace=False); sample.sort()
    h = weights.host()
    ocfg = oracle.Config(*[getattr(cfg, n) for n, _ in z.Config._fields_])
    xs = x.numpy(f32).reshape(T, cfg.hidden)[sample]
    want, tr = oracle.moe_layer(ocfg, h["router"], h["shared_gate"], h["shared_record"], h["records"], h["stride"],
                                xs, len(sample), router_offsets=h["offsets"], threads=16, trace=True)
    assert fast["ids"].reshape(T, cfg.topk)[sample].tobytes() == tr["ids"].tobytes(), "routing ids differ from the oracle"
    assert fast["weights"].reshape(T, cfg.topk)[sample].tobytes() == tr["weights"].tobytes()
    got = fast["out"].reshape(T, cfg.hidden)[sample]
    assert rel(got, want) <= TOLERANCE
    assert exact["out"].reshape(T, cfg.hidden)[sample].tobytes() == want.tobytes()   # the exact path stays byte-equal at full size
    for b in (weights.router, weights.shared_gate, weights.shared_record, weights.records, x):
        ctx.free(b)


@pytest.mark.parametrize("T", [70, 300])   # 300 tokens: the router on bounds with the selection in its launch, and the one-launch dispatch sort
def test_prefill_reports_unroutable_rows(ctx, T):
    # A NaN row gives that token no selectable expert (ids -1): its sorted positions are not covered by any tile.  The
    # call must end normally and the check must report "invalid router output", as the exact path does.
    cfg = workload.tiny_config(512, 32, 4, 128)
    weights = workload.LayerWeights(ctx, cfg, 94, ("normal", 0.5))
    ws = ctx.alloc(ctx.moe_prefill_workspace_bytes(cfg, T)); out = ctx.alloc(T * cfg.hidden * 4)
    good = workload.hidden_rows(ctx, T, cfg.hidden, 95)
    ctx.fill(ws, 0xff)                        # whatever an earlier call could have left in the recomputation map: all bits set
    ctx.moe_prefill(cfg, weights.layer, good, T, out, ws); ctx.moe_check()
    want = out.numpy(f32).reshape(T, cfg.hidden).copy()
    rows = good.numpy(f32).reshape(T, cfg.hidden).copy()
    rows[[3, 41]] = np.nan
    ctx.fill(ws, 0xff)
    ctx.moe_prefill(cfg, weights.layer, ctx.upload(rows.ravel()), T, out, ws)
    with pytest.raises(z.ZcError) as err:
        ctx.moe_check()
    assert "invalid router output" in str(err.value)
    got = out.numpy(f32).reshape(T, cfg.hidden)
    keep = np.setdiff1d(np.arange(T), [3, 41])
    assert got[keep].tobytes() == want[keep].tobytes()      # the other tokens are untouched by their neighbours' failure
    ctx.moe_prefill(cfg, weights.layer, good, T, out, ws); ctx.moe_check()     # and the path is usable afterwards
    assert out.numpy(f32).tobytes() == want.tobytes()


def test_prefill_rejects_what_it_cannot_run(ctx):
    odd = workload.tiny_config(512, 32, 4, 128, group=32)     # only group 64
    assert ctx.moe_prefill_workspace_bytes(odd, 64) == 0
    assert ctx.moe_prefill_workspace_bytes(workload.tiny_config(512, 32, 4, 128, bits=(4, 8, 8, 8)), 64) > 0   # the mixed artifact is taken
    assert ctx.moe_prefill_workspace_bytes(workload.tiny_config(4224, 32, 4, 128), 64) == 0   # K beyond what the product kernel keeps in LDS
    assert ctx.moe_prefill_workspace_bytes(workload.tiny_config(4096, 32, 4, 4096), 64) > 0
    cfg = workload.tiny_config(512, 32, 4, 128)
    weights = workload.LayerWeights(ctx, cfg, 93, None)
    T = 40
    x = ctx.upload(np.full(T * cfg.hidden, 1.0000001, f32))     # not BF16-valued
    out, ws = ctx.alloc(T * cfg.hidden * 4), ctx.alloc(ctx.moe_prefill_workspace_bytes(cfg, T))
    ctx.moe_prefill(cfg, weights.layer, x, T, out, ws)
    with pytest.raises(z.ZcError) as err:
        ctx.moe_check()
    assert "BF16" in str(err.value)
    with pytest.raises(z.ZcError):
        ctx.moe_prefill(odd, weights.layer, x, T, out, ws)


@pytest.mark.parametrize("skew", [None, ("zipf", 1.1)])
def test_prefill_router_on_bounds_picks_the_exact_ids(ctx, skew):
    """From 128 tokens on (and when the logits themselves are not asked for) the prefill router forms every logit with a
    bf16 matrix-core product, bounds its distance from the reference's chains, and recomputes exactly only the experts that
    can be among the top k.  Ids and softmax weights must be the exact path's bits, also where logits tie exactly (router
    rows repeated, an all-zero input row), nearly tie (a row that differs from another in one element's last bit), where an
    input row is huge or tiny, and where it holds inf or NaN (then no expert is selectable: reported, other tokens
    untouched)."""
    cfg = workload.tiny_config(1024, 128, 8, 128)
    weights = workload.LayerWeights(ctx, cfg, 301, skew)
    E, H, T = cfg.experts, cfg.hidden, 200
    router = weights.router.numpy(np.uint16).reshape(E, H).copy()
    router[17] = router[5]; router[90] = router[5]; router[33] = router[64]      # exact ties
    router[70] = router[12]; router[70, 100] ^= 1                                  # one element differs by its last bit
    ctx.upload(router.ravel(), into=weights.router)
    x = workload.hidden_rows(ctx, T, H, 302).numpy(f32).reshape(T, H).copy()
    x[7] = 0.0
    x[8] = oracle.bf(x[8] * f32(2.0 ** 60)); x[9] = oracle.bf(x[9] * f32(2.0 ** -60))
    x[12] = oracle.bf(x[12] * f32(2.0 ** -75)); x[13] = oracle.bf(x[13] * f32(2.0 ** -120))   # squares below the normal range
    x[10] = x[11]                                                                  # two tokens alike
    dx = ctx.upload(x.ravel())
    exact, fast = run_both(ctx, cfg, weights, dx, T)
    assert fast["ids"].tobytes() == exact["ids"].tobytes()
    assert fast["weights"].tobytes() == exact["weights"].tobytes()
    assert (exact["ids"].reshape(T, cfg.topk)[7] == np.arange(cfg.topk)).all() or skew is not None   # all logits equal: the lowest ids
    # rows that no expert can be selected for
    bad = x.copy(); bad[20, 5] = np.nan; bad[21, 9] = np.inf; bad[22, 9] = -np.inf; bad[22, 10] = np.inf
    dbad = ctx.upload(bad.ravel())
    n = T * cfg.topk
    got = {}
    for prefill in (False, True):
        out = ctx.alloc(T * H * 4); ids = ctx.alloc(n * 4)
        ws = ctx.alloc(ctx.moe_prefill_workspace_bytes(cfg, T) if prefill else ctx.moe_workspace_bytes(cfg, T))
        (ctx.moe_prefill if prefill else ctx.moe_forward)(cfg, weights.layer, dbad, T, out, ws, z.Trace(None, ids.ptr, None, None, None, None))
        with pytest.raises(z.ZcError) as err:
            ctx.moe_check()
        assert "invalid router output" in str(err.value)
        got[prefill] = ids.numpy(np.int32).copy()
        for b in (out, ids, ws):
            ctx.free(b)
    assert got[True].tobytes() == got[False].tobytes()
    for b in (weights.router, weights.shared_gate, weights.shared_record, weights.records, dx, dbad):
        ctx.free(b)
