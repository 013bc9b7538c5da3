"""Stacked decode (BASELINE config 5 at reduced size): the persistent single-launch kernel,
the layer-by-layer path and the CPU oracle chained through the same glue must agree byte
for byte on routing ids, softmax weights and every layer's output."""
import numpy as np
import pytest
import oracle
import zerocool_amd as z
from zerocool_amd import workload

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.fixture(scope="module")
def ctx():
    c = z.Context(0)
    yield c
    c.close()


def oracle_cfg(cfg):
    return oracle.Config(*[getattr(cfg, n) for n, _ in z.Config._fields_])


def glue(y):
    """The stack's stand-in glue: x_next = bf(y * (1 / max|y|)) per token."""
    m = np.nanmax(np.abs(y), axis=1, keepdims=True).astype(f32)
    inv = np.where((m > 0) & np.isfinite(m), f32(1) / m, f32(1)).astype(f32)
    return oracle.bf(y * inv)


def oracle_stack(cfg, layers, x, T):
    ocfg = oracle_cfg(cfg)
    ids, weights, outs = [], [], []
    cur = x.reshape(T, cfg.hidden)
    for h in layers:
        y, tr = oracle.moe_layer(ocfg, h["router"], h["shared_gate"], h["shared_record"], h["records"], h["stride"], cur, T,
                                 router_offsets=h["offsets"], threads=8, trace=True)
        ids.append(tr["ids"]); weights.append(tr["weights"]); outs.append(y)
        cur = glue(y)
    return np.stack(ids), np.stack(weights), np.stack(outs)


def run_stack(ctx, cfg, stack, x_dev, T, L, layered):
    n = T * cfg.topk
    ids, w, outs = ctx.alloc(L * n * 4), ctx.alloc(L * n * 4), ctx.alloc(L * T * cfg.hidden * 4)
    out = ctx.alloc(T * cfg.hidden * 4)
    ctx.stack_decode(stack, x_dev, T, out, z.StackTrace(ids.ptr, w.ptr, outs.ptr, None), layered=layered)
    ctx.moe_check()
    r = (ids.numpy(np.int32).reshape(L, T, cfg.topk), w.numpy(f32).reshape(L, T, cfg.topk),
         outs.numpy(f32).reshape(L, T, cfg.hidden), out.numpy(f32).reshape(T, cfg.hidden))
    for b in (ids, w, outs, out):
        ctx.free(b)
    return r


def _check_stack(ctx, cfg, L, tokens, seed, skew, persistent, mutate=None):
    layers = [workload.LayerWeights(ctx, cfg, seed + l, skew) for l in range(L)]
    if mutate:
        for l in layers:
            mutate(l)
    hosts = [l.host() for l in layers]
    stack = ctx.stack_create(cfg, [l.layer for l in layers], max(tokens))
    for T in tokens:
        x_dev = workload.hidden_rows(ctx, T, cfg.hidden, seed * 131 + T)
        x = x_dev.numpy(f32)
        want = oracle_stack(cfg, hosts, x, T)
        assert ctx.stack_is_persistent(stack, T) == (persistent(T) if callable(persistent) else persistent)   # above eight tokens: launches of eight and the rest
        for layered in (True, False):
            got = run_stack(ctx, cfg, stack, x_dev, T, L, layered)
            name = "layered" if layered else "persistent"
            assert got[0].tobytes() == want[0].tobytes(), f"{name}: routing ids differ (T={T})"
            assert got[1].tobytes() == want[1].tobytes(), f"{name}: softmax weights differ (T={T})"
            assert got[2].tobytes() == want[2].tobytes(), f"{name}: layer outputs differ (T={T})"
            assert got[3].tobytes() == want[2][-1].tobytes()
            rel = float(np.max(np.abs(got[3] - want[2][-1])) / np.max(np.abs(want[2][-1])))
            assert rel <= 2e-3
        ctx.free(x_dev)
    ctx.stack_destroy(stack)
    for l in layers:
        for b in (l.router, l.shared_gate, l.shared_record, l.records):
            ctx.free(b)


def check_stack(ctx, cfg, L, tokens, seed=31, skew=("zipf", 1.1), persistent=True, mutate=None):
    return _check_stack(ctx, cfg, L, tokens, seed, skew, persistent, mutate)


def test_few_experts_stack(ctx):  # the single-layer shape (hidden 2048 / intermediate 512) with few experts
    check_stack(ctx, workload.tiny_config(hidden=2048, experts=32, topk=4, inter=512), 3, [1, 2, 3, 5, 8, 11])


def test_single_layer_shape_stack(ctx):
    check_stack(ctx, workload.tiny_config(hidden=2048, experts=128, topk=10, inter=512), 3, [1, 8, 20])


def test_mixed_artifact_stack(ctx):
    # Affine Q8 down projection and shared expert (BASELINE config 4's artifact): one token runs the one-token kernel with
    # those projections on literal lanes, more tokens the kernel for nine to sixty-four tokens.  All against the oracle.
    check_stack(ctx, workload.tiny_config(hidden=1024, experts=64, topk=10, inter=512, bits=(4, 8, 8, 8)), 3, [1, 3, 16, 21])
    check_stack(ctx, workload.tiny_config(hidden=2048, experts=128, topk=10, inter=512, bits=(4, 8, 8, 8)), 2, [1, 16], seed=37)
    check_stack(ctx, workload.tiny_config(hidden=1024, experts=32, topk=4, inter=1024, bits=(4, 8, 4, 8)), 2, [1, 5], seed=41)
    check_stack(ctx, workload.tiny_config(hidden=1024, experts=32, topk=4, inter=1024, bits=(4, 4, 8, 4)), 2, [1, 9], seed=43)


def test_nine_to_sixty_four_tokens_in_one_launch(ctx):
    # The kernel for nine to sixty-four tokens: entries of up to eight tokens per expert (a skewed router sends dozens of
    # tokens to one expert, so its tokens fill several entries), a full launch of 64, and 64 + 6 as two launches.
    check_stack(ctx, workload.tiny_config(hidden=1024, experts=64, topk=10, inter=512), 2, [9, 64, 70], seed=47)
    check_stack(ctx, workload.tiny_config(hidden=2048, experts=512, topk=10, inter=512), 1, [33], seed=53)
    check_stack(ctx, workload.tiny_config(hidden=1024, experts=16, topk=4, inter=1024), 2, [40], seed=59, skew=None)


def test_small_hidden_stack(ctx):
    check_stack(ctx, workload.tiny_config(hidden=1024, experts=64, topk=10, inter=512), 2, [1, 4, 17, 32])


def test_tied_logits_pick_the_lowest_ids(ctx):
    # 512 experts whose router rows repeat in runs of twelve: every run ties exactly, so the ten picks are the ten
    # lowest ids of the best run, in ascending order, and the softmax weights are all equal
    cfg = workload.tiny_config(hidden=1024, experts=512, topk=10, inter=512)

    def repeat_rows(layer):
        rows = layer.router.numpy(np.uint16).reshape(cfg.experts, cfg.hidden)
        rows = rows[(np.arange(cfg.experts) // 12) * 12]
        layer.ctx.upload(np.ascontiguousarray(rows).reshape(-1), into=layer.router)

    check_stack(ctx, cfg, 2, [1, 3], skew=None, mutate=repeat_rows)

    # all 512 rows alike: every logit ties, the picks are experts 0..9 (more candidates than one wave holds: the pick-by-pick path);
    # runs of 40: more tied candidates than picks, still within one wave
    def one_row(layer):
        rows = layer.router.numpy(np.uint16).reshape(cfg.experts, cfg.hidden)
        layer.ctx.upload(np.ascontiguousarray(rows[np.zeros(cfg.experts, np.int64)]).reshape(-1), into=layer.router)

    def long_runs(layer):
        rows = layer.router.numpy(np.uint16).reshape(cfg.experts, cfg.hidden)
        layer.ctx.upload(np.ascontiguousarray(rows[(np.arange(cfg.experts) // 40) * 40]).reshape(-1), into=layer.router)

    check_stack(ctx, cfg, 2, [1, 2], skew=None, mutate=one_row)
    check_stack(ctx, cfg, 2, [1, 2], skew=None, mutate=long_runs)


def test_other_shapes_take_the_layered_path(ctx):  # hidden not a multiple of 512
    check_stack(ctx, workload.tiny_config(hidden=768, experts=64, topk=10, inter=512), 2, [1, 4], persistent=False)


def test_stand_in_stack_shape(ctx):  # hidden 3072 / intermediate 1024, two layers of the 48
    check_stack(ctx, workload.config("F"), 2, [1, 8])


def test_benchmark_shapes_through_the_single_launch_kernels(ctx):
    # The exact shapes the benchmark quotes, 512 experts and top-10, each through the kernel its figure comes from:
    # the single layer (hidden 2048, intermediate 512) with N(0, 0.5) router offsets at 1 token (one-token kernel),
    # 8 (two to eight), 32 and 64 (nine to sixty-four); the mixed 4/8-bit artifact at 1 and 16 tokens.
    check_stack(ctx, workload.config("S"), 1, [1, 8, 32, 64], seed=61, skew=("normal", 0.5))
    check_stack(ctx, workload.config("S-mixed"), 1, [1, 16], seed=67, skew=("normal", 0.5))


def test_stand_in_stack_six_layers(ctx):  # the 48-layer stack's shape and Zipf(1.1) routers, six layers deep, 1 and 8 tokens
    check_stack(ctx, workload.config("F"), 6, [1, 8], seed=71)


def test_stack_reports_invalid_router_output(ctx):
    cfg = workload.tiny_config(hidden=2048, experts=32, topk=4, inter=512)
    layers = [workload.LayerWeights(ctx, cfg, 77 + l, None) for l in range(2)]
    stack = ctx.stack_create(cfg, [l.layer for l in layers], 2)
    bad = ctx.upload(np.full(2 * cfg.hidden, np.nan, f32)); out = ctx.alloc(2 * cfg.hidden * 4)
    ctx.stack_decode(stack, bad, 2, out)
    with pytest.raises(z.ZcError) as err:
        ctx.moe_check()
    assert "invalid router output" in str(err.value)
    notbf = ctx.upload(np.full(2 * cfg.hidden, 1.0000001, f32))
    ctx.stack_decode(stack, notbf, 2, out)
    with pytest.raises(z.ZcError) as err:
        ctx.moe_check()
    assert "BF16" in str(err.value)
    # the single-token kernel has its own phases: the same two reports, and a clean run afterwards
    for values, text in ((np.full(cfg.hidden, np.nan, f32), "invalid router output"), (np.full(cfg.hidden, 1.0000001, f32), "BF16")):
        ctx.stack_decode(stack, ctx.upload(values), 1, out)
        with pytest.raises(z.ZcError) as err:
            ctx.moe_check()
        assert text in str(err.value)
    ctx.stack_decode(stack, ctx.upload(np.full(cfg.hidden, 0.5, f32)), 1, out)
    ctx.moe_check()
    ctx.stack_destroy(stack)


def test_single_token_launches_across_the_tag_wrap(ctx):
    # The one-token kernel marks everything its workgroups exchange with a 16-bit tag that advances with every layer of
    # every one-token launch: some thirty thousand launches of a two-layer stack take it once around, with launches of the
    # several-token kernel (which shares the flags, not the tagged buffers, and must not move the tags) in between.
    # Every launch must give the first one's output.
    cfg = workload.tiny_config(hidden=1024, experts=64, topk=10, inter=512)
    layers = [workload.LayerWeights(ctx, cfg, 401 + l, ("zipf", 1.1)) for l in range(2)]
    stack = ctx.stack_create(cfg, [l.layer for l in layers], 2)
    assert ctx.stack_is_persistent(stack, 1)
    x1, x2 = workload.hidden_rows(ctx, 1, cfg.hidden, 17), workload.hidden_rows(ctx, 2, cfg.hidden, 18)
    out1, out2 = ctx.alloc(cfg.hidden * 4), ctx.alloc(2 * cfg.hidden * 4)
    ctx.stack_decode(stack, x1, 1, out1); ctx.moe_check()
    first = out1.numpy(f32).tobytes()
    ctx.stack_decode(stack, x2, 2, out2); ctx.moe_check()
    first2 = out2.numpy(f32).tobytes()
    launches = 65535 // 2 + 300
    for i in range(launches):
        ctx.stack_decode(stack, x1, 1, out1)
        if i % 97 == 0:
            ctx.stack_decode(stack, x2, 2, out2)
        if i % 4000 == 0 or i > launches - 600 and i % 7 == 0:
            ctx.moe_check()
            assert out1.numpy(f32).tobytes() == first, f"launch {i}"
            assert out2.numpy(f32).tobytes() == first2, f"launch {i}"
    ctx.moe_check()
    assert out1.numpy(f32).tobytes() == first
    # A long run of several-token launches between two one-token launches: however many there are, the one-token launch
    # that follows must not meet a tag its predecessor left (run lengths around a multiple of the tag period included).
    for run in (1, 409, 1228, 1229, 2979):
        for _ in range(run):
            ctx.stack_decode(stack, x2, 2, out2)
        ctx.stack_decode(stack, x1, 1, out1); ctx.moe_check()
        assert out1.numpy(f32).tobytes() == first, f"after {run} two-token launches"
        assert out2.numpy(f32).tobytes() == first2
    ctx.stack_destroy(stack)
    for l in layers:
        for b in (l.router, l.shared_gate, l.shared_record, l.records):
            ctx.free(b)
    for b in (x1, x2, out1, out2):
        ctx.free(b)


def test_a_wait_that_runs_out_is_reported_and_the_stack_stays_usable(ctx):
    # Every wait of the persistent kernel on another workgroup is bounded.  With a bound of one poll some wait runs out
    # in practically every launch: the launch then gives up everywhere, ends normally, and the check reports it.  With the
    # default bound back, the same stack gives the right answer again.
    cfg = workload.tiny_config(hidden=1024, experts=64, topk=10, inter=512)
    layers = [workload.LayerWeights(ctx, cfg, 501 + l, ("zipf", 1.1)) for l in range(4)]
    stack = ctx.stack_create(cfg, [l.layer for l in layers], 12)
    out = {T: ctx.alloc(T * cfg.hidden * 4) for T in (1, 2, 12)}
    xs = {T: workload.hidden_rows(ctx, T, cfg.hidden, 30 + T) for T in (1, 2, 12)}
    want = {}
    for T in (1, 2, 12):
        ctx.stack_decode(stack, xs[T], T, out[T]); ctx.moe_check()
        want[T] = out[T].numpy(f32).tobytes()
    for T in (1, 2, 12):
        ctx.stack_set_wait_limit(stack, 1)
        reported = 0
        for _ in range(5):
            ctx.stack_decode(stack, xs[T], T, out[T])
            try:
                ctx.moe_check()
            except z.ZcError as err:
                assert "synchronise" in str(err)
                reported += 1
        assert reported > 0, "a one-poll bound never ran out"
        ctx.stack_set_wait_limit(stack, 0)
        ctx.stack_decode(stack, xs[T], T, out[T]); ctx.moe_check()
        assert out[T].numpy(f32).tobytes() == want[T]
    ctx.stack_destroy(stack)
    for l in layers:
        for b in (l.router, l.shared_gate, l.shared_record, l.records):
            ctx.free(b)
    for T in (1, 2, 12):
        ctx.free(out[T]); ctx.free(xs[T])


@pytest.mark.parametrize("skew", [None, ("zipf", 1.1)])
def test_guessed_experts_never_change_the_result(ctx, skew):
    # One-token launches start a layer's gate/up tiles on the experts that layer picked at the previous one-token step and redo
    # only the slots that were guessed wrong.  A run of DIFFERENT tokens (without router skew nearly every guess is wrong, with
    # the Zipf offsets most are right), with several-token launches in between, must give the bytes of the layer-by-layer
    # path for every token, and the same with the guessing switched off.
    cfg = workload.tiny_config(hidden=1024, experts=64, topk=10, inter=512)
    L = 3
    layers = [workload.LayerWeights(ctx, cfg, 601 + l, skew) for l in range(L)]
    stack = ctx.stack_create(cfg, [l.layer for l in layers], 2)
    out, out2 = ctx.alloc(cfg.hidden * 4), ctx.alloc(2 * cfg.hidden * 4)
    xs = [workload.hidden_rows(ctx, 1, cfg.hidden, 40 + i) for i in range(6)]
    x2 = workload.hidden_rows(ctx, 2, cfg.hidden, 77)
    want, ids = [], []
    n = cfg.topk
    trace_ids, trace_w = ctx.alloc(L * n * 4), ctx.alloc(L * n * 4)
    for x in xs:
        ctx.stack_decode(stack, x, 1, out, z.StackTrace(trace_ids.ptr, trace_w.ptr, None, None), layered=True); ctx.moe_check()
        want.append(out.numpy(f32).tobytes()); ids.append(trace_ids.numpy(np.int32).reshape(L, n).copy())
    repeats = sum(len(set(a[l]) & set(b[l])) for a, b in zip(ids, ids[1:]) for l in range(L)) / (L * n * (len(ids) - 1))
    print(f"skew {skew}: {repeats:.2f} of a layer's experts repeat from one token to the next")
    for on in (1, 0, 1):
        ctx.stack_set_speculation(stack, on)
        for i in (0, 1, 1, 2, 3, 3, 4, 5, 0):
            ctx.stack_decode(stack, xs[i], 1, out); ctx.moe_check()
            assert out.numpy(f32).tobytes() == want[i], f"token {i}, guessing {'on' if on else 'off'}"
            if i == 2:
                ctx.stack_decode(stack, x2, 2, out2); ctx.moe_check()
    ctx.stack_destroy(stack)
    for l in layers:
        for b in (l.router, l.shared_gate, l.shared_record, l.records):
            ctx.free(b)
    for b in xs + [x2, out, out2, trace_ids, trace_w]:
        ctx.free(b)
