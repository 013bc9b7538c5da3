"""Whole-layer parity (Model::moe, model.cpp:431-557) of the HIP path against the CPU
oracle on the same seeded weights and inputs: routing ids, dispatch permutation and every
intermediate the reference can dump (--trace-dir, model.cpp:447-448, 549-552) byte for byte,
and the layer output within the north-star tolerance max|d|/max|ref| <= 2e-3 (it is in fact
bit-identical: the kernels keep the reference's lane partition and rounding boundaries)."""
import numpy as np
import pytest
import oracle
import zerocool_amd as z
from zerocool_amd import workload

pytestmark = pytest.mark.gpu
f32 = np.float32
TOLERANCE = 2e-3


@pytest.fixture(scope="module")
def ctx():
    c = z.Context(0)
    yield c
    c.close()


def oracle_cfg(cfg):
    return oracle.Config(*[getattr(cfg, n) for n, _ in z.Config._fields_])


def run_layer(ctx, cfg, weights, x_dev, T):
    n = T * cfg.topk
    ws = ctx.alloc(ctx.moe_workspace_bytes(cfg, T))
    out = ctx.alloc(T * cfg.hidden * 4)
    bufs = dict(logits=ctx.alloc(T * cfg.experts * 4), ids=ctx.alloc(n * 4), weights=ctx.alloc(n * 4),
                expert_out=ctx.alloc(n * cfg.hidden * 4), shared=ctx.alloc(T * cfg.hidden * 4), gate=ctx.alloc(T * 4))
    trace = z.Trace(*[bufs[k].ptr for k in ("logits", "ids", "weights", "expert_out", "shared", "gate")])
    ctx.moe_forward(cfg, weights.layer, x_dev, T, out, ws, trace)
    ctx.moe_check()
    got = {k: v.numpy(np.int32 if k == "ids" else f32) for k, v in bufs.items()}
    got["out"] = out.numpy(f32)
    for b in list(bufs.values()) + [ws, out]:
        ctx.free(b)
    return got


def check_layer(ctx, cfg, T, seed, skew):
    weights = workload.LayerWeights(ctx, cfg, seed, skew)
    x_dev = workload.hidden_rows(ctx, T, cfg.hidden, seed * 977 + T)
    x = x_dev.numpy(f32)
    got = run_layer(ctx, cfg, weights, x_dev, T)
    h = weights.host()
    want, tr = oracle.moe_layer(oracle_cfg(cfg), h["router"], h["shared_gate"], h["shared_record"], h["records"],
                                h["stride"], x, T, router_offsets=h["offsets"], threads=8, trace=True)
    assert got["ids"].tobytes() == tr["ids"].tobytes(), "routing ids differ"
    assert got["logits"].tobytes() == tr["logits"].tobytes()
    assert got["weights"].tobytes() == tr["weights"].tobytes()
    assert got["gate"].tobytes() == tr["gate"].tobytes()
    assert got["shared"].tobytes() == tr["shared"].tobytes()
    assert got["expert_out"].tobytes() == tr["expert_out"].tobytes()
    rel = float(np.max(np.abs(got["out"] - want.ravel())) / np.max(np.abs(want)))
    assert rel <= TOLERANCE
    assert got["out"].tobytes() == want.tobytes()
    for b in (weights.router, weights.shared_gate, weights.shared_record, weights.records, x_dev):
        ctx.free(b)
    return tr


@pytest.mark.parametrize("T", [1, 2, 7, 33, 129])
def test_tiny_layer(ctx, T):
    tr = check_layer(ctx, workload.tiny_config(), T, 11, ("normal", 0.5))
    assert len(np.unique(tr["ids"])) <= 32


def test_tiny_layer_mixed_bits_and_group32(ctx):
    check_layer(ctx, workload.tiny_config(bits=(4, 8, 8, 8)), 9, 12, None)
    check_layer(ctx, workload.tiny_config(hidden=512, inter=256, group=32, bits=(8, 4, 4, 8)), 5, 13, None)


@pytest.mark.parametrize("T", [1, 8, 32, 64])
def test_single_layer_config(ctx, T):  # BASELINE configs 1 and 2: every batch size the configuration names
    tr = check_layer(ctx, workload.config("S"), T, 1, ("normal", 0.5))
    print(f"T={T}: {len(np.unique(tr['ids']))} distinct experts for {T * 10} slots")


@pytest.mark.parametrize("T", [1, 16])
def test_mixed_artifact_config(ctx, T):  # BASELINE config 4: decode batch 1 and 16
    check_layer(ctx, workload.config("S-mixed"), T, 4, None)


def test_reference_shape(ctx):  # hidden 2560 / intermediate 640: the narrow-lane (width 8) down projection
    check_layer(ctx, workload.config("ref"), 2, 5, None)


def test_invalid_router_output_is_reported(ctx):  # model.cpp:459
    cfg = workload.tiny_config()
    weights = workload.LayerWeights(ctx, cfg, 3, None)
    T = 2
    x = np.full(T * cfg.hidden, np.nan, f32)      # NaN logits: nothing is selectable, ids = -1
    ws = ctx.alloc(ctx.moe_workspace_bytes(cfg, T)); out = ctx.alloc(T * cfg.hidden * 4)
    ctx.moe_forward(cfg, weights.layer, ctx.upload(x), T, out, ws)
    with pytest.raises(z.ZcError) as err:
        ctx.moe_check()
    assert "invalid router output" in str(err.value)
    ctx.moe_check()      # flag cleared


def test_layer_rejects_bad_geometry(ctx):
    cfg = workload.tiny_config()
    weights = workload.LayerWeights(ctx, cfg, 3, None)
    ws = ctx.alloc(ctx.moe_workspace_bytes(cfg, 1)); x = ctx.zeros(cfg.hidden * 4)
    with pytest.raises(z.ZcError):
        ctx.moe_forward(cfg, weights.layer, x, 1, x, ws)                  # output aliases input
    with pytest.raises(z.ZcError):
        ctx.moe_forward(cfg, weights.layer, x, 0, ctx.alloc(64), ws)      # no tokens
    bad = workload.tiny_config(group=48)
    with pytest.raises(z.ZcError):
        ctx.moe_forward(bad, weights.layer, x, 1, ctx.alloc(cfg.hidden * 4), ws)
    ctx.finish()
