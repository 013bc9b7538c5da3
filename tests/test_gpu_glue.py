"""The callers' glue either side of the MoE layer on the GPU (zc_hip_unary / binary / hc_mix / hc_add / norm) against
the CPU oracle, byte for byte, and the reference's captured activation tables (tests/test_qwen.cpp:876-897)."""
import json
import os
import numpy as np
import pytest
import oracle
import zerocool_amd as z

pytestmark = pytest.mark.gpu
f32 = np.float32
G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


@pytest.fixture(scope="module")
def ctx():
    c = z.Context(0)
    yield c
    c.close()


def bf(a):
    return oracle.bf(np.asarray(a, f32))


def test_unary_tables_and_oracle(ctx):
    a = G["activations"]
    x = np.array(a["x"], f32)
    dev = ctx.upload(x)
    for op, name in ((0, "silu"), (1, "sigmoid"), (4, "softplus")):
        got = ctx.unary(dev, x.size, op).numpy(f32)
        assert got.tobytes() == bf(np.array(a[name], f32)).tobytes(), name
    b = G["activations"]["boundary"]
    assert ctx.unary(ctx.upload(np.array(b["x"], f32)), 2, 0).numpy(f32).tolist() == b["silu"]
    rng = np.random.default_rng(11)
    wide = np.concatenate([bf(rng.normal(size=50000) * 6), np.array([0.0, -0.0, 100.0, -100.0, np.inf, -np.inf, 1e-30, -1e-30], f32)])
    dev = ctx.upload(wide)
    for op in range(5):
        got, want = ctx.unary(dev, wide.size, op).numpy(f32), oracle.unary(wide, op)
        assert got.tobytes() == want.tobytes(), op


def test_binary_mix_add(ctx):
    rng = np.random.default_rng(12)
    T, H = 5, 2560
    x, y = bf(rng.normal(size=T * H)), bf(rng.normal(size=T * H))
    dx, dy = ctx.upload(x), ctx.upload(y)
    for op in (0, 1):
        assert ctx.binary(dx, dy, x.size, op).numpy(f32).tobytes() == oracle.binary(x, y, op).tobytes()
    a, w = bf(rng.normal(size=(T, 4, H))), bf(rng.normal(size=(T, 4, H)))
    assert ctx.hc_mix(ctx.upload(a), ctx.upload(w), T, H).numpy(f32).tobytes() == oracle.hc_mix(a, w, T, H).tobytes()
    inject = bf(rng.normal(size=(T, 4)))
    got = ctx.hc_add(ctx.upload(a), dx, ctx.upload(inject), T, H).numpy(f32)
    assert got.tobytes() == oracle.hc_add(a, x.reshape(T, H), inject, T, H).tobytes()


@pytest.mark.parametrize("D,width,tokens", [(2560, 10240, 1), (2560, 10240, 3), (512, 1024, 2), (320, 640, 1), (128, 128, 7), (4096, 4096, 2)])
def test_norm(ctx, D, width, tokens):   # shapes of tests/test_qwen.cpp:1137-1145 and the limits
    rng = np.random.default_rng(D + tokens)
    x = bf(3 * rng.normal(size=tokens * width))
    wb = (bf(1 + 0.1 * rng.normal(size=width)).view(np.uint32) >> 16).astype(np.uint16)
    got = ctx.norm(ctx.upload(x), ctx.upload(wb), 0, D, width, tokens).numpy(f32)
    assert got.tobytes() == oracle.norm(x, wb, D, width, tokens).tobytes()
    wf = (wb.astype(np.uint32) << 16).view(f32)
    assert ctx.norm(ctx.upload(x), ctx.upload(wf), 1, D, width, tokens).numpy(f32).tobytes() == got.tobytes()


def test_glue_rejects_bad_shapes(ctx):
    x = ctx.alloc(1024)
    with pytest.raises(z.ZcError):
        ctx.unary(x, 16, 9)
    with pytest.raises(z.ZcError):
        ctx.norm(x, x, 0, 48, 100, 1)      # width not a multiple of the group
    with pytest.raises(z.ZcError):
        ctx.norm(x, x, 0, 8192, 8192, 1)   # group beyond 4096
