"""The exact-integer matrix-core form of the affine Q4 products must give the same
bytes as the CPU oracle (and so as the literal lane kernels) on wide shapes, for any
input: BF16-valued rows (the fast case), rows with huge dynamic range, zeros,
subnormals, infinities, NaN and values that are not BF16-representable (all of which
must take the per-block literal fallback)."""
import numpy as np
import pytest
import oracle
import zerocool_amd as z

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.fixture(scope="module")
def ctx():
    c = z.Context(0)
    yield c
    c.close()


def make(rng, K, N):
    return (rng.integers(0, 2 ** 32, N * K // 8, dtype=np.uint64).astype(np.uint32),
            oracle.bf_bits(0.002 + 0.018 * rng.random(N * K // 64)),
            oracle.bf_bits(-0.08 * rng.random(N * K // 64)))


def dev_linear(ctx, w, s, b, K, N):
    bufs = (ctx.upload(w), ctx.upload(s), ctx.upload(b))
    l = z.Linear(bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, K, N, 64, 0, 1, 4)
    l._keep = bufs
    return l


def inputs(rng, K, T, kind):
    x = oracle.bf(rng.standard_normal((T, K)))
    if kind == "wide-range":
        x = oracle.bf(x * np.exp2(rng.integers(-30, 30, (T, K))).astype(f32))
    elif kind == "sparse":
        x[rng.random((T, K)) < 0.7] = 0
        x[0, :64] = 0
    elif kind == "special":
        x[0, 5] = np.inf; x[min(1, T - 1), 17] = np.nan; x[0, 100] = -0.0
        x[0, 200:216] = np.array([1e-40, -3e-41] * 8, f32)          # subnormals
        x[0, 300] = f32(1.0000001)                                   # not BF16-representable
        x[0, 400:416] = oracle.bf(np.array([3e38, -3e38] * 8, f32))
    elif kind == "activations":
        x = oracle.bf(x * x * np.sign(rng.standard_normal((T, K))) * 0.1)   # product-shaped, like SwiGLU outputs
    return np.ascontiguousarray(x, dtype=f32)


@pytest.mark.parametrize("K,N", [(2048, 512), (512, 2048), (3072, 1024), (1024, 3072), (2560, 640), (512, 8), (1024, 24)])
@pytest.mark.parametrize("kind", ["normal", "wide-range", "sparse", "special", "activations"])
def test_xint_matches_oracle(ctx, K, N, kind):
    rng = np.random.default_rng(K * 131 + N + len(kind))
    a, u = make(rng, K, N), make(rng, K, N)
    ol, ou = oracle.make_linear(*a, K, N), oracle.make_linear(*u, K, N)
    dl, du = dev_linear(ctx, *a, K, N), dev_linear(ctx, *u, K, N)
    for T in (1, 3, 9):
        x = inputs(rng, K, T, kind); dx = ctx.upload(x)
        rows = rng.integers(0, T, T).astype(np.int32)
        ctx.configure(1)
        got = [ctx.linear(dl, dx, T).numpy(f32), ctx.linear(dl, dx, T, float_output=True).numpy(f32),
               ctx.gated_linear(dl, du, dx, T, T).numpy(f32), ctx.gated_linear(dl, du, dx, T, T, ctx.upload(rows)).numpy(f32)]
        ctx.configure(0)
        lit = [ctx.linear(dl, dx, T).numpy(f32), ctx.linear(dl, dx, T, float_output=True).numpy(f32),
               ctx.gated_linear(dl, du, dx, T, T).numpy(f32), ctx.gated_linear(dl, du, dx, T, T, ctx.upload(rows)).numpy(f32)]
        ctx.configure(1)
        want = [oracle.linear(ol, x, T), oracle.linear(ol, x, T, float_output=True), oracle.gated_linear(ol, ou, x, T),
                oracle.gated_linear(ol, ou, x, T, rows)]
        for g, l, w in zip(got, lit, want):
            assert l.tobytes() == w.tobytes()
            assert g.tobytes() == w.tobytes(), (K, N, kind, T, int((g.view(np.uint32) != w.ravel().view(np.uint32)).sum()))
        ctx.free(dx)
    for b in dl._keep + du._keep:
        ctx.free(b)


@pytest.mark.parametrize("kind", ["normal", "wide-range", "special", "activations"])
def test_xint_32_column_tiles(ctx, kind):
    """Calls with enough tokens to fill the chip take the tile engine's 32-column form (v_mfma_i32_32x32x32_i8, up to four
    tokens per instruction): the same bytes as the literal lane kernels on every token, and as the oracle on a sample; the
    sizes leave partial tiles (2056 rows) and a partial last group of tokens (130)."""
    K, N, T = 1024, 2056, 130
    rng = np.random.default_rng(77 + len(kind))
    a, u = make(rng, K, N), make(rng, K, N)
    ol, ou = oracle.make_linear(*a, K, N), oracle.make_linear(*u, K, N)
    dl, du = dev_linear(ctx, *a, K, N), dev_linear(ctx, *u, K, N)
    x = inputs(rng, K, T, kind); dx = ctx.upload(x)
    rows = rng.integers(0, T, T).astype(np.int32); drows = ctx.upload(rows)
    ctx.configure(1)
    got = [ctx.linear(dl, dx, T).numpy(f32), ctx.linear(dl, dx, T, float_output=True).numpy(f32),
           ctx.gated_linear(dl, du, dx, T, T).numpy(f32), ctx.gated_linear(dl, du, dx, T, T, drows).numpy(f32)]
    ctx.configure(0)
    lit = [ctx.linear(dl, dx, T).numpy(f32), ctx.linear(dl, dx, T, float_output=True).numpy(f32),
           ctx.gated_linear(dl, du, dx, T, T).numpy(f32), ctx.gated_linear(dl, du, dx, T, T, drows).numpy(f32)]
    ctx.configure(1)
    for g, l in zip(got, lit):
        assert g.tobytes() == l.tobytes(), (kind, int((g.view(np.uint32) != l.view(np.uint32)).sum()))
    sample = np.r_[0:6, T - 2:T]
    want = [oracle.linear(ol, x[sample], len(sample)), oracle.gated_linear(ol, ou, x[sample], len(sample))]
    assert got[0].reshape(T, N)[sample].tobytes() == want[0].tobytes()
    assert got[2].reshape(T, N)[sample].tobytes() == want[1].tobytes()
    for b in dl._keep + du._keep + (dx, drows):
        ctx.free(b)
