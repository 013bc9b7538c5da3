"""Pins the CPU oracle with the reference's own known-answer vectors and with
brute force; each test names the reference test it restates (tests/test_qwen.cpp)."""
import json
import math
import os
import random
import numpy as np
import pytest
import oracle

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
f32 = np.float32


def bits(x):
    return int(np.asarray(x, dtype=np.float32).reshape(-1)[:1].view(np.uint32)[0])


def test_bf16_rounding():  # :277-283 and storage.cpp:30-35
    assert oracle.lib.zco_b16(0x3f80) == 1.0
    assert oracle.lib.zco_bf(1.00390625) == 1.0          # tie -> even
    assert oracle.lib.zco_bf(1.01171875) == 1.015625      # tie -> even, upward
    assert math.isnan(oracle.lib.zco_bf(float("nan")))
    assert math.isinf(oracle.lib.zco_bf(float("inf")))
    x = np.random.default_rng(1).standard_normal(10000).astype(np.float32)
    r = oracle.bf(x)
    assert ((r.view(np.uint32) & 0xffff) == 0).all()
    assert (np.abs(r - x) <= np.abs(x) * 2.0 ** -8).all()
    assert all(oracle.lib.zco_bf(float(v)) == float(w) for v, w in zip(x[:200], r[:200]))


def test_exp_is_accurate():
    xs = np.linspace(-80, 80, 20001).astype(np.float32)
    got = np.array([oracle.lib.zco_expf(float(v)) for v in xs], dtype=np.float64)
    want = np.exp(xs.astype(np.float64))
    assert np.max(np.abs(got - want) / want) < 1.5e-7     # about one fp32 ulp
    assert oracle.lib.zco_expf(0.0) == 1.0
    assert oracle.lib.zco_expf(float("-inf")) == 0.0 and math.isinf(oracle.lib.zco_expf(100.0))
    assert math.isnan(oracle.lib.zco_expf(float("nan")))


def test_bf16_activation_tables():  # :876-889 (unary op 1 = bf(sigmoid_bf), op 0 = bf(v*sigmoid_bf(v)))
    a = G["activations"]
    for x, s, y in zip(a["x"], a["sigmoid"], a["silu"]):
        sig = oracle.lib.zco_sigmoid_bf(x)
        # the table prints BF16 values with ten digits; rounding to BF16 recovers the exact value
        assert bits(sig) == bits(oracle.bf(f32(s))), (x, sig, s)
        assert bits(oracle.bf(f32(x) * f32(sig))) == bits(oracle.bf(f32(y))), (x,)


def test_sigmoid_exp_rounding_boundary():  # :890-897
    b = G["activations"]["boundary"]
    for x, want in zip(b["x"], b["silu"]):
        assert oracle.bf(f32(x) * f32(oracle.lib.zco_sigmoid_bf(x))).item() == want


def _q4_case():
    K, N, T = 128, 7, 3
    w = np.array([(0x76543210 + (i % 8) * 0x11111111) & 0xffffffff for i in range(N * K // 8)], dtype=np.uint32)
    s = np.full(N * K // 64, 0x3d80, np.uint16); b = np.full(N * K // 64, 0xbe80, np.uint16)
    x = np.array([(i % 11 - 5) / 16 for i in range(T * K)], dtype=np.float32)
    return K, N, T, w, s, b, x


def test_q4_matmul_against_double():  # :634-652
    K, N, T, w, s, b, x = _q4_case()
    l = oracle.make_linear(w, s, b, K, N)
    got = oracle.linear(l, x, T)
    for t in range(T):
        for n in range(N):
            total = 0.0
            for k in range(K):
                word = int(w[n * K // 8 + k // 8])
                total += (((word >> (4 * (k % 8))) & 15) / 16.0 - 0.25) * float(x[t * K + k])
            assert got[t, n] == pytest.approx(oracle.bf(f32(total)).item(), rel=1e-4)


def test_swiglu_epilogue_identity():  # :653-659
    K, N, T, w, s, b, x = _q4_case()
    l = oracle.make_linear(w, s, b, K, N)
    lin = oracle.linear(l, x, T).ravel(); fused = oracle.gated_linear(l, l, x, T).ravel()
    for v, f in zip(lin, fused):
        y = oracle.bf(f32(1) / oracle.bf(f32(1) + oracle.bf(f32(math.exp(abs(float(v)))))))
        gate = y if v < 0 else oracle.bf(f32(1) - y)
        assert f == oracle.bf(oracle.bf(f32(v) * gate) * f32(v))


@pytest.mark.parametrize("K,N,Gs", [(320, 7, 64), (640, 8, 32), (2560, 8, 64)])
def test_q8_exact(K, N, Gs):  # :661-683: exact equality with the double-precision dot
    T = 3
    w = np.array([(i * 17 + 251) & 255 for i in range(K * N)], dtype=np.uint8)
    s = np.array([0xbb80 if i % 2 else 0x3b80 for i in range(K * N // Gs)], dtype=np.uint16)
    b = np.array([0xbf00 if i % 3 else 0x3e80 for i in range(K * N // Gs)], dtype=np.uint16)
    x = np.array([(i % 9 - 4) / 16 for i in range(T * K)], dtype=np.float32)
    got = oracle.linear(oracle.make_linear(w, s, b, K, N, Gs, 8), x, T)
    dec = (w.astype(np.float64).reshape(N, K) * np.repeat(oracle.b16(s).astype(np.float64).reshape(N, K // Gs), Gs, 1)
           + np.repeat(oracle.b16(b).astype(np.float64).reshape(N, K // Gs), Gs, 1))
    # the reference decodes in fp32: code*scale+bias, rounded to float once
    dec = (w.astype(np.float32).reshape(N, K) * np.repeat(oracle.b16(s).reshape(N, K // Gs), Gs, 1)
           + np.repeat(oracle.b16(b).reshape(N, K // Gs), Gs, 1)).astype(np.float64)
    want = oracle.bf((x.astype(np.float64).reshape(T, K) @ dec.T).astype(np.float32))
    assert (got == want).all()


def test_q4_bias_uses_bf16_sum_of_four():  # :863-874
    codes = np.zeros(16, np.uint32); sc = np.full(2, 0x3f80, np.uint16); bi = np.full(2, 0x3f80, np.uint16)
    x = np.zeros(128, np.float32); x[0::4] = 1; x[1::4] = 1.0 / 512; x[2::4] = -1
    out = oracle.linear(oracle.make_linear(codes, sc, bi, 128, 1), x, 1)
    assert out[0, 0] == 0.0          # exact dequantise-then-dot would give 1/16


def _router_case():
    r = G["router"]; T, K, N = r["T"], r["K"], r["N"]
    n = np.arange(N, dtype=np.int64)[:, None]; k = np.arange(K, dtype=np.int64)[None, :]
    wf = np.ldexp(((n * 17 + k * 23) % 251 - 125).astype(np.float32), -(k % 20 + 4).astype(np.int32)).astype(np.float32)
    w = (wf.view(np.uint32) >> 16).astype(np.uint16)
    t = np.arange(T, dtype=np.int64)[:, None]
    x = (((k * 13 + t * 31) % 251 - 125).astype(np.float32) / f32(128)).astype(np.float32)
    return r, T, K, N, w, x


def test_router_matches_captured_words():  # :798-814
    r, T, K, N, w, x = _router_case()
    full = oracle.router_logits(w, x, T, K, N).ravel()
    for i, e in zip(r["indices"], r["expected_bits"]):
        assert bits(full[i]) == e, (i, hex(bits(full[i])), hex(e))


def test_router_chunk_invariance_and_accuracy():  # :815-825
    r, T, K, N, w, x = _router_case()
    full = oracle.router_logits(w, x, T, K, N)
    for offset, count in ((0, 1), (1, 7), (8, 3)):
        part = oracle.router_logits(w, x[offset:offset + count], count, K, N)
        assert (part == full[offset:offset + count]).all()
    exact = x.astype(np.float64) @ oracle.b16(w).astype(np.float64).T
    assert np.max(np.abs(exact - full)) < r["max_abs_error_vs_double"]


def _stable_top(values, k=10):
    order = [e for e in range(len(values)) if values[e] > -math.inf]
    order.sort(key=lambda e: -values[e])           # Python's sort is stable
    return (order + [-1] * k)[:k]


def test_route_selects_ten_and_normalises():  # :744-754
    v = np.array([i % 41 - 100 for i in range(512)], dtype=np.float32)
    ids, w = oracle.route(v, 1, 512)
    assert list(ids[0]) == _stable_top(list(v))
    assert float(np.sum(w.astype(np.float64))) == pytest.approx(1, abs=1e-6)


def route_stress_values(T=137, E=512, seed=123):
    """Row types of tests/test_qwen.cpp:755-774 (the random stream differs; expectations are recomputed)."""
    rng = random.Random(seed)
    v = np.empty((T, E), np.float32)
    for t in range(T):
        for e in range(E):
            x = math.ldexp(rng.randrange(2001) - 1000, -rng.randrange(12))
            c = t % 10
            if c == 0: x = float(e)
            elif c == 1: x = -float(e)
            elif c == 2: x = float(e % 13)
            elif c == 3: x = 0.0 if e % 2 else -0.0
            elif c == 4: x = float(e) if e < 9 else -math.inf
            elif c == 5: x = math.nan if e % 41 == 0 else x
            elif c == 6: x = math.inf if e % 33 == 0 else x
            elif c == 7: x = -math.inf
            elif c == 8: x = math.nan
            v[t, e] = x
    return v


def test_route_ties_and_exceptional_scores():  # :755-781
    v = route_stress_values()
    ids, w = oracle.route(v, v.shape[0], 512)
    for t in range(v.shape[0]):
        assert list(ids[t]) == _stable_top([float(a) for a in v[t]]), t
    # finite rows normalise; rows made only of -inf/NaN give NaN weights, as the reference allows
    for t in range(v.shape[0]):
        if t % 10 in (0, 1, 2, 3, 9):
            assert float(np.sum(w[t].astype(np.float64))) == pytest.approx(1, abs=1e-6)
    # sub-batches reproduce the same bytes (:782-792)
    for offset, count in ((0, 1), (1, 7), (8, 31), (39, 97), (136, 1)):
        i2, w2 = oracle.route(v[offset:offset + count], count, 512)
        assert i2.tobytes() == ids[offset:offset + count].tobytes()
        assert w2.tobytes() == w[offset:offset + count].tobytes()


def _softmax64(scores):
    """w_j = exp(s_j - s_0) / sum_i exp(s_i - s_0) in double precision (qwen.metal:758-764)."""
    s = np.asarray(scores, dtype=np.float64)
    e = np.exp(s - s[0])
    return e / e.sum()


def test_route_weight_values_are_the_softmax_of_the_selected_scores():  # qwen.metal:758-764
    """The weight VALUES against an independent float64 softmax over the ten selected scores, relative 1e-6.
    A swapped subtraction (exp(s_0 - s_j)), a base other than e, a sum over more than the ten, or weights
    left in selection order of another row each miss this by orders of magnitude."""
    rng = np.random.default_rng(2718)
    rows = [np.array([i % 41 - 100 for i in range(512)], dtype=np.float32),        # the reference's ramp, ties of 12 or 13
            rng.standard_normal(512).astype(np.float32),
            (rng.standard_normal(512) * 4).astype(np.float32),                     # spread: weights over many decades
            np.round(rng.standard_normal(512) * 2).astype(np.float32),             # heavy exact ties
            (rng.standard_normal(512) * 0.01 + 7).astype(np.float32),              # near ties, nonzero base
            np.where(np.arange(512) % 7 == 0, np.float32(3.5), rng.standard_normal(512).astype(np.float32))]
    v = np.stack(rows).astype(np.float32)
    ids, w = oracle.route(v, v.shape[0], 512)
    for t in range(v.shape[0]):
        assert list(ids[t]) == _stable_top([float(a) for a in v[t]]), t
        scores = v[t][ids[t]]
        assert (np.diff(scores) <= 0).all()                                        # descending, so scores[0] is the base
        want = _softmax64(scores)
        got = w[t].astype(np.float64)
        assert np.max(np.abs(got - want) / want) <= 1e-6, (t, got, want)
        wrong = np.exp(scores[0].astype(np.float64) - scores.astype(np.float64))
        wrong /= wrong.sum()
        if scores[0] != scores[-1]:
            assert np.max(np.abs(got - wrong) / wrong) > 1e-3                       # the swapped subtraction is far away
    # eight selected scores of 3.5 or ties at the top: equal scores give equal weights, bit for bit
    t = 5
    assert len({bits(x) for x in w[t]}) == 1 and w[t][0] == pytest.approx(0.1, rel=1e-6)
    # fewer than ten finite scores: the missing slots carry weight exactly 0 (exp(-inf)) and the rest still sum to 1
    few = np.full((1, 512), -np.inf, np.float32)
    few[0, [5, 77, 300]] = [1.0, 0.0, -1.0]
    ids, w = oracle.route(few, 1, 512)
    assert list(ids[0]) == [5, 77, 300] + [-1] * 7
    assert (w[0, 3:] == 0).all()
    e = math.e
    want = np.array([e * e, e, 1.0]) / (e * e + e + 1.0)                            # closed form
    assert np.max(np.abs(w[0, :3].astype(np.float64) - want) / want) <= 1e-6


def test_exp32_against_double_precision():
    """The fp32 exponential shared by the oracle and the kernels, over the range the softmax uses (arguments <= 0)
    and the activations use, against libm's double exp: relative 2e-7 (about two units in the last place)."""
    xs = np.concatenate([-np.linspace(0, 87, 2001), np.linspace(0, 20, 501), [-0.0, -1e-8, -103.0, -200.0]]).astype(np.float32)
    got = oracle.exp32(xs).astype(np.float64)
    want = np.exp(xs.astype(np.float64))
    normal = want > 1.2e-38
    assert np.max(np.abs(got[normal] - want[normal]) / want[normal]) <= 2e-7
    assert (got[~normal] <= 1.2e-38).all() and (got >= 0).all()
    assert oracle.exp32(np.array([0.0], np.float32))[0] == 1.0


def test_moe_sum_midpoint():  # :827-842
    m = G["moe_sum"]; H = 2560
    e = np.zeros((10, H), np.float32); e[:, 0] = np.array(m["values"], dtype=np.float32)
    w = np.array(m["weight_bits"], dtype=np.uint32).view(np.float32)
    shared = np.zeros(H, np.float32); shared[0] = m["shared"]
    out = oracle.moe_sum(e, w, shared, np.array([m["gate"]], np.float32), 1, H)
    assert out[0, 0] == m["expected"] and m["expected"] != m["serial_order_gives"]
    assert (out[0, 1:] == 0).all()


def test_dispatch_is_stable_counting_sort():  # model.cpp:449-479, :1500-1530
    rng = np.random.default_rng(7)
    for T in (1, 2, 7, 33, 513):
        ids = np.stack([rng.permutation(512)[:10] for _ in range(T)]).astype(np.int32)
        off, slots, sel = oracle.dispatch(ids, T, 10, 512)
        flat = ids.ravel()
        positions = {e: [p for p in range(T * 10) if flat[p] == e] for e in set(flat.tolist())}
        assert list(sel) == sorted(positions)
        for e in sel:
            assert list(slots[off[e]:off[e + 1]]) == positions[int(e)]
        assert off[-1] == T * 10
    bad = np.zeros((1, 10), np.int32); bad[0, 3] = 512
    with pytest.raises(RuntimeError):
        oracle.dispatch(bad, 1, 10, 512)
    bad[0, 3] = -1
    with pytest.raises(RuntimeError):
        oracle.dispatch(bad, 1, 10, 512)


def test_scatter_rows_leave_other_slots_untouched():  # qwen.metal:800-803, :1087-1099
    H = 64; x = np.arange(3 * H, dtype=np.float32).reshape(3, H); out = np.full((12, H), -17, np.float32)
    oracle.scatter_experts(x, [9, 1, 7], H, out)
    assert (out[9] == x[0]).all() and (out[1] == x[1]).all() and (out[7] == x[2]).all()
    assert (np.delete(out, [9, 1, 7], 0) == -17).all()


@pytest.mark.parametrize("K,N", [(2560, 640), (640, 2560), (704, 2560), (2560, 512), (512, 1024)])
def test_q4_lane_width_shapes_track_double(K, N):  # shapes of :1100-1125; value check only
    rng = np.random.default_rng(K * 7 + N)
    w = rng.integers(0, 2 ** 32, N * K // 8, dtype=np.uint64).astype(np.uint32)
    s = oracle.bf_bits(0.01 * np.abs(rng.standard_normal(N * K // 64)) + 1e-4)
    b = oracle.bf_bits(-0.08 * np.abs(rng.standard_normal(N * K // 64)))
    x = oracle.bf(0.7 * rng.standard_normal(K))
    got = oracle.linear(oracle.make_linear(w, s, b, K, N), x, 1, float_output=True)[0]
    codes = ((w.reshape(N, K // 8, 1) >> (4 * np.arange(8, dtype=np.uint32))) & 15).reshape(N, K).astype(np.float64)
    dec = codes * np.repeat(oracle.b16(s).astype(np.float64).reshape(N, -1), 64, 1) + np.repeat(
        oracle.b16(b).astype(np.float64).reshape(N, -1), 64, 1)
    want = dec @ x.astype(np.float64)
    assert np.max(np.abs(got - want)) < 2e-2 * np.max(np.abs(want)) + 1e-3   # BF16 bias-sum rule bounds the gap


# ---- lane partitions pinned by exact arithmetic -------------------------------------------------------------------
# fp32 cannot hold 2^24 + 1: added to 2^24 a one is lost, added to -(2^24) it is kept.  Inputs built from
# {2^24, -2^24, 1} therefore give a result that depends on WHICH additions share an accumulator, while every other
# addition in the kernel is exact, so the expected values below follow from the kernel text alone (which element
# belongs to which lane), not from the order of the final lane sum.
BIG = float(2 ** 24)


@pytest.mark.parametrize("K,N,tokens", [(10240, 4, 1), (2560, 1, 1), (2560, 48, 2), (2560, 64, 1)])   # shapes of :1126-1135
def test_plain_mm_tracks_double(K, N, tokens):  # qwen.metal:499-506
    rng = np.random.default_rng(K + N)
    w = oracle.bf_bits(0.02 * rng.standard_normal(N * K)); x = oracle.bf(rng.standard_normal(tokens * K))
    got = oracle.plain_mm(w, x, K, N, tokens, float_output=True)
    wd = oracle.b16(w).astype(np.float64).reshape(N, K); xd = x.astype(np.float64).reshape(tokens, K)
    want = xd @ wd.T
    bound = 2.0 ** -23 * (K // 32 + 6) * (np.abs(xd) @ np.abs(wd).T)   # a lane chain of K/32 terms, five butterfly steps
    assert (np.abs(got - want) <= bound).all()
    rounded = oracle.plain_mm(w, x, K, N, tokens)
    assert rounded.tobytes() == oracle.bf(got).tobytes()


def test_plain_mm_lane_chain_is_k_mod_32():  # qwen.metal:503: lane l adds k = l, l + 32, l + 64, ... in turn
    K, N, T = 2560, 3, 2
    w = np.full(N * K, 0x3f80, np.uint16)                   # every weight 1.0: the products are the inputs
    x = np.ones((T, K), f32)
    # token 0: 2^24 and -2^24 meet in lane 5 (k = 5 and k = 37), so they cancel before any one is added:
    # lane 5 holds K/32 - 2, every other lane K/32, all exact, and so is their sum whatever its order.
    x[0, 5] = BIG; x[0, 37] = -BIG
    # token 1: the same pair one element apart (lanes 6 and 7): lane 6 loses its 79 ones (2^24 + 1 -> 2^24), lane 7
    # keeps them (-(2^24) + 79 is exact); both lanes together give 79, the other thirty lanes 80 each.
    x[1, 6] = BIG; x[1, 7] = -BIG
    got = oracle.plain_mm(w, x, K, N, T, float_output=True)
    assert (got[0] == K - 2).all(), got          # a k-ascending sum over all lanes gives K - 33, a stride of 64 loses lane 5's ones
    assert (got[1] == 79 + 30 * 80).all(), got
    assert oracle.plain_mm(w, x, K, N, T).tobytes() == oracle.bf(got).tobytes()
    # rows and tokens are indexed as [n][K] and [t][K]: a weight row of zeros silences exactly its own output
    w2 = w.copy(); w2[K:2 * K] = 0
    got2 = oracle.plain_mm(w2, x, K, N, T, float_output=True)
    assert (got2[:, 1] == 0).all() and (got2[:, 0] == got[:, 0]).all() and (got2[:, 2] == got[:, 2]).all()


def _q4_bias_only(K, N, x):
    """Codes 0, every bias 1.0: a row's output is the lane-ordered sum of the blocks' BF16 chain sums."""
    w = np.zeros(N * K // 8, np.uint32)
    s = np.full(N * K // 64, 0x3f80, np.uint16); b = np.full(N * K // 64, 0x3f80, np.uint16)
    return oracle.linear(oracle.make_linear(w, s, b, K, N), np.asarray(x, f32), 1, float_output=True)[0]


def test_q4_lane_width_rule_bit_level():  # qwen.metal:46-62; metal.mm:795-803: sixteen elements per lane step iff K % 512 == 0 and N % 8 == 0
    # elements 0..15 carry the four quads (1, 2^24, 1, -2^24).  In one lane step of sixteen, the chain sums meet in one
    # accumulator: ((1 + 2^24) + 1) - 2^24 = 0.  In steps of eight, lane 0 holds 1 + 2^24 -> 2^24 and lane 1 holds
    # 1 - 2^24 exactly: together 1.  All other lanes hold zero, so the order of the lane sum does not matter.
    def row(K):
        x = np.zeros(K, f32); x[0] = 1; x[4] = BIG; x[8] = 1; x[12] = -BIG
        return x
    assert (_q4_bias_only(512, 8, row(512)) == 0.0).all()      # wide lanes
    assert (_q4_bias_only(1024, 16, row(1024)) == 0.0).all()
    assert (_q4_bias_only(256, 8, row(256)) == 1.0).all()      # K % 512 != 0: narrow lanes
    assert (_q4_bias_only(512, 7, row(512)) == 1.0).all()      # N % 8 != 0: narrow lanes
    assert (_q4_bias_only(704, 8, row(704)) == 1.0).all()      # the reference's own narrow shape (:1103)


def test_q4_lane_revisits_every_32nd_block():  # qwen.metal:51: base = lane * width + j * 32 * width
    # wide lanes, K = 1536: lane 3 owns the blocks at elements 48, 560 and 1072; their chain sums 2^24, 1, -2^24 meet in
    # that order in lane 3's accumulator: (2^24 + 1) - 2^24 = 0.  Contiguous blocks per lane, or any other stride, would
    # leave the one in a lane of its own.
    K = 1536
    x = np.zeros(K, f32); x[48] = BIG; x[560] = 1; x[1072] = -BIG
    assert (_q4_bias_only(K, 8, x) == 0.0).all()
    x = np.zeros(K, f32); x[48] = BIG; x[64] = 1; x[1072] = -BIG     # the one in lane 4 instead: it survives
    assert (_q4_bias_only(K, 8, x) == 1.0).all()
