"""The callers' glue either side of the MoE layer (reference: model.cpp:328-351, 651, 662; qwen.metal:36-40, 545-595):
unary / binary operators, the four-stream mix, the residual injection and the grouped RMS norm of the CPU oracle,
pinned by the reference's captured tables and by what the definitions fix."""
import json
import os
import numpy as np
import oracle

f32 = np.float32
G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


def bf(a):
    return oracle.bf(np.asarray(a, f32))


def test_unary_tables():  # tests/test_qwen.cpp:876-889: SiLU, sigmoid, softplus at 64 points, exact
    a = G["activations"]
    x = np.array(a["x"], f32)
    for op, name in ((0, "silu"), (1, "sigmoid"), (4, "softplus")):
        assert oracle.unary(x, op).tobytes() == bf(np.array(a[name], f32)).tobytes(), name


def test_unary_boundary_and_composites():
    b = G["activations"]["boundary"]  # tests/test_qwen.cpp:890-897
    assert oracle.unary(np.array(b["x"], f32), 0).tolist() == b["silu"]
    x = np.array(G["activations"]["x"], f32)
    quarter = bf(x / f32(4))
    assert oracle.unary(x, 2).tobytes() == oracle.unary(quarter, 0).tobytes()               # SiLU of the BF16 quarter
    assert oracle.unary(x, 3).tobytes() == bf(f32(2) * oracle.unary(quarter, 1)).tobytes()   # twice its sigmoid


def test_softplus_properties():
    x = np.linspace(-30, 30, 4001).astype(f32)
    y = oracle.unary(x, 4).astype(np.float64)
    want = np.logaddexp(0.0, x.astype(np.float64))
    assert np.max(np.abs(y - want) / np.maximum(want, 1e-30)) < 2.0 ** -7      # three BF16 roundings
    assert np.all(np.diff(y) >= 0)
    assert oracle.lib.zco_softplus_bf(f32(40.0)) == 40.0 and oracle.lib.zco_softplus_bf(f32(-200.0)) == 0.0
    y1 = np.linspace(1, 2, 1001).astype(f32)
    oracle.lib.zco_log_1to2.restype = oracle.C.c_float; oracle.lib.zco_log_1to2.argtypes = [oracle.C.c_float]
    got = np.array([oracle.lib.zco_log_1to2(float(v)) for v in y1], f32)
    assert got.tobytes() == np.log(y1.astype(np.float64)).astype(f32).tobytes()  # correctly rounded on this grid


def test_binary():
    rng = np.random.default_rng(3)
    x, y = bf(rng.normal(size=300)), bf(rng.normal(size=300))
    assert oracle.binary(x, y, 0).tobytes() == bf(x + y).tobytes()
    assert oracle.binary(x, y, 1).tobytes() == bf(x * y).tobytes()
    assert oracle.binary(x, x, 0).tobytes() == bf(f32(2) * x).tobytes()   # the reference tests' doubling dispatch


def test_hc_mix_and_add_against_loops():
    rng = np.random.default_rng(5)
    T, H = 3, 96
    x, w = bf(rng.normal(size=(T, 4, H))), bf(rng.normal(size=(T, 4, H)))
    want = np.zeros((T, H), f32)
    for h in range(4):
        want = bf(want + bf(x[:, h] * w[:, h]))
    assert oracle.hc_mix(x, w, T, H).tobytes() == bf(want / f32(4)).tobytes()
    ones = np.ones((T, 4, H), f32)
    assert oracle.hc_mix(x, ones, T, H).tobytes() == bf(bf(bf(bf(x[:, 0] + x[:, 1]) + x[:, 2]) + x[:, 3]) / f32(4)).tobytes()
    hyper, row, inject = bf(rng.normal(size=(T, 4, H))), bf(rng.normal(size=(T, H))), bf(rng.normal(size=(T, 4)))
    want = bf(hyper + bf(row[:, None, :] * inject[:, :, None]))
    assert oracle.hc_add(hyper, row, inject, T, H).tobytes() == want.tobytes()
    assert oracle.hc_add(hyper, row, np.zeros((T, 4), f32), T, H).tobytes() == hyper.tobytes()


def test_norm_closed_forms_and_double_precision():
    # constant rows: the mean square is c*c exactly (power-of-two sizes), so y = bf(bf(c / sqrt(c*c + 1e-6)) * w)
    D, width, T = 512, 1024, 2
    c = f32(3.0)
    w = (np.arange(width) % 7 + 1).astype(f32)
    inv = f32(1) / np.sqrt(f32(c * c + f32(1e-6)), dtype=f32)
    got = oracle.norm(np.full(T * width, c, f32), w, D, width, T)
    assert got.tobytes() == bf(bf(c * inv) * np.tile(w, T)).tobytes()
    # random rows, BF16 weights, shapes of the reference's own test (tests/test_qwen.cpp:1137-1145) incl. 320 = 2.5 blocks
    rng = np.random.default_rng(9)
    for D, width, T in ((2560, 10240, 1), (2560, 10240, 3), (512, 1024, 2), (320, 640, 1)):
        x = bf(3 * rng.normal(size=T * width))
        wb = (bf(1 + 0.1 * rng.normal(size=width)).view(np.uint32) >> 16).astype(np.uint16)
        got = oracle.norm(x, wb, D, width, T).astype(np.float64)
        xd = x.astype(np.float64).reshape(-1, D)
        want = (xd / np.sqrt((xd * xd).mean(1, keepdims=True) + 1e-6)).reshape(T, width) * (wb.astype(np.uint32) << 16).view(f32).astype(np.float64)
        assert np.max(np.abs(got - want.reshape(-1))) <= 2.0 ** -7 * np.max(np.abs(want))   # two BF16 roundings
    # a sum order that ignored the block structure would still pass the tolerance; the per-block lane sums are pinned
    # by a row whose squares need the exact order: one large value per block plus many small ones
    D = 256
    x = np.full(D, 2.0 ** -6, f32); x[0] = x[128] = 64.0
    acc = np.zeros(32, f32)
    blocks = []
    for block in (0, 128):
        lanes = np.zeros(32, f32)
        for lane in range(32):
            for i in range(4):
                lanes[lane] = f32(lanes[lane] + f32(x[block + lane * 4 + i] * x[block + lane * 4 + i]))
        s = lanes.copy()
        for stride in (16, 8, 4, 2, 1):
            s[:stride] = s[:stride] + s[stride:2 * stride]
        blocks.append(s[0])
    total = f32(blocks[0] + blocks[1])
    inv = f32(1) / np.sqrt(f32(total / f32(D) + f32(1e-6)), dtype=f32)
    got = oracle.norm(x, np.ones(D, f32), D, D, 1)
    assert got.tobytes() == bf(bf(x * inv)).tobytes()
