"""The allocation-free layer entry point (zc_hip_moe_forward_static): same kernels as zc_hip_moe_forward with the
workspace in the library's static device array.  Checked through the C ABI against zc_hip_moe_forward on the same
inputs, byte for byte (outputs and every traced intermediate), on two calls in a row, the second with a smaller input,
so that the second call runs over whatever the first one left in the shared array."""
import ctypes as C
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


def run(ctx, cfg, weights, x, T, static):
    n = T * cfg.topk
    out = ctx.alloc(T * cfg.hidden * 4)
    names = ("logits", "ids", "weights", "expert_out", "shared", "gate")
    sizes = dict(logits=T * cfg.experts * 4, ids=n * 4, weights=n * 4, expert_out=n * cfg.hidden * 4, shared=T * cfg.hidden * 4, gate=T * 4)
    bufs = {k: ctx.alloc(sizes[k]) for k in names}
    trace = z.Trace(*[bufs[k].ptr for k in names])
    if static:
        ctx.moe_forward_static(cfg, weights.layer, x, T, out, trace)
    else:
        ws = ctx.alloc(ctx.moe_workspace_bytes(cfg, T))
        ctx.fill(ws, 0xa5)
        ctx.moe_forward(cfg, weights.layer, x, T, out, ws, trace)
    ctx.moe_check()
    got = {k: bufs[k].numpy(np.uint8).tobytes() for k in names}
    got["out"] = out.numpy(np.uint8).tobytes()
    for b in list(bufs.values()) + [out] + ([] if static else [ws]):
        ctx.free(b)
    return got


@pytest.mark.parametrize("name", ["tiny", "S"])
def test_static_scratch_layer_equals_the_workspace_layer(ctx, name):
    cfg = workload.tiny_config() if name == "tiny" else workload.config("S")
    weights = workload.LayerWeights(ctx, cfg, 55, ("normal", 0.5))
    assert ctx.lib.zc_hip_moe_static_scratch_bytes() == 4 << 20
    for T in (7, 3):                      # two calls in a row, the second smaller
        x = workload.hidden_rows(ctx, T, cfg.hidden, 560 + T)
        want = run(ctx, cfg, weights, x, T, static=False)
        allocated = ctx.allocated
        got = run(ctx, cfg, weights, x, T, static=True)
        assert ctx.allocated == allocated          # (the test's own buffers were freed again; the call added none)
        for k in want:
            assert got[k] == want[k], f"{name}, {T} tokens: {k} differs"
        ctx.free(x)
    # a call whose workspace does not fit the array is refused, with both sizes in the message
    big = 4096
    assert ctx.moe_workspace_bytes(cfg, big) > (4 << 20)
    x = ctx.zeros(big * cfg.hidden * 4); out = ctx.alloc(big * cfg.hidden * 4)
    with pytest.raises(z.ZcError) as err:
        ctx.moe_forward_static(cfg, weights.layer, x, big, out)
    assert "bytes of scratch" in str(err.value) and str(4 << 20) in str(err.value)
    for b in (x, out, weights.router, weights.shared_gate, weights.shared_record, weights.records):
        ctx.free(b)


def _free_bytes():
    """Free device memory as the HIP runtime reports it (hipMemGetInfo of the runtime this process has loaded)."""
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(0), C.c_size_t(0)
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_static_scratch_layer_allocates_nothing_while_a_recording_is_on(ctx):
    # With per-operator timing recorded (zc_hip_profile) every ordinary operator call creates two events and a row.  The
    # allocation-free entry point must not: no row, no change in the library's own count, none in the runtime's free memory.
    cfg = workload.tiny_config()
    weights = workload.LayerWeights(ctx, cfg, 57, ("normal", 0.5))
    T = 5
    x = workload.hidden_rows(ctx, T, cfg.hidden, 571)
    out, want = ctx.alloc(T * cfg.hidden * 4), ctx.alloc(T * cfg.hidden * 4)
    ws = ctx.alloc(ctx.moe_workspace_bytes(cfg, T))
    ctx.moe_forward_static(cfg, weights.layer, x, T, out); ctx.moe_check()     # first use of every kernel is behind us
    ctx.profile(True)
    try:
        ctx.moe_forward(cfg, weights.layer, x, T, want, ws); ctx.moe_check()
        rows = len(ctx.stats()["profile"]["rows"])
        assert rows >= 1
        allocated, free = ctx.allocated, _free_bytes()
        for _ in range(3):
            ctx.moe_forward_static(cfg, weights.layer, x, T, out)
        ctx.moe_check()
        assert ctx.allocated == allocated and _free_bytes() == free
        stats = ctx.stats()["profile"]
        assert len(stats["rows"]) == rows and all(r["operator"] != "moe_forward_static" for r in stats["rows"])
        ctx.moe_forward(cfg, weights.layer, x, T, want, ws); ctx.moe_check()   # the recording itself still works afterwards
        assert len(ctx.stats()["profile"]["rows"]) == rows + 1
    finally:
        ctx.profile(False)
    assert out.numpy(np.uint8).tobytes() == want.numpy(np.uint8).tobytes()
    for b in (x, out, want, ws, weights.router, weights.shared_gate, weights.shared_record, weights.records):
        ctx.free(b)
