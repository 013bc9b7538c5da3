"""Host (numpy) statement of the counter-based synthetic-tensor generator that the
HIP library runs on the device (zc_hip_synth_*): element i of a stream depends only on
(seed, i), so any tensor can be regenerated anywhere without storing it."""
import numpy as np

_M1, _M2, _G = np.uint64(0xBF58476D1CE4E5B9), np.uint64(0x94D049BB133111EB), np.uint64(0x9E3779B97F4A7C15)


def mix64(z):
    z = np.asarray(z, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def hash64(seed, i):
    with np.errstate(over="ignore"):
        base = mix64(np.uint64(seed) ^ np.uint64(0x5EEDC0DE5EEDC0DE))
        return mix64(base + (np.asarray(i, dtype=np.uint64) + np.uint64(1)) * _G)


def bf(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    return ((u + np.uint32(0x7fff) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xffff0000)).view(np.float32)


def bf_bits(x):
    return (bf(x).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def words(count, seed):
    i = np.arange(count, dtype=np.uint64)
    h = hash64(seed, i >> np.uint64(1))
    return np.where(i & np.uint64(1), h >> np.uint64(32), h & np.uint64(0xffffffff)).astype(np.uint32)


def scales(count, seed, lo, span, factor):
    u = (hash64(seed, np.arange(count, dtype=np.uint64)) >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
    sc = bf(np.float32(lo) + np.float32(span) * u)
    return bf_bits(sc), bf_bits(sc * np.float32(factor))


def normal(count, seed, sigma=1.0):
    """Irwin-Hall(12) on 16-bit fields of three hashes; BF16-valued fp32."""
    i = np.arange(count, dtype=np.uint64)
    total = np.zeros(count, np.int64)
    for j in range(3):
        h = hash64(seed, np.uint64(3) * i + np.uint64(j))
        for shift in (0, 16, 32, 48):
            total += ((h >> np.uint64(shift)) & np.uint64(0xffff)).astype(np.int64)
    z = (2 * total - 12 * 65535).astype(np.float32) * np.float32(2.0 ** -17)
    return bf(z * np.float32(sigma))


def zipf_offsets(experts, seed, s=1.1):
    """Per-expert logit offsets ln(pmf(rank)) - mean for a Zipf(s) law over a seeded
    permutation of ranks (the stacked-decode workload's load skew)."""
    order = np.argsort(hash64(seed, np.arange(experts, dtype=np.uint64)), kind="stable")
    rank = np.empty(experts, np.int64); rank[order] = np.arange(1, experts + 1)
    logp = -s * np.log(rank.astype(np.float64))
    return (logp - logp.mean()).astype(np.float32)


def normal_offsets(experts, seed, sigma=0.5):
    z = normal(experts, seed).astype(np.float64) * sigma
    return z.astype(np.float32)
