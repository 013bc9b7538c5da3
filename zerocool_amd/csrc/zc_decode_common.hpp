// Pieces shared by the persistent decode kernels (one token: zc_decode.hip; two to eight tokens: zc_decode_multi.hip):
// coherent loads and stores, the flag barrier between workgroups, staging of exchanged rows into LDS, and the
// top-k + softmax of one token by one wavefront.
#pragma once
#include "zc_kernels.hpp"
#include "zc_xint.hpp"

namespace zc {

#define ZC_LD(p) __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define ZC_ST(p, v) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)

// A value every lane holds alike (read from LDS), moved to a scalar register so that control flow on it is scalar.
__device__ __forceinline__ int32_t uniform(int32_t v) { return __builtin_amdgcn_readfirstlane(v); }
// Where expert e's record is: in the layer's own array, or wherever the expert store's table says (an HBM slot, or the
// record's home in pinned host memory).  e is the same in every lane, so the table word comes through a scalar load.
__device__ __forceinline__ const uint8_t* record_of(const DecodeLayer& L, uint32_t e) {
    return L.table ? L.table[e] : L.records + uint64_t(e) * L.stride;
}
// Workgroup barrier that orders LDS traffic only: __syncthreads() also waits for every global load in flight, which would
// end a prefetch early.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ void st_f32(float* p, float v) { ZC_ST(reinterpret_cast<uint32_t*>(p), __float_as_uint(v)); }
__device__ __forceinline__ void st_i32(int32_t* p, int32_t v) { ZC_ST(reinterpret_cast<uint32_t*>(p), uint32_t(v)); }

// Workgroup size: single-token decode runs two waves per SIMD (the tile engine then fits 256 registers), several
// tokens keep one wave per SIMD and the whole register file.
constexpr uint32_t decode_threads(int nt) { return nt == 1 ? 512u : 256u; }
constexpr uint32_t kFlagStride = 32, kReleaseBase = 32 * 1024, kReleaseStride = 64, kAbortWord = kReleaseBase + 8 * kReleaseStride;

// Literal affine Q8 rows (reference: qwen.metal:112-125) against NTOK input rows held in LDS as BF16 (the tokens of one tile
// pass: a row's codes are fetched once and serve all of them).  Each 32-lane half of the wave plays the reference's 32 lanes
// for one output row at a time: lane l takes the eight-element blocks l, l + 32, ... (K is a multiple of 512 here, so the lane
// width is eight and a row of codes is K bytes); per block the plain fp32 sum of the inputs and the multiply-add chain of
// inputs times codes, result += scale * dot + sum * bias, then the xor butterfly.  `codes`, `scales`, `biases` are per-lane
// bases (the two halves may read different matrices); row_of(i) is the half's i-th row, emit(i, t, value) runs in every lane
// with that row's value for token t.  ROWS rows per half are fetched together, CH blocks each.
template <int CH, int ROWS, int NTOK, class RowOf, class Emit>
__device__ __forceinline__ void q8_rows_chunked(const uint8_t* codes, const uint16_t* scales, const uint16_t* biases, uint32_t K,
                                                const uint16_t* const* x, uint32_t rows, RowOf row_of, Emit emit) {
    const uint32_t l32 = threadIdx.x & 31u, per = K / 256u, groups = K / 64u;
    for (uint32_t i0 = 0; i0 < rows; i0 += ROWS) {
        float result[NTOK][ROWS];
#pragma unroll
        for (int t = 0; t < NTOK; ++t)
#pragma unroll
            for (int r = 0; r < ROWS; ++r) result[t][r] = 0.0f;
        for (uint32_t j0 = 0; j0 < per; j0 += CH) {
            uint2 q[ROWS][CH]; uint16_t sb[ROWS][CH], bb[ROWS][CH];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const uint32_t row = row_of(min(i0 + r, rows - 1));
#pragma unroll
                for (int c = 0; c < CH; ++c) {
                    const uint32_t b = l32 + 32u * (j0 + c);
                    q[r][c] = *reinterpret_cast<const uint2*>(codes + uint64_t(row) * K + b * 8u);
                    sb[r][c] = scales[uint64_t(row) * groups + b / 8u]; bb[r][c] = biases[uint64_t(row) * groups + b / 8u];
                }
            }
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                const uint32_t b = l32 + 32u * (j0 + c);
#pragma unroll
                for (int t = 0; t < NTOK; ++t) {
                    const uint4 raw = *reinterpret_cast<const uint4*>(x[t] + b * 8u);
                    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
                    float xb[8];
#pragma unroll
                    for (int e = 0; e < 4; ++e) { xb[2 * e] = __uint_as_float(w[e] << 16); xb[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u); }
                    float sum = 0;
#pragma unroll
                    for (int e = 0; e < 8; ++e) sum += xb[e];
#pragma unroll
                    for (int r = 0; r < ROWS; ++r) {
                        const uint32_t words[2] = {q[r][c].x, q[r][c].y};
                        float dot = 0;
#pragma unroll
                        for (int e = 0; e < 8; ++e) dot += xb[e] * float((words[e / 4] >> (8 * (e % 4))) & 255u);
                        result[t][r] += b16(sb[r][c]) * dot + sum * b16(bb[r][c]);
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < ROWS; ++r)
#pragma unroll
            for (int t = 0; t < NTOK; ++t) {
                const float v = lane_sum32(result[t][r]);
                if (i0 + r < rows) emit(i0 + r, t, v);
            }
    }
}
// One token.  DEEP: four rows per half in flight (short rows: the down projection); otherwise two.
template <bool DEEP, class RowOf, class Emit>
__device__ __forceinline__ void q8_rows(const uint8_t* codes, const uint16_t* scales, const uint16_t* biases, uint32_t K,
                                        const uint16_t* x, uint32_t rows, RowOf row_of, Emit emit) {
    const uint16_t* const rows_in[1] = {x};
    auto emit_one = [&](uint32_t i, int, float v) { emit(i, v); };
    if constexpr (DEEP) q8_rows_chunked<2, 4, 1>(codes, scales, biases, K, rows_in, rows, row_of, emit_one);
    else q8_rows_chunked<2, 2, 1>(codes, scales, biases, K, rows_in, rows, row_of, emit_one);
}

struct Barrier {
    uint32_t* mem; uint32_t epoch, spin_limit; int32_t* status; uint32_t token;   // token: this launch's first epoch
    // Flags: every workgroup stores its epoch in its own 128-byte line and polls the lines of
    // all others.  No cache write-back or invalidate: the data that crosses is written with
    // write-through atomics, read with coherent loads, and each wave has drained its own stores
    // before the flag is stored.
    __device__ __forceinline__ void wait() {
        ++epoch;
        // Every wave waits until its own write-through stores have been acknowledged by the L2 (the point of
        // coherence between workgroups): a workgroup-scope fence alone does not wait for them, and the flag
        // below must not become visible before the data of ANY wave of this workgroup.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        uint32_t me = blockIdx.x, thread = threadIdx.x;
        asm volatile("" : "+s"(me));       // flag addresses are formed here, not kept in registers across the phases
        asm volatile("" : "+v"(thread));
        // every workgroup watches every flag itself (one flag per thread): one store-to-load hop instead of a collector's two
        if (thread == 0) ZC_ST(mem + kFlagStride * me, epoch);
        for (uint32_t w = thread; w < gridDim.x; w += blockDim.x)
            if (w != me) spin(mem + kFlagStride * w);
        __syncthreads();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    }
    // One token: data crosses between workgroups with a tag beside every value and readers poll the data itself (until()).
    // The flag then only says "this workgroup has read everything the others wrote for this layer": it is stored without
    // waiting for anything, and checked before the next layer's first write to those buffers.
    __device__ __forceinline__ void arrive() {
        ++epoch;
        uint32_t me = blockIdx.x, thread = threadIdx.x;
        asm volatile("" : "+s"(me));
        asm volatile("" : "+v"(thread));
        if (thread == 0) ZC_ST(mem + kFlagStride * me, epoch);
    }
    // Repeats attempt() until it succeeds, bounded like spin().
    template <class Attempt>
    __device__ __forceinline__ void until(Attempt attempt) {
        for (uint32_t i = 0; !attempt(); ++i) {
            if ((i & 31u) == 31u && ZC_LD(mem + kAbortWord) == token) return;
            if (i >= spin_limit) { ZC_ST(mem + kAbortWord, token); atomicOr(status, 2); return; }
        }
    }
    // Bounded: a grid that is not fully resident must not hang the GPU.  Epochs only grow,
    // so "reached" is a signed comparison that survives wrap-around.
    __device__ __forceinline__ void spin(uint32_t* word) {
        for (uint32_t i = 0; int32_t(ZC_LD(word) - epoch) < 0; ++i) {
            if ((i & 255u) == 255u && ZC_LD(mem + kAbortWord) == token) return;   // someone gave up in this launch
            if (i >= spin_limit) { ZC_ST(mem + kAbortWord, token); atomicOr(status, 2); return; }
        }
    }
};

// Copies `pairs` pairs of fp32 values written by other workgroups into LDS as BF16 (high
// halves), DEPTH coherent 8-byte loads in flight per thread; returns whether any value
// had low mantissa bits.  transform(pair index, a, b) may rescale the two values first;
// ready() runs once, after the first loads have been issued and before any value is used.
template <int DEPTH = 8, class Ready, class Transform>
__device__ __forceinline__ int stage_bf16(const float* src, uint32_t pairs, uint32_t* dst, Ready ready, Transform transform) {
    int inexact = 0;
    for (uint32_t base = 0; base < pairs; base += blockDim.x * DEPTH) {
        uint64_t v[DEPTH];
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            const uint32_t i = base + u * blockDim.x + threadIdx.x;
            v[u] = i < pairs ? __hip_atomic_load(reinterpret_cast<const uint64_t*>(src) + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
        }
        if (base == 0) ready();
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            const uint32_t i = base + u * blockDim.x + threadIdx.x;
            if (i < pairs) {
                float a = __uint_as_float(uint32_t(v[u])), b = __uint_as_float(uint32_t(v[u] >> 32));
                transform(i, a, b);
                const uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b);
                inexact |= ((ua | ub) & 0xffffu) != 0;
                dst[i] = (ua >> 16) | (ub & 0xffff0000u);
            }
        }
    }
    return inexact;
}
// Copies `count` 8-byte words written by other workgroups into LDS, DEPTH coherent loads in flight per thread.
template <int DEPTH>
__device__ __forceinline__ void stage_copy(const uint64_t* src, uint32_t count, uint64_t* dst) {
    for (uint32_t base = 0; base < count; base += blockDim.x * DEPTH) {
        uint64_t v[DEPTH];
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            const uint32_t i = base + u * blockDim.x + threadIdx.x;
            v[u] = i < count ? __hip_atomic_load(src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
        }
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            const uint32_t i = base + u * blockDim.x + threadIdx.x;
            if (i < count) dst[i] = v[u];
        }
    }
}

// Top-k of one token by one wavefront.  Lane l holds experts l*per .. l*per+per-1, so the
// lowest lane holding the maximum, then the lowest slot inside it, is the lowest expert id:
// one DPP maximum, one ballot and two scalar-lane reads per pick.
//
// With eight candidates per lane (512 experts) a faster way comes first.  The k-th largest of the 64 lane maxima is
// found by a binary search over the bits of an order-preserving integer key (one compare and one ballot per step,
// stopping as soon as exactly k lanes remain); k elements are then known to be at least that large, so the final top-k
// lies among the elements at or above it: usually k to 2k of them.  They are gathered in ascending id order (`scratch`,
// 128 words of LDS owned by this wave), one per lane, and each counts the candidates that beat it (larger value, or
// equal value and lower id): that count is its slot.  More than 64 candidates (masses of equal logits) or fewer than k
// valid lanes take the picks one by one.
//
// fetch(cand, per) fills the lane's logits (-inf where it has no expert); ready() runs once the ids are final, before the
// softmax weights are formed.
template <int PER, class Fetch, class Clock, class Ready>
__device__ __forceinline__ void route_token(Fetch fetch, uint32_t E, uint32_t topk, uint32_t lane,
                                            int32_t* ids, float* weights, uint32_t* scratch, Clock clock, Ready ready) {
    const uint32_t per = PER == 16 ? (E + 63) / 64 : uint32_t(PER);
    const float ninf = __uint_as_float(0xff800000u);
    float cand[PER];
    fetch(cand, per);
#pragma unroll
    for (int i = 0; i < PER; ++i) cand[i] = cand[i] > ninf ? cand[i] : ninf;   // NaN and -inf never win
    float score = ninf, top = ninf;   // lane j keeps score j
    if (__ballot(cand[0] == 12345.678f) == ~0ull) return;   // (forces the loads to complete before the stamp)
    clock();
    bool done = false;
    if constexpr (PER == 8) {
        constexpr uint32_t kLowest = 0x007fffffu;   // key of -inf: nothing valid is at or below it
        uint32_t key[PER], best = 0;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            uint32_t u = __float_as_uint(cand[i]);
            if (u == 0x80000000u) u = 0;             // the two zeros compare equal
            key[i] = u ^ ((u >> 31) ? 0xffffffffu : 0x80000000u);
            best = max(best, key[i]);
        }
        if (uint32_t(__popcll(__ballot(best > kLowest))) >= topk && topk < 64) {
            uint32_t bar = 0;
            for (int b = 31; b >= 0; --b) {
                const uint32_t trial = bar | (1u << b), lanes = uint32_t(__popcll(__ballot(best >= trial)));
                if (lanes >= topk) { bar = trial; if (lanes == topk) break; }
            }
            // candidates in ascending id order: lower lanes first, then the lane's own slots
            const uint64_t below = (1ull << lane) - 1;
            uint32_t before = 0, count = 0;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                const uint64_t m = __ballot(key[i] >= bar);
                before += uint32_t(__popcll(m & below)); count += uint32_t(__popcll(m));
            }
            if (count <= 64) {
                uint32_t mine = 0;
#pragma unroll
                for (int i = 0; i < PER; ++i)
                    if (key[i] >= bar) { scratch[before + mine] = key[i]; scratch[64 + before + mine] = lane * per + uint32_t(i); ++mine; }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const uint32_t k_mine = lane < count ? scratch[lane] : 0u, id_mine = lane < count ? scratch[64 + lane] : 0u;
                // a candidate's slot is the number of candidates that beat it; as one 64-bit compare: the key above the
                // inverted position (lanes from `count` on hold key 0, which beats nothing)
                const uint64_t wide_mine = (uint64_t(k_mine) << 32) | (63u - lane);
                uint32_t rank = 0;
                for (uint32_t j = 0; j < count; j += 4)   // count <= 64, so lane j + 3 exists
#pragma unroll
                    for (uint32_t u = 0; u < 4; ++u) {
                        const uint64_t other = (uint64_t(uint32_t(__builtin_amdgcn_readlane(int(k_mine), int(j + u)))) << 32) | (63u - (j + u));
                        rank += other > wide_mine ? 1u : 0u;
                    }
                if (lane < count && rank < topk) {   // the slots are a permutation of 0 .. count-1: one owner each
                    ids[rank] = int32_t(id_mine);
                    weights[rank] = __uint_as_float(k_mine ^ ((k_mine >> 31) ? 0x80000000u : 0xffffffffu));   // the value back from its key
                }
                done = true;
            }
        }
    }
    if (!done)
    for (uint32_t j = 0; j < topk; ++j) {
        float best = cand[0];
#pragma unroll
        for (int i = 1; i < PER; ++i) if (uint32_t(i) < per) best = fmaxf(best, cand[i]);
        const float m = wave_max_f32(best);
        const uint64_t holders = __ballot(best == m && m > ninf);
        const bool found = holders != 0;
        const uint32_t owner = found ? uint32_t(__ffsll((long long)holders) - 1) : 0u;
        int first = PER;
#pragma unroll
        for (int i = PER - 1; i >= 0; --i) if (uint32_t(i) < per && cand[i] == m) first = i;
        float value = ninf;   // the winner's original bits (signed zero included)
#pragma unroll
        for (int i = 0; i < PER; ++i) if (i == first) value = cand[i];
        const uint32_t winner = uint32_t(__builtin_amdgcn_readlane(int(lane * per + uint32_t(first)), int(owner)));
        value = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, value), int(owner)));
        if (!found) value = ninf;
#pragma unroll
        for (int i = 0; i < PER; ++i) if (found && lane == owner && i == first) cand[i] = ninf;
        if (lane == j) score = value;
        if (j == 0) top = value;
        if (lane == 0) ids[j] = found ? int32_t(winner) : -1;
    }
    ready();
    clock();
    if (done) {   // the scores as the picks above would have left them
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (lane < topk) score = weights[lane];
        top = weights[0];
    }
    // softmax over the selected: reference lane l sums values 4l..4l+3 (qwen.metal:758-764)
    const float v = lane < topk ? exp32(score - top) : 0.0f;
    float s4 = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float other = __shfl(v, (4 * lane + i) & 63u);
        s4 += (4 * lane + i < 64) ? other : 0.0f;
    }
    const float inverse = 1.0f / __shfl(lane_sum32(s4), 0);
    if (lane < topk) weights[lane] = v * inverse;
}

// The same for up to N rows that lie apart (rows[t], t < count; `words` 8-byte words each) into consecutive LDS rows
// of `words` words: the loads of all rows are in flight together, so an entry's rows cost one latency, not one each.
template <int N>
__device__ __forceinline__ void stage_copy_rows(const uint64_t* const (&rows)[N], int count, uint32_t words, uint64_t* dst) {
    for (uint32_t j = threadIdx.x; j < words; j += blockDim.x) {
        uint64_t v[N];
#pragma unroll
        for (int t = 0; t < N; ++t) v[t] = t < count ? __hip_atomic_load(rows[t] + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
#pragma unroll
        for (int t = 0; t < N; ++t)
            if (t < count) dst[uint32_t(t) * words + j] = v[t];
    }
}
// Rows of fp32 values that lie apart (rows[t], t < count; `pairs` pairs of values each) as BF16 into consecutive LDS
// rows of `pairs` dwords, all rows' loads in flight together; transform(t, a, b) may rescale a pair of row t first.
// Returns nonzero if any value had low mantissa bits (see stage_bf16).
template <int N, class Transform>
__device__ __forceinline__ int stage_bf16_rows(const float* const (&rows)[N], int count, uint32_t pairs, uint32_t* dst, Transform transform) {
    int inexact = 0;
    for (uint32_t j = threadIdx.x; j < pairs; j += blockDim.x) {
        uint64_t v[N];
#pragma unroll
        for (int t = 0; t < N; ++t)
            v[t] = t < count ? __hip_atomic_load(reinterpret_cast<const uint64_t*>(rows[t]) + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
#pragma unroll
        for (int t = 0; t < N; ++t)
            if (t < count) {
                float a = __uint_as_float(uint32_t(v[t])), b = __uint_as_float(uint32_t(v[t] >> 32));
                transform(t, a, b);
                const uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b);
                inexact |= ((ua | ub) & 0xffffu) != 0;
                dst[uint32_t(t) * pairs + j] = (ua >> 16) | (ub & 0xffff0000u);
            }
    }
    return inexact;
}

// Workgroup wg's share [i0, i1) of a list of `total` items, cut at multiples of `waves` items.  Every entry of the tile
// lists is a multiple of eight items long (a tile count times a pass count), so with the cuts on such multiples neither a
// workgroup's range nor its part of any entry ends in a round in which some of its waves have no item.
__device__ __forceinline__ void share_of_items(uint32_t wg, uint32_t nwg, uint32_t total, uint32_t waves, uint32_t& i0, uint32_t& i1) {
    const uint32_t rounds = total / waves;
    i0 = uint32_t(uint64_t(wg) * rounds / nwg) * waves;
    i1 = wg + 1 == nwg ? total : uint32_t(uint64_t(wg + 1) * rounds / nwg) * waves;
}

// Which pass of its tile item q of an entry is (tile = q / passes).  The waves of a workgroup take every waves-th item, so
// with a pass count that divides the wave count a wave would meet the same pass -- the same tokens -- in all its items, and
// the wave that holds a token with many unsafe blocks would do all of that token's literal chains while the others wait
// for it at the end of the phase; the pass index is therefore rotated from tile to tile.
__device__ __forceinline__ uint32_t pass_of_item(uint32_t q, uint32_t passes, uint32_t waves) {
    const uint32_t tile = q / passes, base = q % passes;
    if (passes == 1 || waves % passes != 0) return base;
    return (base + tile / (waves / passes)) % passes;
}

}  // namespace zc
