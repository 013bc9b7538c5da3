// Persistent decode kernel for ONE token: a whole stack of MoE layers in ONE launch (two to eight tokens:
// zc_decode_multi.hip; nine to sixty-four: zc_decode_wide.hip).
//
// One workgroup per compute unit stays resident for all layers.  A layer is three phases:
//   R  router logits (16-split chains), shared-expert gate dot
//   G  every workgroup routes (top-k + softmax) for itself, then the gate/up tiles (routed and shared)
//   D  routed + shared down tiles; a workgroup owns 16 output rows for ALL experts, so
//      the weighted combine (moe_sum) runs inside it without another exchange
// Arithmetic is the exact-integer matrix-core form (zc_xint.hpp) and the literal router /
// route / combine expressions, so every value equals the operator kernels bit for bit.
//
// Cross-workgroup data (logits, activations, layer outputs) is written and read ONLY with
// agent-scope relaxed atomics, which write through to / read from device-coherent
// memory; no cache write-back or invalidate is needed, only wait counters.
// Weights are read with ordinary cached loads: nothing writes them.
//
// There is no grid barrier on the path: every exchanged value carries a tag (a 16-bit number that advances with every layer of every launch) and its
// reader polls the data itself until the tag is the expected one (Barrier::until); one flag per workgroup and layer,
// stored without waiting and checked a layer later (Barrier::arrive), keeps a buffer from being overwritten before
// every workgroup has read it.  Inside a workgroup, waves hand work on through flag words in LDS where a workgroup
// barrier would make waves wait that have other work.
//
// Between layers the stacked-decode workload applies a stand-in glue (not reference
// arithmetic): x_next = bf(y * (1 / max|y|)) per token, order independent.
#include "zc_decode_common.hpp"

namespace zc {

constexpr int kRing = 8;         // sixteen-byte pieces of a router partition in flight per lane; tiles keep eight 128-element spans
                                 // in flight with one wave per SIMD and four with two

// MIXED: the down projection and/or the shared expert are affine Q8 and run on literal lanes; that variant leaves out the
// wave-local down phase (whose tile engine is the largest single piece of the kernel), so that both variants fit the
// register file without scratch memory and the all-Q4 variant is exactly what it was.
template <bool MIXED>
__global__ __launch_bounds__(decode_threads(1)) void decode_stack_kernel(DecodeParams p, DecodeLdsPlan lp) {
    constexpr int PT = 1;   // tokens per tile pass
    constexpr uint32_t kDecodeThreads = decode_threads(1), kDecodeWaves = kDecodeThreads / 64;
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, col = lane & 15u, G = lane >> 4;
    const uint32_t wg = blockIdx.x, nwg = gridDim.x;
    const uint32_t H = p.H, E = p.E, I = p.I, k = p.topk, T = p.T, n = T * k;
    int32_t* ids = reinterpret_cast<int32_t*>(lds + lp.ids);
    float* weights = reinterpret_cast<float*>(lds + lp.weights);
    float* gatev = reinterpret_cast<float*>(lds + lp.gatev);
    int32_t* experts = reinterpret_cast<int32_t*>(lds + lp.experts);
    int32_t* misc = reinterpret_cast<int32_t*>(lds + lp.misc);   // [1..8] wave maxima, [10..14] hand-off and ready words
    const uint16_t* xh_all = reinterpret_cast<const uint16_t*>(lds + lp.xh);
    const XintLayout LH{H}, LI{I};
    Barrier bar{p.sync, p.epoch, p.spin_limit, p.status, p.epoch};
    constexpr uint32_t kStamps = kDecodeStamps;   // slots per layer; this kernel fills 0..14, from the first thread of the workgroup
    // stamps of every workgroup: clocks[(layer * kStamps + stamp index) * workgroups + workgroup]
    uint32_t stamp_layer = 0;
    auto clock = [&](uint32_t i) { if (p.clocks && tid == 0) p.clocks[uint64_t(stamp_layer * kStamps + i) * nwg + wg] = wall_clock64(); };
    auto clock_all = [&](uint32_t i) { if (p.clocks) __syncthreads(); clock(i); };   // after the slowest wave of the workgroup

    if (wg == 0) for (uint32_t i = tid; i < p.L * T; i += blockDim.x) ZC_ST(p.maxabs + i, 0u);
    if (tid == 0) { misc[10] = 0; misc[11] = 0; misc[12] = 0; misc[13] = 0; misc[14] = 0; }   // the router chain's hand-off word, the ids-ready word, the staging waves' image-ready words: no tag is 0
    for (uint32_t layer = 0; layer < p.L; ++layer) {
        const DecodeLayer L = p.layers[layer];
        // Per-lane addresses and predicates derived from the thread index are recomputed in every layer: hoisted out of
        // the layer loop they would stay live through all phases and spill.
        auto refresh = [&]() {
            asm volatile("" : "+v"(tid));
            lane = tid & 63u; wave = uint32_t(uniform(int32_t(tid >> 6))); col = lane & 15u; G = lane >> 4;
        };
        refresh();
        stamp_layer = layer; clock(0);
        // One token: the 16-bit tag of everything layer l exchanges, never 0 (the buffers start as zeros) and different
        // from the tags of the layers (and launches) just before it
        auto tag_of = [&](uint32_t l) { return (p.tag_base + l) % 65535u + 1u; };
        const uint32_t tag = tag_of(layer);
        auto st_logit = [&](uint32_t index, float v) { ZC_ST(p.tlogits + index, (uint64_t(tag) << 32) | __float_as_uint(v)); };
        // one token: the experts this layer picked at the previous step (null: no guess), and where every slot's activations are
        const int32_t* pred = p.pred_in ? p.pred_in + uint64_t(layer) * k : nullptr;
        int32_t* spec = reinterpret_cast<int32_t*>(lds + lp.spec);   // [k + 1] source rows, [k + 1] miss list, [1] misses
        // ---------------- phase R: input images, router, shared gate/up, shared gate ----------------
        __syncthreads();
        // One token: the wave's first router unit starts loading its weights while the input row is staged and its image
        // built (the weights do not depend on the input).
        const uint32_t first_unit = wg + nwg * wave;
        // One token with whole rings of router pieces (hidden a multiple of 1024) and a workgroup to spare per router unit:
        // unit u runs on workgroup u with its K partitions cut into segments of eight pieces, one segment per wave.  All
        // segments load at once; the chain value then passes from wave to wave through LDS, so the unit pays one load
        // latency instead of one per ring.  The shared gate dot goes to the next workgroup, all of whose threads form the
        // products before one half-wave adds them in the reference's order.
        const uint32_t router_pieces = H / 128, router_segments = router_pieces / kRing;
        const bool segmented = router_pieces % kRing == 0 && router_segments <= kDecodeWaves && (E + 3) / 4 < nwg;
        uint4 early[kRing];
#pragma unroll
        for (int i = 0; i < kRing; ++i) early[i] = make_uint4(0, 0, 0, 0);
        // One token, a workgroup that owns a router unit, guesses at hand: its guessed gate/up tiles go to the waves AFTER the
        // router's (the staging waves and the ones behind them), which start them as soon as the image is complete -- told
        // so through flag words in LDS, not by a workgroup barrier, for which the router's waves would have to finish their
        // chains first (a tile is then 2.6 us late, and the layer with it: the gate/up burst is what the routing waits for).
        const bool apart = !MIXED && pred != nullptr && segmented && wg < (E + 3) / 4 && 64 * router_segments + H / 16 <= kDecodeThreads &&
                           (k * (I / 8)) % nwg == 0 && (E + 3) / 4 + I / 8 <= nwg && kDecodeWaves - router_segments >= k * (I / 8) / nwg && (H / 16 + 63) / 64 <= 3;
        {
            // One token: thread b fetches the sixteen values of block b, applies the glue's scale, writes the BF16 copy and
            // builds the block's image pieces straight from registers; the shared gate row rides along.  After the first
            // layer the values are the previous layer's tagged words: the thread fetches them again until every tag is that
            // layer's, and the workgroup forms the glue's scale (the largest magnitude of the row) itself.
            uint16_t* xh = reinterpret_cast<uint16_t*>(lds + lp.xh);
            const bool glue = layer != 0;
            const uint64_t* row = glue ? reinterpret_cast<const uint64_t*>(p.tout + ((layer - 1) & 1u) * H) : reinterpret_cast<const uint64_t*>(p.x_in);
            const uint32_t want = tag_of(layer - 1);
            // A workgroup that owns a segmented router unit issues the same loads from every lane in the same order, with
            // clamped addresses where a lane has nothing to fetch: the wait for the input's values can then leave exactly the
            // later router loads in flight (a load under a branch forces a full wait), and its two barriers order LDS traffic
            // only.  The other workgroups have no router loads to keep in flight and fetch only what they need.
            const bool keep_in_flight = uniform(segmented && wg < (E + 3) / 4);
            // In such a workgroup the staging threads are the waves after the router's: those build the image while the router
            // waves already run their chains, which need the BF16 copy only.
            const bool side = keep_in_flight && 64 * router_segments + H / 16 <= kDecodeThreads;
            const uint32_t blk = side ? tid - 64 * router_segments : tid;   // the thread's block; wraps to "none" for the router's waves
            uint64_t v[8];
            uint4 gate_piece = make_uint4(0, 0, 0, 0);
            const uint32_t own = min(blk, H / 16 - 1);
            // the flag of workgroup `tid` (all have finished reading what the previous layer exchanged), checked below
            uint32_t seen = ZC_LD(p.sync + kFlagStride * min(tid, nwg - 1));
            auto stale = [&]() {
                uint32_t bad = 0;
#pragma unroll
                for (int w = 0; w < 8; ++w) bad |= ((uint32_t(v[w]) ^ want) | (uint32_t(v[w] >> 32) ^ want)) & 0xffffu;
                return bad != 0;
            };
            if (side) {
                // the router's waves request their weights and nothing else; the staging waves fetch the input and nothing
                // else (this workgroup never reads the shared gate row)
#pragma unroll
                for (int w = 0; w < 8; ++w) v[w] = 0;
                if (wave < router_segments) {
                    const uint32_t e = wg * 4 + lane / 16, split = lane % 16, P = H / 16;
                    const uint16_t* wr = L.router + uint64_t(e < E ? e : E - 1) * H + split * P;
#pragma unroll
                    for (int i = 0; i < kRing; ++i) early[i] = ldg_u4(wr, wave * kRing + i);
                } else if (blk < H / 16) {
                    // (the staging lanes side by side: word pair w * H/16 + blk, so that a load covers four whole cache lines --
                    // a lane fetching its own block's eight pairs touches thirty-two; the blocks are built from the BF16 copy)
#pragma unroll
                    for (int w = 0; w < 8; ++w) v[w] = ZC_LD(row + uint32_t(w) * (H / 16) + blk);
                }
            } else if (keep_in_flight) {
#pragma unroll
                for (int w = 0; w < 8; ++w) v[w] = ZC_LD(row + own * 8 + w);
                gate_piece = ldg_u4(L.shared_gate, min(tid, H / 8 - 1));
                asm volatile("" ::: "memory");   // the router loads stay behind the loads above
                const uint32_t first_piece = min(wave, router_segments - 1) * kRing;
                const uint32_t e = wg * 4 + lane / 16, split = lane % 16, P = H / 16;
                const uint16_t* wr = L.router + uint64_t(e < E ? e : E - 1) * H + split * P;
#pragma unroll
                for (int i = 0; i < kRing; ++i) early[i] = ldg_u4(wr, first_piece + i);
            } else {
#pragma unroll
                for (int w = 0; w < 8; ++w) v[w] = 0;
                if (tid < H / 16) {
#pragma unroll
                    for (int w = 0; w < 8; ++w) v[w] = ZC_LD(row + tid * 8 + w);
                }
                if (tid < H / 8) gate_piece = ldg_u4(L.shared_gate, tid);
                if (!segmented && first_unit < (E + 3) / 4) {   // issued after the input's loads
                    const uint32_t e = first_unit * 4 + lane / 16, split = lane % 16, P = H / 16;
                    const uint16_t* wr = L.router + uint64_t(e < E ? e : E - 1) * H + split * P;
#pragma unroll
                    for (int i = 0; i < kRing; ++i) if (uint32_t(i) < P / 8) early[i] = ldg_u4(wr, i);
                }
            }
            if (glue) {
                if (blk < H / 16 && stale())
                    bar.until([&]() {
#pragma unroll
                        for (int w = 0; w < 8; ++w) v[w] = ZC_LD(row + (side ? uint32_t(w) * (H / 16) + own : own * 8 + uint32_t(w)));
                        return !stale();
                    });
                // every workgroup has taken what it needed from the buffers this layer is about to overwrite
                for (uint32_t w = tid; w < nwg; w += kDecodeThreads) {
                    if (w != tid) seen = ZC_LD(p.sync + kFlagStride * w);
                    if (int32_t(seen - bar.epoch) < 0) bar.spin(p.sync + kFlagStride * w);
                }
                // largest magnitude of the row (NaN takes no part): per wave here, across the waves after the barrier
                uint32_t m = 0;
                if (blk < H / 16) {
#pragma unroll
                    for (int w = 0; w < 8; ++w) {
                        const uint32_t a = uint32_t(v[w]) & 0x7fff0000u, c = uint32_t(v[w] >> 32) & 0x7fff0000u;
                        m = max(m, a > 0x7f800000u ? 0u : a); m = max(m, c > 0x7f800000u ? 0u : c);
                    }
                }
                m = __float_as_uint(wave_max_f32(__uint_as_float(m)));
                if (lane == 0) misc[1 + wave] = int32_t(m);
            }
            xint_prepare_begin(LH, lds + lp.img_rg, 1);
            if (keep_in_flight) lds_barrier(); else __syncthreads();
            if (blk < H / 16) {
                uint32_t peak = 0;
                if (glue) {
#pragma unroll
                    for (uint32_t w = 0; w < kDecodeWaves; ++w) peak = max(peak, uint32_t(misc[1 + w]));
                }
                const uint32_t keep = glue ? 0xffff0000u : 0xffffffffu;   // a tagged word keeps its tag in the low half
                const float m = __uint_as_float(peak), inv = (m > 0.0f && m < __uint_as_float(0x7f800000u)) ? 1.0f / m : 1.0f;
                RegF32 block; uint32_t low = 0, packed[8];
#pragma unroll
                for (int w = 0; w < 8; ++w) {
                    float a = __uint_as_float(uint32_t(v[w]) & keep), c = __uint_as_float(uint32_t(v[w] >> 32) & keep);
                    if (glue) { a = bf(a * inv); c = bf(c * inv); }
                    const uint32_t ua = __float_as_uint(a), uc = __float_as_uint(c);
                    low |= (ua | uc) & 0xffffu;
                    block.bits[2 * w] = ua & 0xffff0000u; block.bits[2 * w + 1] = uc & 0xffff0000u;
                    packed[w] = (ua >> 16) | (uc & 0xffff0000u);
                }
                if (low) atomicOr(p.status, 4);   // inputs must be BF16-valued
                if (side) {
#pragma unroll
                    for (int w = 0; w < 8; ++w) reinterpret_cast<uint32_t*>(xh)[uint32_t(w) * (H / 16) + blk] = packed[w];
                } else {
                    uint4* copy = reinterpret_cast<uint4*>(xh + blk * 16);
                    copy[0] = make_uint4(packed[0], packed[1], packed[2], packed[3]); copy[1] = make_uint4(packed[4], packed[5], packed[6], packed[7]);
                    xint_prepare_block(block, LH, lds + lp.img_rg, blk);
                }
            }
            if (tid < H / 8) reinterpret_cast<uint4*>(lds + lp.gatew)[tid] = gate_piece;
            lds_barrier();
            if (side && blk < H / 16) xint_prepare_block(LdsBf16{xh}, LH, lds + lp.img_rg, blk);   // from the BF16 copy, beside the router's waves; the tiles come after a barrier
            if (apart && wave >= router_segments && wave < router_segments + (H / 16 + 63) / 64) {   // this staging wave's part of the image is complete
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                if (lane == 0) __hip_atomic_store(misc + 12 + (wave - router_segments), int32_t(tag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        }
        clock(1);
        {
            // One token: the shared gate/up tiles run in phase G beside the routed ones, on waves that have no routed tile;
            // this phase then only has the router.
            const uint32_t router_units = (E + 3) / 4, gate_units = (T + 1) / 2;
            const uint32_t units = router_units + gate_units;
            if (segmented) {
                float* handoff = reinterpret_cast<float*>(lds + lp.gprod);   // 64 chain values; the products table belongs to another workgroup
                if (wg < router_units) {
                    const uint32_t e = wg * 4 + lane / 16, split = lane % 16, P = H / 16;
                    float c = 0;
                    // the chain value passes from one wave to the next through LDS with a flag word of its own: the other
                    // waves of the workgroup are busy with the image and do not come to a barrier here
                    if (wave < router_segments) {
                        const uint32_t seg = wave;
                        if (seg) {
                            for (uint32_t i = 0; uint32_t(__hip_atomic_load(misc + 10, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) != tag * 4 + seg && i < (1u << 22); ++i)
                                __builtin_amdgcn_s_sleep(1);
                            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                            c = handoff[lane];
                        }
                        uint4 xv[kRing];
#pragma unroll
                        for (int j = 0; j < kRing; ++j) xv[j] = *reinterpret_cast<const uint4*>(xh_all + split * P + (seg * kRing + j) * 8);
#pragma unroll
                        for (int j = 0; j < kRing; ++j) {
                            const uint32_t xw[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w}, ww[4] = {early[j].x, early[j].y, early[j].z, early[j].w};
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                c = __builtin_fmaf(__uint_as_float(xw[q] << 16), __uint_as_float(ww[q] << 16), c);
                                c = __builtin_fmaf(__uint_as_float(xw[q] & 0xffff0000u), __uint_as_float(ww[q] & 0xffff0000u), c);
                            }
                        }
                        if (seg + 1 < router_segments) {
                            handoff[lane] = c;
                            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                            if (lane == 0) __hip_atomic_store(misc + 10, int32_t(tag * 4 + seg + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        } else {
                            // partials added 0..15: after step s the lane of partition i <= s holds ((c0 + c1) + ..) + ci
                            const float offset = (L.offsets && e < E) ? ldg_f32(L.offsets, e) : 0.0f;
                            float sum = 0.0f + c;
#pragma unroll
                            for (int step = 1; step < 16; ++step) sum = dpp_row_shr1(sum) + c;
                            if (split == 15 && e < E) st_logit(e, L.offsets ? sum + offset : sum);
                        }
                    }
                } else if (wg == router_units) {
                    // shared_expert_gate (qwen.metal:499-506): reference lane l adds the products of k = l, l + 32, ... in turn
                    float* products = reinterpret_cast<float*>(lds + lp.gprod);     // [32 lanes][hidden / 32 + 1]
                    const uint16_t* gw = reinterpret_cast<const uint16_t*>(lds + lp.gatew);
                    const uint32_t pitch = H / 32 + 1;
                    for (uint32_t kk = tid; kk < H; kk += kDecodeThreads) products[(kk % 32) * pitch + kk / 32] = b16(xh_all[kk]) * b16(gw[kk]);
                    __syncthreads();
                    if (wave == 0) {
                        float sum = 0;
                        if (lane < 32) for (uint32_t j = 0; j < H / 32; ++j) sum += products[lane * pitch + j];
                        sum = lane_sum32(sum);
                        if (lane == 0) st_logit(E, bf(sum));
                    }
                }
            } else
            for (uint32_t u = wg + nwg * wave; u < units; u += nwg * kDecodeWaves) {
                if (u < router_units) {
                    // four experts x sixteen K partitions; k-ascending fused chain per partition
                    const uint32_t e = u * 4 + lane / 16, split = lane % 16, P = H / 16;
                    const uint16_t* wr = L.router + uint64_t(e < E ? e : E - 1) * H + split * P;
                    constexpr int kRouterRing = kRing;
                    const uint32_t pieces = P / 8;   // sixteen-byte pieces of the partition, kRing in flight
                    uint4 wv[kRouterRing];
                    if (u == first_unit) {
#pragma unroll
                        for (int i = 0; i < kRouterRing; ++i) wv[i] = early[i];
                    } else {
#pragma unroll
                        for (int i = 0; i < kRouterRing; ++i) if (uint32_t(i) < pieces) wv[i] = ldg_u4(wr, i);
                    }
                    float c = 0;
                    if (pieces % kRouterRing == 0) {
                        // one token, whole rings (hidden a multiple of 1024): straight-line bodies of eight pieces, the eight input
                        // pieces read from LDS together so that one wait covers them, the next ring requested before the chain runs
                        for (uint32_t i0 = 0; i0 < pieces; i0 += kRouterRing) {
                            uint4 xv[kRouterRing], wc[kRouterRing];
#pragma unroll
                            for (int j = 0; j < kRouterRing; ++j) { xv[j] = *reinterpret_cast<const uint4*>(xh_all + split * P + (i0 + j) * 8); wc[j] = wv[j]; }
                            if (i0 + kRouterRing < pieces) {
#pragma unroll
                                for (int j = 0; j < kRouterRing; ++j) wv[j] = ldg_u4(wr, i0 + kRouterRing + j);
                            }
#pragma unroll
                            for (int j = 0; j < kRouterRing; ++j) {
                                const uint32_t xw[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w}, ww[4] = {wc[j].x, wc[j].y, wc[j].z, wc[j].w};
#pragma unroll
                                for (int q = 0; q < 4; ++q) {
                                    c = __builtin_fmaf(__uint_as_float(xw[q] << 16), __uint_as_float(ww[q] << 16), c);
                                    c = __builtin_fmaf(__uint_as_float(xw[q] & 0xffff0000u), __uint_as_float(ww[q] & 0xffff0000u), c);
                                }
                            }
                        }
                    } else
                    for (uint32_t i0 = 0; i0 < pieces; i0 += kRouterRing) {
#pragma unroll
                        for (int j = 0; j < kRouterRing; ++j) {
                            const uint32_t i = i0 + j;
                            if (i < pieces) {
                                const uint32_t ww[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
                                if (i + kRouterRing < pieces) wv[j] = ldg_u4(wr, i + kRouterRing);
                                const uint4 xv = *reinterpret_cast<const uint4*>(xh_all + split * P + i * 8);
                                const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
                                for (int q = 0; q < 4; ++q) {
                                    c = __builtin_fmaf(__uint_as_float(xw[q] << 16), __uint_as_float(ww[q] << 16), c);
                                    c = __builtin_fmaf(__uint_as_float(xw[q] & 0xffff0000u), __uint_as_float(ww[q] & 0xffff0000u), c);
                                }
                            }
                        }
                    }
                    // partials added 0..15: after step s the lane of partition i <= s holds ((c0 + c1) + ..) + ci
                    const float offset = (L.offsets && e < E) ? ldg_f32(L.offsets, e) : 0.0f;
                    float sum = 0.0f + c;
#pragma unroll
                    for (int step = 1; step < 16; ++step) sum = dpp_row_shr1(sum) + c;
                    if (split == 15 && e < E) st_logit(e, L.offsets ? sum + offset : sum);
                } else {
                    // shared_expert_gate: reference lane chain k = lane + 32 j (qwen.metal:499-506); two tokens per wave
                    const uint32_t t = (u - router_units) * 2 + (lane >> 5), l32 = lane & 31u;
                    const uint16_t* gw = reinterpret_cast<const uint16_t*>(lds + lp.gatew);   // staged with the input rows
                    float sum = 0;
                    if (t < T)
                        for (uint32_t k0 = l32; k0 < H; k0 += 256) {   // eight LDS reads in flight per operand (hidden is a multiple of 512); the sum stays in k order
                            float a[8], g[8];
#pragma unroll
                            for (int j = 0; j < 8; ++j) { a[j] = b16(xh_all[t * H + k0 + 32 * j]); g[j] = b16(gw[k0 + 32 * j]); }
#pragma unroll
                            for (int j = 0; j < 8; ++j) sum += a[j] * g[j];
                        }
                    sum = lane_sum32(sum);
                    if (t < T && l32 == 0) st_logit(E, bf(sum));
                }
            }
        }
        if (apart) {
            clock(2);
            if (wave >= router_segments) {   // the tile waves: until every staging wave has said that its blocks are built
                const uint32_t staging = (H / 16 + 63) / 64;
                for (uint32_t i = 0; i < (1u << 22); ++i) {
                    bool ready = true;
                    for (uint32_t w = 0; w < staging; ++w) ready = ready && uint32_t(__hip_atomic_load(misc + 12 + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) == tag;
                    if (ready) break;
                    __builtin_amdgcn_s_sleep(1);
                }
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            }
        } else {
            clock_all(2);
            __syncthreads();   // the routing below polls the logits themselves
        }
        refresh();
        clock(3);
        // ---------------- phase G: route, group slots by expert, routed gate/up ----------------
        for (uint32_t t = wave; t < T; t += kDecodeWaves)
        {
            uint32_t route_stamp = 4; auto stamp = [&]() { if (t == 0) clock(route_stamp++); };
            // the previous step's ids of this layer, one per lane: requested now, compared when this step's ids are final
            const int32_t guess = (pred && lane < k) ? pred[lane] : -1;
            uint32_t* scratch = reinterpret_cast<uint32_t*>(experts) + 128 * wave;   // the selection's 128 words of scratch per wave
            // the lane's logits: written by other workgroups; one token polls the tagged words until all carry this layer's tag
            auto fetch = [&](auto& cand, uint32_t per) {
                constexpr int PER = int(sizeof(cand) / sizeof(float));
                const float ninf = __uint_as_float(0xff800000u);
                {
                    // polled with the lanes side by side (word i * 64 + lane: four whole cache lines per load; lane-major, as
                    // the selection wants its candidates, a load touched thirty-two), turned lane-major through LDS
                    uint64_t w[PER];
                    bar.until([&]() {
                        uint32_t bad = 0;
#pragma unroll
                        for (int i = 0; i < PER; ++i) {
                            const uint32_t e = uint32_t(i) * 64 + lane;
                            w[i] = e < E ? ZC_LD(p.tlogits + e) : (uint64_t(tag) << 32) | 0xff800000u;
                        }
#pragma unroll
                        for (int i = 0; i < PER; ++i) bad |= uint32_t(w[i] >> 32) ^ tag;
                        return __ballot(bad != 0) == 0;
                    });
                    float* turned = reinterpret_cast<float*>(experts);   // E words: the expert list is built later, the selection's scratch used after this
                    auto wave_order = [&]() {
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                        __builtin_amdgcn_wave_barrier();
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    };
#pragma unroll
                    for (int i = 0; i < PER; ++i) if (uint32_t(i) * 64 + lane < E) turned[uint32_t(i) * 64 + lane] = __uint_as_float(uint32_t(w[i]));
                    wave_order();
#pragma unroll
                    for (int i = 0; i < PER; ++i) cand[i] = (uint32_t(i) < per && lane * per + i < E) ? turned[lane * per + i] : ninf;
                    wave_order();
                }
            };
            // One token: the other waves wait for the ids only (a flag word in LDS), not for the softmax weights, which the
            // combine needs much later; the routing wave takes its tiles last.
            auto ready = [&]() {
                {
                    // Where every slot's gate/up activations come from: the row of the prediction pass that already ran the same
                    // expert (slot j' of the predicted list), or this layer's own row once the tiles below have run (-1: a miss).
                    // The misses form the tile list of the second pass; without a prediction every slot and the shared expert miss.
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // the ids were written by other lanes of this wave
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    const int32_t mine = lane < k ? ids[lane] : -1;
                    int32_t from = -1;
                    if (pred)
                        for (uint32_t j0 = 0; j0 < k; j0 += 4)   // (lanes from k on hold no guess: -1 matches nothing)
#pragma unroll
                            for (uint32_t j = j0; j < j0 + 4; ++j) { const int32_t pj = __builtin_amdgcn_readlane(guess, int(j & 63u)); if (pj == mine && mine >= 0) from = int32_t(j); }
                    const uint64_t missing = __ballot(lane < k && from < 0);
                    if (lane < k) {
                        spec[lane] = from;
                        if (from < 0) spec[(k + 1) + __popcll(missing & ((1ull << lane) - 1))] = int32_t(lane);
                    }
                    if (lane == 0) {
                        uint32_t misses = uint32_t(__popcll(missing));
                        spec[k] = pred ? int32_t(k) : -1;                        // the shared expert's row
                        if (!pred) spec[(k + 1) + misses++] = int32_t(k);
                        spec[2 * (k + 1)] = int32_t(misses);
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                    if (lane == 0) __hip_atomic_store(misc + 11, int32_t(tag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            };
            if (E == 512) route_token<8>(fetch, E, k, lane, ids + t * k, weights + t * k, scratch, stamp, ready);
            else route_token<16>(fetch, E, k, lane, ids + t * k, weights + t * k, scratch, stamp, ready);
        }
        {
            // (the waves other than the routing wave go straight to the prediction pass below and wait for the ids after it)
        }
        clock(6);
        if (tid < n) {
            const int32_t e = ids[tid];
            if (e < 0 || e >= int32_t(E)) atomicOr(p.status, 1);
            if (wg == 0 && p.ids_trace) { st_i32(p.ids_trace + uint64_t(layer) * p.trace_tokens * k + tid, e); st_f32(p.weights_trace + uint64_t(layer) * p.trace_tokens * k + tid, weights[tid]); }
            if (wg == 0 && p.pred_out) p.pred_out[uint64_t(layer) * k + tid] = e;   // the next step's guess for this layer
        }
        // (slot j belongs to expert ids[j] and no two slots share an expert, so there is nothing to group)
        clock(7);
        {
            // Two passes over gate/up tiles.  Pass 0 runs BEFORE the ids are known, on the seven waves that do not route: the
            // tiles of the experts this layer picked at the previous step (the reference predicts a layer's experts for its
            // prefetcher, model.cpp:438-445; here the guess buys the time of the router, the exchange of the logits and the
            // selection), and the shared expert's, which needs no ids at all; results go to the prediction buffer.  Pass 1
            // runs once the ids are final: the tiles of the slots whose expert was not predicted.  Both passes compute a slot
            // with the same arithmetic, so a guess can only cost time, never change a bit.
            const uint32_t tiles = I / 8;
            const bool q8_shared = MIXED && p.shared_bits_gate_up == 8;
            const uint32_t shared_cut = q8_shared ? 4u : 1u;   // pieces a shared gate/up tile is cut into in the first pass
            for (int pass = 0; pass < 2; ++pass) {
                uint32_t first, stride, units;
                bool far_end = false;
                if (pass == 0) {
                    // With whole rounds of routed tiles the shared tiles (one more round, not a full one) go to the workgroups counted
                    // from the far end: the near end owns the router units and comes to the tiles last.
                    if (!pred || wave == 0) continue;
                    far_end = !q8_shared && (k * tiles) % nwg == 0 && tiles <= nwg;
                    first = wg + nwg * (wave - 1); stride = nwg * (kDecodeWaves - 1);
                    if (apart) {   // (this workgroup has no shared tile: those go to the far end)
                        if (wave < router_segments) continue;
                        first = wg + nwg * (wave - router_segments);
                    }
                    units = far_end ? k * tiles + nwg : k * tiles + tiles * shared_cut;
                } else {
                    if (wave != 0) {
                        for (uint32_t i = 0; uint32_t(__hip_atomic_load(misc + 11, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)) != tag && i < (1u << 22); ++i)
                            __builtin_amdgcn_s_sleep(1);
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                    }
                    const uint32_t turn = (wave + kDecodeWaves - 1) % kDecodeWaves;   // the routing wave, still busy with the softmax, comes last
                    first = wg + nwg * turn; stride = nwg * kDecodeWaves; units = uint32_t(uniform(spec[2 * (k + 1)])) * tiles;
                }
                for (uint32_t u = first; u < units; u += stride) {
                    uint32_t slot = u / tiles, tile = u % tiles, piece = 0, pieces = shared_cut;
                    if (pass == 0 && q8_shared && u >= k * tiles) { slot = k; tile = (u - k * tiles) / shared_cut; piece = (u - k * tiles) % shared_cut; pieces = piece + 1; }
                    if (far_end && u >= k * tiles) {
                        const uint32_t s = nwg - 1 - wg;   // the shared tile of this workgroup, if it has one
                        if (s >= tiles) continue;
                        slot = k; tile = s;
                    }
                    if (pass == 1) slot = uint32_t(uniform(spec[(k + 1) + slot]));   // the miss list
                    const int32_t e = slot < k ? (pass == 0 ? uniform(pred[slot]) : uniform(ids[slot])) : 0;
                    if (e < 0 || e >= int32_t(E)) continue;   // no guess for the slot, or an id reported above (the combine drops the slot)
                    uint32_t* out_row = (pass == 0 ? p.tspec : p.tact) + uint64_t(slot) * I;
                    if (MIXED && slot == k && p.shared_bits_gate_up == 8) {
                        // the shared expert's gate/up rows as affine Q8: the lower half of the wave takes gate row tile * 8 + i,
                        // the upper half the up row of the same index
                        // (a row pair is several memory latencies long, so in the first pass a tile is cut into pieces of two
                        // row pairs that different waves take; the second pass, which sees the shared expert only when there was
                        // no guess at all, runs a tile's pieces one after the other)
                        const uint32_t side = lane >> 5, per_piece = 8 / shared_cut;
                        const uint8_t* rec = L.shared_record;
                        for (; piece < pieces; ++piece)
                            q8_rows<false>(rec + p.so[side * 3], reinterpret_cast<const uint16_t*>(rec + p.so[side * 3 + 1]),
                                    reinterpret_cast<const uint16_t*>(rec + p.so[side * 3 + 2]), H, xh_all, per_piece,
                                    [&](uint32_t i) { return tile * 8 + piece * per_piece + i; },
                                    [&](uint32_t i, float v) {
                                        const float up = __shfl(v, 32);
                                        if (lane == 0) ZC_ST(out_row + tile * 8 + piece * per_piece + i, (__float_as_uint(swiglu_bf(v, up)) & 0xffff0000u) | tag);
                                    });
                        continue;
                    }
                    const uint32_t row = tile * 8 + (col & 7u), pr = col < 8 ? 0 : 3;
                    const uint8_t* rec = slot < k ? record_of(L, e) : L.shared_record;
                    const uint64_t* off = slot < k ? p.ro : p.so;
                    const uint8_t* w_row = rec + off[pr] + uint64_t(row) * (H / 2);
                    const uint16_t* s_row = reinterpret_cast<const uint16_t*>(rec + off[pr + 1]) + uint64_t(row) * (H / 64);
                    const uint16_t* b_row = reinterpret_cast<const uint16_t*>(rec + off[pr + 2]) + uint64_t(row) * (H / 64);
                    const uint8_t* img[PT] = {lds + lp.img_rg}; LdsBf16 src[PT] = {LdsBf16{xh_all}};
                    // SwiGLU of the finished tile as tagged words, one per activation: row `slot` of the tagged buffer (row k: shared)
                    auto emit = [&](int, float v) {
                        const float up = __shfl(v, (lane & ~15u) | ((col & 7u) + 8u));
                        const uint32_t a = __float_as_uint(swiglu_bf(v, up));
                        if (lane < 8) ZC_ST(out_row + row, (a & 0xffff0000u) | tag);
                    };
                    xint_run_tile<PT, 4>(w_row, s_row, b_row, H / 128, img, src, LH, lane, 1, emit);
                }
            }
            if (tid == 64) {   // the combine's gate factor (written by another workgroup)
                uint64_t w = 0;
                bar.until([&]() { w = ZC_LD(p.tlogits + E); return uint32_t(w >> 32) == tag; });
                gatev[0] = bf(sigmoid_bf(__uint_as_float(uint32_t(w))));
            }
        }
        clock_all(8);
        __syncthreads();   // the staging below polls the activations themselves
        refresh();
        clock(9);
        // ---------------- phase D: down tiles per 16 output rows, combine ----------------
        float* otile = reinterpret_cast<float*>(lds + lp.otile);
        const uint32_t slots_total = n + T, SB = lp.slots_per_batch;
        if (wg >= H / 16) { clock(10); clock(11); clock(12); }   // workgroups without a row tile keep the stamp count
        { if (wg >= H / 16) bar.arrive(); }
        for (uint32_t rt = wg; rt < H / 16; rt += nwg) {
            const uint32_t row = rt * 16 + col;
            if (!MIXED && SB >= slots_total && I == 1024) {
                // One token, all slots' images resident, tiles of two bodies (intermediate 1024): every wave works alone.  It requests the first weights of its slot's
                // tile, then polls that slot's activations (one 16-element block per lane), builds the slot's image and the
                // BF16 copy under the latency of those loads, and runs the tile; no workgroup barrier until the combine, and
                // a wave starts as soon as its own slot is complete.
                __syncthreads();
                clock(10); clock(11);
                uint16_t* ah = reinterpret_cast<uint16_t*>(lds + lp.ah);
                for (uint32_t slot = wave; slot <= k; slot += kDecodeWaves) {   // slot k is the shared expert's
                    const uint8_t* rec = L.shared_record; const uint64_t* off = p.so;
                    // what the combine adds up: the slot's output times its softmax weight (a dropped slot: zero times it),
                    // the shared expert's output times the gate factor, rounded
                    const float factor = slot < k ? weights[slot] : gatev[0];
                    if (slot < k) {
                        const int32_t e = uniform(ids[slot]);
                        if (e < 0 || e >= int32_t(E)) { if (G == 0) otile[slot * 16 + col] = 0.0f * factor; continue; }
                        rec = record_of(L, e); off = p.ro;
                    }
                    const uint8_t* w_row = rec + off[6] + uint64_t(row) * (I / 2);
                    const uint16_t* s_row = reinterpret_cast<const uint16_t*>(rec + off[7]) + uint64_t(row) * (I / 64);
                    const uint16_t* b_row = reinterpret_cast<const uint16_t*>(rec + off[8]) + uint64_t(row) * (I / 64);
                    uint8_t* image = lds + lp.img_d + slot * LI.bytes();
                    uint16_t* copy_row = ah + slot * I;
                    auto wave_sync = [&]() {   // LDS traffic of this wave's lanes, in program order
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                        __builtin_amdgcn_wave_barrier();
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    };
                    // (the first poll goes out before the tile's weights are requested: loads come back in the order they were sent)
                    const int32_t from = uniform(spec[slot]);   // the prediction pass's row of the same expert, or this layer's own
                    const uint64_t* words = reinterpret_cast<const uint64_t*>(from >= 0 ? p.tspec + uint64_t(from) * I : p.tact + uint64_t(slot) * I) + lane;
                    uint64_t w[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) w[i] = ZC_LD(words + i * 64);
                    auto prologue = [&]() {
                        if (lane < LI.mask_bytes() / 4) reinterpret_cast<uint32_t*>(image + LI.planes_bytes() + LI.info_bytes())[lane] = 0;
                        if (lane < 4) reinterpret_cast<uint32_t*>(image + LI.blocks() * 48)[lane] = 0;
                        wave_sync();
                        {
                            // The slot's 1024 tagged words, polled with the lanes side by side (word pair i * 64 + lane: a load
                            // instruction covers four whole cache lines; with a lane fetching its own block of sixteen it
                            // touched sixty-four), packed into the BF16 copy in LDS, from which every lane then builds the image
                            // of one block.
                            bool again = false;
                            bar.until([&]() {
                                uint32_t bad = 0;
                                if (again) {
#pragma unroll
                                    for (int i = 0; i < 8; ++i) w[i] = ZC_LD(words + i * 64);
                                }
                                again = true;
#pragma unroll
                                for (int i = 0; i < 8; ++i) bad |= ((uint32_t(w[i]) ^ tag) | (uint32_t(w[i] >> 32) ^ tag)) & 0xffffu;
                                return __ballot(bad != 0) == 0;   // the whole row, for every lane
                            });
                            uint32_t* copy = reinterpret_cast<uint32_t*>(copy_row) + lane;
#pragma unroll
                            for (int i = 0; i < 8; ++i) copy[i * 64] = (uint32_t(w[i]) >> 16) | (uint32_t(w[i] >> 32) & 0xffff0000u);
                            wave_sync();
                            xint_prepare_block(LdsBf16{copy_row}, LI, image, lane);
                        }
                        wave_sync();
                    };
                    const uint8_t* img[PT] = {image}; LdsBf16 src[PT] = {LdsBf16{copy_row}};
                    auto emit = [&](int, float v) { if (G == 0) otile[slot * 16 + col] = slot < k ? bf(v) * factor : bf(factor * bf(v)); };
                    xint_run_tile_after<PT, 4, true>(w_row, s_row, b_row, I / 128, img, src, LI, lane, 1, emit, prologue);   // two bodies: both requested at once
                }
            } else
            for (uint32_t s0 = 0; s0 < slots_total; s0 += SB) {
                const uint32_t sn = min(SB, slots_total - s0);
                __syncthreads();
                uint16_t* ah = reinterpret_cast<uint16_t*>(lds + lp.ah);
                auto source_of = [&](uint32_t q) { return LdsBf16{ah + q * I}; };
                {
                    // One token: a thread fetches whole 16-element blocks of the activations (32 bytes) and builds their
                    // image pieces straight from registers; the BF16 copy for the literal chain is written on the way.
                    const uint32_t per = I / 16, total = sn * per;
                    constexpr int kMine = 2;
                    for (uint32_t base = 0; base < total; base += kDecodeThreads * kMine) {
                        uint64_t words[kMine][8];   // sixteen tagged words of a block; a slot without a valid expert stays zero
                        bool wanted[kMine];
#pragma unroll
                        for (int j = 0; j < kMine; ++j) {
                            const uint32_t blk = base + j * kDecodeThreads + tid;
#pragma unroll
                            for (int w = 0; w < 8; ++w) words[j][w] = 0;
                            wanted[j] = false;
                            if (blk < total) {
                                const uint32_t slot = s0 + blk / per;
                                const int32_t e = slot < k ? ids[slot] : 0;
                                wanted[j] = e >= 0 && e < int32_t(E);
                            }
                        }
                        bool prepared = false;
                        auto fetch = [&]() {
                            uint32_t bad = 0;
#pragma unroll
                            for (int j = 0; j < kMine; ++j) {
                                const uint32_t blk = base + j * kDecodeThreads + tid;
                                if (wanted[j]) {
                                    const uint32_t at_slot = s0 + blk / per;
                                    const int32_t from = spec[at_slot];
                                    const uint64_t* src = reinterpret_cast<const uint64_t*>((from >= 0 ? p.tspec + uint64_t(from) * I : p.tact + uint64_t(at_slot) * I) + (blk % per) * 16);
#pragma unroll
                                    for (int w = 0; w < 8; ++w) words[j][w] = ZC_LD(src + w);
                                }
                            }
                            if (base == 0 && !prepared) { xint_prepare_begin(LI, lds + lp.img_d, sn); prepared = true; }   // while the loads are in flight
#pragma unroll
                            for (int j = 0; j < kMine; ++j)
                                if (wanted[j]) {
#pragma unroll
                                    for (int w = 0; w < 8; ++w) bad |= ((uint32_t(words[j][w]) ^ tag) | (uint32_t(words[j][w] >> 32) ^ tag)) & 0xffffu;
                                }
                            return bad == 0;
                        };
                        bar.until(fetch);
                        if (base == 0) __syncthreads();
#pragma unroll
                        for (int j = 0; j < kMine; ++j) {
                            const uint32_t blk = base + j * kDecodeThreads + tid;
                            if (blk < total) {
                                const uint32_t q = blk / per, b = blk % per;
                                RegF32 piece;
                                uint32_t* copy = reinterpret_cast<uint32_t*>(ah + q * I + b * 16);
#pragma unroll
                                for (int w = 0; w < 8; ++w) {
                                    const uint32_t lo = uint32_t(words[j][w]) & 0xffff0000u, hi = uint32_t(words[j][w] >> 32) & 0xffff0000u;
                                    piece.bits[2 * w] = lo; piece.bits[2 * w + 1] = hi;
                                    copy[w] = (lo >> 16) | hi;
                                }
                                xint_prepare_block(piece, LI, lds + lp.img_d + q * LI.bytes(), b);
                            }
                        }
                    }
                    if (s0 == 0) { clock(10); clock(11); }
                    __syncthreads();
                    if (rt + nwg >= H / 16 && s0 + SB >= slots_total) bar.arrive();   // nothing more to read from other workgroups in this layer
                }
                {
                    for (uint32_t slot = wave; slot <= k; slot += kDecodeWaves) {   // slot k is the shared expert's
                        if (slot < s0 || slot >= s0 + sn) continue;
                        const uint8_t* rec = L.shared_record; const uint64_t* off = p.so;
                        if (slot < k) {
                            const int32_t e = uniform(ids[slot]);
                            if (e < 0 || e >= int32_t(E)) continue;
                            rec = record_of(L, e); off = p.ro;
                        }
                        if (MIXED && (slot < k ? p.bits_down : p.shared_bits_down) == 8) {   // affine Q8 down rows: row 2 i of the tile on the lower half of the wave, 2 i + 1 on the upper
                            q8_rows<true>(rec + off[6], reinterpret_cast<const uint16_t*>(rec + off[7]), reinterpret_cast<const uint16_t*>(rec + off[8]), I,
                                    ah + (slot - s0) * I, 8, [&](uint32_t i) { return rt * 16 + 2 * i + (lane >> 5); },
                                    [&](uint32_t i, float v) { if ((lane & 31u) == 0) otile[slot * 16 + 2 * i + (lane >> 5)] = bf(v); });
                            continue;
                        }
                        const uint8_t* w_row = rec + off[6] + uint64_t(row) * (I / 2);
                        const uint16_t* s_row = reinterpret_cast<const uint16_t*>(rec + off[7]) + uint64_t(row) * (I / 64);
                        const uint16_t* b_row = reinterpret_cast<const uint16_t*>(rec + off[8]) + uint64_t(row) * (I / 64);
                        const uint8_t* img[PT] = {lds + lp.img_d + (slot - s0) * LI.bytes()}; LdsBf16 src[PT] = {source_of(slot - s0)};
                        auto emit = [&](int, float v) { if (G == 0) otile[slot * 16 + col] = bf(v); };
                        xint_run_tile<PT, 4>(w_row, s_row, b_row, I / 128, img, src, LI, lane, 1, emit);
                    }
                }
            }
            __syncthreads();
            if (!MIXED && SB >= slots_total && I == 1024 && rt + nwg >= H / 16) bar.arrive();   // every wave has read its slots' activations
            clock(12);
            // weighted combine of the tile (reference: qwen.metal:804-816)
            if (tid < T * 16) {
                const uint32_t t = tid / 16, c = tid % 16;
                float partial[8];
#pragma unroll
                for (int q = 0; q < 8; ++q) partial[q] = 0;
                const bool products = !MIXED && SB >= slots_total && I == 1024;   // the waves left products, not outputs
                if (products) {
                    for (uint32_t base = 0; base < k; base += 8) {
                        float value[8];
#pragma unroll
                        for (int j = 0; j < 8; ++j) value[j] = otile[min(base + j, k - 1) * 16 + c];
#pragma unroll
                        for (int j = 0; j < 8; ++j) if (base + j < k) partial[j] = base == 0 ? value[j] : partial[j] + value[j];
                    }
                } else
                for (uint32_t base = 0; base < k; base += 8) {   // eight independent products at a time, partial j takes slots j, j+8, ...
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const uint32_t kk = base + j;
                        if (kk < k) {
                            const int32_t e = ids[t * k + kk];
                            const float value = (e >= 0 && e < int32_t(E)) ? otile[(t * k + kk) * 16 + c] : 0.0f;
                            const float product = value * weights[t * k + kk];
                            partial[j] = base == 0 ? product : partial[j] + product;
                        }
                    }
                }
                float sum = partial[0];
                for (uint32_t kk = 1; kk < 8 && kk < k; ++kk) sum += partial[kk];
                const float y = bf(bf(sum) + (products ? otile[n * 16 + c] : bf(gatev[t] * otile[(n + t) * 16 + c])));
                const uint64_t at = uint64_t(t) * H + rt * 16 + c;
                ZC_ST(p.tout + (layer & 1u) * H + at, (__float_as_uint(y) & 0xffff0000u) | tag);   // y is BF16-valued
                if (p.out_trace) st_f32(p.out_trace + uint64_t(layer) * p.trace_tokens * H + at, y);
                if (layer + 1 == p.L) st_f32(p.out + at, y);
            }
        }
        clock_all(13);
        __syncthreads();   // the next layer polls the output words themselves
        clock(14);
    }
}

static uint32_t align16(uint32_t v) { return (v + 15u) / 16u * 16u; }

DecodeLdsPlan decode_lds_plan(uint32_t H, uint32_t E, uint32_t topk, uint32_t I, uint32_t NT, uint32_t lds_limit) {
    DecodeLdsPlan lp{};
    const XintLayout LH{H}, LI{I};
    uint32_t at = 0;
    auto take = [&](uint32_t bytes) { const uint32_t o = at; at += align16(bytes); return o; };
    lp.ids = take(NT * topk * 4); lp.weights = take(NT * topk * 4); lp.gatev = take(NT * 4);
    lp.experts = take(E * 4); lp.misc = take(64); lp.gatew = take(H * 2);
    lp.spec = take((2 * (topk + 1) + 1) * 4);
    lp.region = at;
    lp.img_rg = lp.region; lp.xh = lp.img_rg + NT * LH.bytes();
    lp.gprod = lp.xh + align16(NT * H * 2);   // one token: the shared gate dot's products, [32][hidden / 32 + 1] fp32
    const uint32_t rg_end = lp.gprod + (NT == 1 ? align16(32 * (H / 32 + 1) * 4) : 0);
    lp.otile = lp.region;
    const uint32_t slots = NT * (topk + 1);
    lp.img_d = lp.otile + align16(slots * 16 * 4);
    const uint32_t per_slot = LI.bytes() + align16(I * 2);
    uint32_t sb = lp.img_d < lds_limit ? (lds_limit - lp.img_d) / per_slot : 0;
    if (sb > slots) sb = slots;
    lp.slots_per_batch = sb;
    lp.ah = lp.img_d + sb * LI.bytes();
    const uint32_t d_end = lp.ah + sb * align16(I * 2);
    lp.total = rg_end > d_end ? rg_end : d_end;
    // One workgroup per compute unit: ask for more than half of the LDS so that the
    // dispatcher cannot stack two workgroups on one unit and leave another idle.
    const uint32_t exclusive = lds_limit / 2 + 1024;
    if (lp.total < exclusive) lp.total = exclusive;
    return lp;
}

hipError_t launch_decode_stack(hipStream_t s, const DecodeParams& p, uint32_t nt, uint32_t workgroups, const DecodeLdsPlan& lp) {
#define ZC_DECODE(MIXED)                                                                                               \
    do {                                                                                                               \
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(decode_stack_kernel<MIXED>),                \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, int(lp.total));                 \
        if (e != hipSuccess) return e;                                                                                 \
        hipLaunchKernelGGL((decode_stack_kernel<MIXED>), dim3(workgroups), dim3(decode_threads(1)), lp.total, s, p, lp);  \
    } while (0)
    (void)nt;   // two to eight tokens run decode_multi_kernel (zc_decode_multi.hip)
    if (p.bits_down == 4 && p.shared_bits_gate_up == 4 && p.shared_bits_down == 4) ZC_DECODE(false); else ZC_DECODE(true);
#undef ZC_DECODE
    return hipGetLastError();
}
hipError_t decode_stack_occupancy(uint32_t nt, uint32_t lds_bytes, int* blocks_per_cu) {
    (void)nt;
    // both variants have the same launch bounds and dynamic LDS; the mixed one uses no more registers than the other
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(decode_stack_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(decode_stack_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    if (e != hipSuccess) return e;
    int plain = 0, mixed = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&plain, decode_stack_kernel<false>, decode_threads(1), lds_bytes);
    if (e != hipSuccess) return e;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&mixed, decode_stack_kernel<true>, decode_threads(1), lds_bytes);
    *blocks_per_cu = plain < mixed ? plain : mixed;
    return e;
}

}  // namespace zc
