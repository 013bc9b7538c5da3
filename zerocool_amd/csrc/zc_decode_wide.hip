// Persistent decode kernel for nine to sixty-four tokens: a whole stack of MoE layers in ONE launch.
//
// The kernel for two to eight tokens keeps every token's input row and digit-plane image in LDS; sixty-four do not fit.
// Here a workgroup holds the rows and images of at most eight tokens at a time, namely those of the work it is about to do:
//   * the unit of expert work is an ENTRY = (distinct expert, batch of up to eight of the tokens routed to it), the shared
//     expert's entries being the tokens eight at a time; every workgroup derives the same entry list from the routes;
//   * the flat list of (entry, tile, pass of two tokens) is cut into one contiguous range per workgroup, as in the smaller
//     kernel; for each entry in its range a workgroup stages the entry's rows from the previous layer's output (applying the
//     glue's scale), builds their images once, and runs its items -- for the gate/up tiles as for the down tiles;
//   * the router's units are (four experts x sixteen K partitions) for a PAIR of tokens; a workgroup takes a contiguous range
//     of units ordered by pair, so it stages two rows per pair it touches;
//   * routing (top-k + softmax) is one wave per token, spread over the workgroups; ids and weights cross through memory.
// A layer is five phases with a grid barrier after each: R router logits and shared gate dots, T routing, G gate/up tiles,
// D down tiles, C weighted combine.  The reference shares an expert's weights across a tile of tokens the same way
// (kernels/metal/qwen.metal:444-498, affine_multi).  Arithmetic is the exact-integer matrix-core form (zc_xint.hpp) and the
// literal router / route / combine expressions: every value equals the operator kernels bit for bit.
//
// Cross-workgroup data is written and read only with agent-scope relaxed atomics (write-through / coherent), so a barrier
// needs wait counters and flags, no cache maintenance.  Weights are read with ordinary cached loads.
//
// Between layers the stacked-decode workload applies a stand-in glue (not reference arithmetic):
// x_next = bf(y * (1 / max|y|)) per token, order independent.
#include "zc_decode_common.hpp"

namespace zc {

constexpr int kWideBatch = 8;                // tokens whose rows and images a workgroup holds at a time
// Tokens one tile pass holds, chosen at build time: 2 with 512 threads (two waves per SIMD cover each other's latencies), or
// up to 8 with 256 threads (one wave per SIMD with the whole register file; a tile's codes are expanded once for the entry).
#ifndef ZC_WIDE_PASS_TOKENS
#define ZC_WIDE_PASS_TOKENS 2
#endif
constexpr int kWidePass = ZC_WIDE_PASS_TOKENS;
constexpr uint32_t kWideThreads = kWidePass <= 2 ? 512 : 256, kWideWaves = kWideThreads / 64;

template <bool T32, class Emit>
__device__ __forceinline__ void run_tile_wide(const uint8_t* w_row, const uint16_t* s_row, const uint16_t* b_row, uint32_t spans, const uint8_t* const* img,
                                              const LdsBf16* src, const XintLayout L, uint32_t lane, int nt, Emit emit) {
    if constexpr (T32) {   // tiles of 32 weight rows on the 32x32x32 instruction
        if (nt <= 1) xint_run_tile32<1>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
        else if (kWidePass == 2 || nt == 2) xint_run_tile32<2>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
        else if constexpr (kWidePass >= 4) xint_run_tile32<4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    } else if constexpr (kWidePass == 8) xint_run_tile_upto8(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    else if (nt <= 1) xint_run_tile_tokens<1, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    else xint_run_tile_tokens_piped<2, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
}

// MIXED: the down projection and/or the shared expert are affine Q8 and run on literal lanes (q8_rows_chunked); a variant of
// its own, so that the all-Q4 kernel is exactly what it was.  It also serves two to eight tokens of such artifacts.
template <bool MIXED>
__global__ __launch_bounds__(kWideThreads) void decode_wide_kernel(DecodeParams p, WideLdsPlan lp) {
    constexpr int PT = kWidePass, MT = kWideBatch;
    constexpr bool T32 = !MIXED && (kWidePass == 2 || kWidePass == 4);
    constexpr uint32_t TR = T32 ? 16 : 8, DR = T32 ? 32 : 16;   // gate (and up) rows of a gate/up tile, rows of a down tile
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, col = lane & 15u, G = lane >> 4;
    const uint32_t wg = blockIdx.x, nwg = gridDim.x;
    uint32_t H = p.H, E = p.E, I = p.I, k = p.topk, T = p.T, n = T * k;
    int32_t* ids = reinterpret_cast<int32_t*>(lds + lp.ids);
    float* weights = reinterpret_cast<float*>(lds + lp.weights);
    float* gatev = reinterpret_cast<float*>(lds + lp.gatev);     // the combine's gate factor per token
    float* gscale = reinterpret_cast<float*>(lds + lp.gscale);   // the glue's scale per token
    unsigned long long* chosen = reinterpret_cast<unsigned long long*>(lds + lp.chosen);   // per expert: a bit per token routed to it
    int32_t* entries = reinterpret_cast<int32_t*>(lds + lp.entries);   // (expert << 3 | batch); expert == E: the shared expert
    int32_t* cum = reinterpret_cast<int32_t*>(lds + lp.cum);           // cum[i] = passes of the entries before entry i
    int32_t* misc = reinterpret_cast<int32_t*>(lds + lp.misc);
    uint16_t* xh = reinterpret_cast<uint16_t*>(lds + lp.xh);
    const XintLayout LH{H}, LI{I};
    Barrier bar{p.sync, p.epoch, p.spin_limit, p.status, p.epoch};
    // stamps of every workgroup (a tuning aid): clocks[(stamp index) * workgroups + workgroup]; kDecodeStamps per layer: start, scales,
    // router done, barrier, routed, barrier, entries, gate/up done, barrier, down done, barrier, combined, barrier
    uint32_t stamp = 0;
    auto clock = [&]() { if (p.clocks && tid == 0) p.clocks[uint64_t(stamp) * nwg + wg] = wall_clock64(); ++stamp; };
    auto clock_all = [&]() { if (p.clocks) __syncthreads(); clock(); };

    auto store_act = [&](float* buffer, uint32_t slot_row, uint32_t row, float v) {   // SwiGLU of a gate/up tile as packed BF16 pairs
        const float up = T32 ? __shfl(v, (lane & ~31u) | ((lane & 15u) + 16u)) : __shfl(v, (lane & ~15u) | ((col & 7u) + 8u));
        const uint32_t a = __float_as_uint(swiglu_bf(v, up));
        const uint32_t other = uint32_t(__shfl_xor(int(a), 1));
        if (lane < TR && !(lane & 1u))
            ZC_ST(reinterpret_cast<uint32_t*>(buffer) + (uint64_t(slot_row) * I + row) / 2, (a >> 16) | (other & 0xffff0000u));
    };
    // exclusive prefix of `mine` over the threads of the workgroup, and the total; every thread calls it
    auto block_scan = [&](uint32_t mine, uint32_t& before, uint32_t& total) {
        uint32_t incl = mine;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { const uint32_t up = uint32_t(__shfl_up(int(incl), o)); if (int(lane) >= o) incl += up; }
        if (lane == 63) misc[1 + wave] = int32_t(incl);
        __syncthreads();
        before = incl - mine; total = 0;
        for (uint32_t w = 0; w < kWideWaves; ++w) { const uint32_t v = uint32_t(misc[1 + w]); if (w < wave) before += v; total += v; }
        __syncthreads();
    };

    for (uint32_t layer = 0; layer < p.L; ++layer) {
        const DecodeLayer L = p.layers[layer];
        auto refresh = [&]() {   // per-lane values and the shape are formed again per phase: hoisted, they would stay live through all of them
            asm volatile("" : "+v"(tid));
            lane = tid & 63u; wave = uint32_t(uniform(int32_t(tid >> 6))); col = lane & 15u; G = lane >> 4;
            H = p.H; E = p.E; I = p.I; k = p.topk; T = p.T;
            asm volatile("" : "+s"(H), "+s"(E), "+s"(I), "+s"(k), "+s"(T));
            n = T * k;
        };
        refresh();
        stamp = layer * kDecodeStamps;
        clock();
        const bool glue = layer != 0;
        const float* rows_in = glue ? p.layer_out : p.x_in;
        __syncthreads();
        // the glue's scale per token: 1 / max|y| of the previous layer, from the candidates the combine left per 64 columns
        for (uint32_t t = wave; t < T; t += kWideWaves) {
            uint32_t m = 0;
            if (glue) for (uint32_t g = lane; g < H / 64; g += 64) m = max(m, ZC_LD(p.maxabs + t * (H / 64) + g));
            m = __float_as_uint(wave_max_f32(__uint_as_float(m)));
            if (lane == 0) {
                const float v = __uint_as_float(m);
                gscale[t] = (glue && v > 0.0f && v < __uint_as_float(0x7f800000u)) ? 1.0f / v : 1.0f;
            }
        }
        for (uint32_t i = tid; i < H / 8; i += kWideThreads) reinterpret_cast<uint4*>(lds + lp.gatew)[i] = ldg_u4(L.shared_gate, i);
        __syncthreads();
        // Stages `count` whole rows starting at token `first` as BF16 into LDS rows 0.. of xh, scaled; all threads call it.
        auto stage_rows = [&](uint32_t first, uint32_t count, uint16_t* dst) {
            const int bad = stage_bf16<8>(rows_in + uint64_t(first) * H, count * H / 2, reinterpret_cast<uint32_t*>(dst), []() {},
                [&](uint32_t i, float& a, float& b) {
                    if (glue) { const float scale = gscale[first + (2 * i) / H]; a = bf(a * scale); b = bf(b * scale); }
                });
            if (bad) atomicOr(p.status, 4);   // inputs must be BF16-valued
        };
        clock();
        // ---------------- phase R: router logits and shared gate dots ----------------
        {
            // units of a token pair: (E + 3) / 4 router units (four experts x sixteen K partitions each), then the pair's gate dots
            const uint32_t pairs = (T + 1) / 2, per_pair = (E + 3) / 4 + 1, total = pairs * per_pair;
            const uint32_t u0 = uint32_t(uint64_t(wg) * total / nwg), u1 = uint32_t(uint64_t(wg + 1) * total / nwg);
            constexpr int kPieces = 24;   // sixteen-byte pieces of a K partition at hidden 3072
            for (uint32_t at = u0; at < u1;) {
                const uint32_t pair = at / per_pair, seg_end = min(u1, (pair + 1) * per_pair), t0 = pair * 2;
                const bool two = t0 + 1 < T;
                __syncthreads();   // the units of the previous pair have read their rows
                stage_rows(t0, two ? 2u : 1u, xh);
                __syncthreads();
                for (uint32_t u = at + wave; u < seg_end; u += kWideWaves) {
                    const uint32_t unit = u - pair * per_pair;
                    if (unit + 1 < per_pair) {
                        const uint32_t e = unit * 4 + lane / 16, split = lane % 16, P = H / 16;
                        const uint16_t* wr = L.router + uint64_t(e < E ? e : E - 1) * H + split * P;
                        const uint32_t pieces = P / 8;
                        const uint16_t* x0 = xh + split * P;
                        const uint16_t* x1 = xh + (two ? H : 0u) + split * P;
                        float c0 = 0, c1 = 0;
                        auto piece = [&](uint32_t i, const uint4 w) {
                            const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
                            const uint4 xa = *reinterpret_cast<const uint4*>(x0 + i * 8), xb = *reinterpret_cast<const uint4*>(x1 + i * 8);
                            const uint32_t xwa[4] = {xa.x, xa.y, xa.z, xa.w}, xwb[4] = {xb.x, xb.y, xb.z, xb.w};
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                const float wl = __uint_as_float(ww[q] << 16), wh = __uint_as_float(ww[q] & 0xffff0000u);
                                c0 = __builtin_fmaf(__uint_as_float(xwa[q] << 16), wl, c0);
                                c0 = __builtin_fmaf(__uint_as_float(xwa[q] & 0xffff0000u), wh, c0);
                                c1 = __builtin_fmaf(__uint_as_float(xwb[q] << 16), wl, c1);
                                c1 = __builtin_fmaf(__uint_as_float(xwb[q] & 0xffff0000u), wh, c1);
                            }
                        };
                        if (pieces <= uint32_t(kPieces)) {   // every piece requested at once: one memory latency for the unit
                            uint4 wv[kPieces];
#pragma unroll
                            for (int i = 0; i < kPieces; ++i) wv[i] = ldg_u4(wr, min(uint32_t(i), pieces - 1));
#pragma unroll
                            for (int i = 0; i < kPieces; ++i) if (uint32_t(i) < pieces) piece(uint32_t(i), wv[i]);
                        } else {
                            for (uint32_t i = 0; i < pieces; ++i) piece(i, ldg_u4(wr, i));
                        }
                        // partials added 0..15: after step s the lane of partition i <= s holds ((c0 + c1) + ..) + ci
                        const float offset = (L.offsets && e < E) ? ldg_f32(L.offsets, e) : 0.0f;
                        float s0 = 0.0f + c0, s1 = 0.0f + c1;
#pragma unroll
                        for (int step = 1; step < 16; ++step) { s0 = dpp_row_shr1(s0) + c0; s1 = dpp_row_shr1(s1) + c1; }
                        if (split == 15 && e < E) {
                            st_f32(p.logits + uint64_t(t0) * E + e, L.offsets ? s0 + offset : s0);
                            if (two) st_f32(p.logits + uint64_t(t0 + 1) * E + e, L.offsets ? s1 + offset : s1);
                        }
                    } else {
                        // shared_expert_gate: reference lane chain k = lane + 32 j (qwen.metal:499-506); the pair's two tokens on the wave's halves
                        const uint32_t half = lane >> 5, t = t0 + half, l32 = lane & 31u;
                        const uint16_t* gw = reinterpret_cast<const uint16_t*>(lds + lp.gatew);
                        float sum = 0;
                        if (t < T)
                            for (uint32_t k0 = l32; k0 < H; k0 += 256) {   // eight LDS reads in flight per operand; the sum stays in k order
                                float a[8], g[8];
#pragma unroll
                                for (int j = 0; j < 8; ++j) { a[j] = b16(xh[half * H + k0 + 32 * j]); g[j] = b16(gw[k0 + 32 * j]); }
#pragma unroll
                                for (int j = 0; j < 8; ++j) sum += a[j] * g[j];
                            }
                        sum = lane_sum32(sum);
                        if (t < T && l32 == 0) st_f32(p.gate + t, bf(sum));
                    }
                }
                at = seg_end;
            }
        }
        clock_all();
        bar.wait();
        refresh();
        clock();
        // ---------------- phase T: top-k + softmax, one wave per token, spread over the workgroups ----------------
        for (uint32_t t = wg + nwg * wave; t < T; t += nwg * kWideWaves) {
            uint32_t* scratch = reinterpret_cast<uint32_t*>(entries) + 128 * wave;   // the entry list is built later; 128 words per wave
            auto fetch = [&](auto& cand, uint32_t per) {
                constexpr int PER = int(sizeof(cand) / sizeof(float));
                const float ninf = __uint_as_float(0xff800000u);
#pragma unroll
                for (int i = 0; i < PER; ++i) {
                    const uint32_t e = lane * per + i;
                    cand[i] = (uint32_t(i) < per && e < E) ? load_shared_f32(p.logits + uint64_t(t) * E + e) : ninf;
                }
            };
            if (E == 512) route_token<8>(fetch, E, k, lane, ids + t * k, weights + t * k, scratch, []() {}, []() {});
            else route_token<16>(fetch, E, k, lane, ids + t * k, weights + t * k, scratch, []() {}, []() {});
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // the routes were written by other lanes of this wave
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (lane < k) { st_i32(p.route_ids + t * k + lane, ids[t * k + lane]); st_f32(p.route_weights + t * k + lane, weights[t * k + lane]); }
        }
        clock_all();
        bar.wait();
        refresh();
        clock();
        // every workgroup takes all routes and derives the same entry list from them
        for (uint32_t i = tid; i < n; i += kWideThreads) {
            ids[i] = int32_t(ZC_LD(reinterpret_cast<const uint32_t*>(p.route_ids) + i));
            weights[i] = load_shared_f32(p.route_weights + i);
        }
        if (tid < T) gatev[tid] = bf(sigmoid_bf(load_shared_f32(p.gate + tid)));
        for (uint32_t e = tid; e < E; e += kWideThreads) chosen[e] = 0ull;
        __syncthreads();
        for (uint32_t i = tid; i < n; i += kWideThreads) {
            const int32_t e = ids[i];
            if (e < 0 || e >= int32_t(E)) { if (wg == 0) atomicOr(p.status, 1); }
            else atomicOr(&chosen[e], 1ull << (i / k));
            if (wg == 0 && p.ids_trace) { st_i32(p.ids_trace + uint64_t(layer) * p.trace_tokens * k + i, e); st_f32(p.weights_trace + uint64_t(layer) * p.trace_tokens * k + i, weights[i]); }
        }
        __syncthreads();
        // entries: every distinct expert's tokens eight at a time (ascending expert ids, ascending tokens), then the shared expert's
        uint32_t U = 0;
        for (uint32_t e0 = 0; e0 < E; e0 += kWideThreads) {
            const uint32_t e = e0 + tid;
            const uint32_t batches = e < E ? (uint32_t(__popcll(chosen[e])) + MT - 1) / MT : 0u;
            uint32_t before, total;
            block_scan(batches, before, total);
            for (uint32_t b = 0; b < batches; ++b) entries[U + before + b] = int32_t(e << 3 | b);
            U += total;
        }
        const uint32_t shared_entries = (T + MT - 1) / MT, NE = U + shared_entries;
        if (tid < shared_entries) entries[U + tid] = int32_t(E << 3 | tid);
        __syncthreads();
        // the tokens of an entry as a bit mask (at most eight bits set)
        auto tokens_of = [&](uint32_t packed) {
            const uint32_t e = packed >> 3, b = packed & 7u;
            unsigned long long m = e < E ? chosen[e] : (T >= 64 ? ~0ull : (1ull << T) - 1ull);
            for (uint32_t i = 0; i < b * MT && m; ++i) m &= m - 1;   // the batches before this one
            unsigned long long mine = 0;
            for (int i = 0; i < MT && m; ++i) { mine |= m & (~m + 1); m &= m - 1; }
            return mine;
        };
        {   // cum[i + 1] = passes of entries 0..i
            uint32_t carried = 0;
            for (uint32_t i0 = 0; i0 < NE; i0 += kWideThreads) {
                const uint32_t i = i0 + tid;
                const uint32_t mine = i < NE ? (uint32_t(__popcll(tokens_of(uint32_t(entries[i])))) + PT - 1) / PT : 0u;
                uint32_t before, total;
                block_scan(mine, before, total);
                if (i < NE) cum[i + 1] = int32_t(carried + before + mine);
                carried += total;
            }
            if (tid == 0) cum[0] = 0;
            __syncthreads();
        }
        // all slots of entry ei (at most eight), ascending tokens: slot = token * topk + rank for a routed expert, n + token for the shared one
        auto slots_of = [&](uint32_t ei, int32_t (&all)[MT], int32_t (&token)[MT], bool& routed, uint32_t& e) {
            const uint32_t packed = uint32_t(uniform(entries[ei]));
            e = packed >> 3; routed = e < E;
            const uint32_t batch = packed & 7u;
            const unsigned long long whole = routed ? chosen[e] : (T >= 64 ? ~0ull : (1ull << T) - 1ull);
            uint32_t lo = uint32_t(uniform(int32_t(uint32_t(whole)))), hi = uint32_t(uniform(int32_t(uint32_t(whole >> 32))));
            unsigned long long m = (static_cast<unsigned long long>(hi) << 32) | lo;
            for (uint32_t i = 0; i < batch * MT && m; ++i) m &= m - 1;
            int na = 0;
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                all[i] = 0; token[i] = 0;
                if (m) {
                    const uint32_t t = uint32_t(__builtin_ctzll(m));
                    m &= m - 1;
                    uint32_t rank = 0;
                    if (routed) for (uint32_t j = 0; j < k; ++j) if (uniform(ids[t * k + j]) == int32_t(e)) rank = j;
                    all[i] = routed ? int32_t(t * k + rank) : int32_t(n + t);
                    token[i] = int32_t(t);
                    na = i + 1;
                }
            }
            return na;
        };
        auto pass_of = [&](const int32_t (&all)[MT], int na, uint32_t pass, int32_t (&slot)[PT], uint32_t (&index)[PT]) {
            const int nt = min(int(PT), na - int(pass) * PT);
#pragma unroll
            for (int t = 0; t < PT; ++t) {
                index[t] = t < nt ? pass * PT + uint32_t(t) : 0u;
                slot[t] = 0;
#pragma unroll
                for (int a = 0; a < MT; ++a) slot[t] = uint32_t(a) == index[t] ? all[a] : slot[t];
            }
            return nt;
        };
        clock();
        // ---------------- phase G: gate/up tiles; items (entry, tile, pass), one contiguous range per workgroup ----------------
        {
            // A Q8 gate/up tile of the shared expert is several memory latencies long: its items are cut into `cut` pieces of
            // 8 / cut row pairs, i.e. the shared entries (the last ones of the list) count `cut` times their passes here.
            const bool q8_shared = MIXED && p.shared_bits_gate_up == 8;
            const uint32_t cut = q8_shared ? 4u : 1u, routed_passes = uint32_t(cum[U]);
            auto gcum = [&](uint32_t i) { const uint32_t c = uint32_t(uniform(cum[i])); return i <= U ? c : routed_passes + cut * (c - routed_passes); };
            const uint32_t tiles = I / TR, total = tiles * gcum(NE);
            uint32_t i0, i1;
            share_of_items(wg, nwg, total, kWideWaves, i0, i1);
            uint32_t ei = 0;
            while (ei + 1 < NE && tiles * gcum(ei + 1) <= i0) ++ei;
            for (uint32_t at = i0; at < i1; ++ei) {
                const uint32_t first = tiles * gcum(ei), seg_end = min(i1, tiles * gcum(ei + 1));
                int32_t all[MT], token[MT]; bool routed; uint32_t e;
                const int na = slots_of(ei, all, token, routed, e);
                __syncthreads();   // the previous entry's tiles have read their rows and images
                {   // the entry's input rows, all requested at once
                    const float* rows[MT];
#pragma unroll
                    for (int t = 0; t < MT; ++t) rows[t] = rows_in + uint64_t(uint32_t(token[t])) * H;
                    const int bad = stage_bf16_rows(rows, na, H / 2, reinterpret_cast<uint32_t*>(xh), [&](int t, float& a, float& b) {
                        if (glue) { const float scale = gscale[token[t]]; a = bf(a * scale); b = bf(b * scale); }
                    });
                    if (bad) atomicOr(p.status, 4);   // inputs must be BF16-valued
                }
                __syncthreads();
                xint_prepare_batch([&](uint32_t t) { return LdsBf16{xh + t * H}; }, uint32_t(na), LH, lds + lp.img_x);
                const uint8_t* rec = routed ? record_of(L, e) : L.shared_record;
                const uint64_t* off = routed ? p.ro : p.so;
                const uint32_t passes = uint32_t(na + PT - 1) / PT;
                for (uint32_t item = at + wave; item < seg_end; item += kWideWaves) {
                    if (MIXED && !routed && q8_shared) {
                        // affine Q8 rows: the lower half of the wave takes gate rows, the upper half the up rows of the same indices
                        const uint32_t local = item - first, piece = local % cut, pass = (local / cut) % passes, tile = local / (cut * passes);
                        int32_t slot[PT]; uint32_t index[PT];
                        const int nt = pass_of(all, na, pass, slot, index);
                        const uint32_t side = lane >> 5, per_piece = 8 / cut, row0 = tile * 8 + piece * per_piece;
                        const uint16_t* const rows_in[PT] = {xh + index[0] * H, xh + index[PT - 1] * H};
                        q8_rows_chunked<2, 2, PT>(rec + p.so[side * 3], reinterpret_cast<const uint16_t*>(rec + p.so[side * 3 + 1]),
                                reinterpret_cast<const uint16_t*>(rec + p.so[side * 3 + 2]), H, rows_in, per_piece,
                                [&](uint32_t i) { return row0 + i; },
                                [&](uint32_t i, int t, float v) {
                                    const float up = __shfl(v, 32);
                                    const uint32_t a = __float_as_uint(swiglu_bf(v, up)) >> 16;   // BF16 bits
                                    if (lane == 0 && t < nt)
                                        __hip_atomic_store(reinterpret_cast<uint16_t*>(p.shared_act) + uint64_t(uint32_t(slot[t]) - n) * I + row0 + i, uint16_t(a),
                                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                });
                        continue;
                    }
                    const uint32_t tile = (item - first) / passes, pass = pass_of_item(item - first, passes, kWideWaves);
                    const uint32_t row = T32 ? tile * 16 + (lane & 15u) : tile * 8 + (col & 7u), pr = T32 ? ((lane & 31u) < 16 ? 0 : 3) : (col < 8 ? 0 : 3);
                    const uint8_t* w_row = rec + off[pr] + uint64_t(row) * (H / 2);
                    const uint16_t* s_row = reinterpret_cast<const uint16_t*>(rec + off[pr + 1]) + uint64_t(row) * (H / 64);
                    const uint16_t* b_row = reinterpret_cast<const uint16_t*>(rec + off[pr + 2]) + uint64_t(row) * (H / 64);
                    int32_t slot[PT]; uint32_t index[PT];
                    const int nt = pass_of(all, na, pass, slot, index);
                    const uint8_t* img[PT]; LdsBf16 src[PT];
#pragma unroll
                    for (int t = 0; t < PT; ++t) { img[t] = lds + lp.img_x + index[t] * LH.bytes(); src[t] = LdsBf16{xh + index[t] * H}; }
                    auto emit = [&](int t, float v) {
                        if (routed) store_act(p.act, uint32_t(slot[t]), row, v); else store_act(p.shared_act, uint32_t(slot[t]) - n, row, v);
                    };
                    run_tile_wide<T32>(w_row, s_row, b_row, H / 128, img, src, LH, lane, nt, emit);
                }
                at = seg_end;
            }
        }
        clock_all();
        bar.wait();
        refresh();
        clock();
        // ---------------- phase D: down tiles; items (entry, row tile, pass), one contiguous range per workgroup ----------------
        {
            const uint32_t row_tiles = H / DR, total = row_tiles * uint32_t(cum[NE]);
            uint32_t i0, i1;
            share_of_items(wg, nwg, total, kWideWaves, i0, i1);
            uint16_t* ah = reinterpret_cast<uint16_t*>(lds + lp.ah);
            uint32_t ei = 0;
            while (ei + 1 < NE && row_tiles * uint32_t(uniform(cum[ei + 1])) <= i0) ++ei;
            for (uint32_t at = i0; at < i1; ++ei) {
                const uint32_t first = row_tiles * uint32_t(uniform(cum[ei])), seg_end = min(i1, row_tiles * uint32_t(uniform(cum[ei + 1])));
                int32_t all[MT], token[MT]; bool routed; uint32_t e;
                const int na = slots_of(ei, all, token, routed, e);
                __syncthreads();   // the previous entry's tiles have read their images
                {   // the slots' activations (packed BF16 rows of I elements) into LDS, all requested at once, then their images
                    const uint64_t* rows[MT];
#pragma unroll
                    for (int t = 0; t < MT; ++t) {
                        const uint32_t sl = uint32_t(all[t]);
                        rows[t] = sl < n ? reinterpret_cast<const uint64_t*>(p.act) + uint64_t(sl) * I / 4
                                         : reinterpret_cast<const uint64_t*>(p.shared_act) + uint64_t(sl - n) * I / 4;
                    }
                    stage_copy_rows(rows, na, I / 4, reinterpret_cast<uint64_t*>(ah));
                }
                __syncthreads();
                xint_prepare_batch([&](uint32_t t) { return LdsBf16{ah + t * I}; }, uint32_t(na), LI, lds + lp.img_d);
                const uint8_t* rec = routed ? record_of(L, e) : L.shared_record;
                const uint64_t* off = routed ? p.ro : p.so;
                const uint32_t passes = uint32_t(na + PT - 1) / PT;
                for (uint32_t item = at + wave; item < seg_end; item += kWideWaves) {
                    const uint32_t pass = pass_of_item(item - first, passes, kWideWaves);
                    const uint32_t row = ((item - first) / passes) * DR + (T32 ? (lane & 31u) : col);
                    const uint8_t* w_row = rec + off[6] + uint64_t(row) * (I / 2);
                    const uint16_t* s_row = reinterpret_cast<const uint16_t*>(rec + off[7]) + uint64_t(row) * (I / 64);
                    const uint16_t* b_row = reinterpret_cast<const uint16_t*>(rec + off[8]) + uint64_t(row) * (I / 64);
                    int32_t slot[PT]; uint32_t index[PT];
                    const int nt = pass_of(all, na, pass, slot, index);
                    if (MIXED && (routed ? p.bits_down : p.shared_bits_down) == 8) {   // affine Q8 down rows: row 2 i of the tile on the lower half, 2 i + 1 on the upper
                        const uint32_t row0 = ((item - first) / passes) * 16;
                        const uint16_t* const rows_in[PT] = {ah + index[0] * I, ah + index[PT - 1] * I};
                        q8_rows_chunked<2, 4, PT>(rec + off[6], reinterpret_cast<const uint16_t*>(rec + off[7]), reinterpret_cast<const uint16_t*>(rec + off[8]), I,
                                rows_in, 8, [&](uint32_t i) { return row0 + 2 * i + (lane >> 5); },
                                [&](uint32_t i, int t, float v) {
                                    if ((lane & 31u) == 0 && t < nt) st_f32(p.eout + uint64_t(slot[t]) * H + row0 + 2 * i + (lane >> 5), bf(v));
                                });
                        continue;
                    }
                    const uint8_t* img[PT]; LdsBf16 src[PT];
#pragma unroll
                    for (int t = 0; t < PT; ++t) { img[t] = lds + lp.img_d + index[t] * LI.bytes(); src[t] = LdsBf16{ah + index[t] * I}; }
                    auto emit = [&](int t, float v) { if (T32 ? lane < 32 : G == 0) st_f32(p.eout + uint64_t(slot[t]) * H + row, bf(v)); };
                    run_tile_wide<T32>(w_row, s_row, b_row, I / 128, img, src, LI, lane, nt, emit);
                }
                at = seg_end;
            }
        }
        clock_all();
        bar.wait();
        refresh();
        clock();
        // ---------------- phase C: weighted combine (reference: qwen.metal:804-816), spread over the grid ----------------
        for (uint32_t group = wg + nwg * wave; group < T * H / 64; group += nwg * kWideWaves) {   // 64 neighbouring columns of one token per wave
            const uint32_t idx = group * 64 + lane, t = idx / H, c = idx % H;
            float partial[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) partial[q] = 0;
            const float shared_out = load_shared_f32(p.eout + uint64_t(n + t) * H + c);
            for (uint32_t base = 0; base < k; base += 8) {   // eight independent products at a time, partial j takes slots j, j+8, ...
                float value[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t kk = base + j;
                    const int32_t e = kk < k ? ids[t * k + kk] : -1;
                    value[j] = (e >= 0 && e < int32_t(E)) ? load_shared_f32(p.eout + uint64_t(t * k + kk) * H + c) : 0.0f;
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t kk = base + j;
                    if (kk < k) {
                        const float product = value[j] * weights[t * k + kk];
                        partial[j] = base == 0 ? product : partial[j] + product;
                    }
                }
            }
            float sum = partial[0];
            for (uint32_t kk = 1; kk < 8 && kk < k; ++kk) sum += partial[kk];
            const float y = bf(bf(sum) + bf(gatev[t] * shared_out));
            st_f32(p.layer_out + idx, y);
            if (p.out_trace) st_f32(p.out_trace + uint64_t(layer) * p.trace_tokens * H + idx, y);
            if (layer + 1 == p.L) st_f32(p.out + idx, y);
            uint32_t m = __float_as_uint(y) & 0x7fffffffu;
            if (m > 0x7f800000u) m = 0;   // NaN does not take part in the maximum
            m = __float_as_uint(wave_max_f32(__uint_as_float(m)));
            if (lane == 0) ZC_ST(p.maxabs + group, m);   // group = t * (H / 64) + column group: read by the next layer's staging
        }
        clock_all();
        bar.wait();
        clock();
    }
}

static uint32_t align16w(uint32_t v) { return (v + 15u) / 16u * 16u; }

WideLdsPlan decode_wide_lds_plan(uint32_t H, uint32_t E, uint32_t topk, uint32_t I, uint32_t T, uint32_t lds_limit) {
    WideLdsPlan lp{};
    const XintLayout LH{H}, LI{I};
    uint32_t at = 0;
    auto take = [&](uint32_t bytes) { const uint32_t o = at; at += align16w(bytes); return o; };
    lp.ids = take(T * topk * 4); lp.weights = take(T * topk * 4); lp.gatev = take(T * 4); lp.gscale = take(T * 4);
    lp.chosen = take(E * 8);
    // entries: every distinct expert has at least one, plus one more per eight slots, plus the shared expert's; the list's
    // space also serves the routing waves (128 words each) before it is built
    const uint32_t entries = E + T * topk / kWideBatch + T / kWideBatch + 8;
    lp.entries = take((entries > 128 * kWideWaves ? entries : 128 * kWideWaves) * 4);
    lp.cum = take((entries + 2) * 4);
    lp.misc = take(64); lp.gatew = take(H * 2);
    lp.region = at;
    // router and gate/up phases: eight rows and their images; the down phase reuses the space for an entry's activations
    lp.img_x = lp.region; lp.xh = lp.img_x + kWideBatch * LH.bytes();
    const uint32_t rg_end = lp.xh + align16w(kWideBatch * H * 2);
    lp.img_d = lp.region; lp.ah = lp.img_d + kWideBatch * LI.bytes();
    const uint32_t d_end = lp.ah + align16w(kWideBatch * I * 2);
    lp.total = rg_end > d_end ? rg_end : d_end;
    // One workgroup per compute unit: more than half of the LDS, so that two can never share a unit while another idles.
    const uint32_t exclusive = lds_limit / 2 + 1024;
    if (lp.total < exclusive) lp.total = exclusive;
    return lp;
}

static bool wide_mixed(const DecodeParams& p) { return !(p.bits_down == 4 && p.shared_bits_gate_up == 4 && p.shared_bits_down == 4); }
hipError_t launch_decode_wide(hipStream_t s, const DecodeParams& p, uint32_t workgroups, const WideLdsPlan& lp) {
    const void* kernel = wide_mixed(p) ? reinterpret_cast<const void*>(decode_wide_kernel<true>) : reinterpret_cast<const void*>(decode_wide_kernel<false>);
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, int(lp.total));
    if (e != hipSuccess) return e;
    if (wide_mixed(p)) hipLaunchKernelGGL(decode_wide_kernel<true>, dim3(workgroups), dim3(kWideThreads), lp.total, s, p, lp);
    else hipLaunchKernelGGL(decode_wide_kernel<false>, dim3(workgroups), dim3(kWideThreads), lp.total, s, p, lp);
    return hipGetLastError();
}
hipError_t decode_wide_occupancy(uint32_t lds_bytes, int* blocks_per_cu) {
    int plain = 0, mixed = 0;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(decode_wide_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(decode_wide_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    if (e != hipSuccess) return e;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&plain, decode_wide_kernel<false>, kWideThreads, lds_bytes);
    if (e != hipSuccess) return e;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&mixed, decode_wide_kernel<true>, kWideThreads, lds_bytes);
    *blocks_per_cu = plain < mixed ? plain : mixed;
    return e;
}

}  // namespace zc
