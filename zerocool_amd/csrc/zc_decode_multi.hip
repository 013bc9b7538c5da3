// Persistent decode kernel for two to eight tokens: a whole stack of MoE layers in ONE launch.
//
// One workgroup per compute unit stays resident for all layers.  The tokens of a step mostly pick the same few experts
// (continuous batching over a skewed router), so the unit of work is (distinct expert, tile of output rows): a tile's
// weights are streamed ONCE and multiplied with the input rows of every token routed to that expert -- the reference's
// token tiles (kernels/metal/qwen.metal:444-498, affine_multi) with the expert as the shared operand.  A layer is four
// phases separated by grid barriers:
//   R  stage the T input rows (BF16 copies and digit-plane images in LDS), router logits, shared gate dots
//   G  every workgroup routes the T tokens (top-k + softmax) and groups the slots by expert; then gate/up tiles of the
//      distinct experts and of the shared expert over all waves of the chip, SwiGLU activations out (packed BF16)
//   D  down tiles: the flat list (expert, 16 output rows) is cut into one contiguous range per workgroup, so that a
//      workgroup stages the activations of one expert's slots at a time (images built once per workgroup and expert,
//      not once per output tile), outputs out per slot
//   C  weighted combine (moe_sum order) of every (token, column), spread over the grid; layer output out
// Arithmetic is the exact-integer matrix-core form (zc_xint.hpp) and the literal router / route / combine expressions:
// every value equals the operator kernels bit for bit.
//
// Cross-workgroup data is written and read only with agent-scope relaxed atomics (write-through / coherent), so a
// barrier needs wait counters and flags, no cache maintenance.  Weights are read with ordinary cached loads.
//
// Between layers the stacked-decode workload applies a stand-in glue (not reference arithmetic):
// x_next = bf(y * (1 / max|y|)) per token, order independent.
#include "zc_decode_common.hpp"

namespace zc {

constexpr int kMultiTokens = 8;              // tokens per launch at most
// Two ways to run the tiles, chosen at build time:
//   512 threads, one token per tile pass: two waves per SIMD cover each other's LDS and MFMA latencies; an expert's tokens are
//   separate work items on neighbouring waves of ONE workgroup, so the tile's weights come from HBM once and from the
//   compute unit's caches for the other tokens;
//   256 threads, up to eight tokens per pass: one wave per SIMD with the whole register file, the codes of a span expanded once
//   for all tokens, latencies covered by the hand-pipelined engine.
#ifndef ZC_MULTI_PASS_TOKENS
#define ZC_MULTI_PASS_TOKENS 2
#endif
constexpr int kPassTokens = ZC_MULTI_PASS_TOKENS;   // tokens one tile pass holds
#ifndef ZC_MULTI_THREADS
#define ZC_MULTI_THREADS (ZC_MULTI_PASS_TOKENS <= 4 ? 512 : 256)
#endif
constexpr uint32_t kMultiThreads = ZC_MULTI_THREADS, kMultiWaves = kMultiThreads / 64;
constexpr int kMultiRing = 8;                // sixteen-byte pieces of a router partition in flight per lane

template <class Emit>
__device__ __forceinline__ void run_tile(const uint8_t* w_row, const uint16_t* s_row, const uint16_t* b_row, uint32_t spans, const uint8_t* const* img,
                                         const LdsBf16* src, const XintLayout L, uint32_t lane, int nt, Emit emit) {
    if constexpr (kMultiThreads == 256) xint_run_tile_upto8(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    else if constexpr (kPassTokens == 1) xint_run_tile_tokens<1, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    else if constexpr (kPassTokens == 2) {
        if (nt <= 1) xint_run_tile_tokens<1, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
        else xint_run_tile_tokens_piped<2, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    } else xint_run_tile_upto4(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
}

__global__ __launch_bounds__(kMultiThreads) void decode_multi_kernel(DecodeParams p, MultiLdsPlan lp) {
    constexpr int PT = kPassTokens, MT = kMultiTokens;
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, col = lane & 15u, G = lane >> 4;
    const uint32_t wg = blockIdx.x, nwg = gridDim.x;
    uint32_t H = p.H, E = p.E, I = p.I, k = p.topk, T = p.T, n = T * k;
    int32_t* ids = reinterpret_cast<int32_t*>(lds + lp.ids);
    float* weights = reinterpret_cast<float*>(lds + lp.weights);
    float* gatev = reinterpret_cast<float*>(lds + lp.gatev);
    // the tokens of every expert: a bit per token, and the rank at which the token picked the expert (slot = token * topk + rank);
    // unlike linked lists built with atomics, every workgroup derives the SAME slot order from them
    uint32_t* chosen = reinterpret_cast<uint32_t*>(lds + lp.head);
    uint8_t* rank_of = lds + lp.next;   // [E][8]
    int32_t* experts = reinterpret_cast<int32_t*>(lds + lp.experts);
    int32_t* misc = reinterpret_cast<int32_t*>(lds + lp.misc);   // [0] U, [1..] wave counts
    uint16_t* xh = reinterpret_cast<uint16_t*>(lds + lp.xh);
    const XintLayout LH{H}, LI{I};
    Barrier bar{p.sync, p.epoch, p.spin_limit, p.status, p.epoch};
    uint32_t stamp = 0;
    auto clock = [&]() { if (p.clocks && tid == 0) p.clocks[uint64_t(stamp) * nwg + wg] = wall_clock64(); ++stamp; };
    auto clock_all = [&]() { if (p.clocks) __syncthreads(); clock(); };

    // SwiGLU of a finished gate/up tile (gate rows in columns 0-7, up rows in 8-15), stored as packed BF16 pairs: the lane
    // of an even row writes rows r and r+1 of activation row `slot_row` as one word.
    auto store_act = [&](float* buffer, uint32_t slot_row, uint32_t row, float v) {
        const float up = __shfl(v, (lane & ~15u) | ((col & 7u) + 8u));
        const uint32_t a = __float_as_uint(swiglu_bf(v, up));
        const uint32_t other = uint32_t(__shfl_xor(int(a), 1));
        if (lane < 8 && !(lane & 1u))
            ZC_ST(reinterpret_cast<uint32_t*>(buffer) + (uint64_t(slot_row) * I + row) / 2, (a >> 16) | (other & 0xffff0000u));
    };

    for (uint32_t layer = 0; layer < p.L; ++layer) {
        const DecodeLayer L = p.layers[layer];
        // per-lane values derived from the thread index are formed again in every layer: hoisted out of the layer loop they
        // would stay live through all phases
        // (the same for the shape: quotients, reciprocals and LDS addresses derived from it are formed per phase, not kept)
        auto refresh = [&]() {
            asm volatile("" : "+v"(tid));
            lane = tid & 63u; wave = uint32_t(uniform(int32_t(tid >> 6))); col = lane & 15u; G = lane >> 4;
            H = p.H; E = p.E; I = p.I; k = p.topk; T = p.T;
            asm volatile("" : "+s"(H), "+s"(E), "+s"(I), "+s"(k), "+s"(T));
            n = T * k;
        };
        refresh();
        stamp = layer * kDecodeStamps;
        clock();
        // ---------------- phase R: input rows, their images, router logits, shared gate dots ----------------
        __syncthreads();
        // Router units: four experts x sixteen K partitions for TWO tokens (the weights of a unit are read once per token pair;
        // spreading the pairs over the chip keeps a unit's k-ascending chains short).
        const uint32_t pairs = (T + 1) / 2, router_units = ((E + 3) / 4) * pairs, gate_units = (T + 1) / 2;
        constexpr int kPieces = 24;   // sixteen-byte pieces of a K partition at hidden 3072
        const uint32_t u_first = wg + nwg * wave;
        const bool ahead = H / 128 <= uint32_t(kPieces);
        {
            const bool glue = layer != 0;
            // Everything the staging needs is requested in one go -- the input rows, then the candidates of the glue's scale
            // per token (1 / max|y| of the previous layer: the combine left one candidate per 64 columns) and the shared gate's
            // weights -- so that the three fetches cost one trip to the L2, not three in a row.
            auto ready = [&]() {
                uint4 gw[2];
#pragma unroll
                for (int q = 0; q < 2; ++q) { const uint32_t i = tid + q * kMultiThreads; gw[q] = i < H / 8 ? ldg_u4(L.shared_gate, i) : make_uint4(0, 0, 0, 0); }
                if (glue) {
                    const uint32_t groups = H / 64;
                    uint32_t m = 0;
                    for (uint32_t g = lane; g < groups; g += 64) if (wave < T) m = max(m, ZC_LD(p.maxabs + wave * groups + g));
                    m = __float_as_uint(wave_max_f32(__uint_as_float(m)));
                    if (wave < T && lane == 0) {
                        const float v = __uint_as_float(m);
                        gatev[wave] = (v > 0.0f && v < __uint_as_float(0x7f800000u)) ? 1.0f / v : 1.0f;
                    }
                }
#pragma unroll
                for (int q = 0; q < 2; ++q) { const uint32_t i = tid + q * kMultiThreads; if (i < H / 8) reinterpret_cast<uint4*>(lds + lp.gatew)[i] = gw[q]; }
                __syncthreads();
            };
            const int bad = stage_bf16<24>(glue ? p.layer_out : p.x_in, T * H / 2, reinterpret_cast<uint32_t*>(xh), ready,
                [&](uint32_t i, float& a, float& b) {
                    if (glue) { const float scale = gatev[(2 * i) / H]; a = bf(a * scale); b = bf(b * scale); }
                });
            if (bad) atomicOr(p.status, 4);   // inputs must be BF16-valued
        }
        xint_prepare_begin(LH, lds + lp.img_x, T);
        __syncthreads();
        clock();
        // The waves that own a router or gate unit run it now (the BF16 rows are all they need); the other waves of the
        // workgroup build the tokens' images meanwhile.  With more units than waves (a small grid) every wave does both.
        const bool all_build = router_units + gate_units > nwg * kMultiWaves;
        const uint32_t builders_from = all_build ? 0u : min(kMultiWaves - 1, (router_units + gate_units - min(wg, router_units + gate_units) + nwg - 1) / nwg);
        for (uint32_t u = u_first; u < router_units + gate_units; u += nwg * kMultiWaves) {
            if (u < router_units) {
                const uint32_t t0 = (u % pairs) * 2, e = (u / pairs) * 4 + lane / 16, split = lane % 16, P = H / 16;
                const bool two = t0 + 1 < T;
                const uint16_t* wr = L.router + uint64_t(e < E ? e : E - 1) * H + split * P;
                const uint32_t pieces = P / 8;   // sixteen-byte pieces of the partition
                const uint16_t* x0 = xh + uint64_t(t0) * H + split * P;
                const uint16_t* x1 = xh + uint64_t(two ? t0 + 1 : t0) * H + split * P;
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
                if (ahead) {   // every piece requested at once: one memory latency for the unit
                    uint4 wv[kPieces];
#pragma unroll
                    for (int i = 0; i < kPieces; ++i) wv[i] = ldg_u4(wr, min(uint32_t(i), pieces - 1));
#pragma unroll
                    for (int i = 0; i < kPieces; ++i) if (uint32_t(i) < pieces) piece(uint32_t(i), wv[i]);
                } else {
                    uint4 ring[kMultiRing];
#pragma unroll
                    for (int i = 0; i < kMultiRing; ++i) if (uint32_t(i) < pieces) ring[i] = ldg_u4(wr, i);
                    for (uint32_t i0 = 0; i0 < pieces; i0 += kMultiRing) {
#pragma unroll
                        for (int j = 0; j < kMultiRing; ++j) {
                            const uint32_t i = i0 + j;
                            if (i < pieces) {
                                const uint4 w = ring[j];
                                if (i + kMultiRing < pieces) ring[j] = ldg_u4(wr, i + kMultiRing);
                                piece(i, w);
                            }
                        }
                    }
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
                // shared_expert_gate: reference lane chain k = lane + 32 j (qwen.metal:499-506); two tokens per wave
                const uint32_t t = (u - router_units) * 2 + (lane >> 5), l32 = lane & 31u;
                const uint16_t* gw = reinterpret_cast<const uint16_t*>(lds + lp.gatew);
                float sum = 0;
                if (t < T)
                    for (uint32_t k0 = l32; k0 < H; k0 += 256) {   // eight LDS reads in flight per operand (hidden is a multiple of 512); the sum stays in k order
                        float a[8], g[8];
#pragma unroll
                        for (int j = 0; j < 8; ++j) { a[j] = b16(xh[t * H + k0 + 32 * j]); g[j] = b16(gw[k0 + 32 * j]); }
#pragma unroll
                        for (int j = 0; j < 8; ++j) sum += a[j] * g[j];
                    }
                sum = lane_sum32(sum);
                if (t < T && l32 == 0) st_f32(p.gate + t, bf(sum));
            }
        }
        if (wave >= builders_from) {
            const uint32_t builders = (kMultiWaves - builders_from) * 64u, blocks = LH.blocks();
            for (uint32_t i = tid - builders_from * 64u; i < T * blocks; i += builders) {
                const uint32_t q = i / blocks;
                xint_prepare_block(LdsBf16{xh + q * H}, LH, lds + lp.img_x + q * LH.bytes(), i % blocks);
            }
        }
        clock_all();
        bar.wait();
        refresh();
        clock();
        // ---------------- phase G: route, group slots by expert, gate/up tiles ----------------
        for (uint32_t t = wave; t < T; t += kMultiWaves) {
            uint32_t* scratch = reinterpret_cast<uint32_t*>(experts) + 128 * wave;   // the expert list is built later; 128 words per wave
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
        }
        if (tid < T) gatev[tid] = bf(sigmoid_bf(load_shared_f32(p.gate + tid)));   // the combine's gate factor
        for (uint32_t e = tid; e < E; e += kMultiThreads) chosen[e] = 0;
        __syncthreads();
        clock();
        if (tid < n) {
            const int32_t e = ids[tid];
            if (e < 0 || e >= int32_t(E)) atomicOr(p.status, 1);
            else { atomicOr(&chosen[e], 1u << (tid / k)); rank_of[uint32_t(e) * MT + tid / k] = uint8_t(tid % k); }
            if (wg == 0 && p.ids_trace) { st_i32(p.ids_trace + uint64_t(layer) * p.trace_tokens * k + tid, e); st_f32(p.weights_trace + uint64_t(layer) * p.trace_tokens * k + tid, weights[tid]); }
        }
        __syncthreads();
        // the distinct experts that own at least one slot, ascending ids
        uint32_t U = 0;
        {
            uint32_t base = 0;
            for (uint32_t e0 = 0; e0 < E; e0 += kMultiThreads) {
                const uint32_t e = e0 + tid;
                const bool used = e < E && chosen[e] != 0;
                const uint64_t m = __ballot(used);
                if (lane == 0) misc[1 + wave] = __popcll(m);
                __syncthreads();
                uint32_t before = base;
                for (uint32_t w = 0; w < wave; ++w) before += misc[1 + w];
                if (used) experts[before + __popcll(m & ((1ull << lane) - 1))] = int32_t(e);
                for (uint32_t w = 0; w < kMultiWaves; ++w) base += misc[1 + w];
                __syncthreads();
            }
            U = base;
        }
        // cum[ei] = passes of the experts before list index ei (index U: the shared expert; cum[U + 1] = all passes): tile work is
        // shared out by passes, so that a workgroup with many-token experts gets fewer tiles
        int32_t* cum = reinterpret_cast<int32_t*>(lds + lp.cum);
        {
            uint32_t mine = 0;
            if (tid <= U) {
                uint32_t count = T;
                if (tid < U) count = uint32_t(__popc(chosen[experts[tid]]));
                mine = (count + PT - 1) / PT;
            }
            uint32_t incl = mine;   // inclusive scan inside the wave, then the waves' totals
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) { const uint32_t up = uint32_t(__shfl_up(int(incl), o)); if (int(lane) >= o) incl += up; }
            if (lane == 63) misc[1 + wave] = int32_t(incl);
            __syncthreads();
            uint32_t before = 0;
            for (uint32_t w = 0; w < wave; ++w) before += uint32_t(misc[1 + w]);
            if (tid <= U) cum[tid + 1] = int32_t(before + incl);
            if (tid == 0) cum[0] = 0;
            __syncthreads();
        }
        clock();
        // Work of a tile phase: the flat list (expert index, tile) -- index U is the shared expert, whose slots are the T tokens --
        // is cut into one contiguous range per workgroup; inside a range the items (tile, pass of PT tokens) of one expert go to
        // the waves in turn, so the passes of a tile run side by side on one compute unit.
        // all slots of expert index ei (at most T: a token picks an expert once), in list order
        auto slots_of = [&](uint32_t ei, int32_t (&all)[MT], bool& routed, uint32_t& e) {
            routed = ei < U;
            e = routed ? uint32_t(uniform(experts[ei])) : 0u;
            int na = 0;
            uint32_t m = routed ? uint32_t(uniform(int32_t(chosen[e]))) : (1u << T) - 1u;   // ascending tokens
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                all[i] = 0;
                if (m) {
                    const uint32_t t = uint32_t(__builtin_ctz(m));
                    m &= m - 1;
                    all[i] = routed ? int32_t(t * k) + uniform(int32_t(rank_of[e * MT + t])) : int32_t(n + t);
                    na = i + 1;
                }
            }
            return na;
        };
        // the slots of pass `pass` out of `all`: slot[t] = all[pass * PT + t]
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
        {
            // items = (expert index, tile, pass), passes of a tile adjacent; expert ei owns items [tiles * cum[ei], tiles * cum[ei + 1])
            const uint32_t tiles = I / 8, total = tiles * uint32_t(cum[U + 1]);
            uint32_t i0, i1;
            share_of_items(wg, nwg, total, kMultiWaves, i0, i1);
            uint32_t ei = 0;
            while (ei < U && tiles * uint32_t(uniform(cum[ei + 1])) <= i0) ++ei;
            for (uint32_t at = i0; at < i1; ++ei) {
                const uint32_t first = tiles * uint32_t(uniform(cum[ei])), seg_end = min(i1, tiles * uint32_t(uniform(cum[ei + 1])));
                int32_t all[MT]; bool routed; uint32_t e;
                const int na = slots_of(ei, all, routed, e);
                const uint8_t* rec = routed ? record_of(L, e) : L.shared_record;
                const uint64_t* off = routed ? p.ro : p.so;
                const uint32_t passes = uint32_t(na + PT - 1) / PT;
                for (uint32_t item = at + wave; item < seg_end; item += kMultiWaves) {
                    const uint32_t tile = (item - first) / passes, pass = pass_of_item(item - first, passes, kMultiWaves);
                    const uint32_t row = tile * 8 + (col & 7u), pr = col < 8 ? 0 : 3;
                    const uint8_t* w_row = rec + off[pr] + uint64_t(row) * (H / 2);
                    const uint16_t* s_row = reinterpret_cast<const uint16_t*>(rec + off[pr + 1]) + uint64_t(row) * (H / 64);
                    const uint16_t* b_row = reinterpret_cast<const uint16_t*>(rec + off[pr + 2]) + uint64_t(row) * (H / 64);
                    int32_t slot[PT]; uint32_t index[PT];
                    const int nt = pass_of(all, na, pass, slot, index);
                    const uint8_t* img[PT]; LdsBf16 src[PT];
#pragma unroll
                    for (int t = 0; t < PT; ++t) {
                        const uint32_t tt = t < nt ? (routed ? uint32_t(slot[t]) / k : uint32_t(slot[t]) - n) : 0u;
                        img[t] = lds + lp.img_x + tt * LH.bytes(); src[t] = LdsBf16{xh + tt * H};
                    }
                    auto emit = [&](int t, float v) {
                        if (routed) store_act(p.act, uint32_t(slot[t]), row, v); else store_act(p.shared_act, uint32_t(slot[t]) - n, row, v);
                    };
                    run_tile(w_row, s_row, b_row, H / 128, img, src, LH, lane, nt, emit);
                }
                at = seg_end;
            }
        }
        clock_all();
        bar.wait();
        refresh();
        clock();
        // ---------------- phase D: down tiles, one contiguous range of (expert, row tile) per workgroup ----------------
        {
            const uint32_t row_tiles = H / 16, total = row_tiles * uint32_t(cum[U + 1]);
            uint32_t i0, i1;
            share_of_items(wg, nwg, total, kMultiWaves, i0, i1);
            uint16_t* ah = reinterpret_cast<uint16_t*>(lds + lp.ah);
            uint32_t ei = 0;
            while (ei < U && row_tiles * uint32_t(uniform(cum[ei + 1])) <= i0) ++ei;
            for (uint32_t at = i0; at < i1; ++ei) {
                const uint32_t first = row_tiles * uint32_t(uniform(cum[ei])), seg_end = min(i1, row_tiles * uint32_t(uniform(cum[ei + 1])));
                int32_t all[MT]; bool routed; uint32_t e;
                const int na = slots_of(ei, all, routed, e);
                __syncthreads();   // the previous segment's tiles have read their images
                // the slots' activations (packed BF16 rows of I elements) into LDS, then their images
                {
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
                for (uint32_t item = at + wave; item < seg_end; item += kMultiWaves) {
                    const uint32_t pass = pass_of_item(item - first, passes, kMultiWaves);
                    const uint32_t row = ((item - first) / passes) * 16 + col;
                    const uint8_t* w_row = rec + off[6] + uint64_t(row) * (I / 2);
                    const uint16_t* s_row = reinterpret_cast<const uint16_t*>(rec + off[7]) + uint64_t(row) * (I / 64);
                    const uint16_t* b_row = reinterpret_cast<const uint16_t*>(rec + off[8]) + uint64_t(row) * (I / 64);
                    int32_t slot[PT]; uint32_t index[PT];
                    const int nt = pass_of(all, na, pass, slot, index);
                    const uint8_t* img[PT]; LdsBf16 src[PT];
#pragma unroll
                    for (int t = 0; t < PT; ++t) { img[t] = lds + lp.img_d + index[t] * LI.bytes(); src[t] = LdsBf16{ah + index[t] * I}; }
                    auto emit = [&](int t, float v) { if (G == 0) st_f32(p.eout + uint64_t(slot[t]) * H + row, bf(v)); };
                    run_tile(w_row, s_row, b_row, I / 128, img, src, LI, lane, nt, emit);
                }
                at = seg_end;
            }
        }
        clock_all();
        bar.wait();
        refresh();
        clock();
        // ---------------- phase C: weighted combine (reference: qwen.metal:804-816), spread over the grid ----------------
        for (uint32_t group = wg + nwg * wave; group < T * H / 64; group += nwg * kMultiWaves) {   // 64 neighbouring columns of one token per wave
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
            // the lanes of a wave hold consecutive columns; a wave may straddle two tokens only when H is not a multiple of 64
            m = __float_as_uint(wave_max_f32(__uint_as_float(m)));
            if (lane == 0) ZC_ST(p.maxabs + group, m);   // group = t * (H / 64) + column group: read by the next layer's staging
        }
        clock_all();
        bar.wait();
        clock();
    }
}

static uint32_t align16m(uint32_t v) { return (v + 15u) / 16u * 16u; }

MultiLdsPlan decode_multi_lds_plan(uint32_t H, uint32_t E, uint32_t topk, uint32_t I, uint32_t T, uint32_t lds_limit) {
    MultiLdsPlan lp{};
    const XintLayout LH{H}, LI{I};
    uint32_t at = 0;
    auto take = [&](uint32_t bytes) { const uint32_t o = at; at += align16m(bytes); return o; };
    lp.ids = take(T * topk * 4); lp.weights = take(T * topk * 4); lp.gatev = take(kMultiTokens * 4);
    lp.head = take(E * 4); lp.next = take(E * kMultiTokens); lp.experts = take((2 * E > 128 * kMultiWaves ? 2 * E : 128 * kMultiWaves) * 4);
    lp.misc = take(64); lp.gatew = take(H * 2); lp.cum = take((T * topk + 3) * 4);
    lp.region = at;
    // phases R and G: the tokens' images and BF16 rows; phase D reuses the space for one expert's slots
    lp.img_x = lp.region; lp.xh = lp.img_x + T * LH.bytes();
    const uint32_t rg_end = lp.xh + align16m(T * H * 2);
    lp.img_d = lp.region; lp.ah = lp.img_d + T * LI.bytes();
    const uint32_t d_end = lp.ah + align16m(T * I * 2);
    lp.total = rg_end > d_end ? rg_end : d_end;
    // One workgroup per compute unit: more than half of the LDS, so that two can never share a unit while another idles.
    const uint32_t exclusive = lds_limit / 2 + 1024;
    if (lp.total < exclusive) lp.total = exclusive;
    return lp;
}

hipError_t launch_decode_multi(hipStream_t s, const DecodeParams& p, uint32_t workgroups, const MultiLdsPlan& lp) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(decode_multi_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lp.total));
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(decode_multi_kernel, dim3(workgroups), dim3(kMultiThreads), lp.total, s, p, lp);
    return hipGetLastError();
}
hipError_t decode_multi_occupancy(uint32_t lds_bytes, int* blocks_per_cu) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(decode_multi_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds_bytes));
    if (e != hipSuccess) return e;
    return hipOccupancyMaxActiveBlocksPerMultiprocessor(blocks_per_cu, decode_multi_kernel, kMultiThreads, lds_bytes);
}

}  // namespace zc
