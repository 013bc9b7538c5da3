// Host-side launchers of the MoE-path kernels.  Each only enqueues on `s`.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/zc_hip.h"

namespace zc {

struct AffineDesc {
    zc_linear gate, up;          // up used only when gated
    bool gated = false;
    const float* x = nullptr;
    const int32_t* in_rows = nullptr;
    const int32_t* out_rows = nullptr;
    float* out = nullptr;
    uint32_t tokens = 0;
    uint32_t float_output = 0;
};
void launch_affine(hipStream_t s, const AffineDesc& a);          // literal lane arithmetic, any shape
bool xint_supported(const zc_linear& l);                          // wide affine Q4, group 64, 16-byte aligned
void launch_affine_xint(hipStream_t s, const AffineDesc& a);     // exact-integer matrix-core form

struct ExpertPhaseDesc {
    const void* records; uint64_t stride;
    uint64_t off[6];             // w,s,b of the first matrix, then of the second (gate/up phase)
    const int32_t *offsets, *selected, *count, *in_rows, *out_rows;
    const float* x; float* out;
    uint32_t K, N, group, bits, x_sorted, max_jobs;
    bool gated;
};
void launch_expert_phase(hipStream_t s, const ExpertPhaseDesc& d);

void launch_plain(hipStream_t s, const void* w, uint32_t dtype, const float* x, uint32_t K, uint32_t N,
                  uint32_t tokens, float* out, bool float_output);
void launch_router(hipStream_t s, const void* w, const float* x, uint32_t T, uint32_t K, uint32_t E,
                   const float* offsets, float* out);
void launch_route(hipStream_t s, const float* logits, uint32_t T, uint32_t E, uint32_t topk, int32_t* ids, float* weights);
void launch_dispatch(hipStream_t s, const int32_t* ids, uint32_t tokens, uint32_t topk, uint32_t E, int32_t* offsets,
                     int32_t* slots, int32_t* rows, int32_t* selected, int32_t* count, int32_t* status);
void launch_scatter(hipStream_t s, const float* x, const int32_t* positions, uint32_t n, uint32_t H, float* out);
// ---- the callers' glue either side of the layer (zc_glue.hip)
void launch_unary(hipStream_t s, const float* x, uint64_t n, uint32_t op, float* y);
void launch_binary(hipStream_t s, const float* x, const float* y, uint64_t n, uint32_t op, float* out);
void launch_hc_mix(hipStream_t s, const float* x, const float* w, uint32_t tokens, uint32_t hidden, float* out);
void launch_hc_add(hipStream_t s, const float* hyper, const float* x, const float* inject, uint32_t tokens, uint32_t hidden, float* out);
void launch_norm(hipStream_t s, const float* x, const void* w, uint32_t dtype, uint32_t D, uint32_t width, uint32_t tokens, float* out);
void launch_moe_sum(hipStream_t s, const float* experts, const float* weights, const float* shared, const float* gate,
                    uint32_t T, uint32_t H, uint32_t topk, float* out);
void launch_moe_sum_half(hipStream_t s, const uint16_t* experts, const float* weights, const float* shared, const float* gate,
                         uint32_t T, uint32_t H, uint32_t topk, float* out);
void launch_stack_glue(hipStream_t s, const float* y, uint32_t T, uint32_t H, float* out);
void launch_synth_words(hipStream_t s, uint32_t* dst, uint64_t count, uint64_t seed);
void launch_synth_scales(hipStream_t s, uint16_t* sc, uint16_t* bi, uint64_t count, uint64_t seed, float lo, float span, float factor);
void launch_synth_normal(hipStream_t s, void* dst, uint64_t count, uint64_t seed, float sigma, bool half);
void launch_synth_records(hipStream_t s, void* records, uint64_t stride, uint32_t count, const uint64_t* w_off,
                          const uint64_t* s_off, const uint64_t* words, const uint64_t* meta, const uint32_t* bits, uint64_t seed);


// Persistent stacked decode (zc_decode.hip)
struct DecodeLayer {
    const uint16_t* router; const float* offsets; const uint16_t* shared_gate;
    const uint8_t* shared_record; const uint8_t* records; uint64_t stride;
    const uint8_t* const* table;   // if set: expert e's record is at table[e] (an expert store's view); else at records + e * stride
};
struct DecodeParams {
    uint32_t H, E, topk, I, T, L;
    uint32_t bits_down, shared_bits_gate_up, shared_bits_down;   // 4 or 8 (routed gate/up is always 4 in these kernels); 8: literal lanes, one token only
    uint64_t ro[9], so[9];           // byte offsets [projection*3 + {codes, scales, biases}] in a routed / shared record
    const DecodeLayer* layers;       // device array [L]
    const float* x_in; float* out;   // [T][H]
    float *logits, *gate, *shared_act, *act, *layer_out;   // exchange buffers
    float* eout;                     // several tokens: down outputs per slot, [T * topk + T][H] (the last T rows: the shared expert's)
    uint32_t* maxabs;                // [L][T] bit patterns of max |layer output|
    // One token: the exchange buffers carry a tag beside every value, so that a reader polls the data itself instead of
    // waiting at a grid barrier and fetching afterwards.  tlogits [E + 1] words {fp32 bits, tag << 32} (word E: the shared
    // gate dot); tact [topk + 1][I] and tout [2][H] words {BF16 value << 16 | 16-bit tag}.  All zero before the first launch.
    unsigned long long* tlogits; uint32_t *tact, *tout;
    // One token, optional: pred_in [L][topk] = the ids every layer picked at the previous step (its gate/up tiles start on them
    // before this step's ids are known), pred_out [L][topk] receives this step's; tspec [topk + 1][I]: the prediction pass's
    // activations, tagged like tact.
    const int32_t* pred_in; int32_t* pred_out; uint32_t* tspec;
    int32_t* route_ids; float* route_weights;   // nine to sixty-four tokens: [T][topk] routes, written by the routing waves, read by every workgroup
    int32_t* ids_trace; float* weights_trace; float* out_trace;   // optional [L][trace_tokens][topk], [L][trace_tokens][topk], [L][trace_tokens][H],
    uint32_t trace_tokens;           // each already advanced to this launch's first token: a launch may be one piece of a larger batch
    uint32_t* sync; uint32_t epoch; int32_t* status; uint32_t spin_limit;
    uint32_t tag_base;               // one token: layer l exchanges under tag (tag_base + l) % 65535 + 1; advances only with one-token launches
    unsigned long long* clocks;      // optional [L * kDecodeStamps][workgroups] 100 MHz timestamps, one per workgroup
};
constexpr uint32_t kDecodeStamps = 24;
struct DecodeLdsPlan {
    uint32_t ids, weights, gatev, experts, misc, region, total;
    uint32_t img_rg, xh, gprod, img_d, ah, otile, slots_per_batch, gatew, spec;
};
DecodeLdsPlan decode_lds_plan(uint32_t H, uint32_t E, uint32_t topk, uint32_t I, uint32_t NT, uint32_t lds_limit);
hipError_t launch_decode_stack(hipStream_t s, const DecodeParams& p, uint32_t nt, uint32_t workgroups, const DecodeLdsPlan& lp);
hipError_t decode_stack_occupancy(uint32_t nt, uint32_t lds_bytes, int* blocks_per_cu);
constexpr uint32_t kDecodeSyncBytes = (32 * 1024 + 16 * 64) * 4;
// Two to eight tokens (zc_decode_multi.hip)
struct MultiLdsPlan {
    uint32_t ids, weights, gatev, head, next, experts, misc, gatew, region, total;
    uint32_t img_x, xh, img_d, ah, cum;
};
MultiLdsPlan decode_multi_lds_plan(uint32_t H, uint32_t E, uint32_t topk, uint32_t I, uint32_t T, uint32_t lds_limit);
hipError_t launch_decode_multi(hipStream_t s, const DecodeParams& p, uint32_t workgroups, const MultiLdsPlan& lp);
hipError_t decode_multi_occupancy(uint32_t lds_bytes, int* blocks_per_cu);

// Nine to sixty-four tokens (zc_decode_wide.hip)
struct WideLdsPlan {
    uint32_t ids, weights, gatev, gscale, chosen, entries, cum, misc, gatew, region, total;
    uint32_t img_x, xh, img_d, ah;
};
WideLdsPlan decode_wide_lds_plan(uint32_t H, uint32_t E, uint32_t topk, uint32_t I, uint32_t T, uint32_t lds_limit);
hipError_t launch_decode_wide(hipStream_t s, const DecodeParams& p, uint32_t workgroups, const WideLdsPlan& lp);
hipError_t decode_wide_occupancy(uint32_t lds_bytes, int* blocks_per_cu);

// ---- prefill: sorted-token grouped GEMM on the bf16 matrix cores (zc_prefill.hip)
struct PrefillGemm {
    const uint16_t* a;        // bf16 rows [.][K]
    const float* asum;        // per (row, group of 64): sum of the blocks' BF16-rounded sum-of-four chains
    const float* asum16;      // per (row, block of 16): that block's chain sum (read by the recomputation; null: formed there)
    const int32_t* a_rows;    // row of `a` for sorted position pos: a_rows ? a_rows[pos] / a_div : pos
    uint32_t a_div;
    const int32_t* out_rows;  // output row for sorted position pos: out_rows ? out_rows[pos] : pos   (down projection)
    const uint8_t* records; uint64_t stride;   // expert e's record at records + e * stride
    uint64_t off[6];          // byte offsets in a record: codes, scales, biases of the (gate | down) projection, then of up
    const int32_t *tile_expert, *tile_first, *tile_rows, *tile_count;
    uint32_t K, N;            // reduction length, rows of ONE projection
    uint32_t bits;            // 4: nibble codes, asum = the Q4 lanes' BF16-rounded sum-of-four chains; 8: byte codes, asum = the Q8 lanes' plain sums
    uint16_t* out_b;          // gate/up: SwiGLU activations as bf16 [sorted position][N]
    float* out_f;             // down: BF16-rounded fp32 [output row][N]
    uint16_t* out_h;          // down, instead of out_f when not null: the same values as bf16 (what the combine reads is half as long)
    // Sums that land within near_margin * (sum of term magnitudes) of a BF16 rounding boundary are marked in a bit map
    // (bit sorted position * N + row; near_words 32-bit words, all written by the product kernel)
    // and recomputed afterwards with the reference's exact lane arithmetic (launch_prefill_patch).
    uint32_t* near_bits; uint32_t near_words; float near_margin;
    const int32_t* ids;       // expert of sorted position pos: ids ? ids[slots[pos]] : 0 (used by the recomputation)
    const int32_t* slots;
    // Sorted positions the product kernel covered: positions below *covered (the dispatch's offsets[experts]; an id
    // outside [0, experts) leaves the tail uncovered and its map words unwritten) or, when covered is null, all of them.
    const int32_t* covered; uint32_t experts;
};
// Margin of the recomputation, as a fraction of the summed term magnitudes (those of the scale groups' sums: what cancels
// inside a group is not seen).  Rows of fewer than 8 groups keep 2^-22, four fp32 steps: with few groups the additions
// inside a group weigh most, and a flip was seen at two groups with half of that.  From 8 to 32 groups the margin is
// 2^-23 (the largest distance seen between the two orders of additions, on rows of 8 and of 32 groups, is a quarter of it),
// beyond that 2^-28 per group (2^-22 again at 64): the distance grows with the number of additions.
constexpr float prefill_margin(uint32_t K) { return K / 64 < 8 ? 0x1p-22f : (K / 64 <= 32 ? 0x1p-23f : float(K / 64) * 0x1p-28f); }
void launch_prefill_rows(hipStream_t s, const float* x, uint32_t rows, uint32_t K, uint16_t* xb, float* sums, float* sums16, float* plain, int32_t* status);
// ids / weights not null (topk <= 64): the selection runs in the same launch and the logits are not written
void launch_prefill_router(hipStream_t s, const float* x, const uint16_t* xb, const void* w, const float* offsets, uint32_t T, uint32_t K,
                           uint32_t E, uint32_t topk, float* norms, float* logits, int32_t* ids, float* weights);
void launch_prefill_sums(hipStream_t s, const uint16_t* xb, const int32_t* rows_ptr, uint32_t rows_max, uint32_t K, float* sums, float* sums16, bool plain);
void launch_prefill_dispatch(hipStream_t s, const int32_t* ids, uint32_t tokens, uint32_t topk, uint32_t E, int32_t* offsets, int32_t* slots, int32_t* rows,
                             int32_t* status, int32_t* tile_expert, int32_t* tile_first, int32_t* tile_rows, int32_t* tile_count);
bool prefill_dispatch_fits(const int32_t* ids, uint32_t tokens, uint32_t topk, uint32_t E);
void launch_prefill_tiles(hipStream_t s, const int32_t* offsets, uint32_t experts, uint32_t rows, int32_t* tile_expert, int32_t* tile_first,
                          int32_t* tile_rows, int32_t* tile_count);
void launch_prefill_gemm(hipStream_t s, const PrefillGemm& p, bool gated, uint32_t max_tiles);
void launch_prefill_patch(hipStream_t s, const PrefillGemm& p, bool gated);
bool prefill_shape(uint32_t hidden, uint32_t inter, uint32_t experts);

}  // namespace zc
