/*
 * CPU oracle for the ZeroCool mixture-of-experts layer path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the arithmetic of
 * the reference's Metal kernels (kernels/metal/qwen.metal) and of the host
 * orchestration in src/engine/model.cpp:431-557 / src/engine/pipeline.cpp:7-31.
 * It is the checker for the HIP library and the CPU baseline that the benchmark
 * times next to the GPU.  Nothing in the product (the HIP library, its host
 * shim) includes, links or calls this file.
 *
 * Choices the reference leaves to Apple hardware and that this oracle FIXES:
 *   - simd_sum over the 32 reference lanes: xor butterfly with strides
 *     16, 8, 4, 2, 1 (lane l adds lane l^stride at every step).
 *   - exp: one fp32 algorithm (zco_expf), used for both precise::exp
 *     (sigmoid_bf) and fast::exp (route softmax).
 *   - no fused multiply-add except inside the router MAC chain (where products
 *     of BF16-valued operands are exact, so fusing cannot change a bit).
 *
 * Parity pins (tests/test_oracle_golden.py):
 *   bf/b16            closed form  (tests/test_qwen.cpp:277-283)
 *   sigmoid_bf, SiLU  64-point captured tables + boundary (…:876-897)
 *   affine Q4 value   double-precision brute force (…:634-652)
 *   Q4 bias rounding  special case -> exactly 0 (…:863-874)
 *   SwiGLU epilogue   closed-form identity (…:653-659)
 *   affine Q8         exact equality with double dot (…:661-683)
 *   router logits     16 captured fp32 words (…:798-826)
 *   route ids         stable-sort brute force incl. NaN/inf/ties (…:744-797)
 *   moe_sum           captured BF16 midpoint value (…:827-842)
 *   dispatch/scatter  brute force (…:1500-1533)
 *   plain_mm          double precision within the fp32 bound on the reference's four
 *                     shapes (…:1126-1135), and exact closed forms that hold only for
 *                     the lane chain k = lane + 32 j (2^24 / 1 absorption rows)
 *   Q4 lane widths    exact closed forms that tell sixteen-element lane steps from
 *                     eight-element ones, and the every-32nd-block revisit, bit for bit
 *   route softmax     weight VALUES against a float64 softmax over the ten selected
 *                     scores, relative 1e-6 (random, spread, tied and near-tied rows, the
 *                     reference's ramp, a closed form with three finite scores); the
 *                     swapped subtraction is shown to miss; zco_expf against double
 *                     precision, relative 2e-7.  (qwen.metal:758-764)
 *   Still unpinned at BIT level (only an Apple GPU run could pin them): the last
 *   bits of the softmax weights (Metal fast::exp) and the final simd_sum association
 *   of the affine dots.  Both sit far inside the 2e-3 layer tolerance.
 *
 * The callers' glue either side of the layer (tests/test_oracle_glue.py):
 *   softplus, unary   64-point captured softplus table, exact (…:881); ops 2 and 3
 *                     as compositions of the pinned SiLU / sigmoid
 *   log in softplus   correctly rounded fp32 logarithm on a 1001-point grid
 *   binary, hc_mix,   explicit loops with a BF16 rounding after every operation
 *   hc_add
 *   norm              double precision within two BF16 roundings, closed forms, and
 *                     a row whose block sums depend on the order of additions;
 *                     precise::rsqrt (taken as 1/sqrt) and the lane-sum association:
 *                     parity unpinned (the reference tests norm only against norm_wide)
 */
#ifndef ZC_ORACLE_H
#define ZC_ORACLE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* qwen.metal:17-22, storage.cpp:29-35 */
float zco_bf(float x);
float zco_b16(uint16_t h);
uint16_t zco_bf_bits(float x);
/* qwen.metal:33-35 */
float zco_expf(float x);
float zco_sigmoid_bf(float x);

/* One projection: packed codes + BF16 scales/biases, row-major [N][K]. */
typedef struct {
    const void* weight;      /* Q4: uint32 words, nibble i of word w = element 8w+i; Q8: bytes */
    const uint16_t* scales;  /* [N][K/group] BF16 */
    const uint16_t* biases;  /* [N][K/group] BF16 */
    uint32_t input, output, group, bits;
} zco_linear_t;

/* qwen.metal:46-62 (bits 4) and :112-125 (bits 8): one output row, one token. */
float zco_affine_dot(const zco_linear_t* l, const float* x, uint32_t row);
/* qwen.metal:63-70 / :126-133: out[t*N+n] = float_output ? s : bf(s) */
void zco_linear(const zco_linear_t* l, const float* x, uint32_t tokens, float* out, int float_output);
/* qwen.metal:71-81 / :134-144: rows may be NULL (identity gather). */
void zco_gated_linear(const zco_linear_t* gate, const zco_linear_t* up, const float* x,
                      uint32_t tokens, const int32_t* rows, float* out);
/* qwen.metal:499-506; dtype 0 = BF16, 1 = F32. */
void zco_plain_mm(const void* w, uint32_t dtype, const float* x, uint32_t K, uint32_t N,
                  uint32_t tokens, float* out, int float_output);
/* qwen.metal:512-534 + metal.mm:818-822: 16 contiguous K splits. offsets (may be
 * NULL) is a per-expert fp32 value added to the finished logit; it is the synthetic
 * load-skew knob of the benchmark workloads, not part of the reference. */
void zco_router_logits(const uint16_t* w, const float* x, uint32_t tokens, uint32_t K,
                       uint32_t E, const float* offsets, float* out);
/* qwen.metal:742-795 */
void zco_route(const float* logits, uint32_t tokens, uint32_t E, uint32_t topk,
               int32_t* ids, float* weights);
/* model.cpp:449-479: stable counting sort of flat slots by expert.
 * offsets[E+1], slots[tokens*topk], selected[<=E]; returns number of selected
 * experts, or -1 on an id outside [0,E) ("invalid router output"). */
int zco_dispatch(const int32_t* ids, uint32_t tokens, uint32_t topk, uint32_t E,
                 int32_t* offsets, int32_t* slots, int32_t* selected);
/* qwen.metal:800-803 */
void zco_scatter_experts(const float* x, const int32_t* positions, uint32_t n, uint32_t H, float* out);
/* qwen.metal:804-816 (general topk: partial j = k mod 8 accumulates k ascending,
 * then partials are added 0..7; topk 10 gives exactly the reference expression). */
void zco_moe_sum(const float* experts, const float* weights, const float* shared,
                 const float* gate, uint32_t tokens, uint32_t H, uint32_t topk, float* out);

/* The callers' glue either side of the layer (model.cpp:328-351, 651, 662): element-wise operators, the
 * four-stream mix and residual injection, grouped RMS norm. */
float zco_log_1to2(float y);
float zco_softplus_bf(float x);                                                       /* qwen.metal:36-40 */
float zco_unary(float v, uint32_t op);                                                /* qwen.metal:567-577 */
void zco_unary_n(const float* x, uint64_t n, uint32_t op, float* y);
void zco_binary_n(const float* x, const float* y, uint64_t n, uint32_t op, float* out);   /* qwen.metal:578-581 */
void zco_hc_mix(const float* x, const float* w, uint32_t tokens, uint32_t hidden, float* out);   /* qwen.metal:582-588 */
void zco_hc_add(const float* hyper, const float* x, const float* inject, uint32_t tokens, uint32_t hidden, float* out);   /* qwen.metal:589-595 */
void zco_norm(const float* x, const void* w, uint32_t dtype, uint32_t D, uint32_t width, uint32_t tokens, float* out);    /* qwen.metal:545-566 */

/* A whole layer (model.cpp:431-557). */
typedef struct {
    uint32_t hidden, experts, topk, inter, group;
    uint32_t bits_gate_up, bits_down;              /* routed experts */
    uint32_t shared_bits_gate_up, shared_bits_down; /* shared expert */
} zco_config_t;
typedef struct {
    const uint16_t* router;       /* [E][H] BF16 */
    const float* router_offsets;  /* [E] or NULL */
    const uint16_t* shared_gate;  /* [1][H] BF16 (shared_expert_gate) */
    const uint8_t* shared_record; /* gate,up,down projections of the shared expert */
    const uint8_t* expert_records;/* E records, record_stride apart */
    uint64_t record_stride;
} zco_layer_t;
typedef struct {               /* optional intermediates, any may be NULL */
    float* logits;  int32_t* ids;  float* weights;
    float* expert_out; float* shared; float* gate;
} zco_trace_t;
uint64_t zco_projection_bytes(uint32_t K, uint32_t N, uint32_t group, uint32_t bits);
uint64_t zco_record_bytes(const zco_config_t* c, int shared);
/* metal.mm:1124-1129 generalised: projection 0 gate, 1 up, 2 down. */
void zco_expert_linear(const zco_config_t* c, int shared, const uint8_t* record, int projection, zco_linear_t* out);
/* returns 0, or -1 for an invalid router output. threads<=1: serial. */
int zco_moe_layer(const zco_config_t* c, const zco_layer_t* l, const float* x, uint32_t tokens,
                  float* out, zco_trace_t* trace, int threads);
#ifdef __cplusplus
}
#endif
#endif
