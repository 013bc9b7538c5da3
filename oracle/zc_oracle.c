/*
 * CPU oracle for the ZeroCool MoE-layer path: see zc_oracle.h for what it is,
 * what it pins and what it fixes.  TEST INFRASTRUCTURE ONLY.
 *
 * Build: gcc -O3 -fno-fast-math -ffp-contract=off -fopenmp (see Makefile).
 * -ffp-contract=off is part of the definition: every a*b+c below is two
 * roundings unless written as fmaf().
 */
#include "zc_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ZCO_LANES 32u /* the reference SIMD-group width; part of the arithmetic */

static inline uint32_t f2u(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static inline float u2f(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

/* qwen.metal:17-21; storage.cpp:30-35 */
float zco_bf(float x) {
    uint32_t u = f2u(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return NAN;
    return u2f((u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u);
}
uint16_t zco_bf_bits(float x) { return (uint16_t)(f2u(zco_bf(x)) >> 16); }
/* qwen.metal:22 */
float zco_b16(uint16_t h) { return u2f((uint32_t)h << 16); }

/*
 * exp in fp32: n = rint(x*log2(e)); r = x - n*ln2 (two-constant Cody-Waite);
 * degree-5 polynomial on r*r (Cephes expf coefficients); scale by 2^n in two
 * exact power-of-two steps.  Inputs below -87 give 0 so no result is subnormal.
 * Stands in for Metal's precise::exp (qwen.metal:34) and fast::exp (:760).
 */
float zco_expf(float x) {
    if (x != x) return x;
    if (x > 88.72283f) return INFINITY;
    if (x < -87.0f) return 0.0f;
    float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693359375f, x);
    r = fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    float y = fmaf(p, r * r, r) + 1.0f;
    int ni = (int)n, a = ni / 2, b = ni - a;
    return y * u2f((uint32_t)(a + 127) << 23) * u2f((uint32_t)(b + 127) << 23);
}
/* qwen.metal:33-35 */
float zco_sigmoid_bf(float x) {
    float y = zco_bf(1.0f / zco_bf(1.0f + zco_bf(zco_expf(fabsf(x)))));
    return x < 0 ? y : zco_bf(1.0f - y);
}

/*
 * log(y) for y in [1, 2], evaluated in double from basic operations only (division, fused multiply-add), so the
 * device computes the same bits: log y = 2 atanh z, z = (y-1)/(y+1) <= 1/3, odd series to z^35.  Rounded to
 * fp32 once.  Stands in for Metal's log in softplus_bf (qwen.metal:36-40).
 */
float zco_log_1to2(float y) {
    const double z = ((double)y - 1.0) / ((double)y + 1.0), z2 = z * z;
    double p = 1.0 / 35.0;
    for (int k = 33; k >= 1; k -= 2) p = fma(p, z2, 1.0 / (double)k);
    return (float)(2.0 * z * p);
}
/* qwen.metal:36-40 */
float zco_softplus_bf(float x) {
    const float e = zco_bf(zco_expf(-fabsf(x))), one = 1.0f + e;
    const float tail = one == 1.0f ? e : e * (zco_log_1to2(one) / (one - 1.0f));
    return zco_bf(fmaxf(x, 0.0f) + zco_bf(tail));
}
/* kernel unary (qwen.metal:567-577): 0 SiLU, 1 sigmoid, 2 SiLU(x/4), 3 2*sigmoid(x/4), 4 softplus */
float zco_unary(float v, uint32_t op) {
    if (op == 0) v = v * zco_sigmoid_bf(v);
    if (op == 1) v = zco_sigmoid_bf(v);
    if (op == 2) { v = zco_bf(v / 4); v = v * zco_sigmoid_bf(v); }
    if (op == 3) v = 2 * zco_bf(zco_sigmoid_bf(zco_bf(v / 4)));
    if (op == 4) v = zco_softplus_bf(v);
    return zco_bf(v);
}
void zco_unary_n(const float* x, uint64_t n, uint32_t op, float* y) { for (uint64_t i = 0; i < n; ++i) y[i] = zco_unary(x[i], op); }
/* kernel binary (qwen.metal:578-581): op 0 add, otherwise multiply */
void zco_binary_n(const float* x, const float* y, uint64_t n, uint32_t op, float* out) {
    for (uint64_t i = 0; i < n; ++i) out[i] = zco_bf(op ? x[i] * y[i] : x[i] + y[i]);
}
/* kernel hc_mix (qwen.metal:582-588): x, w are [tokens][4][hidden]; BF16 rounding of every product and partial sum */
void zco_hc_mix(const float* x, const float* w, uint32_t tokens, uint32_t hidden, float* out) {
    for (uint32_t t = 0; t < tokens; ++t)
        for (uint32_t d = 0; d < hidden; ++d) {
            float sum = 0;
            for (uint32_t h = 0; h < 4; ++h) { const uint64_t k = ((uint64_t)t * 4 + h) * hidden + d; sum = zco_bf(sum + zco_bf(x[k] * w[k])); }
            out[(uint64_t)t * hidden + d] = zco_bf(sum / 4);
        }
}
/* kernel hc_add (qwen.metal:589-595): hyper [tokens][4][hidden], x [tokens][hidden], inject [tokens][4] */
void zco_hc_add(const float* hyper, const float* x, const float* inject, uint32_t tokens, uint32_t hidden, float* out) {
    for (uint32_t t = 0; t < tokens; ++t)
        for (uint32_t h = 0; h < 4; ++h)
            for (uint32_t d = 0; d < hidden; ++d) {
                const uint64_t k = ((uint64_t)t * 4 + h) * hidden + d;
                out[k] = zco_bf(hyper[k] + zco_bf(x[(uint64_t)t * hidden + d] * inject[t * 4 + h]));
            }
}

/* The fixed association this oracle gives simd_sum: xor butterfly 16,8,4,2,1. */
static float simd_sum(float* lane) {
    for (uint32_t stride = ZCO_LANES / 2; stride; stride >>= 1)
        for (uint32_t l = 0; l < stride; ++l) lane[l] = lane[l] + lane[l + stride];
    return lane[0];
}
/* rms_square_sum + kernel norm (qwen.metal:545-566): grouped RMS norm, D <= 4096 per group.  Each 128-element
 * block gives every lane a sum of four squares, a lane sum, and lane block/128 keeps it; a second lane sum adds the
 * blocks.  precise::rsqrt is taken as 1 / sqrt (two correctly rounded operations).  w: dtype 0 BF16, 1 fp32. */
void zco_norm(const float* x, const void* w, uint32_t dtype, uint32_t D, uint32_t width, uint32_t tokens, float* out) {
    const uint64_t groups = (uint64_t)tokens * (width / D);
    for (uint64_t g = 0; g < groups; ++g) {
        const float* xg = x + g * D;
        float contribution[32] = {0};
        for (uint32_t block = 0; block < D; block += 128) {
            float acc[32];
            for (uint32_t lane = 0; lane < 32; ++lane) {
                acc[lane] = 0;
                for (uint32_t i = 0; i < 4; ++i) { const uint32_t d = block + lane * 4 + i; if (d < D) acc[lane] += xg[d] * xg[d]; }
            }
            contribution[block / 128] = simd_sum(acc);
        }
        const float inv = 1.0f / sqrtf(simd_sum(contribution) / (float)D + 1e-6f);
        for (uint32_t d = 0; d < D; ++d) {
            const uint64_t i = g * D + d; const uint32_t wi = (uint32_t)(i % width);
            const float weight = dtype == 1 ? ((const float*)w)[wi] : zco_b16(((const uint16_t*)w)[wi]);
            out[i] = zco_bf(zco_bf(xg[d] * inv) * weight);
        }
    }
}
/* Note: lane l and lane l^stride compute the same commutative sum, so keeping
 * only the lower half at every step gives lane 0's butterfly value exactly. */

/* qwen.metal:46-62 */
static float affine_dot_q4(const zco_linear_t* l, const float* x, uint32_t row) {
    const uint32_t K = l->input, N = l->output;
    const uint32_t width = (K % 512 == 0 && N % 8 == 0) ? 16 : 8;
    const uint32_t* w = (const uint32_t*)l->weight;
    float lanes[ZCO_LANES];
    for (uint32_t lane = 0; lane < ZCO_LANES; ++lane) {
        float result = 0;
        for (uint32_t base = lane * width; base < K; base += ZCO_LANES * width) {
            float dot = 0, sum = 0;
            for (uint32_t i = 0; i < width && base + i < K; i += 4) {
                uint32_t k = base + i, packed = (w[row * (K / 8) + k / 8] >> (4 * (k % 8))) & 0xffff;
                float a = x[k], c = x[k + 1], d = x[k + 2], e = x[k + 3];
                sum += zco_bf(zco_bf(zco_bf(a + c) + d) + e);
                dot += a * (float)(packed & 15) + c * (float)((packed >> 4) & 15) +
                       d * (float)((packed >> 8) & 15) + e * (float)((packed >> 12) & 15);
            }
            uint32_t g = row * (K / l->group) + base / l->group;
            result += zco_b16(l->scales[g]) * dot + sum * zco_b16(l->biases[g]);
        }
        lanes[lane] = result;
    }
    return simd_sum(lanes);
}
/* qwen.metal:112-125 */
static float affine_dot_q8(const zco_linear_t* l, const float* x, uint32_t row) {
    const uint32_t K = l->input, N = l->output;
    const uint32_t width = (K % 512 == 0 && N % 8 == 0) ? 8 : 4;
    const uint8_t* w = (const uint8_t*)l->weight;
    float lanes[ZCO_LANES];
    for (uint32_t lane = 0; lane < ZCO_LANES; ++lane) {
        float result = 0;
        for (uint32_t base = lane * width; base < K; base += ZCO_LANES * width) {
            float dot = 0, sum = 0;
            for (uint32_t i = 0; i < width && base + i < K; ++i) {
                float value = x[base + i];
                sum += value;
                dot += value * (float)w[(uint64_t)row * K + base + i];
            }
            uint32_t g = row * (K / l->group) + base / l->group;
            result += zco_b16(l->scales[g]) * dot + sum * zco_b16(l->biases[g]);
        }
        lanes[lane] = result;
    }
    return simd_sum(lanes);
}
float zco_affine_dot(const zco_linear_t* l, const float* x, uint32_t row) {
    return l->bits == 8 ? affine_dot_q8(l, x, row) : affine_dot_q4(l, x, row);
}

/* qwen.metal:63-70, 126-133 */
void zco_linear(const zco_linear_t* l, const float* x, uint32_t tokens, float* out, int float_output) {
    const uint32_t K = l->input, N = l->output;
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t t = 0; t < tokens; ++t)
        for (uint32_t n = 0; n < N; ++n) {
            float s = zco_affine_dot(l, x + (uint64_t)t * K, n);
            out[(uint64_t)t * N + n] = float_output ? s : zco_bf(s);
        }
}
/* qwen.metal:71-81, 134-144 */
void zco_gated_linear(const zco_linear_t* gate, const zco_linear_t* up, const float* x,
                      uint32_t tokens, const int32_t* rows, float* out) {
    const uint32_t K = gate->input, N = gate->output;
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t t = 0; t < tokens; ++t)
        for (uint32_t n = 0; n < N; ++n) {
            const float* xr = x + (uint64_t)(rows ? (uint32_t)rows[t] : t) * K;
            float g = zco_bf(zco_affine_dot(gate, xr, n));
            float u = zco_bf(zco_affine_dot(up, xr, n));
            out[(uint64_t)t * N + n] = zco_bf(zco_bf(g * zco_sigmoid_bf(g)) * u);
        }
}
/* qwen.metal:499-506 (and plain_mv :382-398, the same lane chain) */
void zco_plain_mm(const void* w, uint32_t dtype, const float* x, uint32_t K, uint32_t N,
                  uint32_t tokens, float* out, int float_output) {
    for (uint32_t t = 0; t < tokens; ++t)
        for (uint32_t n = 0; n < N; ++n) {
            float lanes[ZCO_LANES];
            for (uint32_t lane = 0; lane < ZCO_LANES; ++lane) {
                float sum = 0;
                for (uint32_t k = lane; k < K; k += ZCO_LANES) {
                    float wv = dtype == 1 ? ((const float*)w)[(uint64_t)n * K + k]
                                          : zco_b16(((const uint16_t*)w)[(uint64_t)n * K + k]);
                    sum += x[(uint64_t)t * K + k] * wv;
                }
                lanes[lane] = sum;
            }
            float s = simd_sum(lanes);
            out[(uint64_t)t * N + n] = float_output ? s : zco_bf(s);
        }
}

/*
 * qwen.metal:512-534, metal.mm:818-822.  The 8x8 simdgroup MAC's internal order
 * is resolved by the reference's 16 captured words (tests/test_qwen.cpp:810-813):
 * only a k-ascending multiply-accumulate chain inside each of the 16 contiguous
 * K partitions, partitions then added 0..15 starting from 0.0f, reproduces them.
 */
void zco_router_logits(const uint16_t* w, const float* x, uint32_t tokens, uint32_t K,
                       uint32_t E, const float* offsets, float* out) {
    const uint32_t P = K / 16;
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t t = 0; t < tokens; ++t)
        for (uint32_t e = 0; e < E; ++e) {
            float sum = 0;
            for (uint32_t s = 0; s < 16; ++s) {
                float c = 0;
                for (uint32_t k = s * P; k < (s + 1) * P; ++k)
                    c = fmaf(x[(uint64_t)t * K + k], zco_b16(w[(uint64_t)e * K + k]), c);
                sum += c;
            }
            out[(uint64_t)t * E + e] = offsets ? sum + offsets[e] : sum;
        }
}

/* qwen.metal:742-765 (serial) == :768-795 (simd): same ids, scores, weights. */
void zco_route(const float* logits, uint32_t tokens, uint32_t E, uint32_t topk,
               int32_t* ids, float* weights) {
    for (uint32_t t = 0; t < tokens; ++t) {
        const float* v = logits + (uint64_t)t * E;
        float scores[128];
        int32_t selected[128];
        for (uint32_t j = 0; j < topk; ++j) { scores[j] = -INFINITY; selected[j] = -1; }
        for (int32_t e = 0; e < (int32_t)E; ++e) {
            float value = v[e];
            for (uint32_t j = 0; j < topk; ++j)
                if (value > scores[j]) {
                    for (uint32_t k = topk - 1; k > j; --k) { scores[k] = scores[k - 1]; selected[k] = selected[k - 1]; }
                    scores[j] = value; selected[j] = e; break;
                }
        }
        /* four values per lane, simd_sum, one reciprocal (qwen.metal:758-764) */
        float lanes[ZCO_LANES], values[128];
        for (uint32_t lane = 0; lane < ZCO_LANES; ++lane) {
            float sum = 0;
            for (uint32_t i = 0; i < 4; ++i) {
                uint32_t j = lane * 4 + i;
                float value = j < topk ? zco_expf(scores[j] - scores[0]) : 0;
                if (j < topk) values[j] = value;
                sum += value;
            }
            lanes[lane] = sum;
        }
        float inverse = 1.0f / simd_sum(lanes);
        for (uint32_t j = 0; j < topk; ++j) {
            ids[(uint64_t)t * topk + j] = selected[j];
            weights[(uint64_t)t * topk + j] = values[j] * inverse;
        }
    }
}

/* model.cpp:449-479 */
int zco_dispatch(const int32_t* ids, uint32_t tokens, uint32_t topk, uint32_t E,
                 int32_t* offsets, int32_t* slots, int32_t* selected) {
    const uint32_t n = tokens * topk;
    memset(offsets, 0, (E + 1) * sizeof(int32_t));
    for (uint32_t p = 0; p < n; ++p) {
        if (ids[p] < 0 || ids[p] >= (int32_t)E) return -1;
        ++offsets[ids[p] + 1];
    }
    for (uint32_t e = 0; e < E; ++e) offsets[e + 1] += offsets[e];
    int32_t* cursor = (int32_t*)malloc(E * sizeof(int32_t));
    memcpy(cursor, offsets, E * sizeof(int32_t));
    for (uint32_t p = 0; p < n; ++p) slots[cursor[ids[p]]++] = (int32_t)p;
    free(cursor);
    int count = 0;
    for (uint32_t e = 0; e < E; ++e) if (offsets[e + 1] > offsets[e]) selected[count++] = (int32_t)e;
    return count;
}
/* qwen.metal:800-803 */
void zco_scatter_experts(const float* x, const int32_t* positions, uint32_t n, uint32_t H, float* out) {
    for (uint32_t r = 0; r < n; ++r)
        memcpy(out + (uint64_t)positions[r] * H, x + (uint64_t)r * H, (size_t)H * 4);
}
/* qwen.metal:804-816 */
void zco_moe_sum(const float* experts, const float* weights, const float* shared,
                 const float* gate, uint32_t tokens, uint32_t H, uint32_t topk, float* out) {
#pragma omp parallel for schedule(static)
    for (uint32_t t = 0; t < tokens; ++t) {
        const float g = zco_bf(zco_sigmoid_bf(gate[t]));
        for (uint32_t c = 0; c < H; ++c) {
            float partial[8] = {0};
            for (uint32_t k = 0; k < topk; ++k) {
                float product = experts[((uint64_t)t * topk + k) * H + c] * weights[(uint64_t)t * topk + k];
                if (k < 8) partial[k] = product; else partial[k % 8] = partial[k % 8] + product;
            }
            float sum = partial[0];
            for (uint32_t k = 1; k < 8 && k < topk; ++k) sum += partial[k];
            out[(uint64_t)t * H + c] = zco_bf(zco_bf(sum) + zco_bf(g * shared[(uint64_t)t * H + c]));
        }
    }
}

uint64_t zco_projection_bytes(uint32_t K, uint32_t N, uint32_t group, uint32_t bits) {
    return (uint64_t)K * N * bits / 8 + 2ull * 2 * (K / group) * N;
}
static void shape(const zco_config_t* c, int shared, int projection, uint32_t* K, uint32_t* N, uint32_t* bits) {
    *K = projection == 2 ? c->inter : c->hidden;
    *N = projection == 2 ? c->hidden : c->inter;
    *bits = shared ? (projection == 2 ? c->shared_bits_down : c->shared_bits_gate_up)
                   : (projection == 2 ? c->bits_down : c->bits_gate_up);
}
uint64_t zco_record_bytes(const zco_config_t* c, int shared) {
    uint64_t total = 0;
    for (int p = 0; p < 3; ++p) { uint32_t K, N, b; shape(c, shared, p, &K, &N, &b); total += zco_projection_bytes(K, N, c->group, b); }
    return total;
}
/* metal.mm:1124-1129: [W,S,B] per projection, projections back to back. */
void zco_expert_linear(const zco_config_t* c, int shared, const uint8_t* record, int projection, zco_linear_t* out) {
    uint64_t offset = 0; uint32_t K, N, bits;
    for (int p = 0; p < projection; ++p) { shape(c, shared, p, &K, &N, &bits); offset += zco_projection_bytes(K, N, c->group, bits); }
    shape(c, shared, projection, &K, &N, &bits);
    const uint64_t wbytes = (uint64_t)K * N * bits / 8, meta = 2ull * (K / c->group) * N;
    out->weight = record + offset;
    out->scales = (const uint16_t*)(record + offset + wbytes);
    out->biases = (const uint16_t*)(record + offset + wbytes + meta);
    out->input = K; out->output = N; out->group = c->group; out->bits = bits;
}

/* model.cpp:431-557 with pipeline.cpp:7-31 for each selected expert. */
int zco_moe_layer(const zco_config_t* c, const zco_layer_t* l, const float* x, uint32_t tokens,
                  float* out, zco_trace_t* trace, int threads) {
#ifdef _OPENMP
    omp_set_num_threads(threads > 1 ? threads : 1);
#else
    (void)threads;
#endif
    const uint32_t H = c->hidden, E = c->experts, k = c->topk, I = c->inter, n = tokens * k;
    float* logits = (float*)malloc((size_t)tokens * E * 4);
    int32_t* ids = (int32_t*)malloc((size_t)n * 4);
    float* weights = (float*)malloc((size_t)n * 4);
    int32_t* offsets = (int32_t*)malloc((size_t)(E + 1) * 4);
    int32_t* slots = (int32_t*)malloc((size_t)n * 4);
    int32_t* selected = (int32_t*)malloc((size_t)E * 4);
    float* expert_out = (float*)calloc((size_t)n * H, 4);
    float* shared_act = (float*)malloc((size_t)tokens * I * 4);
    float* shared = (float*)malloc((size_t)tokens * H * 4);
    float* gate = (float*)malloc((size_t)tokens * 4);
    int status = 0;
    zco_router_logits(l->router, x, tokens, H, E, l->router_offsets, logits);
    zco_route(logits, tokens, E, k, ids, weights);
    const int count = zco_dispatch(ids, tokens, k, E, offsets, slots, selected);
    if (count < 0) status = -1;
    else {
        zco_linear_t g, u, d;
        zco_expert_linear(c, 1, l->shared_record, 0, &g);
        zco_expert_linear(c, 1, l->shared_record, 1, &u);
        zco_expert_linear(c, 1, l->shared_record, 2, &d);
        zco_gated_linear(&g, &u, x, tokens, NULL, shared_act);
        zco_linear(&d, shared_act, tokens, shared, 0);
        zco_plain_mm(l->shared_gate, 0, x, H, 1, tokens, gate, 0);
        for (int s = 0; s < count; ++s) {
            const int32_t e = selected[s];
            const int32_t* pos = slots + offsets[e];
            const uint32_t rows_n = (uint32_t)(offsets[e + 1] - offsets[e]);
            int32_t* rows = (int32_t*)malloc((size_t)rows_n * 4);
            float* act = (float*)malloc((size_t)rows_n * I * 4);
            float* down = (float*)malloc((size_t)rows_n * H * 4);
            for (uint32_t r = 0; r < rows_n; ++r) rows[r] = pos[r] / (int32_t)k;
            const uint8_t* record = l->expert_records + (uint64_t)e * l->record_stride;
            zco_expert_linear(c, 0, record, 0, &g);
            zco_expert_linear(c, 0, record, 1, &u);
            zco_expert_linear(c, 0, record, 2, &d);
            zco_gated_linear(&g, &u, x, rows_n, rows, act);
            zco_linear(&d, act, rows_n, down, 0);
            zco_scatter_experts(down, pos, rows_n, H, expert_out);
            free(rows); free(act); free(down);
        }
        zco_moe_sum(expert_out, weights, shared, gate, tokens, H, k, out);
    }
    if (trace) {
        if (trace->logits) memcpy(trace->logits, logits, (size_t)tokens * E * 4);
        if (trace->ids) memcpy(trace->ids, ids, (size_t)n * 4);
        if (trace->weights) memcpy(trace->weights, weights, (size_t)n * 4);
        if (trace->expert_out) memcpy(trace->expert_out, expert_out, (size_t)n * H * 4);
        if (trace->shared) memcpy(trace->shared, shared, (size_t)tokens * H * 4);
        if (trace->gate) memcpy(trace->gate, gate, (size_t)tokens * 4);
    }
    free(logits); free(ids); free(weights); free(offsets); free(slots); free(selected);
    free(expert_out); free(shared_act); free(shared); free(gate);
    return status;
}
