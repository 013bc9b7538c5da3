/* The CPU oracle (oracle/zc_oracle.c) compiled together with this driver under -fsanitize=address,undefined (make asan):
 * every operator once on small buffers allocated to their exact sizes, so that a read or write past an end, a shift out
 * of range or a signed overflow in the restatement stops the run.  Values are checked elsewhere (tests/test_oracle_*.py);
 * here only two closed forms guard against a driver that calls nothing. */
#include "../../oracle/zc_oracle.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static uint64_t state = 0x5eedull;
static uint32_t next(void) { state = state * 6364136223846793005ull + 1442695040888963407ull; return (uint32_t)(state >> 33); }
static float unit(void) { return (float)(next() % 2001) / 1000.0f - 1.0f; }
static int failures = 0;
#define CHECK(c) do { if (!(c)) { ++failures; printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #c); } } while (0)

static void fill_record(const zco_config_t* c, int shared, uint8_t* record) {
    const uint64_t n = zco_record_bytes(c, shared);
    for (uint64_t i = 0; i < n; ++i) record[i] = (uint8_t)next();
    for (int p = 0; p < 3; ++p) {   /* sane scales and biases: small positive scale, bias = -8 * scale */
        zco_linear_t l; zco_expert_linear(c, shared, record, p, &l);
        const uint64_t groups = (uint64_t)l.output * (l.input / l.group);
        uint16_t* s = (uint16_t*)(uintptr_t)l.scales; uint16_t* b = (uint16_t*)(uintptr_t)l.biases;
        for (uint64_t g = 0; g < groups; ++g) { const float v = 0.002f + 0.018f * (float)(next() % 1000) / 1000.0f; s[g] = zco_bf_bits(v); b[g] = zco_bf_bits(-8.0f * zco_b16(s[g])); }
    }
}

static void layer_case(zco_config_t c, uint32_t tokens, int threads) {
    const uint64_t stride = (zco_record_bytes(&c, 0) + 255) / 256 * 256;
    uint16_t* router = malloc((size_t)c.experts * c.hidden * 2); uint16_t* gate = malloc((size_t)c.hidden * 2);
    float* offsets = malloc((size_t)c.experts * 4);
    uint8_t* shared = malloc(zco_record_bytes(&c, 1));
    uint8_t* records = malloc(stride * (c.experts - 1) + zco_record_bytes(&c, 0));   /* no pad after the last record */
    float* x = malloc((size_t)tokens * c.hidden * 4); float* out = malloc((size_t)tokens * c.hidden * 4);
    for (uint64_t i = 0; i < (uint64_t)c.experts * c.hidden; ++i) router[i] = zco_bf_bits(unit() * 0.05f);
    for (uint32_t i = 0; i < c.hidden; ++i) gate[i] = zco_bf_bits(unit() * 0.05f);
    for (uint32_t e = 0; e < c.experts; ++e) offsets[e] = unit();
    fill_record(&c, 1, shared);
    for (uint32_t e = 0; e < c.experts; ++e) {
        uint8_t* tmp = malloc(zco_record_bytes(&c, 0)); fill_record(&c, 0, tmp);
        memcpy(records + e * stride, tmp, zco_record_bytes(&c, 0)); free(tmp);
    }
    for (uint64_t i = 0; i < (uint64_t)tokens * c.hidden; ++i) x[i] = zco_bf(unit());
    const uint64_t n = (uint64_t)tokens * c.topk;
    zco_trace_t tr = { malloc((size_t)tokens * c.experts * 4), malloc(n * 4), malloc(n * 4), malloc(n * c.hidden * 4), malloc((size_t)tokens * c.hidden * 4), malloc((size_t)tokens * 4) };
    zco_layer_t l = { router, offsets, gate, shared, records, stride };
    CHECK(zco_moe_layer(&c, &l, x, tokens, out, &tr, threads) == 0);
    float sum = 0; for (uint32_t j = 0; j < c.topk; ++j) sum += tr.weights[j];
    CHECK(fabsf(sum - 1.0f) < 1e-5f);
    for (uint64_t i = 0; i < (uint64_t)tokens * c.hidden; ++i) CHECK(out[i] == zco_bf(out[i]));   /* BF16-valued, finite or not */
    CHECK(zco_moe_layer(&c, &l, x, tokens, out, NULL, threads) == 0);
    x[3] = NAN;   /* a row of NaN logits: the call reports an invalid router output and writes nothing past its buffers */
    for (uint32_t k = 0; k < c.hidden; ++k) x[k] = NAN;
    CHECK(zco_moe_layer(&c, &l, x, tokens, out, &tr, threads) == -1);
    free(router); free(gate); free(offsets); free(shared); free(records); free(x); free(out);
    free(tr.logits); free(tr.ids); free(tr.weights); free(tr.expert_out); free(tr.shared); free(tr.gate);
}

int main(void) {
    /* scalar helpers over the whole float range, special values included */
    const uint32_t specials[] = {0u, 0x80000000u, 0x7f800000u, 0xff800000u, 0x7fc00000u, 0x7f7fffffu, 0x00000001u, 0x3f808000u, 0x477fe000u, 0xc2b00000u, 0x42b20000u};
    for (unsigned i = 0; i < sizeof specials / sizeof *specials; ++i) {
        float v; memcpy(&v, &specials[i], 4);
        (void)zco_bf(v); (void)zco_bf_bits(v); (void)zco_expf(v); (void)zco_sigmoid_bf(v); (void)zco_softplus_bf(v);
        for (uint32_t op = 0; op < 5; ++op) (void)zco_unary(v, op);
    }
    for (int i = 0; i < 20000; ++i) { const uint32_t u = next() ^ (next() << 16); float v; memcpy(&v, &u, 4); (void)zco_bf(v); (void)zco_expf(v); (void)zco_unary(v, (uint32_t)i % 5); }
    CHECK(zco_bf(1.00390625f) == 1.0f && zco_bf(1.01171875f) == 1.015625f);    /* ties to even, both directions */

    /* routing on exceptional rows: ramps, ties, signed zeros, too few finite scores, NaN, +inf, all -inf, all NaN */
    enum { E = 512, K = 10, T = 16 };
    float* v = malloc(sizeof(float) * T * E); int32_t* ids = malloc(sizeof(int32_t) * T * K); float* w = malloc(sizeof(float) * T * K);
    for (int t = 0; t < T; ++t) for (int e = 0; e < E; ++e) {
        float a = ldexpf((float)((int)(next() % 2001) - 1000), -(int)(next() % 12));
        switch (t % 10) { case 0: a = (float)e; break; case 1: a = -(float)e; break; case 2: a = (float)(e % 13); break; case 3: a = e % 2 ? 0.0f : -0.0f; break;
            case 4: a = e < 9 ? (float)e : -INFINITY; break; case 5: if (e % 41 == 0) a = NAN; break; case 6: if (e % 33 == 0) a = INFINITY; break;
            case 7: a = -INFINITY; break; case 8: a = NAN; break; default: break; }
        v[t * E + e] = a;
    }
    zco_route(v, T, E, K, ids, w);
    CHECK(ids[0] == 511 && ids[1 * K] == 0 && ids[4 * K + 9] == -1 && ids[7 * K] == -1);
    int32_t* offsets = malloc(sizeof(int32_t) * (E + 1)); int32_t* slots = malloc(sizeof(int32_t) * T * K); int32_t* selected = malloc(sizeof(int32_t) * E);
    CHECK(zco_dispatch(ids, T, K, E, offsets, slots, selected) == -1);          /* the -1 paddings are an invalid router output */
    CHECK(zco_dispatch(ids, 3, K, E, offsets, slots, selected) > 0);            /* rows 0..2 are complete */
    free(v); free(ids); free(w); free(offsets); free(slots); free(selected);

    /* whole layers: Q4 everywhere, the mixed 4/8-bit artifact, a lane-width-16 shape, serial and threaded */
    zco_config_t small = {512, 32, 4, 128, 64, 4, 4, 4, 4};
    layer_case(small, 1, 1); layer_case(small, 5, 4);
    zco_config_t mixed = {512, 16, 4, 128, 64, 4, 8, 8, 8};
    layer_case(mixed, 3, 2);
    zco_config_t wide = {1024, 16, 10, 512, 64, 4, 4, 4, 4};
    layer_case(wide, 2, 4);

    /* glue operators on exact-size buffers */
    enum { TOK = 3, H = 256 };
    float* a = malloc(sizeof(float) * TOK * 4 * H); float* b = malloc(sizeof(float) * TOK * 4 * H); float* o = malloc(sizeof(float) * TOK * 4 * H);
    for (int i = 0; i < TOK * 4 * H; ++i) { a[i] = zco_bf(unit()); b[i] = zco_bf(unit()); }
    for (uint32_t op = 0; op < 5; ++op) zco_unary_n(a, TOK * H, op, o);
    for (uint32_t op = 0; op < 2; ++op) zco_binary_n(a, b, TOK * H, op, o);
    zco_hc_mix(a, b, TOK, H, o);
    float* inj = malloc(sizeof(float) * TOK * 4); for (int i = 0; i < TOK * 4; ++i) inj[i] = zco_bf(unit());
    zco_hc_add(a, b, inj, TOK, H, o);
    uint16_t nw[H]; for (int i = 0; i < H; ++i) nw[i] = zco_bf_bits(1.0f + unit() * 0.1f);
    zco_norm(a, nw, 0, H, H, TOK, o); zco_norm(a, nw, 0, 64, H, TOK, o);
    free(a); free(b); free(o); free(inj);
    printf("oracle under sanitizers: %d failures\n", failures);
    return failures ? 1 : 0;
}
