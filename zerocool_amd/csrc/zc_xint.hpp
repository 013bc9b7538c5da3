// Exact-integer evaluation of the affine Q4 dot on the matrix cores.
//
// The reference evaluates a row as 32 lanes, each summing `scale*dot + sum*bias` over
// its 16-element blocks, where `dot` is an fp32 chain over the block.  For BF16-valued
// inputs every product x*q (8-bit by 4-bit significands) is exact, and when all
// partial sums of a block fit 24 bits the whole chain is exact: `dot` then equals the
// true sum, whatever the order.  Such a block is computed here in integers:
//   x_k = X_k * 2^e   (e = smallest exponent in the block, X_k integer, |X_k| < 2^21)
//   X_k = d0 + 2^7 d1 + 2^14 d2  (two's-complement digits: d0, d1 in [0,127], d2 signed)
//   dot = float(sum_k X_k q_k) * 2^e,  sum_k X_k q_k from three int8 MFMA rows.
// A block is "safe" when 15 * sum_k |X_k| < 2^24 and every x_k is BF16-valued; any
// other block takes the literal fp32 chain.  Per-block terms are then combined in the
// reference's lane order, so results equal the literal kernels bit for bit.
//
// One v_mfma_i32_16x16x64_i8 covers 16 weight rows x 4 blocks for one token: the A
// operand is block-diagonal (row (c,p) holds digit plane p of block c in lane group c,
// zeros elsewhere), the B operand holds each row's 16 codes of block G in lane group G.
// D[(c,p)][j] lands in lane (j, G=c), register p: the lane that loaded (row j, block G)
// receives that block's three digit sums.
#pragma once
#include "zc_device.hpp"

namespace zc {

typedef int v4i __attribute__((ext_vector_type(4)));

// LDS image of one token's input row, K elements: per 16-block three digit planes of
// 16 bytes in MFMA byte order, a {2^e, bias-sum} pair, and an unsafe bit.
struct XintLayout {
    uint32_t K;
    __host__ __device__ constexpr uint32_t blocks() const { return K / 16; }
    __host__ __device__ constexpr uint32_t planes_bytes() const { return blocks() * 48 + 16; }   // + one zero slot
    __host__ __device__ constexpr uint32_t info_bytes() const { return blocks() * 8; }
    __host__ __device__ constexpr uint32_t mask_bytes() const { return (blocks() + 31) / 32 * 4; }
    __host__ __device__ constexpr uint32_t bytes() const { return (planes_bytes() + info_bytes() + mask_bytes() + 15) / 16 * 16; }
};

// The three digit sums of a block recombined, d0 + 2^7 d1 + 2^14 d2, by Horner's rule in two shift-and-add instructions.
// (The empty statement keeps the compiler from regrouping the sum into two shifts and a three-operand add; the instructions
// themselves are the compiler's, so it still places the wait states a read of matrix-core results needs.)
__device__ __forceinline__ int xint_digits(const v4i r) {
    int t = int((uint32_t(r[2]) << 7) + uint32_t(r[1]));
    asm("" : "+v"(t));
    return int((uint32_t(t) << 7) + uint32_t(r[0]));
}

// One of a dword's two BF16 values as fp32, in one byte-permute: select 0x03020c0c takes the upper one, 0x01000c0c the lower.
__device__ __forceinline__ float xint_bf16_of(uint32_t pair, uint32_t select) { return __uint_as_float(__builtin_amdgcn_perm(pair, pair, select)); }

// Byte t of a lane's 16-byte operand holds block element kOrder[t]: the order in which
// (w & 0x0f0f0f0f), ((w >> 4) & 0x0f0f0f0f) of the block's two code words lay nibbles out.
__device__ __forceinline__ uint32_t xint_element_of_byte(uint32_t t) {
    return (t & 8u) + ((t & 3u) << 1) + ((t >> 2) & 1u);
}

// Loads with agent scope: data written by another workgroup of a persistent kernel must
// not come from a stale cache line.
__device__ __forceinline__ float load_shared_f32(const float* p) {
    return __uint_as_float(__hip_atomic_load(reinterpret_cast<const uint32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

// Input sources: a row staged in LDS.  block(b, out) gives the fp32 bit patterns of the
// sixteen elements of block b.  kExactProducts: every element is BF16-valued, so x*q is
// exact and a fused multiply-add equals the reference's separate multiply and add.
struct LdsBf16 {     // BF16 copy of a BF16-valued row
    static constexpr bool kExactProducts = true, kRowInLds = true;
    const uint16_t* x;
    __device__ __forceinline__ void block(uint32_t b, uint32_t* out) const {
        // (native vector types: the compiler then keeps track of where the read comes from, and does not make it wait for
        // loads whose target is another part of LDS)
        const u32x4 lo = *reinterpret_cast<const u32x4*>(x + b * 16), hi = *reinterpret_cast<const u32x4*>(x + b * 16 + 8);
        const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) { out[2 * i] = w[i] << 16; out[2 * i + 1] = w[i] & 0xffff0000u; }
    }
};
struct RegBf16 {     // one block of sixteen BF16 values held in registers (block index ignored)
    static constexpr bool kExactProducts = true, kRowInLds = false;
    uint64_t w[4];
    __device__ __forceinline__ void block(uint32_t, uint32_t* out) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t lo = uint32_t(w[i]), hi = uint32_t(w[i] >> 32);
            out[4 * i] = lo << 16; out[4 * i + 1] = lo & 0xffff0000u; out[4 * i + 2] = hi << 16; out[4 * i + 3] = hi & 0xffff0000u;
        }
    }
};
struct RegF32 {      // one block of sixteen BF16-valued fp32 bit patterns held in registers (block index ignored)
    static constexpr bool kExactProducts = true, kRowInLds = false;
    uint32_t bits[16];
    __device__ __forceinline__ void block(uint32_t, uint32_t* out) const {
#pragma unroll
        for (int i = 0; i < 16; ++i) out[i] = bits[i];
    }
};
struct LdsF32 {      // fp32 copy of an arbitrary row
    static constexpr bool kExactProducts = false, kRowInLds = false;
    const float* x;
    __device__ __forceinline__ void block(uint32_t b, uint32_t* out) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint4 v = *reinterpret_cast<const uint4*>(x + b * 16 + 4 * i);
            out[4 * i] = v.x; out[4 * i + 1] = v.y; out[4 * i + 2] = v.z; out[4 * i + 3] = v.w;
        }
    }
};

// Builds one 16-block `b` of an image: digit planes, {2^e, bias sum}, unsafe bit.
// The image's mask words must have been zeroed (xint_prepare_begin) before.
//
// e = exponent field of the smallest non-zero magnitude; every element times 2^(134-e) is then
// an integer X (8-bit significand shifted left by its exponent distance), obtained with one
// exact scaling and one conversion.  The block is safe when 15 * sum|X| < 2^24, i.e.
// sum|X| <= 1118481: that bound also keeps every |X| below 2^21 (three digit planes), rules out
// infinities and NaN (the sum is then not below the bound), and exponent distances above 13.
// A block whose smallest element is subnormal is left to the literal chain.
template <class Source>
__device__ __forceinline__ void xint_prepare_block(const Source x, const XintLayout L, uint8_t* lds, uint32_t b) {
    uint8_t* planes = lds;
    float2* info = reinterpret_cast<float2*>(lds + L.planes_bytes());
    uint32_t* mask = reinterpret_cast<uint32_t*>(lds + L.planes_bytes() + L.info_bytes());
    uint32_t bits[16];
    x.block(b, bits);
    // bias sum: BF16 rounding after each addition of four inputs (reference: qwen.metal:55).  For BF16-valued
    // inputs the rounding needs no NaN case: a NaN keeps being a NaN under the integer form of the rounding.
    auto round16 = [](float v) {
        if constexpr (Source::kExactProducts) {
            const uint32_t u = __float_as_uint(v);
            return __uint_as_float((u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u);
        } else {
            return bf(v);
        }
    };
    float sum = 0;
#pragma unroll
    for (int i = 0; i < 16; i += 4)
        sum += round16(round16(round16(__uint_as_float(bits[i]) + __uint_as_float(bits[i + 1])) + __uint_as_float(bits[i + 2])) + __uint_as_float(bits[i + 3]));
    // smallest non-zero magnitude: (bits << 1) - 1 wraps zeros to the top of the unsigned range
    uint32_t tmin = 0xffffffffu, lowbits = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        tmin = min(tmin, (bits[i] << 1) - 1u);
        if constexpr (!Source::kExactProducts) lowbits |= bits[i] & 0xffffu;
    }
    const uint32_t smallest = tmin + 1u;                 // (bits << 1) of that element, 0 when the block is all zeros
    const bool subnormal = smallest != 0u && smallest < (1u << 24);
    const uint32_t emin = max(smallest >> 24, 1u);
    // integers on the common exponent, and the sum of their magnitudes (exact while it matters)
    int32_t xs[16];
    float sumabs = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float scaled = __builtin_ldexpf(__uint_as_float(bits[i]), 134 - int(emin));
        sumabs += __builtin_fabsf(scaled);
        xs[i] = int32_t(scaled);
    }
    const bool safe = !lowbits && !subnormal && sumabs <= 1118481.0f;
    // digits of the signed integer Xs in two's complement: Xs = d0 + 2^7 d1 + 2^14 d2 with
    // d0, d1 in [0,127] and d2 = Xs >> 14 in [-128,127]
    uint32_t words[3][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t w0 = 0, w1 = 0, w2 = 0;
#pragma unroll
        for (int q = 3; q >= 0; --q) {
            const uint32_t v = uint32_t(xs[xint_element_of_byte(4 * j + q)]);
            w0 = (w0 << 8) | (v & 127u);
            w1 = (w1 << 8) | ((v >> 7) & 127u);
            w2 = (w2 << 8) | ((v >> 14) & 255u);
        }
        words[0][j] = safe ? w0 : 0u; words[1][j] = safe ? w1 : 0u; words[2][j] = safe ? w2 : 0u;
    }
    if (!safe) atomicOr(mask + b / 32, 1u << (b % 32));
#pragma unroll
    for (int p = 0; p < 3; ++p)
        *reinterpret_cast<uint4*>(planes + b * 48 + p * 16) = make_uint4(words[p][0], words[p][1], words[p][2], words[p][3]);
    // 2^(emin-134): x = sig * 2^(e-127-7)
    const int ex = int(emin) - 134;
    const float scale = ex >= -126 ? __uint_as_float(uint32_t(ex + 127) << 23) : __uint_as_float(1u << (ex + 149));
    info[b] = make_float2(scale, sum);
}
// Clears the unsafe masks and zero slots of `count` consecutive images (stride L.bytes()).
__device__ __forceinline__ void xint_prepare_begin(const XintLayout L, uint8_t* lds, uint32_t count) {
    const uint32_t words = L.mask_bytes() / 4;
    uint32_t first = threadIdx.x;
    asm volatile("" : "+v"(first));   // addresses are formed here, not hoisted out of a caller's outer loop
    for (uint32_t i = first; i < count * words; i += blockDim.x)
        reinterpret_cast<uint32_t*>(lds + (i / words) * L.bytes() + L.planes_bytes() + L.info_bytes())[i % words] = 0;
    for (uint32_t i = first; i < count * 4; i += blockDim.x)
        reinterpret_cast<uint32_t*>(lds + (i / 4) * L.bytes() + L.blocks() * 48)[i % 4] = 0;
}
// Builds `count` images cooperatively: all threads call it; source_of(q) gives image q's
// input row.  Work is the flat list of (image, block) pairs.  Ends with a barrier.
template <class SourceOf>
__device__ __forceinline__ void xint_prepare_batch(const SourceOf source_of, uint32_t count, const XintLayout L, uint8_t* lds) {
    xint_prepare_begin(L, lds, count);
    __syncthreads();
    const uint32_t blocks = L.blocks();
    uint32_t first = threadIdx.x;
    asm volatile("" : "+v"(first));
    for (uint32_t i = first; i < count * blocks; i += blockDim.x) {
        const uint32_t q = i / blocks;
        xint_prepare_block(source_of(q), L, lds + q * L.bytes(), i % blocks);
    }
    __syncthreads();
}

// The literal fp32 chain of one block (reference: qwen.metal:52-57) from the block's
// expanded code bytes (MFMA byte order: element of byte t is xint_element_of_byte(t)).
template <class Source>
__device__ __forceinline__ float xint_literal_dot(const v4i codes, const Source x, uint32_t block) {
    uint32_t xb[16];
    x.block(block, xb);
    float q[16];   // q[element]
#pragma unroll
    for (int t = 0; t < 16; ++t) q[(t & 8) + ((t & 3) << 1) + ((t >> 2) & 1)] = float((uint32_t(codes[t / 4]) >> (8 * (t % 4))) & 255u);
    float dot = 0;
#pragma unroll
    for (int i = 0; i < 16; i += 4) {
        const float a = __uint_as_float(xb[i]), c = __uint_as_float(xb[i + 1]), d = __uint_as_float(xb[i + 2]), e = __uint_as_float(xb[i + 3]);
        if constexpr (Source::kExactProducts)
            dot += __builtin_fmaf(e, q[i + 3], __builtin_fmaf(d, q[i + 2], __builtin_fmaf(c, q[i + 1], a * q[i])));
        else
            dot += a * q[i] + c * q[i + 1] + d * q[i + 2] + e * q[i + 3];
    }
    return dot;
}

// Runs a whole 16-column tile for nt <= PT tokens and hands each finished row sum to
// emit(t, sum).  lane = (j = column, G = lane / 16); acc[t][m][h] is the running sum of
// reference lane 8*m + 2*G + h of the column's row.
//
// Weights stream through a ring of R spans (128 elements each) per lane: R sixteen-byte
// code loads plus the matching scale / bias dwords (dword d of a row's vector holds
// groups 2d, 2d+1) are in flight while earlier spans are multiplied.  Each ring body is
// three straight-line passes so the scheduler can overlap LDS reads, MFMAs and VALU work:
//   1. every span: A operands from LDS, two MFMAs, digit sums -> fp32 block dots
//   2. only if some block of the body is unsafe: those dots again by the literal chain
//   3. every span: acc += scale*dot + sum*bias, in span order
//
// prologue() runs once the first ring of weights has been requested and before anything is read from the images: a caller
// whose images are not built yet builds them there, under the latency of those loads.
//
// PAIR: the tile has exactly two bodies (spans == 2 R) and both are requested before the prologue, each into registers of
// its own: the second body then does not wait for a memory latency of its own either.
template <int PT, int R, bool PAIR = false, class Source, class Emit, class Prologue>
__device__ __forceinline__ void xint_run_tile_after(const uint8_t* w_row, const uint16_t* s_row, const uint16_t* b_row, uint32_t spans,
                                                    const uint8_t* const* img, const Source* src, const XintLayout L, uint32_t lane,
                                                    int nt, Emit emit, Prologue prologue) {
    static_assert(R == 8 || R == 4, "bodies of eight or four spans; spans must be a multiple of R");
    const uint32_t G = lane >> 4, row_a = lane & 15u, c_a = row_a >> 2, p_a = row_a & 3u;
    const uint8_t* c = w_row + 16 * G;   // the lane's 16 bytes of each 64-byte span
    uint4 ring[R], sring[R / 4], bring[R / 4];
#pragma unroll
    for (int j = 0; j < R; ++j) ring[j] = ldg_u4(c, j * 4);
#pragma unroll
    for (int q = 0; q < R / 4; ++q) { sring[q] = ldg_u4(s_row, q); bring[q] = ldg_u4(b_row, q); }
    uint4 ring2[PAIR ? R : 1], sring2[PAIR ? R / 4 : 1], bring2[PAIR ? R / 4 : 1];
    if constexpr (PAIR) {
#pragma unroll
        for (int j = 0; j < R; ++j) ring2[j] = ldg_u4(c, (R + j) * 4);
    }
    float acc[PT][4][2];
#pragma unroll
    for (int t = 0; t < PT; ++t)
#pragma unroll
        for (int m = 0; m < 4; ++m) { acc[t][m][0] = 0; acc[t][m][1] = 0; }
    const uint32_t half = (lane & 32u) ? 0x03020c0cu : 0x01000c0cu;   // group 2d + (G >> 1): the low BF16 of a dword for G < 2
    // A operand: row (c,p) of lane group G holds digit plane p of block 2c (+1) when c == G, zeros otherwise
    const bool live = (c_a == G) && p_a < 3;
    const uint32_t a_first = live ? 2 * G * 48 + p_a * 16 : L.blocks() * 48, a_span = live ? 8 * 48 : 0, a_next = live ? 48 : 0;
    const uint32_t M = 0x0f0f0f0fu;
    const v4i zero = {0, 0, 0, 0};
    auto expand = [&](uint32_t lo, uint32_t hi) { const v4i r = {int(lo & M), int((lo >> 4) & M), int(hi & M), int((hi >> 4) & M)}; return r; };
    prologue();
    // one body: spans d0 .. d0 + R - 1 with their codes and scale / bias dwords
    auto compute = [&](uint32_t d0, const uint4 (&codes)[R], const uint32_t (&sd)[R], const uint32_t (&bd)[R]) {
#pragma unroll
        for (int t = 0; t < PT; ++t) {
            if (t >= nt) break;
            const uint8_t* planes = img[t];
            const float2* info = reinterpret_cast<const float2*>(planes + L.planes_bytes());
            const uint32_t* mask = reinterpret_cast<const uint32_t*>(planes + L.planes_bytes() + L.info_bytes());
            float dot[R][2], bsum[R][2];
            // pass 1
#pragma unroll
            for (int j = 0; j < R; ++j) {
                const uint32_t d = d0 + j;
                {
                    const v4i b0 = expand(codes[j].x, codes[j].y), b1 = expand(codes[j].z, codes[j].w);
                    const uint8_t* a_at = planes + a_first + d * a_span;
                    const v4i a0 = *reinterpret_cast<const v4i*>(a_at), a1 = *reinterpret_cast<const v4i*>(a_at + a_next);
                    const v4i r0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b0, zero, 0, 0, 0);
                    const v4i r1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b1, zero, 0, 0, 0);
                    const float4 fi = *reinterpret_cast<const float4*>(info + 8 * d + 2 * G);   // {2^e, sum} of blocks 2G, 2G+1
                    dot[j][0] = float(xint_digits(r0)) * fi.x; bsum[j][0] = fi.y;
                    dot[j][1] = float(xint_digits(r1)) * fi.z; bsum[j][1] = fi.w;
                }
            }
            // pass 2: blocks 8d + 2G + h of spans d0 .. d0+7 sit in mask words d0/4, d0/4 + 1
            const uint32_t mine = 0x03030303u << (2 * G);
            const uint32_t u0 = mask[d0 / 4] & mine, u1 = R == 8 ? mask[d0 / 4 + 1] & mine : 0u;
            if (__builtin_expect(__ballot((u0 | u1) != 0) != 0, 0)) {
#pragma unroll
                for (int j = 0; j < R; ++j) {
                    const uint32_t d = d0 + j;
                    {
                        const uint32_t bits = ((j < 4 ? u0 : u1) >> (8 * (j % 4) + 2 * G)) & 3u;
                        if (bits & 1u) dot[j][0] = xint_literal_dot(expand(codes[j].x, codes[j].y), src[t], 8 * d + 2 * G);
                        if (bits & 2u) dot[j][1] = xint_literal_dot(expand(codes[j].z, codes[j].w), src[t], 8 * d + 2 * G + 1);
                    }
                }
            }
            // pass 3
#pragma unroll
            for (int j = 0; j < R; ++j) {
                {
                    const float scale = xint_bf16_of(sd[j], half), bias = xint_bf16_of(bd[j], half);
                    acc[t][j & 3][0] += scale * dot[j][0] + bsum[j][0] * bias;
                    acc[t][j & 3][1] += scale * dot[j][1] + bsum[j][1] * bias;
                }
            }
        }
    };
    auto dwords = [&](const uint4 (&from)[R / 4], uint32_t (&to)[R]) {
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint4 q = from[j / 4];
            to[j] = (j % 4 == 0) ? q.x : (j % 4 == 1) ? q.y : (j % 4 == 2) ? q.z : q.w;
        }
    };
    if constexpr (PAIR) {
        // the second body's scales and biases share cache lines with the first body's: requested late, they are close by
#pragma unroll
        for (int q = 0; q < R / 4; ++q) { sring2[q] = ldg_u4(s_row, R / 4 + q); bring2[q] = ldg_u4(b_row, R / 4 + q); }
        uint32_t sd[R], bd[R];
        dwords(sring, sd); dwords(bring, bd);
        compute(0, ring, sd, bd);
        if constexpr (R > 0) {   // (a scope of its own for the second body's dwords)
            uint32_t sd2[R], bd2[R];
            dwords(sring2, sd2); dwords(bring2, bd2);
            compute(R, ring2, sd2, bd2);
        }
    } else
    for (uint32_t d0 = 0; d0 < spans; d0 += R) {
        uint4 codes[R]; uint32_t sd[R], bd[R];
#pragma unroll
        for (int j = 0; j < R; ++j) codes[j] = ring[j];
        dwords(sring, sd); dwords(bring, bd);
        if (d0 + R < spans) {
#pragma unroll
            for (int j = 0; j < R; ++j) ring[j] = ldg_u4(c, (d0 + j + R) * 4);
#pragma unroll
            for (int q = 0; q < R / 4; ++q) { sring[q] = ldg_u4(s_row, (d0 + R) / 4 + q); bring[q] = ldg_u4(b_row, (d0 + R) / 4 + q); }
        }
        compute(d0, codes, sd, bd);
    }
    // Reference lane sum (xor butterfly 16, 8, 4, 2, 1): strides 16 and 8 pair accumulators,
    // 4 and 2 pair lane groups, 1 pairs the two blocks of a lane.
#pragma unroll
    for (int t = 0; t < PT; ++t) {
        if (t >= nt) break;
        float v[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float a0 = acc[t][0][h] + acc[t][2][h], a1 = acc[t][1][h] + acc[t][3][h];
            float sum = a0 + a1;
            sum = sum + __shfl_xor(sum, 32);
            sum = sum + __shfl_xor(sum, 16);
            v[h] = sum;
        }
        emit(t, v[0] + v[1]);
    }
}

// The literal fp32 chain of one block (reference: qwen.metal:52-57) from the block's two raw code words (nibble i of word w
// is element 8 w + i) and the block's sixteen BF16 inputs in LDS.  The four quads' nested sums do not depend on each other:
// all sixteen inputs are read at once and the four chains run side by side, then the quad sums are added in order -- one
// LDS latency and a chain of eight dependent operations instead of four latencies and twenty.
__device__ __forceinline__ float xint_literal_block(const uint16_t* x_block, uint32_t w_lo, uint32_t w_hi) {
    const u32x4 xa = *reinterpret_cast<const u32x4*>(x_block), xb = *reinterpret_cast<const u32x4*>(x_block + 8);
    const uint32_t xw[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
    float quad[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t w = q & 2 ? w_hi : w_lo, x0 = xw[2 * q], x1 = xw[2 * q + 1];
        const int at = 16 * (q & 1);
        const float a = __uint_as_float(x0 << 16), c = __uint_as_float(x0 & 0xffff0000u);
        const float d = __uint_as_float(x1 << 16), e = __uint_as_float(x1 & 0xffff0000u);
        // BF16-valued inputs times 4-bit codes are exact products: a fused multiply-add equals the reference's multiply and add
        quad[q] = __builtin_fmaf(e, float((w >> (at + 12)) & 15u), __builtin_fmaf(d, float((w >> (at + 8)) & 15u),
                  __builtin_fmaf(c, float((w >> (at + 4)) & 15u), a * float((w >> at) & 15u))));
    }
    float dot = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) dot += quad[q];
    return dot;
}

// The same tile for NTOK tokens that share the tile's weights (the tokens of a decode step routed to one expert), for
// workgroups that run two waves per SIMD (the other wave covers this one's LDS and MFMA latencies, so the tokens of a span
// are simply taken in turn).  Per span: the codes are expanded once; every token's block dots come from the MFMAs; then
// ONE loop serves the literal chains of all tokens: every lane takes its next unsafe (token, block) in turn until no lane
// has one left, so the chain's code exists once per span and its cost follows the busiest lane group, not the number
// of tokens; then the accumulators are updated in span order.  src must be BF16 rows in LDS.  Images beyond the live
// tokens (t >= nt) must point at valid images; their sums are computed and dropped.  Per-lane accumulation order and the
// final butterfly are those of xint_run_tile_after.
template <int NTOK, int R, class Emit>
__device__ __forceinline__ void xint_run_tile_tokens(const uint8_t* w_row, const uint16_t* s_row, const uint16_t* b_row, uint32_t spans,
                                                     const uint8_t* const* img, const LdsBf16* src, const XintLayout L, uint32_t lane,
                                                     int nt, Emit emit) {
    static_assert(R == 4, "bodies of four spans: one mask word per token covers a body");
    static_assert(NTOK >= 1 && NTOK <= 8, "the pending set of a lane is sixteen bits");
    const uint32_t G = lane >> 4, row_a = lane & 15u, c_a = row_a >> 2, p_a = row_a & 3u;
    const uint8_t* c = w_row + 16 * G;   // the lane's 16 bytes of each 64-byte span
    uint4 ring[R], sring, bring;
#pragma unroll
    for (int j = 0; j < R; ++j) ring[j] = ldg_u4(c, j * 4);
    sring = ldg_u4(s_row, 0); bring = ldg_u4(b_row, 0);
    float acc[NTOK][4][2];
#pragma unroll
    for (int t = 0; t < NTOK; ++t)
#pragma unroll
        for (int m = 0; m < 4; ++m) { acc[t][m][0] = 0; acc[t][m][1] = 0; }
    const uint32_t half = (lane & 32u) ? 0x03020c0cu : 0x01000c0cu;   // group 2d + (G >> 1): the low BF16 of a dword for G < 2
    const bool live = (c_a == G) && p_a < 3;
    const uint32_t a_first = live ? 2 * G * 48 + p_a * 16 : L.blocks() * 48, a_span = live ? 8 * 48 : 0, a_next = live ? 48 : 0;
    const uint32_t M = 0x0f0f0f0fu;
    const v4i zero = {0, 0, 0, 0};
    const uint32_t info_at = L.planes_bytes() + 2 * G * 8, mask_at = L.planes_bytes() + L.info_bytes();
    for (uint32_t d0 = 0; d0 < spans; d0 += R) {
        uint4 codes[R];
#pragma unroll
        for (int j = 0; j < R; ++j) codes[j] = ring[j];
        const uint32_t sdw[4] = {sring.x, sring.y, sring.z, sring.w}, bdw[4] = {bring.x, bring.y, bring.z, bring.w};
        if (d0 + R < spans) {
#pragma unroll
            for (int j = 0; j < R; ++j) ring[j] = ldg_u4(c, (d0 + j + R) * 4);
            sring = ldg_u4(s_row, (d0 + R) / 4); bring = ldg_u4(b_row, (d0 + R) / 4);
        }
        // the unsafe bits of this body's blocks, per token: blocks 8d + 2G + h of spans d0 .. d0+3 sit in mask word d0/4,
        // moved down so that bits 8j, 8j+1 are the lane's two blocks of span j
        uint32_t unsafe[NTOK], any = 0;
#pragma unroll
        for (int t = 0; t < NTOK; ++t) {
            unsafe[t] = (reinterpret_cast<const uint32_t*>(img[t] + mask_at)[d0 / 4] >> (2 * G)) & 0x03030303u;
            any |= unsafe[t];
        }
        const bool literal_body = __ballot(any != 0) != 0;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint32_t d = d0 + uint32_t(j);
            const v4i b0 = {int(codes[j].x & M), int((codes[j].x >> 4) & M), int(codes[j].y & M), int((codes[j].y >> 4) & M)};
            const v4i b1 = {int(codes[j].z & M), int((codes[j].z >> 4) & M), int(codes[j].w & M), int((codes[j].w >> 4) & M)};
            float dot[NTOK][2], bsum[NTOK][2];
#pragma unroll
            for (int t = 0; t < NTOK; ++t) {
                const uint8_t* a_at = img[t] + a_first + d * a_span;
                const v4i a0 = *reinterpret_cast<const v4i*>(a_at), a1 = *reinterpret_cast<const v4i*>(a_at + a_next);
                const float4 fi = *reinterpret_cast<const float4*>(img[t] + info_at + d * 64);   // {2^e, sum} of blocks 2G, 2G+1
                const v4i r0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b0, zero, 0, 0, 0);
                const v4i r1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b1, zero, 0, 0, 0);
                dot[t][0] = float(xint_digits(r0)) * fi.x; bsum[t][0] = fi.y;
                dot[t][1] = float(xint_digits(r1)) * fi.z; bsum[t][1] = fi.w;
            }
            if (__builtin_expect(literal_body, 0)) {
                // pending (token, block) pairs of this lane in span j: bit 2t + h
                uint32_t pending = 0;
#pragma unroll
                for (int t = 0; t < NTOK; ++t) pending |= ((unsafe[t] >> (8 * j)) & 3u) << (2 * t);
                while (__ballot(pending != 0) != 0) {
                    if (pending) {
                        const uint32_t item = uint32_t(__builtin_ctz(pending)), t = item >> 1, h = item & 1u;
                        const uint16_t* row = src[0].x;
#pragma unroll
                        for (int q = 1; q < NTOK; ++q) row = t == uint32_t(q) ? src[q].x : row;
                        const float lit = xint_literal_block(row + (8 * d + 2 * G + h) * 16, h ? codes[j].z : codes[j].x, h ? codes[j].w : codes[j].y);
#pragma unroll
                        for (int q = 0; q < NTOK; ++q) {
                            dot[q][0] = item == uint32_t(2 * q) ? lit : dot[q][0];
                            dot[q][1] = item == uint32_t(2 * q + 1) ? lit : dot[q][1];
                        }
                        pending &= pending - 1;
                    }
                }
            }
            const float scale = xint_bf16_of(sdw[j], half), bias = xint_bf16_of(bdw[j], half);
#pragma unroll
            for (int t = 0; t < NTOK; ++t) {
                acc[t][j][0] += scale * dot[t][0] + bsum[t][0] * bias;
                acc[t][j][1] += scale * dot[t][1] + bsum[t][1] * bias;
            }
        }
    }
    // Reference lane sum (xor butterfly 16, 8, 4, 2, 1): strides 16 and 8 pair accumulators, 4 and 2 pair lane groups, 1 the two blocks of a lane.
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
        float v[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float x0 = acc[t][0][h] + acc[t][2][h], x1 = acc[t][1][h] + acc[t][3][h];
            float sum = x0 + x1;
            sum = sum + __shfl_xor(sum, 32);
            sum = sum + __shfl_xor(sum, 16);
            v[h] = sum;
        }
        if (t < nt) emit(t, v[0] + v[1]);
    }
}
// The same for workgroups that run ONE wave per SIMD (the whole register file, up to eight tokens per pass): there is no
// other wave to cover this one's LDS and MFMA latencies, so the work of a body is cut into steps of at most four tokens of
// one span and software-pipelined by hand: the MFMAs of step s are issued back to back, then the LDS reads of step s + 1
// (into the other operand buffer), then the vector work of step s.  Scheduling barriers keep the compiler from folding
// the stages of a token back into one dependent chain.
template <int NTOK, int R, class Emit>
__device__ __forceinline__ void xint_run_tile_tokens_piped(const uint8_t* w_row, const uint16_t* s_row, const uint16_t* b_row, uint32_t spans,
                                                           const uint8_t* const* img, const LdsBf16* src, const XintLayout L, uint32_t lane,
                                                           int nt, Emit emit) {
    static_assert(R == 4, "bodies of four spans: one mask word per token covers a body");
    static_assert(NTOK == 1 || NTOK == 2 || NTOK == 4 || NTOK == 8, "token counts are rounded up to 1, 2, 4 or 8");
    constexpr int TG = NTOK < 4 ? NTOK : 4, GROUPS = NTOK / TG, STEPS = R * GROUPS;
    const uint32_t G = lane >> 4, row_a = lane & 15u, c_a = row_a >> 2, p_a = row_a & 3u;
    const uint8_t* c = w_row + 16 * G;   // the lane's 16 bytes of each 64-byte span
    uint4 ring[R], sring, bring;
#pragma unroll
    for (int j = 0; j < R; ++j) ring[j] = ldg_u4(c, j * 4);
    sring = ldg_u4(s_row, 0); bring = ldg_u4(b_row, 0);
    float acc[NTOK][4][2];
#pragma unroll
    for (int t = 0; t < NTOK; ++t)
#pragma unroll
        for (int m = 0; m < 4; ++m) { acc[t][m][0] = 0; acc[t][m][1] = 0; }
    const uint32_t half = (lane & 32u) ? 0x03020c0cu : 0x01000c0cu;   // group 2d + (G >> 1): the low BF16 of a dword for G < 2
    const bool live = (c_a == G) && p_a < 3;
    const uint32_t a_first = live ? 2 * G * 48 + p_a * 16 : L.blocks() * 48, a_span = live ? 8 * 48 : 0, a_next = live ? 48 : 0;
    const uint32_t M = 0x0f0f0f0fu;
    const v4i zero = {0, 0, 0, 0};
    const uint32_t info_at = L.planes_bytes() + 2 * G * 8, mask_at = L.planes_bytes() + L.info_bytes();
    // lane q < NTOK holds where token q's BF16 row starts, in elements from src[0]'s (a select chain over the tokens would be
    // turned into a table in memory by the compiler)
    uint32_t row_table = 0;
#pragma unroll
    for (int q = 1; q < NTOK; ++q) row_table = lane == uint32_t(q) ? uint32_t(src[q].x - src[0].x) : row_table;
    for (uint32_t d0 = 0; d0 < spans; d0 += R) {
        uint4 codes[R];
#pragma unroll
        for (int j = 0; j < R; ++j) codes[j] = ring[j];
        const uint32_t sdw[4] = {sring.x, sring.y, sring.z, sring.w}, bdw[4] = {bring.x, bring.y, bring.z, bring.w};
        if (d0 + R < spans) {
#pragma unroll
            for (int j = 0; j < R; ++j) ring[j] = ldg_u4(c, (d0 + j + R) * 4);
            sring = ldg_u4(s_row, (d0 + R) / 4); bring = ldg_u4(b_row, (d0 + R) / 4);
        }
        uint32_t unsafe[NTOK], any = 0;
#pragma unroll
        for (int t = 0; t < NTOK; ++t) {
            unsafe[t] = (reinterpret_cast<const uint32_t*>(img[t] + mask_at)[d0 / 4] >> (2 * G)) & 0x03030303u;
            any |= unsafe[t];
        }
        const bool literal_body = __ballot(any != 0) != 0;
        // operand buffers of two steps: A operands (digit planes of blocks 2G, 2G+1) and {2^e, sum} pairs of those blocks
        v4i a0[2][TG], a1[2][TG]; float4 fi[2][TG];
        auto load = [&](int buf, int step) {
            const uint32_t d = d0 + uint32_t(step / GROUPS);
            const int g = step % GROUPS;
#pragma unroll
            for (int t = 0; t < TG; ++t) {
                const uint8_t* image = img[g * TG + t];
                const uint8_t* a_at = image + a_first + d * a_span;
                a0[buf][t] = *reinterpret_cast<const v4i*>(a_at); a1[buf][t] = *reinterpret_cast<const v4i*>(a_at + a_next);
                fi[buf][t] = *reinterpret_cast<const float4*>(image + info_at + d * 64);
            }
        };
        load(0, 0);
#pragma unroll
        for (int step = 0; step < STEPS; ++step) {
            const int j = step / GROUPS, g = step % GROUPS, buf = step & 1;
            const uint32_t d = d0 + uint32_t(j);
            const v4i b0 = {int(codes[j].x & M), int((codes[j].x >> 4) & M), int(codes[j].y & M), int((codes[j].y >> 4) & M)};
            const v4i b1 = {int(codes[j].z & M), int((codes[j].z >> 4) & M), int(codes[j].w & M), int((codes[j].w >> 4) & M)};
            v4i r0[TG], r1[TG];
#pragma unroll
            for (int t = 0; t < TG; ++t) {
                r0[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[buf][t], b0, zero, 0, 0, 0);
                r1[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1[buf][t], b1, zero, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (step + 1 < STEPS) load(buf ^ 1, step + 1);
            __builtin_amdgcn_sched_barrier(0);
            float dot[TG][2];
#pragma unroll
            for (int t = 0; t < TG; ++t) {
                dot[t][0] = float(xint_digits(r0[t])) * fi[buf][t].x;
                dot[t][1] = float(xint_digits(r1[t])) * fi[buf][t].z;
            }
            if (__builtin_expect(literal_body, 0)) {
                // pending (token, block) pairs of this lane in this step: bit 2t + h; every lane takes its next one in turn
                uint32_t pending = 0;
#pragma unroll
                for (int t = 0; t < TG; ++t) pending |= ((unsafe[g * TG + t] >> (8 * j)) & 3u) << (2 * t);
                while (__ballot(pending != 0) != 0) {
                    // (every lane is active here: the row of token t is lane t's entry of the table, fetched across lanes)
                    const uint32_t item = uint32_t(__builtin_ctz(pending | 0x80000000u)), t = item >> 1, h = item & 1u;
                    const uint32_t row_at = uint32_t(__builtin_amdgcn_ds_bpermute(int(4 * (uint32_t(g * TG) + (t & uint32_t(TG - 1)))), int(row_table)));
                    if (pending) {
                        const uint16_t* row = src[0].x + int32_t(row_at);   // (a signed distance)
                        const float lit = xint_literal_block(row + (8 * d + 2 * G + h) * 16, h ? codes[j].z : codes[j].x, h ? codes[j].w : codes[j].y);
#pragma unroll
                        for (int q = 0; q < TG; ++q) {
                            dot[q][0] = item == uint32_t(2 * q) ? lit : dot[q][0];
                            dot[q][1] = item == uint32_t(2 * q + 1) ? lit : dot[q][1];
                        }
                        pending &= pending - 1;
                    }
                }
            }
            const float scale = xint_bf16_of(sdw[j], half), bias = xint_bf16_of(bdw[j], half);
#pragma unroll
            for (int t = 0; t < TG; ++t) {
                acc[g * TG + t][j][0] += scale * dot[t][0] + fi[buf][t].y * bias;
                acc[g * TG + t][j][1] += scale * dot[t][1] + fi[buf][t].w * bias;
            }
        }
    }
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
        float v[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float x0 = acc[t][0][h] + acc[t][2][h], x1 = acc[t][1][h] + acc[t][3][h];
            float sum = x0 + x1;
            sum = sum + __shfl_xor(sum, 32);
            sum = sum + __shfl_xor(sum, 16);
            v[h] = sum;
        }
        if (t < nt) emit(t, v[0] + v[1]);
    }
}
template <class Emit>
__device__ __forceinline__ void xint_run_tile_upto8(const uint8_t* w_row, const uint16_t* s_row, const uint16_t* b_row, uint32_t spans,
                                                    const uint8_t* const* img, const LdsBf16* src, const XintLayout L, uint32_t lane,
                                                    int nt, Emit emit) {
    if (nt <= 1) xint_run_tile_tokens_piped<1, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    else if (nt == 2) xint_run_tile_tokens_piped<2, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    else if (nt <= 4) xint_run_tile_tokens_piped<4, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    else xint_run_tile_tokens_piped<8, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
}
// Picks the instance for the number of live tokens: 1, 2 or 4 (the count is rounded up; padded tokens repeat image 0).
template <class Emit>
__device__ __forceinline__ void xint_run_tile_upto4(const uint8_t* w_row, const uint16_t* s_row, const uint16_t* b_row, uint32_t spans,
                                                    const uint8_t* const* img, const LdsBf16* src, const XintLayout L, uint32_t lane,
                                                    int nt, Emit emit) {
    if (nt <= 1) xint_run_tile_tokens<1, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    else if (nt == 2) xint_run_tile_tokens<2, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
    else xint_run_tile_tokens<4, 4>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit);
}

// A tile of 32 weight rows for NTOK <= 4 tokens on v_mfma_i32_32x32x32_i8, which costs a SIMD the same time as the
// 16x16x64 form and has four times the room: its 32 rows hold (token t, block c of two, plane p) as row 8 t + 4 c + p, its
// 32 k are two blocks (half wave h supplies block h of the pair), its 32 columns the tile's weight rows.  lane = (n = column,
// h = lane / 32).  Per span of 128 elements lane (n, h) fetches the 32 bytes of codes of blocks 4 h .. 4 h + 3 of weight row
// n; instruction i of the span multiplies blocks i and 4 + i; result elements 4 t .. 4 t + 2 of lane (n, h) are token t's
// three plane sums for block 4 h + i.  Reference lane 8 (d mod 4) + 4 h + i of the row is acc[t][d mod 4][i] of lane (n, h):
// per-lane accumulation order and the butterfly (strides 16 and 8 pair accumulators, 4 the half waves, 2 and 1 the
// blocks of a lane) are those of xint_run_tile_after, so the sums are the same bits.  Images beyond the live tokens are
// not read (their rows of the operand are zeros).
typedef int v16i __attribute__((ext_vector_type(16)));
template <int NTOK, class Source, class Emit>
__device__ __forceinline__ void xint_run_tile32(const uint8_t* w_row, const uint16_t* s_row, const uint16_t* b_row, uint32_t spans,
                                                const uint8_t* const* img, const Source* src, const XintLayout L, uint32_t lane,
                                                int nt, Emit emit) {
    static_assert(NTOK >= 1 && NTOK <= 4, "four tokens fill the instruction's rows");
    constexpr int R = 4;   // spans per body: one scale / bias vector of 16 bytes and one mask word per token
    const uint32_t h = lane >> 5, m = lane & 31u, t_a = m >> 3, c_a = (m >> 2) & 1u, p_a = m & 3u;
    const uint8_t* c = w_row + 32 * h;   // the lane's 32 bytes of each 64-byte span
    // codes travel two spans at a time (four 16-byte loads per lane in flight while the two spans before are multiplied), the
    // scale and bias vectors four spans at a time
    uint4 ring[4], sring, bring;
#pragma unroll
    for (int j = 0; j < 4; ++j) ring[j] = ldg_u4(c, (j / 2) * 4 + (j & 1));
    sring = ldg_u4(s_row, 0); bring = ldg_u4(b_row, 0);
    float acc[NTOK][4][4];
#pragma unroll
    for (int t = 0; t < NTOK; ++t)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[t][q][i] = 0;
    const uint32_t half = (lane & 32u) ? 0x03020c0cu : 0x01000c0cu;   // group 2d + h: the low BF16 of a dword for h = 0
    // left operand: row (t, c, p) of half wave h holds digit plane p of token t's block 4 h + i when c == h, zeros otherwise
    const bool live = c_a == h && p_a < 3 && t_a < uint32_t(nt);
    const uint8_t* a_image = img[0];
#pragma unroll
    for (int t = 1; t < NTOK; ++t) a_image = t_a == uint32_t(t) ? img[t] : a_image;
    const uint8_t* a_base = live ? a_image + 4 * h * 48 + p_a * 16 : img[0] + L.blocks() * 48;
    const uint32_t a_span = live ? 8 * 48 : 0, a_next = live ? 48 : 0;
    const uint32_t M = 0x0f0f0f0fu;
    v16i zero;
#pragma unroll
    for (int e = 0; e < 16; ++e) zero[e] = 0;
    const uint32_t info_at = L.planes_bytes() + 4 * h * 8, mask_at = L.planes_bytes() + L.info_bytes();
    // lane q < NTOK holds where token q's BF16 row starts, in elements from src[0]'s (a select chain over the tokens would be
    // turned into a table in memory by the compiler)
    uint32_t row_table = 0;
    if constexpr (Source::kRowInLds) {
#pragma unroll
        for (int q = 1; q < NTOK; ++q) row_table = lane == uint32_t(q) ? uint32_t(src[q].x - src[0].x) : row_table;
    }
    for (uint32_t d0 = 0; d0 < spans; d0 += R) {
        const uint32_t sdw[4] = {sring.x, sring.y, sring.z, sring.w}, bdw[4] = {bring.x, bring.y, bring.z, bring.w};
        if (d0 + R < spans) { sring = ldg_u4(s_row, (d0 + R) / 4); bring = ldg_u4(b_row, (d0 + R) / 4); }
        // the unsafe bits of the lane's blocks, per token: block 8 d + 4 h + i is bit 8 (d - d0) + 4 h + i of mask word d0 / 4
        uint32_t unsafe[NTOK], any = 0;
#pragma unroll
        for (int t = 0; t < NTOK; ++t) {
            unsafe[t] = t < nt ? (reinterpret_cast<const uint32_t*>(img[t] + mask_at)[d0 / 4] >> (4 * h)) & 0x0f0f0f0fu : 0u;
            any |= unsafe[t];
        }
        const bool literal_body = __ballot(any != 0) != 0;
#pragma unroll
        for (int part = 0; part < 2; ++part) {
            uint4 codes[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) codes[j] = ring[j];
            if (d0 + 2 * uint32_t(part) + 2 < spans) {
#pragma unroll
                for (int j = 0; j < 4; ++j) ring[j] = ldg_u4(c, (d0 + 2 * uint32_t(part) + 2 + j / 2) * 4 + (j & 1));
            }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            const int j = 2 * part + jj;
            const uint32_t d = d0 + uint32_t(j);
            const uint32_t words[8] = {codes[2 * jj].x, codes[2 * jj].y, codes[2 * jj].z, codes[2 * jj].w,
                                       codes[2 * jj + 1].x, codes[2 * jj + 1].y, codes[2 * jj + 1].z, codes[2 * jj + 1].w};
            float dot[NTOK][4], bsum[NTOK][4];
#pragma unroll
            for (int t = 0; t < NTOK; ++t) {
                const uint8_t* image = t < nt ? img[t] : img[0];   // (two fixed elements, not an index formed at run time: the array stays in registers)
                const float4 f0 = *reinterpret_cast<const float4*>(image + info_at + d * 64);        // {2^e, sum} of blocks 4h, 4h+1
                const float4 f1 = *reinterpret_cast<const float4*>(image + info_at + d * 64 + 16);   // of blocks 4h+2, 4h+3
                dot[t][0] = f0.x; bsum[t][0] = f0.y; dot[t][1] = f0.z; bsum[t][1] = f0.w;
                dot[t][2] = f1.x; bsum[t][2] = f1.y; dot[t][3] = f1.z; bsum[t][3] = f1.w;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const v4i b = {int(words[2 * i] & M), int((words[2 * i] >> 4) & M), int(words[2 * i + 1] & M), int((words[2 * i + 1] >> 4) & M)};
                const v4i a = *reinterpret_cast<const v4i*>(a_base + d * a_span + uint32_t(i) * a_next);
                const v16i r = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, zero, 0, 0, 0);
#pragma unroll
                for (int t = 0; t < NTOK; ++t) {
                    const v4i planes = {r[4 * t], r[4 * t + 1], r[4 * t + 2], 0};
                    dot[t][i] = float(xint_digits(planes)) * dot[t][i];
                }
                if constexpr (!Source::kRowInLds) {
                    if (__builtin_expect(literal_body, 0)) {
#pragma unroll
                        for (int t = 0; t < NTOK; ++t)
                            if ((unsafe[t] >> (8 * j + i)) & 1u) dot[t][i] = xint_literal_dot(b, src[t], 8 * d + 4 * h + uint32_t(i));
                    }
                }
            }
            if constexpr (Source::kRowInLds) {
                // BF16 rows in LDS: ONE loop serves the literal chains of all tokens and blocks of the span, every lane taking its
                // next unsafe (token, block) in turn (bit 4 t + i), so the chain's code exists once per span
                if (__builtin_expect(literal_body, 0)) {
                    uint32_t pending = 0;
#pragma unroll
                    for (int t = 0; t < NTOK; ++t) pending |= ((unsafe[t] >> (8 * j)) & 15u) << (4 * t);
                    while (__ballot(pending != 0) != 0) {
                        // (every lane is active here: the row of token t is lane t's entry of the table, fetched across lanes)
                        const uint32_t item = uint32_t(__builtin_ctz(pending | 0x80000000u)), t = (item >> 2) & uint32_t(NTOK - 1), i = item & 3u;
                        const uint32_t row_at = uint32_t(__builtin_amdgcn_ds_bpermute(int(4 * t), int(row_table)));
                        if (pending) {
                            const uint16_t* row = src[0].x + int32_t(row_at);   // (a signed distance)
                            uint32_t lo = words[0], hi = words[1];
#pragma unroll
                            for (int q = 1; q < 4; ++q) { lo = i == uint32_t(q) ? words[2 * q] : lo; hi = i == uint32_t(q) ? words[2 * q + 1] : hi; }
                            const float lit = xint_literal_block(row + (8 * d + 4 * h + i) * 16, lo, hi);
#pragma unroll
                            for (int q = 0; q < NTOK; ++q)
#pragma unroll
                                for (int ii = 0; ii < 4; ++ii) dot[q][ii] = item == uint32_t(4 * q + ii) ? lit : dot[q][ii];
                            pending &= pending - 1;
                        }
                    }
                }
            }
            const float scale = xint_bf16_of(sdw[j], half), bias = xint_bf16_of(bdw[j], half);
#pragma unroll
            for (int t = 0; t < NTOK; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[t][j][i] += scale * dot[t][i] + bsum[t][i] * bias;
        }
        }
    }
#pragma unroll
    for (int t = 0; t < NTOK; ++t) {
        float z[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float x0 = acc[t][0][i] + acc[t][2][i], x1 = acc[t][1][i] + acc[t][3][i];
            const float y = x0 + x1;
            z[i] = y + __shfl_xor(y, 32);
        }
        const float w0 = z[0] + z[2], w1 = z[1] + z[3];
        if (t < nt) emit(t, w0 + w1);
    }
}

template <int PT, int R, class Source, class Emit>
__device__ __forceinline__ void xint_run_tile(const uint8_t* w_row, const uint16_t* s_row, const uint16_t* b_row, uint32_t spans,
                                              const uint8_t* const* img, const Source* src, const XintLayout L, uint32_t lane,
                                              int nt, Emit emit) {
    xint_run_tile_after<PT, R>(w_row, s_row, b_row, spans, img, src, L, lane, nt, emit, []() {});
}

}  // namespace zc
