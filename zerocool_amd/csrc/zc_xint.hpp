// Exact-integer evaluation of the affine Q4 dot on the matrix cores.
//
// The reference evaluates a row as 32 lanes, each summing `scale*dot + sum*bias` over
// its 16-element blocks, where `dot` is an fp32 chain over the block.  For BF16-valued
// inputs every product x*q (8-bit by 4-bit significands) is exact, and when all
// partial sums of a block fit 24 bits the whole chain is exact: `dot` then equals the
// true sum, whatever the order.  Such a block is computed here in integers:
//   x_k = X_k * 2^e   (e = smallest exponent in the block, X_k integer, |X_k| < 2^21)
//   X_k = d0 + 2^7 d1 + 2^14 d2  (signed 7-bit digits, sign of x_k)
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
    __host__ __device__ uint32_t blocks() const { return K / 16; }
    __host__ __device__ uint32_t planes_bytes() const { return blocks() * 48 + 16; }   // + one zero slot
    __host__ __device__ uint32_t info_bytes() const { return blocks() * 8; }
    __host__ __device__ uint32_t mask_bytes() const { return (blocks() + 31) / 32 * 4; }
    __host__ __device__ uint32_t bytes() const { return (planes_bytes() + info_bytes() + mask_bytes() + 15) / 16 * 16; }
};

// Byte t of a lane's 16-byte operand holds block element kOrder[t]: the order in which
// (w & 0x0f0f0f0f), ((w >> 4) & 0x0f0f0f0f) of the block's two code words lay nibbles out.
__device__ __forceinline__ uint32_t xint_element_of_byte(uint32_t t) {
    return (t & 8u) + ((t & 3u) << 1) + ((t >> 2) & 1u);
}

// Loads with agent scope: inputs may have been written by another workgroup of a
// persistent kernel, so they must not come from a stale cache line.
__device__ __forceinline__ float load_shared_f32(const float* p) {
    return __uint_as_float(__hip_atomic_load(reinterpret_cast<const uint32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

// Input sources.  bits(k) returns the fp32 bit pattern of element k.
struct GlobalF32 {   // a row in global memory, possibly written by another workgroup
    const float* x;
    __device__ __forceinline__ uint32_t bits(uint32_t k) const { return __float_as_uint(load_shared_f32(x + k)); }
    __device__ __forceinline__ float at(uint32_t k) const { return load_shared_f32(x + k); }
};
struct LdsBf16 {     // a BF16 copy of the row in LDS
    const uint16_t* x;
    __device__ __forceinline__ uint32_t bits(uint32_t k) const { return uint32_t(x[k]) << 16; }
    __device__ __forceinline__ float at(uint32_t k) const { return b16(x[k]); }
};

// Builds the LDS image of a K-element row cooperatively (all threads of the workgroup
// call it, then __syncthreads()).  One thread per block.
template <class Source>
__device__ __forceinline__ void xint_prepare(const Source x, const XintLayout L, uint8_t* lds) {
    uint8_t* planes = lds;
    float2* info = reinterpret_cast<float2*>(lds + L.planes_bytes());
    uint32_t* mask = reinterpret_cast<uint32_t*>(lds + L.planes_bytes() + L.info_bytes());
    for (uint32_t i = threadIdx.x; i < L.mask_bytes() / 4; i += blockDim.x) mask[i] = 0;
    if (threadIdx.x < 4) reinterpret_cast<uint32_t*>(planes + L.blocks() * 48)[threadIdx.x] = 0;
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < L.blocks(); b += blockDim.x) {
        uint32_t bits[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) bits[i] = x.bits(b * 16 + i);
        // bias sum: BF16 rounding after each addition of four inputs (reference: qwen.metal:55)
        float sum = 0;
#pragma unroll
        for (int i = 0; i < 16; i += 4)
            sum += bf(bf(bf(__uint_as_float(bits[i]) + __uint_as_float(bits[i + 1])) + __uint_as_float(bits[i + 2])) + __uint_as_float(bits[i + 3]));
        uint32_t emin = 255, lowbits = 0, special = 0;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t e = (bits[i] >> 23) & 255u, m = bits[i] & 0x7fffffu;
            lowbits |= bits[i] & 0xffffu;
            special |= (e == 255u);
            if (e | m) emin = min(emin, max(e, 1u));
        }
        if (emin == 255) emin = 1;   // all zero
        uint32_t sumabs = 0, over = 0;
        uint32_t mag[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t e = (bits[i] >> 23) & 255u;
            const uint32_t sig = ((e ? 128u : 0u) | ((bits[i] >> 16) & 127u));
            const uint32_t shift = max(e, 1u) - emin;
            over |= (shift > 13u);
            mag[i] = sig << min(shift, 13u);
            sumabs += mag[i];
        }
        const bool safe = !lowbits && !special && !over && 15u * sumabs < (1u << 24);
        uint32_t words[3][4] = {};
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const uint32_t i = xint_element_of_byte(t);
            const uint32_t neg = bits[i] >> 31;
#pragma unroll
            for (int p = 0; p < 3; ++p) {
                const uint32_t d = (mag[i] >> (7 * p)) & 127u;
                const uint32_t byte = (neg ? (0u - d) : d) & 255u;
                words[p][t / 4] |= byte << (8 * (t % 4));
            }
        }
        if (!safe) { for (int p = 0; p < 3; ++p) for (int q = 0; q < 4; ++q) words[p][q] = 0; atomicOr(mask + b / 32, 1u << (b % 32)); }
#pragma unroll
        for (int p = 0; p < 3; ++p)
            *reinterpret_cast<uint4*>(planes + b * 48 + p * 16) = make_uint4(words[p][0], words[p][1], words[p][2], words[p][3]);
        // 2^(emin-134): x = sig * 2^(e-127-7)
        const int ex = int(emin) - 134;
        const float scale = ex >= -126 ? __uint_as_float(uint32_t(ex + 127) << 23) : __uint_as_float(1u << (ex + 149));
        info[b] = make_float2(scale, sum);
    }
}

// The literal fp32 chain of one block (reference: qwen.metal:52-57) for a lane that
// holds the block's two code words.
template <class Source>
__device__ __forceinline__ float xint_literal_dot(uint32_t w0, uint32_t w1, const Source x, uint32_t k0) {
    float dot = 0;
#pragma unroll
    for (int i = 0; i < 16; i += 4) {
        const uint32_t packed = ((i < 8 ? w0 : w1) >> (4 * (i % 8))) & 0xffffu;
        dot += x.at(k0 + i) * float(packed & 15u) + x.at(k0 + i + 1) * float((packed >> 4) & 15u) +
               x.at(k0 + i + 2) * float((packed >> 8) & 15u) + x.at(k0 + i + 3) * float((packed >> 12) & 15u);
    }
    return dot;
}

// Per-lane state of one 16-row tile: lane = (j = row in tile, G = lane / 16).
// Processes NT tokens at once; acc[t][m][h] is the running sum of reference lane
// 8*m + 2*G + h of row j.
template <int NT>
struct XintTile {
    float acc[NT][4][2];
    __device__ __forceinline__ void clear() {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int m = 0; m < 4; ++m) { acc[t][m][0] = 0; acc[t][m][1] = 0; }
    }
    // One 128-element span `dg` of the row: codes = the lane's 16 bytes (blocks 2G, 2G+1),
    // scale/bias = the row's group values for group 2*dg + G/2.
    // nt <= NT tokens are live (wave-uniform); lds[t] / x[t] are token t's image and source.
    template <class Source>
    __device__ __forceinline__ void step(uint32_t dg, const uint4 codes, float scale, float bias, const uint8_t* const* lds,
                                         const XintLayout L, const Source* x, uint32_t lane, int nt = NT) {
        const uint32_t G = lane >> 4, i = lane & 15u, c = i >> 2, p = i & 3u;
        const uint32_t M = 0x0f0f0f0fu;
        v4i b0 = {int(codes.x & M), int((codes.x >> 4) & M), int(codes.y & M), int((codes.y >> 4) & M)};
        v4i b1 = {int(codes.z & M), int((codes.z >> 4) & M), int(codes.w & M), int((codes.w >> 4) & M)};
        const uint32_t blk = 8 * dg + 2 * G;                 // this lane's result blocks: blk, blk+1
        const uint32_t ablk = 8 * dg + 2 * (c == G ? G : 0); // A rows: plane p of block 2c(+h) in lane group c
        const bool live = (c == G) && p < 3;
        const uint32_t zero_slot = L.blocks() * 48;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            if (t >= nt) break;
            const uint8_t* planes = lds[t];
            const float2* info = reinterpret_cast<const float2*>(planes + L.planes_bytes());
            const uint32_t* mask = reinterpret_cast<const uint32_t*>(planes + L.planes_bytes() + L.info_bytes());
            const v4i a0 = *reinterpret_cast<const v4i*>(planes + (live ? ablk * 48 + p * 16 : zero_slot));
            const v4i a1 = *reinterpret_cast<const v4i*>(planes + (live ? (ablk + 1) * 48 + p * 16 : zero_slot));
            const v4i z = {0, 0, 0, 0};
            const v4i d0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b0, z, 0, 0, 0);
            const v4i d1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b1, z, 0, 0, 0);
            const uint32_t unsafe = (mask[blk / 32] >> (blk % 32)) & 3u;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const v4i d = h ? d1 : d0;
                const float2 fi = info[blk + h];
                float dot = float(d[0] + (d[1] << 7) + (d[2] << 14)) * fi.x;
                if (unsafe & (1u << h)) dot = xint_literal_dot(h ? codes.z : codes.x, h ? codes.w : codes.y, x[t], (blk + h) * 16);
                acc[t][dg & 3u][h] += scale * dot + fi.y * bias;
            }
        }
    }
    // Reference lane sum (xor butterfly 16, 8, 4, 2, 1) of token t; every lane of row j returns it.
    __device__ __forceinline__ float finish(int t) const {
        float v[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float a0 = acc[t][0][h] + acc[t][2][h], a1 = acc[t][1][h] + acc[t][3][h];   // stride 16
            float s = a0 + a1;                                                                    // stride 8
            s = s + __shfl_xor(s, 32);                                                            // stride 4
            s = s + __shfl_xor(s, 16);                                                            // stride 2
            v[h] = s;
        }
        return v[0] + v[1];                                                                       // stride 1
    }
};

}  // namespace zc
