// Device-side arithmetic primitives shared by every kernel of the MoE path.
// All code here is compiled with -ffp-contract=off: a*b+c is two roundings
// unless written as __builtin_fmaf, exactly as the arithmetic is specified.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace zc {

// Round to nearest even to BF16, kept in fp32 (reference: qwen.metal:17-21).
__device__ __forceinline__ float bf(float x) {
    const uint32_t u = __float_as_uint(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return __uint_as_float(0x7fc00000u);
    return __uint_as_float((u + 0x7fffu + ((u >> 16) & 1u)) & 0xffff0000u);
}
__device__ __forceinline__ float b16(uint16_t h) { return __uint_as_float(uint32_t(h) << 16); }

// exp in plain fp32 operations so that host and device agree bit for bit:
// n = rint(x*log2 e), r = x - n*ln2 (two constants), degree-5 polynomial in r on
// r*r, then two exact power-of-two scalings.  x < -87 gives 0 (no subnormals).
__device__ __forceinline__ float exp32(float x) {
    if (x != x) return x;
    if (x > 88.72283f) return __uint_as_float(0x7f800000u);
    if (x < -87.0f) return 0.0f;
    const float n = __builtin_rintf(x * 1.44269504088896341f);
    float r = __builtin_fmaf(n, -0.693359375f, x);
    r = __builtin_fmaf(n, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    const float y = __builtin_fmaf(p, r * r, r) + 1.0f;
    const int ni = int(n), a = ni / 2, b = ni - a;
    return y * __uint_as_float(uint32_t(a + 127) << 23) * __uint_as_float(uint32_t(b + 127) << 23);
}
// BF16 sigmoid with a rounding after the exponential, the sum and the reciprocal
// (reference: qwen.metal:33-35).
__device__ __forceinline__ float sigmoid_bf(float x) {
    const float y = bf(1.0f / bf(1.0f + bf(exp32(__builtin_fabsf(x)))));
    return x < 0 ? y : bf(1.0f - y);
}
// SwiGLU epilogue of the fused gate/up product (reference: qwen.metal:78-80).
__device__ __forceinline__ float swiglu_bf(float gate_sum, float up_sum) {
    const float g = bf(gate_sum), u = bf(up_sum);
    return bf(bf(g * sigmoid_bf(g)) * u);
}

// Sum over the 32 reference lanes as an xor butterfly with strides 16,8,4,2,1.
// A 64-lane wavefront carries two independent 32-lane groups; strides below 32
// never cross between them.  Every lane of a group ends with the same value.
__device__ __forceinline__ float lane_sum32(float v) {
    v = v + __shfl_xor(v, 16);
    v = v + __shfl_xor(v, 8);
    v = v + __shfl_xor(v, 4);
    v = v + __shfl_xor(v, 2);
    v = v + __shfl_xor(v, 1);
    return v;
}

// Read-only data in device memory, addressed in the GLOBAL address space.  A pointer that
// was itself loaded from memory is generic to the compiler; generic loads share the LDS
// wait counter, so waiting for an LDS read would also wait for every weight prefetch.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <class T> using gptr = const T __attribute__((address_space(1)))*;
template <class T> __device__ __forceinline__ gptr<T> as_global(const void* p) { return (gptr<T>)(uintptr_t)p; }
__device__ __forceinline__ uint4 ldg_u4(const void* p, uint32_t index = 0) {
    const u32x4 v = as_global<u32x4>(p)[index];
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 ldg_u2(const void* p, uint32_t index = 0) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 v = as_global<u32x2>(p)[index];
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint16_t ldg_u16(const void* p, uint32_t index = 0) { return as_global<uint16_t>(p)[index]; }
__device__ __forceinline__ uint32_t ldg_u32(const void* p, uint32_t index = 0) { return as_global<uint32_t>(p)[index]; }
__device__ __forceinline__ float ldg_f32(const void* p, uint32_t index = 0) { return as_global<float>(p)[index]; }

// DPP moves inside rows of 16 lanes.  row_shr:1 hands lane i the value of lane i-1
// (0 for the first lane of a row); the xor patterns are permutations.
__device__ __forceinline__ float dpp_row_shr1(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x111, 0xf, 0xf, true));
}
template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// Maximum over the 64 lanes, returned in every lane: four DPP steps inside each row
// (quad swaps, half mirror, mirror), then the four row values through scalar lanes.
__device__ __forceinline__ float wave_max_f32(float v) {
    v = fmaxf(v, dpp_f32<0xb1>(v));    // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_f32<0x4e>(v));    // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_f32<0x141>(v));   // row_half_mirror
    v = fmaxf(v, dpp_f32<0x140>(v));   // row_mirror
    const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// splitmix64 finaliser: the counter-based generator behind every synthetic tensor.
__host__ __device__ inline uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
// Element i of stream `seed`: independent of every other element.
__host__ __device__ inline uint64_t hash64(uint64_t seed, uint64_t i) {
    return mix64(mix64(seed ^ 0x5EEDC0DE5EEDC0DEull) + (i + 1) * 0x9E3779B97F4A7C15ull);
}

}  // namespace zc
