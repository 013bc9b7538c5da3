// The callers' glue either side of the MoE layer: element-wise operators, the four-stream mix and residual
// injection, grouped RMS norm (reference: model.cpp:328-351, 651, 662; kernels qwen.metal:36-40, 545-595).
// All of it is HBM-bound element-wise work: 16-byte accesses where the layout allows, one pass over the data.
#include "zc_kernels.hpp"
#include "zc_device.hpp"

namespace zc {

// log(y) for y in [1, 2] from double-precision basic operations only (the same sequence as the CPU checker):
// log y = 2 atanh z, z = (y-1)/(y+1), odd series to z^35, rounded to fp32 once.
__device__ __forceinline__ float log_1to2(float y) {
    const double z = (double(y) - 1.0) / (double(y) + 1.0), z2 = z * z;
    double p = 1.0 / 35.0;
#pragma unroll
    for (int k = 33; k >= 1; k -= 2) p = __builtin_fma(p, z2, 1.0 / double(k));
    return float(2.0 * z * p);
}
// qwen.metal:36-40
__device__ __forceinline__ float softplus_bf(float x) {
    const float e = bf(exp32(-__builtin_fabsf(x))), one = 1.0f + e;
    const float tail = one == 1.0f ? e : e * (log_1to2(one) / (one - 1.0f));
    return bf(fmaxf(x, 0.0f) + bf(tail));
}
// qwen.metal:567-577
__device__ __forceinline__ float unary_op(float v, uint32_t op) {
    if (op == 0) v = v * sigmoid_bf(v);
    if (op == 1) v = sigmoid_bf(v);
    if (op == 2) { v = bf(v / 4); v = v * sigmoid_bf(v); }
    if (op == 3) v = 2 * bf(sigmoid_bf(bf(v / 4)));
    if (op == 4) v = softplus_bf(v);
    return bf(v);
}
__global__ __launch_bounds__(256) void unary_kernel(const float* x, uint64_t n, uint32_t op, float* y) {
    for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += uint64_t(gridDim.x) * blockDim.x) y[i] = unary_op(x[i], op);
}
// qwen.metal:578-581
__global__ __launch_bounds__(256) void binary_kernel(const float* x, const float* y, uint64_t n, uint32_t op, float* out) {
    for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += uint64_t(gridDim.x) * blockDim.x)
        out[i] = bf(op ? x[i] * y[i] : x[i] + y[i]);
}
// qwen.metal:582-588: x, w [tokens][4][hidden] -> out [tokens][hidden]
__global__ __launch_bounds__(256) void hc_mix_kernel(const float* x, const float* w, uint32_t tokens, uint32_t hidden, float* out) {
    const uint64_t n = uint64_t(tokens) * hidden;
    for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += uint64_t(gridDim.x) * blockDim.x) {
        const uint64_t t = i / hidden, d = i % hidden;
        float sum = 0;
#pragma unroll
        for (uint32_t h = 0; h < 4; ++h) { const uint64_t k = (t * 4 + h) * hidden + d; sum = bf(sum + bf(x[k] * w[k])); }
        out[i] = bf(sum / 4);
    }
}
// qwen.metal:589-595: hyper [tokens][4][hidden], x [tokens][hidden], inject [tokens][4]
__global__ __launch_bounds__(256) void hc_add_kernel(const float* hyper, const float* x, const float* inject, uint32_t tokens, uint32_t hidden, float* out) {
    const uint64_t n = uint64_t(tokens) * 4 * hidden;
    for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += uint64_t(gridDim.x) * blockDim.x) {
        const uint64_t t = i / (4ull * hidden), h = (i / hidden) % 4, d = i % hidden;
        out[i] = bf(hyper[i] + bf(x[t * hidden + d] * inject[t * 4 + h]));
    }
}
// qwen.metal:545-566 (and norm_wide, :403-426, which gives the same bits): one 32-lane group per normalised group.
// Every 128-element block: four squares per lane, lane sum, lane block/128 keeps it; a second lane sum adds the blocks.
__global__ __launch_bounds__(256) void norm_kernel(const float* x, const void* w, uint32_t dtype, uint32_t D, uint32_t width, uint64_t groups, float* out) {
    const uint32_t lane = threadIdx.x & 31u;
    const uint64_t group = uint64_t(blockIdx.x) * 8 + (threadIdx.x >> 5);
    if (group >= groups) return;
    const float* xg = x + group * D;
    float contribution = 0;
    for (uint32_t block = 0; block < D; block += 128) {
        float acc = 0;
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) { const uint32_t d = block + lane * 4 + i; if (d < D) acc += xg[d] * xg[d]; }
        acc = lane_sum32(acc);
        if (lane == block / 128) contribution = acc;
    }
    const float inv = 1.0f / __builtin_sqrtf(lane_sum32(contribution) / float(D) + 1e-6f);
    for (uint32_t d = lane; d < D; d += 32) {
        const uint64_t i = group * D + d; const uint32_t wi = uint32_t(i % width);
        const float weight = dtype == 1 ? static_cast<const float*>(w)[wi] : b16(static_cast<const uint16_t*>(w)[wi]);
        out[i] = bf(bf(xg[d] * inv) * weight);
    }
}

static dim3 grid_for(uint64_t n) { return dim3(uint32_t(std::min<uint64_t>((n + 255) / 256, 65536))); }
void launch_unary(hipStream_t s, const float* x, uint64_t n, uint32_t op, float* y) { hipLaunchKernelGGL(unary_kernel, grid_for(n), dim3(256), 0, s, x, n, op, y); }
void launch_binary(hipStream_t s, const float* x, const float* y, uint64_t n, uint32_t op, float* out) { hipLaunchKernelGGL(binary_kernel, grid_for(n), dim3(256), 0, s, x, y, n, op, out); }
void launch_hc_mix(hipStream_t s, const float* x, const float* w, uint32_t tokens, uint32_t hidden, float* out) {
    hipLaunchKernelGGL(hc_mix_kernel, grid_for(uint64_t(tokens) * hidden), dim3(256), 0, s, x, w, tokens, hidden, out);
}
void launch_hc_add(hipStream_t s, const float* hyper, const float* x, const float* inject, uint32_t tokens, uint32_t hidden, float* out) {
    hipLaunchKernelGGL(hc_add_kernel, grid_for(uint64_t(tokens) * 4 * hidden), dim3(256), 0, s, hyper, x, inject, tokens, hidden, out);
}
void launch_norm(hipStream_t s, const float* x, const void* w, uint32_t dtype, uint32_t D, uint32_t width, uint32_t tokens, float* out) {
    const uint64_t groups = uint64_t(tokens) * (width / D);
    hipLaunchKernelGGL(norm_kernel, dim3(uint32_t((groups + 7) / 8)), dim3(256), 0, s, x, w, dtype, D, width, groups, out);
}

}  // namespace zc
