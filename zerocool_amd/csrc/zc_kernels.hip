// Operator kernels of the MoE path with the reference's arithmetic kept literally:
// the 32-lane partition of every affine dot, the scalar order inside a lane, every
// BF16 rounding boundary.  One GPU lane plays one reference lane, so a 64-lane
// wavefront carries two output rows.  Results are bit-identical to the CPU statement
// of the same arithmetic for any input.
#include "zc_kernels.hpp"
#include <type_traits>
#include "zc_device.hpp"

namespace zc {

// ---------------------------------------------------------------------------
// Affine Q4 / Q8 rows (reference: qwen.metal:46-81, 112-144)
// ---------------------------------------------------------------------------
// WIDTH = elements one lane takes per step: Q4 16|8, Q8 8|4; always 1 or 2 dwords.
template <int BITS, int WIDTH>
struct Block {
    static constexpr int DW = WIDTH * BITS / 32;
    // x-only part of the bias term.
    __device__ static float xsum(const float* xb) {
        float sum = 0;
        if constexpr (BITS == 4) {
#pragma unroll
            for (int i = 0; i < WIDTH; i += 4) sum += bf(bf(bf(xb[i] + xb[i + 1]) + xb[i + 2]) + xb[i + 3]);
        } else {
#pragma unroll
            for (int i = 0; i < WIDTH; ++i) sum += xb[i];
        }
        return sum;
    }
    __device__ static float dot(const uint32_t* words, const float* xb) {
        float dot = 0;
        if constexpr (BITS == 4) {
#pragma unroll
            for (int i = 0; i < WIDTH; i += 4) {
                const uint32_t packed = (words[i / 8] >> (4 * (i % 8))) & 0xffffu;
                dot += xb[i] * float(packed & 15u) + xb[i + 1] * float((packed >> 4) & 15u) +
                       xb[i + 2] * float((packed >> 8) & 15u) + xb[i + 3] * float((packed >> 12) & 15u);
            }
        } else {
#pragma unroll
            for (int i = 0; i < WIDTH; ++i) dot += xb[i] * float((words[i / 4] >> (8 * (i % 4))) & 255u);
        }
        return dot;
    }
};

struct AffineJob {
    const uint8_t *w0, *w1;          // gate (or the only matrix), up
    const uint16_t *s0, *b0, *s1, *b1;
    const float* x;                  // input rows, K floats each
    const int32_t* in_rows;          // gather of input rows, or null
    const int32_t* out_rows;         // scatter of output rows, or null
    float* out;                      // output rows, N floats each
    uint32_t K, N, group, tokens;
    uint32_t float_output;
};

constexpr int kRowsPerBlock = 8;     // 256 threads = 8 groups of 32 reference lanes

template <int BITS, int WIDTH, bool GATED>
__device__ __forceinline__ void affine_rows(const AffineJob& j, uint32_t tile, float* lds_x, float* lds_sum) {
    using B = Block<BITS, WIDTH>;
    const uint32_t tid = threadIdx.x, lane = tid & 31u, row = tile * kRowsPerBlock + (tid >> 5);
    const uint32_t K = j.K, blocks = K / WIDTH, groups = K / j.group;
    const uint32_t row_dwords = K * BITS / 32;
    for (uint32_t t = 0; t < j.tokens; ++t) {
        const float* xr = j.x + uint64_t(j.in_rows ? uint32_t(j.in_rows[t]) : t) * K;
        __syncthreads();
        for (uint32_t i = tid; i < K / 4; i += blockDim.x)
            reinterpret_cast<float4*>(lds_x)[i] = reinterpret_cast<const float4*>(xr)[i];
        __syncthreads();
        for (uint32_t b = tid; b < blocks; b += blockDim.x) lds_sum[b] = B::xsum(lds_x + b * WIDTH);
        __syncthreads();
        if (row >= j.N) continue;
        float r0 = 0, r1 = 0;
        const uint32_t* w0 = reinterpret_cast<const uint32_t*>(j.w0) + uint64_t(row) * row_dwords;
        const uint32_t* w1 = GATED ? reinterpret_cast<const uint32_t*>(j.w1) + uint64_t(row) * row_dwords : nullptr;
        for (uint32_t b = lane; b < blocks; b += 32) {
            uint32_t q0[B::DW], q1[B::DW];
#pragma unroll
            for (int d = 0; d < B::DW; ++d) {
                q0[d] = w0[b * B::DW + d];
                if constexpr (GATED) q1[d] = w1[b * B::DW + d];
            }
            float xb[WIDTH];
#pragma unroll
            for (int i = 0; i < WIDTH; i += 4) {
                const float4 v = *reinterpret_cast<const float4*>(lds_x + b * WIDTH + i);
                xb[i] = v.x; xb[i + 1] = v.y; xb[i + 2] = v.z; xb[i + 3] = v.w;
            }
            const uint32_t g = row * groups + (b * WIDTH) / j.group;
            const float sum = lds_sum[b];
            r0 += b16(j.s0[g]) * B::dot(q0, xb) + sum * b16(j.b0[g]);
            if constexpr (GATED) r1 += b16(j.s1[g]) * B::dot(q1, xb) + sum * b16(j.b1[g]);
        }
        r0 = lane_sum32(r0);
        if constexpr (GATED) r1 = lane_sum32(r1);
        if (lane == 0) {
            float* o = j.out + uint64_t(j.out_rows ? uint32_t(j.out_rows[t]) : t) * j.N + row;
            if constexpr (GATED) *o = swiglu_bf(r0, r1);
            else *o = j.float_output ? r0 : bf(r0);
        }
    }
}

template <int BITS, int WIDTH, bool GATED>
__global__ __launch_bounds__(256) void affine_op_kernel(AffineJob j) {
    extern __shared__ float lds[];
    affine_rows<BITS, WIDTH, GATED>(j, blockIdx.x, lds, lds + j.K);
}

// Routed experts of one layer: blockIdx.y walks the selected experts that the
// dispatch kernel listed; jobs past the device-side count exit at once.
struct ExpertPhase {
    const uint8_t* records; uint64_t stride;
    uint64_t w0, s0, b0, w1, s1, b1;     // byte offsets inside a record
    const int32_t *offsets, *selected, *count;
    const int32_t *in_rows, *out_rows;   // indexed by sorted slot; either may be null
    const float* x; float* out;          // x: layer input (gate/up) or sorted activations (down)
    uint32_t K, N, group, x_sorted;      // x_sorted: x rows follow the sorted slot order
};
template <int BITS, int WIDTH, bool GATED>
__global__ __launch_bounds__(256) void expert_phase_kernel(ExpertPhase p) {
    extern __shared__ float lds[];
    const uint32_t job = blockIdx.y;
    if (int32_t(job) >= *p.count) return;
    const int32_t e = p.selected[job], first = p.offsets[e], n = p.offsets[e + 1] - first;
    const uint8_t* r = p.records + uint64_t(e) * p.stride;
    AffineJob j;
    j.w0 = r + p.w0; j.s0 = reinterpret_cast<const uint16_t*>(r + p.s0); j.b0 = reinterpret_cast<const uint16_t*>(r + p.b0);
    j.w1 = r + p.w1; j.s1 = reinterpret_cast<const uint16_t*>(r + p.s1); j.b1 = reinterpret_cast<const uint16_t*>(r + p.b1);
    j.x = p.x_sorted ? p.x + uint64_t(first) * p.K : p.x;
    j.in_rows = p.in_rows ? p.in_rows + first : nullptr;
    j.out_rows = p.out_rows ? p.out_rows + first : nullptr;
    j.out = p.out_rows ? p.out : p.out + uint64_t(first) * p.N;
    j.K = p.K; j.N = p.N; j.group = p.group; j.tokens = uint32_t(n); j.float_output = 0;
    affine_rows<BITS, WIDTH, GATED>(j, blockIdx.x, lds, lds + p.K);
}

static bool wide(uint32_t K, uint32_t N) { return K % 512 == 0 && N % 8 == 0; }

template <bool GATED, typename Launch>
static void by_format(uint32_t bits, bool w, Launch&& launch) {
    if (bits == 4) { if (w) launch.template operator()<4, 16, GATED>(); else launch.template operator()<4, 8, GATED>(); }
    else           { if (w) launch.template operator()<8, 8, GATED>();  else launch.template operator()<8, 4, GATED>(); }
}

void launch_affine(hipStream_t s, const AffineDesc& a) {
    AffineJob j{};
    j.w0 = (const uint8_t*)a.gate.weight; j.s0 = (const uint16_t*)a.gate.scales; j.b0 = (const uint16_t*)a.gate.biases;
    if (a.gated) { j.w1 = (const uint8_t*)a.up.weight; j.s1 = (const uint16_t*)a.up.scales; j.b1 = (const uint16_t*)a.up.biases; }
    j.x = a.x; j.in_rows = a.in_rows; j.out_rows = a.out_rows; j.out = a.out;
    j.K = a.gate.input; j.N = a.gate.output; j.group = a.gate.group; j.tokens = a.tokens; j.float_output = a.float_output;
    const dim3 grid((j.N + kRowsPerBlock - 1) / kRowsPerBlock);
    const size_t lds = size_t(j.K) * 4 + size_t(j.K / 4) * 4;
    auto go = [&]<int BITS, int WIDTH, bool GATED>() {
        hipLaunchKernelGGL((affine_op_kernel<BITS, WIDTH, GATED>), grid, dim3(256), lds, s, j);
    };
    if (a.gated) by_format<true>(a.gate.bits, wide(j.K, j.N), go);
    else by_format<false>(a.gate.bits, wide(j.K, j.N), go);
}

void launch_expert_phase(hipStream_t s, const ExpertPhaseDesc& d) {
    ExpertPhase p{};
    p.records = (const uint8_t*)d.records; p.stride = d.stride;
    p.w0 = d.off[0]; p.s0 = d.off[1]; p.b0 = d.off[2]; p.w1 = d.off[3]; p.s1 = d.off[4]; p.b1 = d.off[5];
    p.offsets = d.offsets; p.selected = d.selected; p.count = d.count;
    p.in_rows = d.in_rows; p.out_rows = d.out_rows; p.x = d.x; p.out = d.out;
    p.K = d.K; p.N = d.N; p.group = d.group; p.x_sorted = d.x_sorted;
    const dim3 grid((d.N + kRowsPerBlock - 1) / kRowsPerBlock, d.max_jobs);
    const size_t lds = size_t(d.K) * 4 + size_t(d.K / 4) * 4;
    auto go = [&]<int BITS, int WIDTH, bool GATED>() {
        hipLaunchKernelGGL((expert_phase_kernel<BITS, WIDTH, GATED>), grid, dim3(256), lds, s, p);
    };
    if (d.gated) by_format<true>(d.bits, wide(d.K, d.N), go);
    else by_format<false>(d.bits, wide(d.K, d.N), go);
}

// ---------------------------------------------------------------------------
// Plain (unquantised) rows: lane chain k = lane + 32 j (reference: qwen.metal:499-506)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void plain_kernel(const void* __restrict__ w, uint32_t dtype, const float* __restrict__ x, uint32_t K,
                                                    uint32_t N, uint32_t tokens, float* __restrict__ out, uint32_t float_output) {
    // one 32-lane group per (token, row) pair, eight pairs per workgroup whatever N is (a single row keeps all groups busy)
    const uint32_t lane = threadIdx.x & 31u;
    const uint64_t pair = uint64_t(blockIdx.x) * 8 + (threadIdx.x >> 5);
    if (pair >= uint64_t(N) * tokens) return;
    const uint32_t row = uint32_t(pair % N), t = uint32_t(pair / N);
    const float* xr = x + uint64_t(t) * K;
    float sum = 0;
    uint32_t k = lane;
    // every element's 32-bit word is aligned and inside the array: a four-byte aligned array with an even number of elements
    const bool even_rows = (reinterpret_cast<uintptr_t>(w) & 3u) == 0 && ((uint64_t(N) * K) & 1u) == 0;
    // `count` loads of each operand in flight; the additions stay in k order.  The weight's type is chosen outside the
    // batch: loads on either side of a branch would each be waited for where the sides join.
    auto batch = [&](auto count, auto kind) {
        constexpr int kLoads = decltype(count)::value, kKind = decltype(kind)::value;
        float xv[kLoads], wv[kLoads];
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
            xv[j] = xr[k + 32 * j];
            const uint64_t at = uint64_t(row) * K + k + 32 * j;
            if constexpr (kKind == 0) wv[j] = reinterpret_cast<const float*>(w)[at];
            else if constexpr (kKind == 1) {   // a BF16 weight from the aligned 32-bit word that holds it
                const uint32_t word = reinterpret_cast<const uint32_t*>(w)[at >> 1];
                wv[j] = __uint_as_float((at & 1) ? (word & 0xffff0000u) : (word << 16));
            } else wv[j] = b16(reinterpret_cast<const uint16_t*>(w)[at]);
        }
#pragma unroll
        for (int j = 0; j < kLoads; ++j) sum += xv[j] * wv[j];
        k += kLoads * 32;
    };
    auto batches = [&](auto kind) {   // a row is one memory latency per batch: long rows take sixteen loads at a time
        while (k + 15 * 32 < K) batch(std::integral_constant<int, 16>{}, kind);
        while (k + 7 * 32 < K) batch(std::integral_constant<int, 8>{}, kind);
    };
    if (dtype == 1) batches(std::integral_constant<int, 0>{});
    else if (even_rows) batches(std::integral_constant<int, 1>{});
    else batches(std::integral_constant<int, 2>{});
    for (; k < K; k += 32) {
        const float wv = dtype == 1 ? reinterpret_cast<const float*>(w)[uint64_t(row) * K + k]
                                    : b16(reinterpret_cast<const uint16_t*>(w)[uint64_t(row) * K + k]);
        sum += xr[k] * wv;
    }
    sum = lane_sum32(sum);
    if (lane == 0) out[uint64_t(t) * N + row] = float_output ? sum : bf(sum);
}
void launch_plain(hipStream_t s, const void* w, uint32_t dtype, const float* x, uint32_t K, uint32_t N,
                  uint32_t tokens, float* out, bool float_output) {
    const uint64_t pairs = uint64_t(N) * tokens;
    hipLaunchKernelGGL(plain_kernel, dim3(uint32_t((pairs + 7) / 8)), dim3(256), 0, s, w, dtype, x, K, N, tokens, out,
                       uint32_t(float_output));
}

// ---------------------------------------------------------------------------
// Router logits (reference: qwen.metal:512-534, metal.mm:818-822): sixteen contiguous
// K partitions, a k-ascending multiply-accumulate chain in each, partials added 0..15.
// One lane owns one (expert, partition) chain for TT tokens.
// ---------------------------------------------------------------------------
template <int TT>
__global__ __launch_bounds__(256) void router_kernel(const uint16_t* w, const float* x, uint32_t T, uint32_t K,
                                                     uint32_t E, const float* offsets, float* out) {
    const uint32_t e = blockIdx.x * 16 + threadIdx.x / 16, split = threadIdx.x % 16, t0 = blockIdx.y * TT;
    const uint32_t P = K / 16;
    float c[TT];
#pragma unroll
    for (int t = 0; t < TT; ++t) c[t] = 0;
    if (e < E) {
        const uint16_t* wr = w + uint64_t(e) * K + split * P;
        if (P % 8 == 0) {
            for (uint32_t i = 0; i < P; i += 8) {
                const uint4 wv = *reinterpret_cast<const uint4*>(wr + i);
                const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    const uint32_t tt = t0 + t < T ? t0 + t : T - 1;
                    const float* xr = x + uint64_t(tt) * K + split * P + i;
                    const float4 a = *reinterpret_cast<const float4*>(xr), b = *reinterpret_cast<const float4*>(xr + 4);
                    const float xv[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        c[t] = __builtin_fmaf(xv[k], __uint_as_float((k & 1) ? (ww[k / 2] & 0xffff0000u) : (ww[k / 2] << 16)), c[t]);
                }
            }
        } else {
            for (uint32_t i = 0; i < P; ++i)
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    const uint32_t tt = t0 + t < T ? t0 + t : T - 1;
                    c[t] = __builtin_fmaf(x[uint64_t(tt) * K + split * P + i], b16(wr[i]), c[t]);
                }
        }
    }
    const uint32_t base = (threadIdx.x & 63u) & ~15u;
#pragma unroll
    for (int t = 0; t < TT; ++t) {
        float sum = 0;
        for (uint32_t sidx = 0; sidx < 16; ++sidx) sum += __shfl(c[t], base + sidx);
        if (split == 0 && e < E && t0 + t < T) out[uint64_t(t0 + t) * E + e] = offsets ? sum + offsets[e] : sum;
    }
}
// The same chains for long batches, register-tiled: a lane owns one K partition for 4 tokens x 4 experts, so every
// sixteen-byte weight piece and every eight inputs feed sixteen multiply-accumulate chains.  A workgroup covers
// 16 tokens x 16 experts; lane = (partition, token group, expert group).
__global__ __launch_bounds__(256) void router_tiled_kernel(const uint16_t* w, const float* x, uint32_t T, uint32_t K,
                                                           uint32_t E, const float* offsets, float* out) {
    const uint32_t split = threadIdx.x % 16, pair = threadIdx.x / 16, tg = pair % 4, eg = pair / 4;
    const uint32_t t0 = blockIdx.y * 16 + tg * 4, e0 = blockIdx.x * 16 + eg * 4, P = K / 16;
    float c[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) c[t][e] = 0;
    const float* xr[4]; const uint16_t* wr[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) xr[t] = x + uint64_t(min(t0 + t, T - 1)) * K + split * P;
#pragma unroll
    for (int e = 0; e < 4; ++e) wr[e] = w + uint64_t(min(e0 + e, E - 1)) * K + split * P;
    for (uint32_t i = 0; i < P; i += 8) {
        float xv[4][8], wv[4][8];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float4 a = *reinterpret_cast<const float4*>(xr[t] + i), b = *reinterpret_cast<const float4*>(xr[t] + i + 4);
            xv[t][0] = a.x; xv[t][1] = a.y; xv[t][2] = a.z; xv[t][3] = a.w; xv[t][4] = b.x; xv[t][5] = b.y; xv[t][6] = b.z; xv[t][7] = b.w;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint4 v = *reinterpret_cast<const uint4*>(wr[e] + i);
            const uint32_t ww[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int k = 0; k < 8; ++k) wv[e][k] = __uint_as_float((k & 1) ? (ww[k / 2] & 0xffff0000u) : (ww[k / 2] << 16));
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int k = 0; k < 8; ++k) c[t][e] = __builtin_fmaf(xv[t][k], wv[e][k], c[t][e]);
    }
    const uint32_t base = (threadIdx.x & 63u) & ~15u;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float sum = 0;
            for (uint32_t sidx = 0; sidx < 16; ++sidx) sum += __shfl(c[t][e], base + sidx);
            if (split == 0 && e0 + e < E && t0 + t < T) out[uint64_t(t0 + t) * E + e0 + e] = offsets ? sum + offsets[e0 + e] : sum;
        }
}
// Long batches with K a multiple of 256: a workgroup of 512 threads covers 32 tokens x 16 experts and stages 16 elements
// of every K partition through LDS at a time (whole 64-byte pieces of the inputs, read once per workgroup), so a token
// row is fetched from the L2 by 32 workgroups instead of 128.  Lane = (partition, token group, expert group) with a
// 4 x 4 register tile as above; the chains still run k-ascending inside each partition.  The chunk is small on purpose:
// 52 KB of LDS and few registers let two or three workgroups share a compute unit and hide each other's load latency.
constexpr uint32_t kRouterChunk = 16;
constexpr uint32_t kRouterXPitch = 20, kRouterWPitch = 12;   // words per (row, partition) piece: 16 fp32 + 4, 16 bf16 + 4 (conflict-free 16-/8-byte reads)
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void router_block_kernel(const uint16_t* w, const float* x, uint32_t T, uint32_t K,
                                                              uint32_t E, const float* offsets, float* out) {
    __shared__ __align__(16) uint32_t xs[32 * 16 * kRouterXPitch];   // [token][partition][16 fp32]
    __shared__ __align__(16) uint32_t ws[16 * 16 * kRouterWPitch];   // [expert][partition][16 bf16]
    const uint32_t tid = threadIdx.x, split = tid % 16, pair = tid / 16, tg = pair % 8, eg = pair / 8;
    const uint32_t t0 = blockIdx.y * 32, e0 = blockIdx.x * 16, P = K / 16;
    float c[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) c[t][e] = 0;
    // staging duty per chunk: 32 rows x 16 partitions x 4 sixteen-byte parts of x (4 per thread), 16 x 16 x 2 of w (1 per thread)
    // staging registers as plain 32-bit words (arrays of the vector type end up in scratch memory here)
    uint32_t xr[16], wr[4];
    auto fetch = [&](uint32_t chunk) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t piece = tid + q * 512, part = piece % 4, sp = (piece / 4) % 16, row = piece / 64;
            const uint4 v = *reinterpret_cast<const uint4*>(x + uint64_t(min(t0 + row, T - 1)) * K + sp * P + chunk * kRouterChunk + part * 4);
            xr[4 * q] = v.x; xr[4 * q + 1] = v.y; xr[4 * q + 2] = v.z; xr[4 * q + 3] = v.w;
        }
        {
            const uint32_t part = tid % 2, sp = (tid / 2) % 16, row = tid / 32;
            const uint4 v = ldg_u4(w + uint64_t(min(e0 + row, E - 1)) * K + sp * P + chunk * kRouterChunk + part * 8);
            wr[0] = v.x; wr[1] = v.y; wr[2] = v.z; wr[3] = v.w;
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t piece = tid + q * 512, part = piece % 4, sp = (piece / 4) % 16, row = piece / 64;
            *reinterpret_cast<uint4*>(&xs[(row * 16 + sp) * kRouterXPitch + part * 4]) = make_uint4(xr[4 * q], xr[4 * q + 1], xr[4 * q + 2], xr[4 * q + 3]);
        }
        {
            const uint32_t part = tid % 2, sp = (tid / 2) % 16, row = tid / 32;
            *reinterpret_cast<uint4*>(&ws[(row * 16 + sp) * kRouterWPitch + part * 4]) = make_uint4(wr[0], wr[1], wr[2], wr[3]);
        }
    };
    const uint32_t chunks = P / kRouterChunk;
    fetch(0);
    for (uint32_t chunk = 0; chunk < chunks; ++chunk) {
        __syncthreads();            // the previous chunk has been consumed
        stash();
        __syncthreads();
        if (chunk + 1 < chunks) fetch(chunk + 1);
#pragma unroll
        for (int k = 0; k < int(kRouterChunk); k += 4) {
            float xv[4][4], wv[4][4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint4 v = *reinterpret_cast<const uint4*>(&xs[((tg * 4 + t) * 16 + split) * kRouterXPitch + k]);
                xv[t][0] = __uint_as_float(v.x); xv[t][1] = __uint_as_float(v.y); xv[t][2] = __uint_as_float(v.z); xv[t][3] = __uint_as_float(v.w);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint2 v = *reinterpret_cast<const uint2*>(&ws[((eg * 4 + e) * 16 + split) * kRouterWPitch + k / 2]);
                wv[e][0] = __uint_as_float(v.x << 16); wv[e][1] = __uint_as_float(v.x & 0xffff0000u);
                wv[e][2] = __uint_as_float(v.y << 16); wv[e][3] = __uint_as_float(v.y & 0xffff0000u);
            }
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int i = 0; i < 4; ++i) c[t][e] = __builtin_fmaf(xv[t][i], wv[e][i], c[t][e]);
        }
    }
    const uint32_t base = (tid & 63u) & ~15u;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float sum = 0;
            for (uint32_t sidx = 0; sidx < 16; ++sidx) sum += __shfl(c[t][e], base + sidx);
            const uint32_t tt = t0 + tg * 4 + t, ee = e0 + eg * 4 + e;
            if (split == 0 && ee < E && tt < T) out[uint64_t(tt) * E + ee] = offsets ? sum + offsets[ee] : sum;
        }
}
void launch_router(hipStream_t s, const void* w, const float* x, uint32_t T, uint32_t K, uint32_t E,
                   const float* offsets, float* out) {
    if (T >= 256 && K % 256 == 0) {
        hipLaunchKernelGGL(router_block_kernel, dim3((E + 15) / 16, (T + 31) / 32), dim3(512), 0, s, (const uint16_t*)w, x, T, K, E, offsets, out);
        return;
    }
    if (T >= 64 && K % 128 == 0) {
        hipLaunchKernelGGL(router_tiled_kernel, dim3((E + 15) / 16, (T + 15) / 16), dim3(256), 0, s, (const uint16_t*)w, x, T, K, E, offsets, out);
        return;
    }
    const uint32_t gx = (E + 15) / 16;
    if (T >= 4) hipLaunchKernelGGL(router_kernel<4>, dim3(gx, (T + 3) / 4), dim3(256), 0, s, (const uint16_t*)w, x, T, K, E, offsets, out);
    else hipLaunchKernelGGL(router_kernel<1>, dim3(gx, T), dim3(256), 0, s, (const uint16_t*)w, x, T, K, E, offsets, out);
}

// ---------------------------------------------------------------------------
// Route: top-k by descending value, lowest id on ties, nothing at or below -inf;
// softmax over the selected (reference: qwen.metal:742-795).  One wavefront per token.
// ---------------------------------------------------------------------------
constexpr int kRouteMaxPerLane = 16;   // experts <= 1024
constexpr int kRouteMaxTopK = 128;
__global__ __launch_bounds__(64) void route_kernel(const float* logits, uint32_t T, uint32_t E, uint32_t topk,
                                                   int32_t* ids, float* weights) {
    const uint32_t t = blockIdx.x, lane = threadIdx.x;
    __shared__ float scores[kRouteMaxTopK];
    __shared__ int32_t selected[kRouteMaxTopK];
    const float ninf = __uint_as_float(0xff800000u);
    const float* v = logits + uint64_t(t) * E;
    float cand[kRouteMaxPerLane];
#pragma unroll
    for (int i = 0; i < kRouteMaxPerLane; ++i) {
        const uint32_t e = lane + 64u * i;
        float c = e < E ? v[e] : ninf;
        cand[i] = c > ninf ? c : ninf;   // NaN and -inf never win
    }
    for (uint32_t j = 0; j < topk; ++j) {
        float best = ninf; uint32_t index = 0x7fffffffu;
#pragma unroll
        for (int i = 0; i < kRouteMaxPerLane; ++i) if (cand[i] > best) { best = cand[i]; index = lane + 64u * i; }
        float m = best;
#pragma unroll
        for (int o = 32; o; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
        uint32_t winner = (best == m && best > ninf) ? index : 0x7fffffffu;
#pragma unroll
        for (int o = 32; o; o >>= 1) winner = min(winner, uint32_t(__shfl_xor(int(winner), o)));
        if (lane == 0) {
            selected[j] = winner < E ? int32_t(winner) : -1;
            scores[j] = winner < E ? v[winner] : ninf;   // reload keeps signed zero
        }
#pragma unroll
        for (int i = 0; i < kRouteMaxPerLane; ++i) if (lane + 64u * i == winner) cand[i] = ninf;
    }
    __syncthreads();
    // Four values per reference lane, lane sum, one reciprocal.
    float values[4], sum = 0;
    const float top = scores[0];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t j = lane * 4 + i;
        values[i] = (lane < 32 && j < topk) ? exp32(scores[j] - top) : 0.0f;
        sum += values[i];
    }
    const float inverse = 1.0f / lane_sum32(sum);
    if (lane < 32)
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t j = lane * 4 + i;
            if (j < topk) { ids[uint64_t(t) * topk + j] = selected[j]; weights[uint64_t(t) * topk + j] = values[i] * inverse; }
        }
}
void launch_route(hipStream_t s, const float* logits, uint32_t T, uint32_t E, uint32_t topk, int32_t* ids, float* weights) {
    hipLaunchKernelGGL(route_kernel, dim3(T), dim3(64), 0, s, logits, T, E, topk, ids, weights);
}

// ---------------------------------------------------------------------------
// Dispatch: stable counting sort of the flat slots p = t*topk + k by expert id
// (reference: model.cpp:449-479).  One workgroup; each wavefront owns experts
// e = wave, wave+16, ... and scans the id array in order, so slots of an expert
// come out in ascending p without any atomics.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void dispatch_kernel(const int32_t* ids, uint32_t n, uint32_t topk, uint32_t E,
                                                        int32_t* offsets, int32_t* slots, int32_t* rows,
                                                        int32_t* selected, int32_t* count, int32_t* status) {
    extern __shared__ int32_t cnt[];   // E + 1
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, waves = blockDim.x >> 6;
    int bad = 0;
    for (uint32_t p = tid; p < n; p += blockDim.x) bad |= (ids[p] < 0 || ids[p] >= int32_t(E));
    bad = __syncthreads_or(bad);
    if (tid == 0 && bad) atomicOr(status, 1);
    for (uint32_t e = wave; e < E; e += waves) {
        int32_t c = 0;
        for (uint32_t p0 = 0; p0 < n; p0 += 64) {
            const uint32_t p = p0 + lane;
            c += __popcll(__ballot(p < n && ids[p] == int32_t(e)));
        }
        if (lane == 0) cnt[e] = c;
    }
    __syncthreads();
    if (wave == 0) {
        int32_t running = 0, picked = 0;
        if (lane == 0) offsets[0] = 0;
        for (uint32_t base = 0; base < E; base += 64) {
            const uint32_t e = base + lane;
            const int32_t c = e < E ? cnt[e] : 0;
            int32_t incl = c;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) { const int32_t up = __shfl_up(incl, o); if (int(lane) >= o) incl += up; }
            if (e < E) offsets[e + 1] = running + incl;
            const uint64_t mask = __ballot(c > 0);
            if (c > 0) selected[picked + __popcll(mask & ((1ull << lane) - 1))] = int32_t(e);
            picked += __popcll(mask);
            running += __shfl(incl, 63);
        }
        if (lane == 0) *count = picked;
    }
    __syncthreads();
    __threadfence_block();
    for (uint32_t e = wave; e < E; e += waves) {
        int32_t pos = offsets[e];
        if (cnt[e] == 0) continue;
        for (uint32_t p0 = 0; p0 < n; p0 += 64) {
            const uint32_t p = p0 + lane;
            const bool m = p < n && ids[p] == int32_t(e);
            const uint64_t mask = __ballot(m);
            if (m) { const int32_t at = pos + __popcll(mask & ((1ull << lane) - 1)); slots[at] = int32_t(p); if (rows) rows[at] = int32_t(p / topk); }
            pos += __popcll(mask);
        }
    }
}
// The same sort for many slots (prefill), spread over the device: one wavefront per expert counts, one workgroup
// scans, one wavefront per expert places.  offsets[1 + e] doubles as the count array between the first two steps.
__global__ __launch_bounds__(256) void dispatch_count_kernel(const int32_t* __restrict__ ids, uint32_t n, uint32_t E, int32_t* __restrict__ offsets, int32_t* status, bool aligned) {
    const uint32_t lane = threadIdx.x & 63u, e = blockIdx.x * 4 + (threadIdx.x >> 6);
    {   // every workgroup checks its share of the ids (one workgroup doing all of them was the longest-running one)
        int bad = 0;
        for (uint32_t p = blockIdx.x * blockDim.x + threadIdx.x; p < n; p += gridDim.x * blockDim.x) { const int32_t id = ids[p]; bad |= (id < 0 || id >= int32_t(E)); }
        if (bad) atomicOr(status, 1);
    }
    if (e >= E) return;
    int32_t c = 0;
    uint32_t p0 = 0;
    if (aligned && n >= 8 * 256) {   // eight steps' loads in flight, the next eight requested before these are counted
        int4 v[8], w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = *reinterpret_cast<const int4*>(ids + j * 256 + 4 * lane);
        for (; p0 + 8 * 256 <= n; p0 += 8 * 256) {
            const uint32_t following = p0 + 16 * 256 <= n ? p0 + 8 * 256 : p0;   // none left: the same batch again, not counted
#pragma unroll
            for (int j = 0; j < 8; ++j) w[j] = *reinterpret_cast<const int4*>(ids + following + j * 256 + 4 * lane);
#pragma unroll
            for (int j = 0; j < 8; ++j) c += (v[j].x == int32_t(e)) + (v[j].y == int32_t(e)) + (v[j].z == int32_t(e)) + (v[j].w == int32_t(e));
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = w[j];
        }
    }
    for (; p0 < n; p0 += 256) {   // a lane looks at four neighbouring slots per step
        const uint32_t p = p0 + 4 * lane;
        int4 v = make_int4(-1, -1, -1, -1);
        if (aligned && p + 3 < n) v = *reinterpret_cast<const int4*>(ids + p);   // sixteen-byte loads only from a sixteen-byte aligned array
        else { if (p < n) v.x = ids[p]; if (p + 1 < n) v.y = ids[p + 1]; if (p + 2 < n) v.z = ids[p + 2]; if (p + 3 < n) v.w = ids[p + 3]; }
        c += (v.x == int32_t(e)) + (v.y == int32_t(e)) + (v.z == int32_t(e)) + (v.w == int32_t(e));
    }
#pragma unroll
    for (int o = 32; o; o >>= 1) c += __shfl_xor(c, o);
    if (lane == 0) offsets[1 + e] = c;
}
__global__ __launch_bounds__(64) void dispatch_scan_kernel(uint32_t E, int32_t* offsets, int32_t* selected, int32_t* count) {
    const uint32_t lane = threadIdx.x;
    int32_t running = 0, picked = 0;
    if (lane == 0) offsets[0] = 0;
    for (uint32_t base = 0; base < E; base += 64) {
        const uint32_t e = base + lane;
        const int32_t c = e < E ? offsets[1 + e] : 0;
        int32_t incl = c;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { const int32_t up = __shfl_up(incl, o); if (int(lane) >= o) incl += up; }
        if (e < E) offsets[e + 1] = running + incl;
        const uint64_t mask = __ballot(c > 0);
        if (c > 0) selected[picked + __popcll(mask & ((1ull << lane) - 1))] = int32_t(e);
        picked += __popcll(mask);
        running += __shfl(incl, 63);
    }
    if (lane == 0) *count = picked;
}
__global__ __launch_bounds__(256) void dispatch_place_kernel(const int32_t* __restrict__ ids, uint32_t n, uint32_t topk, uint32_t E, const int32_t* __restrict__ offsets,
                                                             int32_t* __restrict__ slots, int32_t* __restrict__ rows, bool aligned) {
    const uint32_t lane = threadIdx.x & 63u, e = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (e >= E) return;
    int32_t pos = offsets[e];
    if (offsets[e + 1] == pos) return;
    const uint64_t below = (1ull << lane) - 1;
    // eight steps of 256 slots, in order: four neighbouring slots per lane, slots of lower lanes first, then the lane's own
    auto place = [&](const int4 (&batch)[8], uint32_t q0) {
#pragma unroll
        for (int step = 0; step < 8; ++step) {
            if (q0 + step * 256 >= n) break;
            const uint32_t p = q0 + step * 256 + 4 * lane;
            const int4 v = batch[step];
            const bool m[4] = {v.x == int32_t(e), v.y == int32_t(e), v.z == int32_t(e), v.w == int32_t(e)};
            const uint64_t mask[4] = {__ballot(m[0]), __ballot(m[1]), __ballot(m[2]), __ballot(m[3])};
            if ((mask[0] | mask[1] | mask[2] | mask[3]) == 0) continue;   // uniform: none of these 256 slots is the expert's
            int32_t at = pos + __popcll(mask[0] & below) + __popcll(mask[1] & below) + __popcll(mask[2] & below) + __popcll(mask[3] & below);
            uint32_t token = p / topk, rest = p % topk;   // one division per step, not one per slot
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (m[j]) { slots[at] = int32_t(p + j); if (rows) rows[at] = int32_t(token); ++at; }
                if (++rest == topk) { rest = 0; ++token; }
            }
            pos += __popcll(mask[0]) + __popcll(mask[1]) + __popcll(mask[2]) + __popcll(mask[3]);
        }
    };
    uint32_t q0 = 0;
    if (aligned && n >= 8 * 256) {   // whole batches: the next batch is requested before this one is placed
        int4 ahead[8], next[8];
#pragma unroll
        for (int step = 0; step < 8; ++step) ahead[step] = *reinterpret_cast<const int4*>(ids + step * 256 + 4 * lane);
        for (; q0 + 8 * 256 <= n; q0 += 8 * 256) {
            const uint32_t following = q0 + 16 * 256 <= n ? q0 + 8 * 256 : q0;   // none left: the same batch again, not placed
#pragma unroll
            for (int step = 0; step < 8; ++step) next[step] = *reinterpret_cast<const int4*>(ids + following + step * 256 + 4 * lane);
            place(ahead, q0);
#pragma unroll
            for (int step = 0; step < 8; ++step) ahead[step] = next[step];
        }
    }
    for (; q0 < n; q0 += 8 * 256) {   // the ragged end, or an array that is not sixteen-byte aligned
        int4 ahead[8];
#pragma unroll
        for (int step = 0; step < 8; ++step) {
            const uint32_t p = q0 + step * 256 + 4 * lane;
            int4 v = make_int4(-1, -1, -1, -1);
            if (aligned && p + 3 < n) v = *reinterpret_cast<const int4*>(ids + p);   // sixteen-byte loads only from a sixteen-byte aligned array
            else { if (p < n) v.x = ids[p]; if (p + 1 < n) v.y = ids[p + 1]; if (p + 2 < n) v.z = ids[p + 2]; if (p + 3 < n) v.w = ids[p + 3]; }
            ahead[step] = v;
        }
        place(ahead, q0);
    }
}
void launch_dispatch(hipStream_t s, const int32_t* ids, uint32_t tokens, uint32_t topk, uint32_t E, int32_t* offsets,
                     int32_t* slots, int32_t* rows, int32_t* selected, int32_t* count, int32_t* status) {
    const uint32_t n = tokens * topk;
    if (n <= 1024) {   // decode: one launch
        hipLaunchKernelGGL(dispatch_kernel, dim3(1), dim3(1024), size_t(E + 1) * 4, s, ids, n, topk, E, offsets, slots, rows, selected, count, status);
        return;
    }
    const bool aligned = reinterpret_cast<uintptr_t>(ids) % 16 == 0;
    hipLaunchKernelGGL(dispatch_count_kernel, dim3((E + 3) / 4), dim3(256), 0, s, ids, n, E, offsets, status, aligned);
    hipLaunchKernelGGL(dispatch_scan_kernel, dim3(1), dim3(64), 0, s, E, offsets, selected, count);
    hipLaunchKernelGGL(dispatch_place_kernel, dim3((E + 3) / 4), dim3(256), 0, s, ids, n, topk, E, offsets, slots, rows, aligned);
}

// ---------------------------------------------------------------------------
// scatter_experts, moe_sum (reference: qwen.metal:800-816), inter-layer RMS glue
// ---------------------------------------------------------------------------
__global__ void scatter_kernel(const float* x, const int32_t* positions, uint32_t n, uint32_t H, float* out) {
    const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x, r = blockIdx.y;
    if (c < H && r < n) out[uint64_t(uint32_t(positions[r])) * H + c] = x[uint64_t(r) * H + c];
}
void launch_scatter(hipStream_t s, const float* x, const int32_t* positions, uint32_t n, uint32_t H, float* out) {
    hipLaunchKernelGGL(scatter_kernel, dim3((H + 255) / 256, n), dim3(256), 0, s, x, positions, n, H, out);
}
// General top-k keeps the reference's eight strided partials: partial j takes
// k = j, j+8, ...; partials are then added 0..7.  top-k 10 is the reference expression.
template <int V, bool HALF = false>
__global__ __launch_bounds__(256) void moe_sum_kernel(const void* __restrict__ experts_in, const float* __restrict__ weights, const float* __restrict__ shared,
                                                      const float* __restrict__ gate, uint32_t T, uint32_t H, uint32_t topk, float* __restrict__ out) {
    // V neighbouring columns per thread (one 16-byte load per slot when V is 4); every column keeps the scalar arithmetic.
    // HALF: the expert outputs are stored as bf16 (they are BF16 values: the same numbers, half the bytes; V is 4 then).
    typedef float row_t __attribute__((ext_vector_type(V)));
    const uint32_t c = (blockIdx.x * blockDim.x + threadIdx.x) * V, t = blockIdx.y;
    if (c >= H || t >= T) return;
    auto row_of = [&](uint64_t slot) {
        if constexpr (HALF) {
            const uint2 w = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(experts_in) + slot * H + c);
            return row_t{__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xffff0000u)};
        } else return *reinterpret_cast<const row_t*>(static_cast<const float*>(experts_in) + slot * H + c);
    };
    row_t partial[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) partial[k] = row_t(0);
    if (topk == 10) {   // the reference's shape: all ten rows requested before the first is used
        row_t value[10]; float weight[10];
#pragma unroll
        for (int k = 0; k < 10; ++k) { value[k] = row_of(uint64_t(t) * 10 + k); weight[k] = weights[uint64_t(t) * 10 + k]; }
#pragma unroll
        for (int k = 0; k < 10; ++k) {
            const row_t product = value[k] * weight[k];
            if (k < 8) partial[k] = product; else partial[k % 8] = partial[k % 8] + product;
        }
    } else
    for (uint32_t k = 0; k < topk; ++k) {
        const row_t product = row_of(uint64_t(t) * topk + k) * weights[uint64_t(t) * topk + k];
        if (k < 8) partial[k] = product; else partial[k % 8] = partial[k % 8] + product;
    }
    row_t sum = partial[0];
    for (uint32_t k = 1; k < 8 && k < topk; ++k) sum += partial[k];
    const float g = bf(sigmoid_bf(gate[t]));
    const row_t sh = *reinterpret_cast<const row_t*>(shared + uint64_t(t) * H + c);
    row_t y;
    if constexpr (V == 1) y = row_t(bf(bf(sum[0]) + bf(g * sh[0])));
    else {
#pragma unroll
        for (int i = 0; i < V; ++i) y[i] = bf(bf(sum[i]) + bf(g * sh[i]));
    }
    *reinterpret_cast<row_t*>(out + uint64_t(t) * H + c) = y;
}
void launch_moe_sum(hipStream_t s, const float* experts, const float* weights, const float* shared, const float* gate,
                    uint32_t T, uint32_t H, uint32_t topk, float* out) {
    const bool wide = H % 4 == 0 && ((reinterpret_cast<uintptr_t>(experts) | reinterpret_cast<uintptr_t>(shared) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    if (wide) hipLaunchKernelGGL((moe_sum_kernel<4>), dim3((H / 4 + 255) / 256, T), dim3(256), 0, s, experts, weights, shared, gate, T, H, topk, out);
    else hipLaunchKernelGGL((moe_sum_kernel<1>), dim3((H + 255) / 256, T), dim3(256), 0, s, experts, weights, shared, gate, T, H, topk, out);
}
// The same with the expert outputs as bf16 rows (H a multiple of four, every array sixteen-byte aligned).
void launch_moe_sum_half(hipStream_t s, const uint16_t* experts, const float* weights, const float* shared, const float* gate,
                         uint32_t T, uint32_t H, uint32_t topk, float* out) {
    hipLaunchKernelGGL((moe_sum_kernel<4, true>), dim3((H / 4 + 255) / 256, T), dim3(256), 0, s, experts, weights, shared, gate, T, H, topk, out);
}
// Stand-in glue between stacked layers: x_next = bf(y * (1 / max|y|)) per token.
__global__ __launch_bounds__(256) void stack_glue_kernel(const float* y, uint32_t H, float* out) {
    __shared__ uint32_t wave_max[4];
    const float* row = y + uint64_t(blockIdx.x) * H;
    uint32_t m = 0;
    for (uint32_t k = threadIdx.x; k < H; k += blockDim.x) {
        const uint32_t a = __float_as_uint(row[k]) & 0x7fffffffu;
        if (a <= 0x7f800000u) m = max(m, a);   // NaN does not take part
    }
#pragma unroll
    for (int o = 32; o; o >>= 1) m = max(m, uint32_t(__shfl_xor(int(m), o)));
    if ((threadIdx.x & 63u) == 0) wave_max[threadIdx.x >> 6] = m;
    __syncthreads();
    m = max(max(wave_max[0], wave_max[1]), max(wave_max[2], wave_max[3]));
    const float top = __uint_as_float(m);
    const float inv = (top > 0.0f && top < __uint_as_float(0x7f800000u)) ? 1.0f / top : 1.0f;
    for (uint32_t k = threadIdx.x; k < H; k += blockDim.x) out[uint64_t(blockIdx.x) * H + k] = bf(row[k] * inv);
}
void launch_stack_glue(hipStream_t s, const float* y, uint32_t T, uint32_t H, float* out) {
    hipLaunchKernelGGL(stack_glue_kernel, dim3(T), dim3(256), 0, s, y, H, out);
}

// ---------------------------------------------------------------------------
// Counter-based synthetic tensors
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t synth_word(uint64_t seed, uint64_t i) {
    const uint64_t h = hash64(seed, i >> 1);
    return (i & 1) ? uint32_t(h >> 32) : uint32_t(h);
}
__device__ __forceinline__ float synth_scale(uint64_t seed, uint64_t i, float lo, float span) {
    const float u = float(uint32_t(hash64(seed, i) >> 40)) * 5.9604644775390625e-08f;   // 24 bits * 2^-24
    return bf(lo + span * u);
}
// Irwin-Hall(12) on 16-bit fields of three hashes: integer arithmetic, so host and
// device agree exactly; variance (2^32-1)/2^32 of a unit normal, tails cut at 6.
__device__ __forceinline__ float synth_normal(uint64_t seed, uint64_t i, float sigma) {
    int32_t sum = 0;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        const uint64_t h = hash64(seed, 3 * i + j);
        sum += int32_t(h & 0xffff) + int32_t((h >> 16) & 0xffff) + int32_t((h >> 32) & 0xffff) + int32_t(h >> 48);
    }
    return bf(float(2 * sum - 12 * 65535) * 7.62939453125e-06f * sigma);   // * 2^-17
}
__global__ void synth_words_kernel(uint32_t* dst, uint64_t count, uint64_t seed) {
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < count; i += uint64_t(gridDim.x) * blockDim.x)
        dst[i] = synth_word(seed, i);
}
__global__ void synth_scales_kernel(uint16_t* scales, uint16_t* biases, uint64_t count, uint64_t seed, float lo, float span, float factor) {
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < count; i += uint64_t(gridDim.x) * blockDim.x) {
        const float sc = synth_scale(seed, i, lo, span);
        scales[i] = uint16_t(__float_as_uint(sc) >> 16);
        biases[i] = uint16_t(__float_as_uint(bf(sc * factor)) >> 16);
    }
}
template <bool HALF>
__global__ void synth_normal_kernel(void* dst, uint64_t count, uint64_t seed, float sigma) {
    for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < count; i += uint64_t(gridDim.x) * blockDim.x) {
        const float v = synth_normal(seed, i, sigma);
        if constexpr (HALF) reinterpret_cast<uint16_t*>(dst)[i] = uint16_t(__float_as_uint(v) >> 16);
        else reinterpret_cast<float*>(dst)[i] = v;
    }
}
static dim3 flat_grid(uint64_t count) { return dim3(uint32_t(count / 256 + 1 < 65536 ? count / 256 + 1 : 65536)); }
void launch_synth_words(hipStream_t s, uint32_t* dst, uint64_t count, uint64_t seed) {
    hipLaunchKernelGGL(synth_words_kernel, flat_grid(count), dim3(256), 0, s, dst, count, seed);
}
void launch_synth_scales(hipStream_t s, uint16_t* sc, uint16_t* bi, uint64_t count, uint64_t seed, float lo, float span, float factor) {
    hipLaunchKernelGGL(synth_scales_kernel, flat_grid(count), dim3(256), 0, s, sc, bi, count, seed, lo, span, factor);
}
void launch_synth_normal(hipStream_t s, void* dst, uint64_t count, uint64_t seed, float sigma, bool half) {
    if (half) hipLaunchKernelGGL(synth_normal_kernel<true>, flat_grid(count), dim3(256), 0, s, dst, count, seed, sigma);
    else hipLaunchKernelGGL(synth_normal_kernel<false>, flat_grid(count), dim3(256), 0, s, dst, count, seed, sigma);
}
// Whole records: blockIdx.y = record, grid-stride over the record's dwords.
struct RecordLayout { uint64_t w[3], s[3], words[3], meta[3]; float lo[3], span[3], factor[3]; uint64_t bytes; };
__global__ void synth_records_kernel(uint8_t* records, uint64_t stride, RecordLayout l, uint64_t seed) {
    uint8_t* r = records + uint64_t(blockIdx.y) * stride;
    for (int p = 0; p < 3; ++p) {
        const uint64_t ps = seed + uint64_t(blockIdx.y) * 3 + p;
        uint32_t* w = reinterpret_cast<uint32_t*>(r + l.w[p]);
        for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < l.words[p]; i += uint64_t(gridDim.x) * blockDim.x)
            w[i] = synth_word(ps, i);
        uint16_t* sc = reinterpret_cast<uint16_t*>(r + l.s[p]);
        uint16_t* bi = sc + l.meta[p];
        for (uint64_t i = blockIdx.x * uint64_t(blockDim.x) + threadIdx.x; i < l.meta[p]; i += uint64_t(gridDim.x) * blockDim.x) {
            const float v = synth_scale(ps ^ 0x5CA1E5CA1Eull, i, l.lo[p], l.span[p]);
            sc[i] = uint16_t(__float_as_uint(v) >> 16);
            bi[i] = uint16_t(__float_as_uint(bf(v * l.factor[p])) >> 16);
        }
    }
}
void launch_synth_records(hipStream_t s, void* records, uint64_t stride, uint32_t count, const uint64_t* w_off,
                          const uint64_t* s_off, const uint64_t* words, const uint64_t* meta, const uint32_t* bits, uint64_t seed) {
    RecordLayout l{};
    for (int p = 0; p < 3; ++p) {
        l.w[p] = w_off[p]; l.s[p] = s_off[p]; l.words[p] = words[p]; l.meta[p] = meta[p];
        l.lo[p] = bits[p] == 8 ? 0.0002f : 0.002f; l.span[p] = bits[p] == 8 ? 0.0018f : 0.018f;
        l.factor[p] = bits[p] == 8 ? -128.0f : -8.0f;
    }
    hipLaunchKernelGGL(synth_records_kernel, dim3(64, count), dim3(256), 0, s, (uint8_t*)records, stride, l, seed);
}

}  // namespace zc
