// Operator-level kernels on the exact-integer matrix-core path (see zc_xint.hpp):
// the fast form of linear_into / gated_linear for wide affine-Q4 matrices
// (K % 512 == 0, N % 8 == 0, group 64).  Bit-identical to the literal kernels.
#include "zc_kernels.hpp"
#include "zc_xint.hpp"

namespace zc {

struct XintJob {
    const uint8_t *w0, *w1;
    const uint16_t *s0, *b0, *s1, *b1;
    const float* x; const int32_t *in_rows, *out_rows; float* out;
    uint32_t K, N, tokens, float_output;
};

constexpr int kXintWaves = 4;

// One wavefront per 16-column tile; the workgroup shares the tokens' LDS images.
template <int NT, bool GATED>
__device__ __forceinline__ void xint_rows(const XintJob& j, uint32_t tile, uint32_t t0, uint8_t* lds_base) {
    const XintLayout L{j.K};
    const uint32_t lane = threadIdx.x & 63u, col = lane & 15u, G = lane >> 4;
    const uint8_t* lds[NT]; LdsF32 xr[NT];
    float* xf = reinterpret_cast<float*>(lds_base + NT * L.bytes());   // fp32 copies of the rows
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const uint32_t tt = min(t0 + t, j.tokens - 1);
        const float* row = j.x + uint64_t(j.in_rows ? uint32_t(j.in_rows[tt]) : tt) * j.K;
        for (uint32_t i = threadIdx.x; i < j.K / 4; i += blockDim.x)
            reinterpret_cast<float4*>(xf + t * j.K)[i] = reinterpret_cast<const float4*>(row)[i];
        xr[t] = LdsF32{xf + t * j.K};
        lds[t] = lds_base + t * L.bytes();
    }
    __syncthreads();
    xint_prepare_batch([&](uint32_t q) { return LdsF32{xf + q * j.K}; }, NT, L, lds_base);
    uint32_t row; const uint8_t* w; const uint16_t *s, *b;
    if (GATED) {
        row = tile * 8 + (col & 7u);
        w = col < 8 ? j.w0 : j.w1; s = col < 8 ? j.s0 : j.s1; b = col < 8 ? j.b0 : j.b1;
    } else {
        row = tile * 16 + col; w = j.w0; s = j.s0; b = j.b0;
    }
    const bool valid = row < j.N;
    const uint32_t r = valid ? row : j.N - 1;
    auto emit = [&](int t, float v) {
        if (GATED) {
            const float up = __shfl(v, (lane & ~15u) | ((col & 7u) + 8u));
            v = swiglu_bf(v, up);
        } else if (!j.float_output) v = bf(v);
        const bool writer = G == 0 && valid && (!GATED || col < 8) && t0 + t < j.tokens;
        if (writer) j.out[uint64_t(j.out_rows ? uint32_t(j.out_rows[t0 + t]) : t0 + t) * j.N + row] = v;
    };
    const uint8_t* w_row = w + uint64_t(r) * (j.K / 2);
    if ((j.K / 128) % 8 == 0) xint_run_tile<NT, 8>(w_row, s + uint64_t(r) * (j.K / 64), b + uint64_t(r) * (j.K / 64), j.K / 128, lds, xr, L, lane, NT, emit);
    else xint_run_tile<NT, 4>(w_row, s + uint64_t(r) * (j.K / 64), b + uint64_t(r) * (j.K / 64), j.K / 128, lds, xr, L, lane, NT, emit);
}

// One wavefront per tile of 32 columns (gate/up: sixteen gate rows and the up rows of the same indices), two to four
// tokens per workgroup: the form of the tile engine that fills the larger matrix-core instruction.
template <int NT, bool GATED>
__global__ __launch_bounds__(64 * kXintWaves) void xint_op32_kernel(XintJob j) {
    extern __shared__ __align__(16) uint8_t xint_lds[];
    const XintLayout L{j.K};
    const uint32_t tiles = GATED ? (j.N + 15) / 16 : (j.N + 31) / 32;
    const uint32_t tile = min(blockIdx.x * kXintWaves + (threadIdx.x >> 6), tiles - 1);   // tail waves repeat the last tile
    const uint32_t t0 = blockIdx.y * NT, lane = threadIdx.x & 63u, n = lane & 31u, h = lane >> 5;
    const uint8_t* lds[NT]; LdsF32 xr[NT];
    float* xf = reinterpret_cast<float*>(xint_lds + NT * L.bytes());   // fp32 copies of the rows
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const uint32_t tt = min(t0 + t, j.tokens - 1);
        const float* row = j.x + uint64_t(j.in_rows ? uint32_t(j.in_rows[tt]) : tt) * j.K;
        for (uint32_t i = threadIdx.x; i < j.K / 4; i += blockDim.x)
            reinterpret_cast<float4*>(xf + t * j.K)[i] = reinterpret_cast<const float4*>(row)[i];
        xr[t] = LdsF32{xf + t * j.K};
        lds[t] = xint_lds + t * L.bytes();
    }
    __syncthreads();
    xint_prepare_batch([&](uint32_t q) { return LdsF32{xf + q * j.K}; }, NT, L, xint_lds);
    uint32_t row; const uint8_t* w; const uint16_t *s, *b;
    if (GATED) {
        row = tile * 16 + (n & 15u);
        w = n < 16 ? j.w0 : j.w1; s = n < 16 ? j.s0 : j.s1; b = n < 16 ? j.b0 : j.b1;
    } else {
        row = tile * 32 + n; w = j.w0; s = j.s0; b = j.b0;
    }
    const bool valid = row < j.N;
    const uint32_t r = valid ? row : j.N - 1;
    auto emit = [&](int t, float v) {
        if (GATED) {
            const float up = __shfl(v, (lane & ~31u) | ((n & 15u) + 16u));
            v = swiglu_bf(v, up);
        } else if (!j.float_output) v = bf(v);
        const bool writer = h == 0 && valid && (!GATED || n < 16) && t0 + t < j.tokens;
        if (writer) j.out[uint64_t(j.out_rows ? uint32_t(j.out_rows[t0 + t]) : t0 + t) * j.N + row] = v;
    };
    xint_run_tile32<NT>(w + uint64_t(r) * (j.K / 2), s + uint64_t(r) * (j.K / 64), b + uint64_t(r) * (j.K / 64), j.K / 128, lds, xr, L, lane, NT, emit);
}

template <int NT, bool GATED>
__global__ __launch_bounds__(64 * kXintWaves) void xint_op_kernel(XintJob j) {
    extern __shared__ __align__(16) uint8_t xint_lds[];
    const uint32_t tiles = GATED ? j.N / 8 : (j.N + 15) / 16;
    const uint32_t tile = min(blockIdx.x * kXintWaves + (threadIdx.x >> 6), tiles - 1);   // tail waves repeat the last tile
    xint_rows<NT, GATED>(j, tile, blockIdx.y * NT, xint_lds);
}

bool xint_supported(const zc_linear& l) {
    return l.quantized && l.bits == 4 && l.group == 64 && l.input % 512 == 0 && l.output % 8 == 0 &&
           reinterpret_cast<uintptr_t>(l.weight) % 16 == 0;
}

void launch_affine_xint(hipStream_t s, const AffineDesc& a) {
    XintJob j{};
    j.w0 = (const uint8_t*)a.gate.weight; j.s0 = (const uint16_t*)a.gate.scales; j.b0 = (const uint16_t*)a.gate.biases;
    if (a.gated) { j.w1 = (const uint8_t*)a.up.weight; j.s1 = (const uint16_t*)a.up.scales; j.b1 = (const uint16_t*)a.up.biases; }
    j.x = a.x; j.in_rows = a.in_rows; j.out_rows = a.out_rows; j.out = a.out;
    j.K = a.gate.input; j.N = a.gate.output; j.tokens = a.tokens; j.float_output = a.float_output;
    const XintLayout L{j.K};
    const uint32_t tiles = a.gated ? j.N / 8 : (j.N + 15) / 16;
    const uint32_t nt = a.tokens >= 4 ? 4 : a.tokens >= 2 ? 2 : 1;
    const size_t lds = (size_t(L.bytes()) + size_t(j.K) * 4) * nt;
    // Several tokens share a tile: the 32-column form, when its workgroups (half as many) still fill the chip.  (Measured at
    // K = 3072, N = 4096: 256 tokens 460 -> 388 us plain, 897 -> 726 us gate/up; 16 tokens 40 -> 55 us plain.)
    const uint32_t tiles32 = a.gated ? (j.N + 15) / 16 : (j.N + 31) / 32;
    const dim3 grid32((tiles32 + kXintWaves - 1) / kXintWaves, (a.tokens + nt - 1) / nt);
    if (nt >= 2 && grid32.x * grid32.y >= 512) {
#define ZC_GO32(NT, GATED) hipLaunchKernelGGL((xint_op32_kernel<NT, GATED>), grid32, dim3(64 * kXintWaves), lds, s, j)
        if (a.gated) { if (nt == 4) ZC_GO32(4, true); else ZC_GO32(2, true); }
        else { if (nt == 4) ZC_GO32(4, false); else ZC_GO32(2, false); }
#undef ZC_GO32
        return;
    }
    const dim3 grid((tiles + kXintWaves - 1) / kXintWaves, (a.tokens + nt - 1) / nt), block(64 * kXintWaves);
#define ZC_GO(NT, GATED) hipLaunchKernelGGL((xint_op_kernel<NT, GATED>), grid, block, lds, s, j)
    if (a.gated) { if (nt == 4) ZC_GO(4, true); else if (nt == 2) ZC_GO(2, true); else ZC_GO(1, true); }
    else { if (nt == 4) ZC_GO(4, false); else if (nt == 2) ZC_GO(2, false); else ZC_GO(1, false); }
#undef ZC_GO
}

}  // namespace zc
