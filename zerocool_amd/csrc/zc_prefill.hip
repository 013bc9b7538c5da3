// Prefill path of the MoE layer: tokens sorted by expert, then a grouped GEMM on the bf16 matrix cores with
// fp32 accumulation (the reference batches the same work per expert in encode_expert_rows, src/engine/pipeline.cpp:7-31,
// over q4_mm / q4_gate_up, kernels/metal/qwen.metal:289-376).
//
// Arithmetic.  The reference evaluates, per 16-element block, scale * sum(x q) + bias * sum'(x) with sum' the
// BF16-rounded sum-of-four chain (qwen.metal:46-62).  Here the products x * q run on v_mfma_f32_16x16x32_bf16: x is
// BF16-valued (exact as a bf16 operand), q in 0..15 is exact in bf16, products are exact and accumulate in fp32 over one
// scale group of 64; per group the accumulator is folded as  total += scale * dot + bias * chain_sum  with the chain
// sums precomputed per (row, group) exactly as the reference rounds them.  Only the order of the fp32 additions
// differs from the reference, so results agree to a few fp32 steps before the BF16 rounding of the outputs.  Every sum
// that lands within prefill_margin(K) of its term magnitudes of a BF16 rounding boundary is then recomputed with the reference's exact
// lane arithmetic (about 2-3 % of the elements), which removes the rounding flips in practice; the path is still
// specified by a tolerance (max relative error 2e-3 of the layer output), not as bit-exact.  Routing, dispatch and the
// combine use the exact kernels.
//
// Tiling.  One workgroup (4 waves) owns up to 48 sorted token rows of ONE expert and 128 weight rows (gate/up: 64 gate rows
// and the 64 up rows of the same indices, so SwiGLU is fused in registers), and walks K in steps of 64 = one scale
// group.  Each wave multiplies all (two or three) 16-row blocks of the tokens by 2 of the 8 column tiles: the 4-bit codes
// of its 32 weight rows go from memory straight into the lanes that feed them to the matrix cores and are expanded to
// bf16 there (once per workgroup and step), the token rows are gathered into LDS as bf16, double-buffered, and the
// scales, biases and chain sums of all steps are brought into LDS once.  An expert's rows are cut into tiles of 32, except
// that a run of up to 48 rows (a whole expert with few rows, or the last rows of a longer run) is ONE tile: with about
// forty rows per expert -- an unskewed router at 2048 tokens -- every expert's codes are then expanded once, not twice.
#include "zc_kernels.hpp"
#include "zc_device.hpp"
#include "zc_decode_common.hpp"   // route_token: top-k + softmax of one token by one wavefront

namespace zc {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr uint32_t kTileRows = 32, kTileRowsMax = 48, kTileCols = 128, kPitch = 72;   // LDS row pitch in bf16 elements (144 bytes)

// fp32 rows holding BF16 values -> bf16 rows, plus per (row, group of 64) the sum of the four blocks' BF16-rounded
// sum-of-four chains.  One thread per (row, group).  status bit 4: a value was not BF16-valued.
// plain (optional): per (row, group) the sum of the plain fp32 sums of the group's eight 8-element blocks, the affine Q8
// lanes' input sum (qwen.metal:112-125: sum += v, element by element).
__global__ __launch_bounds__(256) void prefill_rows_kernel(const float* x, uint32_t rows, uint32_t K, uint16_t* xb, float* sums, float* sums16, float* plain,
                                                           int32_t* status) {
    const uint32_t groups = K / 64, i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * groups) return;
    const uint32_t r = i / groups, g = i % groups;
    const float4* src = reinterpret_cast<const float4*>(x + uint64_t(r) * K + g * 64);
    uint32_t low = 0;
    float total = 0, total_plain = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        float sum = 0, eight[2] = {0, 0};
        uint32_t packed[8];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 v = src[b * 4 + q];
            sum += bf(bf(bf(v.x + v.y) + v.z) + v.w);
            eight[q / 2] = (((eight[q / 2] + v.x) + v.y) + v.z) + v.w;
            const uint32_t u0 = __float_as_uint(v.x), u1 = __float_as_uint(v.y), u2 = __float_as_uint(v.z), u3 = __float_as_uint(v.w);
            low |= (u0 | u1 | u2 | u3) & 0xffffu;
            packed[2 * q] = (u0 >> 16) | (u1 & 0xffff0000u); packed[2 * q + 1] = (u2 >> 16) | (u3 & 0xffff0000u);
        }
        total += sum;
        total_plain = (total_plain + eight[0]) + eight[1];
        if (sums16) sums16[uint64_t(i) * 4 + b] = sum;
        uint4* dst = reinterpret_cast<uint4*>(xb + uint64_t(r) * K + g * 64 + b * 16);
        dst[0] = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        dst[1] = make_uint4(packed[4], packed[5], packed[6], packed[7]);
    }
    if (sums) sums[i] = total;
    if (plain) plain[i] = total_plain;
    if (low) atomicOr(status, 4);
}
// The same sums for rows that are already bf16 (the SwiGLU activations).
// plain: the affine Q8 lanes' sums instead (see prefill_rows_kernel); no per-block table then.
__global__ __launch_bounds__(256) void prefill_sums_kernel(const uint16_t* xb, const int32_t* rows_ptr, uint32_t rows_max, uint32_t K, float* sums, float* sums16,
                                                           bool plain) {
    const uint32_t groups = K / 64, i = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t rows = rows_ptr ? min(uint32_t(*rows_ptr), rows_max) : rows_max;
    if (i >= rows * groups) return;
    const uint32_t r = i / groups, g = i % groups;
    const uint4* src = reinterpret_cast<const uint4*>(xb + uint64_t(r) * K + g * 64);
    float total = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const uint4 lo = src[2 * b], hi = src[2 * b + 1];
        const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        float sum = 0, eight[2] = {0, 0};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float a = __uint_as_float(w[2 * q] << 16), c = __uint_as_float(w[2 * q] & 0xffff0000u);
            const float d = __uint_as_float(w[2 * q + 1] << 16), e = __uint_as_float(w[2 * q + 1] & 0xffff0000u);
            sum += bf(bf(bf(a + c) + d) + e);
            eight[q / 2] = (((eight[q / 2] + a) + c) + d) + e;
        }
        total = plain ? (total + eight[0]) + eight[1] : total + sum;
        if (sums16 && !plain) sums16[uint64_t(i) * 4 + b] = sum;
    }
    sums[i] = total;
}

// Work list: tile t = (expert, first sorted position, rows).  offsets[e] .. offsets[e+1] are the expert's sorted
// positions (the dispatch kernel's output); a null offsets pointer means ONE group of `rows` rows (the shared expert).
__global__ __launch_bounds__(1024) void prefill_tiles_kernel(const int32_t* offsets, uint32_t experts, uint32_t rows, int32_t* tile_expert,
                                                            int32_t* tile_first, int32_t* tile_rows, int32_t* tile_count) {
    __shared__ int32_t scan[1024];
    const uint32_t e = threadIdx.x;
    const int32_t first = offsets ? (e < experts ? offsets[e] : 0) : 0, count = offsets ? (e < experts ? offsets[e + 1] - offsets[e] : 0) : (e == 0 ? int32_t(rows) : 0);
    // whole tiles of 32 rows; what is left joins the last of them when that gives at most 48 rows, else it is a tile of its own
    const int32_t whole = count / int32_t(kTileRows), left = count % int32_t(kTileRows);
    const int32_t tiles = count == 0 ? 0 : (whole == 0 ? 1 : whole + (left > int32_t(kTileRowsMax - kTileRows) ? 1 : 0));
    scan[e] = tiles;
    __syncthreads();
    for (uint32_t step = 1; step < 1024; step <<= 1) {
        const int32_t add = e >= step ? scan[e - step] : 0;
        __syncthreads();
        scan[e] += add;
        __syncthreads();
    }
    const int32_t begin = scan[e] - tiles;
    for (int32_t t = 0; t < tiles; ++t) {
        tile_expert[begin + t] = int32_t(e); tile_first[begin + t] = first + t * int32_t(kTileRows);
        tile_rows[begin + t] = t + 1 < tiles ? int32_t(kTileRows) : count - t * int32_t(kTileRows);   // the last tile takes what is left (at most 48)
    }
    if (e == 1023) *tile_count = scan[1023];
}

// The dispatch sort of a long batch and the routed experts' work list in ONE launch (the decode path's three dispatch
// kernels and prefill_tiles_kernel hold the same steps as four launches in a row, each of them short: what they cost was
// the four launches).  A workgroup = four experts (one per wave) x one of kDispatchParts stretches of the slots.  Every
// workgroup counts ALL the slots' experts, per stretch, into a table in LDS and keeps its own stretch of the ids there;
// it scans the table (sorted offsets and tile counts of every expert), and each wave then places its expert's slots of
// the workgroup's stretch in ascending slot order, starting where the earlier stretches' slots of that expert end.  The
// workgroups of the first stretch also write their experts' tiles, workgroup (0, 0) the offsets.  Same results as
// launch_dispatch followed by launch_prefill_tiles; the list of selected experts is not written (nothing here reads it).
// ids sixteen-byte aligned; stretch: slots per stretch, a multiple of 1024.
constexpr uint32_t kDispatchParts = 4;
__global__ __launch_bounds__(256) void prefill_dispatch_kernel(const int32_t* __restrict__ ids, uint32_t n, uint32_t topk, uint32_t E, uint32_t stretch,
                                                               int32_t* __restrict__ offsets, int32_t* __restrict__ slots, int32_t* __restrict__ rows, int32_t* status,
                                                               int32_t* tile_expert, int32_t* tile_first, int32_t* tile_rows, int32_t* tile_count) {
    extern __shared__ __align__(16) int32_t table[];   // [parts][E] counts, [E + 1] offsets, [E + 1] tiles before, then the stretch's ids
    __shared__ int32_t wave_sum[2][4];
    int32_t* cnt = table; int32_t* off = table + kDispatchParts * E; int32_t* tiles_before = off + E + 1;
    int32_t* copy = table + ((kDispatchParts + 2) * E + 2 + 3) / 4 * 4;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, part = blockIdx.y, first = part * stretch;
    for (uint32_t i = tid; i < kDispatchParts * E; i += 256) cnt[i] = 0;
    __syncthreads();
    {
        int bad = 0;
        uint32_t at = 0, until = stretch;   // the stretch of slot p: counted up as p goes
        for (uint32_t b0 = 0; b0 < n; b0 += 8 * 1024) {   // eight steps' loads in flight
            int4 batch[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t p = b0 + u * 1024 + 4 * tid;
                int4 v = make_int4(-1, -1, -1, -1);   // (-1: past the end)
                if (p + 3 < n) v = *reinterpret_cast<const int4*>(ids + p);
                else { if (p < n) v.x = ids[p]; if (p + 1 < n) v.y = ids[p + 1]; if (p + 2 < n) v.z = ids[p + 2]; }
                batch[u] = v;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t p0 = b0 + u * 1024, p = p0 + 4 * tid;
                if (p0 >= n) break;
                if (p0 >= until) { ++at; until += stretch; }
                const int32_t four[4] = {batch[u].x, batch[u].y, batch[u].z, batch[u].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (p + j >= n) continue;
                    if (four[j] < 0 || four[j] >= int32_t(E)) bad = 1; else atomicAdd(&cnt[at * E + uint32_t(four[j])], 1);
                }
                if (at == part) *reinterpret_cast<int4*>(copy + (p - first)) = batch[u];
            }
        }
        if (bad && blockIdx.x == 0 && part == 0) atomicOr(status, 1);
    }
    __syncthreads();
    auto count_of = [&](uint32_t e) { int32_t c = 0; for (uint32_t q = 0; q < kDispatchParts; ++q) c += cnt[q * E + e]; return c; };
    {   // exclusive scans over the experts: thread t owns experts t * per .. t * per + per - 1
        const uint32_t per = (E + 255) / 256;
        auto tiles_of = [](int32_t count) {
            const int32_t whole = count / int32_t(kTileRows), left = count % int32_t(kTileRows);
            return count == 0 ? 0 : (whole == 0 ? 1 : whole + (left > int32_t(kTileRowsMax - kTileRows) ? 1 : 0));
        };
        int32_t mine[2] = {0, 0};
        for (uint32_t i = 0; i < per; ++i) { const uint32_t e = tid * per + i; if (e < E) { const int32_t c = count_of(e); mine[0] += c; mine[1] += tiles_of(c); } }
        int32_t incl[2] = {mine[0], mine[1]};
#pragma unroll
        for (int o = 1; o < 64; o <<= 1)
#pragma unroll
            for (int v = 0; v < 2; ++v) { const int32_t up = __shfl_up(incl[v], o); if (int(lane) >= o) incl[v] += up; }
        if (lane == 63) { wave_sum[0][wave] = incl[0]; wave_sum[1][wave] = incl[1]; }
        __syncthreads();
        int32_t at[2];
#pragma unroll
        for (int v = 0; v < 2; ++v) { at[v] = incl[v] - mine[v]; for (uint32_t w = 0; w < wave; ++w) at[v] += wave_sum[v][w]; }
        for (uint32_t i = 0; i < per; ++i) {
            const uint32_t e = tid * per + i;
            if (e < E) { const int32_t c = count_of(e); off[e] = at[0]; tiles_before[e] = at[1]; at[0] += c; at[1] += tiles_of(c); }
        }
        if (tid == 255) { off[E] = at[0]; tiles_before[E] = at[1]; }
        __syncthreads();
    }
    if (blockIdx.x == 0 && part == 0) {
        for (uint32_t e = tid; e <= E; e += 256) offsets[e] = off[e];
        if (tid == 0) *tile_count = tiles_before[E];
    }
    const uint32_t e = blockIdx.x * 4 + wave;
    if (e >= E) return;
    const int32_t count = count_of(e);
    if (count == 0) return;
    if (part == 0) {   // the expert's tiles: whole tiles of 32 rows, the last one takes what is left (at most 48)
        const int32_t tiles = tiles_before[e + 1] - tiles_before[e], begin = tiles_before[e];
        for (int32_t t = int32_t(lane); t < tiles; t += 64) {
            tile_expert[begin + t] = int32_t(e); tile_first[begin + t] = off[e] + t * int32_t(kTileRows);
            tile_rows[begin + t] = t + 1 < tiles ? int32_t(kTileRows) : count - t * int32_t(kTileRows);
        }
    }
    int32_t pos = off[e];
    for (uint32_t q = 0; q < part; ++q) pos += cnt[q * E + e];
    const int32_t end = pos + cnt[part * E + e];
    const uint64_t below = (1ull << lane) - 1;
    const float inverse = 1.0f / float(topk);
    // 256 slots per step, in order: four neighbouring slots per lane, slots of lower lanes first, then the lane's own
    for (uint32_t q0 = first; q0 < n && q0 < first + stretch && pos < end; q0 += 256) {
        const uint32_t p = q0 + 4 * lane;
        const int4 v = *reinterpret_cast<const int4*>(copy + (p - first));
        const bool m[4] = {v.x == int32_t(e), v.y == int32_t(e), v.z == int32_t(e), v.w == int32_t(e)};
        const uint64_t mask[4] = {__ballot(m[0]), __ballot(m[1]), __ballot(m[2]), __ballot(m[3])};
        if ((mask[0] | mask[1] | mask[2] | mask[3]) == 0) continue;   // uniform: none of these 256 slots is the expert's
        int32_t at = pos + __popcll(mask[0] & below) + __popcll(mask[1] & below) + __popcll(mask[2] & below) + __popcll(mask[3] & below);
        // token and rank of slot p (p < 2^24: the rounded quotient is off by one at most)
        uint32_t token = uint32_t(float(p) * inverse);
        int32_t rest = int32_t(p) - int32_t(token * topk);
        if (rest < 0) { --token; rest += int32_t(topk); } else if (rest >= int32_t(topk)) { ++token; rest -= int32_t(topk); }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (m[j]) { slots[at] = int32_t(p + j); if (rows) rows[at] = int32_t(token); ++at; }
            if (++rest == int32_t(topk)) { rest = 0; ++token; }
        }
        pos += __popcll(mask[0]) + __popcll(mask[1]) + __popcll(mask[2]) + __popcll(mask[3]);
    }
}

// BITS: 4 (nibble codes, eight bytes of a row per lane and step) or 8 (byte codes, sixteen bytes; the chain sums are then
// the plain ones of the Q8 lanes).  A byte code is exact in bf16 like a nibble code, and its product with a BF16 value is
// exact in fp32.
template <bool GATED, int BITS>
__global__ __launch_bounds__(256) void prefill_gemm_kernel(PrefillGemm p) {
    __shared__ __align__(16) uint16_t a_s[2][kTileRowsMax * kPitch];
    // The scales and biases of the workgroup's 128 weight rows and the chain sums of its token rows, for every step, are
    // brought in once (whole runs of consecutive bytes: fetched step by step they cost a cache access per row and step
    // for two or four bytes each, more accesses than the codes and the token rows together).
    extern __shared__ __align__(16) uint8_t meta_s[];
    __shared__ uint32_t row_s[kTileRowsMax];
    const uint32_t tile = blockIdx.y;
    if (tile >= uint32_t(*p.tile_count)) return;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, j = lane & 15u, g4 = lane >> 4;
    const uint32_t expert = uint32_t(p.tile_expert[tile]), first = uint32_t(p.tile_first[tile]), rows = uint32_t(p.tile_rows[tile]);
    const uint32_t K = p.K, N = p.N, groups = K / 64;
    const uint32_t n0 = blockIdx.x * (GATED ? 64u : 128u);
    const uint8_t* record = p.records + uint64_t(expert) * p.stride;

    // what this thread fetches every step
    const uint32_t a_r = tid >> 3, a_c = tid & 7u;                       // token row of the tile, 16-byte chunk of the step
    const uint32_t a_pos = first + min(a_r, rows - 1);                   // rows past the end repeat the last one (never stored)
    const uint32_t a_row = p.a_rows ? uint32_t(p.a_rows[a_pos]) / p.a_div : a_pos;
    const uint16_t* a_src = p.a + uint64_t(a_row) * K + a_c * 8;
    const bool tall = rows > kTileRows;                                  // a third block of sixteen rows: threads 0..127 fetch it too
    const uint32_t a_pos2 = first + min(32u + (a_r & 15u), rows - 1);
    const uint32_t a_row2 = p.a_rows ? uint32_t(p.a_rows[a_pos2]) / p.a_div : a_pos2;
    const uint16_t* a_src2 = p.a + uint64_t(a_row2) * K + a_c * 8;
    // The wave's two column tiles (rows of the workgroup's 128 weight rows) for every block of sixteen token rows; gate/up:
    // a gate tile and the up tile of the same rows.  The codes go from memory straight into the lanes that feed them to
    // the matrix cores: lane (j, g4) holds codes 16 g4 .. 16 g4 + 15 of the step for weight row j of each tile (eight
    // bytes), the first eight for one product and the rest for the next; the token rows are read from LDS in the same
    // order, and the order of k inside a step is free.
    uint32_t col_row[2];
    const uint8_t* b_src[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        col_row[q] = (GATED ? (uint32_t(q) * 64u + wave * 16u) : (2 * wave + uint32_t(q)) * 16u) + j;
        const uint32_t b_proj = GATED ? col_row[q] >> 6 : 0u, b_n = n0 + (GATED ? (col_row[q] & 63u) : col_row[q]);
        b_src[q] = record + p.off[b_proj * 3] + uint64_t(b_n) * (K * BITS / 8) + g4 * (2 * BITS);
    }
    // scales then biases as bf16 [128][groups + 2] (the pad keeps sixteen rows on different banks), then the chain sums
    // [groups][48]
    const uint32_t pitch = groups + 2;
    uint16_t* scale_s = reinterpret_cast<uint16_t*>(meta_s);
    uint16_t* bias_s = scale_s + kTileCols * pitch;
    float* sum_s = reinterpret_cast<float*>(bias_s + kTileCols * pitch);
    if (tid < kTileRowsMax) {
        const uint32_t x_pos = first + min(tid, rows - 1);
        row_s[tid] = p.a_rows ? uint32_t(p.a_rows[x_pos]) / p.a_div : x_pos;
    }
    {   // a projection's 64 (gate/up) or 128 rows are consecutive in the record: groups / 2 dwords per row
        const uint32_t half = groups / 2, per_proj = (GATED ? 64u : 128u) * half;
        for (uint32_t i = tid; i < 128u * half; i += 256) {
            const uint32_t proj = GATED ? i / per_proj : 0u, at = GATED ? i % per_proj : i, r = i / half, g2 = i % half;
            const uint32_t sv = ldg_u32(record + p.off[proj * 3 + 1] + uint64_t(n0) * groups * 2, at);
            const uint32_t ov = ldg_u32(record + p.off[proj * 3 + 2] + uint64_t(n0) * groups * 2, at);
            *reinterpret_cast<uint32_t*>(scale_s + r * pitch + 2 * g2) = sv;
            *reinterpret_cast<uint32_t*>(bias_s + r * pitch + 2 * g2) = ov;
        }
    }
    __syncthreads();
    for (uint32_t i = tid; i < kTileRowsMax * groups; i += 256) {
        const uint32_t r = i / groups, g = i % groups;
        sum_s[g * kTileRowsMax + r] = p.asum[uint64_t(row_s[r]) * groups + g];
    }

    // What a step needs is requested two steps ahead and waits in registers (two sets, taken in turn): with one step of
    // lead the loads' latency, several times a step's arithmetic, was paid at every step.
    struct Fetched { uint4 a, a2; uint32_t b[2][BITS / 2]; };   // the lane's sixteen codes of a step: two dwords (Q4) or four (Q8)
    Fetched ahead[2];
    ahead[0] = ahead[1] = Fetched{make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0), {}};
    auto fetch = [&](uint32_t g, Fetched& f) {
        f.a = *reinterpret_cast<const uint4*>(a_src + g * 64);
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            if constexpr (BITS == 4) { const uint2 v = ldg_u2(b_src[q] + g * 32); f.b[q][0] = v.x; f.b[q][1] = v.y; }
            else { const uint4 v = ldg_u4(b_src[q] + g * 64); f.b[q][0] = v.x; f.b[q][1] = v.y; f.b[q][2] = v.z; f.b[q][3] = v.w; }
        }
        if (tall && tid < 128) f.a2 = *reinterpret_cast<const uint4*>(a_src2 + g * 64);
    };
    auto stash = [&](uint32_t buf, const Fetched& f) {   // the token rows
        *reinterpret_cast<uint4*>(&a_s[buf][a_r * kPitch + a_c * 8]) = f.a;
        if (tall && tid < 128) *reinterpret_cast<uint4*>(&a_s[buf][(32 + a_r) * kPitch + a_c * 8]) = f.a2;
    };
    // eight codes -> eight bf16: nibble i of the word is element i
    auto expand = [](uint32_t word) {
        uint32_t even = word & 0x0f0f0f0fu, odd = (word >> 4) & 0x0f0f0f0fu;
        // the masked words are kept from the optimiser, which would otherwise fold mask and shift into a bit-field extract
        // per element and convert that: with whole bytes every element is one byte-to-float conversion
        asm volatile("" : "+v"(even), "+v"(odd));
        uint32_t out[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const f32x2 pair = {float((even >> (8 * q)) & 0xffu), float((odd >> (8 * q)) & 0xffu)};
            out[q] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
        }
        return __builtin_bit_cast(bf16x8, make_uint4(out[0], out[1], out[2], out[3]));
    };
    // eight byte codes (two words, byte i of the pair is element i) -> eight bf16
    auto expand_bytes = [](uint32_t lo, uint32_t hi) {
        uint32_t out[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t word = q < 2 ? lo : hi;
            const f32x2 pair = {float((word >> (16 * (q & 1))) & 0xffu), float((word >> (16 * (q & 1) + 8)) & 0xffu)};
            out[q] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
        }
        return __builtin_bit_cast(bf16x8, make_uint4(out[0], out[1], out[2], out[3]));
    };

    constexpr int kBlocks = int(kTileRowsMax / 16);
    const int blocks = tall ? kBlocks : 2;
    f32x4 total[kBlocks][2], mag[kBlocks][2];   // mag: sum of the magnitudes of the folded terms, the scale of the rounding error
#pragma unroll
    for (int rb = 0; rb < kBlocks; ++rb)
#pragma unroll
        for (int q = 0; q < 2; ++q) total[rb][q] = mag[rb][q] = f32x4{0, 0, 0, 0};

    fetch(0, ahead[0]);
    if (groups > 1) fetch(1, ahead[1]);
    stash(0, ahead[0]);
    __syncthreads();
    // The bias half of the magnitudes, sum over the groups of |bias| * |chain sum|, is a product over the group index:
    // one matrix-core instruction per accumulator tile and 32 groups instead of a multiply-add per element and step (the
    // chain sums rounded to bf16 for it, made up for by the factor below: the magnitudes only scale a margin).
    for (uint32_t g0 = 0; g0 < groups; g0 += 32) {
        bf16x8 bias_abs[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t g = g0 + 8 * g4 + 2 * uint32_t(i);
                w[i] = g < groups ? *reinterpret_cast<const uint32_t*>(bias_s + col_row[q] * pitch + g) & 0x7fff7fffu : 0u;
            }
            bias_abs[q] = __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
        }
#pragma unroll
        for (int rb = 0; rb < kBlocks; ++rb) {
            if (rb >= blocks) break;
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t g = min(g0 + 8 * g4 + 2 * uint32_t(i), groups - 2);   // (past the end: times a zero bias)
                const f32x2 pair = {fabsf(sum_s[g * kTileRowsMax + 16 * rb + j]), fabsf(sum_s[(g + 1) * kTileRowsMax + 16 * rb + j])};
                w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
            }
            const bf16x8 sum_abs = __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
#pragma unroll
            for (int q = 0; q < 2; ++q) mag[rb][q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sum_abs, bias_abs[q], mag[rb][q], 0, 0, 0);
        }
    }
#pragma unroll
    for (int rb = 0; rb < kBlocks; ++rb)
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int r = 0; r < 4; ++r) mag[rb][q][r] *= 1.0078125f;
    // two steps per trip, so that the register sets are named at compile time: step g computes from LDS buffer g & 1, requests
    // step g + 2 into the set that step g's data has just left, and stashes step g + 1 from the other set
    auto step = [&](uint32_t g, Fetched& mine, Fetched& next) {
        const uint32_t buf = g & 1u;
        bf16x8 b[2][2];   // [tile][half of the lane's sixteen codes]
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            if constexpr (BITS == 4) { b[q][0] = expand(mine.b[q][0]); b[q][1] = expand(mine.b[q][1]); }
            else { b[q][0] = expand_bytes(mine.b[q][0], mine.b[q][1]); b[q][1] = expand_bytes(mine.b[q][2], mine.b[q][3]); }
        }
        if (g + 2 < groups) fetch(g + 2, mine);
        f32x4 dot[kBlocks][2];
#pragma unroll
        for (int rb = 0; rb < kBlocks; ++rb)
#pragma unroll
            for (int q = 0; q < 2; ++q) dot[rb][q] = f32x4{0, 0, 0, 0};
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
            for (int rb = 0; rb < kBlocks; ++rb) {
                if (rb >= blocks) break;
                const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&a_s[buf][(16 * rb + j) * kPitch + g4 * 16 + kk * 8]));
#pragma unroll
                for (int q = 0; q < 2; ++q) dot[rb][q] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[q][kk], dot[rb][q], 0, 0, 0);
            }
        }
        float scale[2], bias[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) { scale[q] = b16(scale_s[col_row[q] * pitch + g]); bias[q] = b16(bias_s[col_row[q] * pitch + g]); }
#pragma unroll
        for (int rb = 0; rb < kBlocks; ++rb) {
            if (rb >= blocks) break;
            const float4 sums4 = *reinterpret_cast<const float4*>(sum_s + g * kTileRowsMax + 16 * rb + 4 * g4);
            const float sums[4] = {sums4.x, sums4.y, sums4.z, sums4.w};
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    total[rb][q][r] = __builtin_fmaf(scale[q], dot[rb][q][r], __builtin_fmaf(bias[q], sums[r], total[rb][q][r]));
                    mag[rb][q][r] = __builtin_fmaf(fabsf(scale[q]), fabsf(dot[rb][q][r]), mag[rb][q][r]);
                }
        }
        if (g + 1 < groups) stash(buf ^ 1u, next);
        __syncthreads();
    };
    for (uint32_t g = 0; g < groups; g += 2) {
        step(g, ahead[0], ahead[1]);
        if (g + 1 < groups) step(g + 1, ahead[1], ahead[0]);
    }
    // epilogue: row m of the tile is sorted position first + m.  A sum close to a BF16 rounding boundary could round
    // the other way under the reference's order of additions: such elements are listed for exact recomputation.
    const float margin = p.near_margin;
    auto near_boundary = [margin](float v, float m) { const float e = m * margin; return __float_as_uint(bf(v - e)) != __float_as_uint(bf(v + e)); };
    // One bit per output element (sorted position * N + row); every wave owns whole 16-bit pieces of the map: the sixteen
    // lanes that share a token row hold sixteen neighbouring weight rows.
    uint16_t* bits = reinterpret_cast<uint16_t*>(p.near_bits);
#pragma unroll
    for (int rb = 0; rb < kBlocks; ++rb) {
        if (rb >= blocks) break;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t m = 16 * uint32_t(rb) + 4 * g4 + uint32_t(r);
            const bool live = m < rows;
            const uint32_t pos = first + (live ? m : 0u);
            if constexpr (GATED) {
                const uint32_t n = n0 + wave * 16 + j;
                if (live) p.out_b[uint64_t(pos) * N + n] = uint16_t(__float_as_uint(swiglu_bf(total[rb][0][r], total[rb][1][r])) >> 16);
                const uint64_t marks = __ballot(near_boundary(total[rb][0][r], mag[rb][0][r]) || near_boundary(total[rb][1][r], mag[rb][1][r]));
                if (live && j == 0) bits[(uint64_t(pos) * N + n) / 16] = uint16_t(marks >> (16 * g4));
            } else {
                const uint32_t out_row = p.out_rows ? uint32_t(p.out_rows[pos]) : pos;
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const uint32_t n = n0 + (2 * wave + uint32_t(q)) * 16 + j;
                    if (live) {
                        if (p.out_h) p.out_h[uint64_t(out_row) * N + n] = uint16_t(__float_as_uint(bf(total[rb][q][r])) >> 16);
                        else p.out_f[uint64_t(out_row) * N + n] = bf(total[rb][q][r]);
                    }
                    const uint64_t marks = __ballot(near_boundary(total[rb][q][r], mag[rb][q][r]));
                    if (live && j == 0) bits[(uint64_t(pos) * N + n) / 16] = uint16_t(marks >> (16 * g4));
                }
            }
        }
    }
}

// Exact recomputation of the listed elements: one group of 32 lanes plays the reference's 32 lanes for one row
// (qwen.metal:46-62: lane width 16 when K % 512 == 0 and N % 8 == 0, else 8; xor-butterfly lane sum).
// BITS 8: the affine Q8 lanes (qwen.metal:112-125: lane width 8 when K % 512 == 0 and N % 8 == 0, else 4; the input sum is the
// plain fp32 sum, the dot a multiply-add chain element by element).
constexpr uint32_t kPatchWordsMax = 256;
template <int WIDTH, bool GATED, bool TABLED, int BITS>
__global__ __launch_bounds__(256) void prefill_patch_kernel(PrefillGemm p, uint32_t words_per_group) {
    // each workgroup scans words_per_group words of the map (few for a small map, so that it still spreads over the chip),
    // gathers the marked elements in LDS, then its eight 32-lane groups take them in turn
    __shared__ uint16_t found[kPatchWordsMax * 32];
    __shared__ uint32_t found_count;
    const uint32_t lane = threadIdx.x & 31u;
    const uint32_t K = p.K, N = p.N, groups = K / 64;
    const uint32_t word = blockIdx.x * words_per_group + threadIdx.x;
    if (threadIdx.x == 0) found_count = 0;
    __syncthreads();
    // Only the map words of covered positions were written by the product kernel: a word past them holds whatever the
    // buffer held before.  N is a multiple of 32, so a word never straddles two positions.
    const uint32_t positions = p.near_words / (N / 32u);
    const uint32_t covered = p.covered ? min(uint32_t(max(*p.covered, 0)), positions) : positions;
    uint32_t marks = (threadIdx.x < words_per_group && word < p.near_words && word / (N / 32u) < covered) ? p.near_bits[word] : 0u;
    if (marks) {
        uint32_t at = atomicAdd(&found_count, uint32_t(__popc(marks)));
        while (marks) { found[at++] = uint16_t(threadIdx.x * 32 + (__ffs(marks) - 1)); marks &= marks - 1; }
    }
    __syncthreads();
    const uint32_t listed = found_count;
  for (uint32_t item = threadIdx.x >> 5; item < listed; item += 8) {
    const uint32_t code = blockIdx.x * (words_per_group * 32u) + found[item], pos = code / N, n = code % N;
    const uint32_t expert = p.ids ? uint32_t(p.ids[p.slots[pos]]) : 0u;
    if (p.ids && expert >= p.experts) continue;   // an id the router could not give (reported through the status word)
    const uint8_t* record = p.records + uint64_t(expert) * p.stride;
    const uint32_t a_row = p.a_rows ? uint32_t(p.a_rows[pos]) / p.a_div : pos;
    const uint16_t* xr = p.a + uint64_t(a_row) * K;
    static_assert(WIDTH * BITS >= 32 && !(TABLED && BITS == 8), "a block is whole code words; the table holds Q4 chain sums");
    constexpr int DW = WIDTH * BITS / 32, XV = WIDTH >= 8 ? WIDTH / 8 : 1, kAhead = 4;   // a lane's next four blocks are fetched together: one memory latency, not four
    float result[2] = {0, 0};
    const uint32_t blocks = K / WIDTH;
    for (uint32_t b0 = lane; b0 < blocks; b0 += 32 * kAhead) {
        uint4 xv[kAhead][XV];
        uint32_t words[kAhead][GATED ? 2 : 1][DW];
        uint16_t scale_bits[kAhead][GATED ? 2 : 1], bias_bits[kAhead][GATED ? 2 : 1];
        // the block's BF16-rounded chain sum depends on the row only: with 16-element blocks it comes from the table the
        // row kernels left (the same additions in the same order)
        constexpr bool tabled = TABLED;   // a compile-time choice: with both forms in one kernel the registers of either stay live
        float chain[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const uint32_t b = min(b0 + 32u * u, blocks - 1);   // past the end: the last block again, not used
            if constexpr (WIDTH >= 8) {
#pragma unroll
                for (int i = 0; i < WIDTH / 8; ++i) xv[u][i] = *reinterpret_cast<const uint4*>(xr + b * WIDTH + 8 * i);
            } else {
                const uint2 v = *reinterpret_cast<const uint2*>(xr + b * WIDTH);   // four inputs
                xv[u][0] = make_uint4(v.x, v.y, 0, 0);
            }
            chain[u] = tabled ? p.asum16[uint64_t(a_row) * (K / 16) + b] : 0.0f;
            const uint32_t g = n * groups + (b * WIDTH) / 64;
#pragma unroll
            for (int proj = 0; proj < (GATED ? 2 : 1); ++proj) {
                const uint32_t* src = reinterpret_cast<const uint32_t*>(record + p.off[proj * 3] + uint64_t(n) * (K * BITS / 8)) + b * DW;
#pragma unroll
                for (int i = 0; i < DW; ++i) words[u][proj][i] = src[i];
                scale_bits[u][proj] = reinterpret_cast<const uint16_t*>(record + p.off[proj * 3 + 1])[g];
                bias_bits[u][proj] = reinterpret_cast<const uint16_t*>(record + p.off[proj * 3 + 2])[g];
            }
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            if (b0 + 32u * u >= blocks) break;
            float xb[WIDTH];
#pragma unroll
            for (int i = 0; i < WIDTH; i += 2) {
                const uint4 v = xv[u][i / 8];
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
                xb[i] = __uint_as_float(w[(i % 8) / 2] << 16); xb[i + 1] = __uint_as_float(w[(i % 8) / 2] & 0xffff0000u);
            }
            float sum = chain[u];
            if constexpr (BITS == 8) {
#pragma unroll
                for (int i = 0; i < WIDTH; ++i) sum += xb[i];
            } else if (!tabled) {
#pragma unroll
                for (int i = 0; i < WIDTH; i += 4) sum += bf(bf(bf(xb[i] + xb[i + 1]) + xb[i + 2]) + xb[i + 3]);
            }
#pragma unroll
            for (int proj = 0; proj < (GATED ? 2 : 1); ++proj) {
                float dot = 0;
                if constexpr (BITS == 8) {
                    // (a BF16 value times a byte code is exact in fp32: the fused multiply-add rounds as the reference's multiply and add)
#pragma unroll
                    for (int i = 0; i < WIDTH; ++i) dot = __builtin_fmaf(xb[i], float((words[u][proj][i / 4] >> (8 * (i % 4))) & 0xffu), dot);
                } else
#pragma unroll
                for (int i = 0; i < WIDTH; i += 8) {
                    // nibble j of a word is element j: the even ones and the odd ones as bytes, each converted by one byte-to-float instruction
                    const uint32_t even = words[u][proj][i / 8] & 0x0f0f0f0fu, odd = (words[u][proj][i / 8] >> 4) & 0x0f0f0f0fu;
                    // (a BF16 value times a 4-bit code is exact in fp32, so a fused multiply-add rounds as the reference's
                    // multiply and add do: ((p0 + p1) + p2) + p3, then onto the block's sum)
                    dot += __builtin_fmaf(xb[i + 3], float((odd >> 8) & 0xffu), __builtin_fmaf(xb[i + 2], float((even >> 8) & 0xffu),
                           __builtin_fmaf(xb[i + 1], float(odd & 0xffu), xb[i] * float(even & 0xffu))));
                    dot += __builtin_fmaf(xb[i + 7], float(odd >> 24), __builtin_fmaf(xb[i + 6], float(even >> 24),
                           __builtin_fmaf(xb[i + 5], float((odd >> 16) & 0xffu), xb[i + 4] * float((even >> 16) & 0xffu))));
                }
                result[proj] += b16(scale_bits[u][proj]) * dot + sum * b16(bias_bits[u][proj]);
            }
        }
    }
    result[0] = lane_sum32(result[0]);
    if constexpr (GATED) result[1] = lane_sum32(result[1]);
    if (lane == 0) {
        if constexpr (GATED) p.out_b[uint64_t(pos) * N + n] = uint16_t(__float_as_uint(swiglu_bf(result[0], result[1])) >> 16);
        else {
            const uint64_t at = uint64_t(p.out_rows ? uint32_t(p.out_rows[pos]) : pos) * N + n;
            if (p.out_h) p.out_h[at] = uint16_t(__float_as_uint(bf(result[0])) >> 16); else p.out_f[at] = bf(result[0]);
        }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// Router logits of a long batch without the exact chains for every (token, expert): a bf16 matrix-core product gives
// every logit to within a bound that holds whatever the order of its additions, the top-k can only come from the
// logits within that bound of the k-th largest, and only those are recomputed with the reference's chains
// (qwen.metal:512-534: sixteen contiguous K partitions, a k-ascending multiply-accumulate chain in each, partials added
// 0..15).  The other logits are written as -inf, so the exact selection kernel that follows picks what it would pick from
// all the exact logits: ids and softmax weights are the reference's bits.
//
// The bound.  Inputs and router weights are BF16-valued, so every product is exact in fp32.  Two fp32 sums of the same n
// exact products, each formed with at most n additions that round or truncate to fp32, differ by at most
// n * 2^-22 * sum |x_k w_k| (n * 2^-23 for a truncating accumulator plus n * 2^-24 for the reference's rounded chain
// leaves a factor 1.3), and sum |x_k w_k| <= |x| |w| (Cauchy-Schwarz).  Adding the expert's offset rounds both once more:
// 2^-22 |logit| on top.  With lower bounds a - m and upper bounds a + m of the exact logits: the k-th largest exact logit
// is at least the k-th largest lower bound, which is at least the k-th largest of the 64 lanes' largest lower bounds; an
// expert whose upper bound is below that cannot be among the top k, ties included.  A token with a logit that is not
// finite has every expert recomputed.
// ---------------------------------------------------------------------------------------------------------------------
// |row| of bf16 rows, rounded up a little: one wavefront per row; rows [0, rows_a) come from a, the rest from b.
__global__ __launch_bounds__(256) void row_norms_kernel(const uint16_t* a, uint32_t rows_a, const uint16_t* b, uint32_t rows_b, uint32_t K, float* norms) {
    const uint32_t row = blockIdx.x * 4 + threadIdx.x / 64, lane = threadIdx.x & 63u;
    if (row >= rows_a + rows_b) return;
    const uint16_t* src = row < rows_a ? a + uint64_t(row) * K : b + uint64_t(row - rows_a) * K;
    float sum = 0;
    for (uint32_t i = lane * 8; i < K; i += 512) {
        const uint4 v = *reinterpret_cast<const uint4*>(src + i);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float lo = __uint_as_float(w[q] << 16), hi = __uint_as_float(w[q] & 0xffff0000u);
            sum = __builtin_fmaf(lo, lo, sum); sum = __builtin_fmaf(hi, hi, sum);
        }
    }
#pragma unroll
    for (int o = 32; o; o >>= 1) sum += __shfl_xor(sum, o);
    // (a row so small that its squares leave the normal range has no usable norm: +inf makes the caller recompute everything)
    if (lane == 0) norms[row] = sum < 0x1p-100f ? __uint_as_float(0x7f800000u) : sqrtf(sum) * 1.0001f;
}
// approx[t][e] = sum_k a[t][k] b[e][k] (+ offsets[e]): 64 tokens x 64 experts per workgroup, a wave a 32 x 32 block on
// v_mfma_f32_32x32x16_bf16, K in steps of 64 through LDS (rows padded to 144 bytes), the next step's rows in registers.
__global__ __launch_bounds__(256) void router_product_kernel(const uint16_t* a, const uint16_t* b, uint32_t T, uint32_t E, uint32_t K,
                                                             const float* offsets, float* approx) {
    __shared__ __align__(16) uint16_t a_s[2][64 * kPitch], b_s[2][64 * kPitch];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, m = lane & 31u, h = lane >> 5;
    const uint32_t t0 = blockIdx.y * 64, e0 = blockIdx.x * 64;
    const uint32_t r = tid >> 3, c8 = tid & 7u;   // a thread moves rows r and r + 32, sixteen bytes each, of both operands
    const uint16_t* a_src0 = a + uint64_t(min(t0 + r, T - 1)) * K + c8 * 8;
    const uint16_t* a_src1 = a + uint64_t(min(t0 + r + 32, T - 1)) * K + c8 * 8;
    const uint16_t* b_src0 = b + uint64_t(min(e0 + r, E - 1)) * K + c8 * 8;
    const uint16_t* b_src1 = b + uint64_t(min(e0 + r + 32, E - 1)) * K + c8 * 8;
    uint4 ra0, ra1, rb0, rb1;
    auto fetch = [&](uint32_t g) {
        ra0 = *reinterpret_cast<const uint4*>(a_src0 + g * 64); ra1 = *reinterpret_cast<const uint4*>(a_src1 + g * 64);
        rb0 = *reinterpret_cast<const uint4*>(b_src0 + g * 64); rb1 = *reinterpret_cast<const uint4*>(b_src1 + g * 64);
    };
    auto stash = [&](uint32_t buf) {
        *reinterpret_cast<uint4*>(&a_s[buf][r * kPitch + c8 * 8]) = ra0; *reinterpret_cast<uint4*>(&a_s[buf][(r + 32) * kPitch + c8 * 8]) = ra1;
        *reinterpret_cast<uint4*>(&b_s[buf][r * kPitch + c8 * 8]) = rb0; *reinterpret_cast<uint4*>(&b_s[buf][(r + 32) * kPitch + c8 * 8]) = rb1;
    };
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
    const uint32_t steps = K / 64, row_a = (wave >> 1) * 32 + m, row_b = (wave & 1u) * 32 + m;
    fetch(0); stash(0);
    __syncthreads();
    for (uint32_t g = 0; g < steps; ++g) {
        const uint32_t buf = g & 1u;
        if (g + 1 < steps) fetch(g + 1);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const bf16x8 av = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&a_s[buf][row_a * kPitch + q * 16 + h * 8]));
            const bf16x8 bv = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(&b_s[buf][row_b * kPitch + q * 16 + h * 8]));
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
        }
        if (g + 1 < steps) stash(buf ^ 1u);
        __syncthreads();
    }
    const uint32_t e = e0 + (wave & 1u) * 32 + m;
    const float offset = (offsets && e < E) ? offsets[e] : 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t t = t0 + (wave >> 1) * 32 + 8 * uint32_t(i / 4) + 4 * h + uint32_t(i % 4);
        if (t < T && e < E) approx[uint64_t(t) * E + e] = offsets ? acc[i] + offset : acc[i];
    }
}
// One wavefront per token: bounds, the experts that can be among the top k, their exact logits; everything else -inf.
// (A whole workgroup per token, each wavefront taking a quarter of the list, measured slower: 35 against 29 us.)
// ids / weights not null (topk <= 64): the wavefront also selects its token's top k and forms the softmax weights from the
// row it holds in LDS (route_token, the selection of the decode kernels: the same ids and weights as route_kernel's), and
// the row itself is not written out.
constexpr int kRefinePerLane = 16;   // experts <= 1024
__global__ __launch_bounds__(256) void router_refine_kernel(const uint16_t* xb, const uint16_t* w, const float* offsets, const float* norms,
                                                            uint32_t T, uint32_t E, uint32_t K, uint32_t topk, float* logits,
                                                            int32_t* ids, float* weights) {
    __shared__ float row_s[4][1024];
    __shared__ uint16_t list_s[4][1024];
    __shared__ uint32_t pick_s[4][128];                      // route_token's scratch
    __shared__ int32_t ids_s[4][64]; __shared__ float weights_s[4][64];
    extern __shared__ __align__(16) uint16_t x_s[];   // the four tokens' input rows (BF16-valued, so the bf16 copy is the input)
    const uint32_t wave = threadIdx.x / 64, lane = threadIdx.x & 63u, t = blockIdx.x * 4 + wave;
    if (t >= T) return;
    uint16_t* x_row = x_s + wave * K;
    for (uint32_t i = lane * 8; i < K; i += 512) *reinterpret_cast<uint4*>(x_row + i) = *reinterpret_cast<const uint4*>(xb + uint64_t(t) * K + i);
    const float ninf = __uint_as_float(0xff800000u);
    float* row = logits + uint64_t(t) * E;
    const float reach = float(K) * 0x1p-22f * norms[t];
    float upper[kRefinePerLane], best_lower = ninf;
    bool strange = false;
#pragma unroll
    for (int i = 0; i < kRefinePerLane; ++i) {
        const uint32_t e = lane + 64u * uint32_t(i);
        upper[i] = ninf;
        if (e < E) {
            const float a = row[e], bound = reach * norms[T + e] + 0x1p-22f * fabsf(a);
            strange = strange || !(fabsf(a) < __uint_as_float(0x7f800000u)) || !(bound < __uint_as_float(0x7f800000u));
            upper[i] = a + bound;
            best_lower = fmaxf(best_lower, a - bound);
        }
    }
    // the k-th largest of the lanes' largest lower bounds (fewer than k lanes with an expert: nothing can be ruled out)
    float threshold = ninf;
    bool all = __ballot(strange) != 0;
    {
        float mine = best_lower;
        for (uint32_t j = 0; j < topk && !all; ++j) {
            float top = mine;
#pragma unroll
            for (int o = 32; o; o >>= 1) top = fmaxf(top, __shfl_xor(top, o));
            if (!(top > ninf)) { all = true; break; }
            threshold = top;
            const uint64_t holders = __ballot(mine == top);
            if (lane == uint32_t(__ffsll((long long)holders) - 1)) mine = ninf;
        }
    }
    // the list of experts to recompute, in any order
    uint32_t count = 0;
#pragma unroll
    for (int i = 0; i < kRefinePerLane; ++i) {
        const uint32_t e = lane + 64u * uint32_t(i);
        const bool take = e < E && (all || upper[i] >= threshold);
        const uint64_t takers = __ballot(take);
        if (take) list_s[wave][count + uint32_t(__popcll(takers & ((1ull << lane) - 1)))] = uint16_t(e);
        count += uint32_t(__popcll(takers));
        if (e < E) row_s[wave][e] = ninf;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // four experts at a time: sixteen lanes run an expert's sixteen partition chains (router_kernel's arithmetic).  Eight weight
    // pieces = 64 elements are requested together, and the next eight -- of this expert or of the next four's -- before the
    // current ones are used.
    const uint32_t split = lane % 16, P = K / 16, base = lane & ~15u;
    const uint16_t* xr = x_row + split * P;
    const uint32_t batches = (P + 63) / 64, total = (count + 3) / 4 * batches;
    auto request = [&](uint32_t index, uint4 (&piece)[8]) {
        const uint32_t at = min(index / batches * 4 + lane / 16, count - 1), i0 = index % batches * 64;
        const uint16_t* wr = w + uint64_t(list_s[wave][at]) * K + split * P;
#pragma unroll
        for (int q = 0; q < 8; ++q) piece[q] = *reinterpret_cast<const uint4*>(wr + min(i0 + 8 * uint32_t(q), P - 8));
    };
    uint4 ahead[8];
    if (total) request(0, ahead);
    float c = 0;
    for (uint32_t index = 0; index < total; ++index) {
        uint4 piece[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) piece[q] = ahead[q];
        if (index + 1 < total) request(index + 1, ahead);
        const uint32_t i0 = index % batches * 64;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            if (i0 + 8 * uint32_t(q) >= P) break;
            const uint4 xv4 = *reinterpret_cast<const uint4*>(xr + i0 + 8 * q);
            const uint32_t ww[4] = {piece[q].x, piece[q].y, piece[q].z, piece[q].w}, xw[4] = {xv4.x, xv4.y, xv4.z, xv4.w};
#pragma unroll
            for (int k = 0; k < 8; ++k)
                c = __builtin_fmaf(__uint_as_float((k & 1) ? (xw[k / 2] & 0xffff0000u) : (xw[k / 2] << 16)),
                                   __uint_as_float((k & 1) ? (ww[k / 2] & 0xffff0000u) : (ww[k / 2] << 16)), c);
        }
        if (index % batches + 1 == batches) {   // the expert's chains are complete: partials added 0..15, then the offset
            const uint32_t at = index / batches * 4 + lane / 16;
            float sum = 0;
            for (uint32_t sidx = 0; sidx < 16; ++sidx) sum += __shfl(c, base + sidx);
            if (split == 0 && at < count) { const uint32_t e = list_s[wave][at]; row_s[wave][e] = offsets ? sum + offsets[e] : sum; }
            c = 0;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (!ids) { for (uint32_t e = lane; e < E; e += 64) row[e] = row_s[wave][e]; return; }
    auto fetch = [&](auto& cand, uint32_t per) {
        constexpr int PER = int(sizeof(cand) / sizeof(float));
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const uint32_t e = lane * per + uint32_t(i);
            cand[i] = (uint32_t(i) < per && e < E) ? row_s[wave][e] : ninf;
        }
    };
    if (E == 512) route_token<8>(fetch, E, topk, lane, ids_s[wave], weights_s[wave], pick_s[wave], []() {}, []() {});
    else route_token<16>(fetch, E, topk, lane, ids_s[wave], weights_s[wave], pick_s[wave], []() {}, []() {});
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (lane < topk) { ids[uint64_t(t) * topk + lane] = ids_s[wave][lane]; weights[uint64_t(t) * topk + lane] = weights_s[wave][lane]; }
}
// Router logits for the selection that follows: exact where it can matter, -inf elsewhere.  xb: the inputs as bf16 rows;
// norms: rows + experts floats of scratch.  K % 128 == 0, experts <= 1024.
void launch_prefill_router(hipStream_t s, const float* x, const uint16_t* xb, const void* w, const float* offsets, uint32_t T, uint32_t K,
                           uint32_t E, uint32_t topk, float* norms, float* logits, int32_t* ids, float* weights) {
    const uint16_t* wb = static_cast<const uint16_t*>(w);
    hipLaunchKernelGGL(row_norms_kernel, dim3((T + E + 3) / 4), dim3(256), 0, s, xb, T, wb, E, K, norms);
    hipLaunchKernelGGL(router_product_kernel, dim3((E + 63) / 64, (T + 63) / 64), dim3(256), 0, s, xb, wb, T, E, K, offsets, logits);
    hipLaunchKernelGGL(router_refine_kernel, dim3((T + 3) / 4), dim3(256), 4 * K * 2, s, xb, wb, offsets, norms, T, E, K, topk, logits, ids, weights);
}

void launch_prefill_rows(hipStream_t s, const float* x, uint32_t rows, uint32_t K, uint16_t* xb, float* sums, float* sums16, float* plain, int32_t* status) {
    const uint32_t items = rows * (K / 64);
    hipLaunchKernelGGL(prefill_rows_kernel, dim3((items + 255) / 256), dim3(256), 0, s, x, rows, K, xb, sums, sums16, plain, status);
}
void launch_prefill_sums(hipStream_t s, const uint16_t* xb, const int32_t* rows_ptr, uint32_t rows_max, uint32_t K, float* sums, float* sums16, bool plain) {
    const uint32_t items = rows_max * (K / 64);
    hipLaunchKernelGGL(prefill_sums_kernel, dim3((items + 255) / 256), dim3(256), 0, s, xb, rows_ptr, rows_max, K, sums, sums16, plain);
}
void launch_prefill_tiles(hipStream_t s, const int32_t* offsets, uint32_t experts, uint32_t rows, int32_t* tile_expert, int32_t* tile_first,
                          int32_t* tile_rows, int32_t* tile_count) {
    hipLaunchKernelGGL(prefill_tiles_kernel, dim3(1), dim3(1024), 0, s, offsets, experts, rows, tile_expert, tile_first, tile_rows, tile_count);
}
// LDS beyond the kernel's fixed arrays: the scales and biases of 128 weight rows and the chain sums of 48 token rows for
// every step of K.
void launch_prefill_dispatch(hipStream_t s, const int32_t* ids, uint32_t tokens, uint32_t topk, uint32_t E, int32_t* offsets, int32_t* slots, int32_t* rows,
                             int32_t* status, int32_t* tile_expert, int32_t* tile_first, int32_t* tile_rows, int32_t* tile_count) {
    const uint32_t n = tokens * topk, stretch = ((n + kDispatchParts - 1) / kDispatchParts + 1023) / 1024 * 1024;
    const size_t lds = size_t(((kDispatchParts + 2) * E + 2 + 3) / 4 * 4 + stretch) * 4;
    if (lds > 48 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void*>(prefill_dispatch_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
    hipLaunchKernelGGL(prefill_dispatch_kernel, dim3((E + 3) / 4, kDispatchParts), dim3(256), lds, s, ids, n, topk, E, stretch, offsets, slots, rows, status,
                       tile_expert, tile_first, tile_rows, tile_count);
}
// whether launch_prefill_dispatch takes this batch (else: launch_dispatch and launch_prefill_tiles)
bool prefill_dispatch_fits(const int32_t* ids, uint32_t tokens, uint32_t topk, uint32_t E) {
    const uint64_t n = uint64_t(tokens) * topk;
    return reinterpret_cast<uintptr_t>(ids) % 16 == 0 && n > 1024 && n < (1u << 24) && E <= 1024 && n / kDispatchParts + 1024 <= 24 * 1024;
}
static uint32_t prefill_gemm_lds(uint32_t K) { const uint32_t groups = K / 64; return 2 * kTileCols * (groups + 2) * 2 + groups * kTileRowsMax * 4; }
void launch_prefill_gemm(hipStream_t s, const PrefillGemm& p, bool gated, uint32_t max_tiles) {
    const dim3 grid(gated ? p.N / 64 : p.N / 128, max_tiles);
    const uint32_t lds = prefill_gemm_lds(p.K);
    if (p.bits == 8) {
        if (gated) hipLaunchKernelGGL((prefill_gemm_kernel<true, 8>), grid, dim3(256), lds, s, p);
        else hipLaunchKernelGGL((prefill_gemm_kernel<false, 8>), grid, dim3(256), lds, s, p);
    } else {
        if (gated) hipLaunchKernelGGL((prefill_gemm_kernel<true, 4>), grid, dim3(256), lds, s, p);
        else hipLaunchKernelGGL((prefill_gemm_kernel<false, 4>), grid, dim3(256), lds, s, p);
    }
}
void launch_prefill_patch(hipStream_t s, const PrefillGemm& p, bool gated) {
    const bool wide = p.K % 512 == 0 && p.N % 8 == 0;     // the reference's lane-width rule (metal.mm:649-674)
    const uint32_t per = p.near_words >= kPatchWordsMax * 1024u ? kPatchWordsMax : 64u;   // words of the map per workgroup
    const dim3 grid((p.near_words + per - 1) / per);
    const bool tabled = wide && p.asum16 && p.bits == 4;  // the table holds the Q4 chain sums of 16-element blocks
#define ZC_PATCH(W, G, T, B) hipLaunchKernelGGL((prefill_patch_kernel<W, G, T, B>), grid, dim3(256), 0, s, p, per)
    if (p.bits == 8) {   // the Q8 lanes are half as wide (metal.mm:649-674)
        if (gated) { if (wide) ZC_PATCH(8, true, false, 8); else ZC_PATCH(4, true, false, 8); }
        else { if (wide) ZC_PATCH(8, false, false, 8); else ZC_PATCH(4, false, false, 8); }
    } else if (gated) { if (tabled) ZC_PATCH(16, true, true, 4); else if (wide) ZC_PATCH(16, true, false, 4); else ZC_PATCH(8, true, false, 4); }
    else { if (tabled) ZC_PATCH(16, false, true, 4); else if (wide) ZC_PATCH(16, false, false, 4); else ZC_PATCH(8, false, false, 4); }
#undef ZC_PATCH
}
// (hidden and intermediate sizes up to 4096: the product kernel keeps a whole K of scales, biases and chain sums in LDS)
bool prefill_shape(uint32_t hidden, uint32_t inter, uint32_t experts) {
    return hidden % 128 == 0 && inter % 128 == 0 && hidden <= 4096 && inter <= 4096 && experts <= 1024;
}

}  // namespace zc
