// The C ABI: context, memory, validation and the enqueue of each operator.
// Validation mirrors the reference operator layer (src/engine/metal.mm:261-266,
// 649-661, 775-827, 845-912) so the same misuse is refused with the same class
// of error before anything reaches the GPU.
#include "../../include/zc_hip.h"
#include "zc_kernels.hpp"
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

// Scratch of the allocation-free entry point (zc_hip_moe_forward_static): the workspace that zc_hip_moe_forward takes
// as an argument, as a static device array.  Every GPU the library runs on holds its own copy at its own address until
// the process ends; g_scratch[device] is that address, looked up once per device in zc_hip_create.  Host code never
// uses the array's name as an address: the name is only a handle for hipGetSymbolAddress.
constexpr uint64_t kStaticScratchBytes = 4ull << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch[kMaxDevices] = {};
std::mutex g_scratch_mutex;
thread_local std::string g_error;
zc_status fail(zc_status code, std::string text) { g_error = std::move(text); return code; }
}  // namespace
// Sets the calling thread's error text (shared with the other translation units of the library).
zc_status zc_fail(zc_status code, const std::string& text) { return fail(code, text); }
namespace {

#define ZC_HIP(call)                                                                         \
    do {                                                                                     \
        const hipError_t e_ = (call);                                                        \
        if (e_ != hipSuccess) return fail(ZC_RUNTIME_ERROR, std::string("HIP execution: ") + hipGetErrorString(e_) + " in " #call); \
    } while (0)
#define ZC_REQUIRE(cond, text) do { if (!(cond)) return fail(ZC_INVALID_ARGUMENT, text); } while (0)
#define ZC_LAUNCHED() ZC_HIP(hipGetLastError())

bool overlaps(const void* a, uint64_t an, const void* b, uint64_t bn) {
    const auto x = reinterpret_cast<uintptr_t>(a), y = reinterpret_cast<uintptr_t>(b);
    return a && b && x < y + bn && y < x + an;
}
uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }
}  // namespace

struct zc_hip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    uint64_t budget = 0, allocated = 0, peak = 0;
    std::unordered_map<void*, uint64_t> blocks;
    std::unordered_map<void*, uint64_t> host_blocks;   // pinned host allocations
    std::vector<hipEvent_t> tickets;   // live tickets: ticket t -> tickets[t - retired - 1]
    uint64_t retired = 0;              // tickets known complete and destroyed
    int32_t* moe_status = nullptr;     // device flag: an id outside [0,E) was seen
    hipEvent_t timer[2] = {nullptr, nullptr};
    // The prefill layer runs its shared expert beside the router, the selection and the dispatch sort, which are chains of
    // small kernels: a second stream of default priority, forked from and joined to `stream` by two events per call.
    hipStream_t beside = nullptr; hipEvent_t fork = nullptr, join = nullptr;
    uint32_t affine_policy = 1;        // 0 literal lane kernels, 1 exact-integer matrix-core kernels where possible
    void* static_scratch = nullptr;    // this device's copy of the static scratch array
    std::mutex mutex;
    // Profiling (KernelConfig::profile + Metal::label, metal.mm:267-270): while on, every operator call made through this
    // context records one row: the label current at the call, the operator's name and a pair of events around its launches.
    struct Row { std::string stage; int32_t layer; uint32_t tokens, offset; const char* op; hipEvent_t begin, end; };
    bool profile = false; int profile_depth = 0;
    std::string stage = "unlabelled"; int32_t label_layer = -1; uint32_t label_tokens = 0, label_offset = 0;
    std::vector<Row> rows; uint64_t rows_dropped = 0;
};

namespace {
constexpr size_t kMaxProfileRows = 16384;
// One row per outermost operator call: operators that call other operators (the layer-by-layer stack, the static-scratch
// entry point) count once, under their own name.
struct Timed {
    zc_hip_ctx* ctx; hipEvent_t end = nullptr;
    Timed(zc_hip_ctx* c, const char* op) : ctx(c) {
        if (!ctx || !ctx->profile || ctx->profile_depth++ > 0) return;
        if (ctx->rows.size() >= kMaxProfileRows) { ++ctx->rows_dropped; return; }
        hipEvent_t begin = nullptr;
        if (hipEventCreate(&begin) != hipSuccess || hipEventCreate(&end) != hipSuccess || hipEventRecord(begin, ctx->stream) != hipSuccess) {
            (void)hipGetLastError(); if (begin) (void)hipEventDestroy(begin); if (end) (void)hipEventDestroy(end); end = nullptr; ++ctx->rows_dropped; return;
        }
        ctx->rows.push_back({ctx->stage, ctx->label_layer, ctx->label_tokens, ctx->label_offset, op, begin, end});
    }
    ~Timed() {
        if (!ctx || !ctx->profile) return;
        --ctx->profile_depth;
        if (end) (void)hipEventRecord(end, ctx->stream);
    }
};
// Keeps a recording off for one call: the operators inside see a call already in progress and record nothing, so the
// call creates no event and touches no host container.
struct Untimed {
    zc_hip_ctx* ctx;
    explicit Untimed(zc_hip_ctx* c) : ctx(c && c->profile ? c : nullptr) { if (ctx) ++ctx->profile_depth; }
    ~Untimed() { if (ctx) --ctx->profile_depth; }
};
void json_text(std::string& out, const std::string& text) {
    out += '"';
    for (const char c : text) {
        if (c == '"' || c == '\\') { out += '\\'; out += c; }
        else if (static_cast<unsigned char>(c) < 0x20) { char b[8]; std::snprintf(b, sizeof b, "\\u%04x", c); out += b; }
        else out += c;
    }
    out += '"';
}
}  // namespace

extern "C" {

const char* zc_hip_last_error(void) { return g_error.c_str(); }
const char* zc_hip_version(void) { return "zerocool-moe-mi355x 0.1 (gfx950)"; }

zc_status zc_hip_create(int device, uint64_t budget_bytes, zc_hip_ctx** out) {
    ZC_REQUIRE(out, "null context output");
    int count = 0;
    ZC_HIP(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return fail(ZC_RUNTIME_ERROR, "no such HIP device");
    ZC_HIP(hipSetDevice(device));
    void* device_scratch = nullptr;
    {   // once per device, with that device current: where this GPU keeps its copy of the static scratch array
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (device < kMaxDevices && g_scratch[device]) device_scratch = g_scratch[device];
        else {
            const hipError_t e = hipGetSymbolAddress(&device_scratch, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !device_scratch) return fail(ZC_RUNTIME_ERROR, std::string("HIP execution: cannot locate the static scratch array: ") + hipGetErrorString(e));
            if (device < kMaxDevices) g_scratch[device] = device_scratch;
        }
    }
    auto* ctx = new zc_hip_ctx;
    ctx->device = device; ctx->budget = budget_bytes; ctx->static_scratch = device_scratch;
    if (hipStreamCreate(&ctx->stream) != hipSuccess) { delete ctx; return fail(ZC_RUNTIME_ERROR, "HIP execution: cannot create stream"); }
    if (hipMalloc(&ctx->moe_status, 256) != hipSuccess || hipMemsetAsync(ctx->moe_status, 0, 256, ctx->stream) != hipSuccess) {
        hipStreamDestroy(ctx->stream); delete ctx; return fail(ZC_RUNTIME_ERROR, "HIP execution: cannot allocate status word");
    }
    *out = ctx;
    return ZC_OK;
}
zc_status zc_hip_destroy(zc_hip_ctx* ctx) {
    if (!ctx) return ZC_OK;
    hipSetDevice(ctx->device);
    hipStreamSynchronize(ctx->stream);
    for (auto e : ctx->tickets) hipEventDestroy(e);
    for (auto e : ctx->timer) if (e) hipEventDestroy(e);
    for (auto& r : ctx->rows) { hipEventDestroy(r.begin); hipEventDestroy(r.end); }
    for (auto& b : ctx->blocks) hipFree(b.first);
    for (auto& b : ctx->host_blocks) hipHostFree(b.first);
    hipFree(ctx->moe_status);
    if (ctx->beside) { hipStreamSynchronize(ctx->beside); hipStreamDestroy(ctx->beside); }
    if (ctx->fork) hipEventDestroy(ctx->fork);
    if (ctx->join) hipEventDestroy(ctx->join);
    hipStreamDestroy(ctx->stream);
    delete ctx;
    return ZC_OK;
}
zc_status zc_hip_alloc(zc_hip_ctx* ctx, uint64_t bytes, void** out) {
    ZC_REQUIRE(ctx && out, "null argument");
    std::lock_guard<std::mutex> lock(ctx->mutex);
    if (ctx->budget && (bytes > ctx->budget || ctx->allocated > ctx->budget - bytes))
        return fail(ZC_BUDGET_EXCEEDED, "engine memory budget exceeded");
    void* p = nullptr;
    ZC_HIP(hipSetDevice(ctx->device));
    const hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
    if (e != hipSuccess) { (void)hipGetLastError(); return fail(ZC_BUDGET_EXCEEDED, std::string("device allocation failed: ") + hipGetErrorString(e)); }
    ctx->blocks[p] = bytes; ctx->allocated += bytes;
    if (ctx->allocated > ctx->peak) ctx->peak = ctx->allocated;
    *out = p;
    return ZC_OK;
}
zc_status zc_hip_alloc_host(zc_hip_ctx* ctx, uint64_t bytes, void** out) {
    ZC_REQUIRE(ctx && out, "null argument");
    std::lock_guard<std::mutex> lock(ctx->mutex);
    if (ctx->budget && (bytes > ctx->budget || ctx->allocated > ctx->budget - bytes))
        return fail(ZC_BUDGET_EXCEEDED, "engine memory budget exceeded");
    void* p = nullptr;
    ZC_HIP(hipSetDevice(ctx->device));
    const hipError_t e = hipHostMalloc(&p, bytes ? bytes : 1, hipHostMallocMapped | hipHostMallocCoherent);
    if (e != hipSuccess) { (void)hipGetLastError(); return fail(ZC_BUDGET_EXCEEDED, std::string("host allocation failed: ") + hipGetErrorString(e)); }
    ctx->host_blocks[p] = bytes; ctx->allocated += bytes;
    if (ctx->allocated > ctx->peak) ctx->peak = ctx->allocated;
    *out = p;
    return ZC_OK;
}
zc_status zc_hip_free(zc_hip_ctx* ctx, void* ptr) {
    ZC_REQUIRE(ctx, "null context");
    if (!ptr) return ZC_OK;
    std::lock_guard<std::mutex> lock(ctx->mutex);
    if (auto h = ctx->host_blocks.find(ptr); h != ctx->host_blocks.end()) {
        ZC_HIP(hipStreamSynchronize(ctx->stream));
        ZC_HIP(hipHostFree(ptr));
        ctx->allocated -= h->second; ctx->host_blocks.erase(h);
        return ZC_OK;
    }
    auto it = ctx->blocks.find(ptr);
    if (it == ctx->blocks.end()) return fail(ZC_LOGIC_ERROR, "free of a pointer this context did not allocate");
    ZC_HIP(hipStreamSynchronize(ctx->stream));   // no GPU user may outlive its buffer
    ZC_HIP(hipFree(ptr));
    ctx->allocated -= it->second; ctx->blocks.erase(it);
    return ZC_OK;
}
zc_status zc_hip_memset(zc_hip_ctx* ctx, void* dst, int byte, uint64_t bytes) {
    ZC_REQUIRE(ctx && (dst || !bytes), "null argument");
    if (bytes) ZC_HIP(hipMemsetAsync(dst, byte, bytes, ctx->stream));
    return ZC_OK;
}
zc_status zc_hip_upload(zc_hip_ctx* ctx, void* dst, const void* host_src, uint64_t bytes) {
    ZC_REQUIRE(ctx && ((dst && host_src) || !bytes), "null argument");
    if (bytes) { ZC_HIP(hipMemcpyAsync(dst, host_src, bytes, hipMemcpyHostToDevice, ctx->stream)); ZC_HIP(hipStreamSynchronize(ctx->stream)); }
    return ZC_OK;
}
zc_status zc_hip_download(zc_hip_ctx* ctx, void* host_dst, const void* src, uint64_t bytes) {
    ZC_REQUIRE(ctx && ((host_dst && src) || !bytes), "null argument");
    if (bytes) { ZC_HIP(hipMemcpyAsync(host_dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream)); ZC_HIP(hipStreamSynchronize(ctx->stream)); }
    return ZC_OK;
}
zc_status zc_hip_copy(zc_hip_ctx* ctx, void* dst, const void* src, uint64_t bytes) {
    ZC_REQUIRE(ctx && ((dst && src) || !bytes), "null argument");
    if (bytes) ZC_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return ZC_OK;
}
zc_status zc_hip_configure(zc_hip_ctx* ctx, uint32_t affine_policy) {
    ZC_REQUIRE(ctx, "null context");
    ZC_REQUIRE(affine_policy <= 1, "unknown kernel policy");
    ctx->affine_policy = affine_policy;
    return ZC_OK;
}
zc_status zc_hip_timer_start(zc_hip_ctx* ctx) {
    ZC_REQUIRE(ctx, "null context");
    for (auto& e : ctx->timer) if (!e) ZC_HIP(hipEventCreate(&e));
    ZC_HIP(hipEventRecord(ctx->timer[0], ctx->stream));
    return ZC_OK;
}
zc_status zc_hip_timer_stop(zc_hip_ctx* ctx, float* milliseconds) {
    ZC_REQUIRE(ctx && milliseconds && ctx->timer[0], "timer was not started");
    ZC_HIP(hipEventRecord(ctx->timer[1], ctx->stream));
    ZC_HIP(hipEventSynchronize(ctx->timer[1]));
    ZC_HIP(hipEventElapsedTime(milliseconds, ctx->timer[0], ctx->timer[1]));
    return ZC_OK;
}
zc_status zc_hip_label(zc_hip_ctx* ctx, const char* stage, int32_t layer, uint32_t tokens, uint32_t offset) {
    ZC_REQUIRE(ctx && stage, "null argument");
    if (ctx->profile) { ctx->stage = stage; ctx->label_layer = layer; ctx->label_tokens = tokens; ctx->label_offset = offset; }   // metal.mm:267-270: a no-op unless profiling
    return ZC_OK;
}
zc_status zc_hip_profile(zc_hip_ctx* ctx, int on) {
    ZC_REQUIRE(ctx, "null argument");
    if (on && !ctx->profile) {   // a new recording: earlier rows go
        ZC_HIP(hipStreamSynchronize(ctx->stream));
        for (auto& r : ctx->rows) { (void)hipEventDestroy(r.begin); (void)hipEventDestroy(r.end); }
        ctx->rows.clear(); ctx->rows_dropped = 0; ctx->profile_depth = 0;
        ctx->stage = "unlabelled"; ctx->label_layer = -1; ctx->label_tokens = ctx->label_offset = 0;
    }
    ctx->profile = on != 0;
    return ZC_OK;
}
zc_status zc_hip_stats(zc_hip_ctx* ctx, const zc_hip_store* store, char* json, uint64_t capacity, uint64_t* needed) {
    ZC_REQUIRE(ctx && (json || !capacity), "null argument");
    ZC_HIP(hipStreamSynchronize(ctx->stream));   // every recorded event has happened
    std::string out = "{\"library\": ";
    json_text(out, zc_hip_version());
    out += ", \"device\": " + std::to_string(ctx->device);
    out += ", \"memory\": {\"allocated_bytes\": " + std::to_string(ctx->allocated) + ", \"peak_bytes\": " + std::to_string(ctx->peak) +
           ", \"budget_bytes\": " + std::to_string(ctx->budget) + "}";
    // rows by (stage, operator) in order of first appearance, then the rows themselves
    struct Sum { std::string stage; const char* op; uint64_t calls; double us; };
    std::vector<Sum> sums; std::string rows;
    char number[64];
    for (const auto& r : ctx->rows) {
        float ms = 0;
        if (hipEventElapsedTime(&ms, r.begin, r.end) != hipSuccess) { (void)hipGetLastError(); continue; }
        size_t at = 0;
        while (at < sums.size() && !(sums[at].stage == r.stage && std::strcmp(sums[at].op, r.op) == 0)) ++at;
        if (at == sums.size()) sums.push_back({r.stage, r.op, 0, 0.0});
        ++sums[at].calls; sums[at].us += double(ms) * 1e3;
        rows += rows.empty() ? "" : ", ";
        rows += "{\"stage\": "; json_text(rows, r.stage);
        std::snprintf(number, sizeof number, "%.3f", double(ms) * 1e3);
        rows += ", \"layer\": " + std::to_string(r.layer) + ", \"tokens\": " + std::to_string(r.tokens) + ", \"offset\": " + std::to_string(r.offset) +
                ", \"operator\": \"" + r.op + "\", \"gpu_us\": " + number + "}";
    }
    out += ", \"profile\": {\"recording\": " + std::string(ctx->profile ? "true" : "false") + ", \"rows_recorded\": " + std::to_string(ctx->rows.size()) +
           ", \"rows_dropped\": " + std::to_string(ctx->rows_dropped) + ", \"stages\": [";
    for (size_t i = 0; i < sums.size(); ++i) {
        out += i ? ", " : "";
        out += "{\"stage\": "; json_text(out, sums[i].stage);
        std::snprintf(number, sizeof number, "%.3f", sums[i].us);
        out += ", \"operator\": \"" + std::string(sums[i].op) + "\", \"calls\": " + std::to_string(sums[i].calls) + ", \"gpu_us\": " + number + "}";
    }
    out += "], \"rows\": [" + rows + "]}";
    if (store) {   // Model::stats' "expert_cache" (model.cpp:706-732)
        zc_store_stats c{}; zc_store_table_stats t{};
        if (const zc_status s = zc_hip_store_stats(store, &c)) return s;
        if (const zc_status s = zc_hip_store_table_stats(store, &t)) return s;
        out += ", \"expert_cache\": {\"capacity\": " + std::to_string(zc_hip_store_capacity(store)) + ", \"occupancy\": " + std::to_string(zc_hip_store_occupancy(store)) +
               ", \"hits\": " + std::to_string(c.hits) + ", \"misses\": " + std::to_string(c.misses) + ", \"evictions\": " + std::to_string(c.evictions) +
               ", \"application_read_bytes\": " + std::to_string(c.bytes) + ", \"ready_hits\": " + std::to_string(c.ready_hits) +
               ", \"loading_joins\": " + std::to_string(c.loading_joins) + ", \"prefetches\": " + std::to_string(c.prefetches) +
               ", \"prefetch_claims\": " + std::to_string(c.prefetch_claims) + ", \"prefetch_unclaimed\": " + std::to_string(c.prefetch_unclaimed) +
               ", \"record_table\": {\"reads\": " + std::to_string(t.reads) + ", \"slot_reads\": " + std::to_string(t.slot_reads) +
               ", \"home_reads\": " + std::to_string(t.home_reads) + ", \"home_read_bytes\": " + std::to_string(t.home_read_bytes) +
               ", \"switched\": " + std::to_string(t.switched) + ", \"joined\": " + std::to_string(t.joined) + ", \"not_admitted\": " + std::to_string(t.not_admitted) + "}}";
    }
    out += "}";
    if (needed) *needed = out.size() + 1;
    if (capacity) {
        const size_t n = std::min<size_t>(out.size(), size_t(capacity) - 1);
        std::memcpy(json, out.data(), n); json[n] = 0;
        if (n < out.size()) return fail(ZC_OUT_OF_RANGE, "statistics buffer too small");
    }
    return ZC_OK;
}
uint64_t zc_hip_allocated(const zc_hip_ctx* ctx) { return ctx ? ctx->allocated : 0; }
uint64_t zc_hip_peak(const zc_hip_ctx* ctx) { return ctx ? ctx->peak : 0; }
void* zc_hip_stream(zc_hip_ctx* ctx) { return ctx ? ctx->stream : nullptr; }

zc_status zc_hip_submit(zc_hip_ctx* ctx, uint64_t* ticket) {
    ZC_REQUIRE(ctx && ticket, "null argument");
    hipEvent_t e;
    ZC_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    ZC_HIP(hipEventRecord(e, ctx->stream));
    std::lock_guard<std::mutex> lock(ctx->mutex);
    ctx->tickets.push_back(e);
    *ticket = ctx->retired + ctx->tickets.size();
    return ZC_OK;
}
zc_status zc_hip_wait(zc_hip_ctx* ctx, uint64_t ticket) {
    ZC_REQUIRE(ctx, "null context");
    hipEvent_t e;
    {
        std::lock_guard<std::mutex> lock(ctx->mutex);
        if (!ticket || ticket > ctx->retired + ctx->tickets.size()) return fail(ZC_LOGIC_ERROR, "wait on a ticket that was never submitted");
        if (ticket <= ctx->retired) return ZC_OK;
        e = ctx->tickets[ticket - ctx->retired - 1];
    }
    ZC_HIP(hipEventSynchronize(e));
    return ZC_OK;
}
zc_status zc_hip_finish(zc_hip_ctx* ctx) {
    ZC_REQUIRE(ctx, "null context");
    ZC_HIP(hipStreamSynchronize(ctx->stream));
    std::lock_guard<std::mutex> lock(ctx->mutex);
    for (auto e : ctx->tickets) hipEventDestroy(e);
    ctx->retired += ctx->tickets.size();
    ctx->tickets.clear();
    return ZC_OK;
}

uint64_t zc_hip_projection_bytes(uint32_t K, uint32_t N, uint32_t group, uint32_t bits) {
    return uint64_t(K) * N * bits / 8 + 2ull * 2 * (K / (group ? group : 64)) * N;
}
static void projection_shape(const zc_moe_config* c, int shared, int p, uint32_t* K, uint32_t* N, uint32_t* bits) {
    *K = p == 2 ? c->inter : c->hidden;
    *N = p == 2 ? c->hidden : c->inter;
    *bits = shared ? (p == 2 ? c->shared_bits_down : c->shared_bits_gate_up) : (p == 2 ? c->bits_down : c->bits_gate_up);
}
uint64_t zc_hip_record_bytes(const zc_moe_config* c, int shared) {
    uint64_t total = 0;
    for (int p = 0; p < 3; ++p) { uint32_t K, N, b; projection_shape(c, shared, p, &K, &N, &b); total += zc_hip_projection_bytes(K, N, c->group, b); }
    return total;
}
static zc_status validate_config(const zc_moe_config* c) {
    ZC_REQUIRE(c, "null configuration");
    ZC_REQUIRE(c->hidden && c->inter && c->experts && c->topk, "empty MoE geometry");
    ZC_REQUIRE(c->group == 32 || c->group == 64, "unsupported affine matrix geometry");
    ZC_REQUIRE(c->hidden % c->group == 0 && c->inter % c->group == 0, "unsupported affine matrix geometry");
    ZC_REQUIRE(c->hidden % 16 == 0, "router needs hidden divisible by 16");
    ZC_REQUIRE(c->experts <= 1024 && c->topk <= 128 && c->topk <= c->experts, "route selection supports at most 1024 experts and top-128");
    for (uint32_t b : {c->bits_gate_up, c->bits_down, c->shared_bits_gate_up, c->shared_bits_down})
        ZC_REQUIRE(b == 4 || b == 8, "unsupported affine matrix geometry");
    return ZC_OK;
}
zc_status zc_hip_expert_linear(const zc_moe_config* c, int shared, const void* record, int projection, zc_linear* out) {
    if (const zc_status s = validate_config(c)) return s;
    ZC_REQUIRE(record && out && projection >= 0 && projection <= 2, "invalid expert projection");
    uint64_t offset = 0; uint32_t K, N, bits;
    for (int p = 0; p < projection; ++p) { projection_shape(c, shared, p, &K, &N, &bits); offset += zc_hip_projection_bytes(K, N, c->group, bits); }
    projection_shape(c, shared, projection, &K, &N, &bits);
    const uint64_t wbytes = uint64_t(K) * N * bits / 8, meta = 2ull * (K / c->group) * N;
    const auto* r = static_cast<const uint8_t*>(record);
    *out = zc_linear{r + offset, r + offset + wbytes, r + offset + wbytes + meta, K, N, c->group, 0, 1, bits};
    return ZC_OK;
}

// metal.mm:649-661 without the binding-coverage test (sizes are the shim's business).
static zc_status validate_affine(const zc_linear* l) {
    ZC_REQUIRE(l->input && l->output && (l->bits == 4 || l->bits == 8) && (l->group == 32 || l->group == 64) &&
               l->input % l->group == 0, "unsupported affine matrix geometry");
    ZC_REQUIRE(l->weight && l->scales && l->biases, "affine tensor binding is truncated");
    ZC_REQUIRE(reinterpret_cast<uintptr_t>(l->weight) % 4 == 0 && reinterpret_cast<uintptr_t>(l->scales) % 2 == 0 &&
               reinterpret_cast<uintptr_t>(l->biases) % 2 == 0, "affine tensor binding is misaligned");
    return ZC_OK;
}
static uint64_t weight_bytes(const zc_linear* l) {
    return l->quantized ? uint64_t(l->input) * l->output * l->bits / 8 : uint64_t(l->input) * l->output * (l->dtype == 1 ? 4 : 2);
}

zc_status zc_hip_linear_into(zc_hip_ctx* ctx, const zc_linear* l, const float* x, uint32_t tokens, float* out, int float_output) {
    Timed timed(ctx, "linear");
    ZC_REQUIRE(ctx && l, "null argument");
    ZC_REQUIRE(tokens && l->input && l->output && x, "linear input shape");
    ZC_REQUIRE(l->weight, "missing linear weights");
    if (l->quantized) if (const zc_status s = validate_affine(l)) return s;
    const uint64_t obytes = uint64_t(tokens) * l->output * 4, xbytes = uint64_t(tokens) * l->input * 4;
    ZC_REQUIRE(out && reinterpret_cast<uintptr_t>(out) % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
               !overlaps(out, obytes, x, xbytes) && !overlaps(out, obytes, l->weight, weight_bytes(l)),
               "invalid or overlapping linear output");
    if (l->quantized) {
        zc::AffineDesc a; a.gate = *l; a.x = x; a.out = out; a.tokens = tokens; a.float_output = float_output ? 1 : 0;
        if (ctx->affine_policy == 1 && zc::xint_supported(*l)) zc::launch_affine_xint(ctx->stream, a);
        else zc::launch_affine(ctx->stream, a);
    } else {
        ZC_REQUIRE(l->dtype <= 1, "unsupported plain matrix dtype");
        zc::launch_plain(ctx->stream, l->weight, l->dtype, x, l->input, l->output, tokens, out, float_output != 0);
    }
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_router_logits(zc_hip_ctx* ctx, const void* w, const float* x, uint32_t tokens, uint32_t hidden,
                               uint32_t experts, const float* offsets, float* logits) {
    Timed timed(ctx, "router_logits");
    ZC_REQUIRE(ctx && w && x && logits && tokens && experts, "linear input shape");
    ZC_REQUIRE(hidden && hidden % 16 == 0, "router needs hidden divisible by 16");
    ZC_REQUIRE(reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0, "router operands must be 16-byte aligned");
    ZC_REQUIRE(!overlaps(logits, uint64_t(tokens) * experts * 4, x, uint64_t(tokens) * hidden * 4) &&
               !overlaps(logits, uint64_t(tokens) * experts * 4, w, uint64_t(experts) * hidden * 2), "invalid or overlapping linear output");
    zc::launch_router(ctx->stream, w, x, tokens, hidden, experts, offsets, logits);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_gated_linear(zc_hip_ctx* ctx, const zc_linear* gate, const zc_linear* up, const float* x, uint32_t x_rows,
                              uint32_t tokens, const int32_t* rows, float* out) {
    Timed timed(ctx, "gated_linear");
    ZC_REQUIRE(ctx && gate && up, "null argument");
    ZC_REQUIRE(gate->quantized && up->quantized && gate->input == up->input && gate->output == up->output &&
               gate->group == up->group && gate->bits == up->bits, "fused gate/up requires matching affine matrices");
    if (const zc_status s = validate_affine(gate)) return s;
    if (const zc_status s = validate_affine(up)) return s;
    ZC_REQUIRE(tokens && x && x_rows && (rows || x_rows >= tokens), "fused gate/up input shape");
    ZC_REQUIRE(out && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
               !overlaps(out, uint64_t(tokens) * gate->output * 4, x, uint64_t(x_rows) * gate->input * 4), "invalid or overlapping linear output");
    if (rows) {   // metal.mm:852-856: every gathered row must lie inside x
        std::vector<int32_t> host(tokens);
        ZC_HIP(hipMemcpyAsync(host.data(), rows, uint64_t(tokens) * 4, hipMemcpyDeviceToHost, ctx->stream));
        ZC_HIP(hipStreamSynchronize(ctx->stream));
        for (int32_t r : host) ZC_REQUIRE(r >= 0 && uint32_t(r) < x_rows, "fused gate/up row outside input");
    }
    zc::AffineDesc a; a.gate = *gate; a.up = *up; a.gated = true; a.x = x; a.in_rows = rows; a.out = out; a.tokens = tokens;
    if (ctx->affine_policy == 1 && zc::xint_supported(*gate) && zc::xint_supported(*up)) zc::launch_affine_xint(ctx->stream, a);
    else zc::launch_affine(ctx->stream, a);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_route(zc_hip_ctx* ctx, const float* logits, uint32_t tokens, uint32_t experts, uint32_t topk, int32_t* ids, float* weights) {
    Timed timed(ctx, "route");
    ZC_REQUIRE(ctx && tokens && tokens <= 8192 && logits && ids && weights, "invalid route selection buffers");
    ZC_REQUIRE(experts && experts <= 1024 && topk && topk <= 128 && topk <= experts, "route selection supports at most 1024 experts and top-128");
    zc::launch_route(ctx->stream, logits, tokens, experts, topk, ids, weights);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_build_dispatch(zc_hip_ctx* ctx, const int32_t* ids, uint32_t tokens, uint32_t topk, uint32_t experts,
                                int32_t* offsets, int32_t* slots, int32_t* selected, int32_t* count, int32_t* status) {
    Timed timed(ctx, "build_dispatch");
    ZC_REQUIRE(ctx && ids && offsets && slots && selected && count && status && tokens && topk && experts, "invalid dispatch buffers");
    ZC_REQUIRE(experts <= 8192, "dispatch supports at most 8192 experts");
    zc::launch_dispatch(ctx->stream, ids, tokens, topk, experts, offsets, slots, nullptr, selected, count, status);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_scatter_experts(zc_hip_ctx* ctx, const float* x, const int32_t* positions, uint32_t n, uint32_t hidden, float* out) {
    Timed timed(ctx, "scatter_experts");
    ZC_REQUIRE(ctx && x && positions && out && hidden, "invalid scatter buffers");
    if (!n) return ZC_OK;
    zc::launch_scatter(ctx->stream, x, positions, n, hidden, out);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_moe_sum(zc_hip_ctx* ctx, const float* experts, const float* weights, const float* shared, const float* gate,
                         uint32_t tokens, uint32_t hidden, uint32_t topk, float* out) {
    Timed timed(ctx, "moe_sum");
    ZC_REQUIRE(ctx && experts && weights && shared && gate && out && tokens && hidden && topk, "invalid expert reduction buffers");
    zc::launch_moe_sum(ctx->stream, experts, weights, shared, gate, tokens, hidden, topk, out);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_unary(zc_hip_ctx* ctx, const float* x, uint64_t n, uint32_t op, float* y) {
    Timed timed(ctx, "unary");
    ZC_REQUIRE(ctx && x && y && n && op <= 4, "invalid unary operator or buffers");
    zc::launch_unary(ctx->stream, x, n, op, y);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_binary(zc_hip_ctx* ctx, const float* x, const float* y, uint64_t n, uint32_t op, float* out) {
    Timed timed(ctx, "binary");
    ZC_REQUIRE(ctx && x && y && out && n, "binary shape mismatch");
    zc::launch_binary(ctx->stream, x, y, n, op, out);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_hc_mix(zc_hip_ctx* ctx, const float* x, const float* w, uint32_t tokens, uint32_t hidden, float* out) {
    Timed timed(ctx, "hc_mix");
    ZC_REQUIRE(ctx && x && w && out && tokens && hidden && x != out && w != out, "invalid stream mix buffers");
    zc::launch_hc_mix(ctx->stream, x, w, tokens, hidden, out);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_hc_add(zc_hip_ctx* ctx, const float* hyper, const float* x, const float* inject, uint32_t tokens, uint32_t hidden, float* out) {
    Timed timed(ctx, "hc_add");
    ZC_REQUIRE(ctx && hyper && x && inject && out && tokens && hidden && x != out && inject != out, "invalid residual injection buffers");
    zc::launch_hc_add(ctx->stream, hyper, x, inject, tokens, hidden, out);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_norm(zc_hip_ctx* ctx, const float* x, const void* w, uint32_t dtype, uint32_t group, uint32_t width, uint32_t tokens, float* out) {
    Timed timed(ctx, "norm");
    ZC_REQUIRE(ctx && x && w && out && tokens && group && width && width % group == 0 && group <= 4096 && dtype <= 1, "normalization shape");
    zc::launch_norm(ctx->stream, x, w, dtype, group, width, tokens, out);
    ZC_LAUNCHED();
    return ZC_OK;
}
zc_status zc_hip_grouped_experts(zc_hip_ctx* ctx, const zc_moe_config* cfg, const void* const* records,
                                 const uint32_t* positions, uint32_t n, const float* x, float* out, float* scratch) {
    Timed timed(ctx, "grouped_experts");
    if (const zc_status s = validate_config(cfg)) return s;
    ZC_REQUIRE(ctx && n && n <= 8 && records && positions && x && out && scratch && x != out && x != scratch && out != scratch,
               "invalid grouped expert geometry");
    uint32_t seen = 0;
    for (uint32_t i = 0; i < n; ++i) {
        ZC_REQUIRE(records[i] && positions[i] < cfg->topk && !(positions[i] < 32 && (seen & (1u << positions[i]))) &&
                   records[i] != out && records[i] != scratch, "invalid grouped expert record or destination");
        for (uint32_t k = 0; k < i; ++k) ZC_REQUIRE(positions[k] != positions[i], "invalid grouped expert record or destination");
        if (positions[i] < 32) seen |= 1u << positions[i];
    }
    for (uint32_t i = 0; i < n; ++i) {
        zc_linear g, u, d;
        zc_hip_expert_linear(cfg, 0, records[i], 0, &g); zc_hip_expert_linear(cfg, 0, records[i], 1, &u); zc_hip_expert_linear(cfg, 0, records[i], 2, &d);
        zc::AffineDesc a; a.gate = g; a.up = u; a.gated = true; a.x = x; a.out = scratch + uint64_t(i) * cfg->inter; a.tokens = 1;
        zc::launch_affine(ctx->stream, a);
        zc::AffineDesc b; b.gate = d; b.x = scratch + uint64_t(i) * cfg->inter; b.out = out + uint64_t(positions[i]) * cfg->hidden; b.tokens = 1;
        zc::launch_affine(ctx->stream, b);
    }
    ZC_LAUNCHED();
    return ZC_OK;
}

// Workspace of one zc_hip_moe_forward call.
namespace {
struct Workspace {
    float* logits; int32_t* ids; float* weights;
    int32_t *offsets, *slots, *rows, *selected, *count;
    float *act, *shared_act, *shared, *gate, *expert_out;
    uint64_t bytes;
};
Workspace carve(const zc_moe_config* c, uint32_t T, void* base) {
    Workspace w{};
    uint64_t at = 0;
    auto take = [&](uint64_t bytes) { void* p = base ? static_cast<uint8_t*>(base) + at : nullptr; at += align_up(bytes, 256); return p; };
    const uint64_t n = uint64_t(T) * c->topk;
    w.logits = (float*)take(uint64_t(T) * c->experts * 4);
    w.ids = (int32_t*)take(n * 4); w.weights = (float*)take(n * 4);
    w.offsets = (int32_t*)take(uint64_t(c->experts + 1) * 4); w.slots = (int32_t*)take(n * 4); w.rows = (int32_t*)take(n * 4);
    w.selected = (int32_t*)take(uint64_t(c->experts) * 4); w.count = (int32_t*)take(4);
    w.act = (float*)take(n * c->inter * 4); w.shared_act = (float*)take(uint64_t(T) * c->inter * 4);
    w.shared = (float*)take(uint64_t(T) * c->hidden * 4); w.gate = (float*)take(uint64_t(T) * 4);
    w.expert_out = (float*)take(n * c->hidden * 4);
    w.bytes = at;
    return w;
}
}  // namespace
uint64_t zc_hip_moe_workspace_bytes(const zc_moe_config* cfg, uint32_t tokens) {
    if (validate_config(cfg) != ZC_OK || !tokens) return 0;
    return carve(cfg, tokens, nullptr).bytes;
}
uint64_t zc_hip_moe_static_scratch_bytes(void) { return kStaticScratchBytes; }
// zc_hip_moe_forward with its workspace in the static scratch array of the context's device.  Nothing on this path
// allocates or frees: no hipMalloc / hipFree / hipHostMalloc, no stream or event creation, no host containers --
// also while a recording is on (zc_hip_profile): this call records no row, and neither do the operators inside it.
zc_status zc_hip_moe_forward_static(zc_hip_ctx* ctx, const zc_moe_config* c, const zc_moe_layer* l, const float* x, uint32_t T,
                                    float* out, const zc_moe_trace* trace) {
    Untimed untimed(ctx);
    if (const zc_status s = validate_config(c)) return s;
    ZC_REQUIRE(ctx && T, "invalid MoE layer buffers");
    ZC_REQUIRE(ctx->static_scratch, "the static scratch array was not located for this device");
    const uint64_t need = carve(c, T, nullptr).bytes;
    if (need > kStaticScratchBytes) {
        char text[200];
        snprintf(text, sizeof text, "zc_hip_moe_forward_static: %u tokens of this shape need %llu bytes of scratch, the static array holds %llu; use zc_hip_moe_forward with a workspace",
                 T, (unsigned long long)need, (unsigned long long)kStaticScratchBytes);
        return fail(ZC_INVALID_ARGUMENT, text);
    }
    return zc_hip_moe_forward(ctx, c, l, x, T, out, ctx->static_scratch, trace);
}
zc_status zc_hip_moe_forward(zc_hip_ctx* ctx, const zc_moe_config* c, const zc_moe_layer* l, const float* x, uint32_t T,
                             float* out, void* workspace, const zc_moe_trace* trace) {
    Timed timed(ctx, "moe_forward");
    if (const zc_status s = validate_config(c)) return s;
    ZC_REQUIRE(ctx && l && x && out && workspace && T && T <= 8192, "invalid MoE layer buffers");
    ZC_REQUIRE(l->router && l->shared_gate && l->shared_record && l->expert_records, "missing MoE layer weights");
    ZC_REQUIRE(l->record_stride >= zc_hip_record_bytes(c, 0) && l->record_stride % 4 == 0, "expert record stride is too small");
    ZC_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(workspace) % 256 == 0 &&
               reinterpret_cast<uintptr_t>(l->router) % 16 == 0 && reinterpret_cast<uintptr_t>(l->expert_records) % 4 == 0 &&
               reinterpret_cast<uintptr_t>(l->shared_record) % 4 == 0, "MoE layer operands are misaligned");
    ZC_REQUIRE(x != out, "invalid or overlapping linear output");
    const Workspace w = carve(c, T, workspace);
    hipStream_t s = ctx->stream;
    const uint32_t H = c->hidden, I = c->inter, E = c->experts, k = c->topk;
    // 1-2. router logits, top-k + softmax (model.cpp:434-436)
    zc::launch_router(s, l->router, x, T, H, E, l->router_offsets, w.logits);
    zc::launch_route(s, w.logits, T, E, k, w.ids, w.weights);
    // 4. positions / selected, on the device (model.cpp:449-479)
    zc::launch_dispatch(s, w.ids, T, k, E, w.offsets, w.slots, w.rows, w.selected, w.count, ctx->moe_status);
    // 5. shared expert and its gate (model.cpp:482-485)
    zc_linear g, u, d;
    zc_hip_expert_linear(c, 1, l->shared_record, 0, &g); zc_hip_expert_linear(c, 1, l->shared_record, 1, &u); zc_hip_expert_linear(c, 1, l->shared_record, 2, &d);
    { zc::AffineDesc a; a.gate = g; a.up = u; a.gated = true; a.x = x; a.out = w.shared_act; a.tokens = T; zc::launch_affine(s, a); }
    { zc::AffineDesc a; a.gate = d; a.x = w.shared_act; a.out = w.shared; a.tokens = T; zc::launch_affine(s, a); }
    zc::launch_plain(s, l->shared_gate, 0, x, H, 1, T, w.gate, false);
    // 6. routed experts (pipeline.cpp:18-29): gate/up on gathered rows, down scattered to its slot
    zc_linear rg, ru, rd;
    zc_hip_expert_linear(c, 0, l->expert_records, 0, &rg); zc_hip_expert_linear(c, 0, l->expert_records, 1, &ru); zc_hip_expert_linear(c, 0, l->expert_records, 2, &rd);
    const auto base = reinterpret_cast<uintptr_t>(l->expert_records);
    auto off = [&](const void* p) { return uint64_t(reinterpret_cast<uintptr_t>(p) - base); };
    const uint32_t jobs = uint32_t(std::min<uint64_t>(uint64_t(T) * k, E));
    {
        zc::ExpertPhaseDesc p{};
        p.records = l->expert_records; p.stride = l->record_stride;
        p.off[0] = off(rg.weight); p.off[1] = off(rg.scales); p.off[2] = off(rg.biases);
        p.off[3] = off(ru.weight); p.off[4] = off(ru.scales); p.off[5] = off(ru.biases);
        p.offsets = w.offsets; p.selected = w.selected; p.count = w.count; p.in_rows = w.rows; p.out_rows = nullptr;
        p.x = x; p.out = w.act; p.K = H; p.N = I; p.group = c->group; p.bits = c->bits_gate_up; p.x_sorted = 0; p.max_jobs = jobs; p.gated = true;
        zc::launch_expert_phase(s, p);
    }
    {
        zc::ExpertPhaseDesc p{};
        p.records = l->expert_records; p.stride = l->record_stride;
        p.off[0] = off(rd.weight); p.off[1] = off(rd.scales); p.off[2] = off(rd.biases);
        p.offsets = w.offsets; p.selected = w.selected; p.count = w.count; p.in_rows = nullptr; p.out_rows = w.slots;
        p.x = w.act; p.out = w.expert_out; p.K = I; p.N = H; p.group = c->group; p.bits = c->bits_down; p.x_sorted = 1; p.max_jobs = jobs; p.gated = false;
        zc::launch_expert_phase(s, p);
    }
    // 7. weighted combine (model.cpp:553-556)
    zc::launch_moe_sum(s, w.expert_out, w.weights, w.shared, w.gate, T, H, k, out);
    ZC_LAUNCHED();
    if (trace) {
        const uint64_t n = uint64_t(T) * k;
        if (trace->logits) ZC_HIP(hipMemcpyAsync(trace->logits, w.logits, uint64_t(T) * E * 4, hipMemcpyDeviceToDevice, s));
        if (trace->ids) ZC_HIP(hipMemcpyAsync(trace->ids, w.ids, n * 4, hipMemcpyDeviceToDevice, s));
        if (trace->weights) ZC_HIP(hipMemcpyAsync(trace->weights, w.weights, n * 4, hipMemcpyDeviceToDevice, s));
        if (trace->expert_out) ZC_HIP(hipMemcpyAsync(trace->expert_out, w.expert_out, n * H * 4, hipMemcpyDeviceToDevice, s));
        if (trace->shared) ZC_HIP(hipMemcpyAsync(trace->shared, w.shared, uint64_t(T) * H * 4, hipMemcpyDeviceToDevice, s));
        if (trace->gate) ZC_HIP(hipMemcpyAsync(trace->gate, w.gate, uint64_t(T) * 4, hipMemcpyDeviceToDevice, s));
    }
    return ZC_OK;
}
// Prefill: the same layer with the expert products as a sorted-token grouped GEMM on the bf16 matrix cores.
namespace {
struct PrefillSpace {
    Workspace base;
    uint16_t *xb, *actb, *sactb; float *xsum, *xplain, *asum, *ssum, *xsum16, *asum16, *ssum16;   // xplain: the inputs' sums for affine Q8 gate/up rows
    int32_t *tile_expert, *tile_first, *tile_rows, *tile_count, *stile_expert, *stile_first, *stile_rows, *stile_count;
    uint32_t max_tiles, max_shared_tiles;
    uint32_t* near_bits;      // one bit per product element: recompute exactly
    uint32_t* shared_near_bits;   // the same for the shared expert's products, which run beside the routed ones
    float* norms;             // |row| of the inputs and of the router's rows (the fast router's bound)
    uint64_t bytes;
};
PrefillSpace carve_prefill(const zc_moe_config* c, uint32_t T, void* base) {
    PrefillSpace w{};
    w.base = carve(c, T, base);
    uint64_t at = w.base.bytes;
    auto take = [&](uint64_t bytes) { void* p = base ? static_cast<uint8_t*>(base) + at : nullptr; at += align_up(bytes, 256); return p; };
    const uint64_t n = uint64_t(T) * c->topk;
    w.max_tiles = uint32_t(n / 32 + c->experts); w.max_shared_tiles = (T + 31) / 32;
    w.xb = (uint16_t*)take(uint64_t(T) * c->hidden * 2); w.xsum = (float*)take(uint64_t(T) * (c->hidden / 64) * 4);
    w.actb = (uint16_t*)take(n * c->inter * 2); w.asum = (float*)take(n * (c->inter / 64) * 4);
    w.sactb = (uint16_t*)take(uint64_t(T) * c->inter * 2); w.ssum = (float*)take(uint64_t(T) * (c->inter / 64) * 4);
    w.tile_expert = (int32_t*)take(w.max_tiles * 4ull); w.tile_first = (int32_t*)take(w.max_tiles * 4ull); w.tile_rows = (int32_t*)take(w.max_tiles * 4ull);
    w.tile_count = (int32_t*)take(4);
    w.stile_expert = (int32_t*)take(w.max_shared_tiles * 4ull); w.stile_first = (int32_t*)take(w.max_shared_tiles * 4ull);
    w.stile_rows = (int32_t*)take(w.max_shared_tiles * 4ull); w.stile_count = (int32_t*)take(4);
    w.near_bits = (uint32_t*)take(n * std::max(c->hidden, c->inter) / 8);
    w.xsum16 = (float*)take(uint64_t(T) * (c->hidden / 16) * 4); w.asum16 = (float*)take(n * (c->inter / 16) * 4);
    w.ssum16 = (float*)take(uint64_t(T) * (c->inter / 16) * 4);
    w.norms = (float*)take((uint64_t(T) + c->experts) * 4);
    w.xplain = (float*)take(uint64_t(T) * (c->hidden / 64) * 4);
    w.shared_near_bits = (uint32_t*)take(uint64_t(T) * std::max(c->hidden, c->inter) / 8);
    w.bytes = at;
    return w;
}
bool prefill_config(const zc_moe_config* c) {
    // every projection affine Q4 or affine Q8 (the mixed 4/8-bit artifact: Q4 routed gate/up, Q8 down and shared expert)
    auto q = [](uint32_t bits) { return bits == 4 || bits == 8; };
    return q(c->bits_gate_up) && q(c->bits_down) && q(c->shared_bits_gate_up) && q(c->shared_bits_down) && c->group == 64 &&
           zc::prefill_shape(c->hidden, c->inter, c->experts);
}
}  // namespace
uint64_t zc_hip_moe_prefill_workspace_bytes(const zc_moe_config* cfg, uint32_t tokens) {
    if (validate_config(cfg) != ZC_OK || !tokens || !prefill_config(cfg)) return 0;
    return carve_prefill(cfg, tokens, nullptr).bytes;
}
zc_status zc_hip_moe_prefill(zc_hip_ctx* ctx, const zc_moe_config* c, const zc_moe_layer* l, const float* x, uint32_t T,
                             float* out, void* workspace, const zc_moe_trace* trace) {
    Timed timed(ctx, "moe_prefill");
    if (const zc_status s = validate_config(c)) return s;
    ZC_REQUIRE(prefill_config(c), "the matrix-core prefill path takes affine Q4 and Q8 group 64 with hidden and intermediate sizes that are multiples of 128 up to 4096");
    ZC_REQUIRE(ctx && l && x && out && workspace && T && T <= 8192, "invalid MoE layer buffers");
    ZC_REQUIRE(uint64_t(T) * c->topk * std::max(c->hidden, c->inter) < (1ull << 32), "too many product elements for one prefill call");
    ZC_REQUIRE(l->router && l->shared_gate && l->shared_record && l->expert_records, "missing MoE layer weights");
    ZC_REQUIRE(l->record_stride >= zc_hip_record_bytes(c, 0) && l->record_stride % 16 == 0, "expert record stride is too small or not a multiple of 16");
    ZC_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(workspace) % 256 == 0 &&
               reinterpret_cast<uintptr_t>(l->router) % 16 == 0 && reinterpret_cast<uintptr_t>(l->expert_records) % 16 == 0 &&
               reinterpret_cast<uintptr_t>(l->shared_record) % 16 == 0, "MoE layer operands are misaligned");
    ZC_REQUIRE(x != out, "invalid or overlapping linear output");
    const PrefillSpace w = carve_prefill(c, T, workspace);
    hipStream_t s = ctx->stream;
    const uint32_t H = c->hidden, I = c->inter, E = c->experts, k = c->topk;
    const uint64_t n = uint64_t(T) * k;
    const bool half_out = !(trace && trace->expert_out) && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    // router logits, top-k + softmax, dispatch (model.cpp:434-479), shared gate: the exact kernels, except that a long batch
    // whose logits nobody asks for gets exact logits only where the selection can see the difference (launch_prefill_router)
    const bool x_q4 = c->bits_gate_up == 4 || c->shared_bits_gate_up == 4, x_q8 = c->bits_gate_up == 8 || c->shared_bits_gate_up == 8;
    zc::launch_prefill_rows(s, x, T, H, w.xb, x_q4 ? w.xsum : nullptr, x_q4 ? w.xsum16 : nullptr, x_q8 ? w.xplain : nullptr, ctx->moe_status);
    // the shared expert needs the bf16 rows and nothing of the routing: it runs on a stream of its own from here to the combine
    if (!ctx->beside) {
        ZC_HIP(hipStreamCreateWithFlags(&ctx->beside, hipStreamNonBlocking));
        ZC_HIP(hipEventCreateWithFlags(&ctx->fork, hipEventDisableTiming)); ZC_HIP(hipEventCreateWithFlags(&ctx->join, hipEventDisableTiming));
    }
    hipStream_t s2 = ctx->beside;
    ZC_HIP(hipEventRecord(ctx->fork, s)); ZC_HIP(hipStreamWaitEvent(s2, ctx->fork, 0));
    if (T >= 128 && !(trace && trace->logits)) {
        const bool select = k <= 64;   // the refinement's wavefront selects its token's experts too
        zc::launch_prefill_router(s, x, w.xb, l->router, l->router_offsets, T, H, E, k, w.norms, w.base.logits, select ? w.base.ids : nullptr, select ? w.base.weights : nullptr);
        if (!select) zc::launch_route(s, w.base.logits, T, E, k, w.base.ids, w.base.weights);
    } else {
        zc::launch_router(s, l->router, x, T, H, E, l->router_offsets, w.base.logits);
        zc::launch_route(s, w.base.logits, T, E, k, w.base.ids, w.base.weights);
    }
    // dispatch sort and the routed experts' tile list: one launch for a long batch
    const bool one_dispatch = zc::prefill_dispatch_fits(w.base.ids, T, k, E);
    if (one_dispatch) zc::launch_prefill_dispatch(s, w.base.ids, T, k, E, w.base.offsets, w.base.slots, w.base.rows, ctx->moe_status, w.tile_expert, w.tile_first, w.tile_rows, w.tile_count);
    else zc::launch_dispatch(s, w.base.ids, T, k, E, w.base.offsets, w.base.slots, w.base.rows, w.base.selected, w.base.count, ctx->moe_status);
    // operands of the matrix cores: bf16 rows and their group sums; work lists
    // the per-block chain sums pay where a lane of the recomputation has several blocks of a row (long rows); short rows form them in place
    const bool table_inter = I / 16 >= 128;
    if (!one_dispatch) zc::launch_prefill_tiles(s, w.base.offsets, E, 0, w.tile_expert, w.tile_first, w.tile_rows, w.tile_count);
    zc::launch_prefill_tiles(s2, nullptr, 1, T, w.stile_expert, w.stile_first, w.stile_rows, w.stile_count);
    auto offsets_of = [&](const void* record, int shared, uint64_t* off, int first, int count) {
        for (int q = 0; q < count; ++q) {
            zc_linear lin; zc_hip_expert_linear(c, shared, record, first + q, &lin);
            const auto base = reinterpret_cast<uintptr_t>(record);
            off[3 * q] = reinterpret_cast<uintptr_t>(lin.weight) - base; off[3 * q + 1] = reinterpret_cast<uintptr_t>(lin.scales) - base;
            off[3 * q + 2] = reinterpret_cast<uintptr_t>(lin.biases) - base;
        }
    };
    {   // routed gate/up + SwiGLU on gathered rows (pipeline.cpp:18-24), then down scattered to the slots (pipeline.cpp:25-29)
        zc::PrefillGemm g{};
        g.bits = c->bits_gate_up;
        g.a = w.xb; g.asum = g.bits == 4 ? w.xsum : w.xplain; g.asum16 = g.bits == 4 ? w.xsum16 : nullptr; g.a_rows = w.base.slots; g.a_div = k; g.out_rows = nullptr;
        g.records = static_cast<const uint8_t*>(l->expert_records); g.stride = l->record_stride; offsets_of(l->expert_records, 0, g.off, 0, 2);
        g.tile_expert = w.tile_expert; g.tile_first = w.tile_first; g.tile_rows = w.tile_rows; g.tile_count = w.tile_count;
        g.K = H; g.N = I; g.out_b = w.actb;
        g.near_bits = w.near_bits; g.near_words = uint32_t(uint64_t(n) * I / 32); g.near_margin = zc::prefill_margin(g.K); g.ids = w.base.ids; g.slots = w.base.slots;
        g.covered = w.base.offsets + E; g.experts = E;
        zc::launch_prefill_gemm(s, g, true, w.max_tiles);
        zc::launch_prefill_patch(s, g, true);
        zc::PrefillGemm d{};
        d.bits = c->bits_down;
        zc::launch_prefill_sums(s, w.actb, nullptr, uint32_t(n), I, w.asum, table_inter && d.bits == 4 ? w.asum16 : nullptr, d.bits == 8);
        d.a = w.actb; d.asum = w.asum; d.asum16 = table_inter && d.bits == 4 ? w.asum16 : nullptr; d.a_rows = nullptr; d.a_div = 1; d.out_rows = w.base.slots;
        d.records = g.records; d.stride = g.stride; offsets_of(l->expert_records, 0, d.off, 2, 1);
        d.tile_expert = w.tile_expert; d.tile_first = w.tile_first; d.tile_rows = w.tile_rows; d.tile_count = w.tile_count;
        d.K = I; d.N = H;
        // nobody asks for the slots' outputs: they go to the combine as bf16 (BF16 values either way), in the same space
        if (half_out) d.out_h = reinterpret_cast<uint16_t*>(w.base.expert_out); else d.out_f = w.base.expert_out;
        d.near_bits = w.near_bits; d.near_words = uint32_t(uint64_t(n) * H / 32); d.near_margin = zc::prefill_margin(d.K); d.ids = w.base.ids; d.slots = w.base.slots;
        d.covered = w.base.offsets + E; d.experts = E;
        zc::launch_prefill_gemm(s, d, false, w.max_tiles);
        zc::launch_prefill_patch(s, d, false);
    }
    {   // shared expert (model.cpp:482-485): one group of all the tokens, beside the routed experts
        zc::PrefillGemm g{};
        g.bits = c->shared_bits_gate_up;
        g.a = w.xb; g.asum = g.bits == 4 ? w.xsum : w.xplain; g.asum16 = g.bits == 4 ? w.xsum16 : nullptr; g.a_rows = nullptr; g.a_div = 1;
        g.records = static_cast<const uint8_t*>(l->shared_record); g.stride = 0; offsets_of(l->shared_record, 1, g.off, 0, 2);
        g.tile_expert = w.stile_expert; g.tile_first = w.stile_first; g.tile_rows = w.stile_rows; g.tile_count = w.stile_count;
        g.K = H; g.N = I; g.out_b = w.sactb;
        g.near_bits = w.shared_near_bits; g.near_words = uint32_t(uint64_t(T) * I / 32); g.near_margin = zc::prefill_margin(g.K); g.ids = nullptr; g.slots = nullptr;
        zc::launch_prefill_gemm(s2, g, true, w.max_shared_tiles);
        zc::launch_prefill_patch(s2, g, true);
        zc::PrefillGemm d{};
        d.bits = c->shared_bits_down;
        zc::launch_prefill_sums(s2, w.sactb, nullptr, T, I, w.ssum, table_inter && d.bits == 4 ? w.ssum16 : nullptr, d.bits == 8);
        d.a = w.sactb; d.asum = w.ssum; d.asum16 = table_inter && d.bits == 4 ? w.ssum16 : nullptr; d.a_rows = nullptr; d.a_div = 1; d.out_rows = nullptr;
        d.records = g.records; d.stride = 0; offsets_of(l->shared_record, 1, d.off, 2, 1);
        d.tile_expert = w.stile_expert; d.tile_first = w.stile_first; d.tile_rows = w.stile_rows; d.tile_count = w.stile_count;
        d.K = I; d.N = H; d.out_f = w.base.shared;
        d.near_bits = w.shared_near_bits; d.near_words = uint32_t(uint64_t(T) * H / 32); d.near_margin = zc::prefill_margin(d.K); d.ids = nullptr; d.slots = nullptr;
        zc::launch_prefill_gemm(s2, d, false, w.max_shared_tiles);
        zc::launch_prefill_patch(s2, d, false);
        zc::launch_plain(s2, l->shared_gate, 0, x, H, 1, T, w.base.gate, false);   // the gate dot of the combine: last, it is short
    }
    ZC_HIP(hipEventRecord(ctx->join, s2)); ZC_HIP(hipStreamWaitEvent(s, ctx->join, 0));
    // weighted combine (model.cpp:553-556)
    if (half_out) zc::launch_moe_sum_half(s, reinterpret_cast<const uint16_t*>(w.base.expert_out), w.base.weights, w.base.shared, w.base.gate, T, H, k, out);
    else zc::launch_moe_sum(s, w.base.expert_out, w.base.weights, w.base.shared, w.base.gate, T, H, k, out);
    ZC_LAUNCHED();
    if (trace) {
        if (trace->logits) ZC_HIP(hipMemcpyAsync(trace->logits, w.base.logits, uint64_t(T) * E * 4, hipMemcpyDeviceToDevice, s));
        if (trace->ids) ZC_HIP(hipMemcpyAsync(trace->ids, w.base.ids, n * 4, hipMemcpyDeviceToDevice, s));
        if (trace->weights) ZC_HIP(hipMemcpyAsync(trace->weights, w.base.weights, n * 4, hipMemcpyDeviceToDevice, s));
        if (trace->expert_out) ZC_HIP(hipMemcpyAsync(trace->expert_out, w.base.expert_out, n * H * 4, hipMemcpyDeviceToDevice, s));
        if (trace->shared) ZC_HIP(hipMemcpyAsync(trace->shared, w.base.shared, uint64_t(T) * H * 4, hipMemcpyDeviceToDevice, s));
        if (trace->gate) ZC_HIP(hipMemcpyAsync(trace->gate, w.base.gate, uint64_t(T) * 4, hipMemcpyDeviceToDevice, s));
    }
    return ZC_OK;
}
zc_status zc_hip_moe_check(zc_hip_ctx* ctx) {
    ZC_REQUIRE(ctx, "null context");
    int32_t flag = 0;
    ZC_HIP(hipMemcpyAsync(&flag, ctx->moe_status, 4, hipMemcpyDeviceToHost, ctx->stream));
    ZC_HIP(hipStreamSynchronize(ctx->stream));
    if (flag) {
        ZC_HIP(hipMemsetAsync(ctx->moe_status, 0, 4, ctx->stream));
        if (flag & 2) return fail(ZC_RUNTIME_ERROR, "HIP execution: the persistent decode kernel could not synchronise its workgroups");
        if (flag & 4) return fail(ZC_INVALID_ARGUMENT, "stacked decode input is not BF16-valued");
        return fail(ZC_RUNTIME_ERROR, "invalid router output");
    }
    return ZC_OK;
}
zc_status zc_hip_stack_glue(zc_hip_ctx* ctx, const float* y, uint32_t tokens, uint32_t hidden, float* x_next) {
    Timed timed(ctx, "stack_glue");
    ZC_REQUIRE(ctx && y && x_next && tokens && hidden, "invalid glue buffers");
    zc::launch_stack_glue(ctx->stream, y, tokens, hidden, x_next);
    ZC_LAUNCHED();
    return ZC_OK;
}
}  // extern "C"

struct zc_hip_stack {
    zc_moe_config cfg{};
    std::vector<zc_moe_layer> layers;
    uint32_t max_tokens = 0;
    // persistent path
    zc::DecodeLayer* dev_layers = nullptr;
    uint8_t* arena = nullptr; uint64_t arena_bytes = 0;
    float *logits = nullptr, *gate = nullptr, *shared_act = nullptr, *act = nullptr, *layer_out = nullptr, *eout = nullptr;
    uint32_t* maxabs = nullptr; uint32_t* sync = nullptr;
    unsigned long long* tlogits = nullptr; uint32_t *tact = nullptr, *tout = nullptr;   // tagged exchange buffers of the one-token kernel
    int32_t* wide_ids = nullptr; float* wide_weights = nullptr;   // routes of the nine-to-sixty-four-token kernel
    uint32_t* tspec = nullptr; int32_t* pred[2] = {nullptr, nullptr};   // prediction pass: its activations, the previous / this step's ids per layer
    uint32_t pred_turn = 0; bool pred_valid = false, speculate = true;
    uint32_t epoch = 1u << 12;
    uint32_t tag_base = 0;            // tags of the one-token kernel's exchange words: advanced by that kernel's launches only
    uint32_t wait_limit = 1u << 22;   // polls before a wait on another workgroup gives up
    int cus = 0; uint32_t lds_limit = 0;
    bool persistent_ok = false;
    // layered path
    void* workspace = nullptr; float *xa = nullptr, *xb = nullptr;
    // routed records behind an expert store: the kernels take every record's address from the store's table
    zc_hip_store* store = nullptr;
    // [L][tokens][topk] device copies of a launch's routes and pinned host copies (+ one status word each), two of each: the
    // host may look at one launch's routes while the next launch runs
    int32_t* route_ids[2] = {nullptr, nullptr}; float* route_weights = nullptr;
    int32_t* route_ids_host[2] = {nullptr, nullptr};
    hipEvent_t routes_copied[2] = {nullptr, nullptr};
    uint32_t turn = 0; int pending = -1; uint32_t pending_per_layer = 0;   // pending: the turn whose routes the store has not seen yet
    bool defer = true;                 // the last observed launch read nothing from a record's home: the next one is observed late
};

namespace {
bool all_q4(const zc_moe_config& c) { return c.bits_down == 4 && c.shared_bits_gate_up == 4 && c.shared_bits_down == 4; }
// Routed gate/up is affine Q4 (the exact-integer tiles); the down projection and the shared expert may be affine Q8, which
// the one-token kernel and the kernel for nine to sixty-four tokens run on literal lanes (two to eight tokens of such an
// artifact go through the latter as well; the kernel for two to eight tokens takes Q4 only).
bool persistent_shape(const zc_moe_config& c) {
    return c.bits_gate_up == 4 && (c.bits_down == 4 || c.bits_down == 8) && (c.shared_bits_gate_up == 4 || c.shared_bits_gate_up == 8) &&
           (c.shared_bits_down == 4 || c.shared_bits_down == 8) && c.group == 64 &&
           c.hidden % 512 == 0 && c.inter % 512 == 0 && c.hidden <= 3072 && c.inter <= 1024 && c.experts <= 1024 && c.topk <= 64;
}
}  // namespace

extern "C" {
static zc_status create_stack(zc_hip_ctx* ctx, const zc_moe_config* c, const zc_moe_layer* host_layers, uint32_t n_layers,
                              uint32_t max_tokens, zc_hip_store* store, zc_hip_stack** out) {
    if (const zc_status s = validate_config(c)) return s;
    ZC_REQUIRE(ctx && host_layers && n_layers && max_tokens && max_tokens <= 8192 && out, "invalid stack geometry");
    const void* const* table = nullptr;
    if (store) {
        uint32_t store_layers = 0, store_experts = 0; uint64_t store_record = 0;
        if (const zc_status s = zc_hip_store_geometry(store, &store_layers, &store_experts, &store_record)) return s;
        ZC_REQUIRE(store_layers == n_layers && store_experts == c->experts && store_record == zc_hip_record_bytes(c, 0),
                   "the expert store does not hold this stack's records");
        ZC_REQUIRE(max_tokens <= 64, "a stack behind an expert store decodes at most 64 tokens a call (one launch)");
        if (const zc_status s = zc_hip_store_table(store, &table)) return s;
    }
    for (uint32_t l = 0; l < n_layers; ++l) {
        const zc_moe_layer& y = host_layers[l];
        ZC_REQUIRE(y.router && y.shared_gate && y.shared_record && (store || y.expert_records), "missing MoE layer weights");
        ZC_REQUIRE(store || (y.record_stride >= zc_hip_record_bytes(c, 0) && y.record_stride % 16 == 0), "expert record stride is too small");
        ZC_REQUIRE(reinterpret_cast<uintptr_t>(y.router) % 16 == 0 && reinterpret_cast<uintptr_t>(y.expert_records) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(y.shared_record) % 16 == 0, "MoE layer operands are misaligned");
    }
    auto* st = new zc_hip_stack;
    st->cfg = *c; st->layers.assign(host_layers, host_layers + n_layers); st->max_tokens = max_tokens; st->store = store;
    auto cleanup = [&](zc_status code) { zc_hip_stack_destroy(ctx, st); return code; };
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, ctx->device) != hipSuccess) return cleanup(fail(ZC_RUNTIME_ERROR, "HIP execution: cannot query device"));
    st->cus = prop.multiProcessorCount;
    st->lds_limit = uint32_t(prop.sharedMemPerBlock) - 1024;
    const uint32_t T = max_tokens, H = c->hidden, E = c->experts, k = c->topk, I = c->inter;
    // layered path buffers
    void* p = nullptr;
    if (zc_hip_alloc(ctx, zc_hip_moe_workspace_bytes(c, T), &p)) return cleanup(ZC_BUDGET_EXCEEDED);
    st->workspace = p;
    if (zc_hip_alloc(ctx, uint64_t(T) * H * 4, &p)) return cleanup(ZC_BUDGET_EXCEEDED);
    st->xa = static_cast<float*>(p);
    if (zc_hip_alloc(ctx, uint64_t(T) * H * 4, &p)) return cleanup(ZC_BUDGET_EXCEEDED);
    st->xb = static_cast<float*>(p);
    // persistent path arena
    st->persistent_ok = persistent_shape(*c) && n_layers <= 16384;   // the 16-bit exchange tags tell at most 65535 layers apart
    if (st->persistent_ok) {
        const uint32_t Tp = T < 64 ? T : 64;   // tokens of the largest single launch
        uint64_t at = 0;
        auto take = [&](uint64_t bytes) { const uint64_t o = at; at += align_up(bytes, 256); return o; };
        const uint64_t o_layers = take(sizeof(zc::DecodeLayer) * n_layers), o_logits = take(uint64_t(Tp) * E * 4), o_gate = take(Tp * 4),
                       o_sact = take(uint64_t(Tp) * I * 4), o_act = take(uint64_t(Tp) * k * I * 4), o_lout = take(uint64_t(Tp) * H * 4),
                       o_max = take(std::max<uint64_t>(uint64_t(n_layers) * Tp * 4, uint64_t(Tp) * (H / 64 + 1) * 4)), o_sync = take(zc::kDecodeSyncBytes), o_eout = take(uint64_t(Tp) * (k + 1) * H * 4),
                       o_tlogits = take(uint64_t(E + 1) * 8), o_tact = take(uint64_t(k + 1) * I * 4), o_tout = take(uint64_t(2) * H * 4),
                       o_tspec = take(uint64_t(k + 1) * I * 4), o_pred0 = take(uint64_t(n_layers) * k * 4), o_pred1 = take(uint64_t(n_layers) * k * 4),
                       o_wids = take(uint64_t(Tp) * k * 4), o_wweights = take(uint64_t(Tp) * k * 4);
        if (zc_hip_alloc(ctx, at, &p)) return cleanup(ZC_BUDGET_EXCEEDED);
        st->arena = static_cast<uint8_t*>(p); st->arena_bytes = at;
        st->dev_layers = reinterpret_cast<zc::DecodeLayer*>(st->arena + o_layers);
        st->logits = reinterpret_cast<float*>(st->arena + o_logits); st->gate = reinterpret_cast<float*>(st->arena + o_gate);
        st->shared_act = reinterpret_cast<float*>(st->arena + o_sact); st->act = reinterpret_cast<float*>(st->arena + o_act);
        st->layer_out = reinterpret_cast<float*>(st->arena + o_lout); st->maxabs = reinterpret_cast<uint32_t*>(st->arena + o_max);
        st->sync = reinterpret_cast<uint32_t*>(st->arena + o_sync); st->eout = reinterpret_cast<float*>(st->arena + o_eout);
        st->tlogits = reinterpret_cast<unsigned long long*>(st->arena + o_tlogits); st->tact = reinterpret_cast<uint32_t*>(st->arena + o_tact);
        st->tout = reinterpret_cast<uint32_t*>(st->arena + o_tout);
        st->tspec = reinterpret_cast<uint32_t*>(st->arena + o_tspec);
        st->pred[0] = reinterpret_cast<int32_t*>(st->arena + o_pred0); st->pred[1] = reinterpret_cast<int32_t*>(st->arena + o_pred1);
        st->wide_ids = reinterpret_cast<int32_t*>(st->arena + o_wids); st->wide_weights = reinterpret_cast<float*>(st->arena + o_wweights);
        std::vector<zc::DecodeLayer> host(n_layers);
        for (uint32_t l = 0; l < n_layers; ++l) {
            const zc_moe_layer& y = host_layers[l];
            host[l] = zc::DecodeLayer{static_cast<const uint16_t*>(y.router), y.router_offsets, static_cast<const uint16_t*>(y.shared_gate),
                                      static_cast<const uint8_t*>(y.shared_record), static_cast<const uint8_t*>(y.expert_records), y.record_stride,
                                      table ? reinterpret_cast<const uint8_t* const*>(table) + uint64_t(l) * c->experts : nullptr};
        }
        if (hipMemsetAsync(st->arena, 0, at, ctx->stream) != hipSuccess ||
            hipMemcpyAsync(st->dev_layers, host.data(), sizeof(zc::DecodeLayer) * n_layers, hipMemcpyHostToDevice, ctx->stream) != hipSuccess ||
            hipStreamSynchronize(ctx->stream) != hipSuccess)
            return cleanup(fail(ZC_RUNTIME_ERROR, "HIP execution: cannot initialise the decode stack"));
    }
    if (store) {
        if (!st->persistent_ok) return cleanup(fail(ZC_INVALID_ARGUMENT, "a stack behind an expert store needs a shape the single-launch kernels take"));
        const uint64_t routes = uint64_t(n_layers) * max_tokens * k * 4;
        if (zc_hip_alloc(ctx, routes, &p)) return cleanup(ZC_BUDGET_EXCEEDED);
        st->route_weights = static_cast<float*>(p);
        for (int t = 0; t < 2; ++t) {
            if (zc_hip_alloc(ctx, routes, &p)) return cleanup(ZC_BUDGET_EXCEEDED);
            st->route_ids[t] = static_cast<int32_t*>(p);
            if (zc_hip_alloc_host(ctx, routes + 4, &p)) return cleanup(ZC_BUDGET_EXCEEDED);   // the last word: the status at the end of the launch
            st->route_ids_host[t] = static_cast<int32_t*>(p);
            if (hipEventCreateWithFlags(&st->routes_copied[t], hipEventDisableTiming) != hipSuccess) return cleanup(fail(ZC_RUNTIME_ERROR, "HIP execution: cannot create an event"));
        }
    }
    *out = st;
    return ZC_OK;
}
zc_status zc_hip_stack_create(zc_hip_ctx* ctx, const zc_moe_config* c, const zc_moe_layer* host_layers, uint32_t n_layers,
                              uint32_t max_tokens, zc_hip_stack** out) {
    return create_stack(ctx, c, host_layers, n_layers, max_tokens, nullptr, out);
}
zc_status zc_hip_stack_create_with_store(zc_hip_ctx* ctx, const zc_moe_config* c, const zc_moe_layer* host_layers, uint32_t n_layers,
                                         uint32_t max_tokens, zc_hip_store* store, zc_hip_stack** out) {
    ZC_REQUIRE(store, "null expert store");
    return create_stack(ctx, c, host_layers, n_layers, max_tokens, store, out);
}
zc_status zc_hip_stack_destroy(zc_hip_ctx* ctx, zc_hip_stack* st) {
    if (!st) return ZC_OK;
    ZC_REQUIRE(ctx, "null context");
    for (void* p : {static_cast<void*>(st->workspace), static_cast<void*>(st->xa), static_cast<void*>(st->xb), static_cast<void*>(st->arena),
                    static_cast<void*>(st->route_ids[0]), static_cast<void*>(st->route_ids[1]), static_cast<void*>(st->route_weights),
                    static_cast<void*>(st->route_ids_host[0]), static_cast<void*>(st->route_ids_host[1])})
        if (p) zc_hip_free(ctx, p);
    for (hipEvent_t e : st->routes_copied) if (e) (void)hipEventDestroy(e);
    delete st;
    return ZC_OK;
}
// Which single-launch kernel takes `tokens` rows in one launch, and its LDS plan: nt = 1 (one token), 8 (two to eight) or 64
// (nine to sixty-four); false if none does.
struct LaunchPlan { zc::DecodeLdsPlan one; zc::MultiLdsPlan multi; zc::WideLdsPlan wide; uint32_t nt = 0; };
static bool persistent_plan(zc_hip_ctx* ctx, zc_hip_stack* st, uint32_t tokens, LaunchPlan* plan) {
    if (!st->persistent_ok || !tokens || tokens > 64 || tokens > st->max_tokens) return false;
    const zc_moe_config& c = st->cfg;
    int per_cu = 0;
    (void)ctx;
    if (tokens == 1) {
        plan->nt = 1;
        plan->one = zc::decode_lds_plan(c.hidden, c.experts, c.topk, c.inter, tokens, st->lds_limit);
        if (plan->one.total > st->lds_limit || plan->one.slots_per_batch == 0) return false;
        if (zc::decode_stack_occupancy(1, plan->one.total, &per_cu) != hipSuccess) { (void)hipGetLastError(); return false; }
    } else if (tokens <= 8 && all_q4(c)) {
        plan->nt = 8;
        if (tokens * c.topk > 256) return false;
        plan->multi = zc::decode_multi_lds_plan(c.hidden, c.experts, c.topk, c.inter, tokens, st->lds_limit);
        if (plan->multi.total > st->lds_limit) return false;
        if (zc::decode_multi_occupancy(plan->multi.total, &per_cu) != hipSuccess) { (void)hipGetLastError(); return false; }
    } else {
        plan->nt = 64;
        plan->wide = zc::decode_wide_lds_plan(c.hidden, c.experts, c.topk, c.inter, tokens, st->lds_limit);
        if (plan->wide.total > st->lds_limit) return false;
        if (zc::decode_wide_occupancy(plan->wide.total, &per_cu) != hipSuccess) { (void)hipGetLastError(); return false; }
    }
    return per_cu >= 1;
}
// How a batch is cut into launches: up to eight tokens are one launch; more go sixty-four at a time through the kernel for
// nine to sixty-four tokens where its plan fits, eight at a time otherwise.  0: no single-launch path for this batch.
static uint32_t launch_unit(zc_hip_ctx* ctx, zc_hip_stack* st, uint32_t tokens) {
    LaunchPlan plan;
    if (tokens > st->max_tokens) return 0;
    if (tokens <= 8) return persistent_plan(ctx, st, tokens, &plan) ? 8u : 0u;
    for (const uint32_t unit : {64u, 8u}) {
        bool fits = true;
        for (uint32_t first = 0; first < tokens && fits; first += unit) fits = persistent_plan(ctx, st, std::min(unit, tokens - first), &plan);
        if (fits) return unit;
    }
    return 0;
}
// One launch of the persistent kernels: `tokens` (at most eight) rows starting at token `first` of a batch of `batch`.
static zc_status launch_piece(zc_hip_ctx* ctx, zc_hip_stack* st, const float* x, uint32_t tokens, float* out, const zc_stack_trace* trace,
                              uint32_t first, uint32_t batch, const LaunchPlan& plan) {
    const uint32_t nt = plan.nt;
    const zc_moe_config& c = st->cfg;
    const uint32_t L = uint32_t(st->layers.size()), H = c.hidden, k = c.topk;
    {
        zc::DecodeParams p{};
        p.H = H; p.E = c.experts; p.topk = k; p.I = c.inter; p.T = tokens; p.L = L;
        p.bits_down = c.bits_down; p.shared_bits_gate_up = c.shared_bits_gate_up; p.shared_bits_down = c.shared_bits_down;
        for (int shared = 0; shared < 2; ++shared)
            for (int pr = 0; pr < 3; ++pr) {
                zc_linear l; zc_hip_expert_linear(&c, shared, reinterpret_cast<const void*>(uintptr_t(4096)), pr, &l);
                uint64_t* o = shared ? p.so : p.ro;
                o[pr * 3 + 0] = reinterpret_cast<uintptr_t>(l.weight) - 4096; o[pr * 3 + 1] = reinterpret_cast<uintptr_t>(l.scales) - 4096;
                o[pr * 3 + 2] = reinterpret_cast<uintptr_t>(l.biases) - 4096;
            }
        p.layers = st->dev_layers; p.x_in = x; p.out = out;
        p.logits = st->logits; p.gate = st->gate; p.shared_act = st->shared_act; p.act = st->act; p.layer_out = st->layer_out;
        p.maxabs = st->maxabs; p.eout = st->eout;
        p.tlogits = st->tlogits; p.tact = st->tact; p.tout = st->tout; p.tspec = st->tspec;
        p.route_ids = st->wide_ids; p.route_weights = st->wide_weights;
        if (nt == 1 && st->speculate) {   // this step reads the ids the previous one-token step left, and leaves its own
            p.pred_in = st->pred_valid ? st->pred[st->pred_turn] : nullptr; p.pred_out = st->pred[st->pred_turn ^ 1u];
            st->pred_turn ^= 1u; st->pred_valid = true;
        }
        // trace rows of this piece inside the whole batch's arrays
        p.trace_tokens = batch;
        p.ids_trace = trace && trace->ids ? trace->ids + uint64_t(first) * k : nullptr;
        p.weights_trace = trace && trace->weights ? trace->weights + uint64_t(first) * k : nullptr;
        p.out_trace = trace && trace->outputs ? trace->outputs + uint64_t(first) * H : nullptr;
        if (st->store && !p.ids_trace) { p.ids_trace = st->route_ids[st->turn] + uint64_t(first) * k; p.weights_trace = st->route_weights + uint64_t(first) * k; }
        p.clocks = trace && first == 0 ? reinterpret_cast<unsigned long long*>(trace->clocks) : nullptr;
        p.sync = st->sync; p.epoch = st->epoch; p.status = ctx->moe_status; p.spin_limit = st->wait_limit;
        st->epoch += 5 * L + 16;   // at most five barriers per layer; wraps modulo 2^32, the barrier compares epochs as signed differences
        // The tagged buffers are written by one-token launches only, so their tags advance with those launches only:
        // a launch's layer 0 then expects the tag right after the one its predecessor's last layer left, however many
        // launches of the other kernel ran in between.
        p.tag_base = st->tag_base;
        if (nt == 1) st->tag_base = (st->tag_base + L) % 65535u;
        const uint32_t workgroups = uint32_t(st->cus);
        if (nt == 1) ZC_HIP(zc::launch_decode_stack(ctx->stream, p, nt, workgroups, plan.one));
        else if (nt == 8) ZC_HIP(zc::launch_decode_multi(ctx->stream, p, workgroups, plan.multi));
        else ZC_HIP(zc::launch_decode_wide(ctx->stream, p, workgroups, plan.wide));
    }
    return ZC_OK;
}
zc_status zc_hip_stack_set_wait_limit(zc_hip_ctx* ctx, zc_hip_stack* st, uint32_t polls) {
    ZC_REQUIRE(ctx && st, "null argument");
    st->wait_limit = polls ? polls : 1u << 22;
    return ZC_OK;
}
zc_status zc_hip_stack_set_speculation(zc_hip_ctx* ctx, zc_hip_stack* st, int on) {
    ZC_REQUIRE(ctx && st, "null argument");
    st->speculate = on != 0; st->pred_valid = false;
    return ZC_OK;
}
int zc_hip_stack_is_persistent(zc_hip_ctx* ctx, zc_hip_stack* st, uint32_t tokens) {
    if (!ctx || !st || !tokens) return 0;
    if (st->store && tokens > 64) return 0;
    return launch_unit(ctx, st, tokens) ? 1 : 0;
}
// Waits for the routes of the launch that the store has not seen yet, and shows them to the store.
static zc_status observe_pending(zc_hip_ctx* ctx, zc_hip_stack* st) {
    (void)ctx;
    if (st->pending < 0) return ZC_OK;
    const int turn = st->pending;
    st->pending = -1;
    ZC_HIP(hipEventSynchronize(st->routes_copied[turn]));
    const int32_t status = st->route_ids_host[turn][uint64_t(st->layers.size()) * st->max_tokens * st->cfg.topk];
    // Only a launch that gave up waiting (bit 2) has no routes to observe; the other bits (an unroutable row, an input that is
    // not BF16-valued) are sticky reports of this or an earlier call, and the router's padding id -1 is skipped one by one
    // inside the observation.
    if (status & 2) return ZC_OK;
    zc_store_table_stats before{}, after{};
    if (const zc_status s = zc_hip_store_table_stats(st->store, &before)) return s;
    if (const zc_status s = zc_hip_store_table_observe_layers(st->store, st->route_ids_host[turn], st->pending_per_layer)) return s;
    if (const zc_status s = zc_hip_store_table_stats(st->store, &after)) return s;
    st->defer = after.home_reads == before.home_reads;
    return ZC_OK;
}
zc_status zc_hip_stack_settle(zc_hip_ctx* ctx, zc_hip_stack* st) {
    ZC_REQUIRE(ctx && st, "null argument");
    return st->store ? observe_pending(ctx, st) : ZC_OK;
}
zc_status zc_hip_stack_decode(zc_hip_ctx* ctx, zc_hip_stack* st, const float* x, uint32_t tokens, float* out,
                              const zc_stack_trace* trace, uint32_t flags) {
    Timed timed(ctx, "stack_decode");
    ZC_REQUIRE(ctx && st && x && out && tokens && tokens <= st->max_tokens, "invalid stack decode buffers");
    ZC_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 && x != out, "invalid or overlapping linear output");
    const zc_moe_config& c = st->cfg;
    const uint32_t L = uint32_t(st->layers.size()), H = c.hidden, k = c.topk;
    LaunchPlan plan;
    const uint32_t unit = (flags & 1u) ? 0u : launch_unit(ctx, st, tokens);
    if (st->store) {
        ZC_REQUIRE(unit && tokens <= unit, "a stack behind an expert store runs as one launch only");
        if (const zc_status s = zc_hip_store_table_refresh_joining(st->store)) return s;
    }
    // More than eight tokens go through the single-launch kernels sixty-four (or eight) at a time, one launch per piece (tokens
    // do not interact inside a layer); every piece stays on the device from the first layer to the last.
    if (unit) {
        if (trace && trace->ids) ZC_REQUIRE(trace->weights, "a routing trace needs both ids and weights");
        for (uint32_t first = 0; first < tokens; first += unit) {
            const uint32_t piece = std::min(unit, tokens - first);
            if (!persistent_plan(ctx, st, piece, &plan)) return fail(ZC_LOGIC_ERROR, "no single-launch plan for a piece of the batch");
            if (const zc_status s = launch_piece(ctx, st, x + uint64_t(first) * H, piece, out + uint64_t(first) * H, trace, first, tokens, plan)) return s;
        }
        if (st->store) {
            // The launch reads every record through the store's table; afterwards the store learns which records those were:
            // hits are touched, misses are admitted and their fills start on the side stream (the next launch waits for them on
            // the device, see zc_hip_store_table_refresh_joining).  While launches read nothing from a record's home the routes
            // of one launch are looked at only after the next one has been enqueued, so the host never waits for the GPU; once a
            // launch has read from a home, launches are observed at once again: the sooner a fill starts, the fewer launches read
            // that record over the host link.
            const uint64_t per_layer = uint64_t(tokens) * k;
            const uint32_t turn = st->turn;
            const int32_t* routes = trace && trace->ids ? trace->ids : st->route_ids[turn];
            ZC_HIP(hipMemcpyAsync(st->route_ids_host[turn], routes, L * per_layer * 4, hipMemcpyDeviceToHost, ctx->stream));
            ZC_HIP(hipMemcpyAsync(st->route_ids_host[turn] + uint64_t(L) * st->max_tokens * k, ctx->moe_status, 4, hipMemcpyDeviceToHost, ctx->stream));
            ZC_HIP(hipEventRecord(st->routes_copied[turn], ctx->stream));
            if (st->pending >= 0) { if (const zc_status s = observe_pending(ctx, st)) return s; }
            st->pending = int(turn); st->pending_per_layer = uint32_t(per_layer); st->turn = turn ^ 1u;
            if (!st->defer) { if (const zc_status s = observe_pending(ctx, st)) return s; }
        }
        return ZC_OK;
    }
    // layer by layer: y = moe(x); x_next = glue(y)
    const float* cur = x;
    for (uint32_t l = 0; l < L; ++l) {
        float* y = l + 1 == L ? out : st->xa;
        zc_moe_trace tr{};
        if (trace) {
            tr.ids = trace->ids ? trace->ids + uint64_t(l) * tokens * k : nullptr;
            tr.weights = trace->weights ? trace->weights + uint64_t(l) * tokens * k : nullptr;
        }
        if (const zc_status s = zc_hip_moe_forward(ctx, &c, &st->layers[l], cur, tokens, y, st->workspace, trace ? &tr : nullptr)) return s;
        if (trace && trace->outputs) ZC_HIP(hipMemcpyAsync(trace->outputs + uint64_t(l) * tokens * H, y, uint64_t(tokens) * H * 4, hipMemcpyDeviceToDevice, ctx->stream));
        if (l + 1 < L) { zc::launch_stack_glue(ctx->stream, y, tokens, H, st->xb); cur = st->xb; }
    }
    ZC_LAUNCHED();
    return ZC_OK;
}

zc_status zc_hip_synth_words(zc_hip_ctx* ctx, uint32_t* dst, uint64_t count, uint64_t seed) {
    ZC_REQUIRE(ctx && (dst || !count), "null argument");
    if (count) { zc::launch_synth_words(ctx->stream, dst, count, seed); ZC_LAUNCHED(); }
    return ZC_OK;
}
zc_status zc_hip_synth_scales(zc_hip_ctx* ctx, uint16_t* scales, uint16_t* biases, uint64_t count, uint64_t seed, float lo, float span, float factor) {
    ZC_REQUIRE(ctx && ((scales && biases) || !count), "null argument");
    if (count) { zc::launch_synth_scales(ctx->stream, scales, biases, count, seed, lo, span, factor); ZC_LAUNCHED(); }
    return ZC_OK;
}
zc_status zc_hip_synth_normal_f32(zc_hip_ctx* ctx, float* dst, uint64_t count, uint64_t seed, float sigma) {
    ZC_REQUIRE(ctx && (dst || !count), "null argument");
    if (count) { zc::launch_synth_normal(ctx->stream, dst, count, seed, sigma, false); ZC_LAUNCHED(); }
    return ZC_OK;
}
zc_status zc_hip_synth_normal_bf16(zc_hip_ctx* ctx, uint16_t* dst, uint64_t count, uint64_t seed, float sigma) {
    ZC_REQUIRE(ctx && (dst || !count), "null argument");
    if (count) { zc::launch_synth_normal(ctx->stream, dst, count, seed, sigma, true); ZC_LAUNCHED(); }
    return ZC_OK;
}
zc_status zc_hip_synth_records(zc_hip_ctx* ctx, const zc_moe_config* c, int shared, void* records, uint64_t stride, uint32_t count, uint64_t seed) {
    if (const zc_status s = validate_config(c)) return s;
    ZC_REQUIRE(ctx && records && stride >= zc_hip_record_bytes(c, shared) && stride % 4 == 0, "expert record stride is too small");
    if (!count) return ZC_OK;
    uint64_t w_off[3], s_off[3], words[3], meta[3]; uint32_t bits[3];
    for (int p = 0; p < 3; ++p) {
        zc_linear l; zc_hip_expert_linear(c, shared, records, p, &l);
        w_off[p] = uint64_t(reinterpret_cast<uintptr_t>(l.weight) - reinterpret_cast<uintptr_t>(records));
        s_off[p] = uint64_t(reinterpret_cast<uintptr_t>(l.scales) - reinterpret_cast<uintptr_t>(records));
        words[p] = uint64_t(l.input) * l.output * l.bits / 32; meta[p] = uint64_t(l.input / l.group) * l.output; bits[p] = l.bits;
    }
    zc::launch_synth_records(ctx->stream, records, stride, count, w_off, s_off, words, meta, bits, seed);
    ZC_LAUNCHED();
    return ZC_OK;
}
}  // extern "C"
