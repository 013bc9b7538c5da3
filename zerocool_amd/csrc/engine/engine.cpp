// Host shim: the reference's operator interface over the C ABI.  Validation restates the
// checks of src/engine/metal.mm (cited per method); errors come back from the ABI as status
// codes and leave here as the exception classes the reference throws.
#include "engine.hpp"
#include <algorithm>
#include <array>
#include <bit>
#include <cstring>
#include <limits>
#include <stdexcept>

namespace zerocool::engine {
namespace {
[[noreturn]] void raise(zc_status status) {
    const std::string text = zc_hip_last_error();
    switch (status) {
        case ZC_INVALID_ARGUMENT: throw std::invalid_argument(text);
        case ZC_LOGIC_ERROR: throw std::logic_error(text);
        case ZC_OUT_OF_RANGE: throw std::out_of_range(text);
        default: throw std::runtime_error(text);   // runtime errors and "engine memory budget exceeded"
    }
}
void check(zc_status status) { if (status != ZC_OK) raise(status); }
bool covers(const Binding& b, uint64_t bytes) { return b.buffer && b.offset <= b.buffer->bytes && bytes <= b.buffer->bytes - b.offset; }
void* at(const Binding& b) { return static_cast<std::byte*>(b.buffer->metal) + b.offset; }
// metal.mm:649-661
void validate_affine(const Linear& l) {
    if (!l.input || !l.output || (l.bits != 4 && l.bits != 8) || (l.group != 32 && l.group != 64) || l.input % l.group)
        throw std::invalid_argument("unsupported affine matrix geometry");
    const auto weights = checked_mul(l.input, l.output) / (8 / l.bits);
    const auto metadata = checked_mul(checked_mul(l.input / l.group, l.output), 2);
    if (!covers(l.weight, weights) || !covers(l.scales, metadata) || !covers(l.biases, metadata))
        throw std::invalid_argument("affine tensor binding is truncated");
}
zc_linear abi(const Linear& l) {
    return zc_linear{at(l.weight), l.scales.buffer ? at(l.scales) : nullptr, l.biases.buffer ? at(l.biases) : nullptr,
                     l.input, l.output, l.group, l.dtype, l.quantized ? 1u : 0u, l.bits};
}
}  // namespace

// storage.cpp:20-35
uint64_t checked_add(uint64_t a, uint64_t b) { if (b > UINT64_MAX - a) throw std::overflow_error("tensor size overflow"); return a + b; }
uint64_t checked_mul(uint64_t a, uint64_t b) { if (a && b > UINT64_MAX / a) throw std::overflow_error("tensor size overflow"); return a * b; }
float bf16(uint16_t v) { return std::bit_cast<float>(uint32_t(v) << 16); }
float round_bf16(float v) {
    auto bits = std::bit_cast<uint32_t>(v);
    if ((bits & 0x7fffffff) > 0x7f800000) return std::numeric_limits<float>::quiet_NaN();
    bits += 0x7fff + ((bits >> 16) & 1);
    return std::bit_cast<float>(bits & 0xffff0000);
}

std::shared_ptr<Buffer> Buffer::host(uint64_t bytes) {
    auto b = std::make_shared<Buffer>();
    auto storage = std::shared_ptr<std::byte[]>(new std::byte[bytes ? bytes : 1]());
    b->bytes = bytes; b->data = storage.get(); b->owner = storage; b->metal = storage.get();
    return b;
}
std::span<float> Buffer::floats() const {
    if (!data) throw std::logic_error("buffer lives in HBM only; read it with Metal::read");
    return {reinterpret_cast<float*>(data), size_t(bytes / 4)};
}

void KernelConfig::validate() const {
    if (policy != "reference" && policy != "exact-int") throw std::invalid_argument("unknown kernel policy");
}
zc_moe_config MoeShape::abi() const {
    return zc_moe_config{hidden, experts, topk, inter, group, bits_gate_up, bits_down, shared_bits_gate_up, shared_bits_down};
}
uint64_t MoeShape::expert_bytes(bool shared) const { const auto c = abi(); return zc_hip_record_bytes(&c, shared ? 1 : 0); }

Metal::Metal(MoeShape shape, int device) : shape_(shape) { check(zc_hip_create(device, 0, &ctx_)); }
Metal::~Metal() { if (ctx_) zc_hip_destroy(ctx_); }
void Metal::budget(uint64_t bytes) { budget_ = bytes; }
void Metal::configure(KernelConfig config) {
    config.validate();
    check(zc_hip_configure(ctx_, config.policy == "reference" ? 0u : 1u));
    check(zc_hip_profile(ctx_, config.profile ? 1 : 0));
}
void Metal::label(std::string stage, int layer, uint32_t tokens, uint32_t offset, std::span<const uint32_t>) {
    check(zc_hip_label(ctx_, stage.c_str(), layer, tokens, offset));
}
std::string Metal::statistics(const zc_hip_store* store) const {
    uint64_t needed = 0;
    (void)zc_hip_stats(ctx_, store, nullptr, 0, &needed);
    std::string text(needed, '\0');
    check(zc_hip_stats(ctx_, store, text.data(), needed, &needed));
    text.resize(std::strlen(text.c_str()));
    return text;
}
uint64_t Metal::allocated() const { return zc_hip_allocated(ctx_); }
uint64_t Metal::peak() const { return zc_hip_peak(ctx_); }
std::string Metal::device_name() const { return zc_hip_version(); }

Buf Metal::allocate(uint64_t bytes) { return allocate(bytes, AllocationClass::Temporary); }
Buf Metal::allocate(uint64_t bytes, AllocationClass kind) {
    if (budget_ && checked_add(allocated(), bytes) > budget_) throw std::runtime_error("engine memory budget exceeded");   // metal.mm:395
    const bool hbm = kind == AllocationClass::Resident || kind == AllocationClass::Expert;
    void* p = nullptr;
    check(hbm ? zc_hip_alloc(ctx_, bytes, &p) : zc_hip_alloc_host(ctx_, bytes, &p));
    auto b = std::make_shared<Buffer>();
    b->bytes = bytes; b->metal = p; b->data = hbm ? nullptr : static_cast<std::byte*>(p);
    zc_hip_ctx* ctx = ctx_;
    b->owner = std::shared_ptr<void>(p, [ctx](void* q) { zc_hip_free(ctx, q); });   // waits for GPU users before freeing
    return b;
}
Buf Metal::zeros(uint64_t floats) { return zeros(floats, AllocationClass::Temporary); }
Buf Metal::zeros(uint64_t floats, AllocationClass kind) {
    auto b = allocate(checked_mul(floats, 4), kind);
    if (b->data) std::memset(b->data, 0, b->bytes); else check(zc_hip_memset(ctx_, b->metal, 0, b->bytes));
    return b;
}
Buf Metal::upload(std::span<const float> values) {
    auto b = allocate(values.size_bytes());
    std::memcpy(b->data, values.data(), values.size_bytes());
    return b;
}
void Metal::write(const Buf& d, uint64_t offset, std::span<const std::byte> bytes) {
    if (!d || offset > d->bytes || bytes.size() > d->bytes - offset) throw std::invalid_argument("write outside buffer");
    check(zc_hip_upload(ctx_, static_cast<std::byte*>(d->metal) + offset, bytes.data(), bytes.size()));
}
void Metal::read(const Buf& s, uint64_t offset, std::span<std::byte> bytes) {
    if (!s || offset > s->bytes || bytes.size() > s->bytes - offset) throw std::invalid_argument("read outside buffer");
    check(zc_hip_download(ctx_, bytes.data(), static_cast<std::byte*>(s->metal) + offset, bytes.size()));
}
void Metal::copy(const Buf& s, uint64_t so, const Buf& d, uint64_t doff, uint64_t bytes) {
    if (!s || !d || so > s->bytes || bytes > s->bytes - so || doff > d->bytes || bytes > d->bytes - doff) throw std::invalid_argument("copy outside buffer");
    check(zc_hip_copy(ctx_, static_cast<std::byte*>(d->metal) + doff, static_cast<std::byte*>(s->metal) + so, bytes));
}
Buf Metal::slice(const Buf& s, uint64_t offset, uint64_t bytes) {
    if (!s || offset > s->bytes || bytes > s->bytes - offset) throw std::invalid_argument("slice outside buffer");
    auto b = std::make_shared<Buffer>();
    b->bytes = bytes; b->metal = static_cast<std::byte*>(s->metal) + offset; b->data = s->data ? s->data + offset : nullptr; b->owner = s;
    return b;
}
std::shared_ptr<Metal::Completion> Metal::submit() {
    auto c = std::make_shared<Completion>();
    check(zc_hip_submit(ctx_, &c->ticket));
    return c;
}
void Metal::wait(const std::shared_ptr<Completion>& c) {
    if (!c) throw std::logic_error("wait on an empty completion");
    check(zc_hip_wait(ctx_, c->ticket));
    c->done = true;
}
void Metal::finish() { check(zc_hip_finish(ctx_)); }

// metal.mm:713-716
Buf Metal::linear(const Linear& l, const Buf& x, uint32_t tokens, bool float_output) {
    auto out = allocate(checked_mul(checked_mul(tokens, l.output), 4));
    linear_into(l, x, tokens, {out}, float_output);
    return out;
}
// metal.mm:775-827
void Metal::linear_into(const Linear& l, const Buf& x, uint32_t tokens, Binding out, bool float_output) {
    if (!tokens || !l.input || !l.output || !x || x->bytes < checked_mul(checked_mul(tokens, l.input), 4)) throw std::invalid_argument("linear input shape");
    if (!l.weight.buffer) throw std::invalid_argument("missing linear weights");
    if (l.quantized) validate_affine(l);
    const auto bytes = checked_mul(checked_mul(tokens, l.output), 4);
    if (!out.buffer || out.offset % 4 || out.offset > out.buffer->bytes || bytes > out.buffer->bytes - out.offset ||
        out.buffer->metal == x->metal || out.buffer->metal == l.weight.buffer->metal)
        throw std::invalid_argument("invalid or overlapping linear output");
    float* o = reinterpret_cast<float*>(at(out));
    const float* xi = static_cast<const float*>(x->metal);
    if (!l.quantized && float_output && l.dtype == 0 && l.input == shape_.hidden && l.output == shape_.experts) {   // the router branch, metal.mm:818-822
        check(zc_hip_router_logits(ctx_, at(l.weight), xi, tokens, l.input, l.output, nullptr, o));
        return;
    }
    const zc_linear a = abi(l);
    check(zc_hip_linear_into(ctx_, &a, xi, tokens, o, float_output ? 1 : 0));
}
// metal.mm:845-880
Buf Metal::gated_linear(const Linear& gate, const Linear& up, const Buf& x, uint32_t tokens, const Buf& rows) {
    if (!gate.quantized || !up.quantized || gate.input != up.input || gate.output != up.output || gate.group != up.group || gate.bits != up.bits)
        throw std::invalid_argument("fused gate/up requires matching affine matrices");
    validate_affine(gate); validate_affine(up);
    if (!tokens || !x || x->bytes < gate.input * 4ull || (rows ? rows->bytes < tokens * 4ull : x->bytes < uint64_t(tokens) * gate.input * 4))
        throw std::invalid_argument("fused gate/up input shape");
    auto out = allocate(uint64_t(tokens) * gate.output * 4);
    const zc_linear g = abi(gate), u = abi(up);
    check(zc_hip_gated_linear(ctx_, &g, &u, static_cast<const float*>(x->metal), uint32_t(x->bytes / (gate.input * 4ull)), tokens,
                              rows ? static_cast<const int32_t*>(rows->metal) : nullptr, static_cast<float*>(out->metal)));
    return out;
}
// metal.mm:261-266
void Metal::route(const Buf& logits, const Buf& ids, const Buf& weights, uint32_t tokens) {
    if (!tokens || tokens > 8192 || !logits || !ids || !weights || logits->bytes != uint64_t(tokens) * shape_.experts * 4 ||
        ids->bytes != uint64_t(tokens) * shape_.topk * 4 || weights->bytes != ids->bytes)
        throw std::invalid_argument("invalid route selection buffers");
    check(zc_hip_route(ctx_, static_cast<const float*>(logits->metal), tokens, shape_.experts, shape_.topk,
                       static_cast<int32_t*>(ids->metal), static_cast<float*>(weights->metal)));
}
// metal.mm:881-912
void Metal::grouped_experts(std::span<const Buf> records, std::span<const uint32_t> positions, const Buf& x, const Buf& out, const Buf& scratch) {
    const auto n = records.size();
    if (!n || n > 8 || positions.size() != n || !x || x->bytes < shape_.hidden * 4ull || !out || out->bytes < uint64_t(shape_.topk) * shape_.hidden * 4 ||
        !scratch || scratch->bytes < n * shape_.inter * 4ull || x->metal == out->metal || x->metal == scratch->metal || out->metal == scratch->metal)
        throw std::invalid_argument("invalid grouped expert geometry");
    std::array<const void*, 8> r{};
    for (size_t i = 0; i < n; ++i) {
        if (!records[i] || records[i]->bytes < shape_.expert_bytes()) throw std::invalid_argument("invalid grouped expert record or destination");
        r[i] = records[i]->metal;
    }
    const auto c = shape_.abi();
    check(zc_hip_grouped_experts(ctx_, &c, r.data(), positions.data(), uint32_t(n), static_cast<const float*>(x->metal),
                                 static_cast<float*>(out->metal), static_cast<float*>(scratch->metal)));
}
// metal.mm:510-557 for the two kernels this path dispatches by name
void Metal::dispatch(const std::string& name, std::initializer_list<Binding> buffers, std::initializer_list<uint32_t> params,
                     uint32_t x, uint32_t y, uint32_t, uint32_t, uint32_t, uint32_t) {
    std::vector<Binding> b(buffers); std::vector<uint32_t> p(params);
    for (const auto& v : b) if (!v.buffer || v.offset > v.buffer->bytes) throw std::invalid_argument("invalid kernel binding");
    if (name == "moe_sum") {   // model.cpp:555
        if (b.size() != 5 || p.size() != 1 || x != shape_.hidden || y != p[0]) throw std::invalid_argument("moe_sum dispatch shape");
        check(zc_hip_moe_sum(ctx_, static_cast<const float*>(at(b[0])), static_cast<const float*>(at(b[1])), static_cast<const float*>(at(b[2])),
                             static_cast<const float*>(at(b[3])), p[0], shape_.hidden, shape_.topk, static_cast<float*>(at(b[4]))));
    } else if (name == "scatter_experts") {   // pipeline.cpp:28
        if (b.size() != 3 || p.size() != 1 || x != shape_.hidden || y != p[0]) throw std::invalid_argument("scatter_experts dispatch shape");
        check(zc_hip_scatter_experts(ctx_, static_cast<const float*>(at(b[0])), static_cast<const int32_t*>(at(b[1])), p[0], shape_.hidden,
                                     static_cast<float*>(at(b[2]))));
    } else if (name == "unary") {   // model.cpp:330: {x, out}, {count, op}
        if (b.size() != 2 || p.size() != 2 || x != p[0] || b[0].buffer->bytes - b[0].offset < uint64_t(p[0]) * 4 || b[1].buffer->bytes - b[1].offset < uint64_t(p[0]) * 4)
            throw std::invalid_argument("unary dispatch shape");
        check(zc_hip_unary(ctx_, static_cast<const float*>(at(b[0])), p[0], p[1], static_cast<float*>(at(b[1]))));
    } else if (name == "binary") {   // model.cpp:335: {x, y, out}, {count, op}
        if (b.size() != 3 || p.size() != 2 || x != p[0]) throw std::invalid_argument("binary shape mismatch");
        for (const auto& v : b) if (v.buffer->bytes - v.offset < uint64_t(p[0]) * 4) throw std::invalid_argument("binary shape mismatch");
        check(zc_hip_binary(ctx_, static_cast<const float*>(at(b[0])), static_cast<const float*>(at(b[1])), p[0], p[1], static_cast<float*>(at(b[2]))));
    } else if (name == "hc_mix") {   // model.cpp:343: {n, mix, out}, {tokens}, grid hidden x tokens
        if (b.size() != 3 || p.size() != 1 || x != shape_.hidden || y != p[0]) throw std::invalid_argument("hc_mix dispatch shape");
        check(zc_hip_hc_mix(ctx_, static_cast<const float*>(at(b[0])), static_cast<const float*>(at(b[1])), p[0], shape_.hidden, static_cast<float*>(at(b[2]))));
    } else if (name == "hc_add") {   // model.cpp:651: {hyper, x, inject, out}, {tokens}, grid 4*hidden x tokens
        if (b.size() != 4 || p.size() != 1 || x != 4 * shape_.hidden || y != p[0]) throw std::invalid_argument("hc_add dispatch shape");
        check(zc_hip_hc_add(ctx_, static_cast<const float*>(at(b[0])), static_cast<const float*>(at(b[1])), static_cast<const float*>(at(b[2])), p[0],
                            shape_.hidden, static_cast<float*>(at(b[3]))));
    } else if (name == "norm" || name == "norm_wide") {   // model.cpp:318-325: {x, w, out}, {group, width, tokens, dtype, grouped}
        if (b.size() != 3 || p.size() != 5 || !p[0] || p[1] % p[0]) throw std::invalid_argument("normalization shape");
        check(zc_hip_norm(ctx_, static_cast<const float*>(at(b[0])), at(b[1]), p[3], p[0], p[1], p[2], static_cast<float*>(at(b[2]))));
    } else throw std::invalid_argument("unknown kernel: " + name);
}

Linear expert_linear(const MoeShape& shape, const Buf& record, int projection, bool shared) {
    if (projection < 0 || projection > 2 || !record || record->bytes < shape.expert_bytes(shared)) throw std::invalid_argument("invalid expert projection");
    const auto c = shape.abi();
    zc_linear l;
    check(zc_hip_expert_linear(&c, shared ? 1 : 0, record->metal, projection, &l));
    const auto base = reinterpret_cast<uintptr_t>(record->metal);
    return {{record, uint64_t(reinterpret_cast<uintptr_t>(l.weight) - base)}, {record, uint64_t(reinterpret_cast<uintptr_t>(l.scales) - base)},
            {record, uint64_t(reinterpret_cast<uintptr_t>(l.biases) - base)}, l.input, l.output, l.group, 0, true, l.bits};
}

// Model::moe (model.cpp:431-557) as ONE enqueue: routing, dispatch, expert products and the combine stay on the device
// (zc_hip_moe_forward).  The reference's own host-side orchestration of the same operators (one readback of the ids per
// layer, encode_expert_rows per expert) is what an engine keeps when it only swaps the operator class; it is restated
// next to the C++ tests, which drive this library through it call for call.
Buf moe_resident(Metal& gpu, const MoeLayerWeights& w, const Buf& records, uint64_t stride, const Buf& x, uint32_t tokens) {
    const auto& s = gpu.shape();
    if (!records || !x || !tokens || x->bytes < uint64_t(tokens) * s.hidden * 4 || records->bytes < checked_mul(stride, s.experts))
        throw std::invalid_argument("invalid MoE layer buffers");
    const auto c = s.abi();
    auto ws = gpu.allocate(zc_hip_moe_workspace_bytes(&c, tokens), AllocationClass::Resident);
    auto out = gpu.allocate(uint64_t(tokens) * s.hidden * 4);
    const zc_moe_layer layer{static_cast<std::byte*>(w.router.weight.buffer->metal) + w.router.weight.offset, nullptr,
                             static_cast<std::byte*>(w.shared_gate.weight.buffer->metal) + w.shared_gate.weight.offset,
                             w.shared_record->metal, records->metal, stride};
    check(zc_hip_moe_forward(gpu.context(), &c, &layer, static_cast<const float*>(x->metal), tokens, static_cast<float*>(out->metal), ws->metal, nullptr));
    check(zc_hip_moe_check(gpu.context()));   // drains, and reports "invalid router output" like model.cpp:459
    return out;
}


// ---- expert cache (storage.cpp:525-725 over zc_hip_store_*)
ExpertCache::ExpertCache(Metal& gpu, uint32_t layers, size_t slots) : gpu_(gpu), record_bytes_(gpu.shape().expert_bytes()) {
    check(zc_hip_store_create(gpu.context(), layers, gpu.shape().experts, record_bytes_, slots, &store_));
}
ExpertCache::~ExpertCache() { zc_hip_store_destroy(store_); }
std::span<std::byte> ExpertCache::home(ExpertKey key) {
    void* p = zc_hip_store_backing(store_, key.layer, key.expert);
    if (!p) throw std::out_of_range("invalid expert id");
    return {static_cast<std::byte*>(p), size_t(record_bytes_)};
}
ExpertCache::Lease ExpertCache::acquire(ExpertKey key) {
    Lease lease;
    check(zc_hip_store_acquire(store_, key.layer, key.expert, &lease.lease_));
    lease.store_ = store_; lease.key_ = key;
    lease.slot_ = std::make_shared<Buffer>();
    lease.slot_->bytes = record_bytes_; lease.slot_->metal = lease.lease_.record;
    return lease;
}
bool ExpertCache::prefetch(ExpertKey key) { int issued = 0; check(zc_hip_store_prefetch(store_, key.layer, key.expert, &issued)); return issued != 0; }
bool ExpertCache::ready(ExpertKey key) const { return zc_hip_store_ready(store_, key.layer, key.expert) != 0; }
void ExpertCache::clear() { check(zc_hip_store_clear(store_)); }
void ExpertCache::resize(size_t slots) { check(zc_hip_store_resize(store_, slots)); }
size_t ExpertCache::capacity() const { return zc_hip_store_capacity(store_); }
size_t ExpertCache::occupancy() const { return zc_hip_store_occupancy(store_); }
CacheStats ExpertCache::stats() const {
    zc_store_stats s{}; check(zc_hip_store_stats(store_, &s));
    return CacheStats{s.hits, s.misses, s.evictions, s.bytes, s.ready_hits, s.loading_joins, s.prefetches, s.prefetch_claims, s.prefetch_unclaimed};
}
ExpertCache::Lease::~Lease() { if (store_) zc_hip_store_release(store_, lease_.lease); }
ExpertCache::Lease::Lease(Lease&& o) noexcept : store_(o.store_), lease_(o.lease_), key_(o.key_), slot_(std::move(o.slot_)) { o.store_ = nullptr; }
ExpertCache::Lease& ExpertCache::Lease::operator=(Lease&& o) noexcept {
    if (this != &o) {
        if (store_) zc_hip_store_release(store_, lease_.lease);
        store_ = o.store_; lease_ = o.lease_; key_ = o.key_; slot_ = std::move(o.slot_); o.store_ = nullptr;
    }
    return *this;
}
bool ExpertCache::Lease::ready() const { return store_ && zc_hip_store_ready(store_, key_.layer, key_.expert) != 0; }
const Buf& ExpertCache::Lease::wait() const {
    if (!store_) throw std::logic_error("empty expert lease");
    check(zc_hip_store_wait(store_, lease_.lease));
    return slot_;
}
ExpertKey ExpertCache::Lease::key() const { if (!store_) throw std::logic_error("empty expert lease"); return key_; }
const char* ExpertCache::Lease::acquisition() const { return lease_.acquisition == 0 ? "new_miss" : lease_.acquisition == 1 ? "ready_hit" : "loading_join"; }

}  // namespace zerocool::engine
