// Host side of the MI355X MoE path in the reference's own vocabulary.
//
// The types and signatures below mirror the operator interface the reference's
// Model::moe is written against (include/engine/storage.hpp:54-63, include/engine/metal.hpp:6-13,
// 48-140, 154; include/engine/pipeline.hpp:6-8; include/engine/model.hpp:156), so that code
// written against that interface -- the body of Model::moe, encode_expert_rows, the reference's
// own tests of them -- compiles against this header unchanged apart from the shapes, which
// the reference fixes at compile time (storage.hpp:26-27) and this path takes from a MoeShape.
// Every method only forwards to the C ABI (include/zc_hip.h); there is no arithmetic here.
//
// Memory: the reference runs on unified memory where Buffer::data is CPU-visible.  Here
// Temporary / State / Workspace / Snapshot buffers are pinned host allocations mapped into
// the GPU (same pointer on both sides, readable after finish()); Resident / Expert buffers
// live in HBM (data == nullptr, filled with Metal::write).
#pragma once
#include <atomic>
#include <cstddef>
#include <cstdint>
#include <functional>
#include <initializer_list>
#include <memory>
#include <span>
#include <string>
#include <vector>
#include "../../../include/zc_hip.h"

namespace zerocool::engine {

uint64_t checked_add(uint64_t a, uint64_t b);
uint64_t checked_mul(uint64_t a, uint64_t b);
float bf16(uint16_t value);
float round_bf16(float value);

// storage.hpp:54-63
struct Buffer {
    uint64_t bytes = 0;
    std::byte* data = nullptr;     // CPU-visible contents, or nullptr for HBM-only buffers
    std::shared_ptr<void> owner;
    void* metal = nullptr;         // the device address (the reference's id<MTLBuffer>)
    static std::shared_ptr<Buffer> host(uint64_t bytes);
    std::span<float> floats() const;
};
using Buf = std::shared_ptr<Buffer>;
using Allocator = std::function<Buf(uint64_t)>;

// metal.hpp:6-13
struct Binding { Buf buffer; uint64_t offset = 0; };
enum class AllocationClass { Temporary, Resident, State, Expert, Snapshot, Workspace };
struct Linear {
    Binding weight, scales, biases;
    uint32_t input = 0, output = 0, group = 64, dtype = 0;
    bool quantized = false;
    uint32_t bits = 4;
};
// metal.hpp:17-43, the part that concerns this path
struct KernelConfig {
    std::string policy = "exact-int";   // "reference": literal lane kernels everywhere
    bool profile = false;               // record one timed row per operator call, tagged by Metal::label
    void validate() const;
};

// The shapes storage.hpp:26-27 fixes for the reference's model.
struct MoeShape {
    uint32_t hidden = 2560, experts = 512, topk = 10, inter = 640, group = 64;
    uint32_t bits_gate_up = 4, bits_down = 4, shared_bits_gate_up = 4, shared_bits_down = 4;
    zc_moe_config abi() const;
    uint64_t expert_bytes(bool shared = false) const;   // storage.hpp:32
};

// metal.hpp:48-140, the methods Model::moe and encode_expert_rows use
class Metal {
public:
    struct Completion { std::atomic<bool> done{false}; uint64_t ticket = 0; std::string error; };
    explicit Metal(MoeShape shape = {}, int device = 0);
    ~Metal();
    Metal(const Metal&) = delete;
    Metal& operator=(const Metal&) = delete;
    const MoeShape& shape() const { return shape_; }
    Buf allocate(uint64_t bytes);
    Buf allocate(uint64_t bytes, AllocationClass kind);
    Buf zeros(uint64_t floats);
    Buf zeros(uint64_t floats, AllocationClass kind);
    Buf upload(std::span<const float> values);
    void write(const Buf& destination, uint64_t offset, std::span<const std::byte> bytes);   // fills an HBM buffer
    void read(const Buf& source, uint64_t offset, std::span<std::byte> bytes);              // drains, then copies out
    void copy(const Buf& source, uint64_t source_offset, const Buf& destination, uint64_t destination_offset, uint64_t bytes);
    Buf slice(const Buf& source, uint64_t offset, uint64_t bytes);
    void budget(uint64_t bytes);
    void configure(KernelConfig config);
    bool direct_rows() const { return true; }
    // metal.mm:267-270: names the stage of the calls that follow in the profile rows (nothing unless configure() asked for a profile)
    void label(std::string stage, int layer = -1, uint32_t tokens = 0, uint32_t offset = 0, std::span<const uint32_t> experts = {});
    std::string statistics(const zc_hip_store* store = nullptr) const;   // JSON text: memory, profile rows, expert cache counters
    // "moe_sum" and "scatter_experts" are the two kernels the path dispatches by name (model.cpp:555, pipeline.cpp:28)
    void dispatch(const std::string& name, std::initializer_list<Binding> buffers, std::initializer_list<uint32_t> params,
                  uint32_t x, uint32_t y = 1, uint32_t z = 1, uint32_t tx = 32, uint32_t ty = 1, uint32_t tz = 1);
    std::shared_ptr<Completion> submit();
    void wait(const std::shared_ptr<Completion>& completion);
    void reap() {}
    void finish();
    Buf linear(const Linear& layer, const Buf& x, uint32_t tokens, bool float_output = false);
    void linear_into(const Linear& layer, const Buf& x, uint32_t tokens, Binding output, bool float_output = false);
    void grouped_experts(std::span<const Buf> records, std::span<const uint32_t> positions, const Buf& x, const Buf& output, const Buf& scratch);
    Buf gated_linear(const Linear& gate, const Linear& up, const Buf& x, uint32_t tokens, const Buf& rows = {});
    void route(const Buf& logits, const Buf& ids, const Buf& weights, uint32_t tokens);
    uint64_t allocated() const;
    uint64_t peak() const;
    std::string device_name() const;
    zc_hip_ctx* context() const { return ctx_; }
private:
    MoeShape shape_;
    zc_hip_ctx* ctx_ = nullptr;
    uint64_t budget_ = 0;
};
// metal.hpp:154, metal.mm:1124-1129
Linear expert_linear(const MoeShape& shape, const Buf& record, int projection, bool shared = false);

// storage.hpp:168-172, 183-192, 198-269: the expert cache, with the reference's names.  The records' home is pinned host
// memory (home()), the slots are HBM, fills run on the store's side stream (zc_hip_store_*).  A Lease pins its slot
// until it is destroyed: keep it until the GPU work that reads the slot has finished, as the reference does.
struct ExpertKey {
    uint32_t layer = 0, expert = 0;
    bool operator==(const ExpertKey&) const = default;
};
struct CacheStats {
    uint64_t hits = 0, misses = 0, evictions = 0, bytes = 0, ready_hits = 0, loading_joins = 0;
    uint64_t prefetches = 0, prefetch_claims = 0, prefetch_unclaimed = 0;
};
class ExpertCache {
public:
    class Lease {
    public:
        Lease() = default;
        ~Lease();
        Lease(Lease&& other) noexcept;
        Lease& operator=(Lease&& other) noexcept;
        Lease(const Lease&) = delete;
        bool ready() const;
        const Buf& wait() const;            // the compute stream waits for the slot's fill; the host does not block
        ExpertKey key() const;
        const char* acquisition() const;    // "new_miss", "ready_hit", "loading_join"
    private:
        friend class ExpertCache;
        zc_hip_store* store_ = nullptr;
        zc_store_lease lease_{};
        ExpertKey key_{};
        Buf slot_;
    };
    ExpertCache(Metal& gpu, uint32_t layers, size_t slots);
    ~ExpertCache();
    ExpertCache(const ExpertCache&) = delete;
    std::span<std::byte> home(ExpertKey key);   // where the record lives (pinned host memory): write it before first use
    Lease acquire(ExpertKey key);
    bool prefetch(ExpertKey key);
    bool ready(ExpertKey key) const;
    void clear();
    void resize(size_t slots);
    size_t capacity() const;
    size_t occupancy() const;
    CacheStats stats() const;
private:
    Metal& gpu_;
    zc_hip_store* store_ = nullptr;
    uint64_t record_bytes_ = 0;
};

// What Model::moe reads through Resident and the expert store for one layer.
struct MoeLayerWeights {
    Linear router;            // [experts][hidden] BF16, float output (model.cpp:434)
    Linear shared_gate;       // [1][hidden] BF16 (model.cpp:485)
    Buf shared_record;        // gate, up, down of the shared expert
    std::function<Buf(uint32_t expert)> record;   // the expert store: record of a routed expert
    // Next-layer prediction (model.cpp:437-445, 489-500), a cache hint only that never feeds model arithmetic: a caller
    // that has a `predict` input runs the NEXT layer's router on it beside this layer's, reads its top-k ids back with
    // the same readback, and calls prefetch(expert) for each distinct guess, at most prefetch_depth of them.
    Linear next_router;                             // [experts][hidden] BF16 of layer + 1; unused when empty
    std::function<bool(uint32_t expert)> prefetch;  // e.g. ExpertCache::prefetch({layer + 1, expert}); returns "issued"
    uint32_t prefetch_depth = 10;
};
// The layer as one enqueue with routing and dispatch kept on the device (zc_hip_moe_forward);
// records must be one buffer of experts * stride bytes.
Buf moe_resident(Metal& gpu, const MoeLayerWeights& weights, const Buf& records, uint64_t stride, const Buf& x, uint32_t tokens);

}  // namespace zerocool::engine
