// Expert store: every record has a home in pinned host memory; a fixed pool of HBM slots caches the records in
// use.  Fills are hipMemcpyAsync on a side stream of the store's own, each followed by an event; a compute stream
// that is about to read a slot waits on that event (no host blocking).  The policy (which record, which slot)
// is zc::SlotCache.  With as many slots as records the store is simply HBM-resident after the first touch.
//
// A store created without a context keeps its slots in ordinary host memory and finishes a fill when the caller
// says so (zc_hip_store_hold): the policy can then be tested without a GPU, loading states included.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstring>
#include <memory>
#include <string>
#include <unordered_set>
#include <vector>
#include "../../include/zc_hip.h"
#include "zc_store.hpp"

zc_status zc_fail(zc_status code, const std::string& text);

struct zc_hip_store {
    zc_hip_ctx* ctx = nullptr;          // nullptr: host-memory slots
    uint32_t layers = 0, experts = 0;
    uint64_t record_bytes = 0, stride = 0;
    std::vector<uint8_t*> owned_homes;  // the allocations behind `homes` (fewer than layers when layers share their records' homes)
    std::vector<uint8_t*> homes;        // per layer: [experts] records, pinned host memory (or plain, without a context); one allocation
                                        // per layer, because a single pinned block for a large model can exceed what the driver grants
    uint8_t* pool = nullptr;            // [capacity] slots, HBM (or plain host memory)
    hipStream_t side = nullptr;
    std::vector<hipEvent_t> filled;     // per slot: recorded after the slot's last fill
    std::vector<hipEvent_t> released;   // per slot: recorded on the compute stream at every release of a lease; the slot's next fill waits for it
    std::vector<uint64_t> pending;      // host-memory store: per slot, the key of a fill that waits for its release, or ~0
    std::unordered_set<uint64_t> held;  // host-memory store: keys whose fills wait
    std::unique_ptr<zc::SlotCache> cache;
    std::vector<uint64_t> layer_hits, layer_misses;
    // Device-side view (zc_hip_store_table): one pointer per record, to its slot while the slot holds the finished record,
    // to its home otherwise.  `mirror` is the host's copy (pinned), `table` what kernels read.
    const uint8_t** mirror = nullptr; const uint8_t** table = nullptr;
    bool table_changed = false;
    std::vector<uint64_t> shown;        // per slot: the key whose table entry points at the slot, or ~0
    std::vector<uint64_t> arriving;     // per slot: the key of a fill whose entry has not been switched to the slot yet, or ~0
    std::vector<size_t> in_flight;      // the slots with an `arriving` key
    zc_store_table_stats seen{};
};

namespace {
constexpr uint64_t kNone = ~0ull;
uint64_t key_of(const zc_hip_store* s, uint32_t layer, uint32_t expert) { return uint64_t(layer) * s->experts + expert; }
uint8_t* home_of(const zc_hip_store* s, uint64_t key) { return s->homes[key / s->experts] + (key % s->experts) * s->stride; }

template <class F> zc_status guarded(F f) {
    try { return f(); }
    catch (const std::invalid_argument& e) { return zc_fail(ZC_INVALID_ARGUMENT, e.what()); }
    catch (const std::out_of_range& e) { return zc_fail(ZC_OUT_OF_RANGE, e.what()); }
    catch (const std::logic_error& e) { return zc_fail(ZC_LOGIC_ERROR, e.what()); }
    catch (const std::exception& e) { return zc_fail(ZC_RUNTIME_ERROR, e.what()); }
}
#define ZC_STORE_HIP(call) do { const hipError_t e_ = (call); if (e_ != hipSuccess) throw std::runtime_error(std::string("HIP execution: ") + hipGetErrorString(e_) + " in " #call); } while (0)

void finish_host_fill(zc_hip_store* s, size_t slot) {
    const uint64_t key = s->pending[slot];
    if (key == kNone) return;
    std::memcpy(s->pool + slot * s->stride, home_of(s, key), s->record_bytes);
    s->pending[slot] = kNone;
}
// A fill of `slot` begins: whatever record the table showed there goes back to its home, and the new record's entry
// stays at its home until zc_hip_store_table_refresh finds the fill finished.
void table_fill_begins(zc_hip_store* s, size_t slot, uint64_t key) {
    if (!s->mirror) return;
    if (slot >= s->shown.size()) { s->shown.resize(slot + 1, kNone); s->arriving.resize(slot + 1, kNone); }
    if (s->shown[slot] != kNone) { s->mirror[s->shown[slot]] = home_of(s, s->shown[slot]); s->shown[slot] = kNone; s->table_changed = true; }
    if (s->arriving[slot] == kNone) s->in_flight.push_back(slot);
    s->arriving[slot] = key;
}
zc::SlotCache::Hooks hooks_of(zc_hip_store* s) {
    zc::SlotCache::Hooks h;
    if (s->ctx) {
        h.start = [s](size_t slot, uint64_t key) {
            table_fill_begins(s, slot, key);
            // The slot's previous record may still be read by kernels that were enqueued before its lease was released:
            // the fill is ordered after the compute stream's position at that release, on the device, without the host.
            ZC_STORE_HIP(hipStreamWaitEvent(s->side, s->released[slot], 0));
            ZC_STORE_HIP(hipMemcpyAsync(s->pool + slot * s->stride, home_of(s, key), s->record_bytes, hipMemcpyHostToDevice, s->side));
            ZC_STORE_HIP(hipEventRecord(s->filled[slot], s->side));
        };
        h.done = [s](size_t slot) {
            const hipError_t e = hipEventQuery(s->filled[slot]);
            if (e == hipErrorNotReady) return false;
            ZC_STORE_HIP(e);
            return true;
        };
        h.wait = [s](size_t slot) { ZC_STORE_HIP(hipEventSynchronize(s->filled[slot])); };
        h.move = [s](size_t from, size_t to) {
            ZC_STORE_HIP(hipStreamWaitEvent(s->side, s->released[to], 0));
            ZC_STORE_HIP(hipMemcpyAsync(s->pool + to * s->stride, s->pool + from * s->stride, s->record_bytes, hipMemcpyDeviceToDevice, s->side));
            ZC_STORE_HIP(hipEventRecord(s->filled[to], s->side));
        };
    } else {
        h.start = [s](size_t slot, uint64_t key) { table_fill_begins(s, slot, key); s->pending[slot] = key; if (!s->held.count(key)) finish_host_fill(s, slot); };
        h.done = [s](size_t slot) { return s->pending[slot] == kNone; };
        h.wait = [s](size_t slot) {
            if (s->pending[slot] != kNone && s->held.count(s->pending[slot])) throw std::logic_error("waiting for a fill that the test still holds");
            finish_host_fill(s, slot);
        };
        h.move = [s](size_t from, size_t to) { std::memcpy(s->pool + to * s->stride, s->pool + from * s->stride, s->record_bytes); };
    }
    return h;
}
// After the slots moved or emptied (clear, resize; every fill has finished by then): the table from scratch.
void table_rebuild(zc_hip_store* s) {
    if (!s->mirror) return;
    const uint64_t records = uint64_t(s->layers) * s->experts;
    for (uint64_t key = 0; key < records; ++key) s->mirror[key] = home_of(s, key);
    s->shown.assign(s->cache->capacity(), kNone); s->arriving.assign(s->cache->capacity(), kNone); s->in_flight.clear();
    for (size_t slot = 0; slot < s->cache->capacity(); ++slot)
        if (const int64_t key = s->cache->key_of(slot); key >= 0) { s->mirror[key] = s->pool + slot * s->stride; s->shown[slot] = uint64_t(key); }
    s->table_changed = true;
}
// Slot storage for `slots` slots; keeps the bytes of the first `keep` slots.
void provide_pool(zc_hip_store* s, uint64_t slots, uint64_t keep) {
    uint8_t* fresh = nullptr;
    if (s->ctx) {
        void* p = nullptr;
        if (zc_hip_alloc(s->ctx, slots * s->stride, &p) != ZC_OK) throw std::runtime_error(zc_hip_last_error());
        fresh = static_cast<uint8_t*>(p);
        if (s->pool && keep) { ZC_STORE_HIP(hipMemcpyAsync(fresh, s->pool, keep * s->stride, hipMemcpyDeviceToDevice, s->side)); ZC_STORE_HIP(hipStreamSynchronize(s->side)); }
        if (s->pool) zc_hip_free(s->ctx, s->pool);
        while (s->filled.size() > slots) { (void)hipEventDestroy(s->filled.back()); s->filled.pop_back(); }
        while (s->released.size() > slots) { (void)hipEventDestroy(s->released.back()); s->released.pop_back(); }
        while (s->filled.size() < slots) {
            hipEvent_t e; ZC_STORE_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
            ZC_STORE_HIP(hipEventRecord(e, s->side));   // a slot that was never filled counts as finished
            s->filled.push_back(e);
        }
        while (s->released.size() < slots) {
            hipEvent_t e; ZC_STORE_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
            ZC_STORE_HIP(hipEventRecord(e, s->side));   // a slot that was never leased has no reader to wait for
            s->released.push_back(e);
        }
    } else {
        fresh = new uint8_t[slots * s->stride]();
        if (s->pool && keep) std::memcpy(fresh, s->pool, keep * s->stride);
        delete[] s->pool;
        s->pending.resize(slots, kNone);
    }
    s->pool = fresh;
}
}  // namespace

extern "C" {

zc_status zc_hip_store_create(zc_hip_ctx* ctx, uint32_t layers, uint32_t experts, uint64_t record_bytes, uint64_t slots, zc_hip_store** out) {
    return zc_hip_store_create_with_policy(ctx, layers, experts, record_bytes, slots, "clock", out);
}
zc_status zc_hip_store_create_with_policy(zc_hip_ctx* ctx, uint32_t layers, uint32_t experts, uint64_t record_bytes, uint64_t slots,
                                          const char* policy, zc_hip_store** out) {
    return zc_hip_store_create_shared_homes(ctx, layers, experts, record_bytes, slots, policy, layers, out);
}
zc_status zc_hip_store_create_shared_homes(zc_hip_ctx* ctx, uint32_t layers, uint32_t experts, uint64_t record_bytes, uint64_t slots,
                                           const char* policy, uint32_t home_layers, zc_hip_store** out) {
    if (!out || !layers || !experts || !record_bytes || !slots) return zc_fail(ZC_INVALID_ARGUMENT, "empty expert cache");
    if (!home_layers || home_layers > layers) return zc_fail(ZC_INVALID_ARGUMENT, "invalid number of record homes");
    const std::string name = policy ? policy : "";
    if (name != "clock" && name != "slru") return zc_fail(ZC_INVALID_ARGUMENT, "cache policy must be clock or slru");   // parse_cache_policy, storage.cpp:536-540
    auto s = std::make_unique<zc_hip_store>();
    s->ctx = ctx; s->layers = layers; s->experts = experts; s->record_bytes = record_bytes; s->stride = (record_bytes + 255) / 256 * 256;
    s->layer_hits.assign(layers, 0); s->layer_misses.assign(layers, 0);
    const zc_status status = guarded([&] {
        const uint64_t home = uint64_t(experts) * s->stride;
        for (uint32_t l = 0; l < home_layers; ++l) {
            if (ctx) {
                void* p = nullptr;
                if (zc_hip_alloc_host(ctx, home, &p) != ZC_OK) throw std::runtime_error(zc_hip_last_error());
                s->owned_homes.push_back(static_cast<uint8_t*>(p));
            } else {
                s->owned_homes.push_back(new uint8_t[home]());
            }
        }
        for (uint32_t l = 0; l < layers; ++l) s->homes.push_back(s->owned_homes[l % home_layers]);   // layer l's records live in home l mod home_layers
        if (ctx) ZC_STORE_HIP(hipStreamCreateWithFlags(&s->side, hipStreamNonBlocking));   // default priority
        provide_pool(s.get(), slots, 0);
        s->cache = std::make_unique<zc::SlotCache>(slots, record_bytes, hooks_of(s.get()), name == "slru" ? zc::SlotCache::SegmentedLRU : zc::SlotCache::Clock);
        return ZC_OK;
    });
    if (status != ZC_OK) { zc_hip_store_destroy(s.release()); return status; }
    *out = s.release();
    return ZC_OK;
}
zc_status zc_hip_store_destroy(zc_hip_store* s) {
    if (!s) return ZC_OK;
    if (s->ctx) {
        if (s->side) { (void)hipStreamSynchronize(s->side); }
        for (hipEvent_t e : s->filled) (void)hipEventDestroy(e);
        for (hipEvent_t e : s->released) (void)hipEventDestroy(e);
        if (s->side) (void)hipStreamDestroy(s->side);
        if (s->pool) zc_hip_free(s->ctx, s->pool);
        for (uint8_t* h : s->owned_homes) zc_hip_free(s->ctx, h);
        if (s->table) zc_hip_free(s->ctx, s->table);
        if (s->mirror) zc_hip_free(s->ctx, s->mirror);
    } else {
        delete[] s->pool; for (uint8_t* h : s->owned_homes) delete[] h; delete[] s->mirror;
    }
    delete s;
    return ZC_OK;
}
void* zc_hip_store_backing(zc_hip_store* s, uint32_t layer, uint32_t expert) {
    if (!s || layer >= s->layers || expert >= s->experts) return nullptr;
    return home_of(s, key_of(s, layer, expert));
}
uint64_t zc_hip_store_stride(const zc_hip_store* s) { return s ? s->stride : 0; }
uint64_t zc_hip_store_capacity(const zc_hip_store* s) { return s ? s->cache->capacity() : 0; }
uint64_t zc_hip_store_occupancy(const zc_hip_store* s) { return s ? s->cache->occupancy() : 0; }

zc_status zc_hip_store_acquire(zc_hip_store* s, uint32_t layer, uint32_t expert, zc_store_lease* out) {
    if (!s || !out) return zc_fail(ZC_INVALID_ARGUMENT, "null argument");
    if (layer >= s->layers || expert >= s->experts) return zc_fail(ZC_OUT_OF_RANGE, "invalid expert id");
    return guarded([&] {
        const auto lease = s->cache->acquire(key_of(s, layer, expert));
        if (lease.acquisition == zc::SlotCache::NewMiss) ++s->layer_misses[layer]; else ++s->layer_hits[layer];
        out->lease = lease.slot; out->record = s->pool + lease.slot * s->stride; out->acquisition = int32_t(lease.acquisition);
        return ZC_OK;
    });
}
zc_status zc_hip_store_wait(zc_hip_store* s, uint64_t lease) {
    if (!s || lease >= s->cache->capacity() || !s->cache->pins(lease)) return zc_fail(ZC_LOGIC_ERROR, "empty expert lease");
    return guarded([&] {
        if (s->ctx) ZC_STORE_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(zc_hip_stream(s->ctx)), s->filled[lease], 0));
        else if (s->pending[lease] != kNone) {
            if (s->held.count(s->pending[lease])) throw std::logic_error("waiting for a fill that the test still holds");
            finish_host_fill(s, lease);
        }
        return ZC_OK;
    });
}
zc_status zc_hip_store_release(zc_hip_store* s, uint64_t lease) {
    if (!s) return zc_fail(ZC_INVALID_ARGUMENT, "null argument");
    return guarded([&] {
        s->cache->release(lease);
        // Everything enqueued on the context's stream so far may read the slot; whatever refills it waits for this point.
        if (s->ctx) ZC_STORE_HIP(hipEventRecord(s->released[lease], static_cast<hipStream_t>(zc_hip_stream(s->ctx))));
        return ZC_OK;
    });
}
zc_status zc_hip_store_prefetch(zc_hip_store* s, uint32_t layer, uint32_t expert, int* issued) {
    if (!s) return zc_fail(ZC_INVALID_ARGUMENT, "null argument");
    if (layer >= s->layers || expert >= s->experts) return zc_fail(ZC_OUT_OF_RANGE, "invalid expert id");
    return guarded([&] { const bool did = s->cache->prefetch(key_of(s, layer, expert)); if (issued) *issued = did; return ZC_OK; });
}
int zc_hip_store_ready(zc_hip_store* s, uint32_t layer, uint32_t expert) {
    if (!s || layer >= s->layers || expert >= s->experts) return 0;
    try { return s->cache->ready(key_of(s, layer, expert)) ? 1 : 0; } catch (...) { return 0; }
}
zc_status zc_hip_store_clear(zc_hip_store* s) {
    if (!s) return zc_fail(ZC_INVALID_ARGUMENT, "null argument");
    return guarded([&] { s->cache->clear(); table_rebuild(s); return ZC_OK; });
}
zc_status zc_hip_store_resize(zc_hip_store* s, uint64_t slots) {
    if (!s) return zc_fail(ZC_INVALID_ARGUMENT, "null argument");
    return guarded([&] {
        if (!slots) throw std::invalid_argument("empty expert cache");
        if (s->cache->leased()) throw std::logic_error("cannot resize leased expert slots");   // before any storage moves
        const uint64_t before = s->cache->capacity();
        if (slots > before) { provide_pool(s, slots, before); s->cache->resize(slots); }   // grow: storage first
        else { s->cache->resize(slots); if (slots < before) provide_pool(s, slots, slots); }   // shrink: survivors are compacted to the front first
        table_rebuild(s);
        return ZC_OK;
    });
}
zc_status zc_hip_store_stats(const zc_hip_store* s, zc_store_stats* out) {
    if (!s || !out) return zc_fail(ZC_INVALID_ARGUMENT, "null argument");
    const auto& c = s->cache->stats();
    *out = zc_store_stats{c.hits, c.misses, c.evictions, c.bytes, c.ready_hits, c.loading_joins, c.prefetches, c.prefetch_claims, c.prefetch_unclaimed};
    return ZC_OK;
}
const char* zc_hip_store_policy(const zc_hip_store* s) { return s && s->cache->policy() == zc::SlotCache::SegmentedLRU ? "slru" : "clock"; }
uint64_t zc_hip_store_protected_entries(const zc_hip_store* s) { return s ? s->cache->protected_entries() : 0; }
zc_status zc_hip_store_layer_stats(const zc_hip_store* s, uint32_t layer, uint64_t* hits, uint64_t* misses) {
    if (!s || layer >= s->layers) return zc_fail(ZC_OUT_OF_RANGE, "invalid layer");
    if (hits) *hits = s->layer_hits[layer];
    if (misses) *misses = s->layer_misses[layer];
    return ZC_OK;
}
// ---- the device-side view
zc_status zc_hip_store_table(zc_hip_store* s, const void* const** table) {
    if (!s || !table) return zc_fail(ZC_INVALID_ARGUMENT, "null argument");
    return guarded([&] {
        if (!s->mirror) {
            if (s->cache->occupancy()) throw std::logic_error("the record table must be created while the store is empty");
            const uint64_t records = uint64_t(s->layers) * s->experts;
            if (s->ctx) {
                void* p = nullptr;
                if (zc_hip_alloc_host(s->ctx, records * sizeof(void*), &p) != ZC_OK) throw std::runtime_error(zc_hip_last_error());
                s->mirror = static_cast<const uint8_t**>(p);
                if (zc_hip_alloc(s->ctx, records * sizeof(void*), &p) != ZC_OK) throw std::runtime_error(zc_hip_last_error());
                s->table = static_cast<const uint8_t**>(p);
            } else {
                s->mirror = new const uint8_t*[records];
                s->table = s->mirror;   // host-memory store: one copy serves both
            }
            for (uint64_t key = 0; key < records; ++key) s->mirror[key] = home_of(s, key);
            s->shown.assign(s->cache->capacity(), kNone); s->arriving.assign(s->cache->capacity(), kNone);
            s->table_changed = true;
        }
        *table = reinterpret_cast<const void* const*>(s->table);
        return ZC_OK;
    });
}
static zc_status table_refresh(zc_hip_store* s, bool join) {
    if (!s || !s->mirror) return zc_fail(ZC_LOGIC_ERROR, "the store has no record table");
    return guarded([&] {
        size_t kept = 0;
        for (const size_t slot : s->in_flight) {
            const uint64_t key = s->arriving[slot];
            bool done = s->ctx ? hipEventQuery(s->filled[slot]) == hipSuccess : s->pending[slot] == kNone;
            if (!done && join && s->cache->key_of(slot) == int64_t(key)) {
                // ExpertCache::acquire's "loading join" for a whole launch: what the context's stream runs next waits, on the
                // device, for the fill; the entry can point at the slot at once
                if (s->ctx) ZC_STORE_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(zc_hip_stream(s->ctx)), s->filled[slot], 0));
                else {
                    if (s->held.count(s->pending[slot])) throw std::logic_error("waiting for a fill that the test still holds");
                    finish_host_fill(s, slot);
                }
                done = true; ++s->seen.joined;
            }
            if (!done) { s->in_flight[kept++] = slot; continue; }
            s->arriving[slot] = kNone;
            if (s->cache->key_of(slot) != int64_t(key)) continue;   // replaced before it was ever shown
            s->mirror[key] = s->pool + slot * s->stride; s->shown[slot] = key; s->table_changed = true; ++s->seen.switched;
        }
        s->in_flight.resize(kept);
        if (s->table_changed && s->ctx)
            ZC_STORE_HIP(hipMemcpyAsync(s->table, s->mirror, uint64_t(s->layers) * s->experts * sizeof(void*), hipMemcpyHostToDevice,
                                        static_cast<hipStream_t>(zc_hip_stream(s->ctx))));
        s->table_changed = false;
        return ZC_OK;
    });
}
zc_status zc_hip_store_table_refresh(zc_hip_store* s) { return table_refresh(s, false); }
zc_status zc_hip_store_table_refresh_joining(zc_hip_store* s) { return table_refresh(s, true); }
// What one finished launch read: per layer the distinct valid experts, each classified by what the table showed AT THE LAUNCH
// (nothing below has changed it yet).  First every record that was read from a slot is leased, then the records read from
// home are admitted, then all leases go: a miss can only take the slot of a record that this launch did not use.
static zc_status observe_layers(zc_hip_store* s, uint32_t first_layer, uint32_t layers, const int32_t* ids, uint32_t per_layer) {
    return guarded([&] {
        std::vector<std::pair<uint64_t, uint32_t>> from_slots, from_home;   // (key, layer)
        std::vector<int32_t> distinct;
        for (uint32_t l = 0; l < layers; ++l) {
            distinct.assign(ids + uint64_t(l) * per_layer, ids + uint64_t(l + 1) * per_layer);
            std::sort(distinct.begin(), distinct.end());
            distinct.erase(std::unique(distinct.begin(), distinct.end()), distinct.end());
            for (const int32_t e : distinct) {
                if (e == -1) continue;   // the router's padding for a row with fewer finite logits than picks: no record was read
                if (e < 0 || uint32_t(e) >= s->experts) throw std::out_of_range("invalid expert id");
                const uint64_t key = key_of(s, first_layer + l, uint32_t(e));
                const uint8_t* at = s->mirror[key];
                const bool slot = at >= s->pool && at < s->pool + s->cache->capacity() * s->stride;
                (slot ? from_slots : from_home).push_back({key, first_layer + l});
            }
        }
        s->seen.reads += from_slots.size() + from_home.size();
        s->seen.slot_reads += from_slots.size();
        s->seen.home_reads += from_home.size(); s->seen.home_read_bytes += from_home.size() * s->record_bytes;
        // ExpertCache::acquire's hit for everything that was read from a slot; the leases stay out while the misses are admitted, so
        // that a victim is never a record this launch used, whatever the policy's own preferences
        struct Held {   // whatever happens below, no lease stays out
            zc::SlotCache* cache; std::vector<size_t> slots;
            ~Held() { for (const size_t slot : slots) { try { cache->release(slot); } catch (...) {} } }
        } leases{s->cache.get(), {}};
        std::vector<size_t>& held = leases.slots;
        held.reserve(from_slots.size() + from_home.size());
        for (const auto& [key, layer] : from_slots) {
            held.push_back(s->cache->acquire(key).slot);
            ++s->layer_hits[layer];
        }
        for (const auto& [key, layer] : from_home) {   // acquire's miss (or a join to a fill still in flight): the fill serves later launches
            zc::SlotCache::Lease lease{};
            try { lease = s->cache->acquire(key); }
            catch (const std::runtime_error&) { ++s->seen.not_admitted; continue; }   // no slot to take (all used by this launch, or loading): the record stays at home
            if (lease.acquisition == zc::SlotCache::NewMiss) ++s->layer_misses[layer]; else ++s->layer_hits[layer];
            held.push_back(lease.slot);
        }
        return ZC_OK;
    });
}
zc_status zc_hip_store_table_observe(zc_hip_store* s, uint32_t layer, const int32_t* ids, uint32_t count) {
    if (!s || !s->mirror) return zc_fail(ZC_LOGIC_ERROR, "the store has no record table");
    if (layer >= s->layers || (!ids && count)) return zc_fail(ZC_OUT_OF_RANGE, "invalid layer");
    return observe_layers(s, layer, 1, ids, count);
}
zc_status zc_hip_store_table_observe_layers(zc_hip_store* s, const int32_t* ids, uint32_t per_layer) {
    if (!s || !s->mirror) return zc_fail(ZC_LOGIC_ERROR, "the store has no record table");
    if (!ids && per_layer) return zc_fail(ZC_INVALID_ARGUMENT, "null argument");
    return observe_layers(s, 0, s->layers, ids, per_layer);
}
zc_status zc_hip_store_table_stats(const zc_hip_store* s, zc_store_table_stats* out) {
    if (!s || !out) return zc_fail(ZC_INVALID_ARGUMENT, "null argument");
    *out = s->seen;
    return ZC_OK;
}
zc_status zc_hip_store_geometry(const zc_hip_store* s, uint32_t* layers, uint32_t* experts, uint64_t* record_bytes) {
    if (!s) return zc_fail(ZC_INVALID_ARGUMENT, "null argument");
    if (layers) *layers = s->layers;
    if (experts) *experts = s->experts;
    if (record_bytes) *record_bytes = s->record_bytes;
    return ZC_OK;
}

zc_status zc_hip_store_hold(zc_hip_store* s, uint32_t layer, uint32_t expert, int hold) {
    if (!s || s->ctx) return zc_fail(ZC_LOGIC_ERROR, "fills can only be held in a store without a context");
    if (layer >= s->layers || expert >= s->experts) return zc_fail(ZC_OUT_OF_RANGE, "invalid expert id");
    const uint64_t key = key_of(s, layer, expert);
    if (hold) s->held.insert(key);
    else {
        s->held.erase(key);
        for (size_t slot = 0; slot < s->pending.size(); ++slot) if (s->pending[slot] == key) finish_host_fill(s, slot);
    }
    return ZC_OK;
}

}  // extern "C"
