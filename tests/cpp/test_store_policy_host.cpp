// Host-only harness over the slot cache policy (zerocool_amd/csrc/zc_store.hpp), meant to be built with
// -fsanitize=address,undefined (make asan): long random runs of acquire / release / prefetch / resize / clear under both
// replacement policies, with fills that finish late, checked against the rules the reference states for its cache
// (include/engine/storage.hpp:198-269, src/engine/storage.cpp:525-725):
//   * a victim is never a leased slot and never a slot whose fill has not finished
//   * acquire fails only when no slot can be taken; release of an unleased slot is a logic error
//   * every key maps to at most one slot, occupancy never exceeds capacity, counters add up
//   * resize keeps the survivors' bytes (a survivor's slot still holds its own key's fill)
#include "../../zerocool_amd/csrc/zc_store.hpp"
#include <cstdio>
#include <map>
#include <random>
#include <set>

static int checks = 0, failures = 0;
#define CHECK(cond) do { ++checks; if (!(cond)) { ++failures; std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); } } while (0)

struct Transport {   // what the hooks see: which key's bytes a slot holds and whether its fill has finished
    std::vector<int64_t> holds; std::vector<int> pending;   // pending[slot] > 0: fill finishes after that many polls
    std::mt19937 rng{99};
    zc::SlotCache::Hooks hooks() {
        zc::SlotCache::Hooks h;
        h.start = [this](size_t slot, uint64_t key) { grow(slot); holds[slot] = int64_t(key); pending[slot] = int(rng() % 4); };
        h.done = [this](size_t slot) { grow(slot); if (pending[slot] > 0) --pending[slot]; return pending[slot] == 0; };
        h.wait = [this](size_t slot) { grow(slot); pending[slot] = 0; };
        h.move = [this](size_t from, size_t to) { grow(from); grow(to); holds[to] = holds[from]; pending[to] = 0; };
        return h;
    }
    void grow(size_t slot) { if (slot >= holds.size()) { holds.resize(slot + 1, -1); pending.resize(slot + 1, 0); } }
};

static void run(zc::SlotCache::Policy policy, unsigned seed, size_t slots, uint64_t keys, int steps) {
    Transport t;
    zc::SlotCache cache(slots, 4096, t.hooks(), policy);
    std::mt19937 rng(seed);
    std::multiset<size_t> leases;               // slots this harness holds leases on
    std::map<size_t, uint64_t> leased_key;      // and the key each one was taken for
    uint64_t acquires = 0;
    for (int step = 0; step < steps; ++step) {
        const unsigned op = rng() % 100;
        if (op < 55) {
            const uint64_t key = rng() % keys;
            try {
                const auto lease = cache.acquire(key);
                ++acquires;
                CHECK(lease.slot < cache.capacity() && cache.key_of(lease.slot) == int64_t(key));
                CHECK(t.holds[lease.slot] == int64_t(key));                      // the slot was filled for this key
                if (leased_key.count(lease.slot)) CHECK(leased_key[lease.slot] == key);   // a leased slot was not taken for another key
                leases.insert(lease.slot); leased_key[lease.slot] = key;
            } catch (const std::runtime_error&) {
                // allowed only when nothing can be taken: every slot is leased, or unleased ones are still loading
                size_t free_now = 0;
                for (size_t s = 0; s < cache.capacity(); ++s) if (cache.key_of(s) < 0 || (!cache.pins(s) && t.pending[s] == 0)) ++free_now;
                CHECK(free_now == 0 || policy == zc::SlotCache::Clock);          // CLOCK may also give up after its bounded sweep
            }
        } else if (op < 85 && !leases.empty()) {
            auto it = leases.begin(); std::advance(it, rng() % leases.size());
            const size_t slot = *it; leases.erase(it);
            cache.release(slot);
            if (!leases.count(slot)) leased_key.erase(slot);
        } else if (op < 93) {
            const uint64_t key = rng() % keys;
            const bool was_in = cache.ready(key) || [&] { for (size_t s = 0; s < cache.capacity(); ++s) if (cache.key_of(s) == int64_t(key)) return true; return false; }();
            const bool issued = cache.prefetch(key);
            if (policy == zc::SlotCache::SegmentedLRU || was_in) CHECK(!issued);
        } else if (op < 97 && leases.empty()) {
            const size_t to = 1 + rng() % (2 * slots);
            std::map<int64_t, bool> before;
            for (size_t s = 0; s < cache.capacity(); ++s) if (cache.key_of(s) >= 0) before[cache.key_of(s)] = true;
            cache.resize(to);
            CHECK(cache.capacity() == to && cache.occupancy() <= to);
            for (size_t s = 0; s < cache.capacity(); ++s) if (cache.key_of(s) >= 0) {
                CHECK(before.count(cache.key_of(s)));                            // survivors only, nothing invented
                CHECK(t.holds[s] == cache.key_of(s));                            // and their bytes came along
            }
        } else if (leases.empty()) {
            cache.clear();
            CHECK(cache.occupancy() == 0);
        } else {
            bool refused = false;
            try { cache.clear(); } catch (const std::logic_error&) { refused = true; }
            CHECK(refused);
            refused = false;
            try { cache.resize(cache.capacity() + 1); } catch (const std::logic_error&) { refused = true; }
            CHECK(refused);
        }
        // invariants after every step
        std::set<int64_t> seen; size_t used = 0;
        for (size_t s = 0; s < cache.capacity(); ++s) {
            const int64_t key = cache.key_of(s);
            if (key < 0) { CHECK(cache.pins(s) == 0); continue; }
            ++used; CHECK(seen.insert(key).second);
            CHECK(cache.pins(s) == leases.count(s));
        }
        CHECK(used == cache.occupancy() && used <= cache.capacity());
        if (policy == zc::SlotCache::SegmentedLRU) {
            CHECK(cache.probation_entries() + cache.protected_entries() == used);
            CHECK(cache.protected_entries() <= 3 * cache.capacity() / 4);
        }
        const auto& st = cache.stats();
        CHECK(st.hits + st.misses == acquires && st.ready_hits + st.loading_joins == st.hits);
        CHECK(st.prefetch_claims + st.prefetch_unclaimed <= st.prefetches);
        CHECK(st.bytes == (st.misses + st.prefetches) * 4096);
    }
    while (!leases.empty()) { cache.release(*leases.begin()); leases.erase(leases.begin()); }
    bool twice = false;
    try { cache.release(0); } catch (const std::logic_error&) { twice = true; }
    CHECK(twice);
}

int main() {
    for (unsigned seed = 1; seed <= 6; ++seed) {
        run(zc::SlotCache::Clock, seed, 1 + seed % 5 * 3, 40, 6000);
        run(zc::SlotCache::SegmentedLRU, seed + 100, 2 + seed % 4 * 4, 40, 6000);
    }
    bool refused = false;
    try { Transport t; zc::SlotCache none(0, 16, t.hooks()); } catch (const std::invalid_argument&) { refused = true; }
    CHECK(refused);
    std::printf("%d checks, %d failures\n", checks, failures);
    return failures ? 1 : 0;
}
