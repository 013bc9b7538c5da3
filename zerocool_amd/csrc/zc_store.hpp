// Slot cache policy of the expert store: which record lives in which slot.
//
// The reference streams expert records from SSD into a fixed set of slots (ExpertCache,
// include/engine/storage.hpp:198-269, src/engine/storage.cpp:525-725).  Here the records' home is pinned
// host memory and the slots are HBM; this class keeps the reference's rules and leaves the transport to hooks:
//   * acquire(key): hit (ready or still loading -- a "loading join") or miss; a miss takes a victim by
//     CLOCK second chance and starts a fill.  The returned lease PINS the slot until release().
//   * a victim is never a pinned slot and never a slot whose fill has not finished
//   * prefetch(key): speculative fill into an unpinned, finished slot; the entry is born unreferenced, so an
//     unclaimed guess is the next victim; it never evicts a pinned or loading slot
//   * counters: hits, misses, evictions, bytes, ready_hits, loading_joins, prefetches, prefetch_claims,
//     prefetch_unclaimed (storage.hpp:183-192)
//   * two replacement policies (storage.cpp:536-573): CLOCK second chance (the default), and segmented LRU -- a new
//     record enters a probation queue, a hit moves it to the newest end of a protected queue that holds at most three
//     quarters of the slots (its oldest entry drops back to probation's newest end), the victim is the oldest
//     unpinned, finished entry of probation, then of protected ("a preference, never a pin").  Segmented LRU takes
//     no prefetches, as in the reference.
// One coordinator thread owns the object (storage.hpp:194-197); nothing here is thread safe.
#pragma once
#include <cstdint>
#include <functional>
#include <stdexcept>
#include <unordered_map>
#include <vector>

namespace zc {

struct SlotCacheStats {
    uint64_t hits = 0, misses = 0, evictions = 0, bytes = 0, ready_hits = 0, loading_joins = 0;
    uint64_t prefetches = 0, prefetch_claims = 0, prefetch_unclaimed = 0;
};

class SlotCache {
public:
    struct Hooks {
        std::function<void(size_t slot, uint64_t key)> start;     // begin filling `slot` with the record of `key`
        std::function<bool(size_t slot)> done;                     // has the slot's last fill finished?
        std::function<void(size_t slot)> wait;                     // block the coordinator until it has
        std::function<void(size_t from, size_t to)> move;          // copy a finished slot's bytes (resize compaction)
    };
    enum Acquisition { NewMiss = 0, ReadyHit = 1, LoadingJoin = 2 };
    enum Policy { Clock = 0, SegmentedLRU = 1 };
    struct Lease { size_t slot; Acquisition acquisition; };

    SlotCache(size_t slots, uint64_t record_bytes, Hooks hooks, Policy policy = Clock)
        : slots_(slots), record_bytes_(record_bytes), hooks_(std::move(hooks)), policy_(policy) {
        if (!slots || !record_bytes) throw std::invalid_argument("empty expert cache");
        if (policy != Clock && policy != SegmentedLRU) throw std::invalid_argument("cache policy must be clock or slru");
    }
    Policy policy() const { return policy_; }
    size_t protected_entries() const { return queue_[1].count; }
    size_t probation_entries() const { return policy_ == SegmentedLRU ? queue_[0].count : 0; }
    size_t capacity() const { return slots_.size(); }
    size_t occupancy() const { return lookup_.size(); }
    const SlotCacheStats& stats() const { return stats_; }
    unsigned pins(size_t slot) const { return slots_[slot].pins; }
    bool leased() const { for (const Entry& e : slots_) if (e.used && e.pins) return true; return false; }

    // storage.cpp:628-676
    Lease acquire(uint64_t key) {
        if (auto it = lookup_.find(key); it != lookup_.end()) {
            Entry& e = slots_[it->second];
            touch(it->second); ++stats_.hits;
            const bool ready = hooks_.done(it->second);
            if (ready) ++stats_.ready_hits; else ++stats_.loading_joins;
            if (e.prefetched) { e.prefetched = false; ++stats_.prefetch_claims; }
            ++e.pins;
            return {it->second, ready ? ReadyHit : LoadingJoin};
        }
        size_t selected = slots_.size();
        if (policy_ == SegmentedLRU) {
            if (occupancy() == capacity()) selected = slru_victim();
            else for (size_t trial = 0; trial < slots_.size() && selected == slots_.size(); ++trial) {   // free capacity first
                const size_t slot = hand_; hand_ = (hand_ + 1) % slots_.size();
                if (!slots_[slot].used) selected = slot;
            }
        } else selected = clock_victim();
        while (selected == slots_.size() && policy_ == Clock) {
            // Unclaimed guesses load without a lease.  Wait for one to finish rather than failing an admission
            // that would fit once it does (storage.cpp:650-658).
            size_t guess = slots_.size();
            for (size_t i = 0; i < slots_.size() && guess == slots_.size(); ++i)
                if (slots_[i].used && !slots_[i].pins && slots_[i].prefetched && !hooks_.done(i)) guess = i;
            if (guess == slots_.size()) break;
            hooks_.wait(guess);
            selected = clock_victim();
        }
        if (selected == slots_.size())
            throw std::runtime_error("expert cache exhausted by outstanding leases; finish a batch before acquiring more");
        place(selected, key);
        Entry& e = slots_[selected];
        e.referenced = true; e.prefetched = false; e.pins = 1;
        if (policy_ == SegmentedLRU) link(selected, 0);
        hooks_.start(selected, key);
        ++stats_.misses; stats_.bytes += record_bytes_;
        return {selected, NewMiss};
    }
    void release(size_t slot) {
        if (slot >= slots_.size() || !slots_[slot].pins) throw std::logic_error("expert lease released twice");
        --slots_[slot].pins;
    }
    // storage.cpp:677-692
    bool prefetch(uint64_t key) {
        if (policy_ != Clock || lookup_.count(key)) return false;
        const size_t selected = clock_victim();
        if (selected == slots_.size()) return false;
        place(selected, key);
        Entry& e = slots_[selected];
        e.referenced = false; e.prefetched = true; e.pins = 0;   // unreferenced: an unclaimed guess is the next victim
        hooks_.start(selected, key);
        ++stats_.prefetches; stats_.bytes += record_bytes_;
        return true;
    }
    bool ready(uint64_t key) const {
        const auto it = lookup_.find(key);
        return it != lookup_.end() && hooks_.done(it->second);
    }
    // storage.cpp:697-702
    void clear() {
        for (const Entry& e : slots_) if (e.used && e.pins) throw std::logic_error("cannot clear leased expert slots");
        drain();
        lookup_.clear();
        for (Entry& e : slots_) e = Entry{};
        hand_ = 0; queue_[0] = queue_[1] = Queue{};
    }
    // storage.cpp:708-725: a coordinator boundary; never invalidates a lease or a fill in flight; survivors keep their bytes
    void resize(size_t slots) {
        if (!slots) throw std::invalid_argument("empty expert cache");
        for (const Entry& e : slots_) if (e.used && e.pins) throw std::logic_error("cannot resize leased expert slots");
        drain();
        if (slots >= slots_.size()) { slots_.resize(slots); return; }
        size_t occupied = lookup_.size();
        while (occupied > slots) {
            size_t victim = hand_; hand_ = (hand_ + 1) % slots_.size();
            if (policy_ == SegmentedLRU) victim = slru_victim();   // nothing is pinned or loading here: there always is one
            Entry& e = slots_[victim];
            if (!e.used) continue;
            if (policy_ == Clock && e.referenced) { e.referenced = false; continue; }
            if (e.prefetched) ++stats_.prefetch_unclaimed;
            unlink(victim); lookup_.erase(e.key); e = Entry{}; --occupied; ++stats_.evictions;
        }
        size_t to = 0;
        lookup_.clear();
        for (size_t from = 0; from < slots_.size(); ++from) if (slots_[from].used) {
            if (from != to) { hooks_.move(from, to); relabel(from, to); slots_[to] = slots_[from]; slots_[from] = Entry{}; }
            lookup_[slots_[to].key] = to; ++to;
        }
        drain();
        slots_.resize(slots); hand_ = 0;
        if (policy_ == SegmentedLRU) demote();
    }
    int64_t key_of(size_t slot) const { return slots_[slot].used ? int64_t(slots_[slot].key) : -1; }

private:
    static constexpr size_t kNoSlot = ~size_t(0);
    // A slot's place in the probation (0) or protected (1) queue: links are slot numbers, oldest first.
    struct Entry {
        uint64_t key = 0; unsigned pins = 0; bool used = false, referenced = false, prefetched = false;
        int listed = -1; size_t older = kNoSlot, newer = kNoSlot;
    };
    struct Queue { size_t oldest = kNoSlot, newest = kNoSlot, count = 0; };
    void unlink(size_t slot) {
        Entry& e = slots_[slot];
        if (e.listed < 0) return;
        Queue& q = queue_[e.listed];
        if (e.older != kNoSlot) slots_[e.older].newer = e.newer; else q.oldest = e.newer;
        if (e.newer != kNoSlot) slots_[e.newer].older = e.older; else q.newest = e.older;
        --q.count; e.listed = -1; e.older = e.newer = kNoSlot;
    }
    void link(size_t slot, int which) {
        Entry& e = slots_[slot]; Queue& q = queue_[which];
        e.listed = which; e.older = q.newest; e.newer = kNoSlot;
        if (q.newest != kNoSlot) slots_[q.newest].newer = slot; else q.oldest = slot;
        q.newest = slot; ++q.count;
    }
    void demote() { while (queue_[1].count > 3 * capacity() / 4) { const size_t slot = queue_[1].oldest; unlink(slot); link(slot, 0); } }
    void touch(size_t slot) {   // storage.cpp:563-566
        if (policy_ == Clock) { slots_[slot].referenced = true; return; }
        unlink(slot); link(slot, 1); demote();
    }
    size_t slru_victim() const {   // storage.cpp:567-572
        for (const Queue& q : queue_)
            for (size_t slot = q.oldest; slot != kNoSlot; slot = slots_[slot].newer)
                if (!slots_[slot].pins && hooks_.done(slot)) return slot;
        return slots_.size();
    }
    void relabel(size_t from, size_t to) {   // the entry of slot `from` is about to live in slot `to`: its neighbours and queue ends follow
        const Entry& e = slots_[from];
        if (e.listed < 0) return;
        Queue& q = queue_[e.listed];
        if (e.older != kNoSlot) slots_[e.older].newer = to; else q.oldest = to;
        if (e.newer != kNoSlot) slots_[e.newer].older = to; else q.newest = to;
    }
    void drain() { for (size_t i = 0; i < slots_.size(); ++i) if (slots_[i].used) hooks_.wait(i); }
    void place(size_t slot, uint64_t key) {   // storage.cpp:606-613
        Entry& old = slots_[slot];
        if (old.used) {
            if (old.prefetched) ++stats_.prefetch_unclaimed;
            unlink(slot); lookup_.erase(old.key); ++stats_.evictions;
        }
        old = Entry{}; old.used = true; old.key = key;
        lookup_[key] = slot;
    }
    size_t clock_victim() {   // storage.cpp:614-627
        for (size_t trial = 0; trial < slots_.size() * 2 + 1; ++trial) {
            const size_t slot = hand_; hand_ = (hand_ + 1) % slots_.size();
            Entry& old = slots_[slot];
            if (old.used) {
                if (old.pins) continue;
                if (!hooks_.done(slot)) continue;
                if (old.referenced) { old.referenced = false; continue; }
            }
            return slot;
        }
        return slots_.size();
    }
    std::vector<Entry> slots_;
    std::unordered_map<uint64_t, size_t> lookup_;
    size_t hand_ = 0;
    uint64_t record_bytes_;
    Hooks hooks_;
    Policy policy_ = Clock;
    Queue queue_[2];
    SlotCacheStats stats_;
};

}  // namespace zc
