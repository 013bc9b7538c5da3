"""Slot-cache policy of the expert store, on a store with host-memory slots (no GPU): the reference's cache tests
(tests/test_qwen.cpp:93-100, 336-348, 415-430) restated through the C ABI, plus the prefetch rules of
ExpertCache::prefetch (src/engine/storage.cpp:677-692)."""
import numpy as np
import pytest
import zerocool_amd as z

RECORD = 128


def make(slots, layers=2, experts=512):
    s = z.Store(None, layers, experts, RECORD, slots)
    return s


def put(s, layer, expert):
    s.backing(layer, expert)[:] = np.frombuffer(np.full(RECORD // 4, float(layer * s.experts + expert), np.float32).tobytes(), np.uint8)


def value(s, lease):
    return float(s.slot_bytes(lease).view(np.float32)[0])


def use(s, layer, expert):
    put(s, layer, expert)
    lease = s.acquire(layer, expert)
    s.wait(lease)
    v = value(s, lease)
    s.release(lease)
    return v


def test_clock_leases_protect_in_flight_data():   # test_qwen.cpp:336-348
    s = make(2)
    put(s, 0, 1); put(s, 0, 2); put(s, 0, 3)
    a, b = s.acquire(0, 1), s.acquire(0, 2)
    s.wait(a); s.wait(b)
    assert value(s, a) == 1 and value(s, b) == 2
    with pytest.raises(z.ZcError) as err:
        s.acquire(0, 3)
    assert "exhausted by outstanding leases" in str(err.value)
    with pytest.raises(z.ZcError):
        s.clear()
    with pytest.raises(z.ZcError):
        s.resize(4)
    s.release(b)
    c = s.acquire(0, 3); s.wait(c)
    assert value(s, c) == 3 and value(s, a) == 1
    hit = s.acquire(0, 1)
    assert hit.record == a.record and hit.acquisition == 1
    for lease in (hit, a, c):
        s.release(lease)
    s.resize(4)
    for i in range(32):
        assert use(s, 1, i % 8) == 512 + i % 8
    assert s.stats().evictions > 0
    with pytest.raises(z.ZcError):
        s.release(a)   # released twice
    s.close()


def test_resizing_preserves_survivors_and_refuses_leases():   # test_qwen.cpp:93-100
    s = make(64)
    for i in range(64):
        use(s, 0, i)
    assert s.occupancy == 64
    lease = s.acquire(0, 63)
    with pytest.raises(z.ZcError):
        s.resize(32)
    assert s.capacity == 64
    s.release(lease)
    s.resize(32)
    assert s.capacity == 32 and s.occupancy == 32 and s.stats().evictions == 32
    assert s.ready(0, 63)
    misses = s.stats().misses
    assert use(s, 0, 63) == 63 and s.stats().misses == misses   # a survivor keeps its bytes: a hit, not a reload
    s.close()


def test_loading_joins_count_separately():   # test_qwen.cpp:415-430
    s = make(3)
    put(s, 0, 0)
    s.hold(0, 0)
    a = s.acquire(0, 0)
    join = s.acquire(0, 0)
    st = s.stats()
    assert st.loading_joins == 1 and st.ready_hits == 0 and a.acquisition == 0 and join.acquisition == 2
    assert not s.ready(0, 0)
    with pytest.raises(z.ZcError):
        s.wait(a)           # (a held fill cannot finish; the reference would block here)
    s.hold(0, 0, False)
    s.wait(a); s.wait(join)
    assert a.record == join.record and value(s, a) == 0
    s.release(a); s.release(join)
    use(s, 0, 1); use(s, 0, 2)
    s.resize(2)
    assert s.stats().evictions == 1
    assert sum(s.ready(0, e) for e in range(3)) == 2
    before = s.stats().misses
    s.resize(4)
    for e in range(3):
        if s.ready(0, e):
            assert use(s, 0, e) == e
    assert s.stats().misses == before
    s.close()


def test_loading_slots_are_never_victims():
    s = make(2)
    put(s, 0, 0); put(s, 0, 1); put(s, 0, 2)
    s.hold(0, 0)
    a = s.acquire(0, 0)
    s.release(a)                       # lease gone, but the fill is still in flight: the slot must not be taken
    use(s, 0, 1)
    assert use(s, 0, 2) == 2           # takes the slot of expert 1 (finished), not the loading one
    assert not s.ready(0, 1)
    s.hold(0, 0, False)
    hit = s.acquire(0, 0)
    assert hit.acquisition == 1
    s.wait(hit)
    assert value(s, hit) == 0
    s.release(hit)
    s.close()


def test_prefetch_rules():   # storage.cpp:677-692
    s = make(2)
    for e in range(4):
        put(s, 0, e)
    assert s.prefetch(0, 0) is True
    assert s.prefetch(0, 0) is False                 # present
    st = s.stats()
    assert st.prefetches == 1 and st.misses == 0
    claimed = s.acquire(0, 0)                        # demand claims the guess: a hit
    st = s.stats()
    assert claimed.acquisition == 1 and st.prefetch_claims == 1 and st.hits == 1
    other = s.acquire(0, 1)
    assert s.prefetch(0, 2) is False                 # both slots pinned: a guess never evicts a lease
    s.hold(0, 2)
    s.release(other)
    assert s.prefetch(0, 2) is True                  # takes the unpinned, finished slot ...
    assert s.prefetch(0, 3) is False                 # ... and now one slot is pinned, the other still loading: nothing to take
    s.hold(0, 2, False)
    s.release(claimed)
    s.close()


def test_unclaimed_guess_is_the_next_victim():
    s = make(3)
    for e in range(4):
        put(s, 0, e)
    use(s, 0, 0); use(s, 0, 1)
    assert s.prefetch(0, 2) is True                  # into the free slot, born unreferenced
    assert use(s, 0, 3) == 3                         # the sweep gives 0 and 1 their second chance and takes the guess
    st = s.stats()
    assert st.prefetch_unclaimed == 1 and st.evictions == 1
    assert s.ready(0, 0) and s.ready(0, 1) and s.ready(0, 3) and not s.ready(0, 2)
    s.close()


def test_admission_waits_for_a_loading_guess():   # storage.cpp:650-658
    s = make(1)
    put(s, 0, 0); put(s, 0, 1)
    assert s.prefetch(0, 0) is True                  # the only slot holds a guess whose fill has finished
    lease = s.acquire(0, 1)                          # demand for another record takes it
    s.wait(lease)
    assert value(s, lease) == 1 and s.stats().prefetch_unclaimed == 1
    s.release(lease)
    s.close()


def test_ids_are_checked():
    s = make(2, layers=1, experts=4)
    with pytest.raises(z.ZcError) as err:
        s.acquire(0, 4)
    assert "invalid expert id" in str(err.value)
    with pytest.raises(z.ZcError):
        s.prefetch(1, 0)
    with pytest.raises(z.ZcError):
        z.Store(None, 1, 4, RECORD, 0)
    assert s.layer_stats(0) == (0, 0)
    s.close()


def test_record_table_shows_a_slot_only_while_it_holds_the_finished_record():
    # The device-side view (zc_hip_store_table): entries start at the records' homes, move to a slot when the slot's fill has
    # finished and a refresh has run, and go back home the moment the slot is given to another record.
    import ctypes as C
    s = make(3, layers=2, experts=8)
    for layer in range(2):
        for e in range(8):
            put(s, layer, e)
    homes = np.array([s.lib.zc_hip_store_backing(s.handle, l, e) for l in range(2) for e in range(8)], np.uint64)
    table = s.table_entries()
    assert (table == homes).all()

    def shown_value(key):   # what a kernel would read as the record's first float
        return float(np.ctypeslib.as_array(C.cast(int(table[key]), C.POINTER(C.c_float)), shape=(1,))[0])

    def check_every_entry():
        for key in range(16):
            assert shown_value(key) == key

    s.table_observe(0, [1, 2, 2, 1])            # two distinct records, both read from home; their fills start
    st = s.table_stats()
    assert (st.reads, st.slot_reads, st.home_reads, st.home_read_bytes) == (2, 0, 2, 2 * RECORD)
    assert (table == homes).all()               # nothing moves before a refresh
    s.table_refresh()
    assert table[1] != homes[1] and table[2] != homes[2] and s.table_stats().switched == 2
    check_every_entry()
    s.table_observe(0, [1, 2])
    st = s.table_stats()
    assert (st.reads, st.slot_reads, st.home_reads) == (4, 2, 2)
    assert s.stats().hits == 2 and s.stats().misses == 2

    s.hold(1, 3)                                # a slow fill: the entry stays at home until it has finished
    s.table_observe(1, [3])
    s.table_refresh()
    assert table[8 + 3] == homes[8 + 3]
    s.table_observe(1, [3])                     # read from home again, joined to the fill in flight: no second fill
    assert s.stats().loading_joins == 1 and s.stats().misses == 3
    s.hold(1, 3, False)
    s.table_refresh()
    assert table[8 + 3] != homes[8 + 3]
    check_every_entry()

    # The joining refresh (the "loading join" of a whole launch): the entry of a fill still in flight moves to its slot at
    # once and the fill is waited for -- on a GPU by the stream, here by finishing it; a fill that the test still holds
    # cannot be joined.
    s.hold(1, 5)
    s.table_observe(1, [5])
    s.table_refresh()
    assert table[8 + 5] == homes[8 + 5]
    with pytest.raises(z.ZcError):
        s.table_refresh_joining()
    s.hold(1, 5, False)                        # (letting go of the hold finishes the fill)
    s.hold(1, 6)
    s.table_observe(1, [6])
    s.hold(1, 6, False)
    before = s.table_stats()
    s.table_refresh_joining()
    after = s.table_stats()
    assert table[8 + 5] != homes[8 + 5] and table[8 + 6] != homes[8 + 6] and after.switched == before.switched + 2
    check_every_entry()
    s.table_observe_layers(np.array([[-1, -1], [5, -1]], np.int32))   # the router's padding id is no record
    assert s.table_stats().reads == after.reads + 1

    s.table_observe(0, [4, 5, 6])               # three slots, three more records: earlier ones lose their slots at once
    assert sum(table[k] != homes[k] for k in range(16)) <= 3
    check_every_entry()                         # entries of evicted records are back at home before the slot is overwritten
    s.table_refresh()
    check_every_entry()
    assert s.stats().evictions >= 3
    s.resize(5)
    check_every_entry()
    s.clear()
    assert (table == homes).all()
    with pytest.raises(z.ZcError):
        s.table_observe(0, [8])
    s.close()


def test_record_table_must_be_created_on_an_empty_store():
    s = make(2)
    use(s, 0, 1)
    with pytest.raises(z.ZcError) as err:
        s.table()
    assert "while the store is empty" in str(err.value)
    with pytest.raises(z.ZcError):
        s.table_refresh()
    s.close()


def make_slru(slots, layers=1, experts=16):
    return z.Store(None, layers, experts, RECORD, slots, policy="slru")


def test_slru_matches_an_independent_probation_protected_replay():   # test_qwen.cpp:334-367
    with pytest.raises(z.ZcError) as err:
        z.Store(None, 1, 16, RECORD, 4, policy="adaptive")
    assert "cache policy must be clock or slru" in str(err.value)
    assert make(2).policy == "clock"
    for capacity in range(1, 9):
        s = make_slru(capacity)
        assert s.policy == "slru"
        for e in range(12):
            put(s, 0, e)
        probation, protected, random = [], [], 1234
        for step in range(300):
            random = (random * 1664525 + 1013904223) & 0xffffffff
            key = (random >> 16) % 12
            hit = key in probation or key in protected
            if hit:
                (probation if key in probation else protected).remove(key)
                protected.append(key)
                if len(protected) > capacity * 3 // 4:
                    probation.append(protected.pop(0))
            else:
                if len(probation) + len(protected) == capacity:
                    probation.pop(0)
                probation.append(key)
            before = s.stats()
            hits0, misses0 = before.hits, before.misses
            lease = s.acquire(0, key); s.wait(lease)
            assert value(s, lease) == key
            s.release(lease)
            after = s.stats()
            assert after.hits - hits0 == int(hit) and after.misses - misses0 == int(not hit), (capacity, step)
            assert s.protected_entries == len(protected), (capacity, step)
            for e in range(12):
                assert s.ready(0, e) == (e in probation or e in protected), (capacity, step, e)
        assert s.occupancy == min(capacity, 12)
        s.clear()
        assert s.protected_entries == 0 and s.occupancy == 0
        s.close()


def test_slru_protects_loading_and_leased_slots_and_survives_resizing():   # test_qwen.cpp:368-391
    s = make_slru(4)
    for e in range(10):
        put(s, 0, e)
    for e in range(4):
        use(s, 0, e)
    for e in range(3):
        use(s, 0, e)                       # protected: 0, 1, 2; probation: 3
    s.hold(0, 4)
    pending = s.acquire(0, 4)              # takes probation's 3; its fill stays in flight
    assert pending.acquisition == 0 and not s.ready(0, 3)
    use(s, 0, 5)                           # probation is busy: an eligible protected entry goes
    assert not s.ready(0, 0)
    join = s.acquire(0, 4)
    assert join.acquisition == 2 and s.stats().loading_joins == 1
    s.release(pending); s.release(join)    # the leases go while the read is still active: loading data cannot be overwritten
    a, b, c = s.acquire(0, 1), s.acquire(0, 2), s.acquire(0, 5)
    with pytest.raises(z.ZcError):
        s.acquire(0, 6)
    with pytest.raises(z.ZcError):
        s.resize(2)
    with pytest.raises(z.ZcError):
        s.clear()
    assert not s.prefetch(0, 7)            # segmented LRU takes no prefetches (storage.cpp:679)
    s.hold(0, 4, False)
    lease = s.acquire(0, 4); s.wait(lease)
    assert value(s, lease) == 4
    for l in (lease, a, b, c):
        s.release(l)
    s.resize(2)
    assert s.occupancy == 2 and s.protected_entries <= 1
    survivors = [e for e in range(6) if s.ready(0, e)]
    misses = s.stats().misses
    s.resize(8)
    for e in survivors:
        assert use(s, 0, e) == e
    assert s.stats().misses == misses
    s.clear()
    use(s, 0, 9)
    assert s.occupancy == 1
    s.close()


def test_layers_can_share_their_records_homes():
    # Fewer homes than layers: layer l's records live in home l mod home_layers, the cache still tells the layers apart.
    s = z.Store(None, 4, 8, RECORD, 3, home_layers=2)
    home = lambda l, e: s.lib.zc_hip_store_backing(s.handle, l, e)
    assert home(0, 5) == home(2, 5) and home(1, 5) == home(3, 5) and home(0, 5) != home(1, 5)
    put(s, 0, 5)                                   # also what layer 2 reads
    assert use(s, 0, 5) == 5.0
    lease = s.acquire(2, 5); s.wait(lease)
    assert lease.acquisition == 0 and value(s, lease) == 5.0   # a miss of its own, the same bytes
    s.release(lease)
    assert s.stats().misses == 2 and s.occupancy == 2
    with pytest.raises(z.ZcError):
        z.Store(None, 4, 8, RECORD, 3, home_layers=5)
    s.close()


def test_a_launch_never_loses_a_record_it_used_to_its_own_misses():
    # Twelve slots that hold a launch's twelve records; the next launch uses eleven of them and one new record.  The records
    # read from slots are touched before the new one is admitted, so the victim is the one record this launch did not use --
    # whatever the order of the ids, and across layers when a launch reports all its layers at once.
    s = z.Store(None, 2, 32, RECORD, 12)
    for l in range(2):
        for e in range(32):
            put(s, l, e)
    s.table()
    first = np.array([[0, 1, 2, 3, 4, 5], [10, 11, 12, 13, 14, 15]], np.int32)
    s.table_observe_layers(first); s.table_refresh()
    assert s.table_stats().home_reads == 12
    second = np.array([[20, 0, 1, 2, 3, 4], [10, 11, 12, 13, 14, 15]], np.int32)   # the new record comes FIRST in the list
    s.table_observe_layers(second); s.table_refresh()
    st = s.table_stats()
    assert (st.slot_reads, st.home_reads) == (11, 13)
    assert not s.ready(0, 5) and all(s.ready(0, e) for e in (20, 0, 1, 2, 3, 4)) and all(s.ready(1, e) for e in range(10, 16))
    s.table_observe_layers(second)
    assert s.table_stats().slot_reads == 23 and s.stats().evictions == 1
    with pytest.raises(z.ZcError):
        s.table_observe_layers(np.array([[0], [32]], np.int32))
    s.close()
