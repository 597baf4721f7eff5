"""Caching allocator state machine on a host stand-in for the device (no GPU).

Invariants follow the reference's runtime tests:
dipu/tests/python/individual_scripts/test_memory_stats.py:29-45 (allocated == sum of
512-byte-rounded sizes, reserved >= allocated), test_allocator.py:24-74 (byte-granular
sweep), and the allocator's own rules (DIPUCachingDeviceAllocator.cpp:84-95,584-714,833-837)."""
import random

import pytest

MiB = 1 << 20


@pytest.fixture()
def sim(pkg):
    made = []

    def make(capacity=8 << 30, conf="", **kw):
        a = pkg.runtime.SimAllocator(capacity, conf, **kw)
        made.append(a)
        return a

    yield make
    for a in made:
        a.close()


def round512(n):
    return ((n + 511) // 512) * 512 if n > 512 else 512


def test_rounding_and_segment_sizes(pkg):
    rt = pkg.runtime
    assert rt.roundSize(1) == 512 and rt.roundSize(512) == 512 and rt.roundSize(513) == 1024
    assert rt.roundSize(1000000) == 1000448
    assert rt.segmentSize(512) == 2 * MiB and rt.segmentSize(MiB) == 2 * MiB
    assert rt.segmentSize(MiB + 512) == 20 * MiB and rt.segmentSize(10 * MiB - 512) == 20 * MiB
    assert rt.segmentSize(10 * MiB) == 10 * MiB and rt.segmentSize(11 * MiB + 512) == 12 * MiB
    # >= 1 GiB requests get 64 MiB granular segments (large HBM), unless switched off
    assert rt.segmentSize((1 << 30) + 512) == (1 << 30) + 64 * MiB
    assert rt.segmentSize((1 << 30) + 512, "huge_segments:0") == (1 << 30) + 2 * MiB
    # power-of-two divisions: 1200 KiB with 4 divisions -> next multiple of 256 KiB
    assert rt.roundSize(1200 * 1024, "roundup_power2_divisions:4") == 1280 * 1024
    assert rt.roundSize(123, "bogus_option:1") == 0  # unknown option is rejected


def test_byte_sweep_accounting(sim):
    a = sim()
    ptrs, want = [], 0
    for n in list(range(1, 3000, 7)) + [32767, 65536, MiB, MiB + 1, 3 * MiB]:
        p = a.malloc(n)
        assert p % 512 == 0
        ptrs.append(p)
        want += round512(n)
        st = a.stats()
        assert st["allocated_bytes"] == want
        assert st["reserved_bytes"] >= st["allocated_bytes"]
    assert len(set(ptrs)) == len(ptrs)
    for p in ptrs:
        a.free(p)
    st = a.stats()
    assert st["allocated_bytes"] == 0 and st["allocations"] == 0
    assert st["reserved_bytes"] > 0  # cached, not returned
    a.empty_cache()
    assert a.stats()["reserved_bytes"] == 0
    assert a.backend_usage() == (0, 0)


def test_zero_size_is_null(sim):
    a = sim()
    assert a.malloc(0) == 0
    a.free(0)
    assert a.stats()["allocations"] == 0


def test_live_blocks_never_overlap(sim):
    a = sim()
    rnd = random.Random(0)
    live = {}
    for step in range(3000):
        if live and rnd.random() < 0.45:
            p = rnd.choice(list(live))
            a.free(p)
            del live[p]
        else:
            n = rnd.choice([1, 100, 513, 4096, 70000, MiB - 1, MiB + 1, 5 * MiB, 12 * MiB])
            p = a.malloc(n)
            live[p] = round512(n)
        if step % 250 == 0:
            spans = sorted((p, p + s) for p, s in live.items())
            for (s0, e0), (s1, _) in zip(spans, spans[1:]):
                assert e0 <= s1
            # large-pool blocks whose remainder is <= 1 MiB are handed out whole, so the
            # TORCH algorithm may account more than the rounded sum (never less)
            assert a.stats()["allocated_bytes"] >= sum(live.values())
            assert a.stats()["allocated_bytes"] <= sum(live.values()) + len(live) * MiB


def test_reuse_split_and_merge(sim):
    a = sim()
    p1 = a.malloc(300 * 1024)
    seg_before = a.stats()["segments"]
    p2 = a.malloc(300 * 1024)   # same 2 MiB small segment, split
    assert a.stats()["segments"] == seg_before
    assert p2 == p1 + 300 * 1024
    a.free(p1)
    assert a.malloc(300 * 1024) == p1          # exact-fit reuse
    a.free(p1)
    a.free(p2)
    st = a.stats()
    assert st["inactive_split_bytes"] == 0     # neighbours merged back into one whole segment
    p3 = a.malloc(MiB)
    assert p3 == p1                            # the merged 2 MiB block serves a 1 MiB request
    assert a.stats()["num_device_malloc"] == 1


def test_streams_do_not_share_free_blocks(sim):
    a = sim()
    s1, s2 = 0x1000, 0x2000
    p = a.malloc(4096, s1)
    a.free(p)
    q = a.malloc(4096, s2)
    assert q != p                               # a block freed on s1 is not handed to s2
    assert a.malloc(4096, s1) == p


def test_record_stream_defers_reuse_until_event_completes(sim):
    a = sim()
    s1, s2 = 0x1000, 0x2000
    p = a.malloc(8192, s1)
    a.record_stream(p, s2)
    a.free(p)
    st = a.stats()
    assert st["allocated_bytes"] == 0 and st["active_bytes"] == 8192  # still held by the event
    q = a.malloc(8192, s1)
    assert q != p
    a.complete_events(s2)
    assert a.stats()["active_bytes"] == 8192    # only q is active now
    a.free(q)
    r = a.malloc(16384, s1)                     # p and q merged back after the event
    assert r == p


def test_cache_only_request_queries_no_event(sim):
    # what a workspace request does while its stream is being captured: cached blocks only, no event query
    a = sim()
    s1, s2 = 0x1000, 0x2000
    p = a.malloc(8192, s1)
    a.record_stream(p, s2)
    a.free(p)                                   # parked behind an event on s2 that has not completed
    spare = a.malloc(4096, s1)
    a.free(spare)
    before = a.event_queries()
    assert a.malloc_from_cache(4096, s1) == spare   # a cache hit
    assert a.malloc_from_cache(64 * MiB, s1) == 0   # nothing cached fits: refused, nothing allocated
    assert a.event_queries() == before
    assert a.stats()["active_bytes"] == 8192 + 4096  # p is still held by its event
    a.complete_events(s2)
    q = a.malloc(8192, s1)                      # the next ordinary request sees the event and reuses p
    assert q == p


def test_history_records_each_step_in_order(pkg, sim):
    # recordHistory / trace (DIPUCachingDeviceAllocator.cpp:555-566, 1017-1027): every step, oldest first
    a = sim(capacity=64 * MiB)
    assert a.trace() == []
    p0 = a.malloc(4096)                         # before the switch: not recorded
    a.record_history(True, 64)
    s1, s2 = 0x1000, 0x2000
    p = a.malloc(3000, s1)                      # a new 2 MiB segment on s1
    a.record_stream(p, s2)
    a.free(p)                                   # requested now, completed when s2's event is seen
    a.complete_events(s2)
    q = a.malloc(30 * MiB, s1)
    with pytest.raises(pkg.runtime.RuntimeError_, match="out of memory"):
        a.malloc(60 * MiB, s1)                  # the ladder gives the cached segment back, then fails
    steps = [(e["action"], e["addr"], e["size"], e["stream"]) for e in a.trace()]
    assert steps == [
        ("SEGMENT_ALLOC", p, 2 * MiB, s1), ("ALLOC", p, 3000, s1),
        ("FREE_REQUESTED", p, 3000, s1), ("FREE_COMPLETED", p, 3000, s1),
        ("SEGMENT_ALLOC", q, 30 * MiB, s1), ("ALLOC", q, 30 * MiB, s1),
        ("SEGMENT_FREE", p, 2 * MiB, s1), ("OOM", 60 * MiB, 60 * MiB, s1),
    ]
    a.record_history(False)                     # switching clears the ring and stops recording
    a.free(q)
    a.free(p0)
    assert a.trace() == []


def test_history_ring_keeps_the_newest_entries(sim):
    a = sim()
    a.record_history(True, 5)
    ptrs = [a.malloc(512 * (i + 1)) for i in range(4)]   # SEGMENT_ALLOC + 4 ALLOC
    for p in ptrs:
        a.free(p)                                        # 4 x (FREE_REQUESTED, FREE_COMPLETED)
    t = a.trace()
    assert len(t) == 5
    assert [e["action"] for e in t] == ["FREE_COMPLETED", "FREE_REQUESTED", "FREE_COMPLETED", "FREE_REQUESTED", "FREE_COMPLETED"]
    assert [e["addr"] for e in t] == [ptrs[1], ptrs[2], ptrs[2], ptrs[3], ptrs[3]]
    assert [e["size"] for e in t] == [1024, 1536, 1536, 2048, 2048]


def test_history_of_expandable_segments_and_other_algorithms(sim):
    a = sim(conf="expandable_segments:True")
    a.record_history(True, 32)
    p = a.malloc(3 * MiB)
    a.free(p)
    a.empty_cache()
    acts = [e["action"] for e in a.trace()]
    assert acts[0] == "SEGMENT_MAP" and acts[-1] == "SEGMENT_UNMAP"
    assert acts.count("ALLOC") == 1 and "SEGMENT_ALLOC" not in acts
    mapped = sum(e["size"] for e in a.trace() if e["action"] == "SEGMENT_MAP")
    assert mapped >= 3 * MiB and mapped == sum(e["size"] for e in a.trace() if e["action"] == "SEGMENT_UNMAP")
    b = sim(algorithm="BF")                     # BF and BS keep no history
    b.record_history(True, 8)
    b.free(b.malloc(4096))
    assert b.trace() == []


def test_oom_ladder_releases_cache_then_raises(pkg, sim):
    a = sim(capacity=64 * MiB)
    p = a.malloc(40 * MiB)
    a.free(p)                                   # 40 MiB cached
    q = a.malloc(50 * MiB)                      # needs the cache to be released first
    st = a.stats()
    assert st["num_alloc_retries"] >= 1 and st["num_ooms"] == 0
    assert st["reserved_bytes"] == 50 * MiB
    with pytest.raises(pkg.runtime.RuntimeError_, match="out of memory"):
        a.malloc(30 * MiB)
    assert a.stats()["num_ooms"] == 1
    a.free(q)
    assert a.malloc(30 * MiB) != 0              # works again once memory is back


def test_max_split_size_keeps_oversize_blocks_whole(sim):
    a = sim(conf="max_split_size_mb:32")
    big = a.malloc(100 * MiB)
    a.free(big)
    small = a.malloc(2 * MiB)                   # must not carve the cached 100 MiB block
    assert not (big <= small < big + 100 * MiB)
    again = a.malloc(100 * MiB)
    assert again == big


def test_garbage_collection_threshold(sim):
    a = sim(capacity=100 * MiB, conf="garbage_collection_threshold:0.5")
    ps = [a.malloc(20 * MiB) for _ in range(3)]
    for p in ps:
        a.free(p)                               # 60 MiB cached > 50 MiB threshold
    a.malloc(30 * MiB)                          # no cached block is large enough: GC runs before growing
    assert a.stats()["num_device_free"] >= 1
    assert a.stats()["num_ooms"] == 0


def test_double_free_is_an_error(pkg, sim):
    a = sim()
    p = a.malloc(100)
    a.free(p)
    with pytest.raises(pkg.runtime.RuntimeError_):
        a.free(p)


# ------------------------------------------------------------------ BF algorithm
# DIPU_DEVICE_MEMCACHING_ALGORITHM=BF: dipu/torch_dipu/csrc_dipu/runtime/core/allocator/DIPUBFCachingAllocator.cpp
@pytest.fixture()
def bf(pkg):
    made = []

    def make(capacity=8 << 30, max_extend=0):
        a = pkg.runtime.SimAllocator(capacity, algorithm="BF", max_extend=max_extend)
        made.append(a)
        return a

    yield make
    for a in made:
        a.close()


def bf_round(n):
    return ((n - 1) | 511) + 1


def test_bf_accounting_matches_the_reference_invariant(bf):
    """test_memory_stats.py:29-45: allocated == sum(((n - 1) | 511) + 1), reserved >= allocated, and everything
    returns to zero after the frees (events complete at once here: nothing else uses the blocks)."""
    a = bf()
    ptrs, want = [], 0
    for n in list(range(1, 3000, 7)) + [32767, 65536, MiB, MiB + 1, 3 * MiB, 40 * MiB]:
        p = a.malloc(n)
        assert p % 512 == 0
        ptrs.append((p, bf_round(n)))
        want += bf_round(n)
        st = a.stats()
        assert st["allocated_bytes"] == want
        assert st["reserved_bytes"] >= st["allocated_bytes"]
    spans = sorted(ptrs)
    for (p0, n0), (p1, _) in zip(spans, spans[1:]):
        assert p0 + n0 <= p1, "live chunks overlap"
    for p, _ in ptrs:
        a.free(p)
    a.complete_events()
    assert a.stats()["allocated_bytes"] == 0
    a.empty_cache()
    assert a.stats()["reserved_bytes"] == 0 and a.backend_usage() == (0, 0)


def test_bf_extend_sizes_double_from_8_mib(bf):
    """extend(): the first device request is max(n, 8 MiB) and the extend size doubles after every success
    (DIPUBFCachingAllocator.cpp:303-331), up to the cap."""
    a = bf(max_extend=32 * MiB)
    a.malloc(512)
    assert a.backend_usage() == (8 * MiB, 1)
    held = [a.malloc(6 * MiB)]          # fits in what is left of the first 8 MiB
    assert a.backend_usage() == (8 * MiB, 1)
    held.append(a.malloc(6 * MiB))      # nothing fits: second extend is 16 MiB
    assert a.backend_usage() == (24 * MiB, 2)
    held.append(a.malloc(30 * MiB))     # third: 32 MiB (the cap)
    assert a.backend_usage() == (56 * MiB, 3)
    held.append(a.malloc(31 * MiB))     # capped: stays 32 MiB
    assert a.backend_usage() == (88 * MiB, 4)
    held.append(a.malloc(100 * MiB))    # larger than the cap: exactly the rounded request
    assert a.backend_usage() == (188 * MiB, 5)


def test_bf_split_rule_and_merge_on_free(bf):
    """A chunk at least twice the request (or 8 MiB larger) is split, the rest stays cached; freed neighbours
    merge back into one chunk that serves a request of the whole size (:375-378, :284-301)."""
    a = bf()
    p = a.malloc(3 * MiB)               # 8 MiB from the device, split 3 + 5
    q = a.malloc(5 * MiB)               # exactly the rest: not split
    assert q == p + 3 * MiB and a.backend_usage() == (8 * MiB, 1)
    a.free(p)
    a.free(q)
    a.complete_events()
    r = a.malloc(8 * MiB)               # only possible if the two halves merged
    assert r == p and a.backend_usage() == (8 * MiB, 1)
    a.free(r)
    a.complete_events()
    s = a.malloc(5 * MiB)               # 8 MiB chunk, 5 MiB request: < 2x and < +8 MiB, handed out whole
    t = a.malloc(2 * MiB)
    assert a.backend_usage()[1] == 2, "the 3 MiB tail of an unsplit chunk is not available"
    assert a.stats()["allocated_bytes"] == 7 * MiB
    a.free(s), a.free(t)


def test_bf_reuse_waits_for_events_on_every_stream(bf):
    """free() records an event on the allocation stream and on every recordStream() stream; the chunk is reusable
    only after all of them completed (:525-548). Streams share one set of chunks (:357)."""
    a = bf()
    s1, s2 = 0x10, 0x20
    p = a.malloc(6 * MiB, stream=s1)
    a.record_stream(p, s2)
    a.free(p)
    q = a.malloc(6 * MiB, stream=s1)
    assert q != p, "reused while its events are outstanding"
    a.complete_events(s1)
    q2 = a.malloc(6 * MiB, stream=s1)
    assert q2 != p, "the other stream's event is still outstanding"
    a.complete_events(s2)
    q3 = a.malloc(6 * MiB, stream=s2)   # another stream may take it: one shared set
    assert q3 == p
    for x in (q, q2, q3):
        a.free(x)


def test_bf_out_of_memory_ladder(bf, pkg):
    """Nothing cached fits and the device is full: pending frees are waited for, whole cached chunks go back to the
    device, and only then the request fails."""
    a = bf(capacity=64 * MiB, max_extend=8 * MiB)
    p = a.malloc(40 * MiB)
    a.free(p)                            # pending: its event is not complete
    q = a.malloc(48 * MiB)               # needs the 40 MiB released first
    assert a.backend_usage() == (48 * MiB, 1)
    with pytest.raises(RuntimeError, match="no memory available"):
        a.malloc(32 * MiB)
    assert a.stats()["num_ooms"] == 1
    a.free(q)


def test_bf_size_classes_and_random_stress(bf):
    a = bf(capacity=2 << 30)
    rnd = random.Random(7)
    live = {}
    for step in range(4000):
        if live and (rnd.random() < 0.45 or len(live) > 200):
            p = rnd.choice(list(live))
            a.free(p)
            del live[p]
            if rnd.random() < 0.5:
                a.complete_events()
        else:
            n = rnd.choice([1, 511, 513, 4096, 70000, MiB - 1, 3 * MiB + 5, 9 * MiB])
            p = a.malloc(n, stream=rnd.choice([0, 0x10]))
            assert p % 512 == 0 and p not in live
            live[p] = bf_round(n)
        if step % 500 == 0:
            spans = sorted(live.items())
            for (p0, n0), (p1, _) in zip(spans, spans[1:]):
                assert p0 + n0 <= p1
            st = a.stats()
            assert st["allocated_bytes"] == sum(live.values()) and st["reserved_bytes"] >= st["allocated_bytes"]
    for p in list(live):
        a.free(p)
    a.complete_events()
    a.empty_cache()
    assert a.backend_usage() == (0, 0)


# ------------------------------------------------------------------ BS algorithm
# DIPU_DEVICE_MEMCACHING_ALGORITHM=BS: dipu/torch_dipu/csrc_dipu/runtime/core/allocator/DIPUBSCachingAllocator.cpp
def test_bs_exact_size_lists_and_accounting(pkg):
    a = pkg.runtime.SimAllocator(1 << 30, algorithm="BS")
    try:
        p = a.malloc(1000)                       # 1024: a multiple of 512
        q = a.malloc(1024)                       # same size, second device block
        assert a.backend_usage() == (2048, 2) and a.stats()["allocated_bytes"] == 2048
        a.free(p)
        a.complete_events()
        assert a.malloc(1500) not in (p, q)      # 1536: another size, never served from the 1024 list
        assert a.malloc(513) == p                # 1024 again: the idle block of exactly that size
        assert a.backend_usage() == (2048 + 1536, 3)
        st = a.stats()
        assert st["allocated_bytes"] == 1024 * 2 + 1536 and st["reserved_bytes"] == st["allocated_bytes"]
        a.free(q)
        a.empty_cache()                          # waits for the pending free, then returns idle blocks
        assert a.backend_usage() == (1024 + 1536, 2)
    finally:
        a.close()


def test_bs_power_of_two_sizes(pkg):
    """DIPU_BS_MORE_ADAPTABLE: 1 << bit_length(n), at least 512 (DIPUBSCachingAllocator.cpp:36-52): a power of two
    itself doubles."""
    a = pkg.runtime.SimAllocator(1 << 30, algorithm="BS", power_of_two=True)
    try:
        for n, want in [(1, 512), (511, 512), (512, 1024), (1000, 1024), (1024, 2048), (70000, 131072)]:
            before = a.backend_usage()[0]
            a.malloc(n)
            assert a.backend_usage()[0] - before == want, (n, want)
    finally:
        a.close()


def test_bs_reuse_waits_for_events_and_oom_empties_the_cache(pkg):
    a = pkg.runtime.SimAllocator(64 * MiB, algorithm="BS")
    try:
        p = a.malloc(20 * MiB, stream=0x10)
        a.record_stream(p, 0x20)
        a.free(p)
        q = a.malloc(24 * MiB)                   # another size; the pending 20 MiB is waited for and parked idle
        assert a.backend_usage() == (44 * MiB, 2)
        r = a.malloc(30 * MiB)                   # device full: the idle 20 MiB block goes back, then it fits
        assert a.backend_usage() == (54 * MiB, 2) and a.stats()["num_alloc_retries"] == 1
        with pytest.raises(RuntimeError, match="no memory available"):
            a.malloc(40 * MiB)
        a.free(q), a.free(r)
    finally:
        a.close()


# ---- expandable_segments:True (DIPUCachingDeviceAllocator.cpp:1086-1215, 1633-1705) ----
# The stand-in range is 1 GiB of address space per (stream, pool); its 2 MiB / 20 MiB segments count against the
# capacity only while mapped.
ES = "expandable_segments:True"


def test_expandable_conf_is_parsed(pkg, sim):
    sim(conf="expandable_segments:False")
    with pytest.raises(pkg.runtime.RuntimeError_, match="expandable_segments"):
        sim(conf="expandable_segments:yes")


def test_expandable_range_grows_at_its_end_in_whole_segments(sim):
    a = sim(conf=ES)
    p1 = a.malloc(30 * MiB)                     # two 20 MiB segments mapped
    st = a.stats()
    assert st["reserved_bytes"] == 40 * MiB and st["segments"] == 1
    assert a.backend_usage()[0] == 40 * MiB
    p2 = a.malloc(5 * MiB)                      # fits the mapped remainder
    assert p2 == p1 + 30 * MiB and a.stats()["reserved_bytes"] == 40 * MiB
    p3 = a.malloc(25 * MiB)                     # 5 MiB free + one more segment, contiguous with the rest
    assert p3 == p2 + 5 * MiB
    st = a.stats()
    assert st["reserved_bytes"] == 60 * MiB and st["segments"] == 1
    assert st["allocated_bytes"] == 60 * MiB


def test_expandable_assembles_a_large_block_from_freed_small_ones(sim):
    # the point of the mode: ten 18 MiB blocks freed leave one free run that serves 170 MiB without new memory;
    # fixed segments would hold ten separate 20 MiB segments and need 170 MiB more
    a = sim(capacity=200 * MiB, conf=ES)
    ps = [a.malloc(18 * MiB) for _ in range(10)]
    assert ps == [ps[0] + i * 18 * MiB for i in range(10)]
    assert a.stats()["reserved_bytes"] == 180 * MiB
    for p in ps:
        a.free(p)
    big = a.malloc(170 * MiB)
    assert big == ps[0]
    st = a.stats()
    assert st["reserved_bytes"] == 180 * MiB and st["num_alloc_retries"] == 0

    b = sim(capacity=200 * MiB)                 # same trace without the mode: only after releasing the cache
    qs = [b.malloc(18 * MiB) for _ in range(10)]
    for q in qs:
        b.free(q)
    b.malloc(170 * MiB)
    assert b.stats()["num_alloc_retries"] >= 1


def test_expandable_empty_cache_unmaps_whole_free_segments_only(sim):
    a = sim(conf=ES)
    p1 = a.malloc(30 * MiB)
    p2 = a.malloc(30 * MiB)
    p3 = a.malloc(30 * MiB)                     # 90 MiB -> five segments mapped
    assert a.stats()["reserved_bytes"] == 100 * MiB
    a.free(p2)                                  # [30, 60) free: only segment [40, 60) lies inside it
    a.empty_cache()
    st = a.stats()
    assert st["reserved_bytes"] == 80 * MiB and a.backend_usage()[0] == 80 * MiB
    assert st["segments"] == 1
    q = a.malloc(30 * MiB)                      # maps the hole again, same address
    assert q == p2 and a.stats()["reserved_bytes"] == 100 * MiB
    for p in (p1, p3, q):
        a.free(p)
    a.empty_cache()                             # nothing in use: the range itself goes
    st = a.stats()
    assert st["reserved_bytes"] == 0 and st["segments"] == 0 and a.backend_usage()[0] == 0
    assert a.malloc(30 * MiB) != 0              # and a new one is made on demand
    assert a.stats()["segments"] == 1


def test_expandable_small_pool_streams_and_events(sim):
    a = sim(conf=ES)
    s1, s2 = 0x1000, 0x2000
    p = a.malloc(4096, s1)                      # small pool: 2 MiB segments
    assert a.stats()["reserved_bytes"] == 2 * MiB
    q = a.malloc(4096, s2)                      # another stream gets a range of its own
    assert abs(q - p) >= (1 << 30) and a.stats()["segments"] == 2
    a.record_stream(p, s2)
    a.free(p)
    r = a.malloc(MiB, s1)                       # p still waits for s2's event: served behind it
    assert r == p + 4096
    a.complete_events(s2)
    a.free(r)
    assert a.malloc(MiB, s1) == p               # merged back once the event is done
    assert a.malloc(MiB, s1) == p + MiB         # the first segment is full now
    assert a.malloc(MiB, s1) == p + 2 * MiB     # one more small segment, contiguous
    assert a.stats()["reserved_bytes"] == 4 * MiB + 2 * MiB and a.stats()["segments"] == 2


def test_expandable_out_of_memory_ladder(pkg, sim):
    a = sim(capacity=100 * MiB, conf=ES)
    s1, s2 = 0x1000, 0x2000
    p = a.malloc(60 * MiB, s1)
    a.free(p)                                   # 60 MiB cached on s1's range
    q = a.malloc(50 * MiB, s2)                  # s2's range needs 60 MiB: s1's cache has to be unmapped first
    st = a.stats()
    assert st["num_alloc_retries"] >= 1 and st["num_ooms"] == 0
    assert st["reserved_bytes"] == 60 * MiB
    with pytest.raises(pkg.runtime.RuntimeError_, match="out of memory"):
        a.malloc(60 * MiB, s2)
    a.free(q)
    assert a.malloc(90 * MiB, s2) == q


def test_expandable_random_stress_keeps_the_books(sim):
    rng = random.Random(7)
    a = sim(capacity=900 * MiB, conf=ES)
    live = {}
    for step in range(3000):
        if live and (rng.random() < 0.45 or len(live) > 60):
            p = rng.choice(list(live))
            a.free(p)
            del live[p]
        else:
            n = rng.choice([rng.randint(1, 4096), rng.randint(4096, MiB), rng.randint(MiB, 12 * MiB)])
            p = a.malloc(n)
            assert p not in live
            live[p] = n
        if step % 500 == 499:
            a.empty_cache()
        if step % 100 == 0:
            spans = sorted((p, p + n) for p, n in live.items())
            assert all(x[1] <= y[0] for x, y in zip(spans, spans[1:]))
            st = a.stats()
            want = sum(round512(n) for n in live.values())  # a large block keeps a remainder of up to 1 MiB
            assert want <= st["allocated_bytes"] <= want + len(live) * MiB
            assert st["reserved_bytes"] == a.backend_usage()[0] >= st["allocated_bytes"]
    for p in list(live):
        a.free(p)
    a.empty_cache()
    assert a.stats()["reserved_bytes"] == 0 and a.backend_usage()[0] == 0
