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

    def make(capacity=8 << 30, conf=""):
        a = pkg.runtime.SimAllocator(capacity, conf)
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
