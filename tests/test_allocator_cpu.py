"""The block allocator through the C ABI, without a device: the reference's own allocator tests
(helium/src/cuda/allocator/block.rs:359-399) and the stream rules its doc comments state (block.rs:286-299,
allocator/device.rs:48-89)."""
import numpy as np
from sortedcontainers import SortedList

from helium_amd.allocator import BlockAllocator

GIB = 1 << 30


def test_simple():
    """block.rs:359-376"""
    a = BlockAllocator()
    a.add_page(1024)
    b1 = a.allocate(128, 256)
    assert b1.size == 128
    b2 = a.allocate(1024 - 128, 128)
    assert b2.size == 1024 - 128
    assert a.allocate(1, 1) is None
    a.deallocate(b1)
    a.deallocate(b2)
    assert a.allocate(1024, 8).size == 1024


def test_stress_no_overlap_exact_size_and_alignment():
    """block.rs:378-399: 25,000 operations on a 64 GiB page, sizes in [1 KiB, 32 MiB), alignment 256."""
    a = BlockAllocator()
    a.add_page(64 * GIB)
    rng = np.random.default_rng(66)
    live = SortedList(key=lambda b: b.start)
    for step in range(25_000):
        if not live or rng.random() < 0.4:
            size = int(rng.integers(1024, 32 << 20))
            b = a.allocate(size, 256)
            assert b is not None and b.size == size and b.start % 256 == 0
            i = live.bisect_key_left(b.start)
            assert i == 0 or live[i - 1].end() <= b.start
            assert i == len(live) or b.end() <= live[i].start
            live.add(b)
        else:
            a.deallocate(live.pop(int(rng.integers(len(live)))))
        if step % 2500 == 0:
            s = a.stats()
            assert s["free_bytes"] + sum(b.size for b in live) == 64 * GIB
    for b in list(live):
        a.deallocate(b)
    assert a.stats() == {"free_blocks": 1, "free_bytes": 64 * GIB, "largest_free_block": 64 * GIB, "streams": 0}


def test_best_fit_split_and_coalesce():
    a = BlockAllocator()
    a.add_page(4096)
    blocks = [a.allocate(512, 256) for _ in range(8)]
    assert [b.start for b in blocks] == list(range(0, 4096, 512))
    a.deallocate(blocks[1])                      # hole of 512
    a.deallocate(blocks[4]); a.deallocate(blocks[5])   # hole of 1024 (merged)
    assert a.stats()["free_blocks"] == 2 and a.stats()["largest_free_block"] == 1024
    assert a.allocate(500, 1).start == 512       # the smallest hole that fits, not the first large one
    assert a.allocate(768, 256).start == 2048
    assert a.stats() == {"free_blocks": 2, "free_bytes": 12 + 256, "largest_free_block": 256, "streams": 0}
    # an alignment the block's start does not have: the head is split off and stays free
    a2 = BlockAllocator()
    a2.add_page(1 << 20)
    assert a2.allocate(100, 1).start == 0
    b = a2.allocate(1000, 4096)
    assert b.start == 4096 and b.size == 1000
    assert a2.stats()["free_blocks"] == 2


def test_a_freed_block_waits_for_its_stream():
    """A block freed in a stream may still be in use on the device: until end_stream only that stream and the streams
    that come after it (its descendants) can have it."""
    a = BlockAllocator()
    a.add_page(1024)
    s1 = a.begin_stream()
    other = a.begin_stream()
    b = a.allocate(1024, 256, s1)
    assert b.in_use() == [s1]
    a.deallocate(b)
    assert a.allocate(512, 256) is None              # no stream: only blocks nobody holds
    assert a.allocate(512, 256, other) is None       # an unrelated stream
    child = a.begin_stream(parent=s1)
    grandchild = a.begin_stream(parent=child)
    c = a.allocate(512, 256, grandchild)             # ordered after s1 on the device
    assert c is not None and c.in_use() == [s1, grandchild]
    again = a.allocate(512, 256, s1)                 # the stream itself
    assert again is not None
    a.deallocate(c)
    a.deallocate(again)
    assert a.allocate(512, 256, other) is None
    # blocks held by different stream sets do not merge; they do once the streams have ended
    assert a.stats()["free_blocks"] == 2
    a.end_stream(grandchild)
    assert a.stats()["free_blocks"] == 1
    a.end_stream(s1)
    assert a.stats() == {"free_blocks": 1, "free_bytes": 1024, "largest_free_block": 1024, "streams": 2}
    assert a.allocate(1024, 256, other).in_use() == [other]


def test_ending_a_parent_removes_it_from_its_descendants():
    a = BlockAllocator()
    a.add_page(1024)
    s1 = a.begin_stream()
    s2 = a.begin_stream(parent=s1)
    a.end_stream(s1)
    s3 = a.begin_stream(parent=s1)   # a parent that has ended gives no ancestors (block.rs:217-226)
    b = a.allocate(1024, 256, s2)
    a.deallocate(b)
    assert a.allocate(256, 256, s3) is None
    assert a.allocate(256, 256, s2) is not None


def test_random_streams_never_hand_out_memory_another_stream_may_use():
    """Randomised: streams begin (with the previous stream of their 'thread' as parent) and end in order per thread;
    a block is only ever handed to a stream that is ordered after everyone who may still be using it."""
    rng = np.random.default_rng(7)
    a = BlockAllocator()
    a.add_page(1 << 24)
    threads = {t: [] for t in range(3)}      # live streams per thread, oldest first
    ancestors = {}
    live = []                                # (block, stream)
    holders = {}                             # (start, end) ranges freed while a stream was live -> set of streams
    freed = []                               # (start, end, frozenset of live holders at free time)
    for step in range(6000):
        r = rng.random()
        t = int(rng.integers(3))
        if r < 0.08 or not threads[t]:
            parent = threads[t][-1] if threads[t] else 0
            s = a.begin_stream(parent)
            ancestors[s] = (ancestors.get(parent, set()) | {parent}) if parent else set()
            threads[t].append(s)
        elif r < 0.14 and len(threads[t]) > 1:
            s = threads[t].pop(0)
            # the harness frees what the stream still holds first, as dropping an executor's tensors does
            for item in [x for x in live if x[1] == s]:
                live.remove(item)
                a.deallocate(item[0])
            a.end_stream(s)
            freed = [(lo, hi, h - {s}) for lo, hi, h in freed if h - {s}]
            for k in ancestors:
                ancestors[k].discard(s)
        elif r < 0.6:
            s = threads[t][-1]
            size = int(rng.integers(1, 64)) * 256
            b = a.allocate(size, 256, s)
            if b is None:
                continue
            for other, _ in live:
                assert not (b.start < other.end() and other.start < b.end()), "overlaps a live block"
            for lo, hi, h in freed:
                if b.start < hi and lo < b.end():
                    assert all(x == s or x in ancestors[s] for x in h), (step, h, s, ancestors[s])
            live.append((b, s))
        elif live:
            b, s = live.pop(int(rng.integers(len(live))))
            a.deallocate(b)
            freed.append((b.start, b.end(), frozenset({s})))
        if step % 500 == 0:
            a.stats()
    a.stats()
