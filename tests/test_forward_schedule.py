"""The tile lists of the attention forward with the hand-scheduled loop, on the
host alone: whatever the shape, every (sequence, head, query tile) is launched
exactly once, lists never exceed the table, and the heads that share a kv head
stay on as few XCDs as the partitioning promises (workgroup i runs on XCD i mod
8).  No GPU is needed: the packing is host code behind a test-support export."""
import ctypes
import random

import pytest

from pluto_amd import capi

NO_ITEM = 0xFFFF
CAPACITY = 1536


@pytest.fixture(scope="module")
def library():
    return capi.lib()


def schedule(library, head_dim, q_rows, kv_rows, start, query_heads, group, sequences, resident):
    items = (ctypes.c_uint16 * CAPACITY)()
    workgroups, slots = ctypes.c_int(-1), ctypes.c_int(-1)
    status = library.pluto_hip_test_forward_schedule(
        head_dim, q_rows, kv_rows, start, query_heads, group, sequences, resident, items, CAPACITY,
        ctypes.byref(workgroups), ctypes.byref(slots))
    return status, workgroups.value, slots.value, list(items)


def tile_rows(head_dim):
    return 256 if head_dim == 128 else 128


def check(library, head_dim, q_rows, query_heads, group, sequences, resident, start=0):
    kv_rows = start + q_rows
    status, workgroups, slots, items = schedule(library, head_dim, q_rows, kv_rows, start,
                                                query_heads, group, sequences, resident)
    assert status == 0
    q_tiles = -(-q_rows // tile_rows(head_dim))
    total = q_tiles * query_heads * sequences
    if workgroups == 0:
        return False      # numbered by workgroup index: nothing to check here
    assert workgroups == resident and 0 < slots and workgroups * slots <= CAPACITY
    seen = {}
    for w in range(workgroups):
        ended = False
        for e in range(slots):
            item = items[w * slots + e]
            if item == NO_ITEM:
                ended = True
                continue
            assert not ended, "an entry after the end of a list"
            assert item < total
            assert item not in seen, "tile %d in the lists of workgroups %d and %d" % (item, seen[item], w)
            seen[item] = w
    assert len(seen) == total, "%d of %d tiles are in no list" % (total - len(seen), total)
    # heads of one (sequence, kv head) run on one XCD when the units divide over the eight,
    # on 8 / units XCDs when there are fewer units than XCDs
    kv_heads = query_heads // group
    kv_units = sequences * kv_heads
    xcds = {}
    for item, w in seen.items():
        column = item // q_tiles
        unit = (column // query_heads) * kv_heads + (column % query_heads) // group
        xcds.setdefault(unit, set()).add(w % 8)
    if kv_units % 8 == 0:
        assert all(len(x) == 1 for x in xcds.values())
    elif 8 % kv_units == 0:
        assert all(len(x) <= 8 // kv_units for x in xcds.values())
        assert len(set().union(*xcds.values())) == 8
    # balance: no list carries more than the mean plus one heaviest tile
    def cost(item):
        t = item % q_tiles
        last = min((t + 1) * tile_rows(head_dim), q_rows) - 1
        return -(-min(kv_rows, start + last + 1) // 64) + 8
    loads = [0] * workgroups
    for item, w in seen.items():
        loads[w] += cost(item)
    heaviest = max(cost(i) for i in seen)
    assert max(loads) <= sum(loads) / workgroups + heaviest
    return True


def test_benchmarked_shapes(library):
    assert check(library, 128, 8192, 24, 6, 1, 256)      # the prefill configuration
    assert check(library, 256, 8192, 24, 6, 1, 256)
    assert check(library, 64, 4096, 12, 1, 4, 512)
    assert check(library, 128, 2301, 6, 3, 1, 256) is False   # fewer tiles than workgroups


def test_every_tile_is_launched_once_whatever_the_shape(library):
    rng = random.Random(5)
    listed = 0
    for _ in range(400):
        head_dim = rng.choice([64, 128, 256])
        group = rng.choice([1, 1, 2, 3, 6, 8])
        query_heads = group * rng.randint(1, 6)
        sequences = rng.randint(1, 5)
        q_rows = rng.choice([rng.randint(1, 3000), rng.randint(3000, 40000)])
        start = rng.choice([0, 0, rng.randint(1, 5000)])
        resident = rng.choice([256, 512, 64, 8, 304, 0, 250])
        listed += bool(check(library, head_dim, q_rows, query_heads, group, sequences, resident, start))
    assert listed > 80    # the sample does exercise the packing


def test_rejections(library):
    items = (ctypes.c_uint16 * 4)()
    w, s = ctypes.c_int(), ctypes.c_int()
    call = library.pluto_hip_test_forward_schedule
    assert call(96, 100, 100, 0, 4, 1, 1, 256, items, 4, ctypes.byref(w), ctypes.byref(s)) == capi.EINVAL
    assert call(128, 100, 100, 0, 4, 3, 1, 256, items, 4, ctypes.byref(w), ctypes.byref(s)) == capi.EINVAL
    assert call(128, 8192, 8192, 0, 24, 6, 1, 256, items, 4, ctypes.byref(w), ctypes.byref(s)) == capi.ELIMIT
