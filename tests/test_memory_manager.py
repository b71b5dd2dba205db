"""The device memory manager (pool + array table) driven without a GPU.

A context made with device = -2 takes host memory for device memory; ACCHIP_POOL_LIMIT caps what
it may take, so every rung of the reference's allocation ladder can be forced: free list of the
size class, fresh block, clean hook, purge, eviction of the eldest unused array with copy-back
of dirty data, re-upload on the next use, and failure only when everything is in use
(Array/Remote/Table.hs:170-211, Nursery.hs:43-113, LRU.hs:140-341).  The reference ships no such
test; the same entry points run against a real device in tests/test_gpu_runtime.py.
"""
import ctypes as C

import numpy as np
import pytest

from accelerate_amd import hip

KIB = 1024
CLEAN, DIRTY, UNMANAGED, EVICTED = 0, 1, 2, 3


@pytest.fixture
def small(monkeypatch):
    """a context whose 'device' holds 64 KiB"""
    monkeypatch.setenv("ACCHIP_POOL_LIMIT", str(64 * KIB))
    ctx = hip.Context(-2)
    yield ctx
    ctx.close()


def _read(ctx, devptr, like):
    out = np.empty_like(like)
    ctx.peek(out, devptr)
    return out


def test_pool_rounds_to_1k_and_reuses_blocks_of_the_same_class(small):
    a = small.malloc(1000)
    assert a and small.stat("bytes_allocated_remote") == 1024        # remoteAllocationSize, Table.hs:180-190
    small.free(a)
    b = small.malloc(700)                                            # same class: the block comes back
    assert b == a and small.stat("pool_hits") == 1 and small.stat("bytes_allocated_remote") == 1024
    c = small.malloc(1025)                                           # next class: a new block
    assert c != a and small.stat("bytes_allocated_remote") == 1024 + 2048
    total, avail = small.mem_info()
    assert total == 64 * KIB and avail == 64 * KIB - 3 * KIB


def test_purge_makes_room_when_the_free_lists_hold_the_wrong_sizes(small):
    blocks = [small.malloc(16 * KIB) for _ in range(4)]              # the device is full
    assert all(blocks) and small.malloc(1) is None
    for b in blocks:
        small.free(b)
    # nothing of 48 KiB waits in the free lists and the device is full: they are released, then it fits
    big = small.malloc(48 * KIB)
    assert big and small.stat("bytes_evicted_from_remote") == 64 * KIB
    assert small.malloc(32 * KIB) is None                            # NULL, never an abort (Class.hs:52-54)


def test_poke_and_peek_round_trip(small):
    x = np.arange(5000, dtype=np.int32)
    p = small.malloc(x.nbytes)
    small.poke(p, x)
    assert np.array_equal(_read(small, p, x), x)
    assert small.stat("bytes_copied_to_remote") == x.nbytes and small.stat("bytes_copied_from_remote") == x.nbytes


def test_eviction_of_the_eldest_unused_array_with_copy_back_and_reupload(small):
    ctx = small
    host = {k: np.full(4 * KIB, k, np.int32) for k in range(1, 6)}   # 16 KiB each: four fit
    for k in (1, 2, 3, 4):
        assert ctx.table_malloc(k, host[k], frozen=(k == 2)) is True
        assert ctx.table_malloc(k, host[k]) is False                  # already in the table: a no-op
        ptr = ctx.table_use(k)
        ctx.poke(ptr, host[k] * 10)                                   # the device copy becomes the newer one
        ctx.table_release(k)
    assert [ctx.table_status(k) for k in (1, 2, 3, 4)] == [DIRTY, CLEAN, DIRTY, DIRTY]
    # array 1 is used again: array 2 is now the eldest
    ctx.table_use(1)
    ctx.table_release(1)
    # a fifth array does not fit: the eldest unused one goes -- array 2, frozen, so nothing is copied back
    before = ctx.stat("bytes_copied_from_remote")
    assert ctx.table_malloc(5, host[5]) is True
    assert ctx.table_status(2) == EVICTED and ctx.stat("arrays_evicted") == 1
    assert ctx.stat("bytes_copied_from_remote") == before and np.all(host[2] == 2)
    # using array 2 again evicts the next eldest, array 3: dirty, so its device contents reach the host array
    p2 = ctx.table_use(2)
    assert ctx.table_status(3) == EVICTED and np.all(host[3] == 30)
    assert ctx.table_status(2) == CLEAN and np.array_equal(_read(ctx, p2, host[2]), host[2])   # uploaded from the host copy
    # array 2 is in use: with 4 and 1 and 5 unused the next allocations take those, never array 2
    extra = {k: np.zeros(4 * KIB, np.int32) for k in (6, 7, 8)}
    for k in (6, 7, 8):
        ctx.table_malloc(k, extra[k])
        ctx.table_use(k)                                              # and keeps them in use
    assert ctx.table_status(2) == CLEAN and [ctx.table_status(k) for k in (4, 1, 5)] == [EVICTED] * 3
    assert np.all(host[4] == 40) and np.all(host[1] == 10)
    # everything resident is in use: the ladder ends in "Remote memory exhausted"
    with pytest.raises(hip.AccError, match="Remote memory exhausted") as e:
        ctx.table_malloc(9, np.zeros(4 * KIB, np.int32))
    assert e.value.code == 3
    with pytest.raises(hip.AccError, match="Remote memory exhausted"):
        ctx.table_use(3)                                              # an evicted array cannot come back either
    # once a use ends, its array can make room; the evicted array returns with the data that was copied back
    ctx.table_release(6)
    p3 = ctx.table_use(3)
    assert ctx.table_status(6) == EVICTED and np.all(_read(ctx, p3, host[3]) == 30)


def test_freed_arrays_feed_the_free_lists_and_unknown_ids_are_nothing(small):
    ctx = small
    a = np.zeros(8 * KIB, np.int32)                                   # 32 KiB
    assert ctx.table_use(77) is None                                  # withRemote on an array never allocated: Nothing
    ctx.table_malloc(1, a)
    first = ctx.table_use(1)
    ctx.table_release(1)
    ctx.table_free(1)                                                 # the host array died: block to the free list
    assert ctx.table_status(1) == -1
    ctx.table_malloc(2, a)
    assert ctx.table_use(2) == first and ctx.stat("bytes_allocated_remote") == 32 * KIB
    ctx.table_free(2)
    ctx.table_free(2)                                                 # twice: ignored (Table.hs:253-258)


def test_clean_hook_runs_before_anything_is_purged_or_evicted(small):
    ctx = small
    arrays = {k: np.zeros(8 * KIB, np.int32) for k in (1, 2)}         # 32 KiB each: the device is full
    for k in arrays:
        ctx.table_malloc(k, arrays[k])
    calls = []

    def collect():                                                    # the caller's GC finds array 1 dead
        calls.append(1)
        ctx.table_free(1)

    ctx.set_clean_hook(collect)
    ctx.table_malloc(3, np.zeros(8 * KIB, np.int32))
    assert calls == [1] and ctx.stat("arrays_evicted") == 0 and ctx.table_status(2) == DIRTY
    ctx.set_clean_hook(None)


def test_unmanaged_arrays_are_never_evicted(small):
    ctx = small
    mine = ctx.malloc(32 * KIB)
    lib = hip.lib()
    assert lib.acchip_table_insert_unmanaged(ctx._h, 1, mine) == 0
    assert ctx.table_status(1) == UNMANAGED and ctx.table_use(1) == mine
    ctx.table_release(1)
    ctx.table_malloc(2, np.zeros(4 * KIB, np.int32))                  # 16 KiB: fits beside it
    ctx.table_use(2)
    with pytest.raises(hip.AccError, match="Remote memory exhausted"):
        ctx.table_malloc(3, np.zeros(8 * KIB, np.int32))              # 32 KiB: only the unmanaged block could go
    assert ctx.table_status(1) == UNMANAGED


def test_adopted_results_live_in_the_table(small):
    # a buffer the library allocated (a program's result) becomes the device copy of a host array:
    # the handle may go, the block stays, is evicted with copy-back like any dirty array, and comes back
    from accelerate_amd import ir as A
    ctx = small
    res = ctx.empty((4 * KIB,), A.tarray(1, A.i32))                  # 16 KiB, stands for a result
    p = hip.lib().acchip_array_buffer(res._h, 0)
    ctx.poke(p, np.full(4 * KIB, 7, np.int32))
    host = np.zeros(4 * KIB, np.int32)
    ctx.table_adopt(5, host, res)
    with pytest.raises(hip.AccError, match="does not own"):
        ctx.table_adopt(6, host, res)                                 # once only
    res.release()
    assert ctx.table_use(5) == p and ctx.table_status(5) == DIRTY
    ctx.table_release(5)
    filler = np.zeros(14 * KIB, np.int32)                             # 56 KiB: only fits if the adopted block goes
    ctx.table_malloc(1, filler)
    assert ctx.table_status(5) == EVICTED and np.all(host == 7)       # its contents reached the host array
    ctx.table_free(1)
    assert np.all(_read(ctx, ctx.table_use(5), host) == 7)


def test_contexts_without_memory_refuse(cc_ctx):
    assert cc_ctx.malloc(100) is None
    with pytest.raises(hip.AccError, match="no device"):
        cc_ctx.table_malloc(1, np.zeros(10, np.int32))
    fake = hip.Context(-2)
    with pytest.raises(hip.AccError, match="no device"):             # host memory stands in for memory only
        from accelerate_amd import ir as A, programs as P
        run = fake.compile(P.map_affine())
        run.execute(fake.to_device(np.zeros(4, np.float32), A.tarray(1, A.f32)))
    fake.close()
