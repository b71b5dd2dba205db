"""Array-level control flow (evalOpenAcc, Interpreter.hs:175-259) and the device memory
manager behind the C ABI, on the GPU."""
import ctypes as C

import numpy as np
import pytest

from accelerate_amd import hip
from accelerate_amd import ir as A
from accelerate_amd import programs as P
from oracle import c as OC
from oracle import interp as O

from . import progs as Q
from .cases import same
from .runtime_cases import runtime_cases

pytestmark = pytest.mark.gpu
CASES = runtime_cases()


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_control_flow_matches_oracle(gpu_ctx, case):
    _, prog, args, uses = case
    run = gpu_ctx.compile(prog)
    dev_uses = [gpu_ctx.to_device(u, t) for u, t in uses]
    got = run(*args, uses=dev_uses)
    exp = O.run_n(prog.text(), *args, uses=[O.to_arr(u, t) for u, t in uses])
    assert same(got, exp)


def test_atrace_hands_message_and_arrays_to_the_callback(gpu_ctx, capfd):
    # Atrace (Interpreter.hs:215, atraceOp :873-880): the callback sees the message and the
    # evaluated arrays before the body's result comes back; without one, a line on stderr
    case = [c for c in CASES if c[0] == "atrace_reports_then_continues"][0]
    _, prog, args, _ = case
    run = gpu_ctx.compile(prog)
    seen = []
    gpu_ctx.set_trace(lambda msg, arrays: seen.append((msg, arrays)))
    try:
        got = run(*args)
    finally:
        gpu_ctx.set_trace(None)
    assert same(got, args[0] + 1)
    assert len(seen) == 1 and seen[0][0] == "partial sums"
    assert same(seen[0][1], (np.cumsum(args[0]), np.array(7, np.int64)))
    run(*args)
    assert "partial sums: Array (Z :. 500) i64, Array (Z) i64" in capfd.readouterr().err


def test_fold1seg_reports_an_empty_segment(gpu_ctx):
    # fold1SegOp checks every segment for an element (boundsCheck "empty segment",
    # Interpreter.hs:424); the kernel that walks the boundaries reports it, and the next call
    # that waits for the stream raises it.  The context stays usable.
    from . import progs as Q
    V1 = A.tarray(1, A.i64)
    prog = A.alam([V1, V1], lambda vals, seg: A.alet(
        V1, A.scan("l", Q.binop(A.add, A.i64), A.const(A.i64, 0), seg),
        lambda offs: A.foldseg(A.i64, Q.binop(A.add, A.i64), None, vals, offs)))
    run = gpu_ctx.compile(prog)
    vals = np.arange(10, dtype=np.int64)
    assert same(run(vals, np.array([3, 2, 5], np.int64)), np.array([3, 7, 35], np.int64))
    res = run.execute(gpu_ctx.to_device(vals, V1), gpu_ctx.to_device(np.array([3, 0, 7], np.int64), V1))
    with pytest.raises(hip.AccError, match="empty segment"):
        res.to_host()
    assert same(run(vals, np.array([4, 6], np.int64)), np.array([6, 39], np.int64))
    # with a seed the empty segment is legal and yields the seed (Interpreter.hs:407)
    assert same(gpu_ctx.compile(P.foldseg_sum(A.i64, A.i64, 1, 5))(vals, np.array([3, 0, 7], np.int64)),
                np.array([8, 5, 47], np.int64))


@pytest.mark.parametrize("n", [1000, 1 << 21])
def test_permute_reports_a_target_outside_the_destination(gpu_ctx, n):
    # the reference's toIndex checks the target (Shape.hs:98-106); here such a source is dropped
    # instead of written, reported, and raised by the next call that waits for the stream --
    # through both permute kernels (global atomics; workgroup-private copies from 2^20 sources on)
    keys = (np.arange(n) % 10).astype(np.int32)
    run = gpu_ctx.compile(P.histogram(10))
    assert same(run(keys), np.bincount(keys, minlength=10).astype(np.int32))
    bad = keys.copy()
    bad[n // 2] = 10
    bad[7] = -3
    res = run.execute(gpu_ctx.to_device(bad, A.tarray(1, A.i32)))
    with pytest.raises(hip.AccError, match="index out of bounds"):
        res.to_host()
    assert same(run(keys), np.bincount(keys, minlength=10).astype(np.int32))    # the context goes on


def test_issue255_endurance_blocks_are_recycled():
    # Test/NoFib/Issues/Issue255.hs: a 160 MiB array stepped a hundred times by `zipWith (+) a b`,
    # the function prepared anew for every step, old results dropped as the loop goes.  The kernel
    # cache answers every preparation after the first, and the memory table hands the dropped
    # blocks out again: device memory does not grow with the number of steps.
    ctx = hip.Context(0)
    n = 20 * 1024 * 1024
    V, S0 = A.tarray(1, A.f64), A.tarray(0, A.Int)
    step = A.alam([V, V, S0], lambda a, b, _i: A.zipwith(A.f64, A.lam([A.f64, A.f64], lambda x, y: A.add(A.f64, x, y)), a, b))
    total = A.alam([V], lambda a: A.fold(A.lam([A.f64, A.f64], lambda x, y: A.add(A.f64, x, y)), A.const(A.f64, 0), a))
    a = ctx.to_device(np.zeros(n), V)
    b = ctx.to_device(np.ones(n), V)
    after_two = None
    for i in range(101):
        go = ctx.compile(step)
        a = go.execute(a, b, ctx.to_device(np.array(i, np.int64), S0))     # the old `a` is released here
        if i == 1:
            ctx.sync()
            after_two = ctx.stat("bytes_allocated_remote")
    assert float(ctx.compile(total)(a)) == 101.0 * n
    assert ctx.stat("bytes_allocated_remote") - after_two < 8 * n       # less than one more array
    assert ctx.stat("pool_hits") >= 98
    del a, b, go
    ctx.close()


def test_issue437_identity_allocates_and_copies_nothing(gpu_ctx):
    # Test/NoFib/Issues/Issue437.hs: `runN id` applied to (unit 42, fill (Z:.10000:.10000) 1), itself
    # the result of a run: no remote allocation, nothing copied to the device beyond the unit's 4
    # bytes (here not even those: the pair was made on the device), nothing copied back until the
    # first component is read, and then its 4 bytes only.
    F = A.f32
    sh2 = A.tshape(2)
    make = A.apair(A.unit_(F, A.const(F, 42)),
                   A.generate(A.tarray(2, F), A.sh(A.constI(10000), A.constI(10000)), A.lam([sh2], lambda ix: A.const(F, 1))))
    xs = gpu_ctx.compile(make).execute()
    go = gpu_ctx.compile(Q.issue437())
    gpu_ctx.sync()
    names = ("bytes_allocated_remote", "bytes_copied_to_remote", "bytes_copied_from_remote")
    before = [gpu_ctx.stat(n) for n in names]
    res = go.execute(xs)
    gpu_ctx.sync()
    assert [gpu_ctx.stat(n) for n in names] == before
    a, b = res.parts()
    assert a.to_host() == np.float32(42) and b.shape == (10000, 10000)
    assert gpu_ctx.stat("bytes_copied_from_remote") - before[2] == 4


def test_issue286_repeated_runs_hold_memory_steady(gpu_ctx):
    # Test/NoFib/Issues/Issue286.hs ("check heap profile"): the same prepared function applied to a
    # fresh 120x659 matrix of Word8 over and over; every run's blocks come back from the pool
    go = gpu_ctx.compile(Q.issue286())
    ones = np.ones((120, 659), np.uint8)
    total, steady = 0.0, None
    for n in range(300):
        total += float(go(ones))
        if n == 4:
            steady = gpu_ctx.stat("bytes_allocated_remote")
    assert total == 300 * 79080.0
    assert gpu_ctx.stat("bytes_allocated_remote") == steady


def test_awhile_jacobi_counts_iterations(gpu_ctx):
    # 20 sweeps driven by awhile (Interpreter.hs:222-229).  The loop counter is a rank-0
    # array made by `unit` from index arithmetic, so the host follows its value and the
    # predicate costs no read-back: the only bytes that come back are the result's.
    from .runtime_cases import jacobi_awhile
    g = np.random.default_rng(1).uniform(0, 1, (40, 56)).astype(np.float32)
    run = gpu_ctx.compile(jacobi_awhile(20))
    dg = gpu_ctx.to_device(g, A.tarray(2, A.f32))
    before = gpu_ctx.stat("bytes_copied_from_remote")
    res = run.execute(dg)
    assert gpu_ctx.stat("bytes_copied_from_remote") == before
    assert same(res.to_host(), OC.jacobi_f32(g, 20))


def test_pool_reuses_blocks_and_counts_bytes(gpu_ctx):
    ctx = gpu_ctx
    before_hits, before_alloc = ctx.stat("pool_hits"), ctx.stat("bytes_allocated_remote")
    ctx.purge()                                     # start from empty free lists
    before_hits, before_alloc = ctx.stat("pool_hits"), ctx.stat("bytes_allocated_remote")
    p = ctx.malloc(7777777)
    rounded = (7777777 + 1023) // 1024 * 1024       # requests are rounded up to 1 KiB chunks
    assert p and ctx.stat("bytes_allocated_remote") - before_alloc == rounded
    ctx.free(p)
    q = ctx.malloc(rounded - 5)                     # same size class: the freed block comes back
    assert q == p and ctx.stat("pool_hits") == before_hits + 1
    ctx.free(q)
    evicted = ctx.stat("bytes_evicted_from_remote")
    ctx.purge()
    assert ctx.stat("bytes_evicted_from_remote") - evicted == rounded
    total, avail = ctx.mem_info()
    assert 0 < avail <= total


def test_poke_peek_round_trip_and_events(gpu_ctx):
    import ctypes as C
    from accelerate_amd import hip
    ctx = gpu_ctx
    x = np.random.default_rng(2).integers(0, 255, 3 << 20, dtype=np.uint8)
    p = ctx.malloc(x.nbytes)
    e0 = ctx.event()
    assert hip.lib().acchip_poke(ctx._h, p, x.ctypes.data, x.nbytes) == 0
    y = np.empty_like(x)
    assert hip.lib().acchip_peek(ctx._h, y.ctypes.data, p, y.nbytes) == 0
    e1 = ctx.event()
    e1.sync()
    assert e1.done() and e0.elapsed_ms(e1) >= 0 and np.array_equal(x, y)
    ctx.free(p)


def test_results_stay_on_the_device_between_calls(gpu_ctx):
    # run1 applied repeatedly: the result handle of one call is the argument of the next
    step = gpu_ctx.compile(P.map_affine())
    d = gpu_ctx.to_device(np.ones(1000, np.float32), A.tarray(1, A.f32))
    copied = gpu_ctx.stat("bytes_copied_from_remote")
    for _ in range(5):
        d = step.execute(d)
    assert gpu_ctx.stat("bytes_copied_from_remote") == copied
    assert np.all(d.to_host() == 63.0)      # x -> 2x+1 five times from 1


def test_handles_may_be_released_after_shutdown():
    # arrays, results, events and programs released after acchip_shutdown, in any order
    ctx = hip.Context(0)
    run = ctx.compile(P.map_affine())
    x = np.arange(1000, dtype=np.float32)
    dx = ctx.to_device(x, A.tarray(1, A.f32))
    res = run.execute(dx)
    ev = ctx.event()
    host = res.to_host()
    ctx.close()
    del dx
    del run
    del ev
    del res
    assert np.array_equal(host, 2 * x + 1)


def test_array_table_evicts_and_uploads_again_on_a_real_device(monkeypatch):
    # the ladder of tests/test_memory_manager.py against the GPU, the budget standing in for a
    # full device: 5 arrays of 96 MiB under 256 MiB, each read by a program between use and release
    # (its transfers take several pieces of the staging buffers)
    monkeypatch.setenv("ACCHIP_POOL_LIMIT", str(256 << 20))
    ctx = hip.Context(0)
    try:
        n = 24 << 20
        V = A.tarray(1, A.i32)
        total = ctx.compile(P.fold_sum(A.i32, 1, 0))
        host = {k: np.full(n, k, np.int32) for k in range(1, 6)}
        lib = hip.lib()

        def fold_of(k):
            ptr = ctx.table_use(k)
            h = C.c_void_p()
            shp = (C.c_int64 * 1)(n)
            bufs = (C.c_void_p * 1)(ptr)
            hip._check(lib.acchip_array_wrap(ctx._h, 1, shp, b"i32", bufs, 1, C.byref(h)))
            arr = hip.DeviceArray(ctx, h)
            res = total.execute(arr)
            ctx.table_release(k)                      # the fold may still be running: the event guards the block
            return int(res.to_host())

        for k in host:
            assert ctx.table_malloc(k, host[k], frozen=True)
            ctx.poke(ctx.table_use(k), host[k])
            ctx.table_release(k)
        # 5 x 96 MiB do not fit 256 MiB: the eldest were evicted on the way
        assert ctx.stat("arrays_evicted") >= 3
        assert sorted(ctx.table_status(k) for k in host).count(3) >= 3
        for k in (1, 2, 3, 4, 5, 1, 3, 5):           # every use of an evicted array uploads it again
            assert fold_of(k) == k * n
        total_avail = ctx.mem_info()
        assert total_avail[0] == 256 << 20
        # the budget also binds what programs allocate themselves: a map over 96 MiB needs a second block of
        # 96 MiB, which evicts table arrays; one over 200 MiB cannot be served at all
        ptr = ctx.table_use(2)
        ctx.table_release(2)
        big = ctx.compile(P.map_affine())
        with pytest.raises(hip.AccError, match="Remote memory exhausted") as e:
            big(np.zeros(50 << 20, np.float32))
        assert e.value.code == 3
    finally:
        ctx.close()


def test_transfers_of_many_pieces_round_trip(gpu_ctx):
    # 200 MiB + 12 bytes through the two 32 MiB staging buffers, both directions
    x = np.random.default_rng(5).integers(0, 255, (200 << 20) + 12).astype(np.uint8)
    p = gpu_ctx.malloc(x.nbytes)
    gpu_ctx.poke(p, x)
    y = np.empty_like(x)
    gpu_ctx.peek(y, p)
    gpu_ctx.free(p)
    assert np.array_equal(x, y)
