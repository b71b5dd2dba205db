"""acchip_execute_into: the entry point that allocates no device memory (scans whose tile
descriptors and ticket live in a static device array) against acchip_execute, through the C ABI.

Integer scans must agree bit for bit; Float32 within 1e-4 * sum |x_i| per prefix, the tolerance
of the scan configuration.  Every case runs two calls in a row on the same context, the second
on a smaller input, so that whatever the first call left in the static array is met by the second.
"""
import numpy as np
import pytest

from accelerate_amd import hip, ir as A, programs as P, workloads as W

pytestmark = pytest.mark.gpu


def _both(ctx, prog, x, aty, out_shape, pair_shape=None):
    """(result of acchip_execute, result of acchip_execute_into) as numpy"""
    d = ctx.to_device(x, aty)
    want = prog.execute(d).to_host()
    dest = ctx.empty(out_shape, aty)
    if pair_shape is not None:
        tot = ctx.empty(pair_shape, ("array", len(pair_shape), aty[2]))
        dest = ctx.pair(dest, tot)
    # the pool's counters, and the library's count of every allocation it asks the runtime for
    # outside the pool (hipMalloc, hipMallocAsync, hipHostMalloc) and of code objects it loads
    names = ("bytes_allocated_remote", "pool_hits", "pool_misses", "raw_allocs", "modules_loaded")
    before = [ctx.stat(n) for n in names]
    prog.execute_into(dest, d)
    after = [ctx.stat(n) for n in names]
    assert before == after, "acchip_execute_into allocated or loaded something: %s" % dict(zip(names, zip(before, after)))
    got = dest.to_host()
    return want, got


@pytest.mark.parametrize("sizes", [(3_000_000, 100_000), (1_000_000, 1000), (50_000, 7)])
def test_scanl1_int64_two_calls(gpu_ctx, sizes):
    prog = gpu_ctx.compile(P.scanl1_sum(A.i64))
    aty = A.tarray(1, A.i64)
    for k, n in enumerate(sizes):
        x = W.uniform_int(n, 11 + k)
        want, got = _both(gpu_ctx, prog, x, aty, (n,))
        assert np.array_equal(got, want)
        assert np.array_equal(got, np.cumsum(x))


def test_scanl_seeded_and_right_scans_int32(gpu_ctx):
    aty = A.tarray(1, A.i32)
    for direction in ("l", "r"):
        prog = gpu_ctx.compile(P.scan_sum(direction, A.i32, z=5))
        for k, n in enumerate((2_500_000, 300_000)):
            x = W.uniform_int(n, 21 + k, dtype=np.int32)
            want, got = _both(gpu_ctx, prog, x, aty, (n + 1,))
            assert np.array_equal(got, want)


def test_scan_prime_pair_result(gpu_ctx):
    aty = A.tarray(1, A.i64)
    prog = gpu_ctx.compile(P.scan_prime_sum("l", A.i64, z=3))
    for k, n in enumerate((2_000_000, 4097)):
        x = W.uniform_int(n, 31 + k)
        want, got = _both(gpu_ctx, prog, x, aty, (n,), pair_shape=())
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
        assert int(got[1]) == 3 + int(x.sum())


def test_rows_of_a_matrix(gpu_ctx):
    aty = A.tarray(2, A.i64)
    prog = gpu_ctx.compile(P.scanl1_sum(A.i64, rank=2))
    for k, shape in enumerate(((7, 400_000), (300, 5000), (1000, 20))):
        x = W.uniform_int(shape[0] * shape[1], 41 + k).reshape(shape)
        want, got = _both(gpu_ctx, prog, x, aty, shape)
        assert np.array_equal(got, want)
        assert np.array_equal(got, np.cumsum(x, axis=1))


def test_scanl1_float32_within_tolerance(gpu_ctx):
    aty = A.tarray(1, A.f32)
    prog = gpu_ctx.compile(P.scanl1_sum(A.f32))
    for k, n in enumerate((4_000_000, 123_457)):
        x = W.uniform_f32(n, 51 + k, 0.0, 1.0)
        want, got = _both(gpu_ctx, prog, x, aty, (n,))
        ref = np.cumsum(x.astype(np.float64))
        bound = 1e-4 * np.cumsum(np.abs(x.astype(np.float64)))
        assert np.all(np.abs(got - ref) <= bound)
        assert np.all(np.abs(got - want) <= bound)


def test_long_float32_row_takes_the_pipelined_kernel(gpu_ctx):
    # long rows of 4-byte elements run the persistent pipelined kernel in both entry points (its
    # code object is loaded at compile time like the others); a second, shorter call follows
    aty = A.tarray(1, A.f32)
    prog = gpu_ctx.compile(P.scanl1_sum(A.f32))
    for k, n in enumerate(((1 << 26) + 5, 40_000_003)):
        x = W.uniform_f32(n, 61 + k, 0.0, 1.0)
        want, got = _both(gpu_ctx, prog, x, aty, (n,))
        ref = np.cumsum(x.astype(np.float64))
        assert np.all(np.abs(got - ref) <= 1e-4 * ref) and np.all(np.abs(got - want) <= 1e-4 * ref)


def test_refusals_launch_nothing(gpu_ctx):
    # not a scan
    prog = gpu_ctx.compile(P.map_affine())
    x = gpu_ctx.to_device(W.uniform_f32(1000, 1), A.tarray(1, A.f32))
    dest = gpu_ctx.empty((1000,), A.tarray(1, A.f32))
    with pytest.raises(hip.AccError, match="single scan"):
        prog.execute_into(dest, x)
    # wrong extents of the result
    scan = gpu_ctx.compile(P.scanl1_sum(A.i64))
    xi = gpu_ctx.to_device(W.uniform_int(1000, 2), A.tarray(1, A.i64))
    with pytest.raises(hip.AccError, match="wrong extents"):
        scan.execute_into(gpu_ctx.empty((999,), A.tarray(1, A.i64)), xi)
    with pytest.raises(hip.AccError, match="wrong type"):
        scan.execute_into(gpu_ctx.empty((1000,), A.tarray(1, A.i32)), xi)
    # more tiles than the static array has descriptors for: 70000 rows of one tile each (too long
    # for a workgroup to take several of them), two descriptor words per Int64 tile,
    # against 131072 words (arrays left uninitialised: the call fails before anything is launched)
    rows = gpu_ctx.compile(P.scanl1_sum(A.i64, rank=2))
    shape = (70_000, 4200)
    big = gpu_ctx.empty(shape, A.tarray(2, A.i64))
    launches = gpu_ctx.stat("launches")
    with pytest.raises(hip.AccError, match="static scratch"):
        rows.execute_into(gpu_ctx.empty(shape, A.tarray(2, A.i64)), big)
    assert gpu_ctx.stat("launches") == launches
    # the existing entry point takes the same input
    rows.execute(big).release()
    gpu_ctx.sync()
