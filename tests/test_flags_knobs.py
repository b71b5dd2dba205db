"""The option word of the reference (cbits/flags.h:19-49) and the launch knobs: both belong to a
context, are read from the environment once when it is made, and change afterwards only through
the C ABI."""
import numpy as np
import pytest

from accelerate_amd import hip, ir as A
from accelerate_amd import programs as P
from tests import progs as Q
from oracle import interp as O

C = hip.Context


def test_flag_word_defaults_and_names(monkeypatch):
    monkeypatch.delenv("ACCHIP_FLAGS", raising=False)
    c = C(-1)
    assert c.flags == C.FLAG_INPLACE | C.FLAG_FAST_PERMUTE_CONST
    c.flags = c.flags | C.FLAG_DUMP_GC
    assert c.flags & C.FLAG_DUMP_GC
    c.close()
    monkeypatch.setenv("ACCHIP_FLAGS", "no-inplace,fast-math -dforce-recomp no-fast-permute-const")
    c = C(-1)
    assert c.flags == C.FLAG_FAST_MATH | C.FLAG_FORCE_RECOMP
    c.close()
    monkeypatch.setenv("ACCHIP_FLAGS", "dump-exec-not-a-flag xdump-cc inplace")
    c = C(-1)
    assert c.flags == C.FLAG_INPLACE | C.FLAG_FAST_PERMUTE_CONST   # neither near-miss is a name
    c.close()


def test_knobs_come_from_the_environment_once(monkeypatch):
    monkeypatch.setenv("ACCHIP_SCAN_TILES", "small")
    monkeypatch.setenv("ACCHIP_STREAM_BYTES", "12345")
    c = C(-1)
    assert c.knob("scan_tiles") == 2 and c.knob("stream_bytes") == 12345 and c.knob("fold_target") == 2048
    monkeypatch.setenv("ACCHIP_STREAM_BYTES", "777")          # too late for this context
    assert c.knob("stream_bytes") == 12345
    assert c.set_knob("stream_bytes", 9) == 12345 and c.knob("stream_bytes") == 9
    with pytest.raises(hip.AccError, match="no such knob"):
        c.set_knob("warp_speed", 1)
    c.close()


def test_fast_math_is_part_of_the_kernel_key(tmp_path, monkeypatch):
    monkeypatch.setenv("ACCHIP_CACHE_DIR", str(tmp_path))
    c = C(-1)
    exact = c.compile(P.dotp()).kernel_keys
    c.flags = c.flags | C.FLAG_FAST_MATH
    fast = c.compile(P.dotp()).kernel_keys                  # compiles with the relaxed options
    assert exact and len(exact) == len(fast) and not set(exact) & set(fast)
    assert c.stat("kernels_compiled") == len(exact) + len(fast)
    c.close()


def test_fast_permute_const_picks_the_update(cc_ctx):
    # pairs: plain stores of the two halves when the flag is on, per-element locks when off;
    # one 64-bit value is a single store either way
    pair = A.ttup(A.Int, A.Int)
    before = cc_ctx.flags
    try:
        on_pair, on_one = cc_ctx.compile(Q.scatter(pair)).kernel_keys, cc_ctx.compile(Q.scatter(A.Int)).kernel_keys
        cc_ctx.flags = before & ~C.FLAG_FAST_PERMUTE_CONST
        off_pair, off_one = cc_ctx.compile(Q.scatter(pair)).kernel_keys, cc_ctx.compile(Q.scatter(A.Int)).kernel_keys
    finally:
        cc_ctx.flags = before
    assert on_pair != off_pair and on_one == off_one


@pytest.mark.gpu
def test_permute_const_over_pairs_is_whole_either_way(gpu_ctx):
    # many sources per target: which one wins is open (Language.hs:778-790), but with the flag
    # off every element must be one complete source pair; with it on and distinct targets the
    # result is the oracle's
    pair = A.ttup(A.Int, A.Int)
    rng = np.random.default_rng(11)
    n, m = 1 << 18, 257
    to = rng.integers(0, m, n).astype(np.int64)
    a = np.arange(n, dtype=np.int64)
    xs = (a, a * 3 + 1)
    over = (np.full(m, -1, np.int64), np.full(m, -2, np.int64))
    before = gpu_ctx.flags
    try:
        gpu_ctx.flags = before & ~C.FLAG_FAST_PERMUTE_CONST
        r0, r1 = gpu_ctx.compile(Q.scatter(pair))(to, over, xs)
    finally:
        gpu_ctx.flags = before
    assert np.array_equal(r1, r0 * 3 + 1) and np.array_equal(to[r0], np.arange(m))
    perm = rng.permutation(n).astype(np.int64)
    over = (np.zeros(n, np.int64), np.zeros(n, np.int64))
    prog = Q.scatter(pair)
    got = gpu_ctx.compile(prog)(perm, over, xs)
    exp = O.run_n(prog.text(), perm, over, xs)
    assert all(np.array_equal(g, e) for g, e in zip(got, exp))


@pytest.mark.gpu
def test_no_inplace_copies_the_defaults_and_agrees(gpu_ctx):
    prog = Q.identity_permute(A.Int)
    n = np.array(37, np.int64)
    want = gpu_ctx.compile(prog)(n)
    before = gpu_ctx.flags
    try:
        gpu_ctx.flags = before & ~C.FLAG_INPLACE
        got = gpu_ctx.compile(prog)(n)
    finally:
        gpu_ctx.flags = before
    assert np.array_equal(got, want) and np.array_equal(got, np.eye(37, dtype=np.int64))


@pytest.mark.gpu
def test_fast_math_stays_within_rounding_of_exact(gpu_ctx):
    rng = np.random.default_rng(12)
    x, y = rng.random(1 << 20, dtype=np.float32), rng.random(1 << 20, dtype=np.float32)
    exact = gpu_ctx.compile(P.dotp())(x, y)
    before = gpu_ctx.flags
    try:
        gpu_ctx.flags = before | C.FLAG_FAST_MATH
        fast = gpu_ctx.compile(P.dotp())(x, y)
    finally:
        gpu_ctx.flags = before
    # tolerance: n * eps * sum|x y| bounds any order of summation and contraction
    assert abs(float(fast) - float(exact)) <= (1 << 20) * 2.0 ** -24 * float(np.dot(x.astype(np.float64), y))
