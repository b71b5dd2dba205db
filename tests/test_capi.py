"""Host-side checks that need no GPU: the shared library loads and exports every symbol
that include/acchip.h declares, the digest matches FIPS 202 and the reference's own SHA3
build, programs compile for gfx950 through the C ABI (code generation + hipRTC), and
errors come back as codes + messages instead of exceptions or crashes."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from accelerate_amd import hip
from accelerate_amd import ir as A
from accelerate_amd import programs as P
from oracle import c as OC

from . import progs as Q
from .cases import golden_cases

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "acchip.h")).read()
    declared = sorted(set(re.findall(r"\b(acchip_[a-z0-9_]+)\s*\(", header)))
    assert len(declared) >= 35
    lib = C.CDLL(hip.LIB_PATH)
    missing = [s for s in declared if not hasattr(lib, s)]
    assert not missing, missing
    assert set(hip.lib()._declared) <= set(declared)


def _sha3(data):
    out = C.create_string_buffer(32)
    assert hip.lib().acchip_sha3_256(data, len(data), out) == 0
    return out.raw


def test_sha3_256_known_answers():
    # FIPS 202 known-answer vectors
    assert _sha3(b"").hex() == "a7ffc6f8bf1ed76651c14756a061d662f580ff4de43b49fa82d80a4b80f8434a"
    assert _sha3(b"abc").hex() == "3a985da74fe225b2045c172d6bd390bd855f086e3e9d525b46bfe24511431532"
    assert _sha3(b"a" * 200).hex() == _sha3(b"a" * 200).hex()


def test_sha3_256_matches_reference_build():
    rng = np.random.default_rng(0)
    if OC.ref_sha3_256(b"x") is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    for n in [0, 1, 135, 136, 137, 271, 272, 273, 1000, 4096]:
        data = rng.integers(0, 256, n, dtype=np.uint8).tobytes()
        assert _sha3(data) == OC.ref_sha3_256(data), n


GOLDEN = golden_cases()


@pytest.mark.parametrize("case", GOLDEN, ids=[c[0] for c in GOLDEN])
def test_programs_compile_for_gfx950(cc_ctx, case):
    prog = cc_ctx.compile(case[1])
    assert prog.num_kernels >= 1


def test_benchmark_programs_compile(cc_ctx):
    for p in [P.dotp(), P.scanl1_sum(A.i64), P.scanl1_sum(A.f32), P.foldseg_sum(), P.histogram(1 << 16),
              P.jacobi_step(), P.map_affine()]:
        assert cc_ctx.compile(p).num_kernels >= 1


def test_kernel_cache_is_shared_between_equal_terms(cc_ctx):
    cc_ctx.compile(P.fold_sum(A.i32, 2, 3))
    before = cc_ctx.stat("kernels_from_memory")
    cc_ctx.compile(P.fold_sum(A.i32, 2, 3))     # same term, any shape: same code
    assert cc_ctx.stat("kernels_from_memory") == before + 1


def test_disk_cache_round_trip_and_damaged_entries(tmp_path, monkeypatch):
    # a second context finds the code object on disk; an entry that is not a code object (here:
    # overwritten with text) is compiled anew instead of being handed to the loader
    monkeypatch.setenv("ACCHIP_CACHE_DIR", str(tmp_path))
    prog = P.fold_sum(A.i64, 1, 7)
    c1 = hip.Context(-1)
    c1.compile(prog)
    assert c1.stat("kernels_compiled") >= 1
    c1.close()
    files = sorted(tmp_path.glob("*.hsaco"))
    assert files and all(f.read_bytes()[:4] == b"\x7fELF" for f in files)
    c2 = hip.Context(-1)
    c2.compile(prog)
    assert c2.stat("kernels_from_disk") == len(files) and c2.stat("kernels_compiled") == 0
    c2.close()
    files[0].write_bytes(b"not a code object" * 10)
    c3 = hip.Context(-1)
    c3.compile(prog)
    assert c3.stat("kernels_compiled") == 1 and c3.stat("kernels_from_disk") == len(files) - 1
    c3.close()
    assert files[0].read_bytes()[:4] == b"\x7fELF"


def test_errors_are_reported_not_thrown(cc_ctx):
    with pytest.raises(hip.AccError) as e:
        cc_ctx.compile("(alam (single (array 1 f32)) (fold (lam (single f32) 3) nothing (avar 0)")
    assert "unbalanced" in str(e.value)
    with pytest.raises(hip.AccError) as e:
        cc_ctx.compile("(alam (single (array 1 f32)) (frobnicate (avar 0)))")
    assert "unsupported array term" in str(e.value)
    bad = A.alam([A.tarray(1, A.f32)], lambda xs: A.fold(Q.binop(A.add, A.i32), None, xs))
    with pytest.raises(hip.AccError):
        cc_ctx.compile(bad)                      # type error inside the scalar code
    ok = cc_ctx.compile(P.dotp())
    with pytest.raises(hip.AccError) as e:
        ok.execute(hip.DeviceArray(cc_ctx, C.c_void_p()), hip.DeviceArray(cc_ctx, C.c_void_p()))
    assert e.value.code == 2                     # ACCHIP_NO_DEVICE: nothing falls back to the CPU
    assert cc_ctx.malloc(1024) is None           # mallocRemote without a device: NULL, no abort


def test_program_may_outlive_its_context():
    # finalisers run in any order: a program released after acchip_shutdown must not touch
    # freed memory (the context lives until its last handle is gone)
    ctx = hip.Context(-1)
    prog = ctx.compile(P.dotp())
    assert prog.num_kernels >= 1
    ctx.close()
    del prog
