"""Every program the GPU suite runs is first generated and compiled for gfx950 here, with no
GPU: this catches code-generation errors on the CPU and leaves the code objects in the
in-tree kernel cache that travels to the GPU box.  The oracle is run on the same programs
so that a case the oracle cannot evaluate fails here and not on the GPU box."""
import pytest

from oracle import interp as O

from .cases import gpu_only_programs, parity_cases
from .runtime_cases import jacobi_awhile, runtime_cases
from .scalar_cases import scalar_cases


def _compile_all(cc_ctx, named_programs):
    seen = set()
    for cid, prog in named_programs:
        text = prog.text()
        if text in seen:
            continue
        seen.add(text)
        try:
            assert cc_ctx.compile(prog).num_kernels >= 0
        except Exception as e:  # name the program that failed
            pytest.fail("%s: %s" % (cid, e))


def test_all_parity_programs_compile(cc_ctx):
    from .test_gpu_permute_lds import lds_programs
    _compile_all(cc_ctx, [(c[0], c[1]) for c in parity_cases()] + [(c[0], c[1]) for c in lds_programs()] +
                 gpu_only_programs())


def test_all_scalar_programs_compile_and_oracle_evaluates_them(cc_ctx):
    cases = scalar_cases()
    _compile_all(cc_ctx, [(c[0], c[1]) for c in cases])
    for cid, prog, args, _ in cases:
        try:
            O.run_n(prog.text(), *args)
        except Exception as e:
            pytest.fail("oracle on %s: %r" % (cid, e))


def test_all_runtime_programs_compile_and_oracle_evaluates_them(cc_ctx):
    cases = runtime_cases()
    _compile_all(cc_ctx, [(c[0], c[1]) for c in cases] + [("jacobi_awhile", jacobi_awhile(20))])
    for cid, prog, args, uses in cases:
        try:
            O.run_n(prog.text(), *args, uses=[O.to_arr(u, t) for u, t in uses])
        except Exception as e:
            pytest.fail("oracle on %s: %r" % (cid, e))


def test_programs_print_to_the_committed_term_texts():
    # tests/golden/terms/*.sx are the exact texts of every named program of the suite -- the five
    # configurations, the reference's doctest and issue programs, the control-flow programs, the
    # property-shaped cases and whole programs: the golden files of any printer of the wire format
    # (the Haskell serialiser must produce these bytes for the same programs), so the Python
    # builder must not drift from them either.  tests/golden/make_terms.py writes them.
    import os
    from .golden.make_terms import named_terms
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "terms")
    terms = named_terms()
    assert {"c1_dotp", "c2_scanl1_i64", "c2_scanl1_f32", "c3_foldseg", "c4_histogram", "c5_jacobi_step"} <= set(terms)
    assert sorted(f[:-3] for f in os.listdir(here) if f.endswith(".sx")) == sorted(terms)
    for name, text in terms.items():
        assert open(os.path.join(here, name + ".sx")).read() == text + "\n", name


def test_committed_term_texts_are_accepted_by_the_library(cc_ctx):
    # and the library reads every one of them as it stands in the file
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "terms")
    for f in sorted(os.listdir(here)):
        if f.endswith(".sx"):
            try:
                assert cc_ctx.compile(open(os.path.join(here, f)).read().rstrip("\n")).num_kernels >= 0
            except Exception as e:
                pytest.fail("%s: %s" % (f, e))


def test_unknown_wire_version_is_refused(cc_ctx):
    from accelerate_amd import hip, ir as A, programs as P
    text = P.scanl1_sum(A.i64).text()
    assert text.startswith("(acchip-ir 1 ")
    bare = text[len("(acchip-ir 1 "):-1]
    assert cc_ctx.compile(bare).num_kernels >= 1               # a bare term is version 1
    with pytest.raises(hip.AccError, match="wire format version 2"):
        cc_ctx.compile("(acchip-ir 2 " + bare + ")")


def test_scan_phase_stamps_still_fit_the_kernel():
    # accelerate_amd/scan_phases.py rebuilds acc_scan_pipe with time stamps put in by text
    # substitution: building it here shows that every place it names is still there and that the
    # instrumented kernel compiles for gfx950
    import os
    from accelerate_amd import scan_phases
    exe = scan_phases.build("i64")
    assert os.path.exists(exe)
