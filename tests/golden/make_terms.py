"""Writes tests/golden/terms/: the wire-format text of every named program the test-suite runs.

The files are the golden output of any printer of the wire format (docs/WIRE.md): the Haskell
serialiser (accelerate-hip/.../Serialise.hs) must print these bytes for the same surface programs,
and accelerate_amd/ir.py must keep printing them (tests/test_programs_compile.py compares).  One
file per distinct program text, named after the first test case that uses it:

  c*_...   the five benchmark configurations
  g_...    programs of the reference's doctest / issue vectors (tests/cases.py golden_cases)
  r_...    array-level control flow (tests/runtime_cases.py)
  p_...    property-shaped parity cases and whole programs (tests/cases.py, tests/progs.py)

Run from the repository root:  python -m tests.golden.make_terms
"""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def _safe(cid):
    return re.sub(r"[^A-Za-z0-9_.-]+", "_", cid).strip("_")


def named_terms():
    """{file name without .sx: program text}"""
    from accelerate_amd import ir as A, programs as P
    from tests.cases import golden_cases, gpu_only_programs, parity_cases
    from tests.runtime_cases import jacobi_awhile, runtime_cases
    out, seen = {}, set()

    def add(name, prog):
        text = prog.text()
        if text in seen:
            return
        seen.add(text)
        base, k = name, 2
        while name in out:          # two ids that sanitise alike
            name = "%s_%d" % (base, k)
            k += 1
        out[name] = text

    for name, prog in (("c1_dotp", P.dotp()), ("c2_scanl1_i64", P.scanl1_sum(A.i64)), ("c2_scanl1_f32", P.scanl1_sum(A.f32)),
                       ("c3_foldseg", P.foldseg_sum()), ("c4_histogram", P.histogram(1 << 16)), ("c5_jacobi_step", P.jacobi_step())):
        add(name, prog)
    for c in golden_cases():
        add("g_" + _safe(c[0]), c[1])
    for c in runtime_cases():
        add("r_" + _safe(c[0]), c[1])
    add("r_jacobi_awhile_20", jacobi_awhile(20))
    for c in parity_cases():
        add("p_" + _safe(c[0]), c[1])
    for cid, prog in gpu_only_programs():
        add("p_" + _safe(cid), prog)
    return out


def main():
    d = os.path.join(HERE, "terms")
    os.makedirs(d, exist_ok=True)
    terms = named_terms()
    for f in os.listdir(d):
        if f.endswith(".sx") and f[:-3] not in terms:
            os.remove(os.path.join(d, f))
    for name, text in terms.items():
        with open(os.path.join(d, name + ".sx"), "w") as f:
            f.write(text + "\n")
    print("wrote", len(terms), "term texts to", d)


if __name__ == "__main__":
    main()
