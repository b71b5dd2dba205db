"""Scalar language parity (evalOpenExp / evalPrim, Interpreter.hs:912-1416): every primitive
and control construct, generated HIP C++ against the oracle's restatement of the Haskell
semantics.  Integer and boolean results bit-exact; correctly-rounded float operations
bit-exact; transcendental functions within a few units in the last place."""
import numpy as np
import pytest

from oracle import interp as O

from .cases import same
from .scalar_cases import scalar_cases

pytestmark = pytest.mark.gpu
CASES = scalar_cases()


def _ulp_close(a, b, ulps):
    if isinstance(a, (list, tuple)):
        return all(_ulp_close(x, y, ulps) for x, y in zip(a, b))
    a, b = np.asarray(a), np.asarray(b)
    if a.shape != b.shape:
        return False
    both_nan = np.isnan(a) & np.isnan(b)
    spacing = np.spacing(np.maximum(np.abs(a), np.abs(b)).astype(a.dtype))
    with np.errstate(invalid="ignore"):
        ok = (np.abs(a.astype(np.float64) - b.astype(np.float64)) <= ulps * spacing.astype(np.float64)) | (a == b)
    return bool(np.all(ok | both_nan))


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_scalar_semantics(gpu_ctx, case):
    _, prog, args, ulps = case
    got = gpu_ctx.compile(prog)(*args)
    exp = O.run_n(prog.text(), *args)
    if ulps is None:
        assert same(got, exp), (got, exp)
    else:
        assert _ulp_close(got, exp, ulps)
