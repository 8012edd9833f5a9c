"""
The float32 functions that generated code takes from the device math library (sin, cos, tan, arcsin, arccos, arctan,
sinh, cosh, log10, sqrt, power, arctan2; the reference's generated C++ calls the host C library for them,
opveclib/expression.py:1430-1456, 1632-1672): a strided sweep over all float32 bit patterns (about one million
arguments per function, every exponent, both signs, subnormals, infinities, NaNs) and one million operand pairs for
the two-argument functions, against the CPU oracle.  The stated tolerance for transcendental operators is two units in
the last place; NaN results must coincide.
"""
import numpy as np
import pytest

import opveclib_amd as ovl
import oracle
from tests import cases

pytestmark = pytest.mark.gpu

SWEEPS = dict(cases.library_sweep_outputs())


@pytest.mark.parametrize('name', sorted(SWEEPS))
def test_library_function_within_two_ulp_of_the_oracle(name):
    out = SWEEPS[name]
    want = oracle.evaluate(out)
    got = ovl.evaluate(out, opt_level=0)
    assert got.dtype == want.dtype and got.shape == want.shape
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan), name + ': NaN pattern differs'
    dist = cases.ulp_distance(np.where(nan, 0, got).astype(np.float32), np.where(nan, 0, want).astype(np.float32))
    worst = int(dist.max())
    assert worst <= 2, '%s: %d ulp, %d of %d arguments beyond 2' % (name, worst, int((dist > 2).sum()), dist.size)
