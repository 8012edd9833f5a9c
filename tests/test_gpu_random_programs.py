"""Random element-wise programs (tests/random_programs.py) through the HIP path, with and without the value-range
pruning, against the CPU oracle: bit-exact apart from the sign and payload of NaN; in the 'ulp2' math mode within two
float32 steps (a one-off sweep of 120 programs, in which the mode chose the cheap routine at 186 call sites, found
no output further away)."""
import numpy as np
import pytest

import opveclib_amd as ovl
import oracle
from opveclib_amd import runtime
from tests import random_programs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('seed', random_programs.GPU_SEEDS)
def test_random_program_equals_the_oracle(seed):
    op = random_programs.application(seed)
    outs = [op[0], op[1]]
    ref = oracle.evaluate(outs)
    for options in ({}, {'value_ranges': False}):
        runtime.codegen_options = dict(options)
        try:
            got = ovl.evaluate(outs, opt_level=0)
        finally:
            runtime.codegen_options = {}
        for k, (g, r) in enumerate(zip(got, ref)):
            equal = ((g == r) & (np.signbit(g) == np.signbit(r))) | (np.isnan(g) & np.isnan(r))
            assert equal.all(), 'seed %d %r output %d: %d elements differ' % (seed, options, k, int((~equal).sum()))
    # the fast math mode evaluates the same program without error
    ovl.evaluate(outs, opt_level=0, math_mode='fast')
    # the 'ulp2' mode keeps its promise on arbitrary programs: every output within two float32 steps of the oracle,
    # NaN and infinities in the same places (an inexact value never decides a branch)
    from tests import cases
    got = ovl.evaluate(outs, opt_level=0, math_mode='ulp2')
    for k, (g, r) in enumerate(zip(got, ref)):
        nan = np.isnan(r)
        assert np.array_equal(np.isnan(g), nan), 'seed %d output %d: NaN pattern differs in ulp2 mode' % (seed, k)
        assert np.array_equal(np.isinf(g), np.isinf(r)), 'seed %d output %d: infinities differ in ulp2 mode' % (seed, k)
        distance = cases.ulp_distance(np.where(nan, 0, g).astype(np.float32), np.where(nan, 0, r).astype(np.float32))
        assert int(distance.max()) <= 2, 'seed %d output %d: %d ulp in ulp2 mode' % (seed, k, int(distance.max()))


@pytest.mark.parametrize('seed', random_programs.DAG_SEEDS)
def test_random_dag_fused_and_unfused_equal_the_oracle(seed):
    outs = random_programs.random_dag(seed)
    ref = oracle.evaluate(outs)
    ref = ref if isinstance(ref, list) else [ref]
    for opt_level in (0, 3):
        got = ovl.evaluate(outs, opt_level=opt_level)
        got = got if isinstance(got, list) else [got]
        for k, (g, r) in enumerate(zip(got, ref)):
            equal = ((g == r) & (np.signbit(g) == np.signbit(r))) | (np.isnan(g) & np.isnan(r))
            assert equal.all(), 'seed %d opt_level %d output %d: %d elements differ' % (
                seed, opt_level, k, int((~equal).sum()))


@pytest.mark.parametrize('seed', random_programs.INDEX_SEEDS)
def test_random_index_program_equals_the_oracle(seed):
    """Gathers through computed indices, guarded neighbour reads and stores through one-to-one index maps: bit-exact
    (unwritten elements would show as the 0xFE fill)."""
    op = random_programs.index_application(seed)
    outs = [op[0], op[1]]
    ref = oracle.evaluate(outs)
    runtime.poison_outputs = True
    try:
        got = ovl.evaluate(outs, opt_level=3)
    finally:
        runtime.poison_outputs = False
    for k, (g, r) in enumerate(zip(got, ref)):
        assert g.dtype == r.dtype and g.shape == r.shape and np.array_equal(g, r), 'seed %d output %d' % (seed, k)


@pytest.mark.parametrize('seed', random_programs.SCAN_SEEDS)
def test_random_scan_program_equals_the_oracle(seed):
    """Row scans with one or two loop-carried variables and assorted update rules, through whichever template the
    generator picks (lane-skewed scan when the row length fits, else the map kernel): bit-exact."""
    out = random_programs.scan_application(seed)[0]
    ref = oracle.evaluate([out])
    ref = ref[0] if isinstance(ref, list) else ref
    runtime.poison_outputs = True
    try:
        got = ovl.evaluate(out, opt_level=3)
    finally:
        runtime.poison_outputs = False
    assert got.dtype == ref.dtype and got.shape == ref.shape
    assert np.array_equal(got, ref, equal_nan=(ref.dtype.kind == 'f')), 'seed %d' % seed
    # the 'fast' math mode may run plain sums, products and running extrema as a tree: integer results stay equal,
    # floating point ones agree to rounding; every other scan body keeps its order and its bits
    from opveclib_amd import hipgen
    fast = ovl.evaluate(out, opt_level=3, math_mode='fast')
    template = hipgen.generate(out.parent.expression_dag, 'f' * 57, {'math': 'fast'}).launch['template']
    if template == 'treescan' and ref.dtype.kind == 'f':
        scale = np.max(np.abs(ref), axis=-1, keepdims=True) + np.finfo(ref.dtype).tiny
        assert np.max(np.abs(fast.astype(np.float64) - ref.astype(np.float64)) / scale) <= \
            np.finfo(ref.dtype).eps * 4 * ref.shape[-1], 'seed %d fast' % seed
    else:
        assert np.array_equal(fast, ref, equal_nan=(ref.dtype.kind == 'f')), 'seed %d fast (%s)' % (seed, template)


@pytest.mark.parametrize('seed', random_programs.TYPED_SEEDS)
def test_random_typed_program_equals_the_oracle(seed):
    """Expressions over all ten element types with casts, integer division and remainder, comparisons in the operand
    type, counted loops over worker-local tensors: bit-exact."""
    op = random_programs.typed_application(seed)
    outs = [op[0], op[1]]
    ref = oracle.evaluate(outs)
    got = ovl.evaluate(outs, opt_level=3)
    for k, (g, r) in enumerate(zip(got, ref)):
        assert g.dtype == r.dtype and g.shape == r.shape and np.array_equal(g, r), 'seed %d output %d' % (seed, k)


@pytest.mark.parametrize('seed', random_programs.REDUCE_SEEDS)
def test_random_reduction_program_equals_the_oracle(seed):
    """Reductions along the last or another axis with one or two loop-carried variables, one or two inputs and an
    epilogue on the final state, through whichever template the generator picks (row reduction, column reduction, or
    the map kernel for short lines): the order of the oracle's loop, hence its bits."""
    op = random_programs.reduce_application(seed)
    outs = [op[0], op[1]]
    ref = oracle.evaluate(outs)
    runtime.poison_outputs = True
    try:
        got = ovl.evaluate(outs, opt_level=3)
    finally:
        runtime.poison_outputs = False
    for k, (g, r) in enumerate(zip(got, ref)):
        assert g.dtype == r.dtype and g.shape == r.shape, 'seed %d output %d' % (seed, k)
        assert np.array_equal(g, r, equal_nan=(r.dtype.kind == 'f')), 'seed %d output %d' % (seed, k)
