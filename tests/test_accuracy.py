"""
The 'ulp2' math mode on the CPU: which routine every call site gets (hipgen/accuracy.py), and the once-rounded
log1p / expm1 routines of csrc/ovl_math.h compiled for the host against the reference's formulas
(opveclib/examples/test_log1p.py:22-61, test_expm1.py:22-62) evaluated with the host C library.

The header is plain IEEE double arithmetic, so the host build returns the bits the GPU returns; the sweep here takes
every 31st float32 of the domain on which the code generator uses the routines (the GPU test takes every one).
"""
import os
import subprocess

import numpy as np
import pytest

import opveclib_amd as ovl
from opveclib_amd import language as lang
from opveclib_amd import hipgen, stdops, workloads
from opveclib_amd.examples import log1p, expm1
from opveclib_amd.hipgen import accuracy, ranges
from opveclib_amd.hipgen.analysis import DagInfo
from opveclib_amd.workloads import Spec

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), 'opveclib_amd', 'csrc')


def selection(operator_dag):
    """{expression code or idiom name: [cheap?]} in program order for one operator."""
    info = DagInfo(operator_dag)
    info.math = 'ulp2'
    known = ranges.analyse(info)
    cheap = accuracy.select(info, known)
    kinds = accuracy.candidate_sites(info, known)
    return [(kinds[idx], idx in cheap) for idx in sorted(kinds)]


def test_fused_chain_uses_cheap_routines_where_two_ulp_are_proved():
    outs = workloads.chain8_outputs(Spec((64, 256)), Spec((64, 256)), Spec((1,)))
    op, = workloads.fused_operators(outs)
    chosen = selection(op)
    cheap = [kind for kind, is_cheap in chosen if is_cheap]
    # tanh directly; the three composite formulas as one routine each
    assert lang.TANH in cheap and 'sigmoid' in cheap and 'log1p' in cheap and 'expm1' in cheap
    assert [kind for kind, is_cheap in chosen if kind in accuracy.IDIOM_DOMAIN and not is_cheap] == []


def test_formulas_on_arguments_of_unknown_range_are_replaced_behind_a_run_time_test():
    """Without a known argument range the formula cannot be replaced outright; it is replaced behind a test of the
    arguments at run time, whose other branch is the formula itself with the bit-compatible routines.  The formula's
    own exp / log no longer reach the stored value (a cheap one among them is dead code); an exp that also decides a
    branch of the operator (expm1's ``e == 1``) stays the bit-compatible one."""
    x = Spec((1024,))
    chosen = dict(selection(workloads.unfused_operators([log1p(x)[0]])[0]))
    assert chosen['log1p_guarded'] is True
    chosen = dict(selection(workloads.unfused_operators([expm1(x)[0]])[0]))
    assert chosen['expm1_guarded'] is True and chosen[lang.EXP] is False
    chosen = dict(selection(workloads.unfused_operators([stdops.sigmoid(x)[0]])[0]))
    assert chosen['sigmoid_guarded'] is True
    for op, kind in ((log1p, 'log1p'), (expm1, 'expm1'), (stdops.sigmoid, 'sigmoid')):
        operator_dag, = workloads.unfused_operators([op(x)[0]])
        text = hipgen.generate(operator_dag, 'f' + '7' * 56, {'math': 'ulp2'}).source
        guards = [line for line in text.split('\n') if 'OVL_ALL(' in line]
        assert guards and all('else' in line for line in guards), kind
        routine = {'log1p': 'ovl_log1p_direct(', 'expm1': 'ovl_expm1_direct(', 'sigmoid': 'ovl_sigmoid_ulp2('}[kind]
        exact = {'log1p': 'ovl_logf(', 'expm1': 'ovl_expf(', 'sigmoid': 'ovl_expf('}[kind]
        assert all(routine in line and exact in line for line in guards), kind
        assert 'OVL_DECLARE_MATH_TABLES' in text        # the other branch needs the tables of the exact exp / log
        for lo, hi in accuracy.GUARD_DOMAIN[kind]:
            assert all(repr(float(lo)) + 'f' in line and repr(float(hi)) + 'f' in line for line in guards)
        # the bit-exact mode has no such test
        assert 'OVL_ALL(' not in hipgen.generate(operator_dag, 'f' + '7' * 56, None).source


def test_single_calls_are_cheap_and_cancelling_sums_are_not():
    x = Spec((1024,))
    assert selection(workloads.unfused_operators([stdops.tanh(x)[0]])[0]) == [(lang.TANH, True)]
    # the LSTM cell adds products of either sign: a distance in the operands is unbounded in ulp of the sum
    outs = workloads.lstm_outputs(Spec((8, 64)), Spec((8, 16)))
    assert all(not is_cheap for _, is_cheap in selection(workloads.fused_operators(outs)[0]))
    outs = workloads.lstm_grad_outputs(Spec((8, 64)), Spec((8, 16)), Spec((8, 16)), Spec((8, 16)))
    assert all(not is_cheap for _, is_cheap in selection(workloads.fused_operators(outs)[0]))


def test_the_lstm_cell_composed_of_library_operators_gets_cheap_routines_per_operator():
    """The cell of opveclib/test/test_operator_merge.py:311-321: every sigmoid and tanh is an operator of its own, so
    the promise applies to each of them given its own input (which the fused kernel holds exactly), and the sums of
    products that follow are exact operations on those results."""
    outs = workloads.stdops_lstm_outputs(Spec((8, 64)), Spec((8, 16)))
    op, = workloads.fused_operators(outs)
    chosen = selection(op)
    assert [kind for kind, cheap in chosen if cheap and kind == 'sigmoid_guarded'] == ['sigmoid_guarded'] * 3
    assert [kind for kind, cheap in chosen if cheap and kind == lang.TANH] == [lang.TANH] * 2
    text = hipgen.generate(op, 'f' + '7' * 56, {'math': 'ulp2'}).source
    # (one test per sigmoid and vector element of the thread)
    assert text.count('OVL_ALL(') % 3 == 0 and text.count('OVL_ALL(') >= 3 and 'ovl_fast_tanhf' in text


def test_an_inexact_value_never_decides_a_branch_or_an_index():
    @ovl.operator()
    def branchy(x):
        out = ovl.output_like(x)
        pos = ovl.position_in(x.shape)
        e = ovl.exp(x[pos])
        with ovl.if_(e > 2.0):
            out[pos] = e
        with ovl.else_():
            out[pos] = x[pos]
        return out

    chosen = selection(workloads.unfused_operators([branchy(Spec((256,)))[0]])[0])
    assert chosen == [(lang.EXP, False)]


def test_stage_variables_are_marked_by_the_optimizer():
    outs = workloads.chain8_outputs(Spec((64, 256)), Spec((64, 256)), Spec((1,)))
    op, = workloads.fused_operators(outs)
    marked = [e for e in op.expressions if e.code == lang.VARIABLE and e.io_index == accuracy.STAGE_VARIABLE]
    assert len(marked) == 7         # every internalised edge of the eight-operator chain


def test_generated_text_names_the_chosen_routines():
    from opveclib_amd import hipgen
    outs = workloads.chain8_outputs(Spec((64, 256)), Spec((64, 256)), Spec((1,)))
    op, = workloads.fused_operators(outs)
    text = hipgen.generate(op, 'f' + '0' * 56, {'math': 'ulp2'}).source
    # behind the tanh and the sigmoid the arguments of sigmoid, log1p and expm1 lie in the narrow domains
    for wanted in ('ovl_fast_tanhf(', 'ovl_sigmoid_small(', 'ovl_log1p_unit(', 'ovl_expm1_small('):
        assert wanted in text
    assert 'ovl_tanhf(' not in text
    exact = hipgen.generate(op, 'f' + '0' * 56, None).source
    for unwanted in ('ovl_fast', '_direct', '_unit', '_small'):
        assert unwanted not in exact


def test_narrow_routines_only_where_the_range_allows():
    from opveclib_amd import hipgen

    def clip_op(lo, hi):
        @ovl.operator()
        def clipped(x):
            out = ovl.output_like(x)
            pos = ovl.position_in(x.shape)
            out[pos] = ovl.minimum(ovl.maximum(x[pos], lo), hi)
            return out
        return clipped

    def text(outputs):
        op, = workloads.fused_operators(outputs)
        return hipgen.generate(op, 'f' + '0' * 56, {'math': 'ulp2'}).source

    x = Spec((1024,))
    assert 'ovl_log1p_unit(' in text([log1p(clip_op(0.0625, 0.99)(x))[0]])
    wide = text([log1p(clip_op(0.01, 0.99)(x))[0]])            # below 2^-4: the general once-rounded routine
    assert 'ovl_log1p_direct' in wide and '_unit' not in wide
    reaches_one = text([log1p(clip_op(0.5, 1.0)(x))[0]])        # 1 + 1 = 2 has another exponent
    assert 'ovl_log1p_direct' in reaches_one and '_unit' not in reaches_one
    assert 'ovl_expm1_small(' in text([expm1(clip_op(0.001, 0.68)(x))[0]])
    large = text([expm1(clip_op(0.001, 0.7)(x))[0]])
    assert 'ovl_expm1_direct(' in large and '_small' not in large
    assert 'ovl_sigmoid_small(' in text([stdops.sigmoid(clip_op(-1.0, 5.0)(x))])
    below = text([stdops.sigmoid(clip_op(-1.5, 5.0)(x))])
    assert 'ovl_sigmoid_ulp2(' in below and '_small' not in below


def test_formula_results_are_bounded_by_the_function():
    """log1p of [0.25, 0.75] lies in [0.22, 0.56], not in the [0.07, 1.7] that interval arithmetic over
    log(u) * x / (u - 1) gives: the expm1 behind it sees an argument in its narrow domain."""
    from opveclib_amd.hipgen import analysis, ranges

    @ovl.operator()
    def clipped(x):
        out = ovl.output_like(x)
        pos = ovl.position_in(x.shape)
        out[pos] = ovl.minimum(ovl.maximum(x[pos], 0.25), 0.75)
        return out

    op, = workloads.fused_operators([log1p(clipped(Spec((1024,))))[0]])
    info = analysis.DagInfo(op)
    known = ranges.analyse(info)
    quotients = [n for n in info.nodes if n.code == lang.DIVIDE and accuracy.match_idiom(info, known, n)]
    assert len(quotients) == 1
    r = known.ranges[quotients[0].idx]
    assert 0.2231 < r.lo < 0.2232 and 0.5596 < r.hi < 0.5597


PROGRAM = r'''
#include <math.h>
#include <stdio.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include "ovl_math.h"
static int32_t ordered(float f) { int32_t i; memcpy(&i, &f, 4); return i < 0 ? (int32_t)0x80000000 - i : i; }
static float log1p_formula(float x) {
    volatile float u = 1.0f + x; volatile float d = u - 1.0f;
    if (isinf(x) && x > 0) return x;
    if (d == 0) return x;
    volatile float l = logf(u); volatile float p = l * x; return p / d;
}
static float expm1_formula(float x) {
    volatile float e = expf(x);
    if (isinf(x) && x > 0) return x;
    if (e == 1.0f) return x;
    volatile float em = e - 1.0f;
    if (em == -1.0f) return -1.0f;
    volatile float p = em * x; volatile float l = logf(e); return p / l;
}
int main(int argc, char** argv) {
    int which = atoi(argv[1]); float lo = strtof(argv[2], 0), hi = strtof(argv[3], 0); uint32_t step = atoi(argv[4]);
    uint32_t a, b; memcpy(&a, &lo, 4); memcpy(&b, &hi, 4);
    long total = 0, differing = 0; int worst = 0;
    for (uint64_t i = a; i <= b; i += step) {
        uint32_t bits = (uint32_t)i; float x; memcpy(&x, &bits, 4);
        float want = (which & 1) ? expm1_formula(x) : log1p_formula(x);
        float got = which == 1 ? ovl_math::expm1_direct_(x) : which == 0 ? ovl_math::log1p_direct_<true>(x)
                  : which == 3 ? ovl_math::expm1_small_(x) : ovl_math::log1p_unit_(x);
        int d = abs(ordered(want) - ordered(got));
        ++total; if (d) ++differing; if (d > worst) worst = d;
    }
    float nan_result = which == 1 ? ovl_math::expm1_direct_(NAN) : which == 0 ? ovl_math::log1p_direct_<true>(NAN)
                     : which == 3 ? ovl_math::expm1_small_(NAN) : ovl_math::log1p_unit_(NAN);
    printf("%ld %ld %d %d\n", total, differing, worst, nan_result != nan_result ? 1 : 0);
    return 0;
}
'''


@pytest.fixture(scope='module')
def sweep(tmp_path_factory):
    directory = tmp_path_factory.mktemp('once_rounded')
    src = directory / 'sweep.cpp'
    src.write_text(PROGRAM)
    exe = directory / 'sweep'
    subprocess.check_call(['g++', '-O2', '-ffp-contract=off', '-mfma', '-std=c++17', '-I' + CSRC, str(src), '-o',
                           str(exe)])
    return exe


@pytest.mark.parametrize('kind', ['log1p', 'expm1'])
def test_once_rounded_routines_within_two_ulp_of_the_reference_formulas_on_the_host(sweep, kind):
    """Every 31st argument of the domains the generator replaces the formulas on: the one a value range must prove
    (IDIOM_DOMAIN) and the intervals tested at run time (GUARD_DOMAIN: also negative arguments)."""
    assert accuracy.IDIOM_DOMAIN[kind] in accuracy.GUARD_DOMAIN[kind]
    for lo, hi in accuracy.GUARD_DOMAIN[kind]:
        if hi < 0:
            lo, hi = hi, lo             # the program walks bit patterns upwards: away from zero
        out = subprocess.check_output([str(sweep), '01'[kind == 'expm1'], repr(lo), repr(hi), '31'],
                                      universal_newlines=True).split()
        total, differing, worst, nan_kept = (int(v) for v in out)
        assert total > (4 << 20 if lo > 0 else 2 << 20)
        assert worst <= accuracy.ROUTINE_ULPS[kind] == accuracy.TOLERANCE
        assert 0 < differing < total // 2
        assert nan_kept == 1


@pytest.mark.parametrize('kind', ['log1p', 'expm1'])
def test_narrow_routines_within_two_ulp_of_the_reference_formulas_on_the_host(sweep, kind):
    """Every seventh argument of the narrow domains (all of them: tests/test_gpu_math_exhaustive.py on the GPU)."""
    lo, hi = accuracy.NARROW_DOMAIN[kind]
    out = subprocess.check_output([str(sweep), '23'[kind == 'expm1'], repr(lo), repr(hi), '7'],
                                  universal_newlines=True).split()
    total, differing, worst, nan_kept = (int(v) for v in out)
    assert total > 4 << 20
    assert worst <= accuracy.TOLERANCE
    assert 0 < differing < total // 2
    assert nan_kept == 1


@pytest.mark.parametrize('kind,outside', [('log1p', (2.0 ** -6, 2.0 ** -4)), ('expm1', (0.6824, 0.69))])
def test_the_narrow_domain_limits_are_needed(sweep, kind, outside):
    """Below 2^-4 the table entry's logarithm and the polynomial cancel too far; past 0.682 the scaled argument
    rounds to 32 and the table index wraps."""
    out = subprocess.check_output([str(sweep), '23'[kind == 'expm1'], repr(outside[0]), repr(outside[1]), '1'],
                                  universal_newlines=True).split()
    assert int(out[2]) > accuracy.TOLERANCE


FORMULA_PROGRAM = r"""
#include <math.h>
#include <stdio.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
static int32_t ordered(float f) { int32_t i; memcpy(&i, &f, 4); return i < 0 ? (int32_t)0x80000000 - i : i; }
static float log1p_formula(float x) {
    volatile float u = 1.0f + x; volatile float d = u - 1.0f;
    if (isinf(x) && x > 0) return x;
    if (d == 0) return x;
    volatile float l = logf(u); volatile float p = l * x; return p / d;
}
static float expm1_formula(float x) {
    volatile float e = expf(x);
    if (isinf(x) && x > 0) return x;
    if (e == 1.0f) return x;
    volatile float em = e - 1.0f;
    if (em == -1.0f) return -1.0f;
    volatile float p = em * x; volatile float l = logf(e); return p / l;
}
static float sigmoid_formula(float x) { volatile float n = -x; volatile float e = expf(n); volatile float s = 1.0f + e; return 1.0f / s; }
int main(int argc, char** argv) {
    int which = atoi(argv[1]); float lo = strtof(argv[2], 0), hi = strtof(argv[3], 0); uint32_t step = atoi(argv[4]);
    // every step-th float32 of [lo, hi] in increasing order, both ends included
    int32_t a = ordered(lo), b = ordered(hi);
    float least = INFINITY, most = -INFINITY; int worst = 0;
    for (int64_t i = a; ; i += step) {
        if (i > b) i = b;
        int32_t o = (int32_t)i; int32_t bits = o < 0 ? (int32_t)0x80000000 - o : o; float x; memcpy(&x, &bits, 4);
        float got = which == 0 ? log1p_formula(x) : which == 1 ? expm1_formula(x) : sigmoid_formula(x);
        double exact = which == 0 ? log1p((double)x) : which == 1 ? expm1((double)x) : 1.0 / (1.0 + exp(-(double)x));
        int d = abs(ordered(got) - ordered((float)exact));
        if (d > worst) worst = d;
        if (got < least) least = got;
        if (got > most) most = got;
        if (i == b) break;
    }
    printf("%d %.9g %.9g\n", worst, least, most);
    return 0;
}
"""


@pytest.fixture(scope='module')
def formula_sweep(tmp_path_factory):
    directory = tmp_path_factory.mktemp('formulas')
    src = directory / 'formulas.cpp'
    src.write_text(FORMULA_PROGRAM)
    exe = directory / 'formulas'
    subprocess.check_call(['g++', '-O2', '-ffp-contract=off', '-std=c++17', str(src), '-o', str(exe)])
    return exe


def _formula_division_range(kind, lo, hi):
    """The value range the analysis gives the division that ends the formula of ``kind`` on arguments in [lo, hi]."""
    @ovl.operator()
    def clipped(x, lo=None, hi=None):
        out = ovl.output_like(x)
        pos = ovl.position_in(x.shape)
        out[pos] = ovl.minimum(ovl.maximum(x[pos], lo), hi)
        return out

    formula = {'log1p': log1p, 'expm1': expm1, 'sigmoid': stdops.sigmoid}[kind]
    op, = workloads.fused_operators([formula(clipped(Spec((1024,)), lo=lo, hi=hi))[0]])
    info = DagInfo(op)
    known = ranges.analyse(info)
    quotients = [n for n in info.nodes if n.code == lang.DIVIDE and accuracy.match_idiom(info, known, n)]
    assert len(quotients) == 1, kind
    return known.ranges[quotients[0].idx]


@pytest.mark.parametrize('kind', ['log1p', 'expm1', 'sigmoid'])
def test_formula_values_stay_inside_the_range_the_analysis_narrows_them_to(formula_sweep, kind):
    """The analysis bounds the division that ends a recognised formula by the image of the function itself, widened
    by ranges._SLACK_ULPS float32 steps, in every math mode (guards are pruned and in-range routines chosen from
    it).  That is sound only while the formula evaluated with the host library stays within that many steps of the
    function on the whole compared domain: measured here on a sweep of each domain with both ends, and the narrowed
    range of several sub-intervals is compared with the least and greatest value the formula takes on them."""
    assert ranges._SLACK_ULPS >= 7          # "in every math mode within seven" (ranges.RangeInfo._formula_image)
    which = {'log1p': '0', 'expm1': '1', 'sigmoid': '2'}[kind]
    lo, hi = accuracy.IDIOM_DOMAIN[kind]
    worst, _, _ = subprocess.check_output([str(formula_sweep), which, repr(lo), repr(hi), '61'],
                                          universal_newlines=True).split()
    assert int(worst) <= 3                  # "within three float32 steps of the function itself"
    intervals = {'log1p': [(lo, hi), (lo, 2.0 ** -9), (0.25, 0.75), (0.2689, 0.7311), (1.0, 1.0e19), (2.0 ** 63, hi)],
                 'expm1': [(lo, hi), (lo, 2.0 ** -11), (0.2384, 0.5489), (1.0, 10.0), (60.0, hi)],
                 'sigmoid': [(lo, hi), (lo, -15.0), (-1.0, 1.0), (-0.7616, 0.7616), (20.0, hi)]}[kind]
    for a, b in intervals:
        a32, b32 = float(np.float32(a)), float(np.float32(b))
        if a32 < lo:
            a32 = float(np.nextafter(np.float32(a32), np.float32(np.inf)))
        if b32 > hi:
            b32 = float(np.nextafter(np.float32(b32), np.float32(-np.inf)))
        r = _formula_division_range(kind, a32, b32)
        _, least, most = subprocess.check_output([str(formula_sweep), which, repr(a32), repr(b32), '17'],
                                                 universal_newlines=True).split()
        assert r.lo <= float(least) and float(most) <= r.hi, (kind, a, b, r.lo, r.hi, least, most)


@pytest.mark.parametrize('kind,outside', [('log1p', (8e37, 3e38)), ('expm1', (70.0, 88.0))])
def test_the_domain_limits_are_needed(sweep, kind, outside):
    """Towards overflow the reference's formulas (whose 1 + x and exp(x) become infinite early) leave the once-rounded
    values far behind, which is why the code generator keeps the formula outside the domains."""
    out = subprocess.check_output([str(sweep), '01'[kind == 'expm1'], repr(outside[0]), repr(outside[1]), '1'],
                                  universal_newlines=True).split()
    assert int(out[2]) > accuracy.TOLERANCE


def test_formula_outside_the_domain_is_not_replaced():
    """A consumer of raw input (range unknown) keeps the formula; one behind a clip into the domain gets the
    routine."""
    @ovl.operator()
    def clipped(x):
        out = ovl.output_like(x)
        pos = ovl.position_in(x.shape)
        out[pos] = ovl.minimum(ovl.maximum(x[pos], 0.25), 0.75)
        return out

    raw = dict(selection(workloads.fused_operators([log1p(Spec((1024,)))[0]])[0]))
    assert 'log1p' not in raw
    fused, = workloads.fused_operators([log1p(clipped(Spec((1024,))))[0]])
    assert dict(selection(fused)).get('log1p') is True
    too_wide, = workloads.fused_operators([expm1(stdops.mul(clipped(Spec((1024,))), np.array([200.0], np.float32)))[0]])
    assert 'expm1' not in dict(selection(too_wide))
    fused, = workloads.fused_operators([stdops.sigmoid(clipped(Spec((1024,))))[0]])
    assert dict(selection(fused)).get('sigmoid') is True


def test_rounding_operations_after_an_inexact_value_cost_a_step():
    """exp(x) + 1 stored: the cheap exp is one ulp off and the rounding of the sum can add another: still two.
    (exp(x) + 1) * 3 stored: up to twice that plus one: the exp must be the bit-compatible one."""
    @ovl.operator()
    def exp_plus_one(x):
        out = ovl.output_like(x)
        pos = ovl.position_in(x.shape)
        out[pos] = ovl.exp(x[pos]) + 1.0
        return out

    @ovl.operator()
    def exp_plus_one_times_three(x):
        out = ovl.output_like(x)
        pos = ovl.position_in(x.shape)
        out[pos] = (ovl.exp(x[pos]) + 1.0) * 3.0
        return out

    x = Spec((256,))
    assert selection(workloads.unfused_operators([exp_plus_one(x)[0]])[0]) == [(lang.EXP, True)]
    assert selection(workloads.unfused_operators([exp_plus_one_times_three(x)[0]])[0]) == [(lang.EXP, False)]
