"""
The 'ulp2' float32 math mode on the GPU.

Promise of the mode: every operator's outputs are within two float32 units in the last place (ulp) of what the
reference's generated C++ computes from the same operator inputs (the tolerance stated for transcendental operators);
in a fused chain the promise holds for every operator of the chain.  The CPU oracle is that reference; the 'exact'
mode returns the oracle's bits (tests/test_gpu_parity.py, tests/test_gpu_configs.py), so at sizes the oracle would
need minutes for, the exact mode stands in for it and the oracle itself is applied to a slice of rows.

  * all eight stages of the benchmark chain at full size [8192, 8192], two ways: each stage of the fused kernel
    against the exact operator applied to the same stage input, and each stage's operator fed the exact mode's
    stage input (the oracle's bits) against the exact mode's stage output;
  * the same on a slice of rows against the oracle itself;
  * every transcendental operator on its own, on chain-like inputs and on wide sweeps, against the oracle;
  * fused test cases end to end: absolute error of a few ulp of the O(1) intermediates, NaN / infinity patterns equal;
  * operators without exp / log / tanh / division do not change with the mode.
"""
import numpy as np
import pytest

import opveclib_amd as ovl
import oracle
from opveclib_amd import workloads
from tests import cases

pytestmark = pytest.mark.gpu

TOLERANCE = 2
MATH_STAGES = ('tanh', 'sigmoid', 'log1p', 'expm1')


def _ulps(x, y):
    import torch
    xi, yi = x.view(torch.int32).long(), y.view(torch.int32).long()
    xi = torch.where(xi < 0, -(xi & 0x7fffffff), xi)
    yi = torch.where(yi < 0, -(yi & 0x7fffffff), yi)
    return (xi - yi).abs()


@pytest.fixture(scope='module')
def chain_inputs():
    import torch
    rng = np.random.default_rng(2)
    a = torch.from_numpy(workloads.uniform(rng, -1, 1, cases.CHAIN8_SHAPE)).cuda()
    b = torch.from_numpy(workloads.uniform(rng, -1, 1, cases.CHAIN8_SHAPE)).cuda()
    s = torch.tensor([1.0001], dtype=torch.float32).cuda()
    return a, b, s


def test_every_stage_of_the_fused_chain_at_full_size(chain_inputs):
    """One launch of the fused kernel in 'ulp2' mode with every stage requested; stage k is compared with the exact
    operator applied to the kernel's own stage k-1 output (sub also reads B).  add, mul, sub and abs must be exact."""
    import torch
    a, b, s = chain_inputs
    outs = workloads.chain8_stage_outputs(a, b, s)
    assert len(workloads.fused_operators(outs)) == 1
    stages = ovl.evaluate(outs, opt_level=3, math_mode='ulp2')
    exact_ops = {'add': lambda prev: cases.stdops.add(a, b), 'mul': lambda prev: cases.stdops.mul(prev, s),
                 'sub': lambda prev: cases.stdops.sub(prev, b), 'abs': lambda prev: cases.absolute(prev)}
    for k, name in enumerate(cases.CHAIN8_STAGES):
        prev = stages[k - 1] if k else None
        if name in MATH_STAGES:
            ref = ovl.evaluate(cases.chain8_single_stage(name, prev), opt_level=0, math_mode='exact')
            worst = int(_ulps(stages[k], ref).max())
            assert worst <= TOLERANCE, 'stage %s: %d ulp' % (name, worst)
        else:
            ref = ovl.evaluate(exact_ops[name](prev)[0], opt_level=0, math_mode='exact')
            assert torch.equal(stages[k], ref), 'stage %s is not exact' % name
        del ref
    # the oracle itself on a band of 1024 rows, all 8192 columns, of every transcendental stage
    rows = slice(4000, 4000 + cases.ORACLE_BAND_ROWS)
    for k, name in enumerate(cases.CHAIN8_STAGES):
        if name in MATH_STAGES:
            x = stages[k - 1][rows].cpu().numpy()
            want = oracle.evaluate(cases.chain8_single_stage(name, x))
            got = stages[k][rows].cpu().numpy()
            assert cases.ulp_distance(got, want).max() <= TOLERANCE, name


def test_every_stage_on_the_exact_stage_inputs_at_full_size(chain_inputs):
    """Each stage's operator in 'ulp2' mode is fed the exact mode's stage input (the oracle's bits) and compared with
    the exact mode's stage output.  log1p and expm1 sit behind a clip to their stage's input range, as they sit behind
    sigmoid and log1p in the chain, so that the code generator makes the choices it makes in the fused kernel."""
    import torch
    from opveclib_amd import runtime
    a, b, s = chain_inputs
    exact = ovl.evaluate(workloads.chain8_stage_outputs(a, b, s), opt_level=0, math_mode='exact')
    rows = slice(100, 164)
    want = oracle.evaluate(workloads.chain8_stage_outputs(a[rows].cpu().numpy(), b[rows].cpu().numpy(),
                                                          s.cpu().numpy()))
    for k, name in enumerate(cases.CHAIN8_STAGES):
        assert np.array_equal(exact[k][rows].cpu().numpy(), want[k]), 'exact mode differs from the oracle at ' + name
        if name not in MATH_STAGES:
            continue
        x = exact[k - 1]
        if name in cases.CHAIN8_STAGE_INPUT_RANGE:
            lo, hi = cases.CHAIN8_STAGE_INPUT_RANGE[name]
            assert float(x.min()) >= lo and float(x.max()) <= hi     # the clip changes nothing
        got = ovl.evaluate(cases.chain8_single_stage(name, x, with_range=True), opt_level=3, math_mode='ulp2')
        worst = int(_ulps(got, exact[k]).max())
        assert worst <= TOLERANCE, 'stage %s: %d ulp' % (name, worst)
        del got
    # the kernels that ran are the ones with the cheap routines, not the exact ones
    sources = [c.gen.source for key, c in runtime._loaded.items() if "'math', 'ulp2'" in key[1]]
    # (the chain's stage ranges lie in the narrow domains: the shorter forms of the once-rounded routines)
    assert any('ovl_log1p_unit' in text for text in sources)
    assert any('ovl_expm1_small' in text for text in sources)
    assert any('ovl_sigmoid_small' in text for text in sources)
    assert any('ovl_fast_tanhf' in text for text in sources)


@pytest.mark.parametrize('kind,lo,hi,routine', cases.ULP2_CLIPPED_FORMULAS,
                         ids=['%s_%g_%g' % f[:3] for f in cases.ULP2_CLIPPED_FORMULAS])
def test_formulas_behind_a_clip_use_the_routine_their_range_allows(kind, lo, hi, routine):
    """The clip is exact in every mode, so the formula's stage sees the same input in both runs and the distance of
    the results is the stage's own."""
    from opveclib_amd import runtime
    x = cases.ulp2_clipped_arguments(lo, hi)
    out = cases.ulp2_clipped_formula(kind, lo, hi, x)
    want = ovl.evaluate(out, opt_level=3, math_mode='exact')
    got = ovl.evaluate(out, opt_level=3, math_mode='ulp2')
    assert not np.isnan(want).any() and not np.isnan(got).any()
    worst = int(cases.ulp_distance(got, want).max())
    assert worst <= TOLERANCE, '%s on [%g, %g]: %d ulp' % (kind, lo, hi, worst)
    sources = [c.gen.source for key, c in runtime._loaded.items()
               if "'math', 'ulp2'" in key[1] and c.gen.source.count('ovl_') and 'clip_to_range' in c.gen.source]
    assert any(routine + '(' in text or routine + '_nan(' in text for text in sources)


@pytest.mark.parametrize('case', cases.FAST_CASES, ids=[c.name for c in cases.FAST_CASES])
def test_single_operators_within_two_ulp_of_the_oracle(case):
    for dist in cases.run_fast_case_on_gpu(case, 'ulp2'):
        assert dist.max() <= TOLERANCE, '%s: %d ulp' % (case.name, int(dist.max()))


@pytest.mark.parametrize('name', cases.FAST_FUSED_CASES)
def test_fused_cases_stay_close_end_to_end(name):
    case = cases.CASE_BY_NAME[name]
    outs = case.outputs()
    ref = oracle.profile(outs, 1, 0)[0]
    got = ovl.evaluate(outs, opt_level=3, math_mode='ulp2')
    got = got if isinstance(got, list) else [got]
    for g, r in zip(got, ref):
        finite = np.isfinite(r)
        assert np.array_equal(g[~finite], r[~finite], equal_nan=True), name + ': NaN / infinity pattern differs'
        scale = max(1.0, float(np.abs(r[finite]).max()))
        assert float(np.abs(g[finite].astype(np.float64) - r[finite]).max()) <= 8 * np.finfo(np.float32).eps * scale


def test_small_chain_stagewise_against_the_oracle():
    """The chain at a size the oracle finishes at once: every stage of the fused 'ulp2' kernel against the oracle's
    operator on the same stage input."""
    outs = cases.CASE_BY_NAME['c2_chain_stages'].outputs()
    stages = ovl.evaluate(outs, opt_level=3, math_mode='ulp2')
    for k, name in enumerate(cases.CHAIN8_STAGES):
        if name in MATH_STAGES:
            want = oracle.evaluate(cases.chain8_single_stage(name, stages[k - 1]))
            assert cases.ulp_distance(stages[k], want).max() <= TOLERANCE, name


def _ulps_nan_equal(x, y):
    """Float32 steps between two device tensors, 0 where both are NaN."""
    import torch
    d = _ulps(x, y)
    return torch.where(torch.isnan(x) & torch.isnan(y), torch.zeros_like(d), d)


def test_lstm_cell_composed_of_library_operators_at_full_size():
    """The cell of opveclib/test/test_operator_merge.py:311-321 at [4096, 4 x 1024], fused into one 'ulp2' kernel that
    also stores every operator's output.  Inputs are N(0, 1) with NaN, infinities, zeros of both signs, huge and tiny
    values planted in the first rows.  Every sigmoid and tanh is compared with the bit-exact operator applied to the
    kernel's own value of that operator's input (at most 2 ulp); split, the products and the sum must be exact; and
    on a band of rows that holds the planted values every transcendental operator is compared with the oracle."""
    import torch
    from opveclib_amd import runtime
    concat, c = cases.stdops_lstm_full_size_inputs()
    concat_d, c_d = torch.from_numpy(concat).cuda(), torch.from_numpy(c).cuda()
    outs = workloads.stdops_lstm_stage_outputs(concat_d, c_d)
    fused = workloads.fused_operators(outs)
    assert len(fused) == 1
    got = dict(zip(workloads.STDOPS_LSTM_STAGES, ovl.evaluate(outs, opt_level=3, math_mode='ulp2')))
    source = runtime.load_operator(fused[0], {'math': 'ulp2'}).gen.source
    assert 'ovl_sigmoid_ulp2(' in source and 'OVL_ALL(' in source and 'ovl_fast_tanhf(' in source
    units = c.shape[1]
    for k, name in enumerate('ijfo'):
        assert torch.equal(got[name].view(torch.int32), concat_d[:, k * units:(k + 1) * units].contiguous().view(torch.int32))
    stdops = cases.stdops
    for name, fcn, arg in (('sigmoid_f', stdops.sigmoid, 'f'), ('sigmoid_i', stdops.sigmoid, 'i'),
                           ('tanh_j', stdops.tanh, 'j'), ('tanh_new_c', stdops.tanh, 'new_c'),
                           ('sigmoid_o', stdops.sigmoid, 'o')):
        ref = ovl.evaluate(fcn(got[arg])[0], opt_level=0, math_mode='exact')
        worst = int(_ulps_nan_equal(got[name], ref).max())
        assert worst <= TOLERANCE, '%s: %d ulp' % (name, worst)
        assert torch.equal(torch.isnan(got[name]), torch.isnan(ref)), name
        # the oracle on the band that holds the planted values
        band = slice(0, cases.ORACLE_BAND_ROWS)
        want = oracle.evaluate(fcn(got[arg][band].cpu().numpy())[0])
        mine = got[name][band].cpu().numpy()
        both_nan = np.isnan(want) & np.isnan(mine)
        assert np.array_equal(np.isnan(want), np.isnan(mine)), name
        distance = cases.ulp_distance(np.where(both_nan, 0, mine), np.where(both_nan, 0, want))
        assert distance.max() <= TOLERANCE, '%s against the oracle: %d ulp' % (name, int(distance.max()))
        del ref
    for name, fcn, args in (('c_sigmoid_f', stdops.mul, (c_d, got['sigmoid_f'])),
                            ('sigmoid_i_tanh_j', stdops.mul, (got['sigmoid_i'], got['tanh_j'])),
                            ('new_c', stdops.add, (got['c_sigmoid_f'], got['sigmoid_i_tanh_j'])),
                            ('new_h', stdops.mul, (got['tanh_new_c'], got['sigmoid_o']))):
        ref = ovl.evaluate(fcn(*args)[0], opt_level=0, math_mode='exact')
        same = (got[name].view(torch.int32) == ref.view(torch.int32)) | (torch.isnan(got[name]) & torch.isnan(ref))
        assert bool(same.all()), name + ' is not exact'
        del ref
    # end to end against the bit-exact mode: a few ulp of the O(1) intermediates where nothing is NaN or infinite
    exact_c, exact_h = ovl.evaluate(workloads.stdops_lstm_outputs(concat_d, c_d), opt_level=3, math_mode='exact')
    for mine, ref in ((got['new_c'], exact_c), (got['new_h'], exact_h)):
        finite = torch.isfinite(ref)
        assert torch.equal(torch.isfinite(mine), finite)
        scale = float(ref[finite].abs().max())
        assert float((mine[finite].double() - ref[finite].double()).abs().max()) <= 8 * np.finfo(np.float32).eps * max(1.0, scale)


def test_guarded_formulas_on_arguments_straight_from_a_tensor():
    """sigmoid, log1p and expm1 as single operators on a tensor of unknown range (N(0, 1), a wide sweep, the planted
    special values): the kernel tests its arguments at run time, wavefronts whose arguments all lie in the compared
    domain take the once-rounded routine, the others the formula.  Against the oracle: at most 2 ulp, NaN where it has
    NaN."""
    from opveclib_amd import runtime
    x = cases.guarded_formula_arguments()
    for name, fcn in (('sigmoid', cases.stdops.sigmoid), ('log1p', cases.log1p), ('expm1', cases.expm1)):
        out = fcn(x)[0]
        want = oracle.evaluate(out)
        got = ovl.evaluate(out, opt_level=0, math_mode='ulp2')
        assert np.array_equal(np.isnan(want), np.isnan(got)), name
        both_nan = np.isnan(want)
        distance = cases.ulp_distance(np.where(both_nan, 0, got), np.where(both_nan, 0, want))
        assert distance.max() <= TOLERANCE, '%s: %d ulp' % (name, int(distance.max()))
        # both branches ran: some wavefronts took the routine (results that differ from the formula's bits exist)
        # and the planted values took the formula
        assert (distance > 0).any(), name + ': no result differs from the formula, the routine never ran'
    sources = [c.gen.source for key, c in runtime._loaded.items() if "'math', 'ulp2'" in key[1]]
    assert sum('OVL_ALL(' in text for text in sources) >= 3


def test_lstm_keeps_the_oracle_bits_in_ulp2_mode():
    """The LSTM cell adds products of either sign, so no call site of it may be inexact: the mode changes nothing."""
    for name in ('c4_lstm', 'c4_lstm_grad'):
        outs = cases.CASE_BY_NAME[name].outputs()
        ref = oracle.profile(outs, 1, 0)[0]
        got = ovl.evaluate(outs, opt_level=3, math_mode='ulp2')
        for g, r in zip(got, ref):
            assert np.array_equal(g, r, equal_nan=True), name


def test_an_unmodified_reference_style_call_runs_the_ulp2_kernel(monkeypatch):
    """`ovl.evaluate(outputs)` as the reference's callers write it (opveclib/operator.py:2099-2117: no math argument),
    in a process that has chosen no mode: the 'ulp2' kernel runs, also when the environment says OPVECLIB_MATH=ulp2,
    and OPVECLIB_MATH=exact selects the bit-exact one."""
    import torch
    import importlib
    from opveclib_amd import runtime
    ovl_operator = importlib.import_module('opveclib_amd.operator')
    case = cases.CASE_BY_NAME['c2_chain']
    outs = case.outputs()
    dag, _ = __import__('opveclib_amd.fusion', fromlist=['_merge_op_dag'])._merge_op_dag(
        ovl_operator._build_op_dag(*outs).proto_dag, None)
    assert len(dag.operators) == 1

    def kernel_of_an_unqualified_call():
        before = set(runtime._loaded)
        got = ovl.evaluate(outs)
        key = [k for k in runtime._loaded if k[0] == ovl_operator._op_hash(dag.operators[0])]
        used = [k for k in key if k not in before] or key
        return got, [runtime._loaded[k].lib.info['kernel'] for k in used]

    exact = ovl.evaluate(outs, math_mode='exact')
    for setting, suffix in ((None, '_ulp2'), ('ulp2', '_ulp2')):
        monkeypatch.setattr(ovl_operator, '_default_math_mode', [None])
        if setting is None:
            monkeypatch.delenv('OPVECLIB_MATH', raising=False)
        else:
            monkeypatch.setenv('OPVECLIB_MATH', setting)
        runtime._loaded.clear()
        got, kernels = kernel_of_an_unqualified_call()
        assert ovl.get_math_mode() == 'ulp2'
        assert len(kernels) == 1 and kernels[0].endswith(suffix), kernels
        # close to the bit-exact result (the chain ends in a subtraction, so the bound is absolute)
        assert np.abs(np.asarray(got, np.float64) - np.asarray(exact, np.float64)).max() < 1e-6
    monkeypatch.setattr(ovl_operator, '_default_math_mode', [None])
    monkeypatch.setenv('OPVECLIB_MATH', 'exact')
    runtime._loaded.clear()
    got, kernels = kernel_of_an_unqualified_call()
    assert len(kernels) == 1 and not kernels[0].endswith('_ulp2') and not kernels[0].endswith('_fast')
    assert np.array_equal(np.asarray(got), np.asarray(exact))
