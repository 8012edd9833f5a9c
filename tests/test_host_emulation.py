"""
The generated HIP sources on the CPU: every operator source the code generator emits for the parity cases (all four
kernel templates, fused and unfused, plus the forced template variants and the random programs) is compiled as plain
C++ against tests/native/host_emulation/ovl_device.h, run with one host thread per GPU thread under AddressSanitizer
on buffers of exactly the tensors' sizes, and compared bit for bit with the oracle.  This checks, without a GPU, the
text the GPU compiles: index arithmetic, vector accesses, loads moved ahead of conditions, LDS tiles and barriers,
lane-to-lane moves, and that no access leaves its tensor.  (What only the device can show - its math instructions,
memory model, the lockstep of the 64 lanes of a wavefront, timing - stays with the `gpu` tests.)  The 'fast' math mode is built on device instructions and is
not emulated.
"""
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

import oracle
from tests import cases, host_emulation, random_programs

pytestmark = pytest.mark.skipif(not os.path.exists(host_emulation.CLANG), reason='needs the ROCm clang++ as host compiler')

WORKERS = min(8, os.cpu_count() or 1)


def _same(got, ref):
    return len(got) == len(ref) and all(
        g.dtype == r.dtype and g.shape == r.shape and np.array_equal(g, r, equal_nan=(r.dtype.kind == 'f'))
        for g, r in zip(got, ref))


def _check(job):
    """job = (label, outputs, opt level, code generator options); returns the label when something is wrong."""
    label, outs, level, options = job
    try:
        ref = oracle.profile(outs, 1, 0)[0]
        got = host_emulation.evaluate(outs, level, options)
        return None if _same(got, ref) else label + ': differs from the oracle'
    except Exception as exception:
        return label + ': ' + str(exception)[-1500:]


def _run_all(jobs):
    with ThreadPoolExecutor(WORKERS) as pool:
        return [problem for problem in pool.map(_check, jobs) if problem]


def test_an_access_outside_a_tensor_ends_the_run():
    """Control: an operator that reads one element past its input is reported, not silently accepted."""
    source = r'''
#include "ovl_device.h"
extern "C" __global__ void __launch_bounds__(256) k(const float* __restrict__ in0, float* __restrict__ out0, uint32_t n, uint32_t off) {
    const uint32_t v = blockIdx.x * 256u + threadIdx.x;
    if (v < n) out0[v] = in0[v + off];
}
extern "C" int beyond(const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* stream) {
    hipLaunchKernelGGL(k, dim3(2u), dim3(256u), 0, static_cast<hipStream_t>(stream),
                       static_cast<const float*>(in[0].data), static_cast<float*>(out[0].data), 300u, 1u);
    return OVL_OK;
}
extern "C" int within(const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* stream) {
    hipLaunchKernelGGL(k, dim3(2u), dim3(256u), 0, static_cast<hipStream_t>(stream),
                       static_cast<const float*>(in[0].data), static_cast<float*>(out[0].data), 300u, 0u);
    return OVL_OK;
}
'''
    x = np.arange(300, dtype=np.float32)
    types = [(1, np.float32, [300])]
    good = host_emulation.run_program(host_emulation.build_source(source, 'within'), [x], types, types)
    assert np.array_equal(good[0], x)
    with pytest.raises(host_emulation.EmulationError) as failure:
        host_emulation.run_program(host_emulation.build_source(source, 'beyond'), [x], types, types)
    assert 'AddressSanitizer' in str(failure.value) and 'heap-buffer-overflow' in str(failure.value)


def test_every_parity_case_emulated_on_the_host_equals_the_oracle():
    jobs = []
    for case in cases.CASES:
        outs = case.outputs()
        for level in (0, 3):
            jobs.append(('%s opt_level %d' % (case.name, level), outs, level, None))
    assert _run_all(jobs) == []


def test_forced_templates_emulated_on_the_host_equal_the_oracle():
    jobs = []
    for name, options in cases.TEMPLATE_VARIANTS:
        jobs.append(('%s %r' % (name, options), cases.CASE_BY_NAME[name].outputs(), 3, options))
    assert _run_all(jobs) == []


def test_random_programs_emulated_on_the_host_equal_the_oracle():
    jobs = []
    for seed in random_programs.INDEX_SEEDS:
        op = random_programs.index_application(seed)
        jobs.append(('index program %d' % seed, [op[0], op[1]], 3, None))
    for seed in random_programs.SCAN_SEEDS:
        jobs.append(('scan program %d' % seed, [random_programs.scan_application(seed)[0]], 3, None))
    for seed in random_programs.REDUCE_SEEDS:
        op = random_programs.reduce_application(seed)
        jobs.append(('reduction program %d' % seed, [op[0], op[1]], 3, None))
    for seed in random_programs.TYPED_SEEDS:
        op = random_programs.typed_application(seed)
        jobs.append(('typed program %d' % seed, [op[0], op[1]], 3, None))
    for seed in random_programs.GPU_SEEDS:
        op = random_programs.application(seed)
        jobs.append(('element-wise program %d' % seed, [op[0], op[1]], 3, None))
        jobs.append(('element-wise program %d without value ranges' % seed, [op[0], op[1]], 3,
                     {'value_ranges': False}))
    for seed in random_programs.DAG_SEEDS:
        outs = random_programs.random_dag(seed)
        for level in (0, 3):
            jobs.append(('operator DAG %d opt_level %d' % (seed, level), outs, level, None))
    assert _run_all(jobs) == []


# ----------------------------------------------------------------------------------------------------------------------
# The hand-written kernels with run-time shapes (csrc/ovl_lstm.hip, csrc/ovl_scan.hip) on the host
# ----------------------------------------------------------------------------------------------------------------------
F32, F64, U32 = 1, 2, 10        # dtype codes of the launcher ABI (include/ovl_launch.h)


def _skewed(array, skew):
    """The array as the adapters expect it: behind ``skew`` leading elements (which the kernels must not touch)."""
    flat = np.ascontiguousarray(array).reshape(-1)
    return np.concatenate([np.full(skew, 77, flat.dtype), flat]) if skew else flat


def _lstm_shapes():
    rng = np.random.default_rng(21)
    shapes = [(1, 1), (1, 4), (3, 5), (2, 8), (7, 12), (5, 64), (64, 36), (9, 257), (33, 100), (2, 1024), (130, 20)]
    return [(b, u, int(rng.integers(0, 2))) for b, u in shapes]


@pytest.mark.parametrize('batch,units,skew', _lstm_shapes())
def test_hand_written_lstm_cell_emulated_on_the_host_equals_the_oracle(batch, units, skew):
    from opveclib_amd.lstm import lstm, lstm_grad
    rng = np.random.default_rng(batch * 1000 + units)
    concat = rng.standard_normal((batch, 4 * units)).astype(np.float32) * 3
    c = rng.standard_normal((batch, units)).astype(np.float32)
    d_c = rng.standard_normal((batch, units)).astype(np.float32)
    d_h = rng.standard_normal((batch, units)).astype(np.float32)
    concat[0, 0] = 60.0          # beyond the range of the sigmoid derivative
    bias = np.array([1.0], np.float32)
    dims = np.array([batch, units, skew], np.uint32)
    n, m = batch * units + skew, 4 * batch * units + skew

    ref_c, ref_h = oracle.evaluate(lstm(concat, c, forget_bias=1.0))
    got = host_emulation.run_program(
        host_emulation.build_hand_written('emu_lstm_forward'),
        [_skewed(concat, skew), _skewed(c, skew), bias, dims],
        [(F32, np.float32, [m]), (F32, np.float32, [n]), (F32, np.float32, [1]), (U32, np.uint32, [3])],
        [(F32, np.float32, [n]), (F32, np.float32, [n])])
    assert np.array_equal(got[0][skew:].reshape(batch, units), ref_c)
    assert np.array_equal(got[1][skew:].reshape(batch, units), ref_h)
    # the elements in front of a skewed tensor keep the fill the driver gave them
    assert all(np.all(g[:skew].view(np.uint32) == 0xFEFEFEFE) for g in got)

    ref_dconcat, ref_dc = oracle.evaluate(lstm_grad(concat, c, d_c, d_h, forget_bias=1.0))
    got = host_emulation.run_program(
        host_emulation.build_hand_written('emu_lstm_backward'),
        [_skewed(concat, skew), _skewed(c, skew), _skewed(d_c, skew), _skewed(d_h, skew), bias, dims],
        [(F32, np.float32, [m]), (F32, np.float32, [n]), (F32, np.float32, [n]), (F32, np.float32, [n]),
         (F32, np.float32, [1]), (U32, np.uint32, [3])],
        [(F32, np.float32, [m]), (F32, np.float32, [n])])
    assert np.array_equal(got[0][skew:].reshape(batch, 4 * units), ref_dconcat)
    assert np.array_equal(got[1][skew:].reshape(batch, units), ref_dc)


@pytest.mark.parametrize('rows,cols,skew', [(1, 1, 0), (1, 64, 0), (3, 128, 0), (5, 192, 0), (4, 256, 0), (17, 320, 0),
                                            (9, 64, 1), (6, 100, 0), (2, 7, 1), (70, 33, 0), (67, 512, 0), (1, 1024, 0),
                                            (6, 1536, 0), (5, 2048, 0), (3, 1024, 1), (3, 384, 0), (2, 448, 0), (5, 576, 0),
                                            (2, 832, 0), (3, 1000, 0), (5, 333, 0), (2, 131, 1), (4, 70, 0),
                                            (3, 517, 1), (3, 4608, 0), (2, 6144, 0), (9, 3584, 0)])
def test_hand_written_row_scans_emulated_on_the_host_equal_numpy(rows, cols, skew):
    rng = np.random.default_rng(rows * 1000 + cols)
    dims = np.array([rows, cols, skew], np.uint32)
    n = rows * cols + skew
    for name, code, dtype in (('cumsum_f32', F32, np.float32), ('cumprod_f32', F32, np.float32),
                              ('cumsum_f64', F64, np.float64), ('cumprod_f64', F64, np.float64)):
        x = (rng.uniform(0.7, 1.3, (rows, cols)) * rng.choice([-1.0, 1.0], (rows, cols))).astype(dtype)
        x[0, 0] = -0.0
        got = host_emulation.run_program(host_emulation.build_hand_written('emu_' + name), [_skewed(x, skew), dims],
                                         [(code, dtype, [n]), (U32, np.uint32, [3])], [(code, dtype, [n])])[0]
        ref = (np.cumsum if 'cumsum' in name else np.cumprod)(x, axis=1, dtype=dtype)
        out = got[skew:].reshape(rows, cols)
        assert np.array_equal(out, ref) and np.array_equal(np.signbit(out), np.signbit(ref)), name


@pytest.mark.parametrize('rows,cols,skew', [(1, 4, 0), (2, 1024, 0), (3, 2048, 0), (2, 1028, 0), (5, 4100, 0), (1, 8192, 0),
                                            (4, 100, 0), (3, 258, 0), (2, 7, 0), (3, 64, 1)])
def test_reassociated_row_scans_emulated_on_the_host_are_close_to_numpy(rows, cols, skew):
    """The tree-shaped scan is not the sequential recurrence: it must agree with it to rounding (and bit for bit
    where there is nothing to reassociate: the first column, and shapes that fall back to the sequential kernels)."""
    rng = np.random.default_rng(rows * 1000 + cols)
    dims = np.array([rows, cols, skew], np.uint32)
    n = rows * cols + skew
    for name, code, dtype, tol in (('cumsum_f32', F32, np.float32, 2e-6), ('cumprod_f32', F32, np.float32, 2e-5),
                                   ('cumsum_f64', F64, np.float64, 1e-14), ('cumprod_f64', F64, np.float64, 1e-13)):
        x = rng.uniform(0.9, 1.1, (rows, cols)).astype(dtype)
        got = host_emulation.run_program(host_emulation.build_hand_written('emu_' + name + '_reassociated'),
                                         [_skewed(x, skew), dims], [(code, dtype, [n]), (U32, np.uint32, [3])],
                                         [(code, dtype, [n])])[0]
        out = got[skew:].reshape(rows, cols)
        ref = (np.cumsum if 'cumsum' in name else np.cumprod)(x.astype(np.float64), axis=1)
        assert np.array_equal(out[:, 0], x[:, 0]), name
        assert np.max(np.abs(out - ref) / np.abs(ref)) < tol * max(1.0, np.log2(cols)), name
        if skew or cols % (16 // np.dtype(dtype).itemsize) != 0:
            exact = (np.cumsum if 'cumsum' in name else np.cumprod)(x, axis=1, dtype=dtype)
            assert np.array_equal(out, exact), name + ': sequential fallback'


@pytest.mark.parametrize('name', ['c3_cumsum_f32', 'c3_cumprod_f64', 'c3_rowscan_shapes', 'int_accumulate',
                                  'accumulate_max'])
def test_generated_reassociating_scans_emulated_on_the_host(name):
    """The scans the 'fast' math mode runs as a tree (sums, products, running extrema): close to the oracle's
    sequential results, integer sums and extrema equal to them, no access outside a tensor."""
    outs = cases.CASE_BY_NAME[name].outputs()
    ref = oracle.profile(outs, 1, 0)[0]
    got = host_emulation.evaluate(outs, 3, {'math': 'fast'})
    for g, r in zip(got, ref):
        assert g.dtype == r.dtype and g.shape == r.shape
        if r.dtype.kind != 'f':
            assert np.array_equal(g, r)
        else:
            scale = np.max(np.abs(r), axis=-1, keepdims=True) + np.finfo(r.dtype).tiny
            assert np.max(np.abs(g.astype(np.float64) - r.astype(np.float64)) / scale) <= np.finfo(r.dtype).eps * 4 * r.shape[-1]
