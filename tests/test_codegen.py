"""HIP code generator: access analysis, template selection and that the generated sources compile for gfx950."""
import numpy as np
import pytest

import opveclib_amd as ovl
from opveclib_amd import hipgen, runtime, stdops, compiler
from opveclib_amd.hipgen.analysis import DagInfo
from opveclib_amd.hipgen import map_kernel
from opveclib_amd.operator import _build_op_dag
from opveclib_amd.fusion import _merge_op_dag
from opveclib_amd.examples import shift_cyclic, cumsum, gather_transpose, expm1
from opveclib_amd.lstm import lstm, lstm_grad
from tests import cases


def fused(outputs):
    dag, _ = _merge_op_dag(_build_op_dag(*outputs).proto_dag, None)
    return dag


def test_affine_forms_of_tensor_accesses():
    concat = np.zeros((8, 4 * 16), np.float32)
    c = np.zeros((8, 16), np.float32)
    info = DagInfo(lstm(concat, c, forget_bias=1.0).expression_dag)
    reads = [(t.io_index, a.signature()) for n, t, a in info.tensor_accesses() if n.code == ovl.language.READ_TENSOR]
    p0, p1 = ('p', 0), ('p', 1)
    assert reads == [(0, (((p0, 64), (p1, 1)), 0)), (0, (((p0, 64), (p1, 1)), 16)),
                     (0, (((p0, 64), (p1, 1)), 32)), (0, (((p0, 64), (p1, 1)), 48)),
                     (1, (((p0, 16), (p1, 1)), 0))]
    for _, tensor, aff in info.tensor_accesses():
        assert 0 <= aff.lo and aff.hi < tensor.size


def test_modulo_that_cannot_wrap_is_dropped_and_one_that_can_is_not():
    a = np.zeros((16, 32), np.float32)
    info = DagInfo(gather_transpose(a, a.reshape(-1), alpha=0.5, stride=3).expression_dag)
    by_tensor = {}
    for node, tensor, aff in info.tensor_accesses():
        by_tensor.setdefault((node.code, tensor.io_index), []).append(aff)
    gather = by_tensor[(ovl.language.READ_TENSOR, 1)][0]
    assert gather is not None and gather.signature() == (((('p', 0), 3), (('p', 1), 1)), 0)   # (i*3+j) % 512 == i*3+j
    scatter = by_tensor[(ovl.language.ASSIGN_TENSOR, 0)][0]
    assert scatter.signature() == (((('p', 0), 1), (('p', 1), 16)), 0)                        # out[j, i]

    info = DagInfo(shift_cyclic(np.zeros(64, np.float32)).expression_dag)
    store = [aff for node, _, aff in info.tensor_accesses() if node.code == ovl.language.ASSIGN_TENSOR][0]
    assert store is None                                                                     # (p+1) % n wraps


def test_unsigned_wraparound_is_not_affine():
    info = DagInfo(cases.pad(np.zeros((3, 5)), n=2).expression_dag)
    read = [aff for node, _, aff in info.tensor_accesses() if node.code == ovl.language.READ_TENSOR][0]
    assert read is None             # the row/column come from reassigned variables


def test_vector_width_selection():
    f32 = np.zeros((8, 64), np.float32)
    assert map_kernel.choose_vec(DagInfo(stdops.add(f32, f32).expression_dag)) == 4
    f64 = np.zeros((8, 64), np.float64)
    assert map_kernel.choose_vec(DagInfo(stdops.add(f64, f64).expression_dag)) == 2
    i8 = np.zeros((8, 64), np.int8)
    assert map_kernel.choose_vec(DagInfo(stdops.add(i8, i8).expression_dag)) == 16
    odd = np.zeros((8, 63), np.float32)
    assert map_kernel.choose_vec(DagInfo(stdops.add(odd, odd).expression_dag)) == 1
    two = np.zeros((8, 62), np.float32)
    assert map_kernel.choose_vec(DagInfo(stdops.add(two, two).expression_dag)) == 2
    # accumulate along the last axis: workers are rows, nothing is contiguous across workers
    assert map_kernel.choose_vec(DagInfo(cumsum(f32, axis=1).expression_dag)) == 1


def test_template_selection():
    def template(op, options=None):
        dag = op.expression_dag if hasattr(op, 'expression_dag') else op
        return hipgen.generate(dag, 'f' + '4' * 56, options).launch

    f32 = np.zeros((8, 64), np.float32)
    assert template(stdops.add(f32, f32))['template'] == 'map'
    # last-axis accumulation with a chunkable row length: the order-preserving row scan
    scan = template(cumsum(np.zeros((48, 1024), np.float32), axis=1))
    assert scan['template'] == 'skewscan' and scan['blocks_needed'] == 3       # 16 rows per workgroup
    # 8-byte elements: the lane-skewed recurrence fed from LDS, four rows per workgroup.  With at most one workgroup
    # per compute unit (or whole rounds of them and long rows) the scanning wavefront keeps no results and a second
    # wavefront recomputes them; with more, three of the lockstep variant's workgroups share a compute unit
    carry = template(cumsum(np.zeros((1024, 16384), np.float64), axis=1))
    assert carry['template'] == 'carryscan' and carry['blocks_needed'] == 256 and carry['block'] == 320
    assert template(cumsum(np.zeros((2048, 16384), np.float64), axis=1))['template'] == 'carryscan'
    fed = template(cumsum(np.zeros((4096, 4096), np.float64), axis=1))
    assert fed['template'] == 'fedscan' and fed['blocks_needed'] == 1024
    assert template(cumsum(np.zeros((1500, 8192), np.float64), axis=1))['template'] == 'fedscan'
    assert template(cumsum(np.zeros((1024, 16384), np.float64), axis=1), {'template': 'fedscan'})['template'] == 'fedscan'
    # (rows that are not whole chunks of at least 128 columns keep the lockstep variant or the register-fed scan)
    assert template(cumsum(np.zeros((64, 1088), np.float64), axis=1))['template'] == 'fedscan'
    assert template(cumsum(np.zeros((1024, 16384), np.float64), axis=1), {'template': 'skewscan'})['blocks_needed'] == 64
    lds = template(cumsum(np.zeros((48, 1024), np.float32), axis=1), {'template': 'rowscan'})
    assert lds['template'] == 'rowscan' and lds['blocks_needed'] == 48
    assert template(cumsum(np.zeros((48, 1024), np.float32), axis=1), {'template': 'map'})['template'] == 'map'
    # rows that are not a whole number of groups of 64 columns end in columns scanned by one lane; rows that do not
    # start on 16-byte boundaries are moved with unaligned vectors; rows shorter than one group, other axes and loop
    # bodies with branches use the general template
    ragged = template(cumsum(np.zeros((48, 1000), np.float32), axis=1))
    assert ragged['template'] == 'skewscan' and ragged['align'] == {('in', 0): 16, ('out', 0): 16}
    unaligned = template(cumsum(np.zeros((48, 1001), np.float32), axis=1))
    assert unaligned['template'] == 'skewscan' and unaligned['align'] == {('in', 0): 4, ('out', 0): 4}
    assert template(cumsum(np.zeros((48, 63), np.float32), axis=1))['template'] == 'map'
    # along another axis: a short axis keeps one worker per thread, a long one with few lines gets strips of 64 lines
    assert template(cumsum(np.zeros((48, 1024), np.float32), axis=0))['template'] == 'map'
    # (up to 32768 lines: sixteen lanes per line, strips of 8 to 64 lines for about 256 workgroups)
    col = template(cumsum(np.zeros((1000, 200), np.float64), axis=0))
    # (strips of 8 lines: two scanning wavefronts and four that only move data; 8-byte elements add two finishing ones)
    assert col['template'] == 'colskew' and col['blocks_needed'] == 25 and col['block'] == 128 + 128 + 256
    col = template(cumsum(np.zeros((1000, 200), np.float64), axis=0), {'scan_carry': False})
    assert col['template'] == 'colskew' and col['blocks_needed'] == 25 and col['block'] == 128 + 256
    old = template(cumsum(np.zeros((1000, 200), np.float64), axis=0), {'scan_movers': 0})
    assert old['template'] == 'colskew' and old['block'] == 128
    mid = template(cumsum(np.zeros((3, 500, 96), np.float32), axis=1))
    assert mid['template'] == 'colskew' and mid['blocks_needed'] == 3 * 12
    wide = template(cumsum(np.zeros((200, 16384), np.float32), axis=0))
    assert wide['template'] == 'colskew' and wide['blocks_needed'] == 256 and wide['block'] == 1024
    many = template(cumsum(np.zeros((200, 65536), np.float32), axis=0))
    assert many['template'] == 'colscan' and many['blocks_needed'] == 1024 and many['block'] == 1024
    more = template(cumsum(np.zeros((100, 100000), np.float32), axis=0))
    assert more['template'] == 'colscan' and more['blocks_needed'] == 1563
    assert template(cumsum(np.zeros((128, 1 << 17), np.float32), axis=0))['template'] == 'colscan'    # however many lines
    assert template(cumsum(np.zeros((32, 1 << 17), np.float32), axis=0))['template'] == 'map'         # a short axis
    assert template(cases.dot(np.zeros((16, 64)), np.zeros((16, 64))))['template'] == 'map'
    # transposed store of a rank-2 workgroup: LDS tiles; the gather is one dword-aligned 128-bit load per thread
    tr = template(gather_transpose(np.zeros((192, 320), np.float32), np.zeros(192 * 320, np.float32),
                                   alpha=0.5, stride=3))
    assert tr['template'] == 'transpose' and tr['vector_loads'] == 2 and tr['vector_stores'] == 1
    assert tr['blocks_needed'] == 6 * 2                    # tiles of 32 x 256 workers
    wraps = template(gather_transpose(np.zeros((192, 320), np.float32), np.zeros(192 * 320, np.float32),
                                      alpha=0.5, stride=7919))
    assert wraps['template'] == 'transpose' and wraps['vector_loads'] == 1        # the gather index may wrap: scalar
    odd = template(gather_transpose(np.zeros((6, 9), np.float32), np.zeros(54, np.float32), alpha=0.5, stride=1))
    # (extents that no vector width divides still go through the tile, one element per access)
    assert odd['template'] == 'transpose' and odd['vec'] == 1


def test_a_row_sum_into_one_column_of_a_full_size_output_is_not_taken_for_a_scan():
    """A worker that stores only before its loop (a row sum kept in column 0 of an output as large as the input) has
    the loop shape of a scan but nothing to store per column: the scan templates would write registers that nothing
    assigned over the whole output.  It must go to a template that stores what the worker stores."""
    @ovl.operator()
    def sum_into_first_column(x):
        rows, cols = x.shape
        row = ovl.position_in([rows])[0]
        out = ovl.output_like(x)
        acc = ovl.variable(0, x.dtype)
        acc <<= x[row, 0]
        out[row, 0] = acc
        for i in ovl.arange(1, cols):
            acc <<= acc + x[row, i]
        return out

    generated = hipgen.generate(sum_into_first_column(np.zeros((48, 1024), np.float32)).expression_dag, 'f' + '5' * 56)
    assert generated.launch['template'] not in ('skewscan', 'fedscan', 'carryscan', 'rowscan', 'treescan')
    from opveclib_amd.hipgen import rowscan_kernel
    info = DagInfo(sum_into_first_column(np.zeros((48, 1024), np.float32)).expression_dag)
    assert rowscan_kernel.plan(info, need_chunk=False, multi=True) is None


def test_chain8_kernel_shape():
    a = np.zeros((64, 256), np.float32)
    s = np.array([1.0001], np.float32)
    dag = fused([cases.chain8(a, a.copy(), s)[-1][0]])
    gen = hipgen.generate(dag.operators[0], 'f' + '0' * 56)
    assert gen.launch['template'] == 'map' and gen.launch['vec'] == 4
    assert gen.launch['vector_loads'] == 2          # A and B once each, although B is used twice
    assert gen.launch['vector_stores'] == 1         # stores under if/elif/else chains still become one vector store
    assert gen.algorithmic_bytes == 3 * a.size * 4 + 4
    assert gen.entry == 'f' + '0' * 56 + '_generic_hip'
    assert 'ovl_tanhf' in gen.source and 'ovl_expf' in gen.source and 'ovl_logf' in gen.source


def test_conditional_store_without_else_stays_scalar():
    @ovl.operator()
    def maybe(x):
        out = ovl.output_like(x)
        pos = ovl.position_in(x.shape)
        with ovl.if_(x[pos] > 0):
            out[pos] = x[pos]
        return out
    gen = hipgen.generate(maybe(np.zeros((4, 64), np.float32)).expression_dag, 'f' + '1' * 56)
    assert gen.launch['vector_loads'] == 1 and gen.launch['vector_stores'] == 0


@pytest.mark.parametrize('name', ['c1_shift', 'c2_chain', 'c3_cumsum_f64', 'c4_lstm_grad', 'c5_gather_transpose',
                                  'local_tensor', 'concat_ragged', 'dot', 'binary_mod_int8', 'unary_tan_float64'])
def test_generated_sources_compile(name):
    outs = cases.CASE_BY_NAME[name].outputs()
    for op in fused(outs).operators:
        gen, so_path = runtime.build_operator(op)
        assert so_path.endswith('_generic_hip.so')
        assert compiler.find_library(gen.source) == so_path


def test_entry_point_validates_before_touching_the_gpu(launcher_library):
    """Argument checks of a generated entry point run on the host, so they can be exercised without a device."""
    import ctypes
    from opveclib_amd import launcher
    a = np.zeros(64, np.float32)
    gen, so_path = runtime.build_operator(stdops.add(a, a).expression_dag)
    lib = launcher.OperatorLibrary(so_path, gen.entry, gen.info_symbol)
    assert lib.info['template'] == 'map' and lib.info['algorithmic_bytes'] == 3 * 64 * 4
    good = launcher.tensor_array([(4096, 2, 64), (8192, 2, 64)])
    out = launcher.tensor_array([(12288, 2, 64)])
    L = launcher_library
    assert L.ovl_launch_fn(lib.fn, good, 1, out, 1, None) == launcher.OVL_EARGS         # wrong input count
    assert L.ovl_launch_fn(lib.fn, good, 2, out, 0, None) == launcher.OVL_EARGS         # wrong output count
    bad_len = launcher.tensor_array([(4096, 2, 63), (8192, 2, 64)])
    assert L.ovl_launch_fn(lib.fn, bad_len, 2, out, 1, None) == launcher.OVL_EARGS
    bad_type = launcher.tensor_array([(4096, 3, 64), (8192, 2, 64)])
    assert L.ovl_launch_fn(lib.fn, bad_type, 2, out, 1, None) == launcher.OVL_EARGS
    misaligned = launcher.tensor_array([(4100, 2, 64), (8192, 2, 64)])
    assert L.ovl_launch_fn(lib.fn, misaligned, 2, out, 1, None) == launcher.OVL_EALIGN
    with pytest.raises(launcher.LauncherError) as err:
        lib.launch(bad_len, 2, out, 1, None)
    assert err.value.code == launcher.OVL_EARGS


def test_if_conversion_of_pure_conditional_chains():
    """Chains that only compute and assign become selects; chains with memory accesses of their own stay branches."""
    from opveclib_amd.examples import expm1
    x = np.zeros((8, 64), np.float32)
    converted = hipgen.generate(expm1(x).expression_dag, 'f' + '5' * 56).source
    assert 'if(' not in converted and converted.count('const bool t') == 4      # four branches, four predicates
    assert converted.count(' ? (') == 4
    kept = hipgen.generate(expm1(x).expression_dag, 'f' + '5' * 56, {'if_conversion': False}).source
    assert kept.count('if(') == 3 and 'const bool t' not in kept
    # clip stores a constant or the input under three conditions: also convertible (register-buffered vector store)
    clipped = hipgen.generate(cases.clip(np.zeros(256), threshold1=0.1, threshold2=0.9).expression_dag,
                              'f' + '5' * 56).source
    assert 'if(' not in clipped
    # a branch that reads a tensor at a computed index must not be speculated
    @ovl.operator()
    def guarded_gather(x, idx):
        pos = ovl.position_in(x.shape)
        out = ovl.output_like(x)
        i = idx[pos]
        with ovl.if_(i < x.shape[0]):
            out[pos] = x[i]
        with ovl.else_():
            out[pos] = 0
        return out
    guarded = hipgen.generate(guarded_gather(np.zeros(64, np.float32), np.zeros(64, np.uint32)).expression_dag,
                              'f' + '5' * 56).source
    assert 'if(' in guarded
    # integer division stays guarded
    @ovl.operator()
    def guarded_divide(a, b):
        pos = ovl.position_in(a.shape)
        out = ovl.output_like(a)
        with ovl.if_(b[pos] != 0):
            out[pos] = a[pos] / b[pos]
        with ovl.else_():
            out[pos] = 0
        return out
    ints = hipgen.generate(guarded_divide(np.zeros(64, np.int32), np.zeros(64, np.int32)).expression_dag,
                           'f' + '5' * 56).source
    assert 'if(' in ints
    floats = hipgen.generate(guarded_divide(np.zeros(64, np.float32), np.zeros(64, np.float32)).expression_dag,
                             'f' + '5' * 56).source
    assert 'if(' not in floats


def test_workgroups_beyond_32_bit_positions_are_refused():
    @ovl.operator()
    def fill(shape_like):
        pos = ovl.position_in([1 << 16, 1 << 16])
        out = ovl.output([4], ovl.float32)
        out[pos[0] % 4] = 1
        return out
    with pytest.raises(ValueError):
        hipgen.generate(fill(np.zeros(4, np.float32)).expression_dag, 'f' + '6' * 56)


def test_largest_workgroups_launch_fewer_than_2_to_32_threads_and_step_without_wrapping():
    """A scalar map over 2^32 - 3 workers: 2^24 workgroups of 256 threads would make gridDim.x * 256 wrap to zero (a
    stride of zero never ends), and `v += stride` would wrap for the threads that take a second step."""
    @ovl.operator()
    def fill(shape_like):
        pos = ovl.position_in([(1 << 32) - 3])
        out = ovl.output([7], ovl.float32)
        out[pos[0] % 7] = 1
        return out
    generated = hipgen.generate(fill(np.zeros(4, np.float32)).expression_dag, 'f' + '7' * 56)
    assert generated.launch['vec'] == 1 and generated.launch['blocks_needed'] == 1 << 24
    assert 'uint32_t grid = %du;' % ((1 << 24) - 1) in generated.source
    assert 'v = (num_vectors - v > stride) ? v + stride : num_vectors' in generated.source
    assert 'v += stride' not in generated.source

    # a grid that covers the work needs no loop at all; a capped grid strides
    small = stdops.add(np.zeros(4096, np.float32), np.zeros(4096, np.float32)).expression_dag
    assert 'stride' not in hipgen.generate(small, 'f' + '8' * 56).source
    capped = hipgen.generate(small, 'f' + '8' * 56, {'grid_cap': 1})
    assert 'uint32_t grid = 1u;' in capped.source and 'stride' in capped.source


def test_missing_operators_of_a_dag_are_built_side_by_side(tmp_path, monkeypatch):
    """Cold start: every operator of a DAG without a library is generated and compiled before the first launch."""
    import os
    import threading
    import numpy as np
    from opveclib_amd import compiler, local, runtime, stdops
    from opveclib_amd.operator import _build_op_dag, _normalise_output_list, _op_hash

    monkeypatch.setattr(local, 'cache_directory', str(tmp_path))
    monkeypatch.setattr(local, 'prebuilt_directory', str(tmp_path / 'none'))
    monkeypatch.setattr(compiler, 'prebuild_mode', False)
    seen_threads = set()
    real_build = compiler.build_library

    def recording_build(source):
        seen_threads.add(threading.get_ident())
        return real_build(source)

    monkeypatch.setattr(compiler, 'build_library', recording_build)
    x = np.zeros((3, 20), dtype=np.float32)                # a shape no other test uses
    out = stdops.sub(stdops.mul(stdops.add(x, x), x), x)
    dag = _build_op_dag(*_normalise_output_list(out)).proto_dag
    assert len(dag.operators) == 3
    runtime._build_missing(dag.operators, None)
    for op in dag.operators:
        key = (_op_hash(op), repr([]))
        assert key in runtime._generated
        assert os.path.exists(runtime._generated[key][1])
    assert len(seen_threads) == 3 and threading.get_ident() not in seen_threads
    # nothing left to do the second time
    seen_threads.clear()
    runtime._build_missing(dag.operators, None)
    assert not seen_threads


def test_clear_op_cache_removes_cached_operators_only(tmp_path, monkeypatch):
    """`clear_op_cache` (the reference's local.py:43-50) deletes what was compiled on demand in the per-user cache
    and nothing else: other files there and the prebuilt operators of the package stay."""
    from opveclib_amd import local
    cache = tmp_path / 'cache'
    cache.mkdir()
    prebuilt = tmp_path / 'prebuilt'
    prebuilt.mkdir()
    for name in ('f0123_generic_hip.so', 'f0123_generic_hip.hip', 'fabc_generic_hip.so'):
        (cache / name).write_text('x')
        (prebuilt / name).write_text('x')
    (cache / 'notes.txt').write_text('keep')
    monkeypatch.setattr(local, 'cache_directory', str(cache))
    monkeypatch.setattr(local, 'prebuilt_directory', str(prebuilt))
    local.clear_op_cache()
    assert sorted(p.name for p in cache.iterdir()) == ['notes.txt']
    assert len(list(prebuilt.iterdir())) == 3
    local.clear_op_cache()                      # an empty cache is fine
    monkeypatch.setattr(local, 'cache_directory', str(tmp_path / 'missing'))
    local.clear_op_cache()                      # and so is a cache that does not exist yet


def test_repeated_subexpressions_are_evaluated_once():
    """The reference's LSTM gradient repeats sigmoid(i), sigmoid(f + bias), tanh(j) and tanh(new_c) inside every
    gate's derivative (lstm/lstm.py:84-103): the emitted body evaluates three exponentials and two tanh, as a
    hand-written kernel would, and the operands of a repeated read are requested once."""
    from opveclib_amd import hipgen, workloads
    from opveclib_amd.workloads import Spec
    op, = workloads.fused_operators(workloads.lstm_grad_outputs(Spec((64, 256)), Spec((64, 64)), Spec((64, 64)),
                                                                Spec((64, 64))))
    merged = hipgen.generate(op, 'f' + '0' * 56, {'per_thread': 1}).source
    repeated = hipgen.generate(op, 'f' + '0' * 56, {'cse': False, 'per_thread': 1}).source
    assert (merged.count('ovl_expf'), merged.count('ovl_tanhf(')) == (3, 2)
    assert repeated.count('ovl_expf') > 3 and repeated.count('ovl_tanhf(') > 2
    # a value computed under a condition is not reused outside it
    import opveclib_amd as ovl

    @ovl.operator()
    def guarded(x):
        out = ovl.output_like(x)
        pos = ovl.position_in(x.shape)
        y = ovl.variable(0, x.dtype)
        with ovl.if_(x[pos] > 0):
            y <<= ovl.exp(x[pos])
        out[pos] = y + ovl.exp(x[pos])
        return out

    text = hipgen.generate(guarded(Spec((256,))).expression_dag, 'f' + '1' * 56,
                           {'if_conversion': False, 'per_thread': 1}).source
    assert text.count('ovl_expf') == 2


def test_vectors_per_thread_follow_the_size_of_the_grid():
    """Outside the 'exact' mode a thread of a body with few streams and some arithmetic takes four vectors, but only
    while the grid keeps eight workgroups per compute unit: a small tensor's time is latency."""
    from opveclib_amd import workloads
    from opveclib_amd.workloads import Spec

    def launch(outputs, mode):
        op, = workloads.fused_operators(outputs)
        return hipgen.generate(op, 'f' + '5' * 56, {'math': mode}).launch

    big = [Spec((8192, 8192), np.float32), Spec((8192, 8192), np.float32), Spec((1,), np.float32)]
    assert launch(workloads.chain8_outputs(*big), 'ulp2')['per_thread'] == 4
    assert launch(workloads.chain8_outputs(*big), 'exact')['per_thread'] == 1
    assert launch(workloads.c1_outputs(Spec((1 << 20,), np.float32)), 'ulp2')['per_thread'] == 1
    assert launch(workloads.c1_outputs(Spec((1 << 23,), np.float32)), 'ulp2')['per_thread'] == 4
    assert launch(workloads.c1_outputs(Spec((1 << 22,), np.float32)), 'ulp2')['per_thread'] == 2
