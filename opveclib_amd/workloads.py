"""
The operator graphs of the benchmark configurations, and the step that compiles their kernels ahead of time.

Each ``*_outputs`` function applies operators to its arguments and returns the requested outputs; the arguments may be
arrays, device tensors or :class:`Spec` objects (shape and element type only), which is enough to trace, fuse,
generate and compile an operator without allocating anything.  ``prebuild`` does that for every configuration at its
full size and in every math mode the benchmark reports, into the package's prebuilt directory.
"""

import numpy as np


class Spec(object):
    """Shape and dtype of a tensor, enough to trace an operator without allocating the tensor."""

    def __init__(self, shape, dtype=np.float32):
        self.shape = list(shape)
        self.dtype = np.dtype(dtype).type


def uniform(rng, lo, hi, shape, dtype=np.float32):
    """``lo + (hi - lo) * rng.random(shape)`` in ``dtype``."""
    return (lo + (hi - lo) * rng.random(shape, dtype=dtype)).astype(dtype)


# ----------------------------------------------------------------------------------------------------------------------
# operator graphs
# ----------------------------------------------------------------------------------------------------------------------
def chain8_outputs(a, b, s):
    """The fused 8-op chain (add, mul by scalar, tanh, sigmoid, log1p, expm1, sub, abs): its last stage."""
    from .examples import chain8
    return [chain8(a, b, s)[-1][0]]


def chain8_stage_outputs(a, b, s):
    """Every stage of the 8-op chain as a requested output (the optimizer still fuses them into one kernel)."""
    from .examples import chain8
    return [t[0] for t in chain8(a, b, s)]


def copy_outputs(x):
    """out[pos] = x[pos]: the plain copy kernel that calibrates the profiler's byte counters."""
    import opveclib_amd as ovl

    @ovl.operator()
    def copy(arg):
        pos = ovl.position_in(arg.shape)
        out = ovl.output_like(arg)
        out[pos] = arg[pos]
        return out

    return [copy(x)[0]]


def c1_outputs(x):
    from .examples import shift_cyclic, expm1, log1p
    return [log1p(expm1(shift_cyclic(x)))[0]]


def cumsum_outputs(x, axis=1):
    from .examples import cumsum
    return [cumsum(x, axis=axis)[0]]


def cumprod_outputs(x, axis=1):
    from .examples import cumprod
    return [cumprod(x, axis=axis)[0]]


def lstm_outputs(concat, c):
    from .lstm import lstm
    op = lstm(concat, c, forget_bias=1.0)
    return [op[0], op[1]]


def stdops_lstm_outputs(concat, c):
    """The LSTM cell composed of library operators as the reference's merge test writes it
    (opveclib/test/test_operator_merge.py:311-321; no forget bias there): new_c and new_h.  The optimizer fuses the
    ten operators into one kernel."""
    from . import stdops
    parts = stdops.split(concat, split_dim=1, num_split=4)
    i, j, f, o = (parts[k] for k in range(4))
    new_c = stdops.mul(c, stdops.sigmoid(f)) + stdops.sigmoid(i) * stdops.tanh(j)
    new_h = stdops.tanh(new_c) * stdops.sigmoid(o)
    return [new_c[0], new_h[0]]


#: names of the stages `stdops_lstm_stage_outputs` returns, in its order
STDOPS_LSTM_STAGES = ('i', 'j', 'f', 'o', 'sigmoid_f', 'sigmoid_i', 'tanh_j', 'c_sigmoid_f', 'sigmoid_i_tanh_j', 'new_c',
                      'tanh_new_c', 'sigmoid_o', 'new_h')


def stdops_lstm_stage_outputs(concat, c):
    """Every operator output of the composed cell as a requested output, in the order of `STDOPS_LSTM_STAGES` (the
    optimizer still fuses the operators into one kernel, which then also stores the intermediates)."""
    from . import stdops
    parts = stdops.split(concat, split_dim=1, num_split=4)
    i, j, f, o = (parts[k] for k in range(4))
    sigmoid_f, sigmoid_i, tanh_j = stdops.sigmoid(f), stdops.sigmoid(i), stdops.tanh(j)
    left, right = stdops.mul(c, sigmoid_f), sigmoid_i * tanh_j
    new_c = left + right
    tanh_new_c, sigmoid_o = stdops.tanh(new_c), stdops.sigmoid(o)
    new_h = tanh_new_c * sigmoid_o
    return [i, j, f, o, sigmoid_f[0], sigmoid_i[0], tanh_j[0], left[0], right[0], new_c[0], tanh_new_c[0], sigmoid_o[0],
            new_h[0]]


def conv1d_reference_inputs():
    """The tensors of the reference's conv1D timing run (opveclib/examples/conv1D.py:279-319): TensorFlow sizes
    [5, 1, 1000, 3] and [1, 13, 3, 10] filled with 1, 2, 3, ... as float64, in the 'NEC' layout of the OVL operator:
    input [5 batches, 1000 elements, 3 channels], filters [10 filters, 13 taps, 3 channels]."""
    batches, elements, channels, taps, filters = 5, 1000, 3, 13, 10
    x = np.arange(1, batches * elements * channels + 1, dtype=np.float64).reshape(batches, elements, channels)
    flat = np.arange(1, taps * channels * filters + 1, dtype=np.float64)
    # TensorFlow's filter layout is [tap, channel, filter]; OVL's 'NEC' layout is [filter, tap, channel]
    v = np.ascontiguousarray(flat.reshape(taps, channels, filters).transpose(2, 0, 1))
    return x, v


def conv1d_outputs(x, v):
    """The convolution of that run: mode 'same', filters as they are, 'NEC' layout (conv1D.py:327)."""
    from .examples import conv_1d
    return [conv_1d(x, v, mode='same', kernel_orientation='as-is', data_format='NEC')[0]]


def lstm_grad_outputs(concat, c, dc, dh):
    from .lstm import lstm_grad
    op = lstm_grad(concat, c, dc, dh, forget_bias=1.0)
    return [op[0], op[1]]


def dot_outputs(a, b):
    """One dot product per row, accumulated in the order of the columns: the operator of the reference's dot-product
    test (opveclib/test/test_dot_product.py:27-45), loop bound in a variable as there."""
    import opveclib_amd as ovl

    @ovl.operator()
    def dot(input0, input1):
        num_vectors = input0.shape[0]
        dot_out = ovl.output(num_vectors, input0.dtype)
        pos = ovl.position_in(num_vectors)[0]
        accum = ovl.variable(0.0, input0.dtype)
        num_elements = ovl.variable(input0.shape[1], ovl.uint32)
        for i in ovl.arange(num_elements):
            accum <<= accum + input0[pos, i] * input1[pos, i]
        dot_out[pos] = accum
        return dot_out

    return [dot(a, b)]


def column_sum_outputs(x):
    """The sum of every column of a matrix, rows added in order."""
    import opveclib_amd as ovl

    @ovl.operator()
    def column_sum(arg):
        rows, cols = arg.shape
        out = ovl.output([cols], arg.dtype)
        pos = ovl.position_in([cols])[0]
        acc = ovl.variable(0, arg.dtype)
        for i in ovl.arange(rows):
            acc <<= acc + arg[i, pos]
        out[pos] = acc
        return out

    return [column_sum(x)]


def gather_outputs(a, b_flat):
    from .examples import gather_transpose
    return [gather_transpose(a, b_flat, alpha=0.5, stride=7919)[0]]


#: the LSTM cell sizes the reference's profiler runs (lstm/profile_lstm.py:41-51): batch 20, these unit counts
REFERENCE_LSTM_BATCH = 20
REFERENCE_LSTM_UNITS = (200, 650, 1500)
#: the shape of the reference's accumulate timing (opveclib/examples/test_perf_accumulate.py:35-47): float64, axis 0
REFERENCE_CUMSUM_SHAPE = (10000, 1000)


#: row lengths of the float32 scans that `bench.py --only "row stride"` times for counter collection: rows of 64 KiB,
#: 64 KiB + 256 bytes and 65 KiB
ROW_STRIDE_PROBE_COLUMNS = (16384, 16448, 16640)


def all_workload_outputs():
    """Operator outputs of every benchmark workload at full size, built from shape specs."""
    f32, f64 = np.float32, np.float64
    yield chain8_outputs(Spec((8192, 8192)), Spec((8192, 8192)), Spec((1,)))
    yield chain8_stage_outputs(Spec((8192, 8192)), Spec((8192, 8192)), Spec((1,)))
    yield copy_outputs(Spec((8192, 8192)))
    yield copy_outputs(Spec((1024,)))               # one workgroup: the floor of a launch
    yield c1_outputs(Spec((1 << 20,)))
    yield cumsum_outputs(Spec((4096, 16384), f32))
    yield cumprod_outputs(Spec((4096, 16384), f32))
    yield cumsum_outputs(Spec((1024, 16384), f64))
    yield cumprod_outputs(Spec((1024, 16384), f64))
    yield lstm_outputs(Spec((4096, 4096)), Spec((4096, 1024)))
    yield lstm_grad_outputs(Spec((4096, 4096)), Spec((4096, 1024)), Spec((4096, 1024)), Spec((4096, 1024)))
    yield gather_outputs(Spec((16384, 16384)), Spec((16384 * 16384,)))
    yield stdops_lstm_outputs(Spec((4096, 4096)), Spec((4096, 1024)))
    yield conv1d_outputs(Spec((5, 1000, 3), f64), Spec((10, 13, 3), f64))
    yield cumsum_outputs(Spec(REFERENCE_CUMSUM_SHAPE, f64), axis=0)
    for cols in ROW_STRIDE_PROBE_COLUMNS:           # bench.py --only "row stride"
        yield cumsum_outputs(Spec((4096, cols), f32))
    yield dot_outputs(Spec((4096, 16384), f32), Spec((4096, 16384), f32))
    yield column_sum_outputs(Spec(REFERENCE_CUMSUM_SHAPE, f64))
    for units in REFERENCE_LSTM_UNITS:
        batch = REFERENCE_LSTM_BATCH
        yield lstm_outputs(Spec((batch, 4 * units)), Spec((batch, units)))
        yield lstm_grad_outputs(Spec((batch, 4 * units)), Spec((batch, units)), Spec((batch, units)),
                                Spec((batch, units)))


def fused_operators(outputs):
    """The operators of the fused DAG behind ``outputs``."""
    from .operator import _build_op_dag
    from .fusion import _merge_op_dag
    dag, _ = _merge_op_dag(_build_op_dag(*outputs).proto_dag, None)
    return list(dag.operators)


def unfused_operators(outputs):
    """The operators behind ``outputs`` as written, one kernel each."""
    from .operator import _build_op_dag
    return list(_build_op_dag(*outputs).proto_dag.operators)


def prebuild(force=False, workers=8):
    """
    Compile the kernels of every benchmark workload into the package's prebuilt directory: each in the default
    'exact' math mode, and those that call exp, log, tanh or divide also in the 'ulp2' and 'fast' modes.  Needs
    hipcc, not a GPU.  ``force`` compiles even where a built library exists.  Returns the number of libraries.
    """
    from concurrent.futures import ThreadPoolExecutor
    from . import compiler, runtime
    from . import language as lang

    jobs = {}
    for outputs in all_workload_outputs():
        for op in fused_operators(outputs):
            key = op.SerializeToString()
            jobs[(key, 'exact')] = (op, None)
            if any(e.code in (lang.EXP, lang.LOG, lang.TANH, lang.DIVIDE) for e in op.expressions):
                for mode in ('ulp2', 'fast'):
                    jobs[(key, mode)] = (op, {'math': mode})
            elif op.name == 'accumulate':
                jobs[(key, 'fast')] = (op, {'math': 'fast'})       # the reassociating scan
    # the single operators of the chain at full size, bit-exact: what the benchmark compares each stage with
    headline = chain8_stage_outputs(Spec((8192, 8192)), Spec((8192, 8192)), Spec((1,)))
    for op in unfused_operators(headline):
        jobs[(op.SerializeToString(), 'exact')] = (op, None)
        # ... and each operator on its own in the default mode, compared with the CPU oracle's stages
        jobs[(op.SerializeToString(), 'ulp2')] = (op, {'math': 'ulp2'})
    # the composed LSTM cell: the fused kernel that stores every operator's output, and the single bit-exact
    # operators its stages are compared with
    cell = stdops_lstm_stage_outputs(Spec((4096, 4096)), Spec((4096, 1024)))
    for op in fused_operators(cell):
        jobs[(op.SerializeToString(), 'ulp2')] = (op, {'math': 'ulp2'})
    for op in unfused_operators(cell):
        jobs[(op.SerializeToString(), 'exact')] = (op, None)
    previous = compiler.prebuild_mode, compiler.force_rebuild
    compiler.prebuild_mode, compiler.force_rebuild = True, bool(force)
    try:
        with ThreadPoolExecutor(max_workers=workers) as pool:
            list(pool.map(lambda job: runtime.build_operator(*job), jobs.values()))
    finally:
        compiler.prebuild_mode, compiler.force_rebuild = previous
        if force:
            runtime._generated.clear()
    return len(jobs)
