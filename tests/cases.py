"""
The shared table of parity cases.

Every case builds a small DAG of operators from seeded inputs.  The GPU tests evaluate each case through the HIP
path and compare it with the CPU oracle; the repository build step walks the same table to compile every HIP
operator (and every oracle operator) ahead of time, so that a GPU run only loads binaries.
"""

import numpy as np

import opveclib_amd as ovl
from opveclib_amd import stdops
from opveclib_amd import language as lang
from opveclib_amd.examples import (chain8, shift_cyclic, cumsum, cumprod, accumulate, expm1, log1p, absolute,
                                   gather_transpose)
from opveclib_amd.lstm import lstm, lstm_grad


class Case(object):
    """
    :param name: test id
    :param build: function(rng) -> list of operator outputs
    :param max_ulp: 0 demands bit-exact equality with the oracle; otherwise the largest allowed distance in units in
        the last place (float32) and, for float64 outputs, ``rel`` bounds the relative error instead
    """

    def __init__(self, name, build, max_ulp=0, rel=0.0, seed=0):
        self.name = name
        self.build = build
        self.max_ulp = max_ulp
        self.rel = rel
        self.seed = seed

    def outputs(self):
        return self.build(np.random.default_rng(self.seed))

    def __repr__(self):
        return self.name


def uniform(rng, lo, hi, shape, dtype=np.float32):
    return (lo + (hi - lo) * rng.random(shape, dtype=dtype)).astype(dtype)


def all_outputs(op):
    """Every output of an operator application (gradient-decorated operators already return such a list)."""
    if isinstance(op, (list, tuple)):
        return list(op)
    return [op[i] for i in range(len(op.output_types))]


# ----------------------------------------------------------------------------------------------------------------------
# the five benchmark configurations, at sizes the oracle finishes in well under a second
# ----------------------------------------------------------------------------------------------------------------------
def c1_shift_expm1_log1p(rng, n=1 << 14):
    x = uniform(rng, -0.9, 0.9, n)
    return [log1p(expm1(shift_cyclic(x)))[0]]


def c1_shift_only(rng, n=1 << 14):
    x = uniform(rng, -0.9, 0.9, n)
    return [shift_cyclic(x)[0]]


def c2_chain(rng, shape=(96, 256)):
    a = uniform(rng, -1, 1, shape)
    b = uniform(rng, -1, 1, shape)
    s = np.array([1.0001], np.float32)
    return [chain8(a, b, s)[-1][0]]


def c2_chain_odd(rng):
    """The chain on a last dimension that leaves one element per thread, with more than 4096 workgroups' worth of
    elements: the kernel then strides over the tensor with the math tables copied once per workgroup."""
    return c2_chain(rng, shape=(1025, 1027))


def c2_chain_stages(rng, shape=(96, 256)):
    a = uniform(rng, -1, 1, shape)
    b = uniform(rng, -1, 1, shape)
    s = np.array([1.0001], np.float32)
    return [t[0] for t in chain8(a, b, s)]


def special_values(rng, shape):
    """Random float32 data in which every 7th element is a special value: NaN, infinities, zeros, the largest and
    smallest magnitudes, subnormals, values around the thresholds of exp / log / tanh."""
    specials = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 3.4028235e38, -3.4028235e38, 1.1754944e-38, 1e-45,
                         -1e-45, 88.0, -88.0, 87.3, -87.4, 103.9, -104.0, 22.0, -22.0, 1.0, -1.0, 0.5, 1e-8, -1e-8,
                         1e20, -1e20, 2.0 ** 126, 2.0 ** -126], dtype=np.float32)
    x = rng.standard_normal(shape, dtype=np.float32).ravel()
    x[::7] = specials[np.arange(x[::7].size) % specials.size]
    return x.reshape(shape)


def c2_chain_special(rng, shape=(64, 256)):
    """The 8-op chain on inputs full of special values: what the value-range pruning must leave untouched."""
    a = special_values(rng, shape)
    b = np.roll(special_values(rng, shape), 3)
    s = np.array([1.0001], np.float32)
    return [chain8(a, b, s)[-1][0]]


@ovl.operator()
def _bounded_mix(x):
    """Expressions whose operand ranges are known: exp / log / quotients of bounded activations, a variable that is
    assigned in branches, comparisons that the ranges decide and comparisons that they do not."""
    pos = ovl.position_in(x.shape)
    out0 = ovl.output_like(x)
    out1 = ovl.output_like(x)
    t = ovl.tanh(x[pos])
    s = 1.0 / (1.0 + ovl.exp(-t))
    v = ovl.variable(0.25, x.dtype)
    with ovl.if_(t > 0.5):
        v <<= 3.0
    with ovl.elif_(x[pos] < -2.0):
        v <<= ovl.exp(t) * 2.0
    w = ovl.variable(0.0, x.dtype)
    with ovl.if_(s > 2.0):                      # never
        w <<= 1.0e30
    with ovl.elif_(t >= -1.0):                  # unless t is NaN
        w <<= ovl.log(s + 1.0)
    with ovl.else_():
        w <<= -7.0
    out0[pos] = ovl.exp(v) / (s * (t - 2.0)) + ovl.log(v) * w
    out1[pos] = (t * t + 0.125) / (ovl.exp(t * 3.0) + s) - ovl.sqrt(s) / (t + 1.5)
    return out0, out1


def bounded_mix(rng, shape=(32, 256)):
    return all_outputs(_bounded_mix(special_values(rng, shape)))


def graph_capture_dag(x, y):
    """Several kernels even at opt_level 3: a scan between element-wise stages, two requested outputs."""
    stage = stdops.tanh(stdops.add(x, y))
    scanned = cumsum(stage, axis=1)
    return [log1p(expm1(stdops.mul(scanned, y)))[0], stdops.sub(scanned, x)[0]]


def graph_capture_single(x):
    return [log1p(expm1(shift_cyclic(x)))[0]]


def c3_cumsum_f32(rng, shape=(48, 1024)):
    return [cumsum(rng.standard_normal(shape, dtype=np.float32), axis=1)[0]]


def c3_cumprod_f32(rng, shape=(48, 1024)):
    return [cumprod(uniform(rng, 0.99, 1.01, shape), axis=1)[0]]


def c3_cumsum_f64(rng, shape=(24, 1024)):
    return [cumsum(rng.standard_normal(shape), axis=1)[0]]


def c3_cumprod_f64(rng, shape=(24, 1024)):
    return [cumprod(uniform(rng, 0.99, 1.01, shape, np.float64), axis=1)[0]]


def c3_rowscan_shapes(rng):
    """Row-scan template corner cases: partial last workgroup, several rows per workgroup, rank 3, int32, max, rows that
    end in a shorter burst."""
    outs = [cumsum(rng.standard_normal((515, 64), dtype=np.float32), axis=1)[0],
            cumprod(uniform(rng, 0.9, 1.1, (259, 128), np.float64), axis=1)[0],
            cumsum(rng.standard_normal((4, 70, 128), dtype=np.float32), axis=2)[0],
            cumsum(rng.integers(-1000, 1000, size=(20, 192)).astype(np.int32), axis=1)[0],
            accumulate(rng.standard_normal((7, 256), dtype=np.float32),
                       inner_fcn=lambda acc, x: ovl.maximum(acc, x), axis=1)[0],
            cumsum(rng.standard_normal(4096, dtype=np.float32))[0],
            # rows whose number of groups is not a multiple of the request burst end in a shorter burst
            cumsum(rng.standard_normal((9, 320), dtype=np.float32), axis=1)[0],
            cumprod(uniform(rng, 0.9, 1.1, (5, 448), np.float32), axis=1)[0],
            cumsum(rng.standard_normal((6, 320)), axis=1)[0],
            # rows that are not a whole number of groups, and rows that do not start on 16-byte boundaries: the columns
            # after the last whole group are scanned by one lane, the vectors are moved unaligned
            cumsum(rng.standard_normal((7, 100), dtype=np.float32), axis=1)[0],
            cumsum(rng.standard_normal((5, 1000)), axis=1)[0],
            cumprod(uniform(rng, 0.9, 1.1, (9, 333), np.float32), axis=1)[0],
            cumsum(rng.standard_normal((4, 131)), axis=1)[0],
            cumsum(rng.integers(-1000, 1000, size=(6, 70)).astype(np.int32), axis=1)[0],
            accumulate(rng.standard_normal((3, 2, 203), dtype=np.float32),
                       inner_fcn=lambda acc, x: ovl.maximum(acc, x), axis=2)[0]]
    return outs


def carry_scans(rng):
    """Row scans of 8-byte elements (and, forced, 4-byte ones) whose rows are whole chunks of the LDS-fed variant that
    keeps no results in its scanning wavefront: one to nine chunks per row (the six LDS buffers come round again),
    partial last workgroup, rank 3, sums, products, extrema, integers."""
    return [cumsum(rng.standard_normal((9, 1536)), axis=1)[0],
            cumprod(uniform(rng, 0.9, 1.1, (4, 4096), np.float64), axis=1)[0],
            cumsum(rng.standard_normal((2, 3, 512)), axis=2)[0],
            cumsum(rng.integers(-2 ** 40, 2 ** 40, size=(6, 1024)).astype(np.int64), axis=1)[0],
            accumulate(rng.standard_normal((3, 3584)), inner_fcn=lambda acc, x: ovl.maximum(acc, x), axis=1)[0],
            cumsum(rng.standard_normal((5, 768)), axis=1)[0],
            cumsum(rng.standard_normal((5, 4608), dtype=np.float32), axis=1)[0],
            cumsum(rng.standard_normal((1, 2048)), axis=1)[0]]


def c3_colscan_shapes(rng):
    """Scans along an axis other than the last: partial strips, a partial last chunk of rows, dimensions before the
    axis, 4- and 8-byte elements, a single short chunk, more chunks than register sets with and without a remainder."""
    return [cumsum(rng.standard_normal((200, 100)), axis=0)[0],
            cumsum(rng.standard_normal((700, 30)), axis=0)[0],
            cumsum(rng.standard_normal((1100, 20), dtype=np.float32), axis=0)[0],
            cumprod(uniform(rng, 0.9, 1.1, (130, 70), np.float32), axis=0)[0],
            cumsum(rng.standard_normal((3, 65, 40), dtype=np.float32), axis=1)[0],
            cumsum(rng.integers(-1000, 1000, size=(64, 5)).astype(np.int32), axis=0)[0],
            accumulate(rng.standard_normal((2, 3, 129, 7)), inner_fcn=lambda acc, x: ovl.maximum(acc, x), axis=2)[0],
            cumsum(rng.standard_normal((10, 33)), axis=0)[0]]


def c3_colscan_placements(rng):
    """Scans along the first axis with sixteen strips and more, where strips are placed by XCD: a row pitch that is
    not a multiple of 128 bytes (one contiguous range of strips per XCD), pitches that are (groups of two and of four
    strips that share every line, with left-over strips), and a dimension before the axis."""
    return [cumsum(rng.standard_normal((300, 200)), axis=0)[0],
            # (long axes: the movers' loop over whole chunks runs, with 2 and with 3 chunks of loads in flight; 8-byte
            # integers wrap around like the oracle's; exactly 4 and 5 chunks of 256 rows)
            cumsum(rng.standard_normal((3400, 9)), axis=0)[0],
            cumsum(rng.integers(-2 ** 62, 2 ** 62, size=(3700, 5)), axis=0)[0],
            cumprod(uniform(rng, 0.99, 1.01, (1024, 12), np.float64), axis=0)[0],
            cumsum(rng.standard_normal((1280, 3)), axis=0)[0],
            cumsum(rng.standard_normal((300, 160)), axis=0)[0],
            cumsum(rng.standard_normal((280, 288), dtype=np.float32), axis=0)[0],
            cumsum(rng.standard_normal((2, 270, 72)), axis=1)[0]]


@ovl.operator()
def _swap_last_two(x, scale=None):
    """A batched transpose with some arithmetic and a second, untransposed output: the dimensions before the last two
    of the workgroup are batches of the tile template."""
    shape = list(x.shape)
    swapped = ovl.output(shape[:-2] + [shape[-1], shape[-2]], x.dtype)
    plain = ovl.output_like(x)
    pos = ovl.position_in(x.shape)
    value = x[pos] * scale
    swapped[tuple(pos[k] for k in range(len(shape) - 2)) + (pos[len(shape) - 1], pos[len(shape) - 2])] = value
    plain[pos] = value + 1
    return swapped, plain


@ovl.operator()
def _move_axis_last(x, axis=None, bias=None):
    """out[.., rest.., x.shape[axis]]: the given axis becomes the last one, the others keep their order ([N, C, H, W]
    with axis 1 gives [N, H, W, C]).  The store has unit stride along a workgroup dimension that is neither the last nor
    the one before it, which the tile template takes as its second dimension."""
    shape = list(x.shape)
    order = [k for k in range(len(shape)) if k != axis] + [axis]
    moved = ovl.output([shape[k] for k in order], x.dtype)
    pos = ovl.position_in(x.shape)
    moved[tuple(pos[k] for k in order)] = x[pos] + bias
    return moved


def batched_transposes(rng):
    return (all_outputs(_swap_last_two(rng.standard_normal((3, 70, 100), dtype=np.float32), scale=0.5)) +
            all_outputs(_swap_last_two(rng.standard_normal((2, 3, 66, 34)), scale=2.0)) +
            all_outputs(_swap_last_two(rng.integers(-100, 100, size=(5, 33, 35)).astype(np.int32), scale=3)))


def moved_axes(rng):
    return (all_outputs(_move_axis_last(rng.standard_normal((2, 24, 5, 36), dtype=np.float32), axis=1, bias=1.0)) +
            all_outputs(_move_axis_last(rng.standard_normal((3, 9, 4, 3, 10)), axis=1, bias=0.5)) +
            all_outputs(_move_axis_last(rng.standard_normal((40, 3, 33), dtype=np.float32), axis=0, bias=2.0)) +
            all_outputs(_move_axis_last(rng.integers(-9, 9, size=(2, 3, 7, 64)).astype(np.int32), axis=1, bias=1)))


def c4_lstm(rng, batch=32, units=128):
    concat = rng.standard_normal((batch, 4 * units), dtype=np.float32)
    c = rng.standard_normal((batch, units), dtype=np.float32)
    return all_outputs(lstm(concat, c, forget_bias=1.0))


def c4_lstm_grad(rng, batch=32, units=128):
    concat = rng.standard_normal((batch, 4 * units), dtype=np.float32)
    c = rng.standard_normal((batch, units), dtype=np.float32)
    dc = rng.standard_normal((batch, units), dtype=np.float32)
    dh = rng.standard_normal((batch, units), dtype=np.float32)
    return all_outputs(lstm_grad(concat, c, dc, dh, forget_bias=1.0))


def c5_gather_transpose(rng, shape=(192, 320), stride=7919, dtype=np.float32):
    a = rng.standard_normal(shape, dtype=dtype)
    b = rng.standard_normal(shape, dtype=dtype)
    return [gather_transpose(a, b.reshape(-1), alpha=0.5, stride=stride)[0]]


def c5_variants(rng):
    """Gather index that provably never wraps (dword-aligned vector loads), ragged tile edges, float64 tiles."""
    return (c5_gather_transpose(rng, (192, 320), stride=3) + c5_gather_transpose(rng, (68, 100), stride=5) +
            c5_gather_transpose(rng, (130, 66), stride=7, dtype=np.float64) +
            c5_gather_transpose(rng, (6, 10), stride=1) +
            # extents that leave two elements, or one, per access
            c5_gather_transpose(rng, (70, 102), stride=11) + c5_gather_transpose(rng, (67, 101), stride=3) +
            c5_gather_transpose(rng, (35, 129), stride=2, dtype=np.float64) +
            # (75 tiles along j once the tiles are forced down to 8 x 8)
            c5_gather_transpose(rng, (24, 600), stride=13))


# ----------------------------------------------------------------------------------------------------------------------
# scalar math coverage (the reference's test_unary_math.py / test_binary_math.py inputs)
# ----------------------------------------------------------------------------------------------------------------------
def _unary_op(fcn):
    @ovl.operator()
    def unary(input0):
        out = ovl.output_like(input0)
        pos = ovl.position_in(input0.shape)
        out[pos] = fcn(input0[pos])
        return out
    return unary


def _binary_op(fcn):
    @ovl.operator()
    def binary_math(op_input0, op_input1):
        out = ovl.output_like(op_input0)
        pos = ovl.position_in(op_input0.shape)
        out[pos] = fcn(op_input0[pos], op_input1[pos])
        return out
    return binary_math


UNARY_FLOAT = [
    ('arccos', ovl.arccos, np.arccos, 'one'), ('arcsin', ovl.arcsin, np.arcsin, 'one'),
    ('arctan', ovl.arctan, np.arctan, 'atan'), ('cos', ovl.cos, np.cos, 'any'), ('cosh', ovl.cosh, np.cosh, 'any'),
    ('sin', ovl.sin, np.sin, 'any'), ('sinh', ovl.sinh, np.sinh, 'any'), ('tan', ovl.tan, np.tan, 'any'),
    ('tanh', ovl.tanh, np.tanh, 'any'), ('exp', ovl.exp, np.exp, 'any'), ('log', ovl.log, np.log, 'pos'),
    ('log10', ovl.log10, np.log10, 'pos'), ('sqrt', ovl.sqrt, np.sqrt, 'pos'), ('ceil', ovl.ceil, np.ceil, 'any'),
    ('floor', ovl.floor, np.floor, 'any'), ('absolute', ovl.absolute, np.absolute, 'any'),
    ('negate', lambda x: -x, lambda x: -x, 'any')]

#: float32 functions whose device implementation reproduces the host C library bit for bit
EXACT_F32 = ('tanh', 'exp', 'log', 'sqrt', 'ceil', 'floor', 'absolute', 'negate')


def unary_input(kind, dtype, length=100):
    """Inputs of the reference's unary tests (test_unary_math.py:113-117): RandomState(1), 100 elements."""
    rng = np.random.RandomState(1)
    rand = rng.uniform(-10, 10, length).astype(dtype)
    rand_pos = np.abs(rand) + np.finfo(dtype).eps
    rand_one = rng.uniform(-1.0 + np.finfo(dtype).eps, 1 - np.finfo(dtype).eps, length).astype(dtype)
    return {'any': rand, 'pos': rand_pos, 'one': rand_one, 'atan': (3.14 / 2 * rand_one).astype(dtype)}[kind]


def _unary_case(name, fcn, kind, dtype):
    def build(rng):
        return [_unary_op(fcn)(unary_input(kind, dtype))[0]]
    exact = dtype == np.float32 and name in EXACT_F32 or name in ('sqrt', 'ceil', 'floor', 'absolute', 'negate')
    return Case('unary_%s_%s' % (name, np.dtype(dtype).name), build,
                max_ulp=0 if exact else 2, rel=0 if exact else 1e-12)


BINARY_ALL = [
    ('add', lambda a, b: a + b), ('sub', lambda a, b: a - b), ('mul', lambda a, b: a * b),
    ('div', lambda a, b: a / b), ('mod', lambda a, b: a % b),
    ('eq', lambda a, b: a == b), ('ne', lambda a, b: a != b),
    ('or', lambda a, b: ovl.logical_or(a, b)), ('and', lambda a, b: ovl.logical_and(a, b)),
    ('lt', lambda a, b: a < b), ('le', lambda a, b: a <= b), ('gt', lambda a, b: a > b), ('ge', lambda a, b: a >= b),
    ('min', lambda a, b: ovl.minimum(a, b)), ('max', lambda a, b: ovl.maximum(a, b))]
BINARY_FLOAT = [('pow', lambda a, b: ovl.power(a, b)), ('atan2', lambda a, b: ovl.arctan2(a, b))]

ALL_DTYPES = [np.float32, np.float64, np.int8, np.int16, np.int32, np.int64,
              np.uint8, np.uint16, np.uint32, np.uint64]


def binary_inputs(name, dtype, length=10):
    """Inputs of the reference's binary tests (test_binary_math.py:57-72): RandomState(1), 10 elements."""
    rng = np.random.RandomState(1)

    def cast(arg):
        if np.dtype(dtype).kind == 'u':
            return np.abs(arg).astype(dtype)
        return arg.astype(dtype)

    x = cast(rng.uniform(-10, 10, length))
    y = cast(rng.uniform(-10, 10, length))
    y_nonzero = (y + np.equal(y, 0)).astype(dtype)
    x_binary = cast(rng.uniform(0, 1, length) > 0.5)
    y_binary = cast(rng.uniform(0, 1, length) > 0.5)
    if name in ('div', 'mod'):
        return x, y_nonzero
    if name in ('eq', 'ne', 'or', 'and'):
        return x_binary, y_binary
    if name == 'pow':
        return np.abs(x), y
    return x, y


def _binary_case(name, fcn, dtype):
    def build(rng):
        a, b = binary_inputs(name, dtype)
        return [_binary_op(fcn)(a, b)[0]]
    approx = name in ('pow', 'atan2')
    return Case('binary_%s_%s' % (name, np.dtype(dtype).name), build,
                max_ulp=2 if approx else 0, rel=1e-12 if approx else 0)


# ----------------------------------------------------------------------------------------------------------------------
# control flow, indexing and multi-output operators from the reference's tests
# ----------------------------------------------------------------------------------------------------------------------
@ovl.operator()
def clip(arg, threshold1=None, threshold2=None):
    pos = ovl.position_in(arg.shape)
    clipped = ovl.output_like(arg)
    x = arg[pos]
    with ovl.if_(x < threshold1):
        clipped[pos] = threshold1
    with ovl.elif_(x > threshold2):
        clipped[pos] = threshold2
    with ovl.else_():
        clipped[pos] = x
    return clipped


@ovl.operator()
def set_limits(arg):
    pos = ovl.position_in(arg.shape)
    limits = ovl.output([arg.shape[0], 3], arg.dtype)
    t = arg.dtype
    limits[pos, 0] = ovl.min_value(t)
    limits[pos, 1] = ovl.max_value(t)
    limits[pos, 2] = ovl.epsilon(t)
    return limits


@ovl.operator()
def fill_range(input0):
    assert len(input0.shape) == 1
    ovl.position_in([1])
    num_elements = input0.shape[0]
    out_right = ovl.output(input0.shape, input0.dtype)
    out_left = ovl.output(input0.shape, input0.dtype)
    for i in ovl.arange(num_elements):
        out_right[i] = input0[i] * ovl.cast(i, input0.dtype)
    for i in ovl.arange(num_elements - 1, -1, -1):
        out_left[i] = input0[i] * ovl.cast(i, input0.dtype)
    return out_right, out_left


@ovl.operator()
def dot(input0, input1):
    num_vectors = input0.shape[0]
    dot_out = ovl.output(num_vectors, input0.dtype)
    pos = ovl.position_in(num_vectors)[0]
    accum = ovl.variable(0.0, ovl.float64)
    num_elements = ovl.variable(input0.shape[1], ovl.uint32)
    for i in ovl.arange(num_elements):
        accum <<= accum + input0[pos, i] * input1[pos, i]
    dot_out[pos] = accum
    return dot_out


@ovl.operator()
def _row_dot(a, b):
    """A dot product per row, accumulated in float64, with a statement after the loop."""
    shape = list(a.shape)
    out = ovl.output(shape[:-1], ovl.float64)
    pos = ovl.position_in(shape[:-1])
    acc = ovl.variable(0.0, ovl.float64)
    for j in ovl.arange(shape[-1]):
        index = tuple(pos[k] for k in range(len(shape) - 1)) + (j,)
        acc <<= acc + ovl.cast(a[index] * b[index], ovl.float64)
    out[pos] = acc * 0.5
    return out


@ovl.operator()
def _row_norm_and_max(x):
    """Two carried states and two outputs: the square root of the sum of squares and the running maximum, which
    starts from column 0 (the loop starts at 1)."""
    rows, cols = x.shape
    norm = ovl.output([rows], x.dtype)
    largest = ovl.output([rows], x.dtype)
    pos = ovl.position_in([rows])[0]
    first = x[pos, 0]
    total = ovl.variable(first * first, x.dtype)
    top = ovl.variable(first, x.dtype)
    for j in ovl.arange(1, cols):
        v = x[pos, j]
        total <<= total + v * v
        top <<= ovl.maximum(top, v)
    norm[pos] = ovl.sqrt(total)
    largest[pos] = top
    return norm, largest


@ovl.operator()
def _row_int_sum(x):
    rows, cols = x.shape
    out = ovl.output([rows], x.dtype)
    pos = ovl.position_in([rows])[0]
    acc = ovl.variable(0, x.dtype)
    for j in ovl.arange(cols):
        acc <<= acc + x[pos, j]
    out[pos] = acc
    return out


@ovl.operator()
def _matrix_vector(m, v, first=None, count=None):
    """y[.., r] = sum over columns first .. first+count-1 of m[.., r, c] * v[c - first]: every worker walks a slice
    of its own matrix row and the one vector all workers share."""
    shape = list(m.shape)
    out = ovl.output(shape[:-1], m.dtype)
    pos = ovl.position_in(shape[:-1])
    acc = ovl.variable(0, m.dtype)
    for j in ovl.arange(count):
        index = tuple(pos[k] for k in range(len(shape) - 1)) + (j + first,)
        acc <<= acc + m[index] * v[j]
    out[pos] = acc
    return out


@ovl.operator()
def _two_offsets(x):
    """One tensor read at two offsets in the loop (a row's lag-1 products): not the row reduction's shape."""
    rows, cols = x.shape
    out = ovl.output([rows], x.dtype)
    pos = ovl.position_in([rows])[0]
    acc = ovl.variable(0, x.dtype)
    for j in ovl.arange(cols - 1):
        acc <<= acc + x[pos, j] * x[pos, j + 1]
    out[pos] = acc
    return out


def _gated_body(a, x, b):
    shape = list(x.shape)
    out = ovl.output_like(x)
    pos = ovl.position_in(shape[:-1])

    def at(i):
        return tuple(pos[k] for k in range(len(shape) - 1)) + (i,)

    h = ovl.variable(x[at(0)], x.dtype)
    out[at(0)] = h
    for i in ovl.arange(1, shape[-1]):
        if b is None:
            h <<= a[at(i)] * h + x[at(i)]
        else:
            h <<= a[at(i)] * h + x[at(i)] * b[at(i)]
        out[at(i)] = h
    return out


@ovl.operator()
def _gated_scan(a, x):
    """A gated linear recurrence along the last axis, h = a[.., i] * h + x[.., i]: a row scan whose body reads two
    inputs of the output's shape."""
    return _gated_body(a, x, None)


@ovl.operator()
def _gated_scan3(a, x, b):
    """h = a[.., i] * h + x[.., i] * b[.., i]: three inputs."""
    return _gated_body(a, x, b)


@ovl.operator()
def _cell_scan(f, i, g, o):
    """An LSTM-like recurrence over the last axis with its matrix products taken out: c = f * c + i * g and
    h = o * tanh(c), both stored for every column.  Four inputs, two outputs, one carried variable."""
    shape = list(f.shape)
    cs = ovl.output_like(f)
    hs = ovl.output_like(f)
    pos = ovl.position_in(shape[:-1])

    def at(k):
        return tuple(pos[d] for d in range(len(shape) - 1)) + (k,)

    c = ovl.variable(i[at(0)] * g[at(0)], f.dtype)
    cs[at(0)] = c
    hs[at(0)] = o[at(0)] * ovl.tanh(c)
    for k in ovl.arange(1, shape[-1]):
        c <<= f[at(k)] * c + i[at(k)] * g[at(k)]
        cs[at(k)] = c
        hs[at(k)] = o[at(k)] * ovl.tanh(c)
    return cs, hs


@ovl.operator()
def _sum_and_max(x):
    """Running sum and running maximum of every row: two carried variables, two outputs."""
    rows, cols = x.shape
    sums = ovl.output_like(x)
    tops = ovl.output_like(x)
    r = ovl.position_in([rows])[0]
    total = ovl.variable(x[r, 0], x.dtype)
    top = ovl.variable(x[r, 0], x.dtype)
    sums[r, 0] = total
    tops[r, 0] = top
    for k in ovl.arange(1, cols):
        total <<= total + x[r, k]
        top <<= ovl.maximum(top, x[r, k])
        sums[r, k] = total
        tops[r, k] = top
    return sums, tops


def gated_scans(rng):
    """Row scans over several inputs: whole groups, columns left over, unaligned rows, rank 3, 8-byte elements, a row
    shorter than one group (which stays on the general kernel)."""
    def gate(shape, dtype):
        return rng.uniform(0.5, 1.0, shape).astype(dtype)

    def data(shape, dtype):
        return rng.standard_normal(shape).astype(dtype)
    outs = []
    for shape, dtype, three in [((7, 256), np.float32, False), ((5, 333), np.float32, True), ((3, 131), np.float32, False),
                                ((2, 3, 200), np.float64, True), ((9, 1024), np.float64, False),
                                ((4, 40), np.float32, False), ((67, 640), np.float32, True)]:
        if three:
            outs.append(_gated_scan3(gate(shape, dtype), data(shape, dtype), data(shape, dtype)))
        else:
            outs.append(_gated_scan(gate(shape, dtype), data(shape, dtype)))
    # several outputs
    for shape, dtype in [((6, 256), np.float32), ((2, 3, 333), np.float32), ((5, 131), np.float32)]:
        outs += all_outputs(_cell_scan(gate(shape, dtype), data(shape, dtype), data(shape, dtype), gate(shape, dtype)))
    outs += all_outputs(_sum_and_max(data((9, 517), np.float32)))
    outs += all_outputs(_sum_and_max(data((4, 200), np.float64)))
    outs += all_outputs(_sum_and_max(rng.integers(-50, 50, size=(7, 320)).astype(np.int32)))
    return outs


def row_reductions(rng):
    """Reductions along the last axis: rows of whole groups, rows with columns left over, rows that are not 16-byte
    aligned, a rank-3 tensor, 4- and 8-byte elements, integers."""
    a = rng.standard_normal((7, 256), dtype=np.float32)
    b = rng.standard_normal((7, 256), dtype=np.float32)
    c = rng.standard_normal((5, 333), dtype=np.float32)
    d = rng.standard_normal((5, 333), dtype=np.float32)
    e = rng.standard_normal((2, 3, 200))
    f = rng.standard_normal((2, 3, 200))
    # (the reference's own dot product keeps its loop bound in a variable that nothing writes)
    return ([_row_dot(a, b), _row_dot(c, d), _row_dot(e, f), dot(rng.standard_normal((9, 300)), rng.standard_normal((9, 300)))] +
            all_outputs(_row_norm_and_max(rng.standard_normal((9, 131)))) + all_outputs(_row_norm_and_max(rng.standard_normal((9, 80)))) +
            all_outputs(_row_norm_and_max(rng.standard_normal((70, 1000), dtype=np.float32))) +
            [_row_int_sum(rng.integers(-50, 50, size=(6, 270)).astype(np.int32)),
             # matrix times vector: whole rows, a slice that leaves the rows' vectors unaligned, rank 3
             _matrix_vector(rng.standard_normal((9, 320), dtype=np.float32),
                            rng.standard_normal(320, dtype=np.float32), first=0, count=320),
             _matrix_vector(rng.standard_normal((5, 400)), rng.standard_normal(300), first=37, count=300),
             _matrix_vector(rng.standard_normal((2, 3, 301), dtype=np.float32),
                            rng.standard_normal(301, dtype=np.float32), first=0, count=301),
             _two_offsets(rng.standard_normal((6, 300), dtype=np.float32))])


@ovl.operator()
def _axis_mean_and_max(x, axis=None):
    """Reductions along an axis that is not the last: the mean (a statement after the loop) and the maximum, which
    starts from the first element (the loop starts at 1)."""
    shape = list(x.shape)
    rest = shape[:axis] + shape[axis + 1:]
    mean = ovl.output(rest, x.dtype)
    largest = ovl.output(rest, x.dtype)
    pos = ovl.position_in(rest)

    def at(i):
        return tuple(pos[k] for k in range(axis)) + (i,) + tuple(pos[k] for k in range(axis, len(rest)))
    first = x[at(0)]
    total = ovl.variable(first, x.dtype)
    top = ovl.variable(first, x.dtype)
    for i in ovl.arange(1, shape[axis]):
        v = x[at(i)]
        total <<= total + v
        top <<= ovl.maximum(top, v)
    mean[pos] = total / shape[axis]
    largest[pos] = top
    return mean, largest


@ovl.operator()
def _column_sum(x):
    rows, cols = x.shape
    out = ovl.output([cols], x.dtype)
    pos = ovl.position_in([cols])[0]
    acc = ovl.variable(0, x.dtype)
    for i in ovl.arange(rows):
        acc <<= acc + x[i, pos]
    out[pos] = acc
    return out


def col_reductions(rng):
    """Reductions along an axis other than the last: partial strips, a partial last chunk of rows, dimensions before
    the axis, 4- and 8-byte elements, integers, a loop from 0 and a loop from 1, a long axis."""
    return (all_outputs(_axis_mean_and_max(rng.standard_normal((200, 100)), axis=0)) +
            all_outputs(_axis_mean_and_max(rng.standard_normal((130, 70), dtype=np.float32), axis=0)) +
            all_outputs(_axis_mean_and_max(rng.standard_normal((3, 65, 40), dtype=np.float32), axis=1)) +
            [_column_sum(rng.standard_normal((700, 30))),
             _column_sum(rng.integers(-1000, 1000, size=(64, 5)).astype(np.int32)),
             _column_sum(rng.standard_normal((1100, 20), dtype=np.float32)),
             # (a long axis: the steps of the last, partial chunk alone test their rows against its end)
             _column_sum(rng.standard_normal((8200, 11)))])


@ovl.operator()
def multi_op(input0, input1, input2):
    pos = ovl.position_in(input0.shape)
    output0 = ovl.output_like(input0)
    output1 = ovl.output_like(input0)
    output2 = ovl.output_like(input0)
    a = input0[pos]
    b = input1[pos]
    c = input2[pos]
    d = a + b
    output0[pos] = d
    output1[pos] = d * c
    output2[pos] = d + c
    return output0, output1, output2


@ovl.operator()
def reorder(input0):
    pos = ovl.position_in(input0.shape)
    output3 = ovl.output_like(input0)
    output0 = ovl.output_like(input0)
    output2 = ovl.output_like(input0)
    output1 = ovl.output_like(input0)
    inp = input0[pos]
    output0[pos] = 2 * inp
    output1[pos] = 3 * inp
    output2[pos] = 4 * inp
    output3[pos] = 5 * inp
    return output0, output1, output2, output3


@ovl.operator()
def pad(in0, n=None):
    rows_in, cols_in = in0.shape
    rows = rows_in + 2 * n
    cols = cols_in + 2 * n
    out = ovl.output([rows, cols], in0.dtype)
    pos = ovl.position_in([rows, cols])
    i_row = pos[0]
    i_col = pos[1]
    row_in = ovl.variable(i_row, dtype=pos.dtype)
    col_in = ovl.variable(i_col, dtype=pos.dtype)
    with ovl.if_(row_in < n):
        row_in <<= 0
    with ovl.elif_(row_in >= (rows_in + n)):
        row_in <<= rows_in - 1
    with ovl.else_():
        row_in <<= row_in - n
    with ovl.if_(col_in < n):
        col_in <<= 0
    with ovl.elif_(col_in >= (cols_in + n)):
        col_in <<= cols_in - 1
    with ovl.else_():
        col_in <<= col_in - n
    out[i_row, i_col] = in0[row_in, col_in]
    return out


@ovl.operator()
def crop(in0, n=None):
    rows = in0.shape[0] - 2 * n
    cols = in0.shape[1] - 2 * n
    pos = ovl.position_in([rows, cols])
    i_row = pos[0]
    i_col = pos[1]
    out = ovl.output([rows, cols], in0.dtype)
    out[i_row, i_col] = in0[n + i_row, n + i_col]
    return out


@ovl.operator()
def local_window_sum(x, width=None):
    """Worker-local tensor: gather ``width`` neighbours into a local array, then sum it back to front."""
    n = x.shape[0]
    out = ovl.output_like(x)
    pos = ovl.position_in(n)[0]
    window = ovl.zeros(width, x.dtype)
    for k in ovl.arange(width):
        window[k] = x[(pos + ovl.cast(k, ovl.uint32)) % n]
    acc = ovl.variable(0, x.dtype)
    for k in ovl.arange(width - 1, -1, -1):
        acc <<= acc + window[k]
    out[pos] = acc
    return out


def _simple(name, fcn, max_ulp=0, rel=0.0):
    return Case(name, fcn, max_ulp=max_ulp, rel=rel)


def _stdops_lstm(rng):
    batches, vec_len = 4, 24
    concat_arg = rng.standard_normal((batches, 4 * vec_len), dtype=np.float32)
    c = rng.standard_normal((batches, vec_len), dtype=np.float32)
    i, j, f, o = all_outputs(stdops.split(concat_arg, split_dim=1, num_split=4))
    new_c = stdops.mul(c, stdops.sigmoid(f)) + stdops.sigmoid(i) * stdops.tanh(j)
    new_h = stdops.tanh(new_c) * stdops.sigmoid(o)
    return [new_c[0], new_h[0]]


def _broadcast(rng):
    a = rng.standard_normal((6, 20), dtype=np.float32)
    s = np.array([[2.5]], np.float32)
    return [stdops.mul(a, s)[0], stdops.sub(s, a)[0], stdops.div(a, s)[0], stdops.mod(a, s)[0],
            stdops.less(a, s)[0], stdops.equal(a, a)[0]]


def _concat_ragged(rng):
    a = rng.standard_normal((3, 4))
    b = rng.standard_normal((3, 7))
    c = rng.standard_normal((3, 1))
    return [stdops.concat(a, b, c, concat_dim=1)[0]]


def _split_concat(rng):
    a = rng.standard_normal((8, 12), dtype=np.float32)
    parts = all_outputs(stdops.split(a, split_dim=1, num_split=3))
    return [stdops.concat(parts[2], parts[0], parts[1], concat_dim=0)[0]]


def _int_accumulate(rng):
    b = np.arange(1, 16).reshape(3, 5)
    return [cumsum(b, axis=0)[0], cumprod(b, axis=0)[0], cumsum(np.arange(1, 6))[0]]


def _accumulate_axes(rng):
    a = rng.random((5, 6, 7))
    outs = []
    for axis in range(3):
        outs.append(cumsum(a, axis=axis)[0])
        outs.append(cumprod(a, axis=axis)[0])
    return outs


def _int_tree_scans(rng):
    """Integer sums, products, minima and maxima over rows long enough for the tree-shaped scan, values that wrap."""
    outs = []
    for dtype in (np.int32, np.int64, np.uint32, np.uint64):
        info = np.iinfo(dtype)
        big = rng.integers(info.min // 2, info.max // 2, (6, 2048), dtype=dtype)      # sums wrap around
        small = rng.integers(0 if info.min == 0 else -3, 4, (5, 4096)).astype(dtype)
        outs.append(cumsum(big, axis=1)[0])
        outs.append(cumprod(small | dtype(1), axis=1)[0])                              # odd factors: products wrap
        outs.append(accumulate(big, inner_fcn=lambda acc, x: ovl.maximum(acc, x), axis=1)[0])
        outs.append(accumulate(big, inner_fcn=lambda acc, x: ovl.minimum(x, acc), axis=1)[0])
    # rows that end inside a step of 256 vectors
    outs.append(cumsum(rng.integers(-1000, 1000, (3, 1088)).astype(np.int32), axis=1)[0])
    outs.append(cumsum(rng.integers(-1000, 1000, (2, 2112)).astype(np.int64), axis=1)[0])
    return outs


def _accumulate_max(rng):
    a = rng.standard_normal((9, 130), dtype=np.float32)
    return [accumulate(a, inner_fcn=lambda acc, x: ovl.maximum(acc, x), axis=1)[0]]


def _edge_expm1_log1p(rng):
    a = np.array([1e-10, -1e-10, 0.0, np.inf], dtype=np.float64)
    b = np.array([1e-99, -1e-99, 0.0, np.inf], dtype=np.float64)
    a32 = np.array([1e-10, -1e-10, 0.0, np.inf, -np.inf, 88.0, -104.0, 1e-38, -0.0], dtype=np.float32)
    return [expm1(a)[0], log1p(b)[0], expm1(a32)[0], log1p(np.abs(a32))[0]]


def _conv1d(rng):
    from opveclib_amd.examples.conv1d import conv_1d
    outs = []
    for mode, orientation, taps, dtype in (('same', 'as-is', 5, np.float32), ('valid', 'flipped', 4, np.float32),
                                           ('full', 'as-is', 3, np.float64), ('same', 'flipped', 1, np.float32)):
        x = rng.standard_normal((2, 3, 37)).astype(dtype)
        v = rng.standard_normal((4, 3, taps)).astype(dtype)
        outs.append(conv_1d(x, v, kernel_orientation=orientation, mode=mode)[0])
    x = rng.standard_normal((2, 37, 3))
    v = rng.standard_normal((4, 5, 3))
    outs.append(conv_1d(x, v, mode='same', data_format='NEC')[0])
    return outs


def _triangles(rng):
    from opveclib_amd.examples import graph
    outs = [graph.triangles_op(*graph.adjacency_from_edges(graph.EXAMPLE_EDGES))[0]]
    for vertices, edges in ((40, 300), (300, 4000)):
        outs.append(graph.triangles_op(*graph.adjacency_from_edges(rng.integers(0, vertices, size=(edges, 2))))[0])
    return outs


@ovl.operator()
def scatter_affine(x, a=None, c=None):
    """out[(a * p + c) mod n] = x[p]"""
    n = x.shape[0]
    pos = ovl.position_in(x.shape)
    out = ovl.output_like(x)
    out[(pos[0] * a + c) % n] = x[pos]
    return out


@ovl.operator()
def transpose_scaled(x):
    pos = ovl.position_in(x.shape)
    out = ovl.output([x.shape[1], x.shape[0]], x.dtype)
    out[pos[1], pos[0]] = 2 * x[pos]
    return out


def _adopted_position(rng):
    """Element-wise consumers fused into producers whose store permutes the workgroup."""
    x = uniform(rng, -0.9, 0.9, 1000)
    y = rng.standard_normal(4096, dtype=np.float32)
    w = rng.standard_normal(4096, dtype=np.float32)
    m = rng.standard_normal((96, 160), dtype=np.float32)
    v = rng.standard_normal((160, 96), dtype=np.float32)
    shifted = shift_cyclic(x)
    return [log1p(expm1(shifted))[0], shifted[0],
            stdops.mul(scatter_affine(y, a=3, c=1), w)[0],
            stdops.sub(scatter_affine(y, a=4095, c=7), w)[0],
            stdops.tanh(stdops.neg(transpose_scaled(m)))[0],
            stdops.tanh(stdops.add(transpose_scaled(m), v))[0]]


@ovl.operator()
def store_then_loop_store(x):
    """One element stored at the top level and again, with another value, inside a loop: the last store must win."""
    out = ovl.output_like(x)
    pos = ovl.position_in(x.shape)
    out[pos] = x[pos]
    acc = ovl.variable(0, x.dtype)
    for _ in ovl.arange(3):
        acc <<= acc + x[pos]
        out[pos] = acc
    return out


@ovl.operator()
def scan_late_store(x):
    """A row scan that stores its first column after the loop instead of before it."""
    out = ovl.output_like(x)
    pos = ovl.position_in([x.shape[0]])
    acc = ovl.variable(x[pos[0], 0], x.dtype)
    for i in ovl.arange(1, x.shape[1]):
        acc <<= acc + x[pos[0], i]
        out[pos[0], i] = acc
    out[pos[0], 0] = x[pos[0], 0] * 2
    return out


@ovl.operator()
def scan_two_stores(x):
    """A row scan whose first column is stored twice before the loop."""
    out = ovl.output_like(x)
    pos = ovl.position_in([x.shape[0]])
    acc = ovl.variable(x[pos[0], 0], x.dtype)
    out[pos[0], 0] = acc * 3
    out[pos[0], 0] = acc
    for i in ovl.arange(1, x.shape[1]):
        acc <<= acc + x[pos[0], i]
        out[pos[0], i] = acc
    return out


@ovl.operator()
def diagonal_overwrite(x):
    """Every element stored through the worker's own position, the diagonal stored again through the transposed
    index under a condition: on the diagonal both stores of one worker hit one element, and the second must win."""
    out = ovl.output_like(x)
    pos = ovl.position_in(x.shape)
    out[pos] = x[pos]
    with ovl.if_(pos[0] == pos[1]):
        out[pos[1], pos[0]] = x[pos] * 2
    return out


def _store_order(rng):
    x = rng.standard_normal((64, 256), dtype=np.float32)
    return [store_then_loop_store(rng.standard_normal(1024, dtype=np.float32))[0], scan_late_store(x)[0],
            scan_two_stores(x)[0], diagonal_overwrite(rng.standard_normal((64, 64), dtype=np.float32))[0]]


def _odd_sizes(rng):
    # sizes that are not multiples of the vector width, rank 1 and rank 3
    a = rng.standard_normal(1001, dtype=np.float32)
    b = rng.standard_normal((3, 5, 7), dtype=np.float32)
    return [stdops.tanh(a)[0], stdops.add(b, b)[0], shift_cyclic(a)[0], shift_cyclic(np.array([3.0], np.float32))[0]]


CASES = [
    Case('c1_shift', c1_shift_only),
    Case('c1_shift_expm1_log1p', c1_shift_expm1_log1p),
    Case('c2_chain', c2_chain, seed=2),
    Case('c2_chain_odd', c2_chain_odd, seed=2),
    Case('c2_chain_stages', c2_chain_stages, seed=2),
    Case('c2_chain_special', c2_chain_special, seed=2),
    Case('bounded_mix', bounded_mix, seed=2),
    Case('c3_cumsum_f32', c3_cumsum_f32, seed=3),
    Case('c3_cumprod_f32', c3_cumprod_f32, seed=3),
    Case('c3_cumsum_f64', c3_cumsum_f64, seed=3),
    Case('c3_cumprod_f64', c3_cumprod_f64, seed=3),
    Case('c3_rowscan_shapes', c3_rowscan_shapes, seed=3),
    Case('carry_scans', carry_scans, seed=3),
    Case('c3_colscan_placements', c3_colscan_placements, seed=12),
    Case('c3_colscan_shapes', c3_colscan_shapes, seed=3),
    Case('c4_lstm', c4_lstm, seed=4),
    Case('c4_lstm_grad', c4_lstm_grad, seed=4),
    Case('c5_gather_transpose', c5_gather_transpose, seed=5),
    Case('c5_variants', c5_variants, seed=5),
    Case('batched_transposes', batched_transposes, seed=5),
    Case('moved_axes', moved_axes, seed=6),
    Case('row_reductions', row_reductions, seed=7),
    Case('gated_scans', gated_scans, seed=8),
    Case('col_reductions', col_reductions, seed=8),
    _simple('store_order', _store_order),
    _simple('clip', lambda rng: [clip(rng.random(1000), threshold1=0.1, threshold2=0.9)[0]]),
    _simple('limits_f32', lambda rng: [set_limits(np.array([0], np.float32))[0]]),
    _simple('limits_f64', lambda rng: [set_limits(np.array([0], np.float64))[0]]),
    _simple('arange', lambda rng: all_outputs(fill_range(np.random.RandomState(1).uniform(-1, 1, 10)))),
    _simple('dot', lambda rng: [dot(np.random.RandomState(1).uniform(-1, 1, (100, 10)),
                                    np.random.RandomState(2).uniform(-1, 1, (100, 10)))[0]]),
    _simple('multi_output', lambda rng: all_outputs(multi_op(rng.random(5), rng.random(5), rng.random(5)))),
    _simple('reorder', lambda rng: all_outputs(reorder(rng.random(5)))),
    _simple('pad_crop', lambda rng: [crop(pad(rng.random((3, 5)), n=2), n=2)[0]]),
    _simple('local_tensor', lambda rng: [local_window_sum(rng.standard_normal(37, dtype=np.float32), width=5)[0]]),
    _simple('stdops_lstm', _stdops_lstm),
    _simple('broadcast', _broadcast),
    _simple('concat_ragged', _concat_ragged),
    _simple('split_concat', _split_concat),
    _simple('int_accumulate', _int_accumulate),
    _simple('accumulate_axes', _accumulate_axes),
    _simple('accumulate_max', _accumulate_max),
    _simple('int_tree_scans', _int_tree_scans),
    _simple('edge_expm1_log1p', _edge_expm1_log1p, max_ulp=2, rel=1e-12),
    _simple('odd_sizes', _odd_sizes),
    _simple('adopted_position', _adopted_position),
    _simple('conv1d', _conv1d),
    _simple('triangles', _triangles),
]
for _name, _fcn, _np, _kind in UNARY_FLOAT:
    for _dt in (np.float32, np.float64):
        CASES.append(_unary_case(_name, _fcn, _kind, _dt))
for _name, _fcn in BINARY_ALL:
    for _dt in ALL_DTYPES:
        CASES.append(_binary_case(_name, _fcn, _dt))
for _name, _fcn in BINARY_FLOAT:
    for _dt in (np.float32, np.float64):
        CASES.append(_binary_case(_name, _fcn, _dt))
for _dt in (np.float32, np.float64, np.int8, np.int16, np.int32, np.int64):
    CASES.append(Case('abs_%s' % np.dtype(_dt).name,
                      (lambda dt: lambda rng: [_unary_op(ovl.absolute)(
                          (np.random.RandomState(1).uniform(-100, 100, 100)).astype(dt))[0]])(_dt)))
for _dt in ALL_DTYPES:
    CASES.append(Case('not_%s' % np.dtype(_dt).name,
                      (lambda dt: lambda rng: [_unary_op(ovl.logical_not)(
                          np.random.RandomState(1).randint(0, 2, 100).astype(dt))[0]])(_dt)))
for _dt in (np.float32, np.float64):
    for _pname, _p in (('isinf', ovl.isinf), ('isfinite', ovl.isfinite), ('isnan', ovl.isnan)):
        CASES.append(Case('%s_%s' % (_pname, np.dtype(_dt).name),
                          (lambda dt, p: lambda rng: [_unary_op(p)(
                              np.array([1.5, 0, np.nan, np.inf, -np.inf]).astype(dt))[0]])(_dt, _p)))

CASE_BY_NAME = dict((c.name, c) for c in CASES)


# ----------------------------------------------------------------------------------------------------------------------
# comparison helpers
# ----------------------------------------------------------------------------------------------------------------------
def ulp_distance(a, b):
    """Element-wise distance in representable values between two float arrays of one dtype (NaN == NaN)."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    assert a.dtype == b.dtype and a.shape == b.shape
    if a.dtype == np.float32:
        ia = a.view(np.int32).astype(np.int64)
        ib = b.view(np.int32).astype(np.int64)
        bias = np.int64(0x80000000)
    else:
        ia = a.view(np.int64).astype(np.float64)
        ib = b.view(np.int64).astype(np.float64)
        bias = np.float64(2.0 ** 63)
    ia = np.where(ia < 0, -(ia + bias), ia)
    ib = np.where(ib < 0, -(ib + bias), ib)
    dist = np.abs(ia - ib)
    both_nan = np.isnan(a) & np.isnan(b)
    return np.where(both_nan, 0, dist)


def assert_matches(case, got, ref, what=''):
    assert got.dtype == ref.dtype, '%s %s: dtype %s vs %s' % (case.name, what, got.dtype, ref.dtype)
    assert got.shape == ref.shape, '%s %s: shape %s vs %s' % (case.name, what, got.shape, ref.shape)
    if case.max_ulp == 0 or ref.dtype.kind in 'iu':
        if ref.dtype.kind == 'f':
            equal = (got == ref) | (np.isnan(got) & np.isnan(ref))
            # bit-exact apart from the sign and payload of NaN (an invalid operation gives a NaN with the sign bit
            # set on x86 and clear on the GPU): the sign of zero must agree
            equal &= (np.signbit(got) == np.signbit(ref)) | np.isnan(ref)
        else:
            equal = got == ref
        assert equal.all(), '%s %s: %d of %d elements differ (bit-exact expected)' % (
            case.name, what, int((~equal).sum()), equal.size)
    elif ref.dtype == np.float64:
        finite = np.isfinite(ref)
        assert np.array_equal(got[~finite], ref[~finite], equal_nan=True), case.name + ' non-finite values differ'
        denom = np.maximum(np.abs(ref[finite]), np.finfo(np.float64).tiny)
        err = np.abs(got[finite] - ref[finite]) / denom
        assert err.size == 0 or err.max() <= case.rel, '%s %s: relative error %g > %g' % (
            case.name, what, err.max(), case.rel)
    else:
        dist = ulp_distance(got, ref)
        assert dist.max() <= case.max_ulp, '%s %s: %g ulp > %d' % (case.name, what, dist.max(), case.max_ulp)


# ----------------------------------------------------------------------------------------------------------------------
# ahead-of-time compilation and the smoke check
# ----------------------------------------------------------------------------------------------------------------------
def _operators_of(outputs, opt_level):
    from opveclib_amd.operator import _build_op_dag
    from opveclib_amd.fusion import _merge_op_dag
    dag = _build_op_dag(*outputs).proto_dag
    if opt_level >= 3:
        dag, _ = _merge_op_dag(dag, None)
    return list(dag.operators)


# ----------------------------------------------------------------------------------------------------------------------
# 'fast' math mode: every transcendental operator on its own, compared with the oracle in units in the last place
# ----------------------------------------------------------------------------------------------------------------------
def _log_uniform(rng, lo_exp, hi_exp, n):
    """Magnitudes spread evenly over binades 2^lo_exp .. 2^hi_exp."""
    return np.exp2(rng.uniform(lo_exp, hi_exp, n)).astype(np.float32)


def fast_stage_inputs(rng, n=1 << 16):
    """Stage inputs of the 8-op chain drawn like the benchmark's (A, B uniform[-1, 1]) plus wide-range sweeps."""
    a = uniform(rng, -1, 1, n)
    b = uniform(rng, -1, 1, n)
    t2 = (a + b) * np.float32(1.0001)
    t3 = np.tanh(t2).astype(np.float32)
    t4 = (1.0 / (1.0 + np.exp(-t3.astype(np.float64)))).astype(np.float32)
    t5 = np.log1p(t4.astype(np.float64)).astype(np.float32)
    sign = np.where(rng.random(n) < 0.5, -1.0, 1.0).astype(np.float32)
    return {
        'tanh_chain': t2, 'sigmoid_chain': t3, 'log1p_chain': t4, 'expm1_chain': t5,
        'tanh_wide': sign * _log_uniform(rng, -30, 5, n),
        'sigmoid_wide': sign * _log_uniform(rng, -30, 6.4, n),
        'log1p_wide': np.concatenate([_log_uniform(rng, -30, 30, n // 2), -_log_uniform(rng, -30, -0.01, n // 2)]),
        'expm1_wide': sign * _log_uniform(rng, -30, 6.4, n),
        'exp_wide': sign * _log_uniform(rng, -20, 6.6, n),
        'log_wide': _log_uniform(rng, -140, 127, n),
        'div_wide': (sign * _log_uniform(rng, -60, 60, n), _log_uniform(rng, -60, 60, n)),
    }


def _fast_case(name, key, fcn, max_ulp=2):
    def build(rng):
        x = fast_stage_inputs(rng)[key]
        return [fcn(*x)[0]] if isinstance(x, tuple) else [fcn(x)[0]]
    return Case('fast_' + name, build, max_ulp=max_ulp, seed=2)


def _raw_exp_op():
    @ovl.operator()
    def raw_exp(x):
        pos = ovl.position_in(x.shape)
        out = ovl.output_like(x)
        out[pos] = ovl.exp(x[pos])
        return out
    return raw_exp


def _raw_log_op():
    @ovl.operator()
    def raw_log(x):
        pos = ovl.position_in(x.shape)
        out = ovl.output_like(x)
        out[pos] = ovl.log(x[pos])
        return out
    return raw_log


# Single library calls and the division stay within 2 units in the last place of the oracle.  Operators composed of
# several of them (sigmoid = 1/(1+exp(-x)), log1p = log(u)*x/(u-1), expm1 = (e-1)*x/log(e)) add the differences up:
# 4 units is the largest distance observed over these sweeps.
FAST_CASES = [
    _fast_case('tanh_chain', 'tanh_chain', stdops.tanh),
    _fast_case('sigmoid_chain', 'sigmoid_chain', stdops.sigmoid, 4),
    _fast_case('log1p_chain', 'log1p_chain', log1p, 4),
    _fast_case('expm1_chain', 'expm1_chain', expm1, 4),
    _fast_case('tanh_wide', 'tanh_wide', stdops.tanh),
    _fast_case('sigmoid_wide', 'sigmoid_wide', stdops.sigmoid, 4),
    _fast_case('log1p_wide', 'log1p_wide', log1p, 4),
    _fast_case('expm1_wide', 'expm1_wide', expm1, 4),
    _fast_case('exp_wide', 'exp_wide', _raw_exp_op()),
    _fast_case('log_wide', 'log_wide', _raw_log_op()),
    _fast_case('div_wide', 'div_wide', stdops.div),
]


def run_fast_case_on_gpu(case, math_mode='fast'):
    """The case's operators unfused in ``math_mode`` against the oracle (exact by construction); returns the
    distances."""
    import oracle
    outs = case.outputs()
    ref = oracle.profile(outs, 1, 0)[0]
    got = ovl.evaluate(outs, target_language='hip', opt_level=0, math_mode=math_mode)
    got = got if isinstance(got, list) else [got]
    dists = []
    for g, r in zip(got, ref):
        assert g.dtype == r.dtype and g.shape == r.shape
        nan = np.isnan(r)
        assert np.array_equal(np.isnan(g), nan), case.name + ': NaN pattern differs'
        dists.append(ulp_distance(np.where(nan, 0, g).astype(r.dtype), np.where(nan, 0, r).astype(r.dtype)))
    return dists


# ----------------------------------------------------------------------------------------------------------------------
# strided sweeps of the float32 functions that come from the device math library
# ----------------------------------------------------------------------------------------------------------------------
LIBRARY_SWEEP_STEP = 4099       # every 4099th float32 bit pattern: about one million arguments over all exponents
LIBRARY_UNARY = [('sin', ovl.sin), ('cos', ovl.cos), ('tan', ovl.tan), ('arcsin', ovl.arcsin),
                 ('arccos', ovl.arccos), ('arctan', ovl.arctan), ('sinh', ovl.sinh), ('cosh', ovl.cosh),
                 ('log10', ovl.log10), ('sqrt', ovl.sqrt)]
LIBRARY_BINARY = [('power', ovl.power), ('arctan2', ovl.arctan2)]


def library_sweep_arguments():
    """Every LIBRARY_SWEEP_STEP-th float32 bit pattern (both signs, subnormals, infinities, NaNs included)."""
    bits = np.arange(0, 1 << 32, LIBRARY_SWEEP_STEP, dtype=np.uint64).astype(np.uint32)
    return bits.view(np.float32)


def library_sweep_pairs(n=1 << 20):
    """Operand pairs with magnitudes spread over binades 2^-40 .. 2^40, both signs, some exact small integers."""
    rng = np.random.default_rng(11)
    sign = lambda: np.where(rng.random(n) < 0.5, -1.0, 1.0).astype(np.float32)
    a = sign() * _log_uniform(rng, -40, 40, n)
    b = sign() * _log_uniform(rng, -40, 40, n)
    b[::5] = rng.integers(-8, 9, size=b[::5].size).astype(np.float32)
    a[::7] = sign()[::7] * _log_uniform(rng, -3, 3, a[::7].size)
    return a, b


def library_sweep_outputs():
    """[(name, operator output)] of the sweeps (tests/test_gpu_library_math.py)."""
    x = library_sweep_arguments()
    a, b = library_sweep_pairs()
    found = [(name, _unary_op(fcn)(x)[0]) for name, fcn in LIBRARY_UNARY]
    found += [(name, _binary_op(fcn)(a, b)[0]) for name, fcn in LIBRARY_BINARY]
    return found


# ----------------------------------------------------------------------------------------------------------------------
# 'ulp2' math mode at the benchmark's full size
# ----------------------------------------------------------------------------------------------------------------------
CHAIN8_SHAPE = (8192, 8192)
CHAIN8_STAGES = ('add', 'mul', 'tanh', 'sigmoid', 'log1p', 'expm1', 'sub', 'abs')
#: value ranges of the chain's stage inputs (what the code generator derives in the fused kernel, rounded outward)
CHAIN8_STAGE_INPUT_RANGE = {'log1p': (0.25, 0.75), 'expm1': (0.2, 0.6)}


@ovl.operator()
def clip_to_range(x, lo=0.0, hi=1.0):
    """min(max(x, lo), hi): leaves every value inside [lo, hi] untouched and tells the code generator the range."""
    out = ovl.output_like(x)
    pos = ovl.position_in(x.shape)
    out[pos] = ovl.minimum(ovl.maximum(x[pos], lo), hi)
    return out


def chain8_single_stage(name, x, with_range=False):
    """Operator output of one transcendental stage of the chain applied to ``x``; with ``with_range`` behind a clip
    to the stage's input range, which the optimizer fuses in (so the stage sees the range it sees inside the chain)."""
    fcn = {'tanh': stdops.tanh, 'sigmoid': stdops.sigmoid, 'log1p': log1p, 'expm1': expm1}[name]
    if with_range and name in CHAIN8_STAGE_INPUT_RANGE:
        lo, hi = CHAIN8_STAGE_INPUT_RANGE[name]
        x = clip_to_range(x, lo=lo, hi=hi)
    return fcn(x)[0]


#: (formula, lower and upper end of the clip in front of it, the routine the 'ulp2' mode must choose): the general
#: once-rounded routines on wide ranges, their shorter forms on narrow ones, the test at run time (with the formula as
#: its other branch) where the range leaves the compared domain
ULP2_CLIPPED_FORMULAS = [
    ('log1p', 2.0 ** -9, 1.0e6, 'ovl_log1p_direct'),
    ('log1p', 0.0625, 0.999, 'ovl_log1p_unit'),
    ('log1p', 1.0e-5, 0.5, 'OVL_ALL'),
    ('expm1', 0.001, 50.0, 'ovl_expm1_direct'),
    ('expm1', 0.001, 0.68, 'ovl_expm1_small'),
    ('expm1', -1.0, 0.5, 'OVL_ALL'),
    ('sigmoid', -15.0, 60.0, 'ovl_sigmoid_ulp2'),
    ('sigmoid', -1.0, 60.0, 'ovl_sigmoid_small'),
]
ULP2_CLIPPED_COUNT = 1 << 20


def ulp2_clipped_formula(kind, lo, hi, x):
    fcn = {'sigmoid': stdops.sigmoid, 'log1p': log1p, 'expm1': expm1}[kind]
    return fcn(clip_to_range(x, lo=lo, hi=hi))[0]


def ulp2_clipped_arguments(lo, hi):
    """Arguments spread evenly over the binades of [lo, hi] (both signs where the range has both), some beyond the
    ends (the clip brings them back), the ends themselves."""
    rng = np.random.default_rng(12)
    n = ULP2_CLIPPED_COUNT
    top = max(abs(lo), abs(hi)) * 2.0
    bottom = min(abs(lo), abs(hi)) / 2.0 if lo * hi > 0 else top * 2.0 ** -30
    x = _log_uniform(rng, np.log2(bottom), np.log2(top), n)
    if lo < 0:
        x = x * np.where(rng.random(n) < 0.5, -1.0, 1.0).astype(np.float32)
    x[:2] = (lo, hi)
    return x.astype(np.float32)


#: rows of the band on which the full-size 'ulp2' tests run the oracle itself
ORACLE_BAND_ROWS = 1024


def _special_float32_values():
    return np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 1e30, -1e30, 100.0, -100.0, 88.7, -88.7, 64.0, -16.0, 17.0,
                     -17.0, 1e-30, -1e-30, 1e-45, 2.0 ** -10, -(2.0 ** -10), 2.0 ** -12, -1.0, -0.99999994, -2.0,
                     2.0 ** -24, 2.0 ** -25, 709.0, -709.0], np.float32)


def stdops_lstm_full_size_inputs():
    """concat [4096, 4 x 1024] and c [4096, 1024], N(0, 1) from default_rng(4) (the benchmark's C4 tensors), with
    special values planted in the first rows of every gate and of c."""
    rng = np.random.default_rng(4)
    concat = rng.standard_normal((4096, 4096), dtype=np.float32)
    c = rng.standard_normal((4096, 1024), dtype=np.float32)
    special = _special_float32_values()
    for gate in range(4):
        for row in range(4):
            concat[row, gate * 1024 + 7 * row:gate * 1024 + 7 * row + special.size] = np.roll(special, gate + row)
    c[1, 5:5 + special.size] = special
    return concat, c


def guarded_formula_arguments():
    """float32 [1 << 20]: N(0, 1), a logarithmic sweep of both signs over 2^-30 .. 2^7, positive values, and the
    special values (each planted into an otherwise ordinary stretch, so that single wavefronts leave the compared
    domain)."""
    rng = np.random.default_rng(11)
    n = 1 << 20
    x = rng.standard_normal(n, dtype=np.float32)
    sweep = np.exp2(rng.uniform(-30.0, 7.0, n // 4)).astype(np.float32) * rng.choice([-1.0, 1.0], n // 4).astype(np.float32)
    x[n // 2:n // 2 + n // 4] = sweep
    # (a stretch of positive arguments inside every domain: whole wavefronts that take the routines)
    x[3 * n // 4:] = np.abs(x[3 * n // 4:]) + np.float32(2.0 ** -9)
    special = _special_float32_values()
    x[1000:1000 + special.size * 4096:4096][:special.size] = special
    return x


def ulp2_full_size_operators():
    """[(operator, options)] of tests/test_gpu_ulp2.py that the benchmark's own prebuild step does not cover."""
    from opveclib_amd import workloads
    spec = workloads.Spec(CHAIN8_SHAPE)
    jobs = []
    for name in ('tanh', 'sigmoid', 'log1p', 'expm1'):
        for op in _operators_of([chain8_single_stage(name, spec, with_range=True)], 3):
            jobs.append((op, {'math': 'ulp2'}))
    for kind, lo, hi, _routine in ULP2_CLIPPED_FORMULAS:
        for op in _operators_of([ulp2_clipped_formula(kind, lo, hi, workloads.Spec((ULP2_CLIPPED_COUNT,)))], 3):
            jobs.append((op, {'math': 'ulp2'}))
            jobs.append((op, None))
    # the composed LSTM cell at full size: the fused kernel that stores every stage, the single operators it is
    # compared with, the fused cell in the exact mode
    concat, c = workloads.Spec((4096, 4096)), workloads.Spec((4096, 1024))
    for op in _operators_of(workloads.stdops_lstm_stage_outputs(concat, c), 3):
        jobs.append((op, {'math': 'ulp2'}))
    for op in _operators_of(workloads.stdops_lstm_outputs(concat, c), 3):
        jobs.append((op, None))
    for out in (stdops.sigmoid(c)[0], stdops.tanh(c)[0], stdops.mul(c, c)[0], stdops.add(c, c)[0]):
        for op in _operators_of([out], 0):
            jobs.append((op, None))
    x = workloads.Spec((1 << 20,))
    for out in (stdops.sigmoid(x)[0], log1p(x)[0], expm1(x)[0]):
        for op in _operators_of([out], 0):
            jobs.append((op, {'math': 'ulp2'}))
    return jobs


# (case, code generator options): the same cases through kernel templates the generator would not pick by itself
TEMPLATE_VARIANTS = [
    ('c3_colscan_shapes', {'template': 'colskew', 'scan_strip': 64}),
    ('c3_colscan_shapes', {'template': 'colskew', 'scan_strip': 4, 'scan_sets': 3}),
    ('c3_colscan_shapes', {'template': 'colskew', 'scan_strip': 16, 'scan_sets': 2}),
    ('c3_colscan_shapes', {'template': 'colskew', 'scan_width': 4, 'scan_sets': 5}),
    ('c3_colscan_shapes', {'template': 'colskew', 'scan_movers': 0}),
    ('c3_colscan_shapes', {'template': 'colskew', 'scan_carry': False}),
    ('c3_colscan_shapes', {'template': 'colskew', 'scan_carry': False, 'scan_sets': 3}),
    ('c3_colscan_shapes', {'template': 'colskew', 'scan_movers': 512, 'scan_sets': 3}),
    ('c3_colscan_shapes', {'template': 'colskew', 'scan_sets': 5}),
    ('c3_colscan_shapes', {'template': 'colskew', 'scan_movers': 128, 'scan_strip': 16}),
    ('c3_colscan_placements', {'scan_nt': 's'}),
    ('c3_colscan_placements', {'scan_sets': 3}),
    ('c3_colscan_placements', {'scan_nt': '', 'scan_carry': False}),
    ('c3_colscan_shapes', {'template': 'colscan'}),
    ('c3_colscan_shapes', {'template': 'colscan', 'scan_rows': 32, 'scan_batch': 2}),
    ('c3_colscan_shapes', {'template': 'colscan', 'scan_sets': 3}),
    ('c3_colscan_shapes', {'template': 'map'}),
    ('c3_rowscan_shapes', {'template': 'fedscan'}),
    ('carry_scans', {'template': 'carryscan'}),
    ('carry_scans', {'template': 'carryscan', 'scan_width': 8}),
    ('carry_scans', {'template': 'fedscan'}),
    ('carry_scans', {'template': 'map'}),
    ('c3_cumsum_f32', {'template': 'carryscan'}),
    ('c3_cumprod_f64', {'template': 'carryscan', 'scan_width': 8}),
    ('c3_cumsum_f64', {'template': 'fedscan'}),
    ('c3_cumprod_f64', {'template': 'fedscan', 'scan_width': 2}),
    ('c3_cumsum_f32', {'template': 'fedscan', 'scan_width': 4, 'scan_chunk': 256}),
    ('c3_rowscan_shapes', {'template': 'rowscan'}),
    ('c3_cumsum_f32', {'template': 'rowscan'}),
    ('c3_cumprod_f64', {'template': 'rowscan'}),
    ('c3_rowscan_shapes', {'template': 'map'}),
    ('c3_cumsum_f64', {'template': 'skewscan'}),
    ('c2_chain', {'per_thread': 2}),
    ('c2_chain', {'per_thread': 4}),
    ('c4_lstm_grad', {'per_thread': 2}),
    ('c4_lstm_grad', {'cse': False}),
    ('c3_rowscan_shapes', {'template': 'skewscan', 'scan_depth': 1, 'scan_sets': 3}),
    ('gated_scans', {'scan_depth': 1, 'scan_sets': 3}),
    ('gated_scans', {'scan_interleave': 2}),
    ('gated_scans', {'scan_width': 2, 'scan_nt': 'l'}),
    ('gated_scans', {'template': 'map'}),
    ('gated_scans', {'scan_split': True}),
    ('gated_scans', {'scan_split': False, 'scan_interleave': 2}),
    ('c3_rowscan_shapes', {'template': 'skewscan', 'scan_split': True, 'scan_interleave': 2}),
    ('row_reductions', {'scan_width': 1}),
    ('row_reductions', {'scan_width': 2, 'scan_sets': 3, 'scan_nt': 'l'}),
    ('c3_cumsum_f32', {'template': 'skewscan', 'scan_depth': 2, 'scan_sets': 2}),
    ('c3_cumsum_f32', {'template': 'skewscan', 'scan_width': 2}),
    ('c3_cumprod_f64', {'template': 'skewscan', 'scan_width': 1}),
    ('c3_rowscan_shapes', {'template': 'skewscan', 'scan_width': 4, 'scan_depth': 1}),
    ('c3_rowscan_shapes', {'template': 'skewscan', 'scan_interleave': 2}),
    ('c3_cumprod_f64', {'template': 'skewscan', 'scan_interleave': 3, 'scan_sets': 3}),
    ('accumulate_max', {'template': 'skewscan', 'scan_interleave': 4}),
    ('c5_variants', {'template': 'map'}),
    ('c2_chain', {'vec': 2}),
    ('c2_chain', {'value_ranges': False}),
    ('c2_chain_special', {'value_ranges': False}),
    ('bounded_mix', {'value_ranges': False}),
    # grids smaller than the work: the map and transpose kernels stride over the rest
    ('c2_chain', {'grid_cap': 3}),
    ('odd_sizes', {'grid_cap': 1}),
    ('pad_crop', {'grid_cap': 2}),
    ('c5_variants', {'grid_cap': 2}),
    ('c5_variants', {'nt': 'l'}),
    ('batched_transposes', {'template': 'map'}),
    ('moved_axes', {'template': 'map'}),
    ('moved_axes', {'tile_i': 16, 'tile_j': 64}),
    ('moved_axes', {'tile_order': 'plain'}),
    # (tiles of 8 x 8 workers: groups of 64 stripes, of eight, and stripes left over in one kernel)
    ('c5_variants', {'tile_i': 8, 'tile_j': 8, 'tile_order': 'xcd'}),
    ('batched_transposes', {'tile_i': 8, 'tile_j': 8, 'tile_order': 'xcd'}),
    ('col_reductions', {'template': 'map'}),
    ('col_reductions', {'scan_rows': 32, 'scan_batch': 2}),
    ('col_reductions', {'scan_sets': 3}),
    ('col_reductions', {'scan_skew': False}),
    ('col_reductions', {'scan_movers': 0}),
    ('col_reductions', {'scan_strip': 16, 'scan_movers': 0, 'scan_sets': 2}),
    ('col_reductions', {'scan_strip': 64}),
    ('col_reductions', {'scan_width': 4, 'scan_movers': 128}),
    ('row_reductions', {'template': 'map'}),
    ('row_reductions', {'scan_depth': 1}),
    ('row_reductions', {'scan_depth': 3, 'scan_width': 1}),
    ('batched_transposes', {'tile_i': 16, 'tile_j': 64}),
    ('c5_variants', {'nt': 'ls'}),
    ('c5_variants', {'template': 'map', 'grid_cap': 5}),
]


# fused cases also evaluated end to end in 'fast' mode (tolerance on the absolute error, see the test)
FAST_FUSED_CASES = ['c2_chain', 'c4_lstm', 'c4_lstm_grad', 'c1_shift_expm1_log1p', 'bounded_mix']

# row scans that the 'fast' math mode may run as a reassociating (tree-shaped) scan: sums, products, running extrema
FAST_SCAN_CASES = ['c3_cumsum_f32', 'c3_cumprod_f32', 'c3_cumsum_f64', 'c3_cumprod_f64', 'c3_rowscan_shapes',
                   'int_accumulate', 'accumulate_max', 'accumulate_axes']


def run_variant_on_gpu(name, options):
    from opveclib_amd import runtime
    runtime.codegen_options = dict(options)
    try:
        run_case_on_gpu(CASE_BY_NAME[name], 3)
    finally:
        runtime.codegen_options = {}


def prebuild_all(cases=None, workers=8, with_oracle=True):
    """Compile the HIP library (and the oracle library) of every operator used by the cases and the benchmark."""
    from concurrent.futures import ThreadPoolExecutor
    from opveclib_amd import compiler, runtime
    import oracle
    from opveclib_amd import workloads

    ops = {}
    oracle_ops = {}
    for case in (cases or CASES):
        outs = case.outputs()
        for level in (0, 3):
            for op in _operators_of(outs, level):
                ops[op.SerializeToString()] = op
        for op in _operators_of(outs, 0):
            oracle_ops[op.SerializeToString()] = op
    oracle_o2 = {}
    for outs in workloads.all_workload_outputs():
        for op in _operators_of(outs, 3):
            ops[op.SerializeToString()] = op
        # the benchmark's CPU legs: every workload as written, the headline also fused, with and without -O2
        for op in _operators_of(outs, 0):
            oracle_ops[op.SerializeToString()] = op
    headline = workloads.chain8_outputs(workloads.Spec((8192, 8192)), workloads.Spec((8192, 8192)),
                                        workloads.Spec((1,)))
    for op in _operators_of(headline, 3):
        oracle_ops[op.SerializeToString()] = op
        oracle_o2[op.SerializeToString()] = op

    variants = []
    if cases is None:
        for name, options in TEMPLATE_VARIANTS:
            for op in _operators_of(CASE_BY_NAME[name].outputs(), 3):
                variants.append((op, options))
        for case in FAST_CASES:
            outs = case.outputs()
            for op in _operators_of(outs, 0):
                variants.append((op, {'math': 'fast'}))
                variants.append((op, {'math': 'ulp2'}))
                oracle_ops[op.SerializeToString()] = op
        for name in FAST_FUSED_CASES + FAST_SCAN_CASES:
            for op in _operators_of(CASE_BY_NAME[name].outputs(), 3):
                variants.append((op, {'math': 'fast'}))
        for name in FAST_FUSED_CASES + ['c2_chain_stages']:
            for op in _operators_of(CASE_BY_NAME[name].outputs(), 3):
                variants.append((op, {'math': 'ulp2'}))
        variants.extend(ulp2_full_size_operators())
        for _name, out in library_sweep_outputs():
            for op in _operators_of([out], 0):
                ops[op.SerializeToString()] = op
                oracle_ops[op.SerializeToString()] = op
        # tests/test_gpu_ulp2.py: the oracle on slices of 64 rows of the full-size chain and on the small chain's stages
        rows = np.zeros((64, CHAIN8_SHAPE[1]), np.float32)
        band = np.zeros((ORACLE_BAND_ROWS, CHAIN8_SHAPE[1]), np.float32)
        small = np.zeros((96, 256), np.float32)
        lstm_band = np.zeros((ORACLE_BAND_ROWS, 1024), np.float32)
        guarded = np.zeros(1 << 20, np.float32)
        for x in (rows, small, band, lstm_band, guarded):
            for name in ('tanh', 'sigmoid', 'log1p', 'expm1'):
                for op in _operators_of([chain8_single_stage(name, x)], 0):
                    oracle_ops[op.SerializeToString()] = op
        for op in _operators_of(workloads.chain8_stage_outputs(rows, rows, np.ones(1, np.float32)), 0):
            oracle_ops[op.SerializeToString()] = op
        from tests import random_programs
        for seed in random_programs.GPU_SEEDS:
            program = random_programs.application(seed).expression_dag
            ops[program.SerializeToString()] = program
            oracle_ops[program.SerializeToString()] = program
            variants.append((program, {'value_ranges': False}))
            variants.append((program, {'math': 'fast'}))
            variants.append((program, {'math': 'ulp2'}))
        for seed in random_programs.INDEX_SEEDS:
            program = random_programs.index_application(seed).expression_dag
            ops[program.SerializeToString()] = program
            oracle_ops[program.SerializeToString()] = program
        for seed in random_programs.TYPED_SEEDS:
            program = random_programs.typed_application(seed).expression_dag
            ops[program.SerializeToString()] = program
            oracle_ops[program.SerializeToString()] = program
        for seed in random_programs.SCAN_SEEDS:
            program = random_programs.scan_application(seed).expression_dag
            ops[program.SerializeToString()] = program
            oracle_ops[program.SerializeToString()] = program
            variants.append((program, {'math': 'fast'}))
        for seed in random_programs.REDUCE_SEEDS:
            program = random_programs.reduce_application(seed).expression_dag
            ops[program.SerializeToString()] = program
            oracle_ops[program.SerializeToString()] = program
        for seed in random_programs.DAG_SEEDS:
            outs = random_programs.random_dag(seed)
            for level in (0, 3):
                for op in _operators_of(outs, level):
                    ops[op.SerializeToString()] = op
            for op in _operators_of(outs, 0):
                oracle_ops[op.SerializeToString()] = op
        from tests import golden
        for _name, out, _expected, _sum, _atol in golden.known_answers():
            for op in _operators_of(all_outputs(out), 0):
                ops[op.SerializeToString()] = op
        zeros = np.zeros((48, 256), np.float32)
        for level in (0, 3):
            for op in _operators_of(graph_capture_dag(zeros, zeros), level):
                ops[op.SerializeToString()] = op
        for op in _operators_of(graph_capture_single(np.zeros(4096, np.float32)), 3):
            variants.append((op, {'math': 'fast'}))
        for k in range(4):      # tests/test_gpu_launcher.py: concurrent evaluation on large host arrays
            staged = np.zeros((3 << 20) + k, np.float32)
            for op in _operators_of([stdops.add(staged, staged)[0]], 0):
                ops[op.SerializeToString()] = op
        staged = np.zeros((4096, 4096), np.float32)
        for op in _operators_of([stdops.mul(stdops.add(staged, staged), staged)[0]], 3):
            ops[op.SerializeToString()] = op
        from tests import large_cases
        for op in large_cases.operators_to_build():
            ops[op.SerializeToString()] = op
        from tests import autograd_cases
        for outs in autograd_cases.graphs_to_build():
            for level in (0, 3):
                for op in _operators_of(outs, level):
                    ops[op.SerializeToString()] = op
        for outs in workloads.all_workload_outputs():
            for op in _operators_of(outs, 3):
                if any(e.code in (lang.EXP, lang.LOG, lang.TANH, lang.DIVIDE) for e in op.expressions):
                    variants.append((op, {'math': 'fast'}))

    compiler.prebuild_mode = True
    try:
        with ThreadPoolExecutor(max_workers=workers) as pool:
            list(pool.map(runtime.build_operator, ops.values()))
            list(pool.map(lambda v: runtime.build_operator(*v), variants))
            if with_oracle:
                list(pool.map(oracle.compile_op, oracle_ops.values()))
                list(pool.map(lambda op: oracle.compile_op(op, ('-O2',)), oracle_o2.values()))
    finally:
        compiler.prebuild_mode = False
    return len(ops), len(oracle_ops)


def run_case_on_gpu(case, opt_level):
    import oracle
    outs = case.outputs()
    ref = oracle.profile(outs, 1, 0)[0]
    got = ovl.evaluate(outs, target_language='hip', opt_level=opt_level, math_mode='exact')
    got = got if isinstance(got, list) else [got]
    assert len(got) == len(ref)
    for n, (g, r) in enumerate(zip(got, ref)):
        assert_matches(case, g, r, 'output %d opt_level %d' % (n, opt_level))


SMOKE_CASES = ('c2_chain', 'c4_lstm', 'c1_shift')


def smoke_check():
    for name in SMOKE_CASES:
        run_case_on_gpu(CASE_BY_NAME[name], 3)
