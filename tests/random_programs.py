"""
Random operator programs for differential tests: element-wise programs over two float32 inputs built from the
operations whose results are bit-compatible between the HIP path and the CPU oracle (arithmetic, exp / log / tanh,
sqrt, floor, ceil, min / max, comparisons, logical operations, variables assigned under if / elif / else).  The
program of a seed is the same everywhere (Python's ``random.Random``).
"""
import random

import numpy as np

import opveclib_amd as ovl

UNARY = [ovl.tanh, ovl.exp, ovl.log, ovl.absolute, lambda v: -v, ovl.sqrt, ovl.floor, ovl.ceil]
BINARY = [lambda a, b: a + b, lambda a, b: a - b, lambda a, b: a * b, lambda a, b: a / b, ovl.minimum, ovl.maximum]
COMPARE = [lambda a, b: a < b, lambda a, b: a <= b, lambda a, b: a > b, lambda a, b: a >= b, lambda a, b: a == b,
           lambda a, b: a != b]
CONSTANTS = [0.0, 1.0, -1.0, 0.5, 2.0, -2.0, 50.0, -50.0, 0.25, 3.0, 88.0, 1e-8, 1e30, 0.6, 10.0]


def make_operator(seed):
    @ovl.operator()
    def program(x, y):
        rng = random.Random(seed)
        pos = ovl.position_in(x.shape)
        out0 = ovl.output_like(x)
        out1 = ovl.output_like(x)
        leaves = [x[pos], y[pos]]
        variables = []

        def expr(depth):
            r = rng.random()
            if depth <= 0 or r < 0.15:
                r2 = rng.random()
                if r2 < 0.55 or not variables:
                    return rng.choice(leaves)
                if r2 < 0.8:
                    return rng.choice(variables)
                return rng.choice(leaves) * rng.choice(CONSTANTS)
            if r < 0.45:
                return rng.choice(UNARY)(expr(depth - 1))
            if r < 0.85:
                a = expr(depth - 1)
                b = expr(depth - 1) if rng.random() < 0.7 else rng.choice(CONSTANTS)
                return rng.choice(BINARY)(a, b)
            if r < 0.95:
                other = rng.choice(CONSTANTS) if rng.random() < 0.6 else expr(depth - 1)
                return rng.choice(COMPARE)(expr(depth - 1), other)
            a = rng.choice(COMPARE)(expr(depth - 1), rng.choice(CONSTANTS))
            b = rng.choice(COMPARE)(expr(depth - 1), rng.choice(CONSTANTS))
            return (ovl.logical_and if rng.random() < 0.5 else ovl.logical_or)(a, b)

        for _ in range(rng.randint(1, 3)):
            v = ovl.variable(rng.choice(CONSTANTS), x.dtype)
            cond = rng.choice(COMPARE)(expr(2), rng.choice(CONSTANTS))
            branches = rng.randint(1, 3)
            with ovl.if_(cond):
                v <<= expr(3)
            if branches >= 2:
                with ovl.elif_(rng.choice(COMPARE)(expr(2), rng.choice(CONSTANTS))):
                    v <<= expr(2)
            if branches >= 3 or rng.random() < 0.5:
                with ovl.else_():
                    v <<= expr(2)
            variables.append(v)
            leaves.append(ovl.tanh(v) if rng.random() < 0.3 else v + 0.0)
        out0[pos] = expr(4)
        out1[pos] = expr(4)
        return out0, out1
    return program


def inputs(seed, shape=(4, 128)):
    from tests import cases
    rng = np.random.default_rng(seed)
    return cases.special_values(rng, shape), np.roll(cases.special_values(rng, shape), 5)


def application(seed):
    """The program of ``seed`` applied to its inputs."""
    x, y = inputs(seed)
    return make_operator(seed)(x, y)


GPU_SEEDS = list(range(16))


# ----------------------------------------------------------------------------------------------------------------------
# random DAGs of library operators (fusion)
# ----------------------------------------------------------------------------------------------------------------------
def random_dag(seed):
    """Outputs of a random DAG of 3 to 9 element-wise library operators (cyclic shifts included) over three vectors."""
    from opveclib_amd import stdops
    from opveclib_amd.examples import expm1, log1p, shift_cyclic, absolute
    from tests import cases
    unary = [stdops.tanh, stdops.sigmoid, stdops.neg, lambda t: log1p(t)[0], lambda t: expm1(t)[0],
             lambda t: absolute(t)[0], lambda t: shift_cyclic(t)[0]]
    binary = [stdops.add, stdops.sub, stdops.mul, stdops.div]
    rng = random.Random(seed)
    nrng = np.random.default_rng(seed)
    n = rng.choice([256, 1024, 4096])
    leaves = [cases.special_values(nrng, (n,)) if rng.random() < 0.3 else nrng.uniform(-2, 2, n).astype(np.float32)
              for _ in range(3)]
    scalar = np.array([rng.choice([1.0001, 0.5, -2.0])], np.float32)
    nodes = list(leaves)
    for _ in range(rng.randint(3, 9)):
        r = rng.random()
        if r < 0.45:
            nodes.append(rng.choice(unary)(rng.choice(nodes)))
        elif r < 0.9:
            nodes.append(rng.choice(binary)(rng.choice(nodes), rng.choice(nodes)))
        else:
            nodes.append(stdops.mul(rng.choice(nodes), scalar))
    produced = nodes[3:]
    count = rng.randint(1, min(3, len(produced)))
    outs = [produced[-1]] + (rng.sample(produced[:-1], count - 1) if len(produced) > 1 else [])
    return [o if not hasattr(o, 'output_types') else o[0] for o in outs]


DAG_SEEDS = list(range(100, 112))


# ----------------------------------------------------------------------------------------------------------------------
# Random index programs: gathers through computed indices, guarded neighbour reads, stores through one-to-one index maps.
# They exercise what the code generator decides from index expressions: which accesses become vector accesses, which
# loads may move ahead of the conditions that guard them, which modulo operations cannot wrap, which template runs.
# ----------------------------------------------------------------------------------------------------------------------
INDEX_DTYPES = [np.float32, np.float32, np.float64, np.int32, np.uint8, np.int16]
LAST_DIMS = [4, 8, 12, 16, 20, 32, 64, 100, 7, 33, 128, 256]
OUTER_DIMS = [1, 2, 3, 5, 8, 16, 17]
MULTIPLIERS = [1, 2, 3, 4, 5, 7, 16, 31, 7919, 65537, 2 ** 31 + 1, 2 ** 32 - 1]


def _coprime(rng, n):
    import math
    while True:
        a = rng.choice([1, 3, 5, 7, 11, 13, 7919, n - 1 if n > 1 else 1, n + 1])
        if math.gcd(a, n) == 1:
            return a


def index_program_shapes(seed):
    """(workgroup shape, dtype, shapes of the gathered operands) of the program of ``seed``."""
    rng = random.Random(seed * 7919 + 1)
    rank = rng.choice([1, 2, 2, 3])
    shape = [rng.choice(OUTER_DIMS) for _ in range(rank - 1)] + [rng.choice(LAST_DIMS)]
    dtype = rng.choice(INDEX_DTYPES)
    gathered = []
    for _ in range(2):
        g_rank = rng.choice([1, 1, 2, 3])
        gathered.append([rng.choice([1, 2, 3, 5, 8, 16, 17, 64, 100, 257]) for _ in range(g_rank)])
    return shape, dtype, gathered


def make_index_operator(seed):
    shape, _, _ = index_program_shapes(seed)
    rank = len(shape)

    @ovl.operator()
    def index_program(x, g0, g1):
        rng = random.Random(seed)
        pos = ovl.position_in(x.shape)
        p = [pos[k] for k in range(rank)]

        def component(n):
            """An index expression with values in [0, n)."""
            form = rng.randrange(9)
            k = rng.randrange(rank)
            if form == 0:
                return p[k] % n
            if form == 1:
                return (p[k] + rng.choice([1, 2, 3, n - 1, n, 1000])) % n
            if form == 2:
                return (p[k] * rng.choice(MULTIPLIERS) + rng.choice([0, 1, 5, 2 ** 31])) % n
            if form == 3:
                j = rng.randrange(rank)
                return (p[k] * rng.choice(MULTIPLIERS) + p[j] * rng.choice([1, 2, 3])) % n
            if form == 4:
                return (n - 1) - (p[k] % n)
            if form == 5:
                return (p[k] / rng.choice([1, 2, 3, 4, 7])) % n
            if form == 6:
                return rng.randrange(n)
            if form == 7:
                return ovl.minimum(p[k], n - 1)
            return (p[k] % rng.choice([2, 3, 4, 8])) % n

        def gather(g):
            return g[[component(n) for n in g.shape]]

        value = x[pos] + gather(g0)
        if rng.random() < 0.7:
            value = value + gather(g1)

        # neighbour reads along one dimension, guarded against the ends of the tensor
        for _ in range(rng.randint(0, 2)):
            k = rng.randrange(rank)
            n = x.shape[k]
            delta = rng.choice([1, 1, 2, 4])
            neighbour = ovl.variable(0, x.dtype)
            forward = rng.random() < 0.5
            where = list(p)
            if forward:
                where[k] = p[k] + delta
                with ovl.if_(p[k] + delta < n):
                    neighbour <<= x[where]
                if rng.random() < 0.5:
                    with ovl.else_():
                        neighbour <<= x[pos]
            else:
                where[k] = p[k] - delta
                with ovl.if_(p[k] >= delta):
                    neighbour <<= x[where]
            value = value + neighbour

        # stores: one output at the worker's position, one through a one-to-one map of every dimension
        out0 = ovl.output_like(x)
        out0[pos] = value
        permuted = list(range(rank))
        if rank >= 2 and rng.random() < 0.5:
            a, b = rng.sample(range(rank), 2)
            permuted[a], permuted[b] = permuted[b], permuted[a]
        transposition = rank == 2 and rng.random() < 0.3
        if transposition:
            permuted = [1, 0]
        target = []
        for k in permuted:
            n = x.shape[k]
            form = 0 if transposition else rng.randrange(4)
            if form == 0:
                target.append(p[k])
            elif form == 1:
                target.append((p[k] + rng.choice([1, 2, n - 1, 5])) % n)
            elif form == 2:
                target.append((n - 1) - p[k])
            else:
                target.append((p[k] * _coprime(rng, n) + rng.choice([0, 1, 3])) % n)
        out1 = ovl.output([x.shape[k] for k in permuted], x.dtype)
        out1[target] = value + x[pos]
        return out0, out1
    return index_program


def index_inputs(seed):
    shape, dtype, gathered = index_program_shapes(seed)
    rng = np.random.default_rng(seed)

    def data(s):
        if np.dtype(dtype).kind == 'f':
            return rng.standard_normal(s).astype(dtype)
        return rng.integers(0, 50, s).astype(dtype)
    return [data(shape)] + [data(g) for g in gathered]


def index_application(seed):
    """The index program of ``seed`` applied to its inputs (an operator with two outputs)."""
    return make_index_operator(seed)(*index_inputs(seed))


INDEX_SEEDS = range(200, 224)


# ----------------------------------------------------------------------------------------------------------------------
# Random scan programs: one worker per row walks the last axis with loop-carried state.  The scan templates find the
# carried state in the DAG, so the body can be any straight-line update: one or two state variables, sums, products,
# running extrema, decayed sums, integer and floating point types; row lengths that are whole groups of the lane-skewed
# template (16 vectors), lengths with columns left over, lengths that leave rows unaligned, and rows too short for it.
# ----------------------------------------------------------------------------------------------------------------------
SCAN_DTYPES = [np.float32, np.float32, np.float64, np.int32, np.int64, np.int16]
SCAN_LENGTHS = [64, 128, 192, 256, 320, 512, 1024, 32, 96, 100, 7, 2, 130, 70, 333, 517]
SCAN_ROWS = [[1], [3], [4], [5], [16], [17], [67], [2, 3], [4, 9], [2, 2, 5]]


def scan_program_shape(seed):
    rng = random.Random(seed * 104729 + 7)
    return rng.choice(SCAN_ROWS) + [rng.choice(SCAN_LENGTHS)], rng.choice(SCAN_DTYPES)


def make_scan_operator(seed):
    shape, dtype = scan_program_shape(seed)
    floating = np.dtype(dtype).kind == 'f'

    @ovl.operator()
    def scan_program(x):
        rng = random.Random(seed)
        length = x.shape[-1]
        pos = ovl.position_in(x.shape[:-1])
        out = ovl.output_like(x)

        def at(i):
            return [pos[k] for k in range(x.rank - 1)] + [i]

        def update(state, other, element):
            form = rng.randrange(8)
            if form == 0:
                return state + element
            if form == 1:
                return state * element if floating else state + element * 3
            if form == 2:
                return ovl.maximum(state, element)
            if form == 3:
                return ovl.minimum(state, element)
            if form == 4:
                return state + element * element
            if form == 5:
                return state * 0.5 + element if floating else state - element
            if form == 6 and other is not None:
                return ovl.maximum(state, other)
            if form == 7 and other is not None:
                return state + other
            return element - state

        two_states = rng.random() < 0.4
        first = x[at(0)]
        s0 = ovl.variable(first, x.dtype)
        s1 = ovl.variable(first if rng.random() < 0.5 else 0, x.dtype) if two_states else None
        emit_second = two_states and rng.random() < 0.5
        out[at(0)] = s1 if emit_second else s0
        for i in ovl.arange(1, length):
            element = x[at(i)]
            s0 <<= update(s0, None, element)
            if two_states:
                s1 <<= update(s1, s0, element)
            if emit_second:
                out[at(i)] = s1
            elif rng.random() < 0.3:
                out[at(i)] = s0 + element
            else:
                out[at(i)] = s0
        return out
    return scan_program


def scan_input(seed):
    shape, dtype = scan_program_shape(seed)
    rng = np.random.default_rng(seed)
    if np.dtype(dtype).kind == 'f':
        # magnitudes around one keep running products finite and interesting
        return (rng.uniform(0.7, 1.3, shape) * rng.choice([-1.0, 1.0], shape, p=[0.2, 0.8])).astype(dtype)
    return rng.integers(-3, 4, shape).astype(dtype)


def scan_application(seed):
    return make_scan_operator(seed)(scan_input(seed))


SCAN_SEEDS = range(300, 324)


# ----------------------------------------------------------------------------------------------------------------------
# Random reduction programs: one worker per line walks one axis with loop-carried state and stores only after the loop
# (sums, dot products of two inputs, sums of squares, running extrema, decayed sums; one or two state variables, an
# epilogue on the final state).  Along the last axis the lengths sit on both sides of what the row-reduction template
# wants (four groups of 64 vectors) with columns left over and unaligned rows; along another axis the line counts run
# from one to more than a strip.
# ----------------------------------------------------------------------------------------------------------------------
REDUCE_DTYPES = [np.float32, np.float32, np.float64, np.int32, np.int64]
REDUCE_LAST = [([3], 1024), ([5], 1030), ([2, 3], 1100), ([4], 2049), ([7], 1537), ([2], 512), ([3], 700), ([1], 4096)]
REDUCE_OTHER = [([], 64, 200), ([], 100, 7), ([2], 257, 64), ([], 1000, 33), ([3], 70, 129), ([], 300, 1), ([], 64, 1000)]


def reduce_program_shape(seed):
    """(shape, axis, element type)"""
    rng = random.Random(seed * 7919 + 3)
    dtype = rng.choice(REDUCE_DTYPES)
    if rng.random() < 0.5:
        outer, length = rng.choice(REDUCE_LAST)
        return outer + [length], len(outer), dtype
    outer, length, inner = rng.choice(REDUCE_OTHER)
    return outer + [length, inner], len(outer), dtype


def make_reduce_operator(seed):
    shape, axis, dtype = reduce_program_shape(seed)
    floating = np.dtype(dtype).kind == 'f'

    @ovl.operator()
    def reduce_program(x, y):
        rng = random.Random(seed)
        length = x.shape[axis]
        line_shape = [extent for k, extent in enumerate(x.shape) if k != axis]
        pos = ovl.position_in(line_shape)
        first_out = ovl.output(line_shape, x.dtype)
        second_out = ovl.output(line_shape, x.dtype)

        def at(i):
            index = [pos[k] for k in range(len(line_shape))]
            index.insert(axis, i)
            return index

        use_y = rng.random() < 0.4

        def update(state, other, element, partner):
            form = rng.randrange(8)
            if form == 0:
                return state + element
            if form == 1:
                return state + element * partner if use_y else state + element * element
            if form == 2:
                return ovl.maximum(state, element)
            if form == 3:
                return ovl.minimum(state, element)
            if form == 4:
                return state + element * element
            if form == 5:
                return state * 0.5 + element if floating else state - element
            if form == 6 and other is not None:
                return ovl.maximum(state, other)
            if form == 7 and other is not None:
                return state + other
            return element - state

        two_states = rng.random() < 0.4
        from_first = rng.random() < 0.5
        s0 = ovl.variable(x[at(0)] if from_first else 0, x.dtype)
        s1 = ovl.variable(0, x.dtype) if two_states else None
        for i in ovl.arange(1 if from_first else 0, length):
            element = x[at(i)]
            partner = y[at(i)] if use_y else None
            s0 <<= update(s0, None, element, partner)
            if two_states:
                s1 <<= update(s1, s0, element, partner)
        epilogue = rng.randrange(3)
        if epilogue == 0 or not floating:
            first_out[pos] = s0
        elif epilogue == 1:
            first_out[pos] = s0 / length
        else:
            first_out[pos] = ovl.sqrt(ovl.absolute(s0))
        second_out[pos] = s1 + s0 if two_states else s0 * 2
        return first_out, second_out
    return reduce_program


def reduce_inputs(seed):
    shape, axis, dtype = reduce_program_shape(seed)
    rng = np.random.default_rng(seed)
    if np.dtype(dtype).kind == 'f':
        return [(rng.uniform(0.7, 1.3, shape) * rng.choice([-1.0, 1.0], shape, p=[0.3, 0.7])).astype(dtype)
                for _ in range(2)]
    return [rng.integers(-3, 4, shape).astype(dtype) for _ in range(2)]


def reduce_application(seed):
    return make_reduce_operator(seed)(*reduce_inputs(seed))


REDUCE_SEEDS = range(500, 524)


# ----------------------------------------------------------------------------------------------------------------------
# Random typed programs: element-wise expressions over all ten element types with casts between them, integer
# division and remainder (C truncation), comparisons that yield 0/1 in the operand type, small counted loops and
# worker-local tensors.  Inputs are small integers, so that no signed arithmetic overflows (undefined in C, for the
# reference's generated code as much as for this one) and every float is exactly representable.
# ----------------------------------------------------------------------------------------------------------------------
TYPED_DTYPES = [np.float32, np.float64, np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32,
                np.uint64]


def typed_program_types(seed):
    rng = random.Random(seed * 31337 + 3)
    return rng.choice(TYPED_DTYPES), rng.choice(TYPED_DTYPES), rng.choice([[64], [5, 12], [3, 7], [2, 3, 16], [100]])


def make_typed_operator(seed):
    @ovl.operator()
    def typed_program(x, y):
        rng = random.Random(seed)
        pos = ovl.position_in(x.shape)
        out0 = ovl.output_like(x)
        out1 = ovl.output_like(y)
        dtypes = [ovl.float32, ovl.float64, ovl.int8, ovl.int16, ovl.int32, ovl.int64, ovl.uint8, ovl.uint16,
                  ovl.uint32, ovl.uint64]

        def leaf(dtype):
            source = rng.choice([x, y])
            value = source[pos]
            if source.dtype == dtype:
                return value
            floats = (ovl.float32, ovl.float64)
            if source.dtype in floats and dtype not in floats and dtype != ovl.int32:
                value = ovl.cast(value, ovl.int32)
            return ovl.cast(value, dtype)

        def expr(dtype, depth):
            """An expression of type ``dtype`` whose magnitude stays below a few thousand."""
            if depth <= 0:
                return leaf(dtype)
            form = rng.randrange(10)
            if form == 0:
                return expr(dtype, depth - 1) + expr(dtype, depth - 1)
            if form == 1:
                return expr(dtype, depth - 1) - leaf(dtype)
            if form == 2:
                return leaf(dtype) * leaf(dtype)
            if form == 3:
                # the divisor is made odd, hence never zero
                if dtype in (ovl.float32, ovl.float64):
                    return expr(dtype, depth - 1) / (leaf(dtype) * 2 + 1)
                return expr(dtype, depth - 1) / (leaf(dtype) * 2 + 1)
            if form == 4 and dtype not in (ovl.float32, ovl.float64):
                return expr(dtype, depth - 1) % (leaf(dtype) * 2 + 1)
            if form == 5:
                return ovl.minimum(expr(dtype, depth - 1), leaf(dtype))
            if form == 6:
                return ovl.maximum(expr(dtype, depth - 1), leaf(dtype))
            if form == 7:
                other = rng.choice(dtypes)
                value = expr(other, depth - 1)
                floats = (ovl.float32, ovl.float64)
                if other in floats and dtype not in floats and dtype != ovl.int32:
                    # a float outside the target's range (a negative one for an unsigned target) converts with
                    # undefined behaviour in C: go through int32, which holds every value that occurs here
                    value = ovl.cast(value, ovl.int32)
                return ovl.cast(value, dtype)
            if form == 8:
                a, b = expr(dtype, depth - 1), leaf(dtype)
                return rng.choice([lambda: a < b, lambda: a <= b, lambda: a == b, lambda: a != b, lambda: a >= b])()
            return leaf(dtype) + rng.choice([0, 1, 2, 3])

        first = expr(x.dtype, 3)
        # a small counted loop over a worker-local tensor
        if rng.random() < 0.5:
            taps = rng.randint(2, 5)
            window = ovl.zeros(taps, x.dtype)
            for k in ovl.arange(taps):
                window[k] = leaf(x.dtype) + ovl.cast(k, x.dtype)
            total = ovl.variable(0, x.dtype)
            for k in ovl.arange(taps - 1, -1, -1):
                total <<= total + window[k]
            first = first + total
        out0[pos] = first
        chosen = ovl.variable(0, y.dtype)
        with ovl.if_(expr(x.dtype, 1) < leaf(x.dtype)):
            chosen <<= expr(y.dtype, 2)
        with ovl.else_():
            chosen <<= expr(y.dtype, 3)
        out1[pos] = chosen
        return out0, out1
    return typed_program


def typed_inputs(seed):
    dx, dy, shape = typed_program_types(seed)
    rng = np.random.default_rng(seed)

    def data(dtype):
        lo = 0 if np.dtype(dtype).kind == 'u' else -6
        return rng.integers(lo, 7, shape).astype(dtype)
    return data(dx), data(dy)


def typed_application(seed):
    return make_typed_operator(seed)(*typed_inputs(seed))


TYPED_SEEDS = range(400, 424)
