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
