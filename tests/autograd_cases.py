"""
Differentiable operator graphs shared by the CPU structure tests, the GPU autograd tests and the ahead-of-time build.

Each case names the leaves (numpy arrays, drawn from a seeded generator), which of them are differentiated, the OVL
graph and the same function written with torch operations.  The graphs restate the reference's gradient tests
(opveclib/test/test_gradients.py:18-125, opveclib/stdops/test_math.py:91-157, the merged gradient DAG test
opveclib/test/test_operator_merge.py:395-487 and the stdops LSTM of test_operator_merge.py:311-321) against
``torch.autograd`` instead of TensorFlow.
"""
import numpy as np

import opveclib_amd as ovl
from opveclib_amd import stdops
from opveclib_amd.lstm import lstm


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


@ovl.gradient(clip)
@ovl.operator()
def clip_grad(arg, d_arg, threshold1=None, threshold2=None):
    pos = ovl.position_in(arg.shape)
    g = ovl.output_like(arg)
    x = arg[pos]
    with ovl.if_(x < threshold1):
        g[pos] = 0
    with ovl.elif_(x > threshold2):
        g[pos] = 0
    with ovl.else_():
        g[pos] = d_arg[pos]
    return g


@ovl.operator()
def square_plus(x, y):
    pos = ovl.position_in(x.shape)
    z = ovl.output_like(x)
    z[pos] = x[pos] * x[pos] + 3 * y[pos]
    return z


@ovl.gradient(square_plus)
@ovl.operator()
def square_plus_grad(x, y, dz):
    pos = ovl.position_in(x.shape)
    dx = ovl.output_like(x)
    dy = ovl.output_like(y)
    dx[pos] = 2.0 * x[pos] * dz[pos]
    dy[pos] = 3.0 * dz[pos]
    return dx, dy


@ovl.operator()
def fan_out(in0, in1):
    pos = ovl.position_in(in0.shape)
    out0 = ovl.output_like(in0)
    out1 = ovl.output_like(in1)
    out2 = ovl.output_like(in1)
    out0[pos] = 2 * in0[pos]
    out1[pos] = 3 * in1[pos]
    out2[pos] = 4 * in1[pos]
    return out0, out1, out2


@ovl.gradient(fan_out)
@ovl.operator()
def fan_out_grad(in0, in1, dout0, dout1, dout2):
    pos = ovl.position_in(in0.shape)
    din0 = ovl.output_like(in0)
    din1 = ovl.output_like(in1)
    din0[pos] = 2 * dout0[pos]
    din1[pos] = 3 * dout1[pos] + 4 * dout2[pos]
    return din0, din1


@ovl.operator()
def fan_in(in0, in1, in2, in3):
    pos = ovl.position_in(in0.shape)
    out0 = ovl.output_like(in0)
    out1 = ovl.output_like(in0)
    out0[pos] = 5 * in0[pos] + 6 * in1[pos]
    out1[pos] = 7 * in2[pos] + 8 * in3[pos]
    return out0, out1


@ovl.gradient(fan_in)
@ovl.operator()
def fan_in_grad(in0, in1, in2, in3, dout0, dout1):
    pos = ovl.position_in(in0.shape)
    din0 = ovl.output_like(in0)
    din1 = ovl.output_like(in1)
    din2 = ovl.output_like(in2)
    din3 = ovl.output_like(in3)
    din0[pos] = 5 * dout0[pos]
    din1[pos] = 6 * dout0[pos]
    din2[pos] = 7 * dout1[pos]
    din3[pos] = 8 * dout1[pos]
    return din0, din1, din2, din3


@ovl.operator()
def no_gradient_scale(x):
    """An operator without a registered gradient."""
    pos = ovl.position_in(x.shape)
    out = ovl.output_like(x)
    out[pos] = 2 * x[pos]
    return out


class AutogradCase(object):
    """
    :param make_leaves: function(rng) -> list of numpy arrays
    :param differentiable: indices of the leaves that require grad
    :param graph: function(*leaves) -> list of OVL operator outputs
    :param torch_graph: function(torch, *tensors) -> list of torch tensors (the same math)
    :param exact: gradients must equal torch's bit for bit (plain arithmetic in the same order), else rtol applies
    """

    def __init__(self, name, make_leaves, differentiable, graph, torch_graph, exact=False, rtol=1e-12):
        self.name = name
        self.make_leaves = make_leaves
        self.differentiable = differentiable
        self.graph = graph
        self.torch_graph = torch_graph
        self.exact = exact
        self.rtol = rtol

    def leaves(self):
        return self.make_leaves(np.random.default_rng(11))

    def __repr__(self):
        return self.name


def _pair(n=100):
    def make(rng):
        lhs = rng.random(n)
        rhs = lhs + rng.integers(-1, 2, size=n) + 0.25
        return [lhs, rhs]
    return make


def _binary(name, fcn, torch_fcn, exact=True):
    return AutogradCase('binary_' + name, _pair(), [0, 1],
                        lambda l, r: [fcn(l, r)[0], fcn(r, l)[0]],
                        lambda torch, l, r: [torch_fcn(torch, l, r), torch_fcn(torch, r, l)], exact=exact)


def _unary(name, fcn, torch_fcn):
    return AutogradCase('unary_' + name, lambda rng: [rng.random(100)], [0],
                        lambda x: [fcn(x)[0]], lambda torch, x: [torch_fcn(torch, x)])


def _merge_graph(x0, x1, h3):
    y0, y1, y2 = fan_out(x0, x1)
    z0, z1 = fan_in(y1, y2, y2, h3)
    return [z1, z0, y1, y0]


def _merge_torch(torch, x0, x1, h3):
    y0, y1, y2 = 2 * x0, 3 * x1, 4 * x1
    return [7 * y2 + 8 * h3, 5 * y1 + 6 * y2, 1.0 * y1, y0]


def _stdops_lstm(concat_arg, c):
    i, j, f, o = stdops.split(concat_arg, split_dim=1, num_split=4)
    new_c = stdops.mul(c, stdops.sigmoid(f)) + stdops.sigmoid(i) * stdops.tanh(j)
    new_h = stdops.tanh(new_c) * stdops.sigmoid(o)
    return [new_c, new_h]


def _fused_lstm(concat_arg, c):
    cell = lstm(concat_arg, c, forget_bias=1.0)
    return [cell[0], cell[1]]


def _torch_lstm(forget_bias):
    def fcn(torch, concat_arg, c):
        i, j, f, o = torch.chunk(concat_arg, 4, dim=1)
        new_c = c * torch.sigmoid(f + forget_bias) + torch.sigmoid(i) * torch.tanh(j)
        new_h = torch.tanh(new_c) * torch.sigmoid(o)
        return [new_c, new_h]
    return fcn


def _lstm_leaves(dtype, batches, units):
    def make(rng):
        return [rng.standard_normal((batches, 4 * units)).astype(dtype),
                rng.standard_normal((batches, units)).astype(dtype)]
    return make


CASES = [
    AutogradCase('square_plus', lambda rng: [rng.random(10), rng.random(10)], [0, 1],
                 lambda a, b: [square_plus(a, b)[0]], lambda torch, a, b: [a * a + 3 * b], exact=True),
    AutogradCase('clip', lambda rng: [rng.random(10)], [0],
                 lambda a: [clip(a, threshold1=0.1, threshold2=0.9)[0]],
                 lambda torch, a: [torch.clamp(a, 0.1, 0.9)], exact=True),
    _binary('add', stdops.add, lambda torch, x, y: x + y),
    _binary('sub', stdops.sub, lambda torch, x, y: x - y),
    _binary('mul', stdops.mul, lambda torch, x, y: x * y),
    _binary('div', stdops.div, lambda torch, x, y: x / y, exact=False),
    _unary('neg', stdops.neg, lambda torch, x: -x),
    _unary('tanh', stdops.tanh, lambda torch, x: torch.tanh(x)),
    _unary('sin', stdops.sin, lambda torch, x: torch.sin(x)),
    _unary('cos', stdops.cos, lambda torch, x: torch.cos(x)),
    _unary('tan', stdops.tan, lambda torch, x: torch.tan(x)),
    _unary('sigmoid', stdops.sigmoid, lambda torch, x: torch.sigmoid(x)),
    AutogradCase('fan_out_fan_in', lambda rng: [rng.random(10), rng.random(10), rng.random(10)], [0, 1, 2],
                 _merge_graph, _merge_torch, rtol=1e-14),
    AutogradCase('chain_f32', lambda rng: [rng.standard_normal((64, 128), dtype=np.float32),
                                          rng.standard_normal((64, 128), dtype=np.float32)], [0, 1],
                 lambda a, b: [stdops.sigmoid(stdops.tanh(stdops.mul(stdops.add(a, b), b)))[0]],
                 lambda torch, a, b: [torch.sigmoid(torch.tanh((a + b) * b))], rtol=2e-5),
    AutogradCase('stdops_lstm_f64', _lstm_leaves(np.float64, 4, 24), [0, 1], _stdops_lstm, _torch_lstm(0.0),
                 rtol=1e-11),
    AutogradCase('fused_lstm_f32', _lstm_leaves(np.float32, 32, 128), [0, 1],
                 _fused_lstm,
                 _torch_lstm(1.0), rtol=2e-4),
    AutogradCase('constant_leaf', lambda rng: [rng.random(50), rng.random(50)], [0],
                 lambda a, b: [stdops.mul(stdops.tanh(a), b)[0]], lambda torch, a, b: [torch.tanh(a) * b]),
]
CASE_BY_NAME = dict((c.name, c) for c in CASES)


def graphs_to_build():
    """Forward and backward output lists of every case on numpy leaves, for compiling ahead of time."""
    from opveclib_amd import autograd
    from opveclib_amd.operator import _build_op_dag, _resolve_output
    built = []
    for case in CASES + [NO_GRADIENT]:
        leaves = case.leaves()
        outputs = [_resolve_output(o) for o in case.graph(*leaves)]
        built.append(outputs)
        op_dag = _build_op_dag(*outputs)
        differentiable = [1] if case is NO_GRADIENT else case.differentiable
        wanted = [any(leaf is leaves[k] for k in differentiable) for leaf in op_dag.inputs]
        leaf_grads, _ = autograd.build_backward(op_dag, wanted)
        backward = [g for g in leaf_grads if g is not None]
        if backward:
            built.append(backward)
    return built


NO_GRADIENT = AutogradCase('no_gradient', lambda rng: [rng.random(20), rng.random(20)], [0, 1],
                           lambda a, b: [stdops.mul(no_gradient_scale(a), b)[0]],
                           lambda torch, a, b: [2 * a.detach() * b])
