"""
Structure of the backward operator DAGs that `as_torch` assembles from per-operator gradient DAGs (no GPU needed):
which operators they contain, what the optimizer fuses them into, and which leaves get no gradient.
"""
import numpy as np
import pytest

from opveclib_amd import autograd, stdops
from opveclib_amd.operator import _build_op_dag, _resolve_output, _GradientPlaceholder
from opveclib_amd.fusion import _merge_op_dag
from tests import autograd_cases as ac


def _backward(case, wanted_leaves=None):
    leaves = case.leaves()
    outputs = [_resolve_output(o) for o in case.graph(*leaves)]
    op_dag = _build_op_dag(*outputs)
    wanted_leaves = case.differentiable if wanted_leaves is None else wanted_leaves
    wanted = [any(leaf is leaves[k] for k in wanted_leaves) for leaf in op_dag.inputs]
    leaf_grads, placeholders = autograd.build_backward(op_dag, wanted)
    return leaves, op_dag, leaf_grads, placeholders


def _names(outputs, merged):
    dag = _build_op_dag(*outputs).proto_dag
    if merged:
        dag, _ = _merge_op_dag(dag, None)
    return [op.name for op in dag.operators]


def test_chain_backward_recomputes_forward_and_fuses_into_one_operator():
    leaves, op_dag, grads, placeholders = _backward(ac.CASE_BY_NAME['chain_f32'])
    assert [op.name for op in op_dag.operators] == ['add', 'mul', 'tanh', 'sigmoid']
    assert len(placeholders) == 1 and all(g is not None for g in grads)
    unfused = _names(grads, merged=False)
    # forward operators whose outputs a gradient needs, every gradient operator, one sum for b (used twice)
    assert sorted(unfused) == sorted(['add', 'mul', 'tanh', 'sigmoid_grad', 'tanh_grad', 'mul_grad', 'add_grad',
                                      'gradient_sum'])
    assert len(_names(grads, merged=True)) == 1
    # its inputs: the two leaves and the gradient of the single output
    new_dag = _build_op_dag(*grads)
    kinds = sorted(type(x).__name__ for x in new_dag.inputs)
    assert kinds == ['_GradientPlaceholder', 'ndarray', 'ndarray']
    assert any(x is placeholders[0] for x in new_dag.inputs)


def test_gradient_types_match_leaf_types():
    for case in ac.CASES:
        leaves, op_dag, grads, placeholders = _backward(case)
        for leaf, grad in zip(op_dag.inputs, grads):
            if grad is None:
                continue
            tt = grad.parent.output_types[grad.index]
            assert list(tt.shape) == list(leaf.shape), case.name
            assert tt.dtype.as_numpy() == leaf.dtype, case.name
        for placeholder, out in zip(placeholders, case.graph(*leaves)):
            out = _resolve_output(out)
            assert list(placeholder.shape) == list(out.parent.output_types[out.index].shape)


def test_unwanted_and_gradient_free_leaves_get_none():
    case = ac.CASE_BY_NAME['constant_leaf']
    leaves, op_dag, grads, _ = _backward(case)
    by_leaf = dict((id(leaf), g) for leaf, g in zip(op_dag.inputs, grads))
    assert by_leaf[id(leaves[0])] is not None and by_leaf[id(leaves[1])] is None

    # no gradient is defined for the operator that consumes leaf 0; leaf 1 is reached through mul
    leaves, op_dag, grads, _ = _backward(ac.NO_GRADIENT, wanted_leaves=[1])
    by_leaf = dict((id(leaf), g) for leaf, g in zip(op_dag.inputs, grads))
    assert by_leaf[id(leaves[0])] is None and by_leaf[id(leaves[1])] is not None
    assert 'no_gradient_scale' in '_'.join(_names([by_leaf[id(leaves[1])]], merged=False))


def test_wanted_gradient_through_an_operator_without_gradient_is_an_error():
    """A missing gradient definition must not turn into a silent None (which autograd reads as zero)."""
    with pytest.raises(ValueError, match='no_gradient_scale'):
        _backward(ac.NO_GRADIENT, wanted_leaves=[0, 1])
    with pytest.raises(ValueError, match='no_gradient_scale'):
        _backward(ac.NO_GRADIENT, wanted_leaves=[0])


def test_unused_output_gets_a_zero_gradient_operator():
    a = np.random.rand(6)
    b = np.random.rand(6)
    y0, y1, y2 = (ac.fan_out(a, b)[k] for k in range(3))
    op_dag = _build_op_dag(y1)
    grads, placeholders = autograd.build_backward(op_dag, [True, True])
    assert len(placeholders) == 1
    names = _names([g for g in grads if g is not None], merged=False)
    assert names.count('gradient_zeros') == 2 and 'fan_out_grad' in names


def test_fan_out_contributions_are_summed():
    case = ac.CASE_BY_NAME['fan_out_fan_in']
    leaves, op_dag, grads, placeholders = _backward(case)
    assert len(placeholders) == 4
    names = _names(grads, merged=False)
    # y1 receives its own output gradient plus one from fan_in; y2 two from fan_in
    assert names.count('gradient_sum') == 2
    assert names.count('fan_in_grad') == 1 and names.count('fan_out_grad') == 1


def test_as_torch_argument_errors():
    with pytest.raises(ValueError):
        autograd.as_torch(stdops.tanh(np.zeros(4)), math_mode='sloppy')
