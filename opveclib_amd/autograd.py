"""
OVL operator DAGs as differentiable PyTorch functions.

The reference hands a DAG of OVL operators to its host framework one operator at a time, each with its serialised
gradient DAG, and lets the framework chain the gradients (``as_tensorflow``, opveclib/operator.py:2338-2412, gradient
registration at operator.py:87-121); when the optimizer merges two operators it also has to construct a gradient DAG
for the merged operator that recomputes the upstream operator inside it (operator.py:1701-1921).  Here the whole
requested DAG becomes ONE ``torch.autograd.Function``:

  forward   the (fused) operator DAG, evaluated on the leaf tensors;
  backward  a second OVL operator DAG, assembled from the per-operator gradient DAGs in reverse order: gradient
            contributions to one tensor are summed by a small OVL operator, forward operators whose outputs a gradient
            needs are simply inputs of that gradient's operators.  That DAG goes through the same optimizer, so the
            recomputation of fused-away intermediates and the gradient arithmetic end up in the same kernels - what
            the reference's merged gradient DAGs achieve, without a special case per merge.

Leaves may be torch tensors (differentiable when they require grad) or numpy arrays (constants).
"""

from . import language as lang
from .expression import TensorType, position_in, output_like, output
from .operator import (_Operator, OperatorOutput, _GradientPlaceholder, _build_op_dag, _resolve_output,
                       _normalise_output_list, operator, get_math_mode, MATH_MODES)


def _output_types(expr_dag):
    outs = sorted((e for e in expr_dag.expressions if e.code == lang.OUTPUT), key=lambda e: e.io_index)
    return [TensorType.from_proto(e.tensor_type) for e in outs]


def _reify(op_dag_proto, dag_inputs):
    """Turn a serialised operator DAG back into wired :class:`_Operator` objects; returns its outputs."""
    operators = []
    for op_index, expr_dag in enumerate(op_dag_proto.operators):
        op_inputs = []
        for ref in op_dag_proto.references[op_index].input_refs:
            if ref.is_leaf:
                op_inputs.append(dag_inputs[ref.dag_input_index])
            else:
                op_inputs.append(operators[ref.op_index][ref.op_output_index])
        operators.append(_Operator(expr_dag, _output_types(expr_dag), op_inputs, None, True, expr_dag.name))
    return [operators[ref.op_index][ref.op_output_index] for ref in op_dag_proto.dag_outputs]


@operator()
def gradient_sum(*args):
    """Element-wise sum of gradient contributions to one tensor (operator.py:1838-1851)."""
    out = output_like(args[0])
    pos = position_in(args[0].shape)
    total = args[0][pos]
    for arg in args[1:]:
        if arg.shape != args[0].shape or arg.dtype != args[0].dtype:
            raise TypeError('gradient contributions of one tensor must share its shape and dtype')
        total = total + arg[pos]
    out[pos] = total
    return out


@operator()
def gradient_zeros(shape=None, dtype=None):
    """The gradient of an output nobody differentiated through (operator.py:1853-1858)."""
    out = output(shape, dtype)
    pos = position_in(shape)
    out[pos] = 0
    return out


def _total(contributions, tensor_type):
    if not contributions:
        return gradient_zeros(shape=tensor_type.shape, dtype=tensor_type.dtype)[0]
    if len(contributions) == 1:
        return contributions[0]
    return gradient_sum(*contributions)[0]


def build_backward(op_dag, wanted):
    """
    :param op_dag: the forward ``_OperatorDAG`` (unmerged, as built from the requested outputs)
    :param wanted: one bool per forward DAG input: is its gradient needed?
    :return: (list with an operator output or None per forward DAG input, placeholders of the output gradients)
    """
    proto = op_dag.proto_dag
    ops = op_dag.operators
    pending = {}            # (id(operator), output index) -> [gradient contributions]
    out_grad_placeholders = []
    for ref in proto.dag_outputs:
        tensor_type = ops[ref.op_index].output_types[ref.op_output_index]
        placeholder = _GradientPlaceholder(tensor_type.shape, tensor_type.dtype)
        out_grad_placeholders.append(placeholder)
        pending.setdefault((id(ops[ref.op_index]), ref.op_output_index), []).append(placeholder)

    leaf_slot = dict((id(leaf), n) for n, leaf in enumerate(op_dag.inputs))
    leaf_contributions = [[] for _ in op_dag.inputs]
    # operators and leaves that a gradient reaches only to stop at an operator without a gradient definition
    blocked_ops = {}        # id(operator) -> name of the operator that stops the gradient
    blocked_leaves = {}     # leaf slot -> the same

    for op in reversed(ops):            # operators are sorted by depth, so consumers come before producers here
        received = [pending.get((id(op), k), []) for k in range(len(op.output_types))]
        stopped_by = blocked_ops.get(id(op))
        if op.grad_dag is None and any(received):
            stopped_by = op.name
        if stopped_by is not None:
            for cur_input in op.inputs:
                try:
                    resolved = _resolve_output(cur_input)
                except TypeError:
                    blocked_leaves.setdefault(leaf_slot[id(cur_input)], stopped_by)
                else:
                    blocked_ops.setdefault(id(resolved.parent), stopped_by)
        if op.grad_dag is None or not any(received):
            continue
        grad_inputs = list(op.inputs) + [_total(c, t) for c, t in zip(received, op.output_types)]
        input_grads = _reify(op.grad_dag, grad_inputs)
        for cur_input, cur_grad in zip(op.inputs, input_grads):
            try:
                resolved = _resolve_output(cur_input)
            except TypeError:
                leaf_contributions[leaf_slot[id(cur_input)]].append(cur_grad)
            else:
                pending.setdefault((id(resolved.parent), resolved.index), []).append(cur_grad)

    leaf_grads = []
    for n, leaf in enumerate(op_dag.inputs):
        if wanted[n] and n in blocked_leaves:
            raise ValueError('the gradient of input %d passes through operator "%s", which has no gradient defined'
                             % (n, blocked_leaves[n]))
        if wanted[n] and leaf_contributions[n]:
            leaf_grads.append(_total(leaf_contributions[n], TensorType.like(leaf)))
        else:
            leaf_grads.append(None)
    return leaf_grads, out_grad_placeholders


def _evaluate(outputs, substitutions, opt_level, options):
    """Run the DAG of ``outputs``; ``substitutions`` maps id(DAG input object) -> tensor to feed instead."""
    from .fusion import _merge_op_dag
    from . import runtime
    new_dag = _build_op_dag(*outputs)
    dag = new_dag.proto_dag
    if opt_level >= 3:
        dag, _ = _merge_op_dag(dag, None)
    feeds = [substitutions.get(id(x), x) for x in new_dag.inputs]
    return runtime.run_op_dag(dag, feeds, 1, timed=False, options=options)[0]


def as_torch(output_list, opt_level=3, math_mode=None):
    """
    Evaluate OVL operator outputs as PyTorch tensors that take part in ``torch.autograd``.

    :param output_list: an operator, an operator output, or a list of either; the DAG's leaf inputs are torch tensors
        on a HIP device (differentiable where they require grad) or numpy arrays (copied to the device, constant)
    :param opt_level: operators are fused when opt_level >= 3 (forward and backward)
    :param math_mode: 'exact', 'ulp2' or 'fast'; None uses the current default
    :return: one tensor for a single requested output, otherwise a list in request order
    :raises ValueError: at ``backward()`` time, if the gradient of an input that requires one passes through an
        operator that has no gradient defined
    """
    import torch

    if math_mode is None:
        math_mode = get_math_mode()
    if math_mode not in MATH_MODES:
        raise ValueError('math_mode must be one of ' + str(MATH_MODES))
    options = None if math_mode == 'exact' else {'math': math_mode}

    outputs = _normalise_output_list(output_list)
    op_dag = _build_op_dag(*outputs)
    leaves = op_dag.inputs
    device = None
    for leaf in leaves:
        if isinstance(leaf, torch.Tensor) and leaf.device.type == 'cuda':
            device = leaf.device
            break
    if device is None:
        device = torch.device('cuda', torch.cuda.current_device())
    leaf_tensors = [leaf if isinstance(leaf, torch.Tensor) else torch.from_numpy(leaf).to(device) for leaf in leaves]

    class _OvlDag(torch.autograd.Function):
        @staticmethod
        def forward(ctx, *tensors):
            substitutions = dict((id(leaf), t.detach()) for leaf, t in zip(leaves, tensors))
            results = _evaluate(outputs, substitutions, opt_level, options)
            ctx.save_for_backward(*tensors)
            integral = [r for r in results if not r.dtype.is_floating_point]
            if integral:
                ctx.mark_non_differentiable(*integral)
            return tuple(results)

        @staticmethod
        @torch.autograd.function.once_differentiable
        def backward(ctx, *grad_outputs):
            tensors = ctx.saved_tensors
            wanted = list(ctx.needs_input_grad)
            leaf_grads, placeholders = build_backward(op_dag, wanted)
            requested = [g for g in leaf_grads if g is not None]
            if not requested:
                return tuple(None for _ in tensors)
            substitutions = dict((id(leaf), t.detach()) for leaf, t in zip(leaves, tensors))
            for placeholder, grad, forward_out in zip(placeholders, grad_outputs, outputs):
                if grad is None:
                    tt = TensorType.like(_resolve_output(forward_out))
                    grad = torch.zeros(tt.shape, dtype=tt.dtype.as_torch(), device=device)
                substitutions[id(placeholder)] = grad.contiguous()
            values = _evaluate(requested, substitutions, opt_level, options)
            values = iter(values)
            return tuple(next(values) if g is not None else None for g in leaf_grads)

    results = _OvlDag.apply(*leaf_tensors)
    results = list(results)
    if len(results) == 1:
        return results[0]
    return results
