"""
The fusion optimizer: merges chains of parallel-for operators into one operator whose intermediates are worker-local
scalars, so that a fused chain becomes a single kernel launch with the intermediates held in registers.

Counterpart of the reference's opveclib/operator.py:809-2034 (``_merge_op_dag`` and helpers).  An operator-DAG edge
(producer output -> consumer input) qualifies when (operator.py:1202-1235)

  1. both operators have the same workgroup shape,
  2. the tensor has the same shape on both sides (no broadcast across the edge),
  3. every store of the producer to that output uses one and the same index expression, and
  4. every read of the consumer from that input uses an index expression structurally identical to it,

and a consumer is merged into a producer when all of its operator-produced inputs come from that one producer and all
of those edges qualify (operator.py:1248-1300).  The merged operator keeps the producer's body, turns each
internalised tensor into a VARIABLE (stores become variable assignments; tensors still needed by other operators or
requested as DAG outputs keep their store as well), then appends the consumer's body with its reads of the
internalised tensors rewired to the variables (operator.py:1453-1666).

Deliberate differences from the reference, none of which changes an operator's results:

* rule 3 accepts several stores with identical index expressions (the reference demands exactly one,
  operator.py:1217-1222), so producers that store under disjoint branches (expm1, log1p) fuse too;
* index expressions that depend on a VARIABLE (e.g. an ``arange`` loop counter) never qualify: a scalar cannot stand
  in for a tensor that is written and read at many indices by one worker (the reference lists such edges,
  test_operator_merge.py:213-223, although its merge would then read only the last value);
* rule 4 inspects the reads of the input that the edge actually feeds (the reference always inspects the consumer's
  first input because it indexes with ``dag_input_index``, operator.py:1194, 1226), and the producer of a consumer is
  its first operator-produced input (the reference takes ``input_refs[0].op_index`` even for a leaf, 1271);
* structural matching also compares dtypes and, for reads of input tensors inside an index, which input is read;
* an input tensor that producer and consumer both read becomes one argument of the merged operator;
* expressions that become unused are removed by a reachability pass instead of index-set arithmetic.
"""

import hashlib
from collections import namedtuple

from . import language as lang
from .local import version, logger


class _MergeRef(namedtuple('_MergeRef', ['to_op_index', 'to_in_expr_index', 'to_in_arg_index', 'from_op_index',
                                         'from_out_expr_index', 'from_out_arg_index'])):
    """
    One mergeable tensor edge of the operator DAG (operator.py:1116-1147): output ``from_out_arg_index`` of operator
    ``from_op_index`` (declared by expression ``from_out_expr_index`` of its DAG) feeds input ``to_in_arg_index`` of
    operator ``to_op_index`` (declared by expression ``to_in_expr_index`` of its DAG).
    """
    __slots__ = ()

    def same(self, ref):
        return tuple(self) == tuple(ref)


# ----------------------------------------------------------------------------------------------------------------------
# expression DAG helpers
# ----------------------------------------------------------------------------------------------------------------------
def _io_indices(expr_dag, code):
    """Expression indices of INPUT (or OUTPUT) declarations ordered by io_index."""
    found = [(e.io_index, n) for n, e in enumerate(expr_dag.expressions) if e.code == code]
    return [n for _, n in sorted(found)]


def _accesses(expr_dag, code, tensor_index):
    """Indices of READ_TENSOR / ASSIGN_TENSOR expressions whose tensor operand is ``tensor_index``."""
    return [n for n, e in enumerate(expr_dag.expressions)
            if e.code == code and expr_dag.references[n].operand_indices[0] == tensor_index]


_CONST_FIELDS = ('float_data', 'double_data', 'sint32_data', 'sint64_data', 'uint32_data', 'uint64_data')


def _same_subtree(dag0, index0, dag1, index1):
    """Structural equality of two expression sub-DAGs (codes, dtypes, constants, io indices, arity)."""
    pending = [(index0, index1)]
    seen = set()
    while pending:
        pair = pending.pop()
        if pair in seen:
            continue
        seen.add(pair)
        e0 = dag0.expressions[pair[0]]
        e1 = dag1.expressions[pair[1]]
        if e0.code != e1.code or e0.dtype != e1.dtype:
            return False
        if e0.code in (lang.CONST_SCALAR, lang.CONST_TENSOR, lang.POSITION):
            if e0.tensor_type != e1.tensor_type:
                return False
            for field in _CONST_FIELDS:
                if getattr(e0, field) != getattr(e1, field):
                    return False
        if e0.code in (lang.INPUT, lang.OUTPUT) and (e0.io_index != e1.io_index or e0.tensor_type != e1.tensor_type):
            return False
        ops0 = dag0.references[pair[0]].operand_indices
        ops1 = dag1.references[pair[1]].operand_indices
        if len(ops0) != len(ops1):
            return False
        pending.extend(zip(ops0, ops1))
    return True


def _depends_on_variable(dag, index):
    pending = [index]
    seen = set()
    while pending:
        cur = pending.pop()
        if cur in seen:
            continue
        seen.add(cur)
        if dag.expressions[cur].code in (lang.VARIABLE, lang.TENSOR):
            return True
        pending.extend(dag.references[cur].operand_indices)
    return False


# ----------------------------------------------------------------------------------------------------------------------
# candidate search
# ----------------------------------------------------------------------------------------------------------------------
def _edge_merge_ref(ops, to_op_index, to_in_arg_index, in_ref):
    """Return the _MergeRef of this edge, or None (with the reason logged) when it does not qualify."""
    to_dag = ops[to_op_index]
    from_dag = ops[in_ref.op_index]
    where = '%s input [%d] and %s output [%d]' % (to_dag.name, to_in_arg_index, from_dag.name, in_ref.op_output_index)

    if list(to_dag.workgroup_shape) != list(from_dag.workgroup_shape):
        logger.info('Non-matching workgroup shapes for ' + where)
        return None

    in_expr_index = _io_indices(to_dag, lang.INPUT)[to_in_arg_index]
    out_expr_index = _io_indices(from_dag, lang.OUTPUT)[in_ref.op_output_index]
    if list(to_dag.expressions[in_expr_index].tensor_type.shape) != \
            list(from_dag.expressions[out_expr_index].tensor_type.shape):
        logger.info('Non-matching tensor shapes (broadcasting) for ' + where)
        return None

    writes = _accesses(from_dag, lang.ASSIGN_TENSOR, out_expr_index)
    if not writes:
        logger.info('No write to %s output [%d]' % (from_dag.name, in_ref.op_output_index))
        return None
    first_index = from_dag.references[writes[0]].operand_indices[1]
    if _depends_on_variable(from_dag, first_index):
        logger.info('Write index depends on a variable for ' + where)
        return None
    for other in writes[1:]:
        if not _same_subtree(from_dag, first_index, from_dag, from_dag.references[other].operand_indices[1]):
            logger.info('Multiple write patterns to %s output [%d]' % (from_dag.name, in_ref.op_output_index))
            return None

    for read in _accesses(to_dag, lang.READ_TENSOR, in_expr_index):
        if not _same_subtree(from_dag, first_index, to_dag, to_dag.references[read].operand_indices[1]):
            logger.info('No-matching read/write index pattern for ' + where)
            return None

    return _MergeRef(to_op_index=to_op_index, to_in_expr_index=in_expr_index, to_in_arg_index=to_in_arg_index,
                     from_op_index=in_ref.op_index, from_out_expr_index=out_expr_index,
                     from_out_arg_index=in_ref.op_output_index)


def _get_merge_refs_for_op_dag(proto_op_dag):
    """
    All mergeable tensor edges among the operators that the DAG outputs depend on (operator.py:1150-1245), found by
    walking from every DAG output toward the inputs; duplicates removed, discovery order kept.
    """
    ops = proto_op_dag.operators
    refs = proto_op_dag.references
    merge_refs = []
    visited = set()
    frontier = [out.op_index for out in proto_op_dag.dag_outputs]
    while frontier:
        to_op_index = frontier.pop(0)
        if to_op_index in visited:
            continue
        visited.add(to_op_index)
        for to_in_arg_index, in_ref in enumerate(refs[to_op_index].input_refs):
            if in_ref.is_leaf:
                continue
            frontier.append(in_ref.op_index)
            merge_ref = _edge_merge_ref(ops, to_op_index, to_in_arg_index, in_ref)
            if merge_ref is not None and merge_ref not in merge_refs:
                merge_refs.append(merge_ref)
    return merge_refs


def _group_merge_refs(proto_op_dag, merge_refs):
    """
    (to-op, from-op) pairs that can be merged (operator.py:1248-1300): every operator-produced input of the to-op
    comes from the one from-op and every such edge is in ``merge_refs``; inputs that are DAG leaves are unconstrained.
    """
    mergeable = set((m.to_op_index, m.to_in_arg_index, m.from_op_index, m.from_out_arg_index) for m in merge_refs)
    pairs = []
    for to_op_index, reference in enumerate(proto_op_dag.references):
        producers = set(r.op_index for r in reference.input_refs if not r.is_leaf)
        if len(producers) != 1:
            continue
        from_op_index = producers.pop()
        if all(r.is_leaf or (to_op_index, n, from_op_index, r.op_output_index) in mergeable
               for n, r in enumerate(reference.input_refs)):
            pairs.append((to_op_index, from_op_index))
    return pairs


# ----------------------------------------------------------------------------------------------------------------------
# merging two expression DAGs
# ----------------------------------------------------------------------------------------------------------------------
_ROOT_CODES = (lang.INPUT, lang.OUTPUT, lang.POSITION, lang.ASSIGN_VARIABLE, lang.ASSIGN_TENSOR, lang.RANGE,
               lang.ENDRANGE, lang.IF, lang.ELSEIF, lang.ELSE, lang.ENDIF)


class _Builder(object):
    """Accumulates (expression, operand list) pairs of the merged DAG."""

    def __init__(self):
        self.exprs = []
        self.operands = []

    def add(self, expr, operands):
        copy = lang.Expression()
        copy.CopyFrom(expr)
        self.exprs.append(copy)
        self.operands.append(list(operands))
        return len(self.exprs) - 1

    def add_zero_variable(self, dtype):
        """``T v = 0;`` as a CONST_SCALAR of the tensor's dtype feeding a VARIABLE (operator.py:1409-1450)."""
        zero = lang.Expression()
        zero.code = lang.CONST_SCALAR
        zero.dtype = dtype
        if dtype == lang.FLOAT64:
            zero.double_data.append(0.0)
        elif dtype in (lang.FLOAT32, lang.FLOAT16):
            zero.float_data.append(0.0)
        elif dtype == lang.UINT64:
            zero.uint64_data.append(0)
        elif dtype == lang.INT64:
            zero.sint64_data.append(0)
        elif dtype in (lang.UINT32, lang.UINT16, lang.UINT8):
            zero.uint32_data.append(0)
        elif dtype in (lang.INT32, lang.INT16, lang.INT8):
            zero.sint32_data.append(0)
        else:
            raise TypeError('Tried to add variable for unknown type ' + str(dtype))
        zero_index = self.add(zero, [])
        var = lang.Expression()
        var.code = lang.VARIABLE
        var.dtype = dtype
        return self.add(var, [zero_index])

    def sweep(self):
        """Drop value expressions nothing depends on; returns (exprs, operands) with operands renumbered."""
        live = set()
        pending = [n for n, e in enumerate(self.exprs) if e.code in _ROOT_CODES]
        while pending:
            cur = pending.pop()
            if cur in live:
                continue
            live.add(cur)
            pending.extend(self.operands[cur])
        new_index = {}
        exprs = []
        operands = []
        for n, e in enumerate(self.exprs):
            if n in live:
                new_index[n] = len(exprs)
                exprs.append(e)
                operands.append(self.operands[n])
        operands = [[new_index[o] for o in ops] for ops in operands]
        return exprs, operands


_MergePlan = namedtuple('_MergePlan', [
    'internal',          # {to-op input arg index: from-op output arg index} for edges turned into variables
    'keep_output',       # set of from-op output arg indices that stay outputs of the merged operator
    'shared_inputs',     # {to-op input arg index: from-op input arg index} for inputs both operators read
])


def _plan_merge(proto_op_dag, to_op_index, from_op_index):
    refs = proto_op_dag.references
    to_refs = refs[to_op_index].input_refs
    from_refs = refs[from_op_index].input_refs

    internal = {}
    shared_inputs = {}
    for arg, r in enumerate(to_refs):
        if not r.is_leaf and r.op_index == from_op_index:
            internal[arg] = r.op_output_index
            continue
        for from_arg, fr in enumerate(from_refs):
            same_leaf = r.is_leaf and fr.is_leaf and r.dag_input_index == fr.dag_input_index
            same_edge = (not r.is_leaf) and (not fr.is_leaf) and r.op_index == fr.op_index and \
                r.op_output_index == fr.op_output_index
            if same_leaf or same_edge:
                shared_inputs[arg] = from_arg
                break

    # producer outputs that something other than the consumer still needs
    needed = set()
    for out in proto_op_dag.dag_outputs:
        if out.op_index == from_op_index:
            needed.add(out.op_output_index)
    for op_index, reference in enumerate(refs):
        if op_index in (to_op_index, from_op_index):
            continue
        for r in reference.input_refs:
            if not r.is_leaf and r.op_index == from_op_index:
                needed.add(r.op_output_index)

    num_from_outputs = len(_io_indices(proto_op_dag.operators[from_op_index], lang.OUTPUT))
    consumed = set(internal.values())
    keep_output = set(k for k in range(num_from_outputs) if k in needed or k not in consumed)
    return _MergePlan(internal=internal, keep_output=keep_output, shared_inputs=shared_inputs)


def _merge_expr_dags(to_expr_dag, from_expr_dag, plan):
    """
    Build the merged expression DAG (operator.py:1453-1666).

    Inputs of the result: the producer's inputs, then the consumer's inputs that are neither internalised nor shared.
    Outputs of the result: the producer's kept outputs (original order), then the consumer's outputs.
    """
    b = _Builder()

    from_out_exprs = _io_indices(from_expr_dag, lang.OUTPUT)
    out_arg_of_expr = dict((n, k) for k, n in enumerate(from_out_exprs))
    internal_outs = set(plan.internal.values())
    new_out_index = {}
    for k in range(len(from_out_exprs)):
        if k in plan.keep_output:
            new_out_index[k] = len(new_out_index)

    # ---- producer body ----
    from_map = {}               # producer expression index -> merged index
    var_of_out = {}             # producer output arg index -> merged VARIABLE index
    from_input_merged = {}      # producer input arg index -> merged INPUT index
    for n, expr in enumerate(from_expr_dag.expressions):
        ops = from_expr_dag.references[n].operand_indices
        if expr.code == lang.OUTPUT:
            k = out_arg_of_expr[n]
            if k in plan.keep_output:
                merged = b.add(expr, [])
                b.exprs[merged].io_index = new_out_index[k]
                from_map[n] = merged
            if k in internal_outs:
                var_of_out[k] = b.add_zero_variable(expr.tensor_type.dtype)
            continue
        if expr.code == lang.ASSIGN_TENSOR and ops[0] in out_arg_of_expr:
            k = out_arg_of_expr[ops[0]]
            if k in plan.keep_output:
                from_map[n] = b.add(expr, [from_map[o] for o in ops])
            if k in internal_outs:
                assign = lang.Expression()
                assign.code = lang.ASSIGN_VARIABLE
                b.add(assign, [var_of_out[k], from_map[ops[2]]])
            continue
        from_map[n] = b.add(expr, [from_map[o] for o in ops])
        if expr.code == lang.INPUT:
            from_input_merged[expr.io_index] = from_map[n]

    merged_position = from_map[[n for n, e in enumerate(from_expr_dag.expressions) if e.code == lang.POSITION][0]]
    num_inputs = len(from_input_merged)
    num_outputs = len(new_out_index)

    # ---- consumer body ----
    to_in_exprs = _io_indices(to_expr_dag, lang.INPUT)
    in_arg_of_expr = dict((n, k) for k, n in enumerate(to_in_exprs))
    to_map = {}
    for n, expr in enumerate(to_expr_dag.expressions):
        ops = to_expr_dag.references[n].operand_indices
        if expr.code == lang.POSITION:
            to_map[n] = merged_position
        elif expr.code == lang.INPUT:
            arg = in_arg_of_expr[n]
            if arg in plan.internal:
                continue                                    # its reads are rewired below
            if arg in plan.shared_inputs:
                to_map[n] = from_input_merged[plan.shared_inputs[arg]]
                continue
            to_map[n] = b.add(expr, [])
            b.exprs[to_map[n]].io_index = num_inputs
            num_inputs += 1
        elif expr.code == lang.READ_TENSOR and in_arg_of_expr.get(ops[0]) in plan.internal:
            to_map[n] = var_of_out[plan.internal[in_arg_of_expr[ops[0]]]]
        elif expr.code == lang.OUTPUT:
            to_map[n] = b.add(expr, [])
            b.exprs[to_map[n]].io_index = num_outputs
            num_outputs += 1
        else:
            # operands that only fed the index of a rewired read are never referenced again and may be missing
            to_map[n] = b.add(expr, [to_map[o] for o in ops])

    exprs, operands = b.sweep()
    merged = lang.ExpressionDAG()
    for expr, ops in zip(exprs, operands):
        merged.expressions.add().CopyFrom(expr)
        merged.references.add().operand_indices.extend(ops)
    merged.workgroup_shape.extend(from_expr_dag.workgroup_shape)
    merged.name = from_expr_dag.name + '_' + to_expr_dag.name
    return merged, new_out_index


def _merge_pair(proto_op_dag, to_op_index, from_op_index):
    """Return a new OperatorDAG in which the to-op has been merged into the from-op."""
    ops = proto_op_dag.operators
    refs = proto_op_dag.references
    plan = _plan_merge(proto_op_dag, to_op_index, from_op_index)
    merged_expr_dag, new_out_index = _merge_expr_dags(ops[to_op_index], ops[from_op_index], plan)
    num_kept = len(new_out_index)

    def new_op_index(op_index):
        if op_index == to_op_index:
            return from_op_index
        return op_index - 1 if op_index > to_op_index else op_index

    def new_output_index(op_index, output_index):
        if op_index == from_op_index:
            return new_out_index[output_index]
        if op_index == to_op_index:
            return num_kept + output_index
        return output_index

    result = lang.OperatorDAG()
    for i, op in enumerate(ops):
        if i == from_op_index:
            result.operators.add().CopyFrom(merged_expr_dag)
        elif i != to_op_index:
            result.operators.add().CopyFrom(op)

    def copy_ref(dst_list, r):
        dst = dst_list.input_refs.add()
        dst.is_leaf = r.is_leaf
        dst.dag_input_index = r.dag_input_index
        if not r.is_leaf:
            dst.op_index = new_op_index(r.op_index)
            dst.op_output_index = new_output_index(r.op_index, r.op_output_index)

    for i, reference in enumerate(refs):
        if i == to_op_index:
            continue
        ref_list = result.references.add()
        for r in reference.input_refs:
            copy_ref(ref_list, r)
        if i == from_op_index:
            for arg, r in enumerate(refs[to_op_index].input_refs):
                if arg not in plan.internal and arg not in plan.shared_inputs:
                    copy_ref(ref_list, r)

    for out in proto_op_dag.dag_outputs:
        dst = result.dag_outputs.add()
        dst.op_index = new_op_index(out.op_index)
        dst.op_output_index = new_output_index(out.op_index, out.op_output_index)

    for tt in proto_op_dag.dag_input_types:
        result.dag_input_types.add().CopyFrom(tt)
    return result


# ----------------------------------------------------------------------------------------------------------------------
# driver
# ----------------------------------------------------------------------------------------------------------------------
_merged_dag_registry = {}


def _merge_op_dag(proto_op_dag, grad_dags):
    """
    Merge operators until no candidate is left (operator.py:1672-2034); memoised by the hash of the input DAG.

    :param proto_op_dag: the operator DAG
    :param grad_dags: gradient DAGs per operator or None.  Merged gradient DAGs are not produced: the second element
        of the result is None whenever a merge happened.
    :return: (merged operator DAG, gradient DAGs or None)
    """
    key = hashlib.sha224(proto_op_dag.SerializeToString() + version.encode('utf-8')).hexdigest()
    if key in _merged_dag_registry:
        return _merged_dag_registry[key]

    merged = proto_op_dag
    pairs = _group_merge_refs(merged, _get_merge_refs_for_op_dag(merged))
    while pairs:
        to_op_index, from_op_index = pairs[0]
        logger.info('Merging ' + merged.operators[from_op_index].name + ' and ' + merged.operators[to_op_index].name)
        merged = _merge_pair(merged, to_op_index, from_op_index)
        pairs = _group_merge_refs(merged, _get_merge_refs_for_op_dag(merged))

    result = (merged, grad_dags if merged is proto_op_dag else None)
    _merged_dag_registry[key] = result
    return result
