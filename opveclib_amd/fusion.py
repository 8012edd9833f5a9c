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
* expressions that become unused are removed by a reachability pass instead of index-set arithmetic;
* a producer whose single store permutes its workgroup over the tensor (``out[(p + 1) % n] = ...``, a transposed
  store) merges with an element-wise consumer that reads the tensor at its own position: the consumer's body runs
  in the producer's worker with the producer's store index as its position ("adopted position", `_edge_adoption`).
  The reference rejects such edges (rule 4), so its shift -> expm1 chain stays two operators.
"""

import hashlib
from collections import namedtuple

from . import language as lang
from .local import version, logger
from .operator import _op_hash, _freeze_op


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


def _reads_tensor_data(dag, index):
    """True when the sub-DAG of ``index`` reads an operator input (an index that depends on tensor contents)."""
    pending = [index]
    seen = set()
    while pending:
        cur = pending.pop()
        if cur in seen:
            continue
        seen.add(cur)
        if dag.expressions[cur].code in (lang.INPUT, lang.OUTPUT):
            return True
        pending.extend(dag.references[cur].operand_indices)
    return False


def _constant_int(dag, index):
    """Value of an integer literal (through casts)."""
    expr = dag.expressions[index]
    while expr.code == lang.CAST:
        index = dag.references[index].operand_indices[0]
        expr = dag.expressions[index]
    if expr.code != lang.CONST_SCALAR:
        raise ValueError('position component index is not a literal')
    for field in ('uint32_data', 'uint64_data', 'sint32_data', 'sint64_data'):
        data = getattr(expr, field)
        if len(data):
            return int(data[0])
    raise ValueError('position component index is not an integer literal')


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
# adopted positions
# ----------------------------------------------------------------------------------------------------------------------
def _product(values):
    result = 1
    for v in values:
        result *= int(v)
    return result


def _gcd(a, b):
    while b:
        a, b = b, a % b
    return a


def _index_form(info, idx):
    """('affine', aff, None) or ('mod', aff, n) for an index that is affine in the position, possibly reduced modulo a
    constant and wrapped in casts / multiplications by one / additions of zero; else None."""
    aff = info.affine.get(idx)
    if aff is not None:
        return ('affine', aff, None) if aff.only_position() else None
    node = info.nodes[idx]
    if node.code == lang.CAST and len(node.ops) == 1:
        return _index_form(info, node.ops[0])
    if node.code == lang.MULTIPLY:
        for a, b in ((0, 1), (1, 0)):
            if info._literal_int(node.ops[b]) == 1:
                return _index_form(info, node.ops[a])
        return None
    if node.code == lang.ADD:
        for a, b in ((0, 1), (1, 0)):
            if info._literal_int(node.ops[b]) == 0:
                return _index_form(info, node.ops[a])
        return None
    if node.code == lang.MODULO:
        n = info._literal_int(node.ops[1])
        inner = _index_form(info, node.ops[0])
        if n is not None and 0 < n <= 2 ** 31 and inner is not None and inner[0] == 'affine' and inner[1].lo >= 0:
            return ('mod', inner[1], n)
    return None


def _is_bijection(form, workgroup_shape, size):
    """Does the index form map the workgroup one-to-one onto 0 .. size-1?"""
    kind, aff, n = form
    extents = dict((('p', k), int(d)) for k, d in enumerate(workgroup_shape))
    moving = [s for s, d in extents.items() if d > 1]
    if any(s not in aff.coeffs for s in moving):
        return False
    coeffs = dict((s, c) for s, c in aff.coeffs.items() if extents[s] > 1)
    if kind == 'mod':
        # (a * p + c) mod n over p = 0 .. n-1 with gcd(a, n) = 1
        if n != size or len(coeffs) != 1:
            return False
        (sym, a), = coeffs.items()
        return extents[sym] == n and _gcd(a % n, n) == 1
    # a mixed-radix numbering: coefficients are the strides of some ordering of the position components
    if aff.const != 0:
        return False
    running = 1
    for sym, c in sorted(coeffs.items(), key=lambda item: item[1]):
        if c != running:
            return False
        running *= extents[sym]
    return running == size


def _is_own_position_index(aff, shape):
    """Is the affine form the row-major flat index of the worker's own position in a workgroup of this shape?"""
    if aff is None or aff.const != 0 or not aff.only_position():
        return False
    strides = [_product(shape[k + 1:]) for k in range(len(shape))]
    for k, extent in enumerate(shape):
        if extent > 1 and aff.coeff(('p', k)) != strides[k]:
            return False
    return all(sym[1] < len(shape) for sym in aff.coeffs)


def _edge_adoption(to_dag, in_expr_index, from_dag, out_expr_index):
    """
    The producer's store index expression when the consumer can adopt it as its position, else None.  Conditions: the
    consumer is element-wise over the tensor (its workgroup is the tensor's shape and every read of the tensor uses the
    worker's own position), every store of the producer to the tensor uses one index expression, outside loops, and
    that index is a one-to-one map of the producer's workgroup onto the tensor.
    """
    from .hipgen.analysis import DagInfo
    shape = [int(d) for d in to_dag.expressions[in_expr_index].tensor_type.shape]
    size = _product(shape)
    if [int(d) for d in to_dag.workgroup_shape] != shape or _product(from_dag.workgroup_shape) != size:
        return None
    to_info = DagInfo(to_dag)
    reads = _accesses(to_dag, lang.READ_TENSOR, in_expr_index)
    if not reads:
        return None
    for read in reads:
        if not _is_own_position_index(to_info.affine.get(to_dag.references[read].operand_indices[1]), shape):
            return None
    writes = _accesses(from_dag, lang.ASSIGN_TENSOR, out_expr_index)
    if not writes:
        return None
    from_info = DagInfo(from_dag)
    store_index = from_dag.references[writes[0]].operand_indices[1]
    for write in writes:
        # several stores are fine when they go to the same element (branches of a conditional chain); the index must
        # not change between them, which a loop could make it do
        if from_info.in_loop[write] or \
                not _same_subtree(from_dag, store_index, from_dag, from_dag.references[write].operand_indices[1]):
            return None
    if from_dag.expressions[store_index].dtype != lang.UINT64 or _depends_on_variable(from_dag, store_index):
        return None
    form = _index_form(from_info, store_index)
    if form is None or not _is_bijection(form, from_dag.workgroup_shape, size):
        return None
    # A consumer that adopts a transposing index reads its other tensors transposed as well: measured on MI355X
    # (float32 [8192, 8192], transposed store + add of a second tensor) the merged kernel takes 446 us against 241 us
    # for the two separate ones, whereas a cyclic shift + multiply gains (137 us against 208 us).  Permutations of the
    # position components are therefore adopted only by consumers without further tensor inputs.
    transposing = form[0] == 'affine' and not _is_own_position_index(form[1], [int(d) for d in
                                                                              from_dag.workgroup_shape])
    if transposing and len(_io_indices(to_dag, lang.INPUT)) > 1:
        return None
    return store_index


# ----------------------------------------------------------------------------------------------------------------------
# candidate search
# ----------------------------------------------------------------------------------------------------------------------
def _edge_kind(ops, to_op_index, to_in_arg_index, in_ref):
    """
    How the edge qualifies: ('same', None) when producer and consumer index the tensor identically (the reference's
    rules), ('adopt', producer store index) when the consumer can adopt the producer's store index as its position,
    or (None, reason).
    """
    to_dag = ops[to_op_index]
    from_dag = ops[in_ref.op_index]
    in_expr_index = _io_indices(to_dag, lang.INPUT)[to_in_arg_index]
    out_expr_index = _io_indices(from_dag, lang.OUTPUT)[in_ref.op_output_index]

    def adopted(reason):
        if list(to_dag.expressions[in_expr_index].tensor_type.shape) == \
                list(from_dag.expressions[out_expr_index].tensor_type.shape):
            store_index = _edge_adoption(to_dag, in_expr_index, from_dag, out_expr_index)
            if store_index is not None:
                return 'adopt', store_index
        return None, reason

    if list(to_dag.workgroup_shape) != list(from_dag.workgroup_shape):
        return adopted('Non-matching workgroup shapes for ')
    if list(to_dag.expressions[in_expr_index].tensor_type.shape) != \
            list(from_dag.expressions[out_expr_index].tensor_type.shape):
        return None, 'Non-matching tensor shapes (broadcasting) for '

    writes = _accesses(from_dag, lang.ASSIGN_TENSOR, out_expr_index)
    if not writes:
        return None, 'No write to the producer output for '
    first_index = from_dag.references[writes[0]].operand_indices[1]
    if _depends_on_variable(from_dag, first_index):
        return None, 'Write index depends on a variable for '
    # An index computed from tensor contents never qualifies.  Input numbers are local to each operator, so equal
    # sub-DAGs of two operators may read different tensors (out[idx1[p]] = x[p] followed by y[p] = t[idx2[p]]); and
    # even with one index tensor the store need not be one-to-one, in which case the element a consumer reads was
    # written by another worker.
    if _reads_tensor_data(from_dag, first_index):
        return None, 'Write index depends on tensor contents for '
    for other in writes[1:]:
        if not _same_subtree(from_dag, first_index, from_dag, from_dag.references[other].operand_indices[1]):
            return None, 'Multiple write patterns to the producer output for '
    for read in _accesses(to_dag, lang.READ_TENSOR, in_expr_index):
        read_index = to_dag.references[read].operand_indices[1]
        if _reads_tensor_data(to_dag, read_index):
            return None, 'Read index depends on tensor contents for '
        if not _same_subtree(from_dag, first_index, to_dag, read_index):
            return adopted('No-matching read/write index pattern for ')
    return 'same', None


def _edge_merge_ref(ops, to_op_index, to_in_arg_index, in_ref):
    """Return the _MergeRef of this edge, or None (with the reason logged) when it does not qualify."""
    to_dag = ops[to_op_index]
    from_dag = ops[in_ref.op_index]
    where = '%s input [%d] and %s output [%d]' % (to_dag.name, to_in_arg_index, from_dag.name, in_ref.op_output_index)
    kind, detail = _edge_kind(ops, to_op_index, to_in_arg_index, in_ref)
    if kind is None:
        logger.info(detail + where)
        return None
    if kind == 'adopt':
        logger.info('Consumer adopts the producer\'s store index as its position for ' + where)
    return _MergeRef(to_op_index=to_op_index,
                     to_in_expr_index=_io_indices(to_dag, lang.INPUT)[to_in_arg_index],
                     to_in_arg_index=to_in_arg_index, from_op_index=in_ref.op_index,
                     from_out_expr_index=_io_indices(from_dag, lang.OUTPUT)[in_ref.op_output_index],
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
            edges = [(n, r) for n, r in enumerate(reference.input_refs) if not r.is_leaf]
            kinds = [_edge_kind(proto_op_dag.operators, to_op_index, n, r)[0] for n, r in edges]
            # a consumer that adopts the producer's store index as its position may take only that one tensor from it
            if 'adopt' in kinds and len(edges) != 1:
                continue
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
        # io_index has no meaning of its own on a VARIABLE: 1 marks the variable as standing for an operator's output
        # tensor, which is where the code generator's error analysis starts a new stage (hipgen/accuracy.py)
        var.io_index = 1
        return self.add(var, [zero_index])

    def add_uint64(self, value):
        const = lang.Expression()
        const.code = lang.CONST_SCALAR
        const.dtype = lang.UINT64
        const.uint64_data.append(int(value))
        return self.add(const, [])

    def add_binary(self, code, dtype, lhs, rhs):
        expr = lang.Expression()
        expr.code = code
        expr.dtype = dtype
        return self.add(expr, [lhs, rhs])

    def add_cast(self, dtype, operand):
        expr = lang.Expression()
        expr.code = lang.CAST
        expr.dtype = dtype
        return self.add(expr, [operand])

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


def _merge_expr_dags(to_expr_dag, from_expr_dag, plan, adopted_store_index=None):
    """
    Build the merged expression DAG (operator.py:1453-1666).

    :param adopted_store_index: expression index (in the producer) of the store index the consumer adopts as its
        position, or None for an ordinary merge in which both bodies share the worker's position

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
    adopted = {}                # position component k -> merged expression holding it
    own_index = set()
    flat = None
    if adopted_store_index is not None:
        shape = [int(d) for d in to_expr_dag.workgroup_shape]
        # The store index may have been computed inside a branch of the producer; it depends on the position and on
        # constants only, so a fresh copy at the top level of the merged body has the same value.
        copies = {}

        def clone(index):
            if index not in copies:
                expr = from_expr_dag.expressions[index]
                if expr.code == lang.POSITION:
                    copies[index] = from_map[index]
                else:
                    operands = [clone(o) for o in from_expr_dag.references[index].operand_indices]
                    copies[index] = b.add(expr, operands)
            return copies[index]

        flat = clone(adopted_store_index)
        # flat indices of the consumer's own position are the adopted index itself: no need to take it apart into
        # components and put it together again (and the merged store index keeps a form later merges recognise)
        from .hipgen.analysis import DagInfo
        to_info = DagInfo(to_expr_dag)
        own_index = set(n for n, e in enumerate(to_expr_dag.expressions)
                        if e.dtype == lang.UINT64 and not list(e.tensor_type.shape) and
                        e.code not in (lang.CONST_SCALAR, lang.VARIABLE) and
                        _is_own_position_index(to_info.affine.get(n), shape) and to_info.affine.get(n).coeffs)
        for k, extent in enumerate(shape):
            stride = _product(shape[k + 1:])
            value = flat
            if stride > 1:
                value = b.add_binary(lang.DIVIDE, lang.UINT64, value, b.add_uint64(stride))
            if k > 0:
                value = b.add_binary(lang.MODULO, lang.UINT64, value, b.add_uint64(extent))
            adopted[k] = b.add_cast(lang.UINT32, value)
    to_position = [n for n, e in enumerate(to_expr_dag.expressions) if e.code == lang.POSITION][0]
    for n, expr in enumerate(to_expr_dag.expressions):
        ops = to_expr_dag.references[n].operand_indices
        if expr.code == lang.POSITION:
            to_map[n] = merged_position
        elif adopted and expr.code == lang.READ_TENSOR and ops[0] == to_position:
            to_map[n] = adopted[_constant_int(to_expr_dag, ops[1])]
        elif adopted and n in own_index:
            to_map[n] = flat
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
    adopted_store_index = None
    for n, r in enumerate(refs[to_op_index].input_refs):
        if not r.is_leaf:
            kind, detail = _edge_kind(ops, to_op_index, n, r)
            if kind == 'adopt':
                adopted_store_index = detail
    merged_expr_dag, new_out_index = _merge_expr_dags(ops[to_op_index], ops[from_op_index], plan, adopted_store_index)
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


def _dag_key(proto_op_dag):
    """Content hash of an operator DAG from its operators' content names (computed once per traced operator) and
    the serialised wiring."""
    wiring = lang.OperatorDAG()
    wiring.dag_input_types.extend(proto_op_dag.dag_input_types)
    wiring.references.extend(proto_op_dag.references)
    wiring.dag_outputs.extend(proto_op_dag.dag_outputs)
    digest = hashlib.sha224()
    for op in proto_op_dag.operators:
        digest.update(_op_hash(op).encode('utf-8'))
    digest.update(wiring.SerializeToString())
    digest.update(version.encode('utf-8'))
    return digest.hexdigest()


def _merge_op_dag(proto_op_dag, grad_dags):
    """
    Merge operators until no candidate is left (operator.py:1672-2034); memoised by the hash of the input DAG.

    :param proto_op_dag: the operator DAG
    :param grad_dags: gradient DAGs per operator or None.  Merged gradient DAGs are not produced: the second element
        of the result is None whenever a merge happened.
    :return: (merged operator DAG, gradient DAGs or None)
    """
    key = _dag_key(proto_op_dag)
    if key in _merged_dag_registry:
        return _merged_dag_registry[key]

    merged = proto_op_dag
    pairs = _group_merge_refs(merged, _get_merge_refs_for_op_dag(merged))
    while pairs:
        to_op_index, from_op_index = pairs[0]
        logger.info('Merging ' + merged.operators[from_op_index].name + ' and ' + merged.operators[to_op_index].name)
        merged = _merge_pair(merged, to_op_index, from_op_index)
        pairs = _group_merge_refs(merged, _get_merge_refs_for_op_dag(merged))

    if merged is not proto_op_dag:
        for op in merged.operators:
            _freeze_op(op)
    result = (merged, grad_dags if merged is proto_op_dag else None)
    _merged_dag_registry[key] = result
    return result
