"""
Static analysis of an expression DAG for the HIP code generator.

Turns the serialised DAG (the form the reference's generator walks in opveclib/expression.py:521-566) into a node
list, parses its control flow into a block tree, and derives for every integer-valued expression an affine form in
the workgroup position components whenever one exists.  The affine forms tell the kernel templates which tensor
accesses are contiguous along the last workgroup dimension (vector loads/stores), which are transposed, which are
uniform, and which must stay scalar.
"""

from .. import language as lang

INT_RANGE = {
    lang.INT8: (-2 ** 7, 2 ** 7 - 1), lang.INT16: (-2 ** 15, 2 ** 15 - 1),
    lang.INT32: (-2 ** 31, 2 ** 31 - 1), lang.INT64: (-2 ** 63, 2 ** 63 - 1),
    lang.UINT8: (0, 2 ** 8 - 1), lang.UINT16: (0, 2 ** 16 - 1),
    lang.UINT32: (0, 2 ** 32 - 1), lang.UINT64: (0, 2 ** 64 - 1)}

ITEMSIZE = {lang.FLOAT16: 2, lang.FLOAT32: 4, lang.FLOAT64: 8, lang.INT8: 1, lang.INT16: 2, lang.INT32: 4,
            lang.INT64: 8, lang.UINT8: 1, lang.UINT16: 2, lang.UINT32: 4, lang.UINT64: 8}


class Node(object):
    """One expression of the DAG with its operands resolved to node indices."""
    __slots__ = ('idx', 'code', 'dtype', 'shape', 'io_index', 'data', 'ops')

    def __init__(self, idx, expr, ops):
        self.idx = idx
        self.code = expr.code
        self.ops = list(ops)
        self.io_index = expr.io_index
        if expr.code in (lang.INPUT, lang.OUTPUT, lang.CONST_TENSOR, lang.POSITION, lang.TENSOR):
            self.dtype = expr.tensor_type.dtype
            self.shape = list(expr.tensor_type.shape)
        else:
            self.dtype = expr.dtype
            self.shape = None
        self.data = None
        if expr.code == lang.POSITION:
            self.data = list(expr.uint32_data)
        elif expr.code in (lang.CONST_SCALAR, lang.CONST_TENSOR):
            self.data = list(const_data(expr, self.dtype))

    @property
    def size(self):
        n = 1
        for d in self.shape:
            n *= d
        return n


def const_data(expr, dtype):
    if dtype in (lang.FLOAT16, lang.FLOAT32):
        return expr.float_data
    if dtype == lang.FLOAT64:
        return expr.double_data
    if dtype in (lang.INT8, lang.INT16, lang.INT32):
        return expr.sint32_data
    if dtype == lang.INT64:
        return expr.sint64_data
    if dtype in (lang.UINT8, lang.UINT16, lang.UINT32):
        return expr.uint32_data
    return expr.uint64_data


class Affine(object):
    """
    value = const + sum(coeff[s] * s) over symbols s, exact in unbounded integers, together with the value range
    [lo, hi] it takes over the whole workgroup.  Symbols are ('p', k) for workgroup position component k and
    ('v', node) for the counter of a counted loop with constant bounds.
    """
    __slots__ = ('coeffs', 'const', 'lo', 'hi')

    def __init__(self, coeffs, const, lo, hi):
        self.coeffs = dict((s, c) for s, c in coeffs.items() if c != 0)
        self.const = const
        self.lo = lo
        self.hi = hi

    @staticmethod
    def constant(value):
        return Affine({}, value, value, value)

    @staticmethod
    def symbol(sym, lo, hi):
        return Affine({sym: 1}, 0, lo, hi)

    def is_constant(self):
        return not self.coeffs

    def signature(self):
        return (tuple(sorted(self.coeffs.items())), self.const)

    def coeff(self, sym):
        return self.coeffs.get(sym, 0)

    def only_position(self):
        return all(s[0] == 'p' for s in self.coeffs)


def _combine(a, b, sign, ranges):
    coeffs = dict(a.coeffs)
    for s, c in b.coeffs.items():
        coeffs[s] = coeffs.get(s, 0) + sign * c
    return _with_range(coeffs, a.const + sign * b.const, ranges)


def _with_range(coeffs, const, ranges):
    lo = hi = const
    for s, c in coeffs.items():
        s_lo, s_hi = ranges[s]
        if c >= 0:
            lo += c * s_lo
            hi += c * s_hi
        else:
            lo += c * s_hi
            hi += c * s_lo
    return Affine(coeffs, const, lo, hi)


class Item(object):
    """Element of a block: a plain statement node, a conditional chain or a counted loop."""
    __slots__ = ('kind', 'node', 'branches', 'has_else', 'body')

    def __init__(self, kind, node=None, branches=None, has_else=False, body=None):
        self.kind = kind            # 'stmt' | 'if' | 'loop'
        self.node = node            # node index (stmt: the node, loop: the RANGE node)
        self.branches = branches    # if: list of (condition node index or None, [Item])
        self.has_else = has_else
        self.body = body            # loop: [Item]


class DagInfo(object):
    """Parsed DAG: nodes, inputs/outputs by io_index, workgroup shape, block tree and affine forms."""

    def __init__(self, dag):
        self.name = dag.name
        self.nodes = [Node(n, e, dag.references[n].operand_indices) for n, e in enumerate(dag.expressions)]
        self.workgroup_shape = list(dag.workgroup_shape)
        self.num_workers = 1
        for d in self.workgroup_shape:
            self.num_workers *= d

        self.inputs = {}
        self.outputs = {}
        self.position = None
        for node in self.nodes:
            if node.code == lang.INPUT:
                self.inputs[node.io_index] = node
            elif node.code == lang.OUTPUT:
                self.outputs[node.io_index] = node
            elif node.code == lang.POSITION:
                self.position = node
        if self.position is None:
            raise ValueError('expression DAG has no POSITION expression')
        if sorted(self.inputs) != list(range(len(self.inputs))) or \
                sorted(self.outputs) != list(range(len(self.outputs))):
            raise ValueError('expression DAG inputs/outputs are not numbered contiguously')

        self.depth = {}             # node index -> nesting depth of control flow (0 = top level of the worker)
        self.in_loop = {}           # node index -> True when inside a counted loop
        self.tree = self._parse_blocks()
        # variables that anything writes after their declaration (an assignment, or a loop that counts in them)
        self.written_variables = set(n.ops[0] for n in self.nodes if n.code in (lang.ASSIGN_VARIABLE, lang.RANGE))
        self.loop_counters = self._find_loop_counters()
        self.ranges = {}
        for k, extent in enumerate(self.workgroup_shape):
            self.ranges[('p', k)] = (0, extent - 1)
        for var, (lo, hi) in self.loop_counters.items():
            self.ranges[('v', var)] = (lo, hi)
        self.affine = {}
        for node in self.nodes:
            self.affine[node.idx] = self._affine_of(node)

    # -- control flow --------------------------------------------------------------------------------------------
    def _parse_blocks(self):
        pos = [0]
        nodes = self.nodes

        def block(depth, looping, terminators):
            items = []
            while pos[0] < len(nodes):
                node = nodes[pos[0]]
                if node.code in terminators:
                    return items
                pos[0] += 1
                self.depth[node.idx] = depth
                self.in_loop[node.idx] = looping
                if node.code == lang.IF:
                    branches = [(node.ops[0], block(depth + 1, looping, (lang.ELSEIF, lang.ELSE, lang.ENDIF)))]
                    has_else = False
                    while True:
                        closer = nodes[pos[0]]
                        pos[0] += 1
                        self.depth[closer.idx] = depth
                        self.in_loop[closer.idx] = looping
                        if closer.code == lang.ELSEIF:
                            branches.append((closer.ops[0],
                                             block(depth + 1, looping, (lang.ELSEIF, lang.ELSE, lang.ENDIF))))
                        elif closer.code == lang.ELSE:
                            has_else = True
                            branches.append((None, block(depth + 1, looping, (lang.ENDIF,))))
                        else:
                            break
                    items.append(Item('if', node=node.idx, branches=branches, has_else=has_else))
                elif node.code == lang.RANGE:
                    body = block(depth + 1, True, (lang.ENDRANGE,))
                    closer = nodes[pos[0]]
                    pos[0] += 1
                    self.depth[closer.idx] = depth
                    self.in_loop[closer.idx] = looping
                    items.append(Item('loop', node=node.idx, body=body))
                else:
                    items.append(Item('stmt', node=node.idx))
            if terminators:
                raise ValueError('unterminated control flow block in expression DAG')
            return items

        return block(0, False, ())

    def _find_loop_counters(self):
        """VARIABLEs that are only ever written by one RANGE with constant start/stop and a constant positive step:
        {variable node: (lowest value, highest value inside the loop body)}."""
        assigned = set()
        for node in self.nodes:
            if node.code == lang.ASSIGN_VARIABLE:
                assigned.add(node.ops[0])
        counters = {}
        used = {}
        for node in self.nodes:
            if node.code == lang.RANGE:
                used[node.ops[0]] = used.get(node.ops[0], 0) + 1
        for node in self.nodes:
            if node.code != lang.RANGE:
                continue
            var = node.ops[0]
            if var in assigned or used[var] != 1:
                continue
            bounds = [self._literal_int(o) for o in node.ops[1:]]
            if any(b is None for b in bounds):
                continue
            start, stop, step = bounds
            if step <= 0 or stop <= start:
                continue
            last = start + ((stop - 1 - start) // step) * step
            counters[var] = (start, last)
        return counters

    def _literal_int(self, idx):
        """Integer value of a literal or a chain of casts and never-written variables ending in a literal (the
        reference's dot-product test keeps its loop bound in a variable, opveclib/test/test_dot_product.py:34-36),
        else None."""
        node = self.nodes[idx]
        chain = []
        while node.code == lang.CAST or (node.code == lang.VARIABLE and node.idx not in self.written_variables):
            if node.dtype not in INT_RANGE:
                return None
            chain.append(node.dtype)
            node = self.nodes[node.ops[0]]
        if node.code == lang.CONST_SCALAR and node.dtype in INT_RANGE:
            value = int(node.data[0])
            # a literal that does not fit a type on the way (variable(300, uint8)) is not the value the code sees
            for dtype in chain + [node.dtype]:
                lo, hi = INT_RANGE[dtype]
                if not lo <= value <= hi:
                    return None
            return value
        return None

    # -- affine forms --------------------------------------------------------------------------------------------
    def _fits(self, aff, dtype):
        lo, hi = INT_RANGE[dtype]
        return aff is not None and lo <= aff.lo and aff.hi <= hi

    def _affine_of(self, node):
        code = node.code
        if node.shape is not None or node.dtype not in INT_RANGE:
            return None
        get = self.affine.get
        if code == lang.CONST_SCALAR:
            return Affine.constant(int(node.data[0]))
        if code == lang.READ_TENSOR:
            tensor = self.nodes[node.ops[0]]
            index = get(node.ops[1])
            if tensor.code == lang.POSITION and index is not None and index.is_constant():
                k = index.const
                return Affine.symbol(('p', k), 0, self.workgroup_shape[k] - 1)
            return None
        if code == lang.VARIABLE:
            if node.idx in self.loop_counters:
                lo, hi = self.loop_counters[node.idx]
                return Affine.symbol(('v', node.idx), lo, hi)
            return None
        if code == lang.CAST:
            src = get(node.ops[0])
            if self.nodes[node.ops[0]].dtype not in INT_RANGE:
                return None
            return src if self._fits(src, node.dtype) else None
        if code in (lang.ADD, lang.SUBTRACT):
            a, b = get(node.ops[0]), get(node.ops[1])
            if a is None or b is None:
                return None
            out = _combine(a, b, 1 if code == lang.ADD else -1, self.ranges)
            return out if self._fits(out, node.dtype) else None
        if code == lang.MULTIPLY:
            a, b = get(node.ops[0]), get(node.ops[1])
            if a is None or b is None:
                return None
            if b.is_constant():
                a, b = b, a
            if not a.is_constant():
                return None
            out = _with_range(dict((s, c * a.const) for s, c in b.coeffs.items()), b.const * a.const, self.ranges)
            return out if self._fits(out, node.dtype) else None
        if code == lang.MODULO:
            a, b = get(node.ops[0]), get(node.ops[1])
            if a is None or b is None or not b.is_constant() or b.const <= 0:
                return None
            if a.lo >= 0 and a.hi < b.const:
                return a            # the remainder never wraps: x % m == x
            return None
        return None

    # -- queries ---------------------------------------------------------------------------------------------------
    def uses_math_tables(self):
        """True when the body calls the table-driven float32 exp or log."""
        mode = getattr(self, 'math', 'exact')
        calls = [n for n in self.nodes if n.code in (lang.EXP, lang.LOG) and n.dtype == lang.FLOAT32]
        if mode in ('ulp2', 'fast'):
            # the call sites that keep the bit-compatible routine (none in 'fast' mode) and the once-rounded
            # log1p / expm1 that stand in for the reference's formulas
            from . import accuracy
            cheap = accuracy.cheap_sites(self, self.known_ranges())
            calls = [] if mode == 'fast' else [n for n in calls if n.idx not in cheap]
            calls += [k for k in cheap.values() if k in ('log1p', 'expm1', 'log1p_guarded', 'expm1_guarded')]
            # a formula replaced behind a run-time test of its argument keeps the formula itself as the other branch,
            # evaluated with the bit-compatible exp and log in the 'ulp2' mode
            if mode == 'ulp2':
                calls += [k for k in cheap.values() if k == 'sigmoid_guarded']
        return bool(calls)

    def known_ranges(self):
        """The value-range analysis of this DAG (None when it is switched off), computed once per setting."""
        enabled = (bool(getattr(self, 'value_ranges', True)), getattr(self, 'math', 'exact'))
        cached = getattr(self, '_known_ranges', None)
        if cached is None or cached[0] != enabled:
            from . import ranges
            cached = (enabled, ranges.analyse(self) if enabled[0] else None)
            self._known_ranges = cached
        return cached[1]

    def tensor_accesses(self):
        """[(node, tensor node, affine or None)] for reads of inputs and stores to outputs, in program order."""
        found = []
        for node in self.nodes:
            if node.code == lang.READ_TENSOR and self.nodes[node.ops[0]].code == lang.INPUT:
                found.append((node, self.nodes[node.ops[0]], self.affine[node.ops[1]]))
            elif node.code == lang.ASSIGN_TENSOR and self.nodes[node.ops[0]].code == lang.OUTPUT:
                found.append((node, self.nodes[node.ops[0]], self.affine[node.ops[1]]))
        return found

    def bufferable_outputs(self, buffers):
        """
        Output node indices whose stores may be held in registers (or an LDS tile) until the end of the worker's
        iteration.  ``buffers(node, tensor, affine) -> bool`` says whether the template would buffer that one store;
        a tensor qualifies when it says so for every store to it.  A store that is not buffered (inside a loop,
        through a computed index, under a condition that not every path takes) is written at once; buffering another
        store to the same tensor would write it later and so reverse the program's order whenever both hit one element.
        """
        allowed = {}
        for node, tensor, aff in self.tensor_accesses():
            if node.code == lang.ASSIGN_TENSOR:
                ok = aff is not None and not self.in_loop[node.idx] and bool(buffers(node, tensor, aff))
                allowed[tensor.idx] = allowed.get(tensor.idx, True) and ok
        return set(idx for idx, ok in allowed.items() if ok)

    def definitely_stores(self, keys):
        """
        Subset of ``keys`` (each a (output node index, affine signature)) that every worker is certain to store on
        every path: a store at the top level of the worker, or in every branch of a conditional that ends in else.
        """
        def stored(items):
            done = set()
            for item in items:
                if item.kind == 'stmt':
                    node = self.nodes[item.node]
                    if node.code == lang.ASSIGN_TENSOR:
                        aff = self.affine[node.ops[1]]
                        if aff is not None:
                            done.add((node.ops[0], aff.signature()))
                elif item.kind == 'if' and item.has_else:
                    common = None
                    for _, branch in item.branches:
                        cur = stored(branch)
                        common = cur if common is None else (common & cur)
                    done |= common
            return done

        return stored(self.tree) & set(keys)
