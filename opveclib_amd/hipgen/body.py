"""
Emission of the per-worker body of an operator as HIP device code.

One statement per expression in DAG order, the same sequence of typed operations that the reference's generator
emits for the CPU and CUDA targets (opveclib/expression.py: every ``gen_c``, statement forms listed at
1293-1306, 1351-1352, 1386-1387, 1422-1423, 1479-1481, 1739-1742, 1794-1795, 1881-1882, 1904-1905, 1996-2006,
2064-2183), so a worker performs the same arithmetic in the same order.  Kernel templates customise how tensor
reads and stores are realised through the ``read_hook`` / ``store_hook`` callbacks (vector register lanes, LDS
tiles, plain global accesses).
"""

from .. import language as lang
from . import ranges as value_ranges
from . import accuracy

CTYPE = {
    lang.FLOAT32: 'float', lang.FLOAT64: 'double',
    lang.INT8: 'int8_t', lang.INT16: 'int16_t', lang.INT32: 'int32_t', lang.INT64: 'long long',
    lang.UINT8: 'uint8_t', lang.UINT16: 'uint16_t', lang.UINT32: 'uint32_t', lang.UINT64: 'uint64_t'}

# device math entry points (ovl_* are defined in csrc/ovl_device.h)
UNARY = {
    lang.ACOS: {lang.FLOAT32: 'acosf', lang.FLOAT64: 'acos'},
    lang.ASIN: {lang.FLOAT32: 'asinf', lang.FLOAT64: 'asin'},
    lang.ATAN: {lang.FLOAT32: 'atanf', lang.FLOAT64: 'atan'},
    lang.COS: {lang.FLOAT32: 'cosf', lang.FLOAT64: 'cos'},
    lang.COSH: {lang.FLOAT32: 'coshf', lang.FLOAT64: 'cosh'},
    lang.SIN: {lang.FLOAT32: 'sinf', lang.FLOAT64: 'sin'},
    lang.SINH: {lang.FLOAT32: 'sinhf', lang.FLOAT64: 'sinh'},
    lang.TAN: {lang.FLOAT32: 'tanf', lang.FLOAT64: 'tan'},
    lang.TANH: {lang.FLOAT32: 'ovl_tanhf', lang.FLOAT64: 'tanh'},
    lang.EXP: {lang.FLOAT32: 'ovl_expf', lang.FLOAT64: 'exp'},
    lang.LOG: {lang.FLOAT32: 'ovl_logf', lang.FLOAT64: 'log'},
    lang.LOG10: {lang.FLOAT32: 'log10f', lang.FLOAT64: 'log10'},
    lang.SQRT: {lang.FLOAT32: 'sqrtf', lang.FLOAT64: 'sqrt'},
    lang.CEIL: {lang.FLOAT32: 'ceilf', lang.FLOAT64: 'ceil'},
    lang.FLOOR: {lang.FLOAT32: 'floorf', lang.FLOAT64: 'floor'},
    lang.ABS: {lang.FLOAT32: 'fabsf', lang.FLOAT64: 'fabs', lang.INT8: 'ovl_abs_8', lang.INT16: 'ovl_abs_16',
               lang.INT32: 'abs', lang.INT64: 'llabs'},
    lang.ISINF: {lang.FLOAT32: 'isinf', lang.FLOAT64: 'isinf'},
    lang.ISFINITE: {lang.FLOAT32: 'isfinite', lang.FLOAT64: 'isfinite'},
    lang.ISNAN: {lang.FLOAT32: 'isnan', lang.FLOAT64: 'isnan'},
}
# Float32 math per mode: {mode: {expression code: function name}}; DIVIDE maps to a two-argument function.
# 'exact' (the default) is the table above plus the IEEE '/' operator: the host C library's bits.  'fast' calls the
# routines of csrc/ovl_fast_math.h (hardware exp2 / log2 / reciprocal with extended-precision range handling, each
# within two units in the last place of the host library's result).  The third mode, 'ulp2', has no table of its own:
# every call site takes its routine from 'exact' or from 'fast', as accuracy.select decides.
MATH_MODES = {
    'exact': {},
    'fast': {lang.TANH: 'ovl_fast_tanhf', lang.EXP: 'ovl_fast_expf', lang.LOG: 'ovl_fast_logf',
             lang.DIVIDE: 'ovl_fast_divf'},
}
# Variants without the rare-argument block, chosen when the value-range analysis (ranges.py) proves that no argument
# can need it: {mode: {expression code: function name}}.  The exact mode's logarithm works on the bits of its
# argument and has a second variant that also passes NaN on.
IN_RANGE = {
    'exact': {lang.EXP: 'ovl_expf_inrange', lang.LOG: 'ovl_logf_inrange', 'log nan': 'ovl_logf_inrange_nan',
              lang.DIVIDE: 'ovl_divf_inrange'},
    'fast': {lang.EXP: 'ovl_fast_expf_inrange', lang.LOG: 'ovl_fast_logf_inrange', 'log nan': 'ovl_fast_logf_inrange',
             lang.DIVIDE: 'ovl_fast_divf_inrange'},
}

_NEGATABLE = (lang.FLOAT32, lang.FLOAT64, lang.INT8, lang.INT16, lang.INT32, lang.INT64)
UNARY[lang.NEGATE] = dict((t, '-') for t in _NEGATABLE)
UNARY[lang.NOT] = dict((t, '!') for t in CTYPE)

INFIX = {lang.ADD: '+', lang.SUBTRACT: '-', lang.MULTIPLY: '*', lang.DIVIDE: '/', lang.MODULO: '%',
         lang.EQUAL: '==', lang.NOTEQUAL: '!=', lang.LESS: '<', lang.LESS_EQ: '<=', lang.GREATER: '>',
         lang.GREATER_EQ: '>=', lang.AND: '&&', lang.OR: '||'}

LIMITS = {lang.MIN_VALUE: {lang.FLOAT32: 'FLT_MIN', lang.FLOAT64: 'DBL_MIN'},
          lang.MAX_VALUE: {lang.FLOAT32: 'FLT_MAX', lang.FLOAT64: 'DBL_MAX'},
          lang.EPSILON: {lang.FLOAT32: 'FLT_EPSILON', lang.FLOAT64: 'DBL_EPSILON'}}


def literal(value, dtype=None):
    """
    Text of a numeric literal.  Floating point literals are written as C double literals exactly like Python prints
    them, so the conversion to the destination type happens in the compiled code, as it does for the reference's
    generated text (a ``float e = 1.0001;`` statement rounds the double literal to float).
    """
    if isinstance(value, float):
        if value != value:
            return '__builtin_nan("")'
        if value == float('inf'):
            return '__builtin_inf()'
        if value == float('-inf'):
            return '(-__builtin_inf())'
        return repr(float(value))
    value = int(value)
    if dtype == lang.UINT64 or value > 2 ** 63 - 1:
        return str(value) + 'ull'
    if value < -2 ** 31 or value > 2 ** 31 - 1:
        return str(value) + 'll'
    return str(value)


def binary_text(code, dtype, a, b):
    if code == lang.MIN:
        return '(((' + a + ')<(' + b + '))?(' + a + '):(' + b + '))'
    if code == lang.MAX:
        return '(((' + a + ')>(' + b + '))?(' + a + '):(' + b + '))'
    if code == lang.POW:
        return ('powf(' if dtype == lang.FLOAT32 else 'pow(') + a + ',' + b + ')'
    if code == lang.ATAN2:
        return ('ovl_atan2f(' if dtype == lang.FLOAT32 else 'atan2(') + a + ',' + b + ')'
    if code == lang.MODULO and dtype == lang.FLOAT32:
        return 'fmodf(' + a + ',' + b + ')'
    if code == lang.MODULO and dtype == lang.FLOAT64:
        return 'fmod(' + a + ',' + b + ')'
    return '(' + a + ' ' + INFIX[code] + ' ' + b + ')'


class BodyEmitter(object):
    """
    Walks the DAG and produces the statement list of one worker.

    :param info: the analysed DAG (:class:`analysis.DagInfo`)
    :param position_exprs: list of C expressions, one per workgroup dimension, giving this worker's position
    :param read_hook: ``f(node, tensor_node, index_name) -> C expression or None``; None selects the plain global
        read ``in<k>[index]``
    :param store_hook: ``f(node, tensor_node, index_name, value_name) -> C statement or None``; None selects the
        plain global store ``out<k>[index] = value;``
    """

    def __init__(self, info, position_exprs, read_hook=None, store_hook=None, suffix='', register_stores=True):
        self.info = info
        self.position_exprs = position_exprs
        self.read_hook = read_hook
        self.store_hook = store_hook
        self.suffix = suffix
        # True when every statement the store hook returns assigns a register (so it may be turned into a select)
        self.register_stores = register_stores

    def tensor_name(self, node):
        if node.code == lang.INPUT:
            return 'in' + str(node.io_index)
        if node.code == lang.OUTPUT:
            return 'out' + str(node.io_index)
        if node.code == lang.POSITION:
            return 'position'
        return 'e' + str(node.idx) + self.suffix

    def _is_constant_one(self, idx):
        """The expression is the literal 1, directly or through casts (a VARIABLE could be reassigned: excluded)."""
        node = self.info.nodes[idx]
        while node.code == lang.CAST:
            node = self.info.nodes[node.ops[0]]
        return node.code == lang.CONST_SCALAR and len(node.data) == 1 and float(node.data[0]) == 1.0

    # ------------------------------------------------------------------------------------------------------------
    # If-conversion.  A conditional chain whose branches only compute values and assign variables (or registers that
    # buffer a vector store) is emitted as straight-line code: every branch is evaluated and each assignment becomes a
    # select on "this branch is the one taken".  Lanes of a wavefront that disagree execute all branches anyway; what
    # the conversion removes is the execution-mask bookkeeping around every branch, and it lets the compiler schedule
    # across the chain.  Speculating a branch is safe when it cannot fault or trap: no memory access of its own, no
    # integer division.  At most one branch may be expensive (the others would otherwise be pure overhead when the
    # whole wavefront takes the same branch).
    # ------------------------------------------------------------------------------------------------------------
    _CHEAP_BRANCH = 6

    def _plan_if_conversion(self):
        info = self.info
        self._predicate = {}        # statement node index -> name of the bool "its branch is taken"
        self._converted = {}        # IF node index -> [(predicate name, condition node index or None)]
        if not getattr(info, 'if_conversion', True):
            return
        expensive_codes = (lang.DIVIDE, lang.MODULO, lang.POW, lang.ATAN2, lang.EXP, lang.LOG, lang.LOG10, lang.TANH,
                           lang.SIN, lang.COS, lang.TAN, lang.SINH, lang.COSH, lang.ASIN, lang.ACOS, lang.ATAN,
                           lang.SQRT)

        def branch_cost(items):
            """Number of operations of a branch, or None when it cannot be speculated."""
            cost = 0
            for item in items:
                if item.kind != 'stmt':
                    return None
                node = info.nodes[item.node]
                code = node.code
                if code in (lang.CONST_SCALAR, lang.MIN_VALUE, lang.MAX_VALUE, lang.EPSILON):
                    continue
                if code in (lang.CAST, lang.VARIABLE):
                    cost += 1 if node.dtype in (lang.FLOAT32, lang.FLOAT64) else 0
                elif code == lang.ASSIGN_VARIABLE:
                    cost += 1
                elif code == lang.READ_TENSOR and info.nodes[node.ops[0]].code == lang.POSITION:
                    continue                # a component of the worker's position: a register
                elif code == lang.READ_TENSOR:
                    tensor = info.nodes[node.ops[0]]
                    if tensor.code != lang.INPUT or self.read_hook is None or \
                            self.read_hook(node, tensor, 'index') is None:
                        return None         # a memory access of its own
                    cost += 1
                elif code == lang.ASSIGN_TENSOR:
                    tensor = info.nodes[node.ops[0]]
                    if tensor.code != lang.OUTPUT or self.store_hook is None or not self.register_stores:
                        return None
                    text = self.store_hook(node, tensor, 'index', 'value')
                    if not text or not text.endswith('= value;'):
                        return None         # a real store, not a register that buffers one
                    cost += 1
                elif code in UNARY or code in INFIX or code in (lang.MIN, lang.MAX, lang.POW, lang.ATAN2):
                    if code in (lang.DIVIDE, lang.MODULO) and node.dtype not in (lang.FLOAT32, lang.FLOAT64):
                        return None         # integer division by zero must stay guarded
                    if node.dtype in (lang.FLOAT32, lang.FLOAT64):
                        cost += 20 if code in expensive_codes else 1
                    # integer arithmetic in a branch is almost always index arithmetic that folds away: not counted
                else:
                    return None
            return cost

        def walk(items):
            for item in items:
                if item.kind == 'loop':
                    walk(item.body)
                elif item.kind == 'if':
                    costs = [branch_cost(body) for _, body in item.branches]
                    if all(c is not None for c in costs) and \
                            sum(1 for c in costs if c > self._CHEAP_BRANCH) <= 1:
                        names = []
                        for k, (cond, body) in enumerate(item.branches):
                            pred = 't%d_%d%s' % (item.node, k, self.suffix)
                            names.append((pred, cond))
                            for stmt in body:
                                self._predicate[stmt.node] = pred
                        self._converted[item.node] = names
                    else:
                        for _, body in item.branches:
                            walk(body)

        walk(info.tree)

    def emit(self):
        """All statements of the worker, in order."""
        return [text for _, text in self.emit_tagged()]

    def emit_tagged(self):
        """[(index of the expression that produced it, statement text)] in program order."""
        info = self.info
        math_mode = getattr(info, 'math', 'exact')
        known = info.known_ranges()
        cheap_sites = accuracy.cheap_sites(info, known)

        def site_mode(node):
            """The math mode of one call site."""
            if math_mode != 'ulp2':
                return math_mode
            return 'fast' if node.idx in cheap_sites else 'exact'
        self._plan_if_conversion()
        names = {}
        stmts = []
        # Common subexpressions.  The worker functions of the reference repeat whole sub-expressions (its LSTM gradient
        # evaluates sigmoid(i), sigmoid(f + bias), tanh(j) and tanh(new_c) once for the forward recomputation and again
        # inside every gate's derivative, lstm/lstm.py:84-103); the same operation on the same operands gives the same
        # bits, so a repeated expression takes the name of its first evaluation at the top level of the worker.  The
        # C++ compiler finds only some of these across the rare-argument blocks of the math routines.
        value_key = {}          # node index -> hashable description of a pure expression, or None
        first_value = {}        # description -> name of its first unconditional evaluation
        cse = getattr(info, 'cse', True)

        def describe(node):
            code = node.code
            if code == lang.CONST_SCALAR:
                return ('const', node.dtype, repr(node.data[0]))
            if code in LIMITS:
                return ('limit', code, node.dtype)
            operands = tuple(value_key.get(o) for o in node.ops)
            if code == lang.READ_TENSOR:
                tensor = info.nodes[node.ops[0]]
                if tensor.code == lang.POSITION and operands[1] is not None:
                    return ('position', operands[1])
                if tensor.code == lang.INPUT and operands[1] is not None and not info.in_loop[node.idx]:
                    return ('read', tensor.io_index, operands[1])
                return None
            if any(o is None for o in operands) or not operands:
                return None
            if code == lang.CAST:
                return ('cast', node.dtype, operands[0])
            if code in UNARY or code in INFIX or code in (lang.MIN, lang.MAX, lang.POW, lang.ATAN2):
                return (code, node.dtype, site_mode(node) if code in accuracy.ROUTINE_ULPS else None) + operands
            return None

        indent = 0
        current = [0]
        open_chains = []        # True for a converted chain, False for one emitted as branches

        def assign(node, target, value):
            """target = value, as a select when the statement sits in a converted branch."""
            pred = self._predicate.get(node.idx)
            if pred is None:
                return target + ' = ' + value + ';'
            return target + ' = ' + pred + ' ? (' + value + ') : ' + target + ';'

        def put(text):
            stmts.append((current[0], '    ' * indent + text))

        for node in info.nodes:
            current[0] = node.idx
            code = node.code
            ops = node.ops
            name = 'e' + str(node.idx) + self.suffix
            key = value_key[node.idx] = describe(node) if cse else None
            if key is not None and code not in (lang.CONST_SCALAR,) and code not in LIMITS:
                if key in first_value:
                    names[node.idx] = first_value[key]
                    continue
                if info.depth[node.idx] == 0:
                    first_value[key] = name
            if code in (lang.INPUT, lang.OUTPUT):
                name = self.tensor_name(node)
            elif code == lang.POSITION:
                name = 'position'
                put('const uint32_t position[' + str(len(self.position_exprs)) + '] = {' +
                    ', '.join(self.position_exprs) + '};')
            elif code == lang.CONST_SCALAR:
                name = literal(node.data[0], node.dtype)
            elif code == lang.CONST_TENSOR:
                name = '{' + ', '.join(literal(v, node.dtype) for v in node.data) + '}'
            elif code in LIMITS:
                name = LIMITS[code][node.dtype]
            elif code in (lang.VARIABLE, lang.CAST):
                put(CTYPE[node.dtype] + ' ' + name + ' = ' + names[ops[0]] + ';')
            elif code == lang.TENSOR:
                put(CTYPE[node.dtype] + ' ' + name + '[' + str(node.size) + '] = ' + names[ops[0]] + ';')
            elif code == lang.ASSIGN_VARIABLE:
                put(assign(node, names[ops[0]], names[ops[1]]))
            elif code == lang.ASSIGN_TENSOR:
                tensor = info.nodes[ops[0]]
                text = None
                if tensor.code == lang.OUTPUT and self.store_hook is not None:
                    text = self.store_hook(node, tensor, names[ops[1]], names[ops[2]])
                    if text and node.idx in self._predicate:
                        target = text[:text.index(' = ')]
                        text = assign(node, target, names[ops[2]])
                if text is None:
                    text = names[ops[0]] + '[' + names[ops[1]] + '] = ' + names[ops[2]] + ';'
                if text:
                    put(text)
            elif code == lang.READ_TENSOR:
                tensor = info.nodes[ops[0]]
                text = None
                if tensor.code == lang.INPUT and self.read_hook is not None:
                    text = self.read_hook(node, tensor, names[ops[1]])
                if text is None:
                    text = names[ops[0]] + '[' + names[ops[1]] + ']'
                put(CTYPE[node.dtype] + ' ' + name + ' = ' + text + ';')
            elif code == lang.RANGE:
                i, start, stop, step = (names[o] for o in ops)
                put('for(' + i + ' = ' + start + '; ((' + i + ' < ' + stop + ')&&(' + step + '>0)) || ((' +
                    i + ' > ' + stop + ')&&(' + step + '<0)); ' + i + '+=' + step + '){')
                indent += 1
            elif code == lang.ENDRANGE:
                indent -= 1
                put('}')
            elif code == lang.ENDIF:
                if not open_chains.pop():
                    indent -= 1
                    put('}')
            elif code == lang.IF:
                if node.idx in self._converted:
                    open_chains.append(True)
                    earlier = []
                    for pred, cond in self._converted[node.idx]:
                        terms = ['!' + e for e in earlier]
                        if cond is not None:
                            terms.append('(' + names[cond] + ' != 0)')
                        put('const bool ' + pred + ' = ' + (' && '.join(terms) if terms else 'true') + ';')
                        earlier.append(pred)
                else:
                    open_chains.append(False)
                    put('if(' + names[ops[0]] + '){')
                    indent += 1
            elif code == lang.ELSEIF:
                if not open_chains[-1]:
                    indent -= 1
                    put('} else if(' + names[ops[0]] + '){')
                    indent += 1
            elif code == lang.ELSE:
                if not open_chains[-1]:
                    indent -= 1
                    put('} else {')
                    indent += 1
            elif known is not None and known.constant(node.idx) is not None:
                # the operands' value ranges decide this comparison / logical operation / predicate
                put(CTYPE[node.dtype] + ' ' + name + ' = ' + str(known.constant(node.idx)) + ';')
            elif code in UNARY:
                fcn = UNARY[code][node.dtype]
                mode = site_mode(node)
                if node.dtype == lang.FLOAT32 and code in MATH_MODES[mode]:
                    fcn = MATH_MODES[mode][code]
                if node.dtype == lang.FLOAT32 and known is not None:
                    x = known.operand(node.idx, 0)
                    if code == lang.EXP and value_ranges.exp_in_range(x, mode):
                        fcn = IN_RANGE[mode][code]
                    elif code == lang.LOG and value_ranges.log_in_range(x):
                        fcn = IN_RANGE[mode]['log nan' if x.nan else code]
                put(CTYPE[node.dtype] + ' ' + name + ' = ' + fcn + '(' + names[ops[0]] + ');')
            elif code == lang.DIVIDE and cheap_sites.get(node.idx) in accuracy.GUARDED:
                # the same formula with an argument of unknown range: the routine when every lane of the wavefront
                # holds an argument of the compared domain, else the formula itself (with the routines the other
                # call sites of this mode use: the bit-compatible ones in 'ulp2')
                kind, x = accuracy.match_guarded(info, known, node)
                arg = names[x]
                fallback = 'fast' if math_mode == 'fast' else 'exact'
                exp_fn = MATH_MODES[fallback].get(lang.EXP, UNARY[lang.EXP][lang.FLOAT32])
                log_fn = MATH_MODES[fallback].get(lang.LOG, UNARY[lang.LOG][lang.FLOAT32])
                quotient = (lambda a, b: MATH_MODES[fallback][lang.DIVIDE] + '(' + a + ', ' + b + ')') \
                    if lang.DIVIDE in MATH_MODES[fallback] else (lambda a, b: '(' + a + ' / ' + b + ')')
                routine = {'sigmoid': 'ovl_sigmoid_ulp2', 'log1p': 'ovl_log1p_direct', 'expm1': 'ovl_expm1_direct'}[kind]
                if kind == 'sigmoid':
                    formula = 'ovl_recipf(1.0f + ' + exp_fn + '(-' + arg + '))'
                elif kind == 'log1p':
                    formula = quotient('(' + log_fn + '(1.0f + ' + arg + ') * ' + arg + ')', '((1.0f + ' + arg + ') - 1.0f)')
                else:
                    formula = quotient('((' + exp_fn + '(' + arg + ') - 1.0f) * ' + arg + ')',
                                       log_fn + '(' + exp_fn + '(' + arg + '))')
                inside = ' || '.join('(%s >= %s && %s <= %s)' % (arg, literal(lo) + 'f', arg, literal(hi) + 'f')
                                     for lo, hi in accuracy.GUARD_DOMAIN[kind])
                put('float ' + name + ';')
                put('if (OVL_ALL(' + inside + ')) { ' + name + ' = ' + routine + '(' + arg + '); } else { ' +
                    name + ' = ' + formula + '; }')
            elif code == lang.DIVIDE and cheap_sites.get(node.idx) in accuracy.IDIOM_DOMAIN:
                # the division that ends the reference's sigmoid / log1p / expm1 formula: one routine on x instead
                kind, x, seen = accuracy.match_idiom(info, known, node)
                fcn = {'sigmoid': 'ovl_sigmoid_ulp2', 'log1p': 'ovl_log1p_direct_nan' if seen.nan else 'ovl_log1p_direct',
                       'expm1': 'ovl_expm1_direct'}[kind]
                if accuracy.in_narrow_domain(kind, seen):
                    fcn = {'log1p': 'ovl_log1p_unit', 'expm1': 'ovl_expm1_small', 'sigmoid': 'ovl_sigmoid_small'}[kind]
                put('float ' + name + ' = ' + fcn + '(' + names[x] + ');')
            elif code == lang.DIVIDE and node.dtype == lang.FLOAT32 and self._is_constant_one(ops[0]):
                # 1/x: the verified correctly rounded reciprocal (ovl_math.h) instead of the general division, in
                # every math mode (it is also the cheapest form: hardware reciprocal and one refinement)
                fcn = 'ovl_recipf'
                if known is not None and value_ranges.recip_in_range(known.operand(node.idx, 1)):
                    fcn = 'ovl_recipf_inrange'
                put('float ' + name + ' = ' + fcn + '(' + names[ops[1]] + ');')
            elif code == lang.DIVIDE and node.dtype == lang.FLOAT32 and known is not None and \
                    value_ranges.div_in_range(known.operand(node.idx, 0), known.operand(node.idx, 1)):
                put('float ' + name + ' = ' + IN_RANGE[site_mode(node)][code] + '(' + names[ops[0]] + ', ' +
                    names[ops[1]] + ');')
            elif code == lang.DIVIDE and node.dtype == lang.FLOAT32 and code in MATH_MODES[site_mode(node)]:
                put('float ' + name + ' = ' + MATH_MODES[site_mode(node)][code] + '(' + names[ops[0]] + ', ' +
                    names[ops[1]] + ');')
            elif code in INFIX or code in (lang.MIN, lang.MAX, lang.POW, lang.ATAN2):
                put(CTYPE[node.dtype] + ' ' + name + ' = ' +
                    binary_text(code, node.dtype, names[ops[0]], names[ops[1]]) + ';')
            else:
                raise NotImplementedError('expression code ' + str(code))
            names[node.idx] = name
        return stmts
