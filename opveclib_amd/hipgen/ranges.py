"""
Value ranges of the floating point expressions of an operator.

A forward interval analysis over the expression DAG in program order.  Every float32 / float64 expression gets an
interval ``[lo, hi]`` that contains its value whenever the value is a number, plus a flag saying whether it may be
NaN.  The code generator uses the result for two things only, both of which leave results unchanged:

  * a comparison, logical operation or ``isinf`` / ``isnan`` / ``isfinite`` whose outcome is the same for every value
    in the operands' ranges is emitted as that constant, so the compiler deletes the conditional chains that hang on
    it (the guards of the reference's ``log1p`` / ``expm1`` against infinities, ``u == 1`` and ``u - 1 == -1`` once a
    preceding ``tanh`` or ``sigmoid`` has bounded the argument);
  * ``exp``, ``log``, reciprocal and division are emitted without their rare-argument block when the operand ranges
    show that no argument can need it.

Soundness rests on two facts.  Rounding is monotonic, so the image of an interval under ``+ - * /`` in the
expression's own precision is bounded by the images of its end points evaluated in that precision (numpy scalars
here).  The math routines are not guaranteed monotonic, so their images are widened by several units in the last
place, more than the measured error of the routines of either math mode.  Anything not understood is "any value,
possibly NaN".  Variables assigned inside a counted loop are "any value" throughout the loop and after it; after a
conditional chain a variable has the union of what the branches that can execute leave in it.
"""

import math

import numpy as np

from .. import language as lang

INF = float('inf')
_FLOATS = (lang.FLOAT32, lang.FLOAT64)
_NP = {lang.FLOAT32: np.float32, lang.FLOAT64: np.float64}

#: widening of math routine images, in units in the last place of the end point
_SLACK_ULPS = 8

_COMPARISONS = (lang.EQUAL, lang.NOTEQUAL, lang.LESS, lang.LESS_EQ, lang.GREATER, lang.GREATER_EQ)
_PREDICATES = (lang.ISINF, lang.ISNAN, lang.ISFINITE)
_LOGICAL = (lang.AND, lang.OR, lang.NOT)


class Range(object):
    """``lo <= value <= hi`` for every non-NaN value; ``nan`` says whether NaN is possible."""
    __slots__ = ('lo', 'hi', 'nan')

    def __init__(self, lo, hi, nan):
        self.lo = float(lo)
        self.hi = float(hi)
        self.nan = bool(nan)

    def __repr__(self):
        return 'Range(%r, %r%s)' % (self.lo, self.hi, ', nan' if self.nan else '')

    def __eq__(self, other):
        return isinstance(other, Range) and (self.lo, self.hi, self.nan) == (other.lo, other.hi, other.nan)

    def __ne__(self, other):
        return not self == other

    __hash__ = None

    @property
    def finite(self):
        return self.lo > -INF and self.hi < INF

    @property
    def point(self):
        """The single value of the range, or None."""
        return self.lo if (self.lo == self.hi and not self.nan) else None

    def within(self, lo, hi):
        return self.lo >= lo and self.hi <= hi

    def magnitude(self):
        """(smallest, largest) absolute value."""
        if self.lo >= 0:
            return self.lo, self.hi
        if self.hi <= 0:
            return -self.hi, -self.lo
        return 0.0, max(-self.lo, self.hi)


def top(nan=True):
    return Range(-INF, INF, nan)


def hull(ranges):
    ranges = list(ranges)
    return Range(min(r.lo for r in ranges), max(r.hi for r in ranges), any(r.nan for r in ranges))


BOOL_UNKNOWN = Range(0.0, 1.0, False)
BOOL_TRUE = Range(1.0, 1.0, False)
BOOL_FALSE = Range(0.0, 0.0, False)


def _truth(r):
    """True / False when every value of the range is nonzero / zero (NaN counts as nonzero, as in C), else None."""
    if r is None:
        return None
    if r.lo > 0 or r.hi < 0:
        return True
    if r.lo == 0 and r.hi == 0 and not r.nan:
        return False
    return None


def _from_truth(value):
    if value is None:
        return BOOL_UNKNOWN
    return BOOL_TRUE if value else BOOL_FALSE


def _widen(lo, hi, dtype, floor=-INF, ceiling=INF):
    """Move both ends outward by _SLACK_ULPS units in the last place of ``dtype``, clipped to [floor, ceiling]."""
    cast = _NP[dtype]
    tiny = float(np.finfo(cast).smallest_subnormal)

    def step(v):
        if v in (INF, -INF) or v != v:
            return 0.0
        return _SLACK_ULPS * max(float(np.spacing(cast(abs(v)))), tiny)

    lo = max(lo - step(lo), floor)
    hi = min(hi + step(hi), ceiling)
    return lo, hi


def _round(v, dtype):
    """``v`` (a Python float) rounded to ``dtype``; overflow gives an infinity."""
    with np.errstate(all='ignore'):
        return float(_NP[dtype](v))


def _arith(code, a, b, dtype):
    """Image of ``a op b`` in ``dtype`` arithmetic for finite ranges; None when not representable as an interval."""
    cast = _NP[dtype]
    nan = a.nan or b.nan
    if not (a.finite and b.finite):
        return top()
    with np.errstate(all='ignore'):
        if code == lang.ADD:
            return Range(float(cast(a.lo) + cast(b.lo)), float(cast(a.hi) + cast(b.hi)), nan)
        if code == lang.SUBTRACT:
            return Range(float(cast(a.lo) - cast(b.hi)), float(cast(a.hi) - cast(b.lo)), nan)
        if code == lang.MULTIPLY:
            products = [float(cast(x) * cast(y)) for x in (a.lo, a.hi) for y in (b.lo, b.hi)]
            return Range(min(products), max(products), nan)
        if code == lang.DIVIDE:
            if not (b.lo > 0 or b.hi < 0):
                return top()
            quotients = [float(cast(x) / cast(y)) for x in (a.lo, a.hi) for y in (b.lo, b.hi)]
            return Range(min(quotients), max(quotients), nan)
    return top()


def _monotone(fn, r, dtype, floor=-INF, ceiling=INF):
    """Image of an increasing math routine, widened."""
    def value(v):
        try:
            return _round(fn(v), dtype)
        except OverflowError:
            return INF
    lo, hi = _widen(value(r.lo), value(r.hi), dtype, floor, ceiling)
    return Range(lo, hi, r.nan)


def _exp(v):
    if v == -INF:
        return 0.0
    if v == INF:
        return INF
    return math.exp(v)


def _compare(code, a, b):
    """Outcome of a comparison of two ranges as True / False / None."""
    if a is None or b is None:
        return None
    maybe_nan = a.nan or b.nan
    if code == lang.NOTEQUAL:
        if a.hi < b.lo or b.hi < a.lo:
            return True
        if a.point is not None and a.point == b.point:
            return False
        return None
    if code == lang.EQUAL:
        if a.hi < b.lo or b.hi < a.lo:
            return False
        if a.point is not None and a.point == b.point:
            return True
        return None
    if code in (lang.GREATER, lang.GREATER_EQ):
        a, b = b, a
        code = lang.LESS if code == lang.GREATER else lang.LESS_EQ
    if code == lang.LESS:
        if a.hi < b.lo and not maybe_nan:
            return True
        if a.lo >= b.hi:
            return False
        return None
    if code == lang.LESS_EQ:
        if a.hi <= b.lo and not maybe_nan:
            return True
        if a.lo > b.hi:
            return False
        return None
    return None


class RangeInfo(object):
    """
    Result of the analysis.

    ``ranges[idx]``  Range of expression ``idx`` where it is evaluated (floating point expressions and the 0/1 results
                     of comparisons on them); for a VARIABLE, its range right after the declaration.
    ``operand(idx, k)``  Range of operand ``k`` of expression ``idx`` at that point of the program (differs from
                     ``ranges`` for variables, whose value changes with assignments).
    ``constant(idx)``  0 or 1 when expression ``idx`` is a comparison / logical operation / float predicate with a
                     known outcome, else None.
    """

    def __init__(self, info):
        self.info = info
        # quotients of the 'fast' math mode are not correctly rounded: their images are widened like a routine's
        self.inexact_division = getattr(info, 'math', 'exact') != 'exact'
        self.ranges = {}
        self._operands = {}
        self._run(info.tree, {})

    # -- queries ---------------------------------------------------------------------------------------------------
    def operand(self, idx, k):
        return self._operands.get((idx, k))

    def constant(self, idx):
        node = self.info.nodes[idx]
        if node.code not in _COMPARISONS and node.code not in _PREDICATES and node.code not in _LOGICAL:
            return None
        r = self.ranges.get(idx)
        if r is None or r.point is None:
            return None
        return int(r.point)

    # -- interpretation ----------------------------------------------------------------------------------------------
    def _assigned_in(self, items, out):
        for item in items:
            if item.kind == 'stmt':
                node = self.info.nodes[item.node]
                if node.code == lang.ASSIGN_VARIABLE:
                    out.add(node.ops[0])
            elif item.kind == 'if':
                for _, body in item.branches:
                    self._assigned_in(body, out)
            else:
                out.add(self.info.nodes[item.node].ops[0])      # the loop counter
                self._assigned_in(item.body, out)
        return out

    def _run(self, items, env):
        """Interpret ``items`` in order; ``env`` maps VARIABLE node index -> current Range and is updated in place."""
        nodes = self.info.nodes
        for item in items:
            if item.kind == 'stmt':
                self._transfer(nodes[item.node], env)
            elif item.kind == 'loop':
                # the loop header's operands are evaluated as statements before it; anything the body assigns is
                # unknown from here on
                for var in self._assigned_in([item], set()):
                    env[var] = top() if nodes[var].dtype in _FLOATS else None
                self._run(item.body, env)
                for var in self._assigned_in([item], set()):
                    env[var] = top() if nodes[var].dtype in _FLOATS else None
            else:
                exits = []
                reachable = True
                for cond, body in item.branches:
                    if not reachable:
                        self._run(body, dict(env))      # still gives its expressions (sound) ranges
                        continue
                    taken = True if cond is None else _truth(self._value(cond, env))
                    branch_env = dict(env)
                    self._run(body, branch_env)
                    if taken is False:
                        continue
                    exits.append(branch_env)
                    if taken is True:
                        reachable = False
                if reachable:
                    exits.append(dict(env))             # no branch taken
                merged = {}
                for var in set().union(*[set(e) for e in exits]):
                    values = [e.get(var) for e in exits]
                    merged[var] = None if any(v is None for v in values) else hull(values)
                env.clear()
                env.update(merged)

    def _value(self, idx, env):
        node = self.info.nodes[idx]
        if node.code == lang.VARIABLE:
            return env.get(idx)
        return self.ranges.get(idx)

    def _transfer(self, node, env):
        code = node.code
        dtype = node.dtype
        ops = [self._value(o, env) for o in node.ops]
        for k, r in enumerate(ops):
            if r is not None:
                self._operands[(node.idx, k)] = r
        result = None

        if code == lang.ASSIGN_VARIABLE:
            var = self.info.nodes[node.ops[0]]
            value = ops[1]
            if var.dtype in _FLOATS:
                env[var.idx] = self._converted(value, self.info.nodes[node.ops[1]], var.dtype)
            else:
                env[var.idx] = None
            return
        if code == lang.CONST_SCALAR and dtype in _FLOATS:
            v = _round(float(node.data[0]), dtype)
            result = top() if v != v else Range(v, v, False)
        elif code == lang.CONST_SCALAR and len(node.data) == 1 and abs(int(node.data[0])) < 2 ** 53:
            result = Range(int(node.data[0]), int(node.data[0]), False)
        elif code in (lang.MIN_VALUE, lang.MAX_VALUE, lang.EPSILON) and dtype in _FLOATS:
            fi = np.finfo(_NP[dtype])
            v = float({lang.MIN_VALUE: fi.tiny, lang.MAX_VALUE: fi.max, lang.EPSILON: fi.eps}[code])
            result = Range(v, v, False)
        elif code in (lang.VARIABLE, lang.CAST) and dtype in _FLOATS:
            result = self._converted(ops[0], self.info.nodes[node.ops[0]], dtype)
            if code == lang.VARIABLE:
                env[node.idx] = result
        elif code == lang.READ_TENSOR and dtype in _FLOATS:
            result = top()
        elif code in _COMPARISONS:
            result = _from_truth(_compare(code, ops[0], ops[1]))
        elif code == lang.AND:
            a, b = _truth(ops[0]), _truth(ops[1])
            result = _from_truth(False if (a is False or b is False) else (True if (a and b) else None))
        elif code == lang.OR:
            a, b = _truth(ops[0]), _truth(ops[1])
            result = _from_truth(True if (a or b) else (False if (a is False and b is False) else None))
        elif code == lang.NOT:
            a = _truth(ops[0])
            result = _from_truth(None if a is None else not a)
        elif code in _PREDICATES:
            result = self._predicate(code, ops[0])
        elif dtype in _FLOATS:
            result = self._float_op(code, dtype, ops)
            if code == lang.DIVIDE and dtype == lang.FLOAT32:
                result = self._formula_image(node, result)
        if result is not None:
            self.ranges[node.idx] = result

    def _formula_image(self, node, result):
        """The division that ends the reference's sigmoid / log1p / expm1 formula (accuracy.match_idiom): interval
        arithmetic over the formula's parts forgets that they share x (log(u) * x / (u - 1) with x in [0.27, 0.73]
        comes out as [0.09, 1.5]), but on the domains where the formulas were compared with the once-rounded
        routines on every argument their value is within three float32 steps of the function itself, in every math
        mode within seven: the function's image, widened like a routine's, bounds it."""
        from . import accuracy
        found = accuracy.match_idiom(self.info, self, node)
        if found is None:
            return result
        kind, _, seen = found
        fn = {'sigmoid': lambda v: 1.0 / (1.0 + _exp(-v)), 'log1p': math.log1p, 'expm1': math.expm1}[kind]
        image = _monotone(fn, seen, node.dtype)
        lo, hi = max(result.lo, image.lo), min(result.hi, image.hi)
        if lo > hi:
            return result
        return Range(lo, hi, result.nan)

    @staticmethod
    def _converted(value, source_node, dtype):
        """Range of ``value`` converted to the float type ``dtype``."""
        if value is None:
            # an integer of unknown value is some number, never NaN
            return top(nan=source_node.dtype in _FLOATS)
        return Range(_round(value.lo, dtype), _round(value.hi, dtype), value.nan)

    @staticmethod
    def _predicate(code, x):
        if x is None:
            return BOOL_UNKNOWN
        if code == lang.ISNAN:
            return BOOL_FALSE if not x.nan else BOOL_UNKNOWN
        if code == lang.ISINF:
            return BOOL_FALSE if x.finite else BOOL_UNKNOWN
        if code == lang.ISFINITE:
            return BOOL_TRUE if (x.finite and not x.nan) else BOOL_UNKNOWN
        return BOOL_UNKNOWN

    def _float_op(self, code, dtype, ops):
        if any(r is None for r in ops) or not ops:
            return top()
        a = ops[0]
        if code in (lang.ADD, lang.SUBTRACT, lang.MULTIPLY, lang.DIVIDE):
            r = _arith(code, a, ops[1], dtype)
            if code == lang.DIVIDE and self.inexact_division and r.finite:
                lo, hi = _widen(r.lo, r.hi, dtype)
                r = Range(lo, hi, r.nan)
            return r
        if code in (lang.MIN, lang.MAX):
            # emitted as (a < b) ? a : b and (a > b) ? a : b: the smaller (larger) of two numbers; the comparison is
            # false when a is NaN, which selects b whatever its value, and a NaN in b comes through
            b = ops[1]
            pick = min if code == lang.MIN else max
            result = Range(pick(a.lo, b.lo), pick(a.hi, b.hi), b.nan)
            return hull([result, b]) if a.nan else result
        if code == lang.NEGATE:
            return Range(-a.hi, -a.lo, a.nan)
        if code == lang.ABS:
            lo, hi = a.magnitude()
            return Range(lo, hi, a.nan)
        if code == lang.TANH:
            return _monotone(math.tanh, a, dtype, -1.0, 1.0)
        if code == lang.EXP:
            return _monotone(_exp, a, dtype, 0.0, INF)
        if code == lang.LOG:
            if a.lo <= 0:
                return top()
            return _monotone(lambda v: INF if v == INF else math.log(v), a, dtype)
        if code == lang.SQRT:
            if a.lo < 0:
                return top()
            return _monotone(lambda v: INF if v == INF else math.sqrt(v), a, dtype, 0.0, INF)
        if code in (lang.SIN, lang.COS):
            lo, hi = _widen(-1.0, 1.0, dtype)
            return Range(lo, hi, a.nan or not a.finite)
        if code in (lang.CEIL, lang.FLOOR):
            return Range(math.floor(a.lo) if a.lo > -INF else -INF, math.ceil(a.hi) if a.hi < INF else INF, a.nan)
        return top()


def analyse(info):
    """RangeInfo of a DagInfo, computed once."""
    cached = getattr(info, '_range_info', None)
    if cached is None:
        cached = RangeInfo(info)
        info._range_info = cached
    return cached


# ---------------------------------------------------------------------------------------------------------------------
# Conditions under which the math routines of csrc/ovl_math.h and csrc/ovl_fast_math.h need no rare-argument block
# ---------------------------------------------------------------------------------------------------------------------
def exp_in_range(x, math_mode):
    """|x| below the routine's threshold (88 for the table driven routine, 87 for the hardware based one)."""
    limit = 87.5 if math_mode == 'exact' else 86.5
    return x is not None and x.within(-limit, limit)


def log_in_range(x):
    """x a positive normal float32 (or NaN)."""
    return x is not None and x.lo >= 2.0 ** -126 and x.hi <= 3.0e38


def recip_in_range(b):
    if b is None:
        return False
    lo, hi = b.magnitude()
    return lo >= 2.0 ** -125 and hi <= 2.0 ** 125


def div_in_range(a, b):
    """Operands for which the division needs neither operand scaling nor a fix-up (see ovl_math::divf_inrange_)."""
    if a is None or b is None:
        return False
    alo, ahi = a.magnitude()
    blo, bhi = b.magnitude()
    if not (alo >= 2.0 ** -99 and ahi <= 2.0 ** 119 and blo >= 2.0 ** -119 and bhi <= 2.0 ** 119):
        return False
    return ahi / blo <= 2.0 ** 88 and alo / bhi >= 2.0 ** -118
