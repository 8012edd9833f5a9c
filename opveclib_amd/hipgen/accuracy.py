"""
Choice of float32 math routines under an error budget (the ``ulp2`` math mode).

The reference's generated C++ calls the host C library (opveclib/expression.py:1430-1456).  The ``exact`` math mode
reproduces those results bit for bit, which costs several times the arithmetic of routines built on the hardware's
exp2 / log2 / reciprocal instructions (csrc/ovl_fast_math.h), each of which stays within one or two units in the last
place (ulp) of the host library for every argument.  The ``ulp2`` mode promises that **every value an operator stores
is within two float32 ulp of what the reference's code computes from the same operator inputs** and uses the cheap
routines wherever a static error analysis shows that the promise holds; every other call site keeps the bit-compatible
routine.  In a fused chain the promise holds per operator of the chain (a VARIABLE that stands for a tensor the fusion
optimizer internalised is marked by ``fusion.py`` and starts a new stage here), exactly as it would if the operators
ran one by one.

The analysis interprets the worker in program order and carries, for every float32 value, an upper bound on the
number of float32 steps between this build's value and the reference's, together with the set of call sites the
bound depends on:

  * inputs, constants and the results of operations on exact operands are exact (IEEE arithmetic is deterministic);
  * a cheap routine adds its measured worst distance from the host library (`ROUTINE_ULPS`);
  * negation, absolute value, minimum and maximum keep the operands' distance;
  * an operation that rounds turns a distance of D result-ulp between the unrounded values into at most floor(D) + 1
    steps (the two roundings can go opposite ways, also on ties): a sum of operands of one sign has D = the sum of
    the operands' distances, so it adds one; a product or quotient has D up to twice that sum (the ulp of the result
    can be half as large relative to its value as the ulp of an operand); a sum that can cancel scales by the worst
    ratio of the operand's ulp to the result's ulp over the value ranges (`ranges.py`), unbounded when the result can
    be zero;
  * a comparison with an inexact operand that the value ranges do not decide makes everything it controls unbounded,
    and so does any use of an inexact value as an integer, an index or an argument of a routine that has no rule here.

So a cheap routine passes when its result is stored as it is (or negated, clamped, ...), and a cheap division when it
is the last operation; anything computed from an inexact value loses at least one more step.  Composite formulas are
therefore handled as units: the reference's sigmoid, log1p and expm1 formulas are recognised in the DAG
(`match_idiom`) and replaced by one routine each, whose distance from the formula (evaluated with the host library)
was measured on every float32 argument of a domain; the replacement happens only when the value range of the argument
lies inside that domain.

While a stored value (or a stage's result) exceeds the tolerance, one of the call sites it depends on is switched back
to the bit-compatible routine: one that repairs the value on its own if there is one (the cheapest such), else the last
in program order.  With every site switched back all bounds are zero, so the loop ends; sites that were switched back
without need get their cheap routine again afterwards.
"""

import math

import numpy as np

from .. import language as lang

INF = float('inf')

#: the promise of the mode, in float32 units in the last place per operator output
TOLERANCE = 2

#: marker the fusion optimizer puts into ``io_index`` of a VARIABLE that stands for an internalised operator output
STAGE_VARIABLE = 1

#: worst distance of the routines of csrc/ovl_fast_math.h from the host C library over all 2^32 arguments (the
#: division: from the correctly rounded quotient), and of the once-rounded log1p / expm1 of csrc/ovl_math.h from the
#: reference's formulas evaluated with the host C library over every argument of `IDIOM_DOMAIN`; asserted by
#: tests/test_gpu_math_exhaustive.py
ROUTINE_ULPS = {lang.TANH: 2, lang.EXP: 1, lang.LOG: 2, lang.DIVIDE: 1, 'sigmoid': 2, 'log1p': 2, 'expm1': 2,
                'sigmoid_guarded': 2, 'log1p_guarded': 2, 'expm1_guarded': 2}

#: what a site saves when it may use the cheap routine (issue clocks per element, measured); orders the repairs
_GAIN = {lang.TANH: 225, lang.EXP: 60, lang.LOG: 50, lang.DIVIDE: 19, 'sigmoid': 60, 'log1p': 25, 'expm1': 100,
         'sigmoid_guarded': 50, 'log1p_guarded': 15, 'expm1_guarded': 90}

#: argument ranges on which the once-rounded routines were compared with the reference's formulas
IDIOM_DOMAIN = {'sigmoid': (-16.0, 64.0), 'log1p': (2.0 ** -10, 2.0 ** 64), 'expm1': (2.0 ** -12, 64.0)}

#: A formula whose argument's range is not known to lie in `IDIOM_DOMAIN` (it comes straight from a tensor: every
#: sigmoid of an LSTM cell, opveclib/stdops/math.py:91-93) is replaced behind a test at run time: when every lane of
#: the wavefront holds an argument inside these intervals the once-rounded routine runs, otherwise the wavefront
#: evaluates the formula itself with the bit-compatible routines.  Either way the value is within `TOLERANCE` of the
#: reference's.  The intervals are those on which the routines were compared with the formulas on every float32
#: argument: `IDIOM_DOMAIN`, for log1p also the negative arguments down to the last float32 above -1, for expm1 the
#: negative ones from -2^-5 down (between -2^-5 and -2^-10 the reference's formula is itself up to 2.5 ulp from the
#: function, so a few arguments differ by 3).
GUARD_DOMAIN = {'sigmoid': ((-16.0, 64.0),),
                'log1p': ((-(1.0 - 2.0 ** -24), -(2.0 ** -10)), (2.0 ** -10, 2.0 ** 64)),
                'expm1': ((-64.0, -(2.0 ** -5)), (2.0 ** -12, 64.0))}
#: kind of a guarded call site -> the formula it stands for
GUARDED = {'sigmoid_guarded': 'sigmoid', 'log1p_guarded': 'log1p', 'expm1_guarded': 'expm1'}

#: narrower argument ranges on which shorter forms of the once-rounded routines hold the same bound (also compared
#: with the formulas on every argument): for 2^-4 <= x < 1 the sum 1 + x has a known exponent (`ovl_log1p_unit`), up
#: to 0.68 the exponential's table entry needs no exponent (`ovl_expm1_small`), from -1 on the sigmoid's exponential
#: needs no second term for the rounding of its scaled argument (`ovl_sigmoid_small`).  About a tenth fewer
#: instructions in the 8-op chain; that kernel runs at the board's power limit, so its time follows the instruction
#: count (143-147 -> 133-137 us on one box).
NARROW_DOMAIN = {'log1p': (2.0 ** -4, float(np.nextafter(np.float32(1.0), np.float32(0.0)))),
                 'expm1': (2.0 ** -12, float(np.float32(0.68))),
                 'sigmoid': (-1.0, 64.0)}


def in_narrow_domain(kind, seen):
    """Whether the value range ``seen`` of an idiom's argument (NaN aside) lies in the kind's narrow domain."""
    if kind not in NARROW_DOMAIN or seen is None:
        return False
    lo, hi = NARROW_DOMAIN[kind]
    return seen.lo >= lo and seen.hi <= hi

_COMPARISONS = (lang.EQUAL, lang.NOTEQUAL, lang.LESS, lang.LESS_EQ, lang.GREATER, lang.GREATER_EQ)
_BOOLEAN = _COMPARISONS + (lang.AND, lang.OR, lang.NOT, lang.ISINF, lang.ISNAN, lang.ISFINITE)
_NO_SITES = frozenset()


def _ulp32(v):
    """Size of one float32 step at magnitude ``v`` (the smallest step for zero and subnormal magnitudes)."""
    v = abs(float(v))
    if v == INF or v != v:
        return INF
    return max(float(np.spacing(np.float32(v))), float(np.finfo(np.float32).smallest_subnormal))


def _is_one(info, idx):
    """The expression is the literal 1, directly or through casts."""
    node = info.nodes[idx]
    while node.code == lang.CAST:
        node = info.nodes[node.ops[0]]
    return node.code == lang.CONST_SCALAR and len(node.data) == 1 and float(node.data[0]) == 1.0


def _same_value(info, a, b, depth=12):
    """Two expressions certainly hold the same value: the same node, or pure expressions of the same operation on
    operands that hold the same values (a worker that writes ``x[pos]`` twice reads the tensor twice; inputs are
    never written, and positions do not change)."""
    if a == b:
        return True
    if depth == 0:
        return False
    na, nb = info.nodes[a], info.nodes[b]
    if na.code != nb.code or na.dtype != nb.dtype or len(na.ops) != len(nb.ops):
        return False
    if na.code == lang.CONST_SCALAR:
        return list(na.data) == list(nb.data)
    if na.code in (lang.INPUT, lang.POSITION):
        return False                    # (the same tensor is the same node)
    if na.code == lang.READ_TENSOR:
        if info.nodes[na.ops[0]].code not in (lang.INPUT, lang.POSITION) or info.in_loop.get(a) or info.in_loop.get(b):
            return False
    elif na.code not in (lang.CAST, lang.ADD, lang.SUBTRACT, lang.MULTIPLY, lang.NEGATE):
        return False
    return all(_same_value(info, x, y, depth - 1) for x, y in zip(na.ops, nb.ops))


def _match_formula(info, node):
    """The structure of `match_idiom` without the condition on the argument's range: (kind, index of x, index of the
    expression that takes x, which of its operands x is) or None."""
    nodes = info.nodes
    if node.code != lang.DIVIDE or node.dtype != lang.FLOAT32:
        return None
    product, divisor = nodes[node.ops[0]], nodes[node.ops[1]]

    def one_plus(idx):
        """x when expression idx is 1 + x or x + 1, else None."""
        n = nodes[idx]
        if n.code != lang.ADD:
            return None
        if _is_one(info, n.ops[0]):
            return n.ops[1]
        if _is_one(info, n.ops[1]):
            return n.ops[0]
        return None

    def finish(kind, x, user, operand, parts):
        first = min(parts)
        # the formula's parts must all have seen the same x
        if nodes[x].code == lang.VARIABLE and any(n.code == lang.ASSIGN_VARIABLE and n.ops[0] == x
                                                  for n in nodes[first:node.idx]):
            return None
        if info.in_loop.get(node.idx):
            return None
        return kind, x, user, operand

    if _is_one(info, node.ops[0]):
        inner = one_plus(divisor.idx)
        e = nodes[inner] if inner is not None else None
        if e is not None and e.code == lang.EXP and nodes[e.ops[0]].code == lang.NEGATE:
            negation = nodes[e.ops[0]]
            return finish('sigmoid', negation.ops[0], negation.idx, 0, (negation.idx, e.idx, divisor.idx))
        return None
    if product.code != lang.MULTIPLY or product.dtype != lang.FLOAT32:
        return None

    found = None
    for first, x in ((product.ops[0], product.ops[1]), (product.ops[1], product.ops[0])):
        factor = nodes[first]
        if factor.code == lang.LOG and divisor.code == lang.SUBTRACT and divisor.ops[0] == factor.ops[0] and \
                _is_one(info, divisor.ops[1]) and one_plus(factor.ops[0]) is not None and \
                _same_value(info, one_plus(factor.ops[0]), x):
            found = ('log1p', x, (factor.ops[0],))
        elif factor.code == lang.SUBTRACT and _is_one(info, factor.ops[1]) and divisor.code == lang.LOG and \
                divisor.ops[0] == factor.ops[0] and nodes[factor.ops[0]].code == lang.EXP and \
                _same_value(info, nodes[factor.ops[0]].ops[0], x):
            found = ('expm1', x, (factor.ops[0],))
        if found:
            break
    if found is None:
        return None
    kind, x, parts = found
    return finish(kind, x, product.idx, 0 if product.ops[0] == x else 1, parts + (product.idx, divisor.idx))


def match_idiom(info, known, node):
    """
    Recognise, at the division that ends them, the reference's formulas for the logistic function
    (opveclib/stdops/math.py:93) and its numerically careful ones for log(1 + x) and exp(x) - 1
    (opveclib/examples/test_log1p.py:55-60, test_expm1.py:57-61):

        sigmoid:  1 / (1 + exp(-x))
        log1p:    log(u) * x / (u - 1)   with u = 1 + x
        expm1:    (e - 1) * x / log(e)   with e = exp(x)

    Returns (kind, index of x, value range of x there) when ``node`` is such a division in float32 and the range lies
    inside the domain on which the once-rounded routine was compared with the formula, else None.  (The formulas exist to avoid
    the rounding of ``1 + x`` and the cancellation in ``e - 1``; a routine that forms the result in double precision
    and rounds it once has neither problem.)
    """
    if known is None:
        return None
    found = _match_formula(info, node)
    if found is None:
        return None
    kind, x, user, operand = found
    lo, hi = IDIOM_DOMAIN[kind]
    seen = known.operand(user, operand)
    if seen is None or not seen.within(lo, hi):
        return None
    return kind, x, seen


def match_guarded(info, known, node):
    """(kind, index of x) when ``node`` is the division that ends one of the formulas of `match_idiom` and the range
    of x is not known to lie in the compared domain: the replacement then happens behind a test of the arguments at
    run time (`GUARD_DOMAIN`).  None for a formula `match_idiom` already takes, and for anything else."""
    found = _match_formula(info, node)
    if found is None or match_idiom(info, known, node) is not None:
        return None
    return found[0], found[1]


def site_kind(info, known, node):
    """What kind of call site the expression is: 'log1p' / 'expm1' for a recognised formula, its own code for a
    float32 tanh, exp, log or division (``1/x`` excepted: the reciprocal of csrc/ovl_math.h is correctly rounded and
    already the cheapest form), else None."""
    if node.dtype != lang.FLOAT32 or node.code not in ROUTINE_ULPS:
        return None
    if node.code == lang.DIVIDE:
        idiom = match_idiom(info, known, node)
        if idiom is not None:
            return idiom[0]
        guarded = match_guarded(info, known, node)
        if guarded is not None:
            return guarded[0] + '_guarded'
        if _is_one(info, node.ops[0]):
            return None
    return node.code


class _Bound(object):
    """Distance bound of one value: ``ulps`` float32 steps (INF: unbounded), depending on call sites ``sites``."""
    __slots__ = ('ulps', 'sites')

    def __init__(self, ulps=0, sites=_NO_SITES):
        self.ulps = ulps
        self.sites = sites if ulps else _NO_SITES


_EXACT = _Bound()


def _join(bounds):
    bounds = [b for b in bounds if b is not None]
    if not bounds:
        return _EXACT
    sites = _NO_SITES
    for b in bounds:
        sites = sites | b.sites
    return _Bound(max(b.ulps for b in bounds), sites)


class _Violation(Exception):
    def __init__(self, bound, where):
        Exception.__init__(self)
        self.bound = bound
        self.where = where              # index of the violating statement


class _Interpreter(object):
    """One pass over the worker with a fixed assignment of routines to call sites."""

    def __init__(self, info, known, cheap, kinds):
        self.info = info
        self.known = known
        self.cheap = cheap                  # set of call-site node indices that use the cheap routine
        self.kinds = kinds                  # call-site node index -> kind (see site_kind)
        self.value = {}                     # node index -> _Bound (float32 values and 0/1 results)
        self.control = []                   # stack of _Bound: the conditions the current statement depends on

    # -- helpers -----------------------------------------------------------------------------------------------------
    def _range(self, idx, k=None):
        if self.known is None:
            return None
        return self.known.ranges.get(idx) if k is None else self.known.operand(idx, k)

    def _get(self, idx, env):
        node = self.info.nodes[idx]
        if node.code in (lang.VARIABLE, lang.TENSOR):
            return env.get(idx, _EXACT)
        return self.value.get(idx, _EXACT)

    def _controlled(self, bound):
        """``bound`` joined with the conditions in force: an inexact condition makes what it controls unbounded."""
        if not any(c.ulps for c in self.control):
            return bound
        sites = bound.sites
        for c in self.control:
            sites = sites | c.sites
        return _Bound(INF, sites)

    # -- statements ----------------------------------------------------------------------------------------------------
    def run(self, items, env):
        nodes = self.info.nodes
        for item in items:
            if item.kind == 'stmt':
                self._statement(nodes[item.node], env)
            elif item.kind == 'loop':
                header = _join([self._get(o, env) for o in nodes[item.node].ops[1:]])
                self.control.append(header)
                before = dict(env)
                self.run(item.body, env)
                # a distance that grows in one trip grows without bound over the trips
                grown = [v for v in env if env[v].ulps > before.get(v, _EXACT).ulps]
                if grown:
                    for v in grown:
                        env[v] = _Bound(INF, env[v].sites)
                    self.run(item.body, env)
                self.control.pop()
            else:
                exits = []
                earlier = []
                for cond, body in item.branches:
                    if cond is not None:
                        earlier.append(self._get(cond, env))
                    self.control.append(_join(earlier))
                    branch_env = dict(env)
                    self.run(body, branch_env)
                    self.control.pop()
                    exits.append(branch_env)
                if not item.has_else:
                    exits.append(dict(env))
                chain = _join(earlier)
                merged = {}
                for var in set().union(*[set(e) for e in exits]):
                    joined = _join([e.get(var) for e in exits])
                    changed = any(e.get(var) is not env.get(var) for e in exits)
                    if changed and chain.ulps:
                        joined = _Bound(INF, joined.sites | chain.sites)
                    merged[var] = joined
                env.clear()
                env.update(merged)

    def _statement(self, node, env):
        code, dtype = node.code, node.dtype
        nodes = self.info.nodes
        ops = [self._get(o, env) for o in node.ops]

        if code == lang.ASSIGN_VARIABLE:
            var = nodes[node.ops[0]]
            bound = self._controlled(ops[1])
            if var.code == lang.VARIABLE and var.io_index == STAGE_VARIABLE:
                # the result of one operator of a fused chain: held to the tolerance, and the next operator's input
                if bound.ulps > TOLERANCE:
                    raise _Violation(bound, node.idx)
                bound = _EXACT
            env[var.idx] = bound
            return
        if code == lang.ASSIGN_TENSOR:
            tensor = nodes[node.ops[0]]
            bound = self._controlled(_join([ops[2], _Bound(INF, ops[1].sites) if ops[1].ulps else None]))
            if tensor.code == lang.OUTPUT:
                if bound.ulps > TOLERANCE:
                    raise _Violation(bound, node.idx)
            else:
                env[tensor.idx] = _join([env.get(tensor.idx), bound])      # a worker-local tensor: any element
            return
        if code in (lang.VARIABLE, lang.CAST):
            source = nodes[node.ops[0]]
            bound = ops[0]
            if bound.ulps and not (dtype == lang.FLOAT32 and source.dtype == lang.FLOAT32):
                bound = _Bound(INF, bound.sites)
            if code == lang.VARIABLE:
                env[node.idx] = bound
            else:
                self.value[node.idx] = bound
            return
        if code == lang.TENSOR:
            env[node.idx] = ops[0] if ops else _EXACT
            return
        if code == lang.READ_TENSOR:
            tensor = nodes[node.ops[0]]
            bound = ops[0] if tensor.code == lang.TENSOR else _EXACT
            if ops[1].ulps:
                bound = _Bound(INF, bound.sites | ops[1].sites)
            self.value[node.idx] = bound
            return
        if code in (lang.INPUT, lang.OUTPUT, lang.POSITION, lang.CONST_SCALAR, lang.CONST_TENSOR, lang.MIN_VALUE,
                    lang.MAX_VALUE, lang.EPSILON, lang.RANGE, lang.ENDRANGE, lang.IF, lang.ELSEIF, lang.ELSE,
                    lang.ENDIF):
            return
        if self.kinds.get(node.idx) in GUARDED and node.idx in self.cheap:
            # the once-rounded routine where the arguments allow it, else the formula with the bit-compatible
            # routines: within the routine's distance of the reference either way, given an exact x
            kind, x = match_guarded(self.info, self.known, node)
            bound = self._get(x, env)
            sites = bound.sites | frozenset([node.idx])
            self.value[node.idx] = _Bound(INF if bound.ulps else ROUTINE_ULPS[kind], sites)
            return
        if self.kinds.get(node.idx) in IDIOM_DOMAIN and node.idx in self.cheap:
            # the once-rounded routine takes x itself: nothing of the formula's parts enters
            kind, x, seen = match_idiom(self.info, self.known, node)
            bound = self._get(x, env)
            sites = bound.sites | frozenset([node.idx])
            ulps = ROUTINE_ULPS[kind]
            if bound.ulps:
                condition = 1.0 if kind == 'log1p' else max(abs(seen.lo), abs(seen.hi)) + 1.0
                ulps = INF if bound.ulps == INF else int(math.ceil(2.0 * condition * bound.ulps)) + 2 + ulps
            self.value[node.idx] = _Bound(ulps, sites)
            return
        self.value[node.idx] = self._operation(node, ops)

    # -- values --------------------------------------------------------------------------------------------------------
    def _operation(self, node, ops):
        code, dtype = node.code, node.dtype
        inexact = [b for b in ops if b.ulps]
        sites = _NO_SITES
        for b in inexact:
            sites = sites | b.sites
        is_site = node.idx in self.cheap and self.kinds.get(node.idx) == code
        own = ROUTINE_ULPS[code] if is_site else 0
        if is_site:
            sites = sites | frozenset([node.idx])

        if code in _BOOLEAN:
            if not inexact or (self.known is not None and self.known.constant(node.idx) is not None):
                return _EXACT
            return _Bound(INF, sites)
        if not inexact:
            return _Bound(own, sites)
        if dtype != lang.FLOAT32 or any(b.ulps == INF for b in inexact):
            return _Bound(INF, sites)

        total = sum(b.ulps for b in inexact)
        second_order = 1 if len(inexact) > 1 else 0
        if code in (lang.NEGATE, lang.ABS):
            return _Bound(total, sites)
        if code in (lang.MIN, lang.MAX):
            return _Bound(max(b.ulps for b in inexact), sites)
        # operations that round: unrounded values D result-ulp apart end up at most floor(D) + 1 steps apart
        if code in (lang.ADD, lang.SUBTRACT):
            return _Bound(self._sum(node, ops) + 1, sites)
        if code == lang.MULTIPLY:
            return _Bound(2 * total + second_order + 1, sites)
        if code == lang.DIVIDE:
            return _Bound(2 * total + second_order + 1 + own, sites)
        # a routine applied to an inexact argument: the argument's distance times the routine's relative condition
        # number, doubled (relative size of an ulp), plus two for the host library's own rounding on either argument
        x = self._range(node.idx, 0)
        condition = None
        if code == lang.TANH:
            condition = 1.0
        elif code == lang.SQRT:
            condition = 0.5
        elif code == lang.EXP and x is not None and x.finite:
            condition = max(abs(x.lo), abs(x.hi))
        elif code == lang.LOG and x is not None and (x.lo > 1.0 or (x.hi < 1.0 and x.lo > 0.0)):
            condition = 1.0 / min(abs(math.log(x.lo)), abs(math.log(x.hi)))
        if condition is None:
            return _Bound(INF, sites)
        return _Bound(int(math.ceil(2.0 * condition * total)) + 2 + own, sites)

    def _sum(self, node, ops):
        """Distance bound of ``a + b`` / ``a - b`` with at least one inexact operand."""
        a, b = self._range(node.idx, 0), self._range(node.idx, 1)
        if a is None or b is None:
            return INF
        if node.code == lang.SUBTRACT:
            b = type(b)(-b.hi, -b.lo, b.nan)
        growing = (a.lo >= 0 and b.lo >= 0) or (a.hi <= 0 and b.hi <= 0)
        if growing:
            # |a + b| is at least as large as either operand: a step of an operand is at most a step of the sum
            return sum(bound.ulps for bound in ops)
        z = self._range(node.idx)
        if z is None or not z.finite or not (z.lo > 0 or z.hi < 0):
            return INF
        step = _ulp32(z.magnitude()[0])
        total = 0.0
        for bound, r in zip(ops, (a, b)):
            if bound.ulps:
                if not r.finite:
                    return INF
                total += bound.ulps * _ulp32(r.magnitude()[1]) / step
        return int(math.floor(total))


def _violation(info, known, cheap, kinds):
    try:
        _Interpreter(info, known, cheap, kinds).run(info.tree, {})
    except _Violation as found:
        return found
    return None


def candidate_sites(info, known):
    """{node index: kind} of the call sites that have a cheap routine."""
    kinds = {}
    for node in info.nodes:
        kind = site_kind(info, known, node)
        if kind is not None:
            kinds[node.idx] = kind
    return kinds


def formula_sites(info, known):
    """{node index: kind} of the divisions that end a recognised sigmoid / log1p / expm1 formula (kind + '_guarded'
    when the argument is not known to lie in the compared domain).  The 'fast' math mode replaces these too: the one
    routine is both closer to the reference and shorter than the formula composed of cheap routines."""
    return dict((idx, kind) for idx, kind in candidate_sites(info, known).items()
                if kind in IDIOM_DOMAIN or kind in GUARDED)


def cheap_sites(info, known):
    """The call sites that do not use the bit-compatible routine, by math mode: none ('exact'), those `select` allows
    ('ulp2'); for 'fast', where every routine is the cheap one anyway, the recognised formulas."""
    mode = getattr(info, 'math', 'exact')
    if mode == 'ulp2':
        return select(info, known)
    if mode == 'fast':
        return formula_sites(info, known)
    return {}


def select(info, known):
    """
    ``{node index: kind}`` of the call sites that may use the cheap routine while every operator output stays within
    `TOLERANCE` ulp of the reference's value; all other sites use the bit-compatible routine.  ``kind`` is the
    expression code of a tanh, exp, log or division, or 'log1p' / 'expm1' for a division that ends one of the
    reference's formulas and is replaced by the once-rounded routine (see `match_idiom`).
    """
    cached = getattr(info, '_cheap_sites', None)
    if cached is not None:
        return cached
    kinds = candidate_sites(info, known)
    cheap = set(kinds)
    removed = []
    while cheap:
        found = _violation(info, known, cheap, kinds)
        if found is None:
            break
        suspects = sorted(found.bound.sites & cheap)
        if not suspects:
            raise AssertionError('an inexact value that depends on no call site')
        repairs = []
        for site in suspects:
            after = _violation(info, known, cheap - set([site]), kinds)
            # repaired when the pass gets further than before: nothing is violated, or a later statement is
            if after is None or after.where > found.where:
                repairs.append(site)
        if repairs:
            site = min(repairs, key=lambda s: (_GAIN[kinds[s]], -s))
        else:
            site = suspects[-1]
        cheap.discard(site)
        removed.append(site)
    # a site switched back before the one that mattered may not have needed it: give those their cheap routine again
    for site in sorted(removed, key=lambda s: -_GAIN[kinds[s]]):
        if _violation(info, known, cheap | set([site]), kinds) is None:
            cheap.add(site)
    info._cheap_sites = dict((site, kinds[site]) for site in cheap)
    return info._cheap_sites
