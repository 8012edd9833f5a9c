# Derived from opveclib/operator.py of opveclib (https://github.com/opveclib/opveclib),
# Copyright 2016 Hewlett Packard Enterprise Development LP, licensed under the Apache License, Version 2.0
# (http://www.apache.org/licenses/LICENSE-2.0); see the NOTICE file at the root of this repository.
# Changes: the decorator, the lazy operator handles and the operator DAG builder follow that file's interface and error
# messages; tracing caches, the re-binding check on current bytecode, evaluation on device tensors and the launcher are new.
"""
Operator front-end: the ``@operator`` decorator, lazy operator handles, gradient registration, the operator-DAG
builder and the ``evaluate``/``profile`` entry points that run a DAG of operators on the GPU.

Behavioural counterpart of the reference's opveclib/operator.py:128-806 and 2099-2335.  ``evaluate`` and ``profile``
keep their signatures; the only supported ``target_language`` is ``'hip'``: every operator of the (optionally fused)
DAG is turned into a HIP kernel for gfx950, compiled with hipcc, loaded through the C-ABI launcher and enqueued on the
current PyTorch HIP stream.  There is no CPU execution path in this package.
"""

import dis
import hashlib
import inspect
import threading
import types
from collections import namedtuple

import numpy as np

from . import language as lang
from .expression import TensorType, ExpressionDAG, input, OutputTensor
from .local import version, logger


class _TensorParam(object):
    """Placeholder kept for API familiarity; the launcher's parameter struct lives in ``opveclib_amd.launcher``."""


# ----------------------------------------------------------------------------------------------------------------------
# lazy handles
# ----------------------------------------------------------------------------------------------------------------------
_INFIX = (('add', '__add__', '__radd__'), ('sub', '__sub__', '__rsub__'), ('mul', '__mul__', '__rmul__'),
          ('div', '__truediv__', '__rtruediv__'), ('mod', '__mod__', '__rmod__'))
_COMPARE = (('eq', '__eq__'), ('ne', '__ne__'), ('lt', '__lt__'), ('le', '__le__'), ('gt', '__gt__'),
            ('ge', '__ge__'))


class OperatorOutput(object):
    """
    An un-evaluated output tensor of an operator, used for building lazily evaluated DAGs of operators
    (operator.py:134-221).  Infix arithmetic dispatches to the element-wise operators that
    ``opveclib_amd.stdops`` registers with :meth:`register_magic_method`.
    """

    # raise operator priority so that numpy does not try to use its own operator
    __array_priority__ = 1
    _builtin_ops = {}

    @staticmethod
    def register_magic_method(key, value):
        OperatorOutput._builtin_ops[key] = value

    def __init__(self, parent, index):
        if not isinstance(parent, _Operator):
            raise TypeError('parent must be an Operator')
        if not isinstance(index, int):
            raise TypeError('index must be an int')

        self.parent = parent
        self.index = index
        self.tensor_type = parent.output_types[index]
        self.shape = self.tensor_type.shape
        self.dtype = self.tensor_type.dtype
        self.size = self.tensor_type.size
        self.rank = self.tensor_type.rank

    def __neg__(self):
        return OperatorOutput._builtin_ops['neg'](self)

    def __bool__(self):
        raise SyntaxError('Cannot resolve operator values at interpretation time.')

    __hash__ = None


class _Operator(object):
    """
    One application of an operator function to concrete input types: its expression DAG, output types, inputs
    and (optionally) its gradient DAG (operator.py:232-334).  Indexing yields :class:`OperatorOutput` handles.
    """

    __array_priority__ = 1

    def __init__(self, dag, output_types, inputs, grad_dag, from_gradient, name):
        self.inputs = inputs
        self.expression_dag = dag
        self.output_types = output_types
        self.name = name
        self.grad_dag = grad_dag
        self.from_gradient = from_gradient
        logger.debug('Operator created: ' + str(dag.name))

    def __getitem__(self, item):
        if not isinstance(item, int):
            raise TypeError('index must be an int')
        if item < 0 or item >= len(self.output_types):
            raise IndexError('operator ' + str(self.name) + ' has ' + str(len(self.output_types)) + ' outputs')
        return OperatorOutput(self, item)

    def __len__(self):
        return len(self.output_types)

    def check_binary(self):
        if len(self.output_types) != 1:
            raise SyntaxError('Cannot use binary infix operators on multi-output operators. '
                              'Explicitly index an output.')

    def __neg__(self):
        self.check_binary()
        return -self[0]

    __hash__ = None


def _install_infix():
    def out_forward(key):
        return lambda self, other: OperatorOutput._builtin_ops[key](self, other)

    def out_reverse(key):
        return lambda self, other: OperatorOutput._builtin_ops[key](other, self)

    def op_forward(dunder):
        def method(self, other):
            self.check_binary()
            return getattr(self[0], dunder)(other)
        return method

    for key, fwd, rev in _INFIX:
        setattr(OperatorOutput, fwd, out_forward(key))
        setattr(OperatorOutput, rev, out_reverse(key))
        setattr(_Operator, fwd, op_forward(fwd))
        setattr(_Operator, rev, op_forward(rev))
    for key, dunder in _COMPARE:
        setattr(OperatorOutput, dunder, out_forward(key))
        setattr(_Operator, dunder, op_forward(dunder))
    OperatorOutput.__div__ = OperatorOutput.__truediv__
    OperatorOutput.__rdiv__ = OperatorOutput.__rtruediv__


_install_infix()


class _GradientPlaceholder(object):
    """Stands for an operator input or an upstream gradient while a gradient function is traced."""

    def __init__(self, shape, dtype):
        self.tensor_type = TensorType(shape, dtype)
        self.rank = self.tensor_type.rank
        self.shape = shape
        self.dtype = dtype


def _resolve_output(x):
    """
    Convert single-output Operators to an OperatorOutput (operator.py:337-354).

    :raises ValueError: When argument is a multi-output Operator
    :raises TypeError: When argument is neither an Operator nor an OperatorOutput
    """
    if isinstance(x, _Operator):
        if len(x.output_types) != 1:
            raise ValueError('Only a single-output Operator can be used as an input to another operator. '
                             'Index a specific output from multi-output Operators.')
        return x[0]
    if not isinstance(x, OperatorOutput):
        raise TypeError('Only operator outputs can be used to build an op dag. Received a ' + str(type(x)))
    return x


_frozen_hashes = {}      # id(expression DAG message) -> (the message, its content name)


def _freeze_op(op):
    """Declare that ``op`` (an ExpressionDAG message) will not be modified any more; its name is computed once."""
    entry = _frozen_hashes.get(id(op))
    if entry is None or entry[0] is not op:
        entry = (op, 'f' + hashlib.sha224(op.SerializeToString() + version.encode('utf-8')).hexdigest())
        _frozen_hashes[id(op)] = entry
    return entry[1]


def _op_hash(op):
    """Content name of an operator: 'f' + sha224(serialised DAG + library version) (operator.py:357-358)."""
    entry = _frozen_hashes.get(id(op))
    if entry is not None and entry[0] is op:
        return entry[1]
    return 'f' + hashlib.sha224(op.SerializeToString() + version.encode('utf-8')).hexdigest()


# ----------------------------------------------------------------------------------------------------------------------
# tracing
# ----------------------------------------------------------------------------------------------------------------------
def _as_list(x):
    try:
        len(x)
    except TypeError:
        return [x]
    return list(x)


def _with_full_inputs(found_dag, full_inputs):
    """
    A traced gradient DAG may use only some of its possible inputs, in any order.  Return a copy of its proto whose
    ``dag_input_types`` list all of ``full_inputs`` in order and whose leaf references are renumbered to match
    (operator.py:526-553).
    """
    remap = {}
    for found_index, found_input in enumerate(found_dag.inputs):
        for full_index, candidate in enumerate(full_inputs):
            if candidate is found_input:
                remap[found_index] = full_index
                break
        else:
            raise ValueError('Gradient DAG depends on a tensor that is not one of its declared inputs.')

    reordered = lang.OperatorDAG()
    reordered.operators.extend(found_dag.proto_dag.operators)       # traced expression DAGs are shared, not copied
    for ref in found_dag.proto_dag.references:
        reordered.references.add().CopyFrom(ref)
    for ref in found_dag.proto_dag.dag_outputs:
        reordered.dag_outputs.add().CopyFrom(ref)
    for placeholder in full_inputs:
        reordered.dag_input_types.add().CopyFrom(placeholder.tensor_type.as_proto())
    for ref in reordered.references:
        for input_ref in ref.input_refs:
            if input_ref.is_leaf:
                input_ref.dag_input_index = remap[input_ref.dag_input_index]
    return reordered


class _Uncacheable(Exception):
    pass


def _freeze(value):
    """A hashable stand-in that distinguishes any two constants an operator function could tell apart."""
    if value is None or isinstance(value, (bool, str, bytes)):
        return (type(value).__name__, value)
    if isinstance(value, int):
        return ('int', value)
    if isinstance(value, float):
        return ('float', value.hex())
    if isinstance(value, (tuple, list)):
        return (type(value).__name__,) + tuple(_freeze(v) for v in value)
    if isinstance(value, np.generic):
        return ('numpy', value.dtype.str, value.tobytes())
    if isinstance(value, np.ndarray) and value.size <= 4096:
        return ('ndarray', value.dtype.str, value.shape, value.tobytes())
    if isinstance(value, np.dtype):
        return ('numpy dtype', value.str)
    from .expression import DType as _DType
    if isinstance(value, _DType):
        return ('ovl dtype', value.proto_dtype)
    if isinstance(value, type):
        return ('type', value)
    if isinstance(value, types.FunctionType):
        # a function passed as a constant (accumulate's inner function): the same code with the same defaults and
        # surroundings is the same function, even when a lambda expression creates a new object on every call
        return ('function', value.__code__, tuple(_freeze(d) for d in (value.__defaults__ or ())),
                _environment_key(value))
    if type(value).__module__ == 'torch' and type(value).__name__ == 'dtype':
        return ('torch dtype', str(value))
    raise _Uncacheable()


class _ById(object):
    """Key component for an object compared by identity; holds the object, so its id cannot be re-used by another
    object while a cache entry refers to it."""
    __slots__ = ('obj',)

    def __init__(self, obj):
        self.obj = obj

    def __hash__(self):
        return id(self.obj)

    def __eq__(self, other):
        return isinstance(other, _ById) and other.obj is self.obj

    def __ne__(self, other):
        return not self == other


def _freeze_environment_value(value):
    # functions, modules and classes that an operator function names count by identity (looking into them would
    # never end for functions that name each other); so does anything else that cannot be frozen by value
    if isinstance(value, (types.FunctionType, types.ModuleType, type, types.BuiltinFunctionType)):
        return _ById(value)
    try:
        return _freeze(value)
    except _Uncacheable:
        return _ById(value)


_code_names_cache = {}


def _code_names(code):
    """Global names a code object refers to, nested functions and lambdas included (code objects are immutable)."""
    names = _code_names_cache.get(code)
    if names is None:
        names = list(code.co_names)
        for const in code.co_consts:
            if hasattr(const, 'co_names'):
                names.extend(_code_names(const))
        names = tuple(dict.fromkeys(names))
        _code_names_cache[code] = names
    return names


def _environment_key(function):
    """
    What an operator function can see besides its arguments: the contents of its closure cells and the globals its
    code names.  Part of the trace key, so rebinding such a name to another value (``scale = 3``) traces again;
    objects that cannot be frozen count by identity (changing one in place is not noticed).
    """
    code = function.__code__
    items = []
    for name, cell in zip(code.co_freevars, function.__closure__ or ()):
        try:
            items.append((name, _freeze_environment_value(cell.cell_contents)))
        except ValueError:                  # an empty cell
            items.append((name, ('empty',)))
    module_globals = function.__globals__
    for name in _code_names(code):
        if name in module_globals:
            items.append((name, _freeze_environment_value(module_globals[name])))
    return tuple(items)


_trace_lock = threading.RLock()

#: re-use the trace of an operator function applied again to the same input types and constants
trace_cache_enabled = [True]
_MAX_TRACES_PER_OPERATOR = 256


def set_trace_cache(enabled):
    """
    Operator functions are pure functions of their input types, their constants and the closure variables and
    globals they name, so a repeated application with all of those unchanged re-uses the expression DAG (and gradient
    DAG) traced the first time.  Switch this off for operator functions that depend on anything else (an object
    modified in place, a file, a random number).
    """
    trace_cache_enabled[0] = bool(enabled)


class _OpGenerator(object):
    """The callable that ``@operator()`` returns: calling it traces the function for the given input types."""

    def __init__(self, op_function, forbid_none_valued_constants, name):
        self.op_function = op_function
        self.forbid_none_valued_constants = forbid_none_valued_constants
        self.name = op_function.__name__ if name is None else name
        self.grad_function = None
        self._spec = inspect.getfullargspec(op_function)
        self._traces = {}

    def __str__(self):
        return self.op_function.__name__

    def __call__(self, *inputs, **defined_constants):
        # ops applied inside a gradient graph do not get gradient DAGs of their own
        from_gradient = False
        for inp in inputs:
            if getattr(inp, 'from_gradient', False) or isinstance(inp, _GradientPlaceholder):
                from_gradient = True
            elif isinstance(inp, OperatorOutput) and inp.parent.from_gradient:
                from_gradient = True

        spec = self._spec
        if spec.defaults is None:
            input_names = spec.args
            constants = dict(defined_constants)
        else:
            input_names = spec.args[:-len(spec.defaults)]
            constants = dict(zip(spec.args[-len(spec.defaults):], spec.defaults))
            constants.update(defined_constants)

        if self.forbid_none_valued_constants:
            for key in constants.keys():
                if constants[key] is None:
                    raise ValueError(self.name + ' argument ' + key + ' is None, which implies an unset constant.\n'
                                     '  If a None constant is meaningful for this operator, the operator should be '
                                     'defined with the appropriate decorator flag.')

        input_types = []
        for inp_n, inp in enumerate(inputs):
            try:
                inp = _resolve_output(inp)
            except TypeError:
                pass
            try:
                input_types.append(TensorType.like(inp))
            except AttributeError:
                raise TypeError('Unexpectedly received a ' + inp.__class__.__name__ +
                                ' instead of a tensor at argument position ' +
                                str(inp_n + 1) + ' in the call to ' + self.name + '.  '
                                'Should this argument be passed as a constant (keyword argument) instead?')

        num_inputs = len(input_types)
        if len(input_names) != num_inputs and spec.varargs is None:
            err_msg = '\n'
            err_msg += self.name + ' function signature expects ' + str(len(input_names)) + \
                ' input tensor argument(s):\n' + str(input_names) + '\n'
            err_msg += 'but was supplied with ' + str(num_inputs) + '.\n'
            if len(input_names) > num_inputs:
                remaining_names = input_names[num_inputs - len(input_names):]
                err_msg += 'Should ' + str(remaining_names) + ' be passed to constructor as constant?'
            raise TypeError(err_msg)

        trace_key = None
        if trace_cache_enabled[0]:
            try:
                trace_key = (tuple((tuple(t.shape), t.dtype.proto_dtype) for t in input_types),
                             tuple(sorted((k, _freeze(v)) for k, v in constants.items())), from_gradient,
                             _environment_key(self.op_function))
            except _Uncacheable:
                trace_key = None
            else:
                cached = self._traces.get(trace_key)
                if cached is not None and cached[0] is self.grad_function:
                    return _Operator(cached[1], list(cached[2]), inputs, cached[3], from_gradient, self.name)

        expression_dag, output_types = self._trace(input_types, constants)

        grad_dag = None
        if self.grad_function is not None and not from_gradient:
            grad_inputs = [_GradientPlaceholder(t.shape, t.dtype) for t in input_types + output_types]
            grad_outputs = _as_list(self.grad_function(*grad_inputs, **constants))

            # a None among the gradient outputs means "no gradient defined": no gradient DAG at all
            if not any(g is None for g in grad_outputs):
                for grad_output_index, grad_output in enumerate(grad_outputs):
                    if isinstance(grad_output, _Operator) and len(grad_output.output_types) != 1:
                        raise TypeError('A multi-output operator was returned from a gradient function, '
                                        'but the meaning of this is ambiguous: explicitly index each '
                                        'output from operator: ' + str(grad_output.name))
                    cur_input_type = input_types[grad_output_index]
                    cur_grad_output_type = TensorType.like(_resolve_output(grad_output))
                    if cur_input_type != cur_grad_output_type:
                        raise TypeError('Gradient output index ' + str(grad_output_index) + ', with TensorType: ' +
                                        str(cur_grad_output_type) + ' is inconsistent with operator input index ' +
                                        str(grad_output_index) + ', with TensorType: ' + str(cur_input_type))
                grad_dag = _with_full_inputs(_build_op_dag(*grad_outputs), grad_inputs)

        if trace_key is not None:
            if len(self._traces) >= _MAX_TRACES_PER_OPERATOR:
                self._traces.clear()
            _freeze_op(expression_dag)
            self._traces[trace_key] = (self.grad_function, expression_dag, tuple(output_types), grad_dag)
        return _Operator(expression_dag, output_types, inputs, grad_dag, from_gradient, self.name)

    def _trace(self, input_types, constants):
        """Run the operator function on input expressions; returns (expression DAG, output types).  The recorder of
        expressions is one global list (as in the reference, expression.py:250-352), so traces take turns."""
        with _trace_lock:
            ExpressionDAG.clear()
            input_exprs = [input(cur_type) for cur_type in input_types]

            # interpret function to build up ExpressionDAG
            output_exprs = self.op_function(*input_exprs, **constants)
            if output_exprs is None:
                raise ValueError('No outputs returned from op function')
            output_exprs = _as_list(output_exprs)

            if len(output_exprs) != ExpressionDAG.num_outputs:
                raise ValueError('Defined ' + str(ExpressionDAG.num_outputs) + ' outputs, but returned ' +
                                 str(len(output_exprs)) +
                                 '. Number of defined outputs must equal number of returned outputs.')

            # outputs are numbered by return position, not by declaration order, and their declarations are permuted
            # so that they appear in the DAG in that order too
            output_types = []
            slots = []
            for index, expr in enumerate(output_exprs):
                if type(expr) is not OutputTensor:
                    raise TypeError('User functions must only return outputs. Instead got:\n' + str(expr))
                slots.append(ExpressionDAG.expr_index(expr))
                output_types.append(TensorType.like(expr))
            for index, expr in enumerate(output_exprs):
                expr.proto_expr.io_index = index
            for slot, expr in zip(sorted(slots), output_exprs):
                ExpressionDAG.replace(slot, expr)

            expression_dag = ExpressionDAG.as_proto()
            ExpressionDAG.clear()
            expression_dag.name = self.name
            return expression_dag, output_types

    def add_grad(self, grad_function):
        if self.grad_function is not None:
            raise ValueError('Gradient function is already defined for operator ' + str(self.name) + '.')
        self.grad_function = grad_function


def _check_variable_rebinding(op_function):
    """
    A name bound to ``variable(...)`` must afterwards only be updated with ``<<=``; a plain re-assignment would
    silently rebind the Python name instead of emitting an assignment into the operator
    (operator.py:566-641, pinned by test_operator.py:246-278).  Raises SyntaxError at decoration time.
    """
    co = op_function.__code__
    variable_names = set()
    line_instrs = []
    cur_line = None
    prev = None
    for instr in dis.get_instructions(co):
        if instr.starts_line is not None:
            cur_line = instr.starts_line
            line_instrs = []
        if instr.opname == 'STORE_FAST':
            binds_variable = any(i.opname in ('LOAD_GLOBAL', 'LOAD_ATTR', 'LOAD_METHOD') and i.argval == 'variable'
                                 for i in line_instrs)
            via_lshift = prev is not None and (
                prev.opname == 'INPLACE_LSHIFT' or (prev.opname == 'BINARY_OP' and prev.argrepr == '<<='))
            if instr.argval in variable_names and not via_lshift:
                raise SyntaxError('Cannot reassign to symbol "' + instr.argval + '" in operator "' + co.co_name +
                                  '" because it refers to an OVL variable. Use the <<= operator'
                                  ' to assign to OVL variables. \n' +
                                  '  File "' + co.co_filename + '", line ' + str(cur_line))
            if binds_variable:
                variable_names.add(instr.argval)
        line_instrs.append(instr)
        prev = instr


def operator(forbid_none_valued_constants=True, name=None):
    """
    Decorator that turns a worker function into an operator (operator.py:564-648).  Positional parameters of the
    function are tensors, keyword / defaulted parameters are compile-time constants.
    """
    def wrapper(op_function):
        _check_variable_rebinding(op_function)
        op = _OpGenerator(op_function, forbid_none_valued_constants, name)
        op.__name__ = op_function.__name__
        op.__doc__ = op_function.__doc__
        return op

    return wrapper


def gradient(op_function):
    """
    Decorator that registers the gradient of ``op_function`` (operator.py:651-673).  The gradient function receives
    the operator's inputs followed by the gradients of its outputs (plus the same constants) and returns one
    gradient per input; it may itself be an ``@operator()`` or a plain function composing operators.
    """
    if not isinstance(op_function, _OpGenerator):
        raise TypeError('gradient decorator argument must be a function decorated as an operator')

    def wrapper(grad_function):
        if isinstance(grad_function, _OpGenerator):
            def resolved(*args, **defaults):
                op = grad_function(*args, **defaults)
                return [op[output_index] for output_index in range(len(op.output_types))]
        else:
            resolved = grad_function

        op_function.add_grad(resolved)
        resolved.__name__ = grad_function.__name__
        resolved.__doc__ = grad_function.__doc__
        return resolved

    return wrapper


# ----------------------------------------------------------------------------------------------------------------------
# operator DAG
# ----------------------------------------------------------------------------------------------------------------------
_OperatorDAG = namedtuple('_OperatorDAG', ['proto_dag', 'inputs', 'operators', 'grad_dags'])


def _build_op_dag(*outputs):
    """
    Collect every operator the requested outputs depend on (operator.py:679-806).  Operators are ordered by their
    depth in the DAG (ties keep discovery order), tensors that do not come from an operator become DAG inputs
    (deduplicated by identity, in discovery order).

    :param outputs: operator outputs (or single-output operators) from which to build the dag
    :return: an _OperatorDAG(proto_dag, inputs, operators, grad_dags)
    """
    ops = []            # discovery order
    slot_of = {}        # id(op) -> index in ops
    depth = []
    wiring = []         # per op: list of (parent_slot, parent_output, dag_input_index)
    dag_inputs = []
    dag_input_slot = {}

    def visit(node):
        if not isinstance(node, _Operator):
            raise TypeError()
        if id(node) in slot_of:
            return slot_of[id(node)]
        slot = len(ops)
        slot_of[id(node)] = slot
        ops.append(node)
        depth.append(None)
        wiring.append(None)

        edges = []
        deepest_parent = -1
        for cur_input in node.inputs:
            try:
                resolved = _resolve_output(cur_input)
            except TypeError:
                key = id(cur_input)
                if key not in dag_input_slot:
                    dag_input_slot[key] = len(dag_inputs)
                    dag_inputs.append(cur_input)
                edges.append((None, None, dag_input_slot[key]))
            else:
                parent_slot = visit(resolved.parent)
                deepest_parent = max(deepest_parent, depth[parent_slot])
                edges.append((parent_slot, resolved.index, None))
        wiring[slot] = edges
        depth[slot] = deepest_parent + 1
        return slot

    requested = []
    for dag_output in outputs:
        cur_output = _resolve_output(dag_output)
        requested.append((visit(cur_output.parent), cur_output.index))

    order = sorted(range(len(ops)), key=lambda slot: (depth[slot], slot))
    position = dict((slot, new) for new, slot in enumerate(order))
    sorted_ops = [ops[slot] for slot in order]

    op_dag = lang.OperatorDAG()
    for op in sorted_ops:
        # expression DAGs are never modified once traced: the operator DAG shares them instead of copying
        op_dag.operators.append(op.expression_dag)
    for dag_input in dag_inputs:
        op_dag.dag_input_types.add().CopyFrom(TensorType.like(dag_input).as_proto())
    for slot in order:
        ref_list = op_dag.references.add()
        for parent_slot, parent_output, dag_input_index in wiring[slot]:
            proto_ref = ref_list.input_refs.add()
            if parent_slot is None:
                proto_ref.is_leaf = True
                proto_ref.dag_input_index = dag_input_index
            else:
                proto_ref.op_index = position[parent_slot]
                proto_ref.op_output_index = parent_output
    for parent_slot, parent_output in requested:
        proto_ref = op_dag.dag_outputs.add()
        proto_ref.op_index = position[parent_slot]
        proto_ref.op_output_index = parent_output

    grad_dags = [op.grad_dag for op in sorted_ops]
    return _OperatorDAG(proto_dag=op_dag, inputs=dag_inputs, operators=sorted_ops, grad_dags=grad_dags)


# ----------------------------------------------------------------------------------------------------------------------
# evaluation
# ----------------------------------------------------------------------------------------------------------------------
def _normalise_output_list(output_list):
    if isinstance(output_list, (_Operator, OperatorOutput)):
        if isinstance(output_list, _Operator):
            return [output_list[i] for i in range(len(output_list.output_types))]
        return [output_list]
    return list(output_list)


MATH_MODES = ('exact', 'ulp2', 'fast')
_default_math_mode = [None]


def set_math_mode(mode):
    """
    Choose the float32 math library of operators evaluated from now on.

    'ulp2' (the default) keeps every value an operator stores within two float32 units in the last place of what the
    reference's generated C++ computes from the same operator inputs: a static error analysis (hipgen/accuracy.py)
    gives each exp/log/tanh/division call site the hardware-based routine where that bound is proved and the
    bit-compatible one elsewhere.  In a fused chain the bound holds for every operator of the chain given its own
    inputs, not end to end.  (The reference's own GPU path is compiled with --use_fast_math, opveclib/operator.py:2081,
    and its tests loosen their tolerances for it, test/test_unary_math.py:146-161.)
    'exact' reproduces the host C library's expf/logf/tanhf bit for bit and divides with IEEE rounding, so results
    equal those of the reference's generated C++ on the same inputs; it costs about twice the time on chains of
    transcendental operators.  'fast' uses the hardware-based routines and a reciprocal-based division everywhere:
    every single exp/log/tanh and every quotient is within one or two units in the last place of the exact mode's,
    operators composed of several calls can be further off.  Integer and float64 arithmetic, data movement and the
    order of accumulations are the same in 'ulp2' and 'exact'.  The environment variable OPVECLIB_MATH sets the
    initial mode.
    """
    if mode not in MATH_MODES:
        raise ValueError('math mode must be one of ' + str(MATH_MODES))
    _default_math_mode[0] = mode


DEFAULT_MATH_MODE = 'ulp2'


def get_math_mode():
    if _default_math_mode[0] is None:
        import os
        set_math_mode(os.environ.get('OPVECLIB_MATH', DEFAULT_MATH_MODE))
    return _default_math_mode[0]


def evaluate(output_list, target_language='hip', opt_level=3, math_mode=None):
    """
    Evaluate a collection of OVL operator outputs on the GPU (operator.py:2099-2117).

    :param output_list: an operator, an operator output, or a list of either
    :param target_language: must be 'hip'
    :param opt_level: operators are fused when opt_level >= 3
    :param math_mode: 'exact', 'ulp2' or 'fast' for this call (see :func:`set_math_mode`); None uses the current default
    :return: one array for a single requested output, otherwise a list in request order.  Arrays are numpy arrays
        when every DAG input was a numpy array, otherwise torch tensors on the inputs' device.
    """
    evaluated_outputs = _run(output_list, target_language, 1, opt_level, timed=False, math_mode=math_mode)[0]
    if len(evaluated_outputs) == 1:
        return evaluated_outputs[0]
    return evaluated_outputs


def profile(output_list, target_language='hip', profiling_iterations=1, opt_level=3, math_mode=None):
    """
    Evaluate a collection of OVL operator outputs and time every generated operator (operator.py:2120-2335).

    :param profiling_iterations: number of timed launches per operator, a positive int
    :return: (outputs, {operator hash name: float64[profiling_iterations] milliseconds})
    """
    return _run(output_list, target_language, profiling_iterations, opt_level, timed=True, math_mode=math_mode)


def _run(output_list, target_language, profiling_iterations, opt_level, timed, math_mode=None):
    if target_language != 'hip':
        raise ValueError('Unsupported target_language: ' + str(target_language) +
                         '. This package generates HIP kernels for gfx950 only (target_language=\'hip\').')
    if not isinstance(profiling_iterations, int) or profiling_iterations < 1:
        raise ValueError('profiling_iterations must be a positive int')
    if math_mode is None:
        math_mode = get_math_mode()
    if math_mode not in MATH_MODES:
        raise ValueError('math_mode must be one of ' + str(MATH_MODES))

    from .fusion import _merge_op_dag
    from . import runtime

    op_dag = _build_op_dag(*_normalise_output_list(output_list))
    dag = op_dag.proto_dag
    if opt_level >= 3:
        dag, _ = _merge_op_dag(dag, None)
    options = None if math_mode == 'exact' else {'math': math_mode}
    return runtime.run_op_dag(dag, op_dag.inputs, profiling_iterations, timed=timed, options=options)
