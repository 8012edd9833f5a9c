# Derived from opveclib/expression.py of opveclib (https://github.com/opveclib/opveclib),
# Copyright 2016 Hewlett Packard Enterprise Development LP, licensed under the Apache License, Version 2.0
# (http://www.apache.org/licenses/LICENSE-2.0); see the NOTICE file at the root of this repository.
# Changes: class and function names, signatures, the dtype table and the error messages follow that file so that its
# callers and tests run unchanged; the recorder, the schema messages behind it and everything about code generation are new.
"""
The OVL expression language: data types, tensor types and the tracer that records a worker function as an
expression DAG.

Behavioural counterpart of the reference's opveclib/expression.py (DSL half, lines 20-518 and 718-2183).  The user's
operator function is interpreted once with symbolic arguments; every DSL call appends one node to the recorder
(``ExpressionDAG``), which is finally serialised to the schema of :mod:`opveclib_amd.language`.

Differences from the reference that do not change what an operator computes:

* code generation is not part of the expression classes; the HIP emitter (``opveclib_amd.hipgen``) walks the
  serialised DAG instead;
* a constant index (``x[0, 3]``) folds to an integer directly, without leaving an unused CONST_TENSOR node behind
  (reference: expression.py:875-879);
* the ``elif`` hoisting pass visits every dependency once even when a condition shares sub-expressions
  (reference: expression.py:386-392 would list them twice).
"""

import ctypes

import numpy as np

from . import language as lang

_INT_TYPES = (int,)


# ----------------------------------------------------------------------------------------------------------------------
# data types
# ----------------------------------------------------------------------------------------------------------------------
# one row per storage type: (schema code, numpy scalar type, ctypes type, C spelling)
_DTYPE_ROWS = (
    (lang.FLOAT16, np.float16, None, None),
    (lang.FLOAT32, np.float32, ctypes.c_float, 'float'),
    (lang.FLOAT64, np.float64, ctypes.c_double, 'double'),
    (lang.INT8, np.int8, ctypes.c_int8, 'int8_t'),
    (lang.INT16, np.int16, ctypes.c_int16, 'int16_t'),
    (lang.INT32, np.int32, ctypes.c_int32, 'int32_t'),
    (lang.INT64, np.int64, ctypes.c_int64, 'int64_tf'),
    (lang.UINT8, np.uint8, ctypes.c_uint8, 'uint8_t'),
    (lang.UINT16, np.uint16, ctypes.c_uint16, 'uint16_t'),
    (lang.UINT32, np.uint32, ctypes.c_uint32, 'uint32_t'),
    (lang.UINT64, np.uint64, ctypes.c_uint64, 'uint64_t'),
)
_ROW_BY_CODE = dict((row[0], row) for row in _DTYPE_ROWS)


def _code_from_numpy(candidate):
    """Match a numpy scalar type or numpy dtype object by equality (expression.py:78-81); None when unknown."""
    if isinstance(candidate, str):
        # np.dtype('float32') == 'float32' is True in numpy; strings are not valid dtypes here
        return None
    for code, np_type, _, _ in _DTYPE_ROWS:
        try:
            if candidate == np_type:
                return code
        except (TypeError, ValueError):
            continue
    return None


def _code_from_torch(candidate):
    """torch dtypes are accepted so device tensors can be operator inputs; None when not a torch dtype."""
    mod = type(candidate).__module__
    if not mod.startswith('torch'):
        return None
    name = str(candidate).replace('torch.', '')
    table = {'float16': lang.FLOAT16, 'float32': lang.FLOAT32, 'float64': lang.FLOAT64,
             'int8': lang.INT8, 'int16': lang.INT16, 'int32': lang.INT32, 'int64': lang.INT64,
             'uint8': lang.UINT8, 'uint16': lang.UINT16, 'uint32': lang.UINT32, 'uint64': lang.UINT64}
    return table.get(name)


class DType(object):
    """
    Data type object which indicates a low level storage type (expression.py:20-118).

    Accepts another DType, a numpy scalar type or dtype, a torch dtype, or a schema enum value.
    """

    def __init__(self, dtype):
        if type(dtype) is DType:
            self.proto_dtype = dtype.proto_dtype
            return
        if isinstance(dtype, bool):
            raise TypeError('dtype ' + str(dtype) + ' is not valid.')
        if isinstance(dtype, _INT_TYPES):
            if dtype not in lang.DType.values():
                raise ValueError('dtype ' + str(dtype) + ' is not valid.')
            self.proto_dtype = dtype
            return
        code = _code_from_torch(dtype)
        if code is None:
            code = _code_from_numpy(dtype)
        if code is None:
            raise TypeError('dtype ' + str(dtype) + ' is not valid.')
        self.proto_dtype = code

    def __eq__(self, other):
        return type(other) is DType and self.proto_dtype == other.proto_dtype

    def __ne__(self, other):
        return not self == other

    def __hash__(self):
        return hash(self.proto_dtype)

    def __str__(self):
        return lang.DType.Name(self.proto_dtype)

    __repr__ = __str__

    def as_numpy(self):
        return _ROW_BY_CODE[self.proto_dtype][1]

    def as_ctypes(self):
        ct = _ROW_BY_CODE[self.proto_dtype][2]
        if ct is None:
            raise KeyError(self.proto_dtype)
        return ct

    def as_cstr(self):
        cstr = _ROW_BY_CODE[self.proto_dtype][3]
        if cstr is None:
            raise KeyError(self.proto_dtype)
        return cstr

    _torch_dtypes = {}

    def as_torch(self):
        found = DType._torch_dtypes.get(self.proto_dtype)
        if found is None:
            import torch
            found = getattr(torch, np.dtype(self.as_numpy()).name)
            DType._torch_dtypes[self.proto_dtype] = found
        return found

    def as_proto(self):
        return self.proto_dtype

    def itemsize(self):
        return np.dtype(self.as_numpy()).itemsize

    def is_float(self):
        return self.proto_dtype in (lang.FLOAT16, lang.FLOAT32, lang.FLOAT64)

    def is_signed_int(self):
        return self.proto_dtype in (lang.INT8, lang.INT16, lang.INT32, lang.INT64)

    def is_unsigned_int(self):
        return self.proto_dtype in (lang.UINT8, lang.UINT16, lang.UINT32, lang.UINT64)


#: The half-precision floating point DType
float16 = DType(lang.FLOAT16)
#: The single precision floating point DType
float32 = DType(lang.FLOAT32)
#: The double precision floating point DType
float64 = DType(lang.FLOAT64)
#: The 8 bit signed integer DType
int8 = DType(lang.INT8)
#: The 16 bit signed integer DType
int16 = DType(lang.INT16)
#: The 32 bit signed integer DType
int32 = DType(lang.INT32)
#: The 64 bit signed integer DType
int64 = DType(lang.INT64)
#: The 8 bit unsigned integer DType
uint8 = DType(lang.UINT8)
#: The 16 bit unsigned integer DType
uint16 = DType(lang.UINT16)
#: The 32 bit unsigned integer DType
uint32 = DType(lang.UINT32)
#: The 64 bit unsigned integer DType
uint64 = DType(lang.UINT64)

supported_types = [float16, float32, float64, int8, int16, int32, int64, uint8, uint16, uint32, uint64]


class TensorType(object):
    """A tensor is defined by its data type and its (static, fully known) shape (expression.py:146-238)."""

    def __init__(self, shape, dtype):
        self.dtype = DType(dtype)

        if isinstance(shape, _INT_TYPES):
            dims = [shape]
        elif isinstance(shape, str):
            raise TypeError('Shape must be an iterable of ints.')
        else:
            dims = []
            for elem in shape:
                if elem is None:
                    raise TypeError('All dimensions must be defined.')
                if isinstance(elem, bool) or not isinstance(elem, _INT_TYPES):
                    raise TypeError('Shape must be an iterable of ints.')
                dims.append(elem)

        for elem in dims:
            if elem <= 0:
                raise ValueError('All tensor dimensions must be positive, but got: ' + str(dims))

        self.shape = dims
        self.rank = len(dims)
        self.size = 1
        for elem in dims:
            self.size *= elem

        self._proto_tensor_type = lang.TensorType()
        self._proto_tensor_type.dtype = self.dtype.proto_dtype
        self._proto_tensor_type.shape.extend(dims)

    def __eq__(self, other):
        return isinstance(other, TensorType) and self._proto_tensor_type == other._proto_tensor_type

    def __ne__(self, other):
        return not self == other

    __hash__ = None

    def __str__(self):
        return str(self._proto_tensor_type)

    @staticmethod
    def like(other):
        """
        Resolve the TensorType of the argument: anything with ``shape`` and ``dtype`` (numpy arrays, torch tensors,
        operator outputs, tensor expressions, other TensorTypes) or the TensorFlow-style ``get_shape()``.
        """
        try:
            other_shape = other.shape
        except AttributeError:
            other_shape = other.get_shape().as_list()

        try:
            other_dtype = other.dtype.as_numpy_dtype().dtype
        except AttributeError:
            other_dtype = other.dtype

        return TensorType([int(d) for d in other_shape], other_dtype)

    @staticmethod
    def from_proto(proto):
        return TensorType(list(proto.shape), proto.dtype)

    def as_proto(self):
        tt = lang.TensorType()
        tt.CopyFrom(self._proto_tensor_type)
        return tt


# ----------------------------------------------------------------------------------------------------------------------
# the recorder
# ----------------------------------------------------------------------------------------------------------------------
class ExpressionDAG(object):
    """
    Recorder of expressions in definition order (expression.py:250-352, 708-715).  There is one recorder per process;
    expressions register themselves on construction.
    """
    exprs = []
    expr_ids = []
    workgroup_shape = None
    num_outputs = 0
    num_inputs = 0
    _index_of = {}

    @staticmethod
    def clear():
        ExpressionDAG.exprs = []
        ExpressionDAG.expr_ids = []
        ExpressionDAG.workgroup_shape = None
        ExpressionDAG.num_outputs = 0
        ExpressionDAG.num_inputs = 0
        ExpressionDAG._index_of = {}

    @staticmethod
    def append(item):
        if not isinstance(item, _Expression):
            raise TypeError('Can only append expressions.')

        kind = type(item)
        if kind is PositionTensor:
            if ExpressionDAG.workgroup_shape is not None:
                raise ValueError('Already defined the position tensor.')
            ExpressionDAG.workgroup_shape = list(item.proto_expr.uint32_data)
        elif kind is OutputTensor:
            if item.proto_expr.io_index != ExpressionDAG.num_outputs:
                raise ValueError('Trying to add outputs to expression dag out of order')
            ExpressionDAG.num_outputs += 1
        elif kind is InputTensor:
            if item.proto_expr.io_index != ExpressionDAG.num_inputs:
                raise ValueError('Trying to add inputs to expression dag out of order')
            ExpressionDAG.num_inputs += 1

        ExpressionDAG._index_of[id(item)] = len(ExpressionDAG.exprs)
        ExpressionDAG.exprs.append(item)
        ExpressionDAG.expr_ids.append(id(item))

    @staticmethod
    def _reindex():
        ExpressionDAG.expr_ids = [id(e) for e in ExpressionDAG.exprs]
        ExpressionDAG._index_of = dict((i, n) for n, i in enumerate(ExpressionDAG.expr_ids))

    @staticmethod
    def expr_index(expr):
        """Resolve the index of a particular expression in the current DAG (ValueError when it is not recorded)."""
        try:
            return ExpressionDAG._index_of[id(expr)]
        except KeyError:
            raise ValueError('Expression is not part of the current expression DAG.')

    @staticmethod
    def replace(index, expr):
        """Put ``expr`` at position ``index`` of the recorded list (used to order outputs by return position)."""
        ExpressionDAG.exprs[index] = expr
        ExpressionDAG._reindex()

    @staticmethod
    def remove_endif():
        """Drop the most recent ENDIF so an elif/else continues the open conditional (expression.py:338-352)."""
        for back in range(len(ExpressionDAG.exprs) - 1, -1, -1):
            if type(ExpressionDAG.exprs[back]) is _EndIf:
                del ExpressionDAG.exprs[back]
                ExpressionDAG._reindex()
                return
        raise SyntaxError('Could not find prior if block')

    @staticmethod
    def io_types():
        input_types = ExpressionDAG.num_inputs * [None]
        output_types = ExpressionDAG.num_outputs * [None]
        for expr in ExpressionDAG.exprs:
            if expr.proto_expr.code == lang.INPUT:
                input_types[expr.proto_expr.io_index] = TensorType.from_proto(expr.proto_expr.tensor_type)
            elif expr.proto_expr.code == lang.OUTPUT:
                output_types[expr.proto_expr.io_index] = TensorType.from_proto(expr.proto_expr.tensor_type)
        return input_types, output_types

    @staticmethod
    def as_proto():
        """
        Serialise the recorded DAG.  Sub-expressions of ``elif`` conditions are recorded inside the preceding branch
        (Python evaluates ``elif_(cond)`` before the ``with`` body is entered); they are moved in front of the
        opening IF so that every branch condition is computed before the conditional starts
        (expression.py:374-439).
        """
        if ExpressionDAG.workgroup_shape is None:
            raise ValueError('Workgroup shape must be defined with "position_in" function.')

        exprs = [e.proto_expr for e in ExpressionDAG.exprs]
        operands = [[ExpressionDAG.expr_index(op) for op in e.input_exprs] for e in ExpressionDAG.exprs]
        exprs, operands = _hoist_elif_conditions(exprs, operands)

        proto = lang.ExpressionDAG()
        proto.workgroup_shape.extend(ExpressionDAG.workgroup_shape)
        for expr, ops in zip(exprs, operands):
            proto.expressions.add().CopyFrom(expr)
            proto.references.add().operand_indices.extend(ops)
        return proto

    @staticmethod
    def from_proto(expression_dag):
        """Clear the recorder and rebuild expression objects from a serialised DAG (expression.py:443-519)."""
        ExpressionDAG.clear()
        for i, expr in enumerate(expression_dag.expressions):
            inputs = [ExpressionDAG.exprs[ref] for ref in expression_dag.references[i].operand_indices]
            _class_of_code(expr.code).from_proto(expr, inputs)


def _hoist_elif_conditions(exprs, operands):
    """Return (exprs, operands) reordered so elif-condition dependencies precede their IF."""
    open_ifs = []       # start index of each open conditional
    pending = []        # per open conditional: set of indices to move in front of it
    n = 0
    while n < len(exprs):
        code = exprs[n].code
        if code == lang.IF:
            open_ifs.append(n)
            pending.append(set())
        elif code == lang.ELSEIF:
            start = open_ifs[-1]
            stack = [operands[n][0]] if operands[n][0] > start else []
            while stack:
                cur = stack.pop()
                if cur in pending[-1]:
                    continue
                pending[-1].add(cur)
                stack.extend(ref for ref in operands[cur] if ref > start)
        elif code == lang.ENDIF:
            start = open_ifs.pop()
            moved = sorted(pending.pop())
            if moved:
                last = moved[-1]
                moved_set = set(moved)
                order = list(range(start)) + moved + \
                    [i for i in range(start, last + 1) if i not in moved_set] + \
                    list(range(last + 1, len(exprs)))
                new_index = dict((old, new) for new, old in enumerate(order))
                exprs = [exprs[old] for old in order]
                operands = [[new_index[ref] for ref in operands[old]] for old in order]
                # positions after ``last`` are unchanged, so ``n`` still points at this ENDIF;
                # enclosing conditionals started before ``start`` and keep their index as well
        n += 1
    return exprs, operands


# ----------------------------------------------------------------------------------------------------------------------
# expression base classes
# ----------------------------------------------------------------------------------------------------------------------
class _Expression(object):
    """Base of everything recorded in the DAG (expression.py:718-754)."""

    def __init__(self, expression_code):
        if expression_code not in lang.ExpressionCode.values():
            raise ValueError('Expression code ' + str(expression_code) + ' is not valid.')
        self.proto_expr = lang.Expression()
        self.proto_expr.code = expression_code
        self.input_exprs = []
        self.name = None

    def _register(self):
        ExpressionDAG.append(self)

    def __str__(self):
        return str(self.proto_expr)

    def __ilshift__(self, other):
        raise SyntaxError('Can only use assignment operator <<= on a variable.')

    @staticmethod
    def from_proto(proto, input_exprs):
        raise NotImplementedError('Abstract Class')

    def __bool__(self):
        raise SyntaxError('Attempting to interpret the truth of an expression. This typically happens when trying to '
                          'use a python native "if", "min", or "max" statement to create a data-dependent conditional '
                          'inside of an operator, which is not supported. To do so you must use the corresponding '
                          '"with if_(...)", "minimum", and "maximum" functions.')

    __nonzero__ = __bool__


def _binary(code, swap=False):
    if swap:
        return lambda self, other: _BinaryMath(other, self, code)
    return lambda self, other: _BinaryMath(self, other, code)


class Scalar(_Expression):
    """An expression that refers to a single data value which has a data type (expression.py:757-832)."""

    def __init__(self, expr_code, dtype):
        if not isinstance(dtype, DType):
            raise TypeError('Scalar expressions must be initialized with a DType')
        super(Scalar, self).__init__(expr_code)
        self.dtype = dtype
        self.proto_expr.dtype = dtype.as_proto()

    __add__ = _binary(lang.ADD)
    __radd__ = _binary(lang.ADD, swap=True)
    __sub__ = _binary(lang.SUBTRACT)
    __rsub__ = _binary(lang.SUBTRACT, swap=True)
    __mul__ = _binary(lang.MULTIPLY)
    __rmul__ = _binary(lang.MULTIPLY, swap=True)
    __truediv__ = _binary(lang.DIVIDE)
    __rtruediv__ = _binary(lang.DIVIDE, swap=True)
    __div__ = __truediv__
    __rdiv__ = __rtruediv__
    __mod__ = _binary(lang.MODULO)
    __rmod__ = _binary(lang.MODULO, swap=True)
    __eq__ = _binary(lang.EQUAL)
    __ne__ = _binary(lang.NOTEQUAL)
    __lt__ = _binary(lang.LESS)
    __le__ = _binary(lang.LESS_EQ)
    __gt__ = _binary(lang.GREATER)
    __ge__ = _binary(lang.GREATER_EQ)
    __hash__ = None

    def __neg__(self):
        return _UnaryMath(self, lang.NEGATE)


class _TensorExpression(_Expression):
    """An expression that refers to a tensor of data which has a TensorType (expression.py:835-856)."""

    def __init__(self, expr_code, tensor_type):
        super(_TensorExpression, self).__init__(expr_code)
        self.dtype = tensor_type.dtype
        self.shape = tensor_type.shape
        self.size = tensor_type.size
        self.rank = tensor_type.rank
        self.tensor_type = tensor_type
        self.proto_expr.tensor_type.CopyFrom(tensor_type.as_proto())


# ----------------------------------------------------------------------------------------------------------------------
# indexing
# ----------------------------------------------------------------------------------------------------------------------
def _row_major_strides(shape):
    strides = [1] * len(shape)
    for dim in range(len(shape) - 2, -1, -1):
        strides[dim] = strides[dim + 1] * shape[dim + 1]
    return strides


def _static_component(value, extent):
    """A compile-time index component: floor it and bounds-check it (expression.py:908-916, 941-948)."""
    cur_value = int(np.floor(value))
    if cur_value >= extent or cur_value < 0:
        raise IndexError('Expected index to be in range [0, ' + str(extent) +
                         '), but received index value ' + str(cur_value))
    return cur_value


def _is_number(x):
    return isinstance(x, (int, float, np.integer, np.floating))


def _to_scalar_index(target_shape, index):
    """
    Resolve an N-dimensional index into the index of the C-ordered flat buffer (expression.py:859-973).

    ``index`` may be a number, a list/tuple/array of numbers (static, bounds-checked, folds to a Python int), a
    scalar expression, a mixed list/tuple of scalar expressions, size-1 tensors and numbers, or a rank-1 tensor
    expression (position, local or input tensor) whose length equals the target rank.  Every non-constant component
    is cast to uint64, multiplied by its row-major stride and summed left to right.
    """
    target_rank = len(target_shape)
    strides = _row_major_strides(target_shape)

    if isinstance(index, Scalar):
        index = [index]
    elif _is_number(index):
        index = np.array([index])

    if isinstance(index, (list, tuple)) and all(_is_number(v) for v in index):
        index = np.array(index)

    if isinstance(index, np.ndarray):
        if index.ndim != 1:
            raise IndexError('Index must be one dimensional')
        if index.shape[0] != target_rank:
            raise IndexError('length of index tensor (' + str(index.shape[0]) +
                             ') must match indexed tensor rank (' + str(target_rank) + ')')
        flat = 0
        for dim, elem in enumerate(index.tolist()):
            flat += _static_component(elem, target_shape[dim]) * strides[dim]
        return flat

    if isinstance(index, (list, tuple)):
        if len(index) != target_rank:
            raise IndexError('length of index list (' + str(len(index)) +
                             ') must match indexed tensor rank (' + str(target_rank) + ')')
        components = []
        for dim, value in enumerate(index):
            if isinstance(value, _Expression):
                if not isinstance(value, Scalar):
                    if isinstance(value, _TensorExpression) and value.size == 1:
                        # a 1-D workgroup's position tensor used as one component
                        value = value[0]
                    else:
                        raise TypeError('Must index tensors with an int or a scalar expression. Instead got:\n' +
                                        str(value))
                components.append(value)
            else:
                components.append(_static_component(value, target_shape[dim]))

        flat = None
        for dim, comp in enumerate(components):
            term = comp if isinstance(comp, _INT_TYPES) else cast(comp, uint64)
            term = term * strides[dim]
            flat = term if flat is None else flat + term
        return flat

    if type(index) in (LocalTensor, PositionTensor, InputTensor):
        if len(index.shape) != 1:
            raise IndexError('Index must be one dimensional')
        if index.shape[0] != target_rank:
            raise IndexError('length of index tensor (' + str(index.shape[0]) +
                             ') must match indexed tensor rank (' + str(target_rank) + ')')
        flat = None
        for dim in range(target_rank):
            term = cast(_ReadTensor(index, dim), uint64) * strides[dim]
            flat = term if flat is None else flat + term
        return flat

    raise TypeError('Cannot index a tensor with a ' + str(type(index)))


class _Readable(object):
    """A trait for tensors which enables them to be read"""

    def __getitem__(self, item):
        return _ReadTensor(self, _to_scalar_index(self.shape, item))


class _Writable(object):
    """A trait for tensors which enables them to be written"""

    def __setitem__(self, key, value):
        _AssignTensor(self, _to_scalar_index(self.shape, key), value)


def _tensor_type_polymorphic(*args):
    err_msg = 'Expected a TensorType or a shape and a dtype as arguments'
    if len(args) == 1:
        if type(args[0]) is not TensorType:
            raise TypeError(err_msg)
        return args[0]
    if len(args) == 2:
        return TensorType(args[0], args[1])
    raise TypeError(err_msg)


def _check_io(tensor_type, io_index):
    if not isinstance(tensor_type, TensorType):
        raise TypeError('tensor_type must be a TensorType')
    if isinstance(io_index, bool) or not isinstance(io_index, _INT_TYPES):
        raise TypeError('io_index must be an int')
    if io_index < 0 or io_index > 2 ** 32 - 1:
        raise ValueError('io_index out of range')


# ----------------------------------------------------------------------------------------------------------------------
# tensors
# ----------------------------------------------------------------------------------------------------------------------
def input(*args):
    """Create a new operator input; args are a TensorType, or a shape and a DType (expression.py:1011-1018)."""
    return InputTensor(_tensor_type_polymorphic(*args), ExpressionDAG.num_inputs)


class InputTensor(_TensorExpression, _Readable):
    """A read-only input tensor expression (expression.py:1021-1053)."""

    def __init__(self, tensor_type, io_index):
        _check_io(tensor_type, io_index)
        super(InputTensor, self).__init__(lang.INPUT, tensor_type)
        self.proto_expr.io_index = io_index
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return InputTensor(TensorType.from_proto(proto.tensor_type), proto.io_index)


def output(*args):
    """
    Define a new output; args are a TensorType, or a shape and a DType (expression.py:1056-1079)::

        out = output(in0.tensor_type)
        out = output(in0.shape, in1.dtype)
    """
    return OutputTensor(_tensor_type_polymorphic(*args), ExpressionDAG.num_outputs)


def output_like(other):
    """Define a new output with the same TensorType as another tensor (expression.py:1082-1090)."""
    return output(TensorType.like(other))


class OutputTensor(_TensorExpression, _Writable):
    """A write-only output expression (expression.py:1093-1125)."""

    def __init__(self, tensor_type, io_index):
        _check_io(tensor_type, io_index)
        super(OutputTensor, self).__init__(lang.OUTPUT, tensor_type)
        self.proto_expr.io_index = io_index
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return OutputTensor(TensorType.from_proto(proto.tensor_type), proto.io_index)


class _ConstScalar(Scalar):
    """A Python int (int64) or float (float64) literal (expression.py:1128-1166)."""

    def __init__(self, value):
        if type(value) is float:
            super(_ConstScalar, self).__init__(lang.CONST_SCALAR, float64)
            self.proto_expr.double_data.append(value)
        elif isinstance(value, _INT_TYPES):
            super(_ConstScalar, self).__init__(lang.CONST_SCALAR, int64)
            self.proto_expr.sint64_data.append(int(value))
        else:
            raise TypeError('Tried to wrap a ' + str(type(value)) + ' as a ConstScalar. Can only wrap an int or float')
        self._register()

    def value(self):
        if self.proto_expr.dtype == lang.FLOAT64:
            return float(self.proto_expr.double_data[0])
        if self.proto_expr.dtype == lang.INT64:
            return int(self.proto_expr.sint64_data[0])
        raise ValueError('Can only get a value from float64 or int64 constants.')

    @staticmethod
    def from_proto(proto, input_exprs):
        if proto.dtype == lang.FLOAT64:
            return _ConstScalar(float(proto.double_data[0]))
        if proto.dtype == lang.FLOAT32:
            return _ConstScalar(float(proto.float_data[0]))
        if proto.dtype == lang.INT64:
            return _ConstScalar(int(proto.sint64_data[0]))
        raise ValueError('Cannot recover constant scalar protobuf.')


def _const_data_field(proto_expr, dtype):
    """The repeated field that stores constant data of ``dtype`` (expression.py:1175-1187)."""
    code = dtype.proto_dtype
    if code in (lang.FLOAT16, lang.FLOAT32):
        return proto_expr.float_data
    if code == lang.FLOAT64:
        return proto_expr.double_data
    if code in (lang.INT8, lang.INT16, lang.INT32):
        return proto_expr.sint32_data
    if code == lang.INT64:
        return proto_expr.sint64_data
    if code in (lang.UINT8, lang.UINT16, lang.UINT32):
        return proto_expr.uint32_data
    if code == lang.UINT64:
        return proto_expr.uint64_data
    raise TypeError('No constant storage for ' + str(dtype))


class _ConstTensor(_TensorExpression, _Readable):
    """A constant tensor expression built from a list, tuple, number or numpy array (expression.py:1169-1242)."""

    def __init__(self, value):
        if type(value) in (list, tuple):
            array = np.array(value)
        elif type(value) is np.ndarray:
            array = value
        elif isinstance(value, _INT_TYPES) or type(value) is float:
            array = np.array([value])
        else:
            raise TypeError('ConstTensors can wrap lists, tuples, and numpy arrays')

        super(_ConstTensor, self).__init__(lang.CONST_TENSOR, TensorType.like(array))
        _const_data_field(self.proto_expr, self.dtype).extend(array.flatten(order='C').tolist())
        self._register()

    def to_array(self):
        return np.array(_const_data_field(self.proto_expr, self.dtype), dtype=self.dtype.as_numpy())

    @staticmethod
    def from_proto(proto, input_exprs):
        dtype = DType(proto.tensor_type.dtype)
        data = np.array(_const_data_field(proto, dtype), dtype=dtype.as_numpy())
        return _ConstTensor(data.reshape(list(proto.tensor_type.shape)))


def position_in(workgroup_shape):
    """
    Define the workgroup shape and retrieve a tensor expression that refers to the current position in that
    workgroup shape (expression.py:1245-1253).

    :param workgroup_shape: An int or an iterable of ints defining the shape of the workgroup
    :return: a tensor expression which references the current workgroup position
    """
    return PositionTensor(workgroup_shape)


class PositionTensor(_TensorExpression, _Readable):
    """The current position within the workgroup shape, a uint32 tensor of rank 1 (expression.py:1256-1306)."""

    def __init__(self, workgroup_shape):
        if isinstance(workgroup_shape, _INT_TYPES):
            dims = [workgroup_shape]
        else:
            try:
                dims = list(workgroup_shape)
                for elem in dims:
                    if isinstance(elem, bool) or not isinstance(elem, _INT_TYPES):
                        raise TypeError
            except TypeError:
                raise TypeError('workgroup_shape must be an int or an iterable of ints')
        self.workgroup_shape = dims

        super(PositionTensor, self).__init__(lang.POSITION, TensorType([len(dims)], uint32))
        self.proto_expr.uint32_data.extend(dims)
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return PositionTensor(list(proto.uint32_data))


class LocalTensor(_TensorExpression, _Readable, _Writable):
    """A worker-local tensor initialised from a constant tensor (expression.py:1769-1795)."""

    def __init__(self, initial_value):
        if type(initial_value) is not _ConstTensor:
            raise TypeError('Tensors must be initialized by ConstTensors')
        super(LocalTensor, self).__init__(lang.TENSOR, initial_value.tensor_type)
        self.input_exprs = [initial_value]
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return LocalTensor(input_exprs[0])


def zeros(shape, dtype):
    """Declare a new worker-local tensor with all elements initialized to zero (expression.py:1798-1808)."""
    return LocalTensor(_ConstTensor(np.zeros(shape, dtype=DType(dtype).as_numpy())))


def ones(shape, dtype):
    """Declare a new worker-local tensor with all elements initialized to one (expression.py:1811-1821)."""
    return LocalTensor(_ConstTensor(np.ones(shape, dtype=DType(dtype).as_numpy())))


# ----------------------------------------------------------------------------------------------------------------------
# scalars
# ----------------------------------------------------------------------------------------------------------------------
def variable(initial_value, dtype):
    """
    Declare a new worker-local scalar variable; assign to it with ``<<=`` (expression.py:1309-1324).

    :param initial_value: a numeric constant or a scalar expression
    :param dtype: The DType of the variable
    """
    if isinstance(initial_value, _INT_TYPES) or isinstance(initial_value, float):
        return Variable(dtype, _ConstScalar(initial_value))
    if isinstance(initial_value, Scalar):
        var = Variable(dtype, _ConstScalar(0))
        var <<= initial_value
        return var
    raise TypeError('Must initialize a variable with a numeric constant or a scalar expression.')


class Variable(Scalar):
    """A mutable scalar (expression.py:1327-1352)."""

    def __init__(self, dtype, intial_const):
        if not isinstance(intial_const, _ConstScalar):
            raise TypeError('Variables must be initialized with a constant scalar')
        if not isinstance(dtype, DType):
            raise TypeError('dtype must be a DType')
        super(Variable, self).__init__(lang.VARIABLE, dtype)
        self.input_exprs = [intial_const]
        self._register()

    def __ilshift__(self, other):
        _AssignVariable(self, other)
        return self

    @staticmethod
    def from_proto(proto, input_exprs):
        return Variable(DType(proto.dtype), input_exprs[0])


def cast(value, dtype):
    """Cast a scalar expression as a new data type (expression.py:1355-1363)."""
    return _Cast(dtype, value)


class _Cast(Scalar):
    def __init__(self, dtype, target):
        if not isinstance(dtype, DType):
            raise TypeError('dtype must be a DType')
        if not isinstance(target, Scalar):
            raise TypeError('Can only cast scalar expressions. Received ' + str(type(target)) + ': ' + str(target))
        super(_Cast, self).__init__(lang.CAST, dtype)
        self.input_exprs = [target]
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _Cast(DType(proto.dtype), input_exprs[0])


def _as_value_of(dtype, value):
    """Numbers become literals cast to ``dtype``; scalar expressions pass through (expression.py:1398-1402)."""
    if isinstance(value, _Expression):
        return value
    return cast(_ConstScalar(value), dtype)


class _AssignVariable(_Expression):
    def __init__(self, scalar_expr, value_expr):
        if not isinstance(scalar_expr, Variable):
            raise TypeError('Can only assign to a variable')
        value = _as_value_of(scalar_expr.dtype, value_expr)
        super(_AssignVariable, self).__init__(lang.ASSIGN_VARIABLE)

        t1 = scalar_expr.proto_expr.dtype
        t2 = value.proto_expr.dtype
        if t1 != t2:
            raise TypeError('cannot assign ' + lang.DType.Name(t2) + ' to ' + lang.DType.Name(t1) + ' scalar')

        self.input_exprs = [scalar_expr, value]
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _AssignVariable(input_exprs[0], input_exprs[1])


def _check_index(target_expr, index_expr):
    """Wrap a flat index as an expression and bounds-check it when it is a literal (expression.py:1824-1844)."""
    index = index_expr if isinstance(index_expr, _Expression) else _ConstScalar(index_expr)
    if index.proto_expr.dtype == lang.UNDEFINED_TYPE:
        raise TypeError('Can only index with a scalar.')
    if type(index) is _ConstScalar:
        if target_expr.size <= index.value() or index.value() < 0:
            raise IndexError('Index out of bounds.')
    return index


class _AssignTensor(_Expression):
    def __init__(self, tensor_expr, index_expr, value_expr):
        super(_AssignTensor, self).__init__(lang.ASSIGN_TENSOR)
        if not isinstance(tensor_expr, _Writable):
            raise TypeError('Can only assign to writable tensors.')

        index = _check_index(tensor_expr, index_expr)
        value = _as_value_of(tensor_expr.dtype, value_expr)

        t1 = tensor_expr.proto_expr.tensor_type.dtype
        t2 = value.proto_expr.dtype
        if t1 != t2:
            raise TypeError('cannot assign ' + lang.DType.Name(t2) + ' to ' + lang.DType.Name(t1) + ' tensor')

        self.input_exprs = [tensor_expr, index, value]
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _AssignTensor(input_exprs[0], input_exprs[1], input_exprs[2])


class _ReadTensor(Scalar):
    def __init__(self, tensor_expr, index_expr):
        if not isinstance(tensor_expr, _Readable):
            raise TypeError('Can only index a readable tensor.')
        index = _check_index(tensor_expr, index_expr)
        super(_ReadTensor, self).__init__(lang.READ_TENSOR, tensor_expr.dtype)
        self.input_exprs = [tensor_expr, index]
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _ReadTensor(input_exprs[0], input_exprs[1])


# ----------------------------------------------------------------------------------------------------------------------
# math
# ----------------------------------------------------------------------------------------------------------------------
_FLOATS = (lang.FLOAT32, lang.FLOAT64)
_SIGNED = (lang.INT8, lang.INT16, lang.INT32, lang.INT64)
_UNSIGNED = (lang.UINT8, lang.UINT16, lang.UINT32, lang.UINT64)
_ALL_TYPES = tuple(t.proto_dtype for t in supported_types)

#: unary code -> dtypes it accepts (expression.py:1430-1456)
UNARY_DOMAIN = dict((code, _FLOATS) for code in (
    lang.ACOS, lang.ASIN, lang.ATAN, lang.COS, lang.COSH, lang.SIN, lang.SINH, lang.TAN, lang.TANH, lang.EXP,
    lang.LOG, lang.LOG10, lang.SQRT, lang.CEIL, lang.FLOOR, lang.ISINF, lang.ISFINITE, lang.ISNAN))
UNARY_DOMAIN[lang.ABS] = _FLOATS + _SIGNED
UNARY_DOMAIN[lang.NEGATE] = _FLOATS + _SIGNED
UNARY_DOMAIN[lang.NOT] = _FLOATS + _SIGNED + _UNSIGNED

#: binary code -> dtypes it accepts (expression.py:1632-1672)
BINARY_DOMAIN = dict((code, _ALL_TYPES) for code in (
    lang.ADD, lang.SUBTRACT, lang.MULTIPLY, lang.DIVIDE, lang.MODULO, lang.EQUAL, lang.NOTEQUAL, lang.LESS,
    lang.LESS_EQ, lang.GREATER, lang.GREATER_EQ, lang.MIN, lang.MAX, lang.AND, lang.OR))
BINARY_DOMAIN[lang.POW] = _FLOATS
BINARY_DOMAIN[lang.ATAN2] = _FLOATS


class _UnaryMath(Scalar):
    """Unary expressions which transform a single scalar expression; the result has the argument's dtype."""

    def __init__(self, arg, expr_code):
        if expr_code not in UNARY_DOMAIN:
            raise ValueError(lang.ExpressionCode.Name(expr_code) + 'is an invalid unary math code.')
        if not isinstance(arg, Scalar):
            raise TypeError('Must apply math functions to scalar expressions. Received: ' + str(arg))
        if arg.dtype.proto_dtype not in UNARY_DOMAIN[expr_code]:
            raise ValueError(lang.DType.Name(arg.dtype.proto_dtype) +
                             ' arguments not supported for unary math function ' +
                             lang.ExpressionCode.Name(expr_code))
        super(_UnaryMath, self).__init__(expr_code, arg.dtype)
        self.input_exprs = [arg]
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _UnaryMath(input_exprs[0], proto.code)


def _unary_function(code, doc):
    def fcn(x):
        return _UnaryMath(x, code)
    fcn.__doc__ = doc
    return fcn


arccos = _unary_function(lang.ACOS, 'Inverse cosine of a floating point scalar expression.')
arcsin = _unary_function(lang.ASIN, 'Inverse sine of a floating point scalar expression.')
arctan = _unary_function(lang.ATAN, 'Inverse tangent of a floating point scalar expression.')
cos = _unary_function(lang.COS, 'Cosine of a floating point scalar expression.')
cosh = _unary_function(lang.COSH, 'Hyperbolic cosine of a floating point scalar expression.')
sin = _unary_function(lang.SIN, 'Sine of a floating point scalar expression.')
sinh = _unary_function(lang.SINH, 'Hyperbolic sine of a floating point scalar expression.')
tan = _unary_function(lang.TAN, 'Tangent of a floating point scalar expression.')
tanh = _unary_function(lang.TANH, 'Hyperbolic tangent of a floating point scalar expression.')
exp = _unary_function(lang.EXP, 'Natural exponential of a floating point scalar expression.')
log = _unary_function(lang.LOG, 'Natural logarithm of a floating point scalar expression.')
log10 = _unary_function(lang.LOG10, 'Base 10 logarithm of a floating point scalar expression.')
sqrt = _unary_function(lang.SQRT, 'Square root of a floating point scalar expression.')
ceil = _unary_function(lang.CEIL, 'Ceiling of a floating point scalar expression.')
floor = _unary_function(lang.FLOOR, 'Floor of a floating point scalar expression.')
absolute = _unary_function(lang.ABS, 'Absolute value of a floating point or signed integer scalar expression.')
logical_not = _unary_function(lang.NOT, 'Logical negation; the 0/1 result has the dtype of the argument.')
isinf = _unary_function(lang.ISINF, 'Infinity predicate; the 0/1 result has the dtype of the argument.')
isfinite = _unary_function(lang.ISFINITE, 'Finiteness predicate; the 0/1 result has the dtype of the argument.')
isnan = _unary_function(lang.ISNAN, 'NaN predicate; the 0/1 result has the dtype of the argument.')


class _Limits(Scalar):
    """Numeric limits of the floating point types (expression.py:1564-1596)."""

    def __init__(self, expr_code, t):
        if expr_code not in (lang.MIN_VALUE, lang.MAX_VALUE, lang.EPSILON):
            raise ValueError(lang.ExpressionCode.Name(expr_code) + 'is an invalid limits code.')
        if not isinstance(t, DType):
            raise TypeError('Must apply limits functions to dtypes. Received: ' + str(t))
        if t.as_proto() not in _FLOATS:
            raise ValueError(str(t) + ' arguments not supported for limits function ' +
                             lang.ExpressionCode.Name(expr_code))
        super(_Limits, self).__init__(expr_code, t)
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _Limits(proto.code, DType(proto.dtype))


def min_value(dtype):
    """The minimum normalized positive value of a floating point type (expression.py:1598-1606)."""
    return _Limits(lang.MIN_VALUE, dtype)


def max_value(dtype):
    """The maximum finite value of a floating point type (expression.py:1608-1615)."""
    return _Limits(lang.MAX_VALUE, dtype)


def epsilon(dtype):
    """The difference between 1.0 and the next representable value (expression.py:1617-1625)."""
    return _Limits(lang.EPSILON, dtype)


def _wrap_operand(arg):
    """Numbers become literals; anything else is passed through for the type checks (expression.py:1679-1688)."""
    try:
        return _ConstScalar(arg)
    except TypeError:
        return arg


class _BinaryMath(Scalar):
    """
    Binary expressions which transform two scalars into another.  Both operands must have the same dtype; a Python
    number next to an expression is cast to the expression's dtype first; two bare numbers are an error
    (expression.py:1674-1733).  Comparisons and logical operators yield 0/1 in the operand dtype.
    """

    def __init__(self, arg1, arg2, expr_code):
        if expr_code not in BINARY_DOMAIN:
            raise ValueError('Invalid binary math code')
        code_str = lang.ExpressionCode.Name(expr_code)

        lhs = _wrap_operand(arg1)
        rhs = _wrap_operand(arg2)

        if not isinstance(lhs, _Expression):
            raise TypeError('Cannot apply ' + code_str + ' to first non-expression argument:\n' + str(lhs))
        if not isinstance(rhs, _Expression):
            raise TypeError('Cannot apply ' + code_str + ' to second non-expression argument:\n' + str(rhs))
        if not isinstance(lhs, Scalar):
            raise TypeError('First argument to ' + code_str + ' must be a scalar expression, got:\n' + str(lhs))
        if not isinstance(rhs, Scalar):
            raise TypeError('Second argument to ' + code_str + ' must be a scalar expression, got:\n' + str(rhs))

        lhs_literal = type(lhs) is _ConstScalar
        rhs_literal = type(rhs) is _ConstScalar
        if lhs_literal and rhs_literal:
            raise TypeError('Cannot apply binary operator to two constants.')
        if rhs_literal:
            rhs = cast(rhs, lhs.dtype)
        elif lhs_literal:
            lhs = cast(lhs, rhs.dtype)

        t1 = lhs.proto_expr.dtype
        t2 = rhs.proto_expr.dtype
        if t1 != t2:
            raise TypeError('arg1 type (' + lang.DType.Name(t1) + ') must be the same as arg2 type (' +
                            lang.DType.Name(t2) + ')')
        if t1 not in BINARY_DOMAIN[expr_code]:
            raise ValueError(lang.DType.Name(t1) + ' arguments not supported for binary math function ' + code_str)

        super(_BinaryMath, self).__init__(expr_code, lhs.dtype)
        self.input_exprs = [lhs, rhs]
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _BinaryMath(input_exprs[0], input_exprs[1], proto.code)


def minimum(x, y):
    """Element minimum, evaluated as ``(x < y) ? x : y``."""
    return _BinaryMath(x, y, lang.MIN)


def maximum(x, y):
    """Element maximum, evaluated as ``(x > y) ? x : y``."""
    return _BinaryMath(x, y, lang.MAX)


def power(x, y):
    """x raised to the power y (floating point only)."""
    return _BinaryMath(x, y, lang.POW)


def arctan2(x, y):
    """Two-argument inverse tangent (floating point only)."""
    return _BinaryMath(x, y, lang.ATAN2)


def logical_and(x, y):
    """Logical and; the 0/1 result has the dtype of the operands."""
    return _BinaryMath(x, y, lang.AND)


def logical_or(x, y):
    """Logical or; the 0/1 result has the dtype of the operands."""
    return _BinaryMath(x, y, lang.OR)


# ----------------------------------------------------------------------------------------------------------------------
# control flow
# ----------------------------------------------------------------------------------------------------------------------
def arange(start, stop=None, step=None):
    """
    Create an iterator to iterate over a range inside the worker (expression.py:1908-1961)::

        accum = variable(0, uint64)
        for i in arange(10):
            accum <<= accum + 1

    The loop variable has the dtype of the first argument that is an expression, int64 for an all-integer range.
    """
    if stop is None:
        bounds = [0, start]
    else:
        bounds = [start, stop]
    bounds.append(1 if step is None else step)

    first_type = None
    wrapped = []
    for val in bounds:
        if isinstance(val, _Expression):
            wrapped.append(val)
            if first_type is None:
                first_type = val.dtype
        else:
            wrapped.append(_ConstScalar(val))
    if first_type is None:
        first_type = _ConstScalar(start).dtype

    limits = [cast(e, first_type) if type(e) is _ConstScalar else e for e in wrapped]
    index = variable(0, first_type)
    return _Range(index, limits[0], limits[1], limits[2])


class _Range(_Expression):
    """Head of a counted loop; iterating it yields the loop variable once, then closes the loop."""

    def __init__(self, index, start, stop, step):
        self.block_done = False
        for expr in (start, stop, step):
            if expr.dtype != index.dtype:
                raise TypeError('All input expressions must have the same type.')
        super(_Range, self).__init__(lang.RANGE)
        self.input_exprs = [index, start, stop, step]
        self._register()

    def __iter__(self):
        return self

    def __next__(self):
        if not self.block_done:
            self.block_done = True
            return self.input_exprs[0]
        _EndRange()
        raise StopIteration

    next = __next__

    @staticmethod
    def from_proto(proto, input_exprs):
        return _Range(*input_exprs)


class _EndRange(_Expression):
    def __init__(self):
        super(_EndRange, self).__init__(lang.ENDRANGE)
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _EndRange()


def if_(condition):
    """
    Conditional execution, must be used as part of a ``with`` block (expression.py:2025-2041)::

        y = variable(0, input_tensor.dtype)
        y <<= input_tensor[some_index]
        with if_(y > 1):
            y <<= 1
        output_tensor[some_index] = y
    """
    return _If(condition)


def elif_(condition):
    """Else-if branch; must directly follow an ``if_`` or ``elif_`` block (expression.py:2074-2096)."""
    return _ElseIf(condition)


def else_():
    """Else branch; must directly follow an ``if_`` or ``elif_`` block (expression.py:2125-2145)."""
    return _Else()


class _If(_Expression):
    def __init__(self, condition):
        if not isinstance(condition, Scalar):
            if isinstance(condition, bool):
                raise TypeError('Attempting to use a constant boolean, %s, with the operator if_ expression. Use the '
                                'python if instead since this can be interpreted at operator '
                                'definition time.' % condition)
            raise TypeError('Condition must be a scalar expression, instead got: ' + str(condition))
        super(_If, self).__init__(lang.IF)
        self.input_exprs = [condition]
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _If(input_exprs[0])

    def __enter__(self):
        pass

    def __exit__(self, exc_type, exc_val, exc_tb):
        _EndIf()


class _ElseIf(_Expression):
    def __init__(self, condition):
        if not isinstance(condition, Scalar):
            raise TypeError('Condition must be a scalar expression')
        super(_ElseIf, self).__init__(lang.ELSEIF)
        self.input_exprs = [condition]
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _ElseIf(input_exprs[0])

    def __enter__(self):
        ExpressionDAG.remove_endif()

    def __exit__(self, exc_type, exc_val, exc_tb):
        _EndIf()


class _Else(_Expression):
    def __init__(self):
        super(_Else, self).__init__(lang.ELSE)
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _Else()

    def __enter__(self):
        ExpressionDAG.remove_endif()

    def __exit__(self, exc_type, exc_val, exc_tb):
        _EndIf()


class _EndIf(_Expression):
    def __init__(self):
        super(_EndIf, self).__init__(lang.ENDIF)
        self._register()

    @staticmethod
    def from_proto(proto, input_exprs):
        return _EndIf()


def _class_of_code(code):
    fixed = {
        lang.INPUT: InputTensor, lang.OUTPUT: OutputTensor, lang.CONST_SCALAR: _ConstScalar,
        lang.CONST_TENSOR: _ConstTensor, lang.POSITION: PositionTensor, lang.VARIABLE: Variable, lang.CAST: _Cast,
        lang.TENSOR: LocalTensor, lang.ASSIGN_VARIABLE: _AssignVariable, lang.ASSIGN_TENSOR: _AssignTensor,
        lang.READ_TENSOR: _ReadTensor, lang.RANGE: _Range, lang.ENDRANGE: _EndRange, lang.IF: _If,
        lang.ELSEIF: _ElseIf, lang.ELSE: _Else, lang.ENDIF: _EndIf,
        lang.MIN_VALUE: _Limits, lang.MAX_VALUE: _Limits, lang.EPSILON: _Limits}
    if code in fixed:
        return fixed[code]
    if code in UNARY_DOMAIN:
        return _UnaryMath
    if code in BINARY_DOMAIN:
        return _BinaryMath
    raise ValueError('No expression class for code ' + str(code))
