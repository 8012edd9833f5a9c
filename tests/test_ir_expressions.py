"""
IR-level unit tests of the expression language: constructing expressions directly, the fields of their serialised
form, ``from_proto`` round trips and the error type raised for every kind of misuse.  Covers the behaviours the
reference pins in opveclib/test/test_expressions.py:28-547; nothing is compiled or run.
"""
import numpy as np
import pytest

from opveclib_amd import language as lang
from opveclib_amd.expression import (
    DType, TensorType, ExpressionDAG, float16, float32, float64, int8, int16, int32, int64, uint8, uint16, uint32,
    uint64, supported_types, variable, cast, zeros, ones, arange, position_in, output, input,
    arccos, arcsin, arctan, cos, cosh, sin, sinh, tan, tanh, exp, log, log10, sqrt, ceil, floor, absolute,
    logical_not, isinf, isfinite, isnan, minimum, maximum, power, arctan2, logical_and, logical_or,
    min_value, max_value, epsilon, if_, elif_, else_)
from opveclib_amd.expression import (
    _Expression, InputTensor, OutputTensor, _ConstScalar, _ConstTensor, Variable, LocalTensor, _AssignVariable,
    _AssignTensor, _ReadTensor, _UnaryMath, _Cast, _Limits, _BinaryMath, _to_scalar_index, PositionTensor, _Range,
    _If, _ElseIf, _Else, _EndIf)


@pytest.fixture(autouse=True)
def fresh_dag():
    ExpressionDAG.clear()
    yield
    ExpressionDAG.clear()


NUMPY_TWINS = [(float16, np.float16), (float32, np.float32), (float64, np.float64), (int8, np.int8),
               (int16, np.int16), (int32, np.int32), (int64, np.int64), (uint8, np.uint8), (uint16, np.uint16),
               (uint32, np.uint32), (uint64, np.uint64)]


class TestTypes:
    @pytest.mark.parametrize('bad, err', [('string', TypeError), (1.0, TypeError), (np.longdouble, TypeError),
                                          (np.ndarray, TypeError), (100000, ValueError)])
    def test_dtype_rejects(self, bad, err):
        with pytest.raises(err):
            DType(bad)

    @pytest.mark.parametrize('ovl_type, np_type', NUMPY_TWINS)
    def test_dtype_numpy_twins(self, ovl_type, np_type):
        assert ovl_type == DType(np_type)
        assert ovl_type == DType(np.zeros(3, dtype=np_type).dtype)
        assert ovl_type.as_numpy() == np_type
        assert DType(ovl_type) == ovl_type
        assert DType(ovl_type.as_proto()) == ovl_type
        assert hash(DType(np_type)) == hash(ovl_type)

    def test_dtype_torch_twins(self):
        torch = pytest.importorskip('torch')
        assert DType(torch.float32) == float32
        assert DType(torch.int64) == int64
        assert float64.as_torch() == torch.float64
        assert TensorType.like(torch.zeros((2, 3), dtype=torch.int16)) == TensorType([2, 3], int16)

    def test_dtype_c_spelling(self):
        assert float32.as_cstr() == 'float'
        assert int64.as_cstr() == 'int64_tf'
        assert str(uint16) == 'UINT16'

    @pytest.mark.parametrize('shape, err', [('string', TypeError), ((1, 2, 3.3), TypeError),
                                            (np.array([1.0, 2.0, 3.0]), TypeError), ([0, 5], ValueError),
                                            ([3, None], TypeError), ([-1], ValueError)])
    def test_tensor_type_rejects(self, shape, err):
        with pytest.raises(err):
            TensorType(shape, float32)

    def test_tensor_type_semantics(self):
        assert TensorType((1, 2, 3), float32) == TensorType([1, 2, 3], float32)
        assert TensorType((1, 2, 3), float32) == TensorType([1, 2, 3], np.float32)
        assert TensorType(5, float32) == TensorType([5], float32)
        assert TensorType(5, float32) != TensorType([5], float16)
        assert TensorType(5, float32) != 'something else'
        assert TensorType((5, 10, 100), float32).size == 5000
        assert TensorType((5, 10, 100), float32).rank == 3
        assert TensorType.like(np.zeros(10, dtype=np.uint8)) == TensorType(10, uint8)
        assert TensorType.like(np.zeros((10, 10), dtype=np.float64)) == TensorType([10, 10], float64)
        tt = TensorType([4, 6], int32)
        assert TensorType.from_proto(tt.as_proto()) == tt


class TestTensors:
    def test_expression_code_must_exist(self):
        with pytest.raises(ValueError):
            _Expression(-1)

    @pytest.mark.parametrize('cls', [InputTensor, OutputTensor])
    def test_io_tensor(self, cls):
        a_type = TensorType.like(np.empty((5, 5), dtype=np.uint64))
        t = cls(a_type, 0)
        assert t.proto_expr.io_index == 0
        assert t.proto_expr.tensor_type.shape == [5, 5]
        assert t.proto_expr.tensor_type.dtype == uint64.proto_dtype
        for bad, err in ((-1, ValueError), (2 ** 32, ValueError), ('string', TypeError)):
            with pytest.raises(err):
                cls(a_type, bad)
        with pytest.raises(TypeError):
            cls('string', 0)
        with pytest.raises(ValueError):
            cls(a_type, 5)          # out of order declaration
        ExpressionDAG.clear()
        assert cls.from_proto(t.proto_expr, []).proto_expr == t.proto_expr

    def test_output_is_write_only_and_input_read_only(self):
        a_type = TensorType([5, 5], float32)
        out = OutputTensor(a_type, 0)
        out[0, 0] = 0
        with pytest.raises(TypeError):
            out[0, 0]
        inp = InputTensor(a_type, 0)
        inp[0, 0]
        with pytest.raises(TypeError):
            inp[0, 0] = 1.0

    def test_input_output_helpers_number_sequentially(self):
        a = input([3], float32)
        b = input(TensorType([3], float64))
        o = output([3], float32)
        assert (a.proto_expr.io_index, b.proto_expr.io_index, o.proto_expr.io_index) == (0, 1, 0)
        assert ExpressionDAG.num_inputs == 2 and ExpressionDAG.num_outputs == 1
        with pytest.raises(TypeError):
            output([3])
        in_types, out_types = ExpressionDAG.io_types()
        assert in_types == [TensorType([3], float32), TensorType([3], float64)]
        assert out_types == [TensorType([3], float32)]

    def test_const_scalar(self):
        for bad in ('string', np.arange(1)):
            with pytest.raises(TypeError):
                _ConstScalar(bad)
        t = _ConstScalar(1)
        assert t.proto_expr.code == lang.CONST_SCALAR
        assert t.proto_expr.dtype == lang.INT64
        assert list(t.proto_expr.sint64_data) == [1]
        assert _ConstScalar.from_proto(t.proto_expr, []).proto_expr == t.proto_expr

        t = _ConstScalar(1.1)
        assert t.proto_expr.dtype == lang.FLOAT64
        assert list(t.proto_expr.double_data) == [1.1]
        assert t.value() == 1.1
        assert _ConstScalar.from_proto(t.proto_expr, []).proto_expr == t.proto_expr

        t.proto_expr.dtype = lang.UNDEFINED_TYPE
        with pytest.raises(ValueError):
            t.value()
        with pytest.raises(ValueError):
            _ConstScalar.from_proto(t.proto_expr, [])

    def test_const_tensor(self):
        with pytest.raises(TypeError):
            _ConstTensor('string')
        assert _ConstTensor([1, 2, 3]).proto_expr == _ConstTensor((1, 2, 3)).proto_expr
        assert _ConstTensor(np.arange(1, 4, dtype=np.int64)).proto_expr == _ConstTensor((1, 2, 3)).proto_expr
        assert _ConstTensor(np.arange(1, 4, dtype=np.int32)).proto_expr != _ConstTensor((1, 2, 3)).proto_expr
        rng = np.random.default_rng(0)
        for data in (rng.random(10).astype(np.float32),
                     rng.integers(-2 ** 63, 2 ** 63 - 1, size=10, dtype=np.int64),
                     rng.integers(0, 2 ** 64 - 1, size=6, dtype=np.uint64).reshape(2, 3)):
            a = _ConstTensor(data)
            again = _ConstTensor.from_proto(a.proto_expr, [])
            assert again.proto_expr == a.proto_expr
            assert np.array_equal(again.to_array(), data.reshape(-1))

    def test_position(self):
        pos = PositionTensor((5, 5))
        assert pos.dtype == uint32 and pos.shape == [2]
        assert list(pos.proto_expr.uint32_data) == [5, 5]
        with pytest.raises(ValueError):
            PositionTensor((2, 2))      # only one position per operator
        ExpressionDAG.clear()
        assert PositionTensor.from_proto(pos.proto_expr, []).proto_expr == pos.proto_expr
        ExpressionDAG.clear()
        assert position_in(7).workgroup_shape == [7]
        ExpressionDAG.clear()
        for bad in ('ab', [1.5], 2.0):
            with pytest.raises(TypeError):
                position_in(bad)

    def test_local_tensor(self):
        with pytest.raises(TypeError):
            LocalTensor('string')
        for maker, value in ((zeros, 0), (ones, 1)):
            a = maker((5, 5), int8)
            assert a.proto_expr.tensor_type.dtype == int8.proto_dtype
            init = a.input_exprs[0]
            assert list(init.proto_expr.sint32_data) == [value] * 25
        assert LocalTensor.from_proto(a.proto_expr, a.input_exprs).proto_expr == a.proto_expr


class TestScalars:
    def test_variable(self):
        with pytest.raises(TypeError):
            variable('string', float32)
        a = variable(1.0, float32)
        assert a.proto_expr.dtype == float32.proto_dtype
        assert len(a.input_exprs) == 1
        a <<= 5
        assignment = ExpressionDAG.exprs[-1]
        assert type(assignment) is _AssignVariable
        assert ExpressionDAG.expr_index(a) == ExpressionDAG.expr_index(assignment.input_exprs[0])
        b = variable(2.0, float32)
        assert b.proto_expr == Variable.from_proto(b.proto_expr, b.input_exprs).proto_expr
        c = variable(a + 1, float32)       # initialised from an expression: declared as 0, then assigned
        assert type(ExpressionDAG.exprs[-1]) is _AssignVariable
        assert c.input_exprs[0].value() == 0

    def test_only_variables_accept_ilshift(self):
        a = variable(1.0, float32)
        b = a + 1
        with pytest.raises(SyntaxError):
            b <<= 2

    def test_assign_variable(self):
        for bad_value, err in (('string', TypeError), (None, TypeError)):
            with pytest.raises(err):
                _AssignVariable(variable(0, float32), bad_value)
        with pytest.raises(TypeError):
            _AssignVariable(variable(0, float32), variable(0, float64))
        with pytest.raises(TypeError):
            _AssignVariable('string', variable(0, float32))

        a = variable(1.0, float32)
        b = variable(2.0, float32)
        c = _AssignVariable(a, b)
        assert c.input_exprs[0].proto_expr.dtype == float32.proto_dtype and len(c.input_exprs) == 2
        c = _AssignVariable(a, 2)
        assert c.input_exprs[1].proto_expr.dtype == float32.proto_dtype
        assert type(c.input_exprs[1]) is _Cast
        assert c.proto_expr == _AssignVariable.from_proto(c.proto_expr, c.input_exprs).proto_expr

    def test_cast(self):
        for bad in ('string', 1.0):
            with pytest.raises(TypeError):
                cast(bad, float32)
        with pytest.raises(TypeError):
            cast(PositionTensor((5, 5)), float32)
        a = variable(1.0, float32)
        with pytest.raises(TypeError):
            cast(a, np.float32)
        b = cast(a, float64)
        assert b.proto_expr.dtype == float64.proto_dtype and len(b.input_exprs) == 1
        assert b.proto_expr == _Cast.from_proto(b.proto_expr, b.input_exprs).proto_expr

    def test_assign_tensor(self):
        a = zeros(5, dtype=float32)
        with pytest.raises(TypeError):
            _AssignTensor(InputTensor(TensorType.like(a), 0), 0, 1.0)   # inputs are read-only
        with pytest.raises(TypeError):
            _AssignTensor(a, 'string', 1.0)
        with pytest.raises(TypeError):
            _AssignTensor(a, zeros(1, uint8), 1.0)                      # a tensor is not an index
        for bad in (100, -1):
            with pytest.raises(IndexError):
                _AssignTensor(a, bad, 1.0)
        with pytest.raises(TypeError):
            _AssignTensor(a, 0, 'string')
        with pytest.raises(TypeError):
            _AssignTensor(a, 0, variable(1.0, float64))

        b = _AssignTensor(a, 1, 1)
        assert b.input_exprs[0] is a
        assert b.input_exprs[1].proto_expr == _ConstScalar(1).proto_expr
        assert b.input_exprs[2].proto_expr == cast(_ConstScalar(1), a.dtype).proto_expr
        n = variable(5, uint8)
        v = variable(1.1, float32)
        b = _AssignTensor(a, n, v)
        assert b.input_exprs[1] is n and b.input_exprs[2] is v
        assert b.proto_expr == _AssignTensor.from_proto(b.proto_expr, b.input_exprs).proto_expr

    def test_read_tensor(self):
        a = zeros((5, 5), float32)
        for bad in (-1, 25):
            with pytest.raises(IndexError):
                _ReadTensor(a, bad)
        with pytest.raises(TypeError):
            _ReadTensor(OutputTensor(TensorType.like(a), 0), 5)
        c = _ReadTensor(a, 0)
        assert c.input_exprs[0] is a
        assert c.input_exprs[1].proto_expr == _ConstScalar(0).proto_expr
        assert c.dtype == float32
        d = variable(0, uint8)
        e = _ReadTensor(a, d)
        assert e.input_exprs[1] is d
        assert e.proto_expr == _ReadTensor.from_proto(e.proto_expr, e.input_exprs).proto_expr


class TestIndexing:
    shape = (5, 5)

    def test_static_indices_fold_to_integers(self):
        assert _to_scalar_index(self.shape, [0, 0]) == 0
        assert _to_scalar_index(self.shape, (2, 3)) == 13
        assert _to_scalar_index(self.shape, np.array([4, 4])) == 24
        assert _to_scalar_index(self.shape, [1.9, 2]) == 7     # components are floored
        assert _to_scalar_index((6,), 3) == 3
        before = len(ExpressionDAG.exprs)
        _to_scalar_index(self.shape, [1, 1])
        assert len(ExpressionDAG.exprs) == before               # nothing is recorded for a static index

    @pytest.mark.parametrize('bad', [[1], [0, 0, 0], [0, 5], [5, 0], [-1, 0], np.zeros((2, 1))])
    def test_static_index_errors(self, bad):
        with pytest.raises(IndexError):
            _to_scalar_index(self.shape, bad)

    def test_tensor_indices(self):
        for bad in (zeros(1, float32), zeros(3, float32), zeros((2, 1), float32)):
            with pytest.raises(IndexError):
                _to_scalar_index(self.shape, bad)
        idx = _to_scalar_index(self.shape, zeros(2, float32))
        assert idx.dtype == uint64

    def test_mixed_indices(self):
        v = variable(0, uint32)
        with pytest.raises(IndexError):
            _to_scalar_index(self.shape, [v])
        with pytest.raises(IndexError):
            _to_scalar_index(self.shape, [v, 0, 0])
        with pytest.raises(IndexError):
            _to_scalar_index(self.shape, [v, 5])
        with pytest.raises(TypeError):
            _to_scalar_index(self.shape, [v, zeros(2, uint32)])
        with pytest.raises(TypeError):
            _to_scalar_index(self.shape, _EndIf)
        idx = _to_scalar_index(self.shape, [v, 0])
        assert idx.dtype == uint64 and idx.proto_expr.code == lang.ADD
        # each dynamic component is cast to uint64 and multiplied by its row-major stride
        lhs = idx.input_exprs[0]
        assert lhs.proto_expr.code == lang.MULTIPLY
        assert lhs.input_exprs[0].proto_expr.code == lang.CAST and lhs.input_exprs[0].input_exprs[0] is v
        assert lhs.input_exprs[1].input_exprs[0].value() == 5

    def test_size_one_tensor_as_component(self):
        pos = position_in(4)
        idx = _to_scalar_index((4, 3), (pos, 2))
        assert idx.dtype == uint64


class TestMath:
    UNARY = [(arccos, lang.ACOS), (arcsin, lang.ASIN), (arctan, lang.ATAN), (cos, lang.COS), (cosh, lang.COSH),
             (sin, lang.SIN), (sinh, lang.SINH), (tan, lang.TAN), (tanh, lang.TANH), (exp, lang.EXP),
             (log, lang.LOG), (log10, lang.LOG10), (sqrt, lang.SQRT), (ceil, lang.CEIL), (floor, lang.FLOOR),
             (absolute, lang.ABS), (logical_not, lang.NOT), (lambda x: -x, lang.NEGATE), (isinf, lang.ISINF),
             (isfinite, lang.ISFINITE), (isnan, lang.ISNAN)]

    @staticmethod
    def same_unary(x, y):
        assert x.proto_expr == y.proto_expr
        assert x.input_exprs[0] is y.input_exprs[0]
        assert x.dtype == y.dtype

    @pytest.mark.parametrize('dtype', [float32, float64])
    def test_unary_functions(self, dtype):
        a = variable(1.1, dtype)
        for fcn, code in self.UNARY:
            self.same_unary(fcn(a), _UnaryMath(a, code))
            assert fcn(a).dtype == dtype                  # predicates keep the argument dtype too

    @pytest.mark.parametrize('dtype', [int8, int16, int32, int64])
    def test_unary_on_signed_ints(self, dtype):
        x = variable(1, dtype)
        for fcn, code in ((absolute, lang.ABS), (logical_not, lang.NOT), (lambda v: -v, lang.NEGATE)):
            self.same_unary(fcn(x), _UnaryMath(x, code))
        with pytest.raises(ValueError):
            exp(x)

    def test_unary_errors(self):
        a = variable(1.1, float32)
        with pytest.raises(ValueError):
            _UnaryMath(a, lang.POSITION)
        with pytest.raises(ValueError):
            _UnaryMath(variable(1.1, float16), lang.EXP)
        with pytest.raises(ValueError):
            -variable(1, uint32)
        with pytest.raises(TypeError):
            exp(zeros(3, float32))
        c = absolute(a)
        assert c.proto_expr == _UnaryMath.from_proto(c.proto_expr, c.input_exprs).proto_expr

    def test_limits(self):
        with pytest.raises(ValueError):
            _Limits(lang.POSITION, float32)
        with pytest.raises(ValueError):
            _Limits(lang.MIN_VALUE, float16)
        with pytest.raises(TypeError):
            _Limits(lang.MAX_VALUE, 1.0)
        for t in (float32, float64):
            for fcn, code in ((min_value, lang.MIN_VALUE), (max_value, lang.MAX_VALUE), (epsilon, lang.EPSILON)):
                x, y = fcn(t), _Limits(code, t)
                assert x.proto_expr == y.proto_expr and x.dtype == y.dtype == t
                assert _Limits.from_proto(x.proto_expr, []).proto_expr == x.proto_expr

    def test_binary_construction(self):
        a = variable(1.1, float32)
        b = variable(1.2, float32)
        with pytest.raises(TypeError):
            _BinaryMath(a, variable(0, float64), lang.ADD)
        with pytest.raises(TypeError):
            _BinaryMath(1, 2, lang.ADD)
        with pytest.raises(TypeError):
            _BinaryMath(a, 'string', lang.ADD)
        with pytest.raises(TypeError):
            _BinaryMath(a, zeros(2, float32), lang.ADD)
        with pytest.raises(ValueError):
            _BinaryMath(a, b, lang.POSITION)
        with pytest.raises(ValueError):
            power(variable(1, int32), variable(1, int32))

        c = _BinaryMath(a, b, lang.ADD)
        assert c.input_exprs[0] is a and c.input_exprs[1] is b and c.dtype == float32
        # a Python number is cast to the dtype of the expression next to it
        d = _BinaryMath(a, 1, lang.ADD)
        assert d.dtype == float32 and type(d.input_exprs[1]) is _Cast and d.input_exprs[1].dtype == float32
        d = _BinaryMath(1.5, a, lang.ADD)
        assert d.dtype == float32 and type(d.input_exprs[0]) is _Cast
        assert c.proto_expr == _BinaryMath.from_proto(c.proto_expr, c.input_exprs).proto_expr

    def test_binary_magic_methods(self):
        a = variable(1.1, float32)

        def same(x, y):
            assert x.proto_expr == y.proto_expr
            assert x.input_exprs[0].proto_expr == y.input_exprs[0].proto_expr
            assert x.input_exprs[1].proto_expr == y.input_exprs[1].proto_expr

        same(a + 1, _BinaryMath(a, 1, lang.ADD))
        same(1 + a, _BinaryMath(1, a, lang.ADD))
        same(a - 1, _BinaryMath(a, 1, lang.SUBTRACT))
        same(1 - a, _BinaryMath(1, a, lang.SUBTRACT))
        same(a * 1, _BinaryMath(a, 1, lang.MULTIPLY))
        same(1 * a, _BinaryMath(1, a, lang.MULTIPLY))
        same(a / 1, _BinaryMath(a, 1, lang.DIVIDE))
        same(1 / a, _BinaryMath(1, a, lang.DIVIDE))
        same(a % 1, _BinaryMath(a, 1, lang.MODULO))
        same(1 % a, _BinaryMath(1, a, lang.MODULO))
        same(a == 1, _BinaryMath(a, 1, lang.EQUAL))
        same(1 == a, _BinaryMath(a, 1, lang.EQUAL))
        same(a != 1, _BinaryMath(a, 1, lang.NOTEQUAL))
        same(a < 1, _BinaryMath(a, 1, lang.LESS))
        same(1 < a, _BinaryMath(a, 1, lang.GREATER))
        same(a <= 1, _BinaryMath(a, 1, lang.LESS_EQ))
        same(1 <= a, _BinaryMath(a, 1, lang.GREATER_EQ))
        same(a > 1, _BinaryMath(a, 1, lang.GREATER))
        same(1 > a, _BinaryMath(a, 1, lang.LESS))
        same(a >= 1, _BinaryMath(a, 1, lang.GREATER_EQ))
        same(1 >= a, _BinaryMath(a, 1, lang.LESS_EQ))

    def test_binary_functions(self):
        def same(x, y):
            assert x.proto_expr == y.proto_expr
            assert x.input_exprs[0] is y.input_exprs[0] and x.input_exprs[1] is y.input_exprs[1]
            assert x.dtype == y.dtype

        for t in (float32, float64):
            a1, a2 = variable(1.0, t), variable(1.0, t)
            same(power(a1, a2), _BinaryMath(a1, a2, lang.POW))
            same(arctan2(a1, a2), _BinaryMath(a1, a2, lang.ATAN2))
        for t in supported_types:
            a1, a2 = variable(1.0, t), variable(1.0, t)
            same(minimum(a1, a2), _BinaryMath(a1, a2, lang.MIN))
            same(maximum(a1, a2), _BinaryMath(a1, a2, lang.MAX))
            same(logical_or(a1, a2), _BinaryMath(a1, a2, lang.OR))
            same(logical_and(a1, a2), _BinaryMath(a1, a2, lang.AND))
            assert (a1 < a2).dtype == t                 # comparisons yield 0/1 in the operand dtype


class TestControlFlow:
    def test_arange(self):
        def loop(x):
            for i in arange(x, variable(10, uint16), 1):
                assert i.dtype == x.dtype
        loop(variable(0, uint16))
        codes = [e.proto_expr.code for e in ExpressionDAG.exprs]
        assert codes.count(lang.RANGE) == 1 and codes.count(lang.ENDRANGE) == 1
        with pytest.raises(TypeError):
            loop(variable(0, float32))
        a = arange(10)
        assert a.input_exprs[0].dtype == int64          # all-integer ranges count in int64
        assert a.proto_expr == _Range.from_proto(a.proto_expr, a.input_exprs).proto_expr

    def test_if_elif_else_structure(self):
        with pytest.raises(TypeError):
            _If(zeros((5, 5), float32))
        with pytest.raises(TypeError):
            _If(True)
        with pytest.raises(TypeError):
            _ElseIf(zeros((5, 5), float32))
        a = variable(1.0, float32)
        b = variable(0.0, float32)
        with if_(a < 5):
            b <<= 2
        with elif_(a < 4):
            b <<= 1
        with else_():
            b <<= 0
        codes = [e.proto_expr.code for e in ExpressionDAG.exprs]
        order = [c for c in codes if c in (lang.IF, lang.ELSEIF, lang.ELSE, lang.ENDIF)]
        assert order == [lang.IF, lang.ELSEIF, lang.ELSE, lang.ENDIF]

    def test_elif_without_if(self):
        a = variable(1.0, float32)
        with pytest.raises(SyntaxError):
            with elif_(a < 4):
                pass

    def test_elif_conditions_are_hoisted_before_the_if(self):
        position_in(4)
        a = variable(1.0, float32)
        b = variable(0.0, float32)
        with if_(a < 5):
            b <<= 2
        with elif_((a + 1) * 2 < 4):
            b <<= 1
        with else_():
            b <<= 0
        proto = ExpressionDAG.as_proto()
        codes = [e.code for e in proto.expressions]
        first_if = codes.index(lang.IF)
        elif_at = codes.index(lang.ELSEIF)
        cond = proto.references[elif_at].operand_indices[0]
        assert cond < first_if
        # every operand precedes its user and the condition's whole dependency cone sits before the IF
        for n, ref in enumerate(proto.references):
            for o in ref.operand_indices:
                assert o < n
        pending = [cond]
        while pending:
            cur = pending.pop()
            assert cur < first_if
            pending.extend(proto.references[cur].operand_indices)
        # nothing but the assignment is left inside the first branch
        assert codes[first_if + 1:elif_at].count(lang.ASSIGN_VARIABLE) == 1

    def test_truth_value_of_an_expression_is_an_error(self):
        a = variable(0.0, float32)
        with pytest.raises(SyntaxError):
            if a == 0:
                pass
        with pytest.raises(SyntaxError):
            bool(a)
        with pytest.raises(SyntaxError):
            max(a, 1)
        with pytest.raises(SyntaxError):
            min(a, 1)

    def test_workgroup_shape_is_required(self):
        variable(0.0, float32)
        with pytest.raises(ValueError):
            ExpressionDAG.as_proto()

    def test_dag_round_trip_through_proto(self):
        x = input([4, 6], float32)
        out = output([4, 6], float32)
        pos = position_in([4, 6])
        acc = variable(0, float32)
        for i in arange(3):
            with if_(x[pos] > 0):
                acc <<= acc + x[pos] * cast(i, float32)
            with else_():
                acc <<= minimum(acc, x[pos[0], 0])
        out[pos] = acc
        proto = ExpressionDAG.as_proto()
        ExpressionDAG.from_proto(proto)
        again = ExpressionDAG.as_proto()
        assert again == proto
