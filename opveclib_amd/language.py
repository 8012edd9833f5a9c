"""
The IR schema of the expression/operator DAGs.

This module plays the part that the protoc-generated ``language_pb2`` module plays in the reference
(schema: opveclib/language.proto:16-429).  It is written by hand so that it depends on neither ``protoc`` nor a
particular protobuf runtime: messages are small Python objects with the same field names as the schema, value
equality, ``CopyFrom``, and a ``SerializeToString``/``ParseFromString`` pair that uses the proto3 wire encoding of
that schema (varint / zig-zag / fixed32 / fixed64 / length-delimited, repeated scalars packed, default values
omitted, fields in tag order).  The byte string is deterministic, so it doubles as the content key of the operator
compile cache.

Enum values are module-level ints (``lang.FLOAT32``, ``lang.READ_TENSOR`` ...) plus two helper objects ``DType`` and
``ExpressionCode`` offering ``Name()``, ``Value()``, ``values()``, ``keys()`` and ``items()``.
"""

import struct


class _Enum(object):
    """A named group of integer constants (language.proto:16-37 and 46-371)."""

    def __init__(self, name, pairs):
        self._name = name
        self._by_name = dict(pairs)
        self._by_value = dict((v, k) for k, v in pairs)
        self._order = [k for k, _ in pairs]

    def Name(self, value):
        try:
            return self._by_value[value]
        except KeyError:
            raise ValueError('Enum %s has no name defined for value %r' % (self._name, value))

    def Value(self, name):
        try:
            return self._by_name[name]
        except KeyError:
            raise ValueError('Enum %s has no value defined for name %r' % (self._name, name))

    def values(self):
        return [self._by_name[k] for k in self._order]

    def keys(self):
        return list(self._order)

    def items(self):
        return [(k, self._by_name[k]) for k in self._order]


DType = _Enum('DType', [
    ('UNDEFINED_TYPE', 0), ('FLOAT16', 1), ('FLOAT32', 2), ('FLOAT64', 3),
    ('INT8', 4), ('INT16', 5), ('INT32', 6), ('INT64', 7),
    ('UINT8', 8), ('UINT16', 9), ('UINT32', 10), ('UINT64', 11), ('LITERAL', 12)])

ExpressionCode = _Enum('ExpressionCode', [
    ('UNDEFINED_CODE', 0),
    # tensors, scalars, storage
    ('INPUT', 1), ('OUTPUT', 2), ('CONST_SCALAR', 3), ('CONST_TENSOR', 4), ('POSITION', 5), ('VARIABLE', 6),
    ('CAST', 7), ('TENSOR', 8), ('ASSIGN_VARIABLE', 9), ('ASSIGN_TENSOR', 10), ('READ_TENSOR', 11),
    # control flow
    ('RANGE', 12), ('ENDRANGE', 13), ('IF', 14), ('ELSEIF', 15), ('ELSE', 16), ('ENDIF', 17),
    # unary math
    ('ACOS', 100), ('ASIN', 101), ('ATAN', 102), ('COS', 104), ('COSH', 105), ('SIN', 106), ('SINH', 107),
    ('TAN', 108), ('TANH', 109), ('EXP', 150), ('LOG', 151), ('LOG10', 152), ('SQRT', 154),
    ('CEIL', 201), ('FLOOR', 202), ('ABS', 203), ('NEGATE', 204), ('NOT', 205),
    # binary math
    ('ADD', 250), ('SUBTRACT', 251), ('MULTIPLY', 252), ('DIVIDE', 253), ('MODULO', 254), ('AND', 255),
    ('OR', 256), ('EQUAL', 257), ('NOTEQUAL', 258), ('LESS', 259), ('LESS_EQ', 260), ('GREATER', 261),
    ('GREATER_EQ', 262), ('MIN', 300), ('MAX', 301), ('POW', 302), ('ATAN2', 303),
    # predicates and limits
    ('ISINF', 304), ('ISFINITE', 305), ('ISNAN', 306), ('MIN_VALUE', 307), ('MAX_VALUE', 308), ('EPSILON', 309)])

# export every enum member as a module constant, the way generated protobuf modules do
for _k, _v in DType.items() + ExpressionCode.items():
    globals()[_k] = _v
del _k, _v


# ----------------------------------------------------------------------------------------------------------------------
# wire primitives
# ----------------------------------------------------------------------------------------------------------------------
_VARINT, _FIXED64, _BYTES, _FIXED32 = 0, 1, 2, 5


def _put_varint(buf, value):
    value &= 0xFFFFFFFFFFFFFFFF
    while value > 0x7F:
        buf.append((value & 0x7F) | 0x80)
        value >>= 7
    buf.append(value)


def _get_varint(data, pos):
    shift = 0
    result = 0
    while True:
        b = data[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7


def _zigzag(value, bits):
    return ((value << 1) ^ (value >> (bits - 1))) & ((1 << bits) - 1)


def _unzigzag(value):
    return (value >> 1) ^ -(value & 1)


# kind -> (wire type, encoder(buf, v), decoder(data, pos) -> (v, pos), default)
def _enc_fixed(fmt):
    def enc(buf, v):
        buf.extend(struct.pack(fmt, v))
    return enc


def _dec_fixed(fmt, size):
    def dec(data, pos):
        return struct.unpack_from(fmt, data, pos)[0], pos + size
    return dec


def _dec_uvar(mask):
    def dec(data, pos):
        v, pos = _get_varint(data, pos)
        return v & mask, pos
    return dec


def _dec_svar(data, pos):
    v, pos = _get_varint(data, pos)
    return _unzigzag(v), pos


def _dec_bool(data, pos):
    v, pos = _get_varint(data, pos)
    return bool(v), pos


_SCALAR_KINDS = {
    'enum':   (_VARINT, _put_varint, _dec_uvar(0xFFFFFFFF), 0),
    'uint32': (_VARINT, _put_varint, _dec_uvar(0xFFFFFFFF), 0),
    'uint64': (_VARINT, _put_varint, _dec_uvar(0xFFFFFFFFFFFFFFFF), 0),
    'sint32': (_VARINT, lambda b, v: _put_varint(b, _zigzag(v, 32)), _dec_svar, 0),
    'sint64': (_VARINT, lambda b, v: _put_varint(b, _zigzag(v, 64)), _dec_svar, 0),
    'bool':   (_VARINT, lambda b, v: _put_varint(b, 1 if v else 0), _dec_bool, False),
    'float':  (_FIXED32, _enc_fixed('<f'), _dec_fixed('<f', 4), 0.0),
    'double': (_FIXED64, _enc_fixed('<d'), _dec_fixed('<d', 8), 0.0),
}


class _Field(object):
    __slots__ = ('number', 'name', 'kind', 'repeated', 'message')

    def __init__(self, number, name, kind, repeated=False, message=None):
        self.number = number
        self.name = name
        self.kind = kind
        self.repeated = repeated
        self.message = message


class _Repeated(list):
    """Repeated field container: a list with protobuf's ``add()`` for message elements."""

    def __init__(self, message_cls=None):
        super(_Repeated, self).__init__()
        self._message_cls = message_cls

    def add(self):
        item = self._message_cls()
        self.append(item)
        return item


class Message(object):
    """
    Base class of the schema messages: field table driven storage, equality and wire codec.

    Storage is sparse: a field lives in the instance dictionary only once it has been read or written, so creating,
    copying and encoding a message cost in proportion to the fields in use (an Expression has ten fields and
    typically uses two or three).
    """
    _fields = ()
    _by_name = {}
    _by_number = {}

    def __init_subclass__(cls, **kwargs):
        super(Message, cls).__init_subclass__(**kwargs)
        cls._by_name = dict((f.name, f) for f in cls._fields)
        cls._by_number = dict((f.number, f) for f in cls._fields)

    @staticmethod
    def _default(f):
        if f.repeated:
            return _Repeated(f.message)
        if f.kind == 'message':
            return f.message()
        if f.kind == 'string':
            return ''
        return _SCALAR_KINDS[f.kind][3]

    def __getattr__(self, key):
        # reached only for names that are not in the instance dictionary yet: materialise the field's default
        f = type(self)._by_name.get(key)
        if f is None:
            raise AttributeError('%s has no field "%s"' % (type(self).__name__, key))
        # (setdefault: when two threads materialise the same field, both get the one container that is kept)
        return self.__dict__.setdefault(key, self._default(f))

    def __setattr__(self, key, value):
        f = self._by_name.get(key)
        if f is None:
            raise AttributeError('%s has no field "%s"' % (type(self).__name__, key))
        if f.repeated or f.kind == 'message':
            raise AttributeError('Assignment not allowed to composite field "%s"; use CopyFrom/extend.' % key)
        self.__dict__[key] = value

    def __eq__(self, other):
        if type(other) is not type(self):
            return False
        mine, theirs = self.__dict__, other.__dict__
        for f in self._fields:
            if f.name in mine or f.name in theirs:
                if getattr(self, f.name) != getattr(other, f.name):
                    return False
        return True

    def __ne__(self, other):
        return not self == other

    __hash__ = None

    def CopyFrom(self, other):
        if type(other) is not type(self):
            raise TypeError('CopyFrom expects a %s' % type(self).__name__)
        if other is self:
            return
        mine, theirs = self.__dict__, other.__dict__
        # containers and sub-messages handed out earlier keep their identity: they are emptied, not replaced
        for name in list(mine):
            if name not in theirs:
                f = self._by_name[name]
                if f.repeated:
                    del mine[name][:]
                elif f.kind == 'message':
                    mine[name].Clear()
                else:
                    del mine[name]
        # (a snapshot: traced DAGs are shared between threads, and a reader of `other` in another thread may materialise
        # a default there meanwhile)
        for name, src in list(theirs.items()):
            f = self._by_name[name]
            if f.repeated:
                dst = getattr(self, name)
                del dst[:]
                if f.kind == 'message':
                    for item in src:
                        dst.add().CopyFrom(item)
                else:
                    dst.extend(src)
            elif f.kind == 'message':
                getattr(self, name).CopyFrom(src)
            else:
                mine[name] = src

    def Clear(self):
        self.CopyFrom(type(self)())

    def __getstate__(self):
        return self.__dict__

    def __setstate__(self, state):
        self.__dict__.update(state)

    # -- encoding ------------------------------------------------------------------------------------------------
    def _encode(self, buf):
        stored = self.__dict__
        for f in self._fields:
            value = stored.get(f.name)
            if value is None:
                continue
            if f.kind == 'message':
                items = value if f.repeated else [value]
                for item in items:
                    body = bytearray()
                    item._encode(body)
                    if not f.repeated and not body:
                        continue
                    _put_varint(buf, (f.number << 3) | _BYTES)
                    _put_varint(buf, len(body))
                    buf.extend(body)
            elif f.kind == 'string':
                if value:
                    raw = value.encode('utf-8')
                    _put_varint(buf, (f.number << 3) | _BYTES)
                    _put_varint(buf, len(raw))
                    buf.extend(raw)
            else:
                wire, enc, _, default = _SCALAR_KINDS[f.kind]
                if f.repeated:
                    if len(value):
                        body = bytearray()
                        for v in value:
                            enc(body, v)
                        _put_varint(buf, (f.number << 3) | _BYTES)
                        _put_varint(buf, len(body))
                        buf.extend(body)
                elif value != default:
                    _put_varint(buf, (f.number << 3) | wire)
                    enc(buf, value)

    def SerializeToString(self):
        buf = bytearray()
        self._encode(buf)
        return bytes(buf)

    # -- decoding ------------------------------------------------------------------------------------------------
    def _decode(self, data, pos, end):
        by_number = self._by_number
        while pos < end:
            key, pos = _get_varint(data, pos)
            number, wire = key >> 3, key & 7
            f = by_number.get(number)
            if f is None:
                raise ValueError('Unknown field number %d in %s' % (number, type(self).__name__))
            if f.kind == 'message':
                size, pos = _get_varint(data, pos)
                target = getattr(self, f.name).add() if f.repeated else getattr(self, f.name)
                target._decode(data, pos, pos + size)
                pos += size
            elif f.kind == 'string':
                size, pos = _get_varint(data, pos)
                object.__setattr__(self, f.name, bytes(data[pos:pos + size]).decode('utf-8'))
                pos += size
            else:
                _, _, dec, _ = _SCALAR_KINDS[f.kind]
                if f.repeated and wire == _BYTES:
                    size, pos = _get_varint(data, pos)
                    stop = pos + size
                    dst = getattr(self, f.name)
                    while pos < stop:
                        v, pos = dec(data, pos)
                        dst.append(v)
                elif f.repeated:
                    v, pos = dec(data, pos)
                    getattr(self, f.name).append(v)
                else:
                    v, pos = dec(data, pos)
                    object.__setattr__(self, f.name, v)
        return pos

    def ParseFromString(self, data):
        self.Clear()
        self._decode(memoryview(data), 0, len(data))

    @classmethod
    def FromString(cls, data):
        msg = cls()
        msg.ParseFromString(data)
        return msg

    # -- debugging -----------------------------------------------------------------------------------------------
    def _lines(self, indent):
        pad = '  ' * indent
        out = []
        for f in self._fields:
            value = getattr(self, f.name)
            if f.kind == 'message':
                for item in (value if f.repeated else [value]):
                    body = item._lines(indent + 1)
                    if body or f.repeated:
                        out.append('%s%s {' % (pad, f.name))
                        out.extend(body)
                        out.append('%s}' % pad)
            elif f.repeated:
                for v in value:
                    out.append('%s%s: %r' % (pad, f.name, v))
            elif f.kind == 'enum':
                if value:
                    enum = DType if f.name == 'dtype' else ExpressionCode
                    out.append('%s%s: %s' % (pad, f.name, enum.Name(value)))
            elif value != self._default(f):
                out.append('%s%s: %r' % (pad, f.name, value))
        return out

    def __str__(self):
        return '\n'.join(self._lines(0)) + '\n'

    __repr__ = __str__


# ----------------------------------------------------------------------------------------------------------------------
# schema (language.proto:39-42, 374-429)
# ----------------------------------------------------------------------------------------------------------------------
class TensorType(Message):
    _fields = (_Field(1, 'dtype', 'enum'),
               _Field(2, 'shape', 'uint32', repeated=True))


class Expression(Message):
    _fields = (_Field(1, 'code', 'enum'),
               _Field(2, 'tensor_type', 'message', message=TensorType),
               _Field(3, 'dtype', 'enum'),
               _Field(4, 'io_index', 'uint32'),
               _Field(5, 'float_data', 'float', repeated=True),
               _Field(6, 'double_data', 'double', repeated=True),
               _Field(7, 'sint32_data', 'sint32', repeated=True),
               _Field(8, 'sint64_data', 'sint64', repeated=True),
               _Field(9, 'uint32_data', 'uint32', repeated=True),
               _Field(10, 'uint64_data', 'uint64', repeated=True))


class _OperandList(Message):
    _fields = (_Field(1, 'operand_indices', 'uint32', repeated=True),)


class ExpressionDAG(Message):
    OperandList = _OperandList
    _fields = (_Field(1, 'expressions', 'message', repeated=True, message=Expression),
               _Field(2, 'references', 'message', repeated=True, message=_OperandList),
               _Field(3, 'workgroup_shape', 'uint32', repeated=True),
               _Field(4, 'name', 'string'))


class _OperatorInputReference(Message):
    _fields = (_Field(1, 'is_leaf', 'bool'),
               _Field(2, 'op_index', 'uint32'),
               _Field(3, 'op_output_index', 'uint32'),
               _Field(4, 'dag_input_index', 'uint32'))


class _OperatorInputReferences(Message):
    _fields = (_Field(1, 'input_refs', 'message', repeated=True, message=_OperatorInputReference),)


class _DAGOutputReference(Message):
    _fields = (_Field(1, 'op_index', 'uint32'),
               _Field(2, 'op_output_index', 'uint32'))


class OperatorDAG(Message):
    OperatorInputReference = _OperatorInputReference
    OperatorInputReferences = _OperatorInputReferences
    DAGOutputReference = _DAGOutputReference
    _fields = (_Field(1, 'operators', 'message', repeated=True, message=ExpressionDAG),
               _Field(2, 'dag_input_types', 'message', repeated=True, message=TensorType),
               _Field(3, 'references', 'message', repeated=True, message=_OperatorInputReferences),
               _Field(4, 'dag_outputs', 'message', repeated=True, message=_DAGOutputReference))
