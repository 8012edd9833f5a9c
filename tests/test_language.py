"""The hand-written IR schema module: message semantics and the proto3 wire codec."""
import numpy as np
import pytest

from opveclib_amd import language as lang


def sample_dag():
    dag = lang.ExpressionDAG()
    dag.name = 'sample'
    dag.workgroup_shape.extend([3, 5])
    e = dag.expressions.add()
    e.code = lang.INPUT
    e.tensor_type.dtype = lang.FLOAT32
    e.tensor_type.shape.extend([3, 5])
    dag.references.add()
    e = dag.expressions.add()
    e.code = lang.CONST_SCALAR
    e.dtype = lang.INT64
    e.sint64_data.append(-7)
    dag.references.add()
    e = dag.expressions.add()
    e.code = lang.CONST_TENSOR
    e.tensor_type.dtype = lang.FLOAT64
    e.tensor_type.shape.append(3)
    e.double_data.extend([1.5, -2.25, 1e-300])
    e.float_data.extend([0.5])
    e.uint64_data.append(2 ** 64 - 1)
    e.sint32_data.extend([-2 ** 31, 2 ** 31 - 1])
    e.uint32_data.append(2 ** 32 - 1)
    dag.references.add().operand_indices.extend([0, 1])
    return dag


def test_enum_helpers():
    assert lang.DType.Name(lang.FLOAT32) == 'FLOAT32'
    assert lang.ExpressionCode.Name(lang.READ_TENSOR) == 'READ_TENSOR'
    assert lang.ExpressionCode.Value('ISNAN') == 306
    assert 12 in lang.DType.values() and 13 not in lang.DType.values()
    with pytest.raises(ValueError):
        lang.DType.Name(99)


def test_equality_and_copy():
    a = sample_dag()
    b = lang.ExpressionDAG()
    b.CopyFrom(a)
    assert a == b
    b.expressions[1].sint64_data[0] = 8
    assert a != b
    with pytest.raises(AttributeError):
        a.workgroup_shape = [1]
    with pytest.raises(AttributeError):
        a.no_such_field = 1


def test_wire_round_trip():
    a = sample_dag()
    data = a.SerializeToString()
    assert data == sample_dag().SerializeToString()
    b = lang.ExpressionDAG.FromString(data)
    assert a == b

    op_dag = lang.OperatorDAG()
    op_dag.operators.add().CopyFrom(a)
    refs = op_dag.references.add()
    r = refs.input_refs.add()
    r.is_leaf = True
    r.dag_input_index = 3
    r = refs.input_refs.add()
    r.op_index = 2
    r.op_output_index = 1
    out = op_dag.dag_outputs.add()
    out.op_index = 0
    out.op_output_index = 4
    op_dag.dag_input_types.add().CopyFrom(a.expressions[0].tensor_type)
    again = lang.OperatorDAG.FromString(op_dag.SerializeToString())
    assert again == op_dag
    assert again.references[0].input_refs[0].is_leaf is True


def test_wire_format_matches_protobuf_runtime():
    """The byte encoding equals what the protobuf runtime produces for the same schema (language.proto)."""
    pb = pytest.importorskip('google.protobuf')
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

    f = descriptor_pb2.FileDescriptorProto()
    f.name = 'ovl_test_language.proto'
    f.package = 'ovl_test'
    f.syntax = 'proto3'
    T = descriptor_pb2.FieldDescriptorProto

    def add_field(msg, name, number, ftype, repeated=False, type_name=None):
        fld = msg.field.add()
        fld.name = name
        fld.number = number
        fld.type = ftype
        fld.label = T.LABEL_REPEATED if repeated else T.LABEL_OPTIONAL
        if type_name:
            fld.type_name = type_name

    tt = f.message_type.add()
    tt.name = 'TensorType'
    add_field(tt, 'dtype', 1, T.TYPE_UINT32)
    add_field(tt, 'shape', 2, T.TYPE_UINT32, True)
    ex = f.message_type.add()
    ex.name = 'Expression'
    add_field(ex, 'code', 1, T.TYPE_UINT32)
    add_field(ex, 'tensor_type', 2, T.TYPE_MESSAGE, False, '.ovl_test.TensorType')
    add_field(ex, 'dtype', 3, T.TYPE_UINT32)
    add_field(ex, 'io_index', 4, T.TYPE_UINT32)
    add_field(ex, 'float_data', 5, T.TYPE_FLOAT, True)
    add_field(ex, 'double_data', 6, T.TYPE_DOUBLE, True)
    add_field(ex, 'sint32_data', 7, T.TYPE_SINT32, True)
    add_field(ex, 'sint64_data', 8, T.TYPE_SINT64, True)
    add_field(ex, 'uint32_data', 9, T.TYPE_UINT32, True)
    add_field(ex, 'uint64_data', 10, T.TYPE_UINT64, True)
    ol = f.message_type.add()
    ol.name = 'OperandList'
    add_field(ol, 'operand_indices', 1, T.TYPE_UINT32, True)
    dg = f.message_type.add()
    dg.name = 'ExpressionDAG'
    add_field(dg, 'expressions', 1, T.TYPE_MESSAGE, True, '.ovl_test.Expression')
    add_field(dg, 'references', 2, T.TYPE_MESSAGE, True, '.ovl_test.OperandList')
    add_field(dg, 'workgroup_shape', 3, T.TYPE_UINT32, True)
    add_field(dg, 'name', 4, T.TYPE_STRING)

    pool = descriptor_pool.DescriptorPool()
    pool.Add(f)
    cls = message_factory.GetMessageClass(pool.FindMessageTypeByName('ovl_test.ExpressionDAG'))

    ours = sample_dag()
    theirs = cls()
    theirs.ParseFromString(ours.SerializeToString())
    assert theirs.name == 'sample'
    assert list(theirs.workgroup_shape) == [3, 5]
    assert list(theirs.expressions[2].double_data) == [1.5, -2.25, 1e-300]
    assert list(theirs.expressions[2].sint32_data) == [-2 ** 31, 2 ** 31 - 1]
    assert list(theirs.expressions[2].uint64_data) == [2 ** 64 - 1]
    assert list(theirs.expressions[1].sint64_data) == [-7]
    assert theirs.SerializeToString(deterministic=True) == ours.SerializeToString()


def test_real_dag_round_trip():
    import opveclib_amd as ovl
    from opveclib_amd.lstm import lstm_grad
    x = np.zeros((2, 8), np.float32)
    c = np.zeros((2, 2), np.float32)
    op = lstm_grad(x, c, c, c, forget_bias=1.0)
    dag = op[0].parent.expression_dag
    data = dag.SerializeToString()
    assert lang.ExpressionDAG.FromString(data) == dag


def test_sparse_storage_keeps_message_semantics():
    # fields exist only once touched, yet unset and default-valued fields are indistinguishable from outside
    a, b = lang.Expression(), lang.Expression()
    assert a == b
    assert a.io_index == 0 and list(a.float_data) == [] and a.tensor_type == lang.TensorType()
    assert a == b                                  # reading a field does not change equality
    b.io_index = 0
    assert a == b and a.SerializeToString() == b.SerializeToString() == b''
    b.io_index = 3
    assert a != b

    # CopyFrom empties what the source leaves unset, keeping containers handed out earlier alive
    target = lang.Expression()
    kept_list = target.sint64_data
    kept_list.extend([1, 2])
    kept_type = target.tensor_type
    kept_type.shape.extend([4])
    target.dtype = lang.INT64
    source = lang.Expression()
    source.code = lang.CONST_SCALAR
    source.double_data.append(2.5)
    target.CopyFrom(source)
    assert target == source
    assert target.sint64_data is kept_list and kept_list == []
    assert target.tensor_type is kept_type and list(kept_type.shape) == []
    assert target.dtype == 0

    with pytest.raises(AttributeError):
        target.no_such_field
    with pytest.raises(AttributeError):
        target.no_such_field = 1
    with pytest.raises(AttributeError):
        target.tensor_type = lang.TensorType()

    import copy
    import pickle
    dag = sample_dag()
    assert copy.deepcopy(dag) == dag
    assert pickle.loads(pickle.dumps(dag)) == dag


def test_copy_from_a_message_that_another_thread_is_reading():
    # Traced DAGs are shared between threads.  Reading an unset field materialises its default in the message's
    # storage, so a reader in one thread changes the dictionary that CopyFrom in another thread walks.
    import threading
    names = [f.name for f in lang.Expression._fields]
    messages = []
    for k in range(4000):
        m = lang.Expression()
        m.code = lang.CONST_SCALAR
        m.double_data.append(float(k))
        messages.append(m)
    errors = []
    position = [0]

    def reader():
        while position[0] < len(messages):
            m = messages[min(position[0], len(messages) - 1)]
            for name in names:
                getattr(m, name)

    def copier():
        try:
            for k, m in enumerate(messages):
                position[0] = k
                target = lang.Expression()
                target.CopyFrom(m)
                assert target == m
        except Exception as exception:      # noqa: B902 - reported by the main thread
            errors.append(exception)
        finally:
            position[0] = len(messages)

    import sys
    threads = [threading.Thread(target=reader) for _ in range(3)] + [threading.Thread(target=copier)]
    interval = sys.getswitchinterval()
    sys.setswitchinterval(1e-6)             # hand the interpreter from thread to thread as often as possible
    try:
        for t in threads:
            t.start()
        for t in threads:
            t.join()
    finally:
        sys.setswitchinterval(interval)
    assert errors == []
