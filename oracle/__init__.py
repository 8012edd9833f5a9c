"""
TEST ORACLE - not part of the product.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; nothing under ``opveclib_amd/`` does.

CPU restatement of the reference's generated-C++ evaluation path (opveclib/operator.py:2099-2335 with
``target_language='cpp'``): every operator of the operator DAG is emitted as reference-shaped C++
(:mod:`oracle.cpp_emitter`), compiled with g++ using the reference's code-generation flags
(``-fPIC -std=c++11 -pedantic -Wall -Wextra -shared`` and no ``-O`` flag, operator.py:2051-2055; ``-g`` is left out
because debug information does not change the generated instructions) and run by the std::thread driver
(:mod:`oracle.cpu_driver`, restating opveclib/testcop.cc).  Intermediate operator outputs stay in host numpy
buffers and feed later operators, as in operator.py:2279-2303.

What pins this oracle is listed in the header of :mod:`oracle.cpp_emitter`.
"""

import ctypes
import hashlib
import os
import threading
import subprocess

import numpy as np

from opveclib_amd import language as lang
from opveclib_amd.expression import TensorType
from opveclib_amd.operator import _build_op_dag, _op_hash, _normalise_output_list

from . import cpp_emitter

_here = os.path.dirname(os.path.abspath(__file__))
build_directory = os.path.join(_here, '_build')
driver_source = os.path.join(_here, 'cpu_driver.cpp')
driver_library = os.path.join(_here, 'libovl_cpu_driver.so')

cxx = os.getenv('OPVECLIB_CXX', 'g++')

#: code generation flags of the reference (operator.py:2051-2055) minus -g
REFERENCE_FLAGS = ('-fPIC', '-std=c++11', '-pedantic', '-Wall', '-Wextra', '-shared')


class OvlTensor(ctypes.Structure):
    _fields_ = [('data', ctypes.c_void_p), ('dtype', ctypes.c_int32), ('len', ctypes.c_uint64)]


def _run(cmd):
    try:
        subprocess.check_output(cmd, stderr=subprocess.STDOUT, universal_newlines=True)
    except subprocess.CalledProcessError as exception:
        raise RuntimeError('c++ compiler error:\n' + ' '.join(cmd) + '\n' + exception.output)


def build_driver(force=False):
    """Compile the std::thread driver next to its source; returns the library path."""
    if force or not os.path.exists(driver_library) or \
            os.path.getmtime(driver_library) < os.path.getmtime(driver_source):
        tmp = driver_library + '.tmp.%d' % os.getpid()
        _run([cxx, '-O2', '-fPIC', '-shared', '-std=c++11', '-pthread', driver_source, '-o', tmp, '-ldl'])
        os.replace(tmp, driver_library)
    return driver_library


_driver = None


def driver():
    global _driver
    if _driver is None:
        lib = ctypes.CDLL(build_driver())
        lib.ovl_cpu_run.restype = ctypes.c_int32
        lib.ovl_cpu_run.argtypes = [ctypes.c_char_p, ctypes.c_char_p,
                                    ctypes.POINTER(OvlTensor), ctypes.c_uint32,
                                    ctypes.POINTER(OvlTensor), ctypes.c_uint32,
                                    ctypes.c_uint32, ctypes.POINTER(ctypes.c_double), ctypes.c_uint32]
        lib.ovl_cpu_hardware_threads.restype = ctypes.c_uint
        _driver = lib
    return _driver


def hardware_threads():
    return int(driver().ovl_cpu_hardware_threads())


_compile_locks_guard = threading.Lock()
_compile_locks = {}


def compile_op(dag, extra_flags=()):
    """Emit and compile one operator; returns (library path, entry name).  Cached by source text and flags."""
    name = _op_hash(dag)
    src = cpp_emitter.emit_cpp(dag, name)
    flags = list(REFERENCE_FLAGS) + list(extra_flags)
    key = hashlib.sha224((src + ' '.join(flags)).encode('utf-8')).hexdigest()[:24]
    os.makedirs(build_directory, exist_ok=True)
    so_path = os.path.join(build_directory, 'o' + key + '_generic_cpp.so')
    with _compile_locks_guard:
        lock = _compile_locks.setdefault(key, threading.Lock())
    with lock:      # threads that ask for the same operator at the same time: one compiles, the others wait
        if not os.path.exists(so_path):
            cpp_path = os.path.join(build_directory, 'o' + key + '_generic_cpp.cpp')
            with open(cpp_path, 'w') as f:
                f.write(src)
            tmp = so_path + '.tmp.%d.%d' % (os.getpid(), threading.get_ident())
            _run([cxx] + flags + ['-o', tmp, cpp_path])
            os.replace(tmp, so_path)
    return so_path, name + '_generic_cpp'


def _as_host_array(x):
    if isinstance(x, np.ndarray):
        return x
    if hasattr(x, 'detach') and hasattr(x, 'cpu'):
        return x.detach().cpu().numpy()
    return np.asarray(x)


def profile(output_list, profiling_iterations=1, opt_level=0, num_threads=0, extra_flags=()):
    """
    Run the operator DAG behind ``output_list`` on the host.

    :param opt_level: >= 3 fuses operators with the product's optimizer before emitting; 0 evaluates the operators
        exactly as they were defined, one generated function per operator (the reference-shaped path).
    :param num_threads: host threads, 0 = hardware concurrency
    :return: (list of numpy outputs in request order, {operator name: ms per iteration})
    """
    op_dag = _build_op_dag(*_normalise_output_list(output_list))
    dag = op_dag.proto_dag
    if opt_level >= 3:
        from opveclib_amd.fusion import _merge_op_dag
        dag, _ = _merge_op_dag(dag, None)
    leaves = [np.ascontiguousarray(_as_host_array(x)) for x in op_dag.inputs]

    lib = driver()
    buffers = []
    times = {}
    for op_index, op in enumerate(dag.operators):
        so_path, entry = compile_op(op, extra_flags)
        in_exprs = sorted((e for e in op.expressions if e.code == lang.INPUT), key=lambda e: e.io_index)
        out_exprs = sorted((e for e in op.expressions if e.code == lang.OUTPUT), key=lambda e: e.io_index)

        in_params = (OvlTensor * max(1, len(in_exprs)))()
        keep = []
        for i, ref in enumerate(dag.references[op_index].input_refs):
            buf = leaves[ref.dag_input_index] if ref.is_leaf else buffers[ref.op_index][ref.op_output_index]
            tt = TensorType.from_proto(in_exprs[i].tensor_type)
            if buf.dtype != np.dtype(tt.dtype.as_numpy()) or buf.size != tt.size:
                raise TypeError('input %d of %s: expected %s, got %s %s' % (i, op.name, tt, buf.dtype, buf.shape))
            keep.append(buf)
            in_params[i] = OvlTensor(buf.ctypes.data, tt.dtype.proto_dtype, tt.size)

        out_params = (OvlTensor * max(1, len(out_exprs)))()
        cur = []
        for i, e in enumerate(out_exprs):
            tt = TensorType.from_proto(e.tensor_type)
            buf = np.empty(tt.shape, dtype=tt.dtype.as_numpy())
            cur.append(buf)
            out_params[i] = OvlTensor(buf.ctypes.data, tt.dtype.proto_dtype, tt.size)
        buffers.append(cur)

        ms = np.full(profiling_iterations, np.nan, dtype=np.float64)
        err = lib.ovl_cpu_run(so_path.encode('ascii'), entry.encode('ascii'),
                              in_params, len(in_exprs), out_params, len(out_exprs),
                              num_threads, ms.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), profiling_iterations)
        if err != 0:
            raise RuntimeError('oracle operator %s failed with error code %d' % (op.name, err))
        times[entry] = ms

    outputs = [buffers[ref.op_index][ref.op_output_index] for ref in dag.dag_outputs]
    return outputs, times


def evaluate(output_list, opt_level=0, num_threads=0):
    """Host evaluation of ``output_list``: one numpy array for a single output, else a list in request order."""
    outputs = profile(output_list, 1, opt_level, num_threads)[0]
    return outputs[0] if len(outputs) == 1 else outputs
