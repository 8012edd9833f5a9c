"""
Generated HIP operator sources compiled as plain C++ and run on the host (test infrastructure, never used by the
package): tests/native/host_emulation/ovl_device.h stands in for the device header, one host thread plays one GPU
thread.  The program is built with AddressSanitizer and gets buffers of exactly the tensors' sizes, so an access
outside a tensor ends the run; the outputs come back as numpy arrays for comparison with the oracle.
"""
import hashlib
import os
import subprocess
import tempfile
import threading

import numpy as np

from opveclib_amd import hipgen, language as lang, local
from opveclib_amd.expression import TensorType
from opveclib_amd.operator import _op_hash

HERE = os.path.dirname(os.path.abspath(__file__))
SHIM = os.path.join(HERE, 'native', 'host_emulation')
BUILD = os.path.join(HERE, 'native', '_generated', 'host_emulation')
CLANG = os.path.join(os.path.dirname(os.path.realpath(local.hipcc)), '..', 'llvm', 'bin', 'clang++')
if not os.path.exists(CLANG):
    CLANG = '/opt/rocm/llvm/bin/clang++'

FLAGS = ['-x', 'c++', '-std=c++17', '-O1', '-gline-tables-only', '-fsanitize=address', '-shared-libasan',
         '-fno-omit-frame-pointer', '-ffp-contract=off', '-fno-fast-math', '-pthread', '-Wno-unused-value',
         '-Wno-unknown-attributes']


def _sanitizer_runtime_directory():
    """Where the compiler keeps the shared AddressSanitizer runtime (programs find it through their run path)."""
    path = subprocess.check_output([CLANG, '-print-file-name=libclang_rt.asan-x86_64.so'], universal_newlines=True)
    return os.path.dirname(os.path.realpath(path.strip()))


_build_locks_guard = threading.Lock()
_build_locks = {}


class EmulationError(RuntimeError):
    pass


def _io_types(op):
    ins = sorted((e for e in op.expressions if e.code == lang.INPUT), key=lambda e: e.io_index)
    outs = sorted((e for e in op.expressions if e.code == lang.OUTPUT), key=lambda e: e.io_index)
    return ([TensorType.from_proto(e.tensor_type) for e in ins], [TensorType.from_proto(e.tensor_type) for e in outs])


def build_source(source, entry, extra_flags=()):
    """Compile operator source text (one text, or a list of texts that become one translation unit each) with entry
    point ``entry`` for the host; returns the program's path."""
    sources = [source] if isinstance(source, str) else list(source)
    with open(os.path.join(SHIM, 'ovl_device.h'), 'rb') as f:
        shim = f.read()
    with open(os.path.join(SHIM, 'main.cpp'), 'rb') as f:
        shim += f.read()
    for name in sorted(os.listdir(local.csrc_directory)):      # the product's own headers are compiled in as well
        if name.endswith('.h'):
            with open(os.path.join(local.csrc_directory, name), 'rb') as f:
                shim += f.read()
    digest = hashlib.sha224('\0'.join(sources).encode('utf-8') + entry.encode('utf-8') + shim).hexdigest()[:32]
    os.makedirs(BUILD, exist_ok=True)
    program = os.path.join(BUILD, 'emu_' + digest)
    with _build_locks_guard:
        lock = _build_locks.setdefault(digest, threading.Lock())
    with lock:      # two threads that want the same program: the second finds it built
        _build_program(program, sources, entry, extra_flags)
    return program


def _build_program(program, sources, entry, extra_flags):
    if not os.path.exists(program):
        paths = []
        for k, text in enumerate(sources):
            paths.append(program + ('.cpp' if k == 0 else '.%d.cpp' % k))
            with open(paths[-1], 'w') as f:
                f.write(text)
        tmp = program + '.tmp.%d.%d' % (os.getpid(), threading.get_ident())
        cmd = [CLANG] + FLAGS + list(extra_flags) + ['-I' + SHIM, '-I' + local.csrc_directory, '-DOVL_ENTRY=' + entry,
                                                     '-Wl,-rpath,' + _sanitizer_runtime_directory(),
                                                     os.path.join(SHIM, 'main.cpp')] + paths + ['-o', tmp]
        try:
            subprocess.check_output(cmd, stderr=subprocess.STDOUT, universal_newlines=True)
        except subprocess.CalledProcessError as exception:
            raise EmulationError('host build of the generated source failed:\n' + exception.output)
        os.replace(tmp, program)


class _Adapter(str):
    """Path of the hand-written kernels' program plus the adapter it is to run (see run_program)."""
    function = None


def build_hand_written(entry):
    """The hand-written kernel libraries (csrc/ovl_lstm.hip, csrc/ovl_scan.hip) compiled for the host together with
    the adapters of hand_written_adapters.cpp, as one program for all adapters; ``entry`` names the adapter that
    run_program is to select.  The sources are compiled from copies in the build directory, so that their
    ``#include "ovl_device.h"`` finds the stand-in."""
    parts = []
    for name in ('ovl_lstm.hip', 'ovl_scan.hip'):
        with open(os.path.join(local.csrc_directory, name)) as f:
            parts.append(f.read())
    with open(os.path.join(SHIM, 'hand_written_adapters.cpp')) as f:
        parts.append(f.read())
    include = os.path.normpath(os.path.join(local.csrc_directory, '..', '..', 'include'))
    program = _Adapter(build_source(parts, 'emu_dispatch', ['-I' + include]))
    program.function = entry
    return program


def build(op, options=None):
    """Compile the operator's generated source for the host; returns the program's path."""
    generated = hipgen.generate(op, _op_hash(op), options)
    return build_source(generated.source, generated.entry)


def run_program(program, inputs, in_types, out_types, timeout=300):
    """``in_types`` / ``out_types``: (dtype code of the launcher ABI, numpy dtype, shape) per tensor."""
    with tempfile.TemporaryDirectory() as work:
        args = [program, str(len(in_types)), str(len(out_types))]
        for k, (x, (code, dtype, shape)) in enumerate(zip(inputs, in_types)):
            x = np.ascontiguousarray(x, dtype=dtype)
            assert list(x.shape) == list(shape)
            path = os.path.join(work, 'in%d' % k)
            x.tofile(path)
            args += [str(code), str(x.dtype.itemsize), str(x.size), path]
        for k, (code, dtype, shape) in enumerate(out_types):
            args += [str(code), str(np.dtype(dtype).itemsize), str(int(np.prod(shape, dtype=np.int64))),
                     os.path.join(work, 'out%d' % k)]
        env = dict(os.environ, ASAN_OPTIONS='detect_leaks=0')
        if getattr(program, 'function', None):
            env['OVL_EMU_FUNCTION'] = program.function
        program = str(program)
        args[0] = program
        done = subprocess.run(args, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, universal_newlines=True,
                              timeout=timeout, env=env)
        if done.returncode != 0:
            raise EmulationError('emulated operator ended with status %d:\n%s' % (done.returncode, done.stdout[-4000:]))
        return [np.fromfile(os.path.join(work, 'out%d' % k), dtype=dtype).reshape(shape)
                for k, (code, dtype, shape) in enumerate(out_types)]


def run(op, inputs, options=None, timeout=300):
    """Run one operator (an expression DAG) on the host; ``inputs`` are numpy arrays.  Returns the output arrays."""
    program = build(op, options)
    in_types, out_types = _io_types(op)
    assert len(inputs) == len(in_types)

    def described(t):
        return int(t.dtype.proto_dtype), t.dtype.as_numpy(), list(t.shape)
    return run_program(program, inputs, [described(t) for t in in_types], [described(t) for t in out_types], timeout)


def evaluate(output_list, opt_level=3, options=None):
    """Like ``ovl.evaluate`` for numpy leaves, with every operator of the (fused) DAG run on the host."""
    from opveclib_amd.operator import _build_op_dag, _normalise_output_list
    from opveclib_amd.fusion import _merge_op_dag
    op_dag = _build_op_dag(*_normalise_output_list(output_list))
    dag = op_dag.proto_dag
    if opt_level >= 3:
        dag, _ = _merge_op_dag(dag, None)
    buffers = []
    for op_index, op in enumerate(dag.operators):
        ins = []
        for ref in dag.references[op_index].input_refs:
            ins.append(np.asarray(op_dag.inputs[ref.dag_input_index]) if ref.is_leaf
                       else buffers[ref.op_index][ref.op_output_index])
        buffers.append(run(op, ins, options))
    return [buffers[ref.op_index][ref.op_output_index] for ref in dag.dag_outputs]
