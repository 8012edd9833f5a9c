"""
ctypes binding of the C-ABI launcher ``libovl_launch.so`` (declared in include/ovl_launch.h).

The Python side of the boundary that the reference crosses with
``libtest.testCUDAOperator(lib_path, f_name, inputs, n, outputs, n, threads_per_block, times, iters)``
(opveclib/operator.py:2244-2251, 2316-2324).  The library must have been built (``python -m opveclib_amd.build``);
there is no fallback when it is missing.
"""

import ctypes
import os
import subprocess

from . import local

library_path = os.path.join(local.csrc_directory, 'libovl_launch.so')
source_path = os.path.join(local.csrc_directory, 'ovl_launch.cpp')
include_directory = os.path.normpath(os.path.join(local.csrc_directory, '..', '..', 'include'))

EXPORTED_SYMBOLS = ('ovl_lib_open', 'ovl_lib_sym', 'ovl_lib_close', 'ovl_launch', 'ovl_launch_fn', 'ovl_time',
                    'ovl_poison', 'ovl_dtype_size', 'ovl_strerror', 'ovl_last_error', 'ovl_abi_version')

OVL_OK, OVL_EARGS, OVL_EOPEN, OVL_ESYMBOL, OVL_EHIP, OVL_EALIGN, OVL_EINVAL = range(7)


class OvlTensor(ctypes.Structure):
    """``ovl_tensor``: device pointer, dtype code, element count."""
    _fields_ = [('data', ctypes.c_void_p), ('dtype', ctypes.c_int32), ('len', ctypes.c_uint64)]


ENTRY_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.POINTER(OvlTensor), ctypes.c_uint32,
                            ctypes.POINTER(OvlTensor), ctypes.c_uint32, ctypes.c_void_p)


class LauncherError(RuntimeError):
    def __init__(self, code, detail):
        RuntimeError.__init__(self, 'ovl launcher error %d: %s' % (code, detail))
        self.code = code


def build(force=False):
    """Compile the launcher with hipcc next to its source; returns the library path."""
    if not force and os.path.exists(library_path) and \
            os.path.getmtime(library_path) >= os.path.getmtime(source_path):
        return library_path
    tmp = library_path + '.tmp.%d' % os.getpid()
    cmd = [local.hipcc, '-O2', '-fPIC', '-shared', '-std=c++17', '-I' + include_directory,
           source_path, '-o', tmp, '-ldl']
    try:
        subprocess.check_output(cmd, stderr=subprocess.STDOUT, universal_newlines=True)
    except subprocess.CalledProcessError as exception:
        raise RuntimeError('hipcc failed for the launcher:\n' + exception.output)
    os.replace(tmp, library_path)
    return library_path


_lib = None


def library():
    """The loaded launcher (loads it on first use)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(library_path):
        raise RuntimeError('The OVL launcher library ' + library_path + ' has not been built. '
                           'Run "python -m opveclib_amd.build" first.')
    lib = ctypes.CDLL(library_path)
    tensors = ctypes.POINTER(OvlTensor)
    lib.ovl_lib_open.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]
    lib.ovl_lib_sym.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(ENTRY_FN)]
    lib.ovl_lib_close.argtypes = [ctypes.c_void_p]
    lib.ovl_launch.argtypes = [ctypes.c_void_p, ctypes.c_char_p, tensors, ctypes.c_uint32, tensors,
                               ctypes.c_uint32, ctypes.c_void_p]
    lib.ovl_launch_fn.argtypes = [ENTRY_FN, tensors, ctypes.c_uint32, tensors, ctypes.c_uint32, ctypes.c_void_p]
    lib.ovl_time.argtypes = [ENTRY_FN, tensors, ctypes.c_uint32, tensors, ctypes.c_uint32, ctypes.c_void_p,
                             ctypes.c_uint32, ctypes.POINTER(ctypes.c_double)]
    lib.ovl_poison.argtypes = [tensors, ctypes.c_uint32, ctypes.c_void_p]
    lib.ovl_dtype_size.argtypes = [ctypes.c_int32]
    lib.ovl_dtype_size.restype = ctypes.c_uint32
    lib.ovl_strerror.argtypes = [ctypes.c_int]
    lib.ovl_strerror.restype = ctypes.c_char_p
    lib.ovl_last_error.restype = ctypes.c_char_p
    lib.ovl_abi_version.restype = ctypes.c_uint32
    for name in ('ovl_lib_open', 'ovl_lib_sym', 'ovl_lib_close', 'ovl_launch', 'ovl_launch_fn', 'ovl_time',
                 'ovl_poison'):
        getattr(lib, name).restype = ctypes.c_int
    _lib = lib
    return lib


def check(code):
    if code != OVL_OK:
        lib = library()
        detail = lib.ovl_last_error().decode('utf-8', 'replace') or lib.ovl_strerror(code).decode('utf-8')
        raise LauncherError(code, detail)


class OperatorLibrary(object):
    """An open operator library and one resolved entry point."""

    def __init__(self, so_path, entry, info_symbol=None):
        lib = library()
        self.so_path = so_path
        self.entry = entry
        self.handle = ctypes.c_void_p()
        check(lib.ovl_lib_open(so_path.encode('utf-8'), ctypes.byref(self.handle)))
        self.fn = ENTRY_FN()
        check(lib.ovl_lib_sym(self.handle, entry.encode('utf-8'), ctypes.byref(self.fn)))
        self.info = None
        if info_symbol is not None:
            import json
            dl = ctypes.CDLL(so_path)
            getter = getattr(dl, info_symbol)
            getter.restype = ctypes.c_char_p
            self.info = json.loads(getter().decode('utf-8'))

    def launch(self, in_params, n_in, out_params, n_out, stream):
        check(library().ovl_launch_fn(self.fn, in_params, n_in, out_params, n_out, stream))

    def time(self, in_params, n_in, out_params, n_out, stream, iters):
        times = (ctypes.c_double * iters)()
        check(library().ovl_time(self.fn, in_params, n_in, out_params, n_out, stream, iters, times))
        return list(times)


def tensor_array(tensors):
    """ctypes array of OvlTensor from (data_ptr, dtype code, element count) triples (at least one slot)."""
    arr = (OvlTensor * max(1, len(tensors)))()
    for i, (ptr, dtype, length) in enumerate(tensors):
        arr[i] = OvlTensor(ptr, dtype, length)
    return arr
