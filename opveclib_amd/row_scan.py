"""
The hand-written row scan kernels (``csrc/ovl_scan.hip``, C ABI in ``include/ovl_scan.h``) from Python.

Running sum and running product along the last axis with the strict left-to-right order of the reference's
``accumulate`` operator (opveclib/examples/test_accumulate.py:22-147) - the same bits as the generated operator and as
``numpy.cumsum`` / ``numpy.cumprod`` - for shapes given at run time: nothing is traced, generated or compiled when they
are called.  Inputs are float32 or float64 torch tensors on a HIP device; launches go to the current PyTorch HIP stream
and do not synchronise.  ``reassociate=True`` selects the tree-shaped wavefront scan instead (not the reference's bits).
"""

import ctypes
import os
import subprocess

from . import local

library_path = os.path.join(local.csrc_directory, 'libovl_scan.so')
source_path = os.path.join(local.csrc_directory, 'ovl_scan.hip')
include_directory = os.path.normpath(os.path.join(local.csrc_directory, '..', '..', 'include'))

SCAN_SYMBOLS = ('ovl_cumsum_f32', 'ovl_cumprod_f32', 'ovl_cumsum_f64', 'ovl_cumprod_f64',
                'ovl_cumsum_f32_reassociated', 'ovl_cumprod_f32_reassociated',
                'ovl_cumsum_f64_reassociated', 'ovl_cumprod_f64_reassociated')
EXPORTED_SYMBOLS = SCAN_SYMBOLS + ('ovl_strip_copy_f64', 'ovl_scan_last_error')


def build(force=False):
    """Compile the library with hipcc next to its source (same flags as generated operators); returns its path."""
    from .compiler import HIPCC_FLAGS
    newest = max(os.path.getmtime(p) for p in (source_path, os.path.join(local.csrc_directory, 'ovl_device.h'),
                                                 os.path.join(local.csrc_directory, 'ovl_wave_scan.h')))
    if not force and os.path.exists(library_path) and os.path.getmtime(library_path) >= newest:
        return library_path
    tmp = library_path + '.tmp.%d' % os.getpid()
    cmd = [local.hipcc] + list(HIPCC_FLAGS) + ['-I' + include_directory, '-I' + local.csrc_directory,
                                               source_path, '-o', tmp]
    try:
        subprocess.check_output(cmd, stderr=subprocess.STDOUT, universal_newlines=True)
    except subprocess.CalledProcessError as exception:
        raise RuntimeError('hipcc failed for the row scan library:\n' + exception.output)
    os.replace(tmp, library_path)
    return library_path


_lib = None


def library():
    """The loaded library (loads it on first use); there is no fallback when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(library_path):
        raise RuntimeError('The row scan library ' + library_path + ' has not been built. '
                           'Run "python -m opveclib_amd.build" first.')
    lib = ctypes.CDLL(library_path)
    for name in SCAN_SYMBOLS:
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p]
        fn.restype = ctypes.c_int
    lib.ovl_strip_copy_f64.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p,
                                       ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p]
    lib.ovl_strip_copy_f64.restype = ctypes.c_int
    lib.ovl_scan_last_error.restype = ctypes.c_char_p
    _lib = lib
    return lib


class RowScanError(RuntimeError):
    def __init__(self, code, detail):
        RuntimeError.__init__(self, 'ovl_scan error %d: %s' % (code, detail))
        self.code = code


def _scan(kind, x, reassociate=False):
    import torch
    if not isinstance(x, torch.Tensor):
        raise TypeError('x must be a torch tensor')
    if x.device.type != 'cuda':
        raise RuntimeError('the row scan kernels run on an AMD GPU: x must live on a HIP device')
    if x.dtype == torch.float32:
        entry = kind + '_f32'
    elif x.dtype == torch.float64:
        entry = kind + '_f64'
    else:
        raise TypeError('x must be float32 or float64, got ' + str(x.dtype))
    if x.dim() < 1 or x.numel() == 0:
        raise TypeError('x must have at least one axis and one element, got shape ' + str(tuple(x.shape)))
    x = x.detach().contiguous()
    cols = x.shape[-1]
    rows = x.numel() // cols
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream(x.device).cuda_stream
        entry = 'ovl_' + entry + ('_reassociated' if reassociate else '')
        code = getattr(library(), entry)(x.data_ptr(), rows, cols, out.data_ptr(), stream)
    if code != 0:
        raise RowScanError(code, library().ovl_scan_last_error().decode('utf-8', 'replace'))
    return out


def cumsum(x, reassociate=False):
    """Running sum along the last axis in the dtype of ``x``: accumulated strictly left to right (the reference's
    bits), or with ``reassociate=True`` as a tree over the threads of a workgroup, at the speed of memory, with
    results that differ from the sequential ones by rounding."""
    return _scan('cumsum', x, reassociate)


def cumprod(x, reassociate=False):
    """Running product along the last axis in the dtype of ``x``; ``reassociate`` as for :func:`cumsum`."""
    return _scan('cumprod', x, reassociate)
