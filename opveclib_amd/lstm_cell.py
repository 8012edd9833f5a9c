"""
The hand-written LSTM cell kernels (``csrc/ovl_lstm.hip``, C ABI in ``include/ovl_lstm.h``) from Python.

Same two functions as the DSL operators ``opveclib_amd.lstm.lstm`` / ``lstm_grad`` (the reference's lstm/lstm.py:32-105)
and the same bits, but the shape is a run-time argument: nothing is traced, generated or compiled when they are
called, which is what a recurrent loop over many shapes, or a machine without a compiler, needs.  Inputs are float32
torch tensors on a HIP device; launches go to the current PyTorch HIP stream and do not synchronise.
"""

import ctypes
import os
import subprocess

from . import local

library_path = os.path.join(local.csrc_directory, 'libovl_lstm.so')
source_path = os.path.join(local.csrc_directory, 'ovl_lstm.hip')
include_directory = os.path.normpath(os.path.join(local.csrc_directory, '..', '..', 'include'))

EXPORTED_SYMBOLS = ('ovl_lstm_forward', 'ovl_lstm_backward', 'ovl_lstm_last_error')


def build(force=False):
    """Compile the library with hipcc next to its source (same flags as generated operators); returns its path."""
    from .compiler import HIPCC_FLAGS
    headers = [os.path.join(local.csrc_directory, n) for n in ('ovl_device.h', 'ovl_math.h', 'ovl_fast_math.h', 'ovl_index_div.h')]
    newest = max(os.path.getmtime(p) for p in [source_path] + headers)
    if not force and os.path.exists(library_path) and os.path.getmtime(library_path) >= newest:
        return library_path
    tmp = library_path + '.tmp.%d' % os.getpid()
    cmd = [local.hipcc] + list(HIPCC_FLAGS) + ['-I' + include_directory, '-I' + local.csrc_directory,
                                               source_path, '-o', tmp]
    try:
        subprocess.check_output(cmd, stderr=subprocess.STDOUT, universal_newlines=True)
    except subprocess.CalledProcessError as exception:
        raise RuntimeError('hipcc failed for the LSTM cell library:\n' + exception.output)
    os.replace(tmp, library_path)
    return library_path


_lib = None


def library():
    """The loaded library (loads it on first use); there is no fallback when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(library_path):
        raise RuntimeError('The LSTM cell library ' + library_path + ' has not been built. '
                           'Run "python -m opveclib_amd.build" first.')
    lib = ctypes.CDLL(library_path)
    p = ctypes.c_void_p
    lib.ovl_lstm_forward.argtypes = [p, p, ctypes.c_float, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int32, p, p, p]
    lib.ovl_lstm_forward.restype = ctypes.c_int
    lib.ovl_lstm_backward.argtypes = [p, p, p, p, ctypes.c_float, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int32,
                                      p, p, p]
    lib.ovl_lstm_backward.restype = ctypes.c_int
    lib.ovl_lstm_last_error.restype = ctypes.c_char_p
    _lib = lib
    return lib


class LstmCellError(RuntimeError):
    def __init__(self, code, detail):
        RuntimeError.__init__(self, 'ovl_lstm error %d: %s' % (code, detail))
        self.code = code


def _check(code):
    if code != 0:
        raise LstmCellError(code, library().ovl_lstm_last_error().decode('utf-8', 'replace'))


def _fast(math_mode):
    from .operator import get_math_mode, MATH_MODES
    if math_mode is None:
        math_mode = get_math_mode()
    if math_mode not in MATH_MODES:
        raise ValueError('math_mode must be one of ' + str(MATH_MODES))
    # the cell adds products of either sign, so only the 'fast' mode, which promises nothing per operator, may use the
    # hardware-based routines; 'ulp2' keeps the bit-compatible ones here, as the code generator does for this operator
    return 1 if math_mode == 'fast' else 0


def _prepare(torch, tensors, names):
    device = tensors[0].device
    if device.type != 'cuda':
        raise RuntimeError('the LSTM cell kernels run on an AMD GPU: tensors must live on a HIP device')
    out = []
    for t, name in zip(tensors, names):
        if not isinstance(t, torch.Tensor):
            raise TypeError(name + ' must be a torch tensor')
        if t.dtype != torch.float32:
            raise TypeError(name + ' must be float32, got ' + str(t.dtype))
        if t.device != device:
            raise TypeError(name + ' is on ' + str(t.device) + ', expected ' + str(device))
        out.append(t.detach().contiguous())
    return device, out


def _shapes(concat, others, names):
    if concat.dim() != 2 or concat.shape[1] % 4 != 0 or concat.shape[1] == 0 or concat.shape[0] == 0:
        raise TypeError('concat must be [batch, 4 * units], got ' + str(tuple(concat.shape)))
    batch, units = concat.shape[0], concat.shape[1] // 4
    for t, name in zip(others, names):
        if tuple(t.shape) != (batch, units):
            raise TypeError('%s must be [%d, %d], got %s' % (name, batch, units, tuple(t.shape)))
    return batch, units


def lstm_cell(concat, c, forget_bias, math_mode=None):
    """
    ``new_c = c * sigmoid(f + forget_bias) + sigmoid(i) * tanh(j)``, ``new_h = tanh(new_c) * sigmoid(o)`` with the
    gates i, j, f, o side by side in ``concat`` [batch, 4 * units] (lstm/lstm.py:32-59).

    :return: (new_c, new_h), each [batch, units]
    """
    import torch
    device, (concat, c) = _prepare(torch, [concat, c], ['concat', 'c'])
    batch, units = _shapes(concat, [c], ['c'])
    new_c = torch.empty_like(c)
    new_h = torch.empty_like(c)
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        _check(library().ovl_lstm_forward(concat.data_ptr(), c.data_ptr(), float(forget_bias), batch, units,
                                          _fast(math_mode), new_c.data_ptr(), new_h.data_ptr(), stream))
    return new_c, new_h


def lstm_cell_grad(concat, c, d_new_c, d_new_h, forget_bias, math_mode=None):
    """
    Gradients of :func:`lstm_cell` with respect to ``concat`` and ``c`` given those of ``new_c`` and ``new_h``
    (lstm/lstm.py:62-105; the cell state is recomputed).

    :return: (d_concat [batch, 4 * units], d_c [batch, units])
    """
    import torch
    device, (concat, c, d_new_c, d_new_h) = _prepare(torch, [concat, c, d_new_c, d_new_h],
                                                     ['concat', 'c', 'd_new_c', 'd_new_h'])
    batch, units = _shapes(concat, [c, d_new_c, d_new_h], ['c', 'd_new_c', 'd_new_h'])
    d_concat = torch.empty_like(concat)
    d_c = torch.empty_like(c)
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        _check(library().ovl_lstm_backward(concat.data_ptr(), c.data_ptr(), d_new_c.data_ptr(), d_new_h.data_ptr(),
                                           float(forget_bias), batch, units, _fast(math_mode),
                                           d_concat.data_ptr(), d_c.data_ptr(), stream))
    return d_concat, d_c


def lstm_cell_torch(concat, c, forget_bias, math_mode=None):
    """:func:`lstm_cell` as a differentiable PyTorch function (gradients through :func:`lstm_cell_grad`)."""
    import torch

    class _LstmCell(torch.autograd.Function):
        @staticmethod
        def forward(ctx, concat_t, c_t):
            ctx.save_for_backward(concat_t, c_t)
            return lstm_cell(concat_t, c_t, forget_bias, math_mode)

        @staticmethod
        @torch.autograd.function.once_differentiable
        def backward(ctx, d_new_c, d_new_h):
            concat_t, c_t = ctx.saved_tensors
            if d_new_c is None:
                d_new_c = torch.zeros_like(c_t)
            if d_new_h is None:
                d_new_h = torch.zeros_like(c_t)
            return lstm_cell_grad(concat_t, c_t, d_new_c, d_new_h, forget_bias, math_mode)

    return _LstmCell.apply(concat, c)
