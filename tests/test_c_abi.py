"""The C-ABI launcher library: it loads, exports every function its header declares, and reports errors by code."""
import ctypes
import os
import re

import pytest

from opveclib_amd import launcher

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'ovl_launch.h')


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(ovl_[a-z_0-9]+)\s*\(', text)) - {'ovl_entry_fn'})


def test_header_and_binding_agree():
    assert declared_functions() == sorted(launcher.EXPORTED_SYMBOLS)


def test_every_declared_symbol_is_exported(launcher_library):
    raw = ctypes.CDLL(launcher.library_path)
    for name in declared_functions():
        assert hasattr(raw, name), name
    assert launcher_library.ovl_abi_version() == 1


def test_struct_layout_matches_header():
    # { void* data; int32_t dtype; uint64_t len; } on LP64: 8 + 4 (+4 padding) + 8
    assert ctypes.sizeof(launcher.OvlTensor) == 24
    assert launcher.OvlTensor.data.offset == 0
    assert launcher.OvlTensor.dtype.offset == 8
    assert launcher.OvlTensor.len.offset == 16


def test_dtype_sizes_and_messages(launcher_library):
    L = launcher_library
    sizes = {1: 2, 2: 4, 3: 8, 4: 1, 5: 2, 6: 4, 7: 8, 8: 1, 9: 2, 10: 4, 11: 8, 0: 0, 12: 0, 99: 0}
    for code, size in sizes.items():
        assert L.ovl_dtype_size(code) == size
    assert L.ovl_strerror(0) == b'success'
    for code in range(1, 7):
        assert len(L.ovl_strerror(code)) > 0
    assert b'unknown' in L.ovl_strerror(1234)


def test_error_codes_without_a_gpu(launcher_library, tmp_path):
    L = launcher_library
    handle = ctypes.c_void_p()
    assert L.ovl_lib_open(b'/nonexistent/operator.so', ctypes.byref(handle)) == launcher.OVL_EOPEN
    assert b'/nonexistent/operator.so' in L.ovl_last_error()
    assert L.ovl_lib_open(None, ctypes.byref(handle)) == launcher.OVL_EINVAL
    assert L.ovl_lib_close(None) == launcher.OVL_EINVAL

    # any shared object opens; a missing entry point is reported, not called
    assert L.ovl_lib_open(launcher.library_path.encode(), ctypes.byref(handle)) == launcher.OVL_OK
    fn = launcher.ENTRY_FN()
    assert L.ovl_lib_sym(handle, b'no_such_operator_generic_hip', ctypes.byref(fn)) == launcher.OVL_ESYMBOL
    assert L.ovl_launch(handle, b'no_such_operator_generic_hip', None, 0, None, 0, None) == launcher.OVL_ESYMBOL
    assert L.ovl_lib_close(handle) == launcher.OVL_OK

    null_fn = launcher.ENTRY_FN()
    assert L.ovl_launch_fn(null_fn, None, 0, None, 0, None) == launcher.OVL_EINVAL
    assert L.ovl_time(null_fn, None, 0, None, 0, None, 0, None) == launcher.OVL_EINVAL
    with pytest.raises(launcher.LauncherError):
        launcher.check(launcher.OVL_EOPEN)


def test_missing_launcher_is_a_loud_error(monkeypatch):
    monkeypatch.setattr(launcher, '_lib', None)
    monkeypatch.setattr(launcher, 'library_path', '/nonexistent/libovl_launch.so')
    with pytest.raises(RuntimeError):
        launcher.library()


# ----------------------------------------------------------------------------------------------------------------------
# the hand-written LSTM cell library (include/ovl_lstm.h)
# ----------------------------------------------------------------------------------------------------------------------
LSTM_HEADER = os.path.join(ROOT, 'include', 'ovl_lstm.h')


def lstm_declared_functions():
    text = open(LSTM_HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(ovl_[a-z_0-9]+)\s*\(', text)))


@pytest.fixture(scope='module')
def lstm_library():
    from opveclib_amd import lstm_cell
    if not os.path.exists(lstm_cell.library_path):
        lstm_cell.build()
    return lstm_cell.library()


def test_lstm_header_and_binding_agree(lstm_library):
    from opveclib_amd import lstm_cell
    assert lstm_declared_functions() == sorted(lstm_cell.EXPORTED_SYMBOLS)
    raw = ctypes.CDLL(lstm_cell.library_path)
    for name in lstm_declared_functions():
        assert hasattr(raw, name), name


def test_lstm_argument_errors_are_reported_before_any_gpu_work(lstm_library):
    L = lstm_library
    p = ctypes.c_void_p(64)             # never dereferenced: every call below is refused first
    assert L.ovl_lstm_forward(None, p, 1.0, 4, 8, 0, p, p, None) == launcher.OVL_EINVAL
    assert b'null' in L.ovl_lstm_last_error()
    assert L.ovl_lstm_forward(p, p, 1.0, 0, 8, 0, p, p, None) == launcher.OVL_EINVAL
    assert L.ovl_lstm_forward(p, p, 1.0, 4, 0, 0, p, p, None) == launcher.OVL_EINVAL
    assert L.ovl_lstm_forward(p, p, 1.0, 1 << 16, 1 << 16, 0, p, p, None) == launcher.OVL_EINVAL
    assert b'2^32' in L.ovl_lstm_last_error()
    assert L.ovl_lstm_backward(p, p, p, None, 1.0, 4, 8, 0, p, p, None) == launcher.OVL_EINVAL
    assert L.ovl_lstm_backward(p, p, p, p, 1.0, 0, 8, 0, p, p, None) == launcher.OVL_EINVAL


def test_lstm_python_wrapper_validates_its_arguments():
    import numpy as np
    import torch
    from opveclib_amd import lstm_cell
    concat = torch.zeros(4, 32)
    c = torch.zeros(4, 8)
    with pytest.raises(RuntimeError):
        lstm_cell.lstm_cell(concat, c, 1.0)                         # host tensors
    with pytest.raises((TypeError, AttributeError)):
        lstm_cell.lstm_cell(np.zeros((4, 32), np.float32), c, 1.0)
    with pytest.raises(ValueError):
        lstm_cell._fast('sloppy')
    with pytest.raises(TypeError):
        lstm_cell._shapes(torch.zeros(4, 30), [], [])
    with pytest.raises(TypeError):
        lstm_cell._shapes(concat, [torch.zeros(4, 9)], ['c'])
    assert lstm_cell._shapes(concat, [c], ['c']) == (4, 8)


# ----------------------------------------------------------------------------------------------------------------------
# the hand-written row scan library (include/ovl_scan.h)
# ----------------------------------------------------------------------------------------------------------------------
SCAN_HEADER = os.path.join(ROOT, 'include', 'ovl_scan.h')


def scan_declared_functions():
    text = open(SCAN_HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(ovl_[a-z_0-9]+)\s*\(', text)))


def test_scan_header_binding_and_argument_errors():
    from opveclib_amd import row_scan
    if not os.path.exists(row_scan.library_path):
        row_scan.build()
    L = row_scan.library()
    assert scan_declared_functions() == sorted(row_scan.EXPORTED_SYMBOLS)
    raw = ctypes.CDLL(row_scan.library_path)
    for name in scan_declared_functions():
        assert hasattr(raw, name), name
    p = ctypes.c_void_p(64)             # never dereferenced: every call below is refused first
    for entry in [getattr(L, name) for name in row_scan.SCAN_SYMBOLS]:
        assert entry(None, 4, 8, p, None) == launcher.OVL_EINVAL
        assert b'null' in L.ovl_scan_last_error()
        assert entry(p, 4, 8, None, None) == launcher.OVL_EINVAL
        assert entry(p, 0, 8, p, None) == launcher.OVL_EINVAL
        assert entry(p, 4, 0, p, None) == launcher.OVL_EINVAL
        assert entry(p, 1 << 16, 1 << 16, p, None) == launcher.OVL_EINVAL
        assert b'2^32' in L.ovl_scan_last_error()
    # the measurement aid: strips of 4, 8 or 16 lines; load, store or copy
    assert L.ovl_strip_copy_f64(None, 4, 8, p, 8, 3, None) == launcher.OVL_EINVAL
    assert L.ovl_strip_copy_f64(p, 4, 8, None, 8, 3, None) == launcher.OVL_EINVAL
    assert L.ovl_strip_copy_f64(p, 0, 8, p, 8, 3, None) == launcher.OVL_EINVAL
    assert L.ovl_strip_copy_f64(p, 1 << 16, 1 << 16, p, 8, 3, None) == launcher.OVL_EINVAL
    assert L.ovl_strip_copy_f64(p, 4, 8, p, 5, 3, None) == launcher.OVL_EINVAL
    assert b'lines per workgroup' in L.ovl_scan_last_error()
    assert L.ovl_strip_copy_f64(p, 4, 8, p, 8, 0, None) == launcher.OVL_EINVAL
    assert L.ovl_strip_copy_f64(p, 4, 8, p, 8, 4, None) == launcher.OVL_EINVAL
    assert b'mode' in L.ovl_scan_last_error()


def test_scan_python_wrapper_validates_its_arguments():
    import numpy as np
    import torch
    from opveclib_amd import row_scan
    with pytest.raises(TypeError):
        row_scan.cumsum(np.zeros((4, 8), np.float32))
    with pytest.raises(RuntimeError):
        row_scan.cumsum(torch.zeros(4, 8))                          # a host tensor
