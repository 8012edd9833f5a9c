"""
Exhaustive checks of the device float32 math on the GPU, through the native test library of tests/native.

`test_device_math_equals_host_libm_*`: the device expf / logf / tanhf and the reciprocal that generated kernels call are
evaluated for float bit patterns and compared bit for bit with the host C library's expf / logf / tanhf / (1.0f / x) on
the machine the test runs on: all 2^32 arguments of each (about a second per function with 16 host threads;
OVL_EXHAUSTIVE=0 compares every 16th bit pattern only: 2^28 arguments per function, all exponents and both signs).
`test_tanh_shortened_divisions_*`: all 2^32 arguments, device against device.
`test_in_range_variants_*`: the variants of expf / logf / reciprocal / division without a rare-argument block, on every
argument the code generator may hand them (division: 2^32 operand pairs), device against device.
`test_fast_mode_routines_*`: the optional fast routines against the host C library, largest distance in units in the
last place (measured over all 2^32 arguments: expf 1, logf 2, tanhf 2, reciprocal 0).
`test_formula_routines_*`: the sigmoid / log1p / expm1 routines that the 'ulp2' math mode puts in place of the
reference's formulas, against those formulas evaluated with the host C library, on every float32 of the domain on which the code
generator uses them: at most 2 units in the last place.
"""
import ctypes
import os

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY = os.path.join(HERE, 'native', 'libexhaustive_math.so')
FUNCTIONS = {'expf': 0, 'logf': 1, 'tanhf': 2, 'reciprocal': 3}


@pytest.fixture(scope='module')
def lib():
    if not os.path.exists(LIBRARY):
        from tests.native import build
        build.build()
    handle = ctypes.CDLL(LIBRARY)
    handle.ovl_exh_against_host.argtypes = [ctypes.c_int, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32,
                                            ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint32)]
    handle.ovl_exh_tanh_division.argtypes = [ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint32)]
    return handle


@pytest.mark.parametrize('name', sorted(FUNCTIONS))
def test_device_math_equals_host_libm(lib, name):
    step = 16 if os.environ.get('OVL_EXHAUSTIVE') == '0' else 1
    count = (1 << 32) // step
    bad = ctypes.c_uint64(0)
    first = ctypes.c_uint32(0)
    threads = min(16, os.cpu_count() or 1)
    err = lib.ovl_exh_against_host(FUNCTIONS[name], count, step, threads, ctypes.byref(bad), ctypes.byref(first))
    assert err == 0, 'HIP error %d' % err
    assert bad.value == 0, '%s: %d of %d arguments differ from the host C library, first at bits 0x%08x' % (
        name, bad.value, count, first.value)


FAST_FUNCTIONS = {'expf': (5, 1), 'logf': (6, 2), 'tanhf': (7, 2), 'reciprocal': (8, 0)}


@pytest.mark.parametrize('name', sorted(FAST_FUNCTIONS))
def test_fast_mode_routines_within_two_ulp_of_host_libm(lib, name):
    """The routines of the optional 'fast' math mode: distance from the host C library in units in the last place."""
    lib.ovl_exh_ulp_against_host.argtypes = [ctypes.c_int, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32,
                                             ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64),
                                             ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32)]
    fn, bound = FAST_FUNCTIONS[name]
    step = 16 if os.environ.get('OVL_EXHAUSTIVE') == '0' else 1
    differing, beyond = ctypes.c_uint64(0), ctypes.c_uint64(0)
    largest, where = ctypes.c_uint32(0), ctypes.c_uint32(0)
    err = lib.ovl_exh_ulp_against_host(fn, (1 << 32) // step, step, min(16, os.cpu_count() or 1),
                                       ctypes.byref(differing), ctypes.byref(beyond), ctypes.byref(largest),
                                       ctypes.byref(where))
    assert err == 0, 'HIP error %d' % err
    assert beyond.value == 0 and largest.value <= bound, '%s: %d ulp at bits 0x%08x, %d arguments beyond 2 ulp' % (
        name, largest.value, where.value, beyond.value)


def test_checker_reports_a_library_that_differs_in_the_last_place(lib):
    """Self-test: the device math library's own expf is a correct expf but not the host's; the checker must see it."""
    bad = ctypes.c_uint64(0)
    first = ctypes.c_uint32(0)
    err = lib.ovl_exh_against_host(4, (1 << 32) // 16, 16, 16, ctypes.byref(bad), ctypes.byref(first))
    assert err == 0
    assert bad.value > 1000


def test_tanh_shortened_divisions_equal_ieee_divisions_for_all_arguments(lib):
    bad = ctypes.c_uint64(0)
    first = ctypes.c_uint32(0)
    err = lib.ovl_exh_tanh_division(ctypes.byref(bad), ctypes.byref(first))
    assert err == 0, 'HIP error %d' % err
    assert bad.value == 0, '%d arguments differ, first at bits 0x%08x' % (bad.value, first.value)


IN_RANGE = {'expf': (0, 1 << 31), 'logf': (1, 1 << 30), 'reciprocal': (2, 1 << 31), 'division': (3, 1 << 31)}


@pytest.mark.parametrize('name', sorted(IN_RANGE))
def test_in_range_variants_equal_the_full_routines(lib, name):
    """What the code generator emits for arguments it has proved harmless returns the same bits as the full routine
    (for division: as the IEEE '/' operator) on all of those arguments."""
    lib.ovl_exh_in_range.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64),
                                     ctypes.POINTER(ctypes.c_uint32)]
    which, at_least = IN_RANGE[name]
    bad, compared = ctypes.c_uint64(0), ctypes.c_uint64(0)
    first = ctypes.c_uint32(0)
    err = lib.ovl_exh_in_range(which, ctypes.byref(bad), ctypes.byref(compared), ctypes.byref(first))
    assert err == 0, 'HIP error %d' % err
    assert compared.value >= at_least, 'only %d arguments were compared' % compared.value
    assert bad.value == 0, '%s: %d of %d arguments differ, first at 0x%08x' % (name, bad.value, compared.value,
                                                                               first.value)


def _bits(value):
    import struct
    return struct.unpack('<I', struct.pack('<f', value))[0]


@pytest.mark.parametrize('kind', ['sigmoid', 'log1p', 'expm1', 'log1p_unit', 'expm1_small', 'sigmoid_small'])
def test_formula_routines_within_two_ulp_of_the_reference_formulas(lib, kind):
    """Every float32 argument of the domain the code generator allows (hipgen/accuracy.py: IDIOM_DOMAIN, and
    NARROW_DOMAIN for the shorter forms `_unit` / `_small`)."""
    from opveclib_amd.hipgen import accuracy
    lib.ovl_exh_ulp_in_range.argtypes = [ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32] + \
        [ctypes.POINTER(ctypes.c_uint64)] * 3 + [ctypes.POINTER(ctypes.c_uint32)] * 2
    narrow = {'log1p_unit': 'log1p', 'expm1_small': 'expm1', 'sigmoid_small': 'sigmoid'}.get(kind)
    # (the intervals tested at run time include the one a value range must prove, IDIOM_DOMAIN)
    intervals = [accuracy.NARROW_DOMAIN[narrow]] if narrow else list(accuracy.GUARD_DOMAIN[kind])
    assert narrow or accuracy.IDIOM_DOMAIN[kind] in intervals
    bound = accuracy.TOLERANCE if narrow else accuracy.ROUTINE_ULPS[kind]
    # ranges of bit patterns of one sign each: consecutive patterns are consecutive floats
    spans = []
    for lo, hi in intervals:
        if lo > 0:
            spans.append((_bits(lo), _bits(hi)))
        elif hi < 0:
            spans.append((_bits(hi), _bits(lo)))
        else:
            spans += [(_bits(-0.0), _bits(lo)), (_bits(0.0), _bits(hi))]
    total = total_differing = 0
    for first, last in spans:
        compared, differing, beyond = ctypes.c_uint64(0), ctypes.c_uint64(0), ctypes.c_uint64(0)
        largest, where = ctypes.c_uint32(0), ctypes.c_uint32(0)
        fn = {'log1p': 9, 'expm1': 10, 'sigmoid': 11, 'log1p_unit': 12, 'expm1_small': 13, 'sigmoid_small': 14}[kind]
        err = lib.ovl_exh_ulp_in_range(fn, first, last, min(16, os.cpu_count() or 1), ctypes.byref(compared),
                                       ctypes.byref(differing), ctypes.byref(beyond), ctypes.byref(largest),
                                       ctypes.byref(where))
        assert err == 0, 'HIP error %d' % err
        assert beyond.value == 0 and largest.value <= bound, \
            '%s: %d ulp at bits 0x%08x, %d arguments beyond 2 ulp' % (kind, largest.value, where.value, beyond.value)
        total += compared.value
        total_differing += differing.value
    assert total >= {'log1p_unit': 32 << 20, 'expm1_small': 90 << 20}.get(kind, 140 << 20)
    assert total_differing > 0          # it is not the formula itself
