import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: test needs an AMD GPU (runs the HIP path through the C-ABI launcher)')
    # The parity tests compare with the oracle bit for bit, which is the promise of the 'exact' math mode: an
    # `evaluate` call of this suite that names no mode means that one.  The package's own default ('ulp2', within two
    # float32 units in the last place per operator) has tests that name it or reset this pin (test_frontend.py,
    # test_gpu_ulp2.py).
    import opveclib_amd
    opveclib_amd.set_math_mode('exact')


def _gpu_available():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_available():
        return
    skip = pytest.mark.skip(reason='no HIP device in this environment')
    for item in items:
        if 'gpu' in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope='session')
def launcher_library():
    from opveclib_amd import launcher
    launcher.build()
    return launcher.library()


@pytest.fixture(scope='session', autouse=True)
def _oracle_driver():
    import oracle
    oracle.build_driver()
