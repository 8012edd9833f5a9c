"""
Local runtime environment: version, logger, operator cache directories and the hipcc toolchain location.

Counterpart of the reference's opveclib/local.py (version string, ``logger``, ``cache_directory``,
``clear_op_cache``, compiler selection through environment variables, lines 17-63).

Two directories hold compiled operators, both keyed by content hash:

* ``prebuilt_directory`` - inside the package; filled ahead of time (``python -m opveclib_amd.prebuild`` or the
  repository's build step) and only ever read at run time;
* ``cache_directory`` - per user (``$OPVECLIB_HOME`` or ``~/.opveclib_amd``), filled on demand by the JIT path.
"""

import errno
import logging
import os
import shutil

#: Version string for current version; part of every operator hash
version = '0.1.0-gfx950'

#: The log
logger = logging.getLogger('opveclib_amd')

_package_directory = os.path.dirname(os.path.abspath(__file__))

#: ROCm installation that provides hipcc
rocm_directory = os.getenv('ROCM_PATH', os.getenv('ROCM_HOME', '/opt/rocm'))

#: The HIP compiler driver
hipcc = os.getenv('OPVECLIB_HIPCC', os.path.join(rocm_directory, 'bin', 'hipcc'))

#: The only code object target of this package
gpu_arch = 'gfx950'

_base_cache_directory = os.getenv('OPVECLIB_HOME', os.path.join(os.path.expanduser('~'), '.opveclib_amd'))

#: Directory where operators compiled on demand are stored
cache_directory = os.path.join(_base_cache_directory, version)

#: Directory of operators compiled ahead of time and shipped with the package (read-only at run time)
prebuilt_directory = os.path.join(_package_directory, '_prebuilt')

#: Directory of the package's native sources and the built launcher library
csrc_directory = os.path.join(_package_directory, 'csrc')


def _ensure_directory(path):
    try:
        os.makedirs(path)
    except OSError as exception:
        if exception.errno != errno.EEXIST:
            raise


def ensure_cache_directory():
    _ensure_directory(cache_directory)
    return cache_directory


def clear_op_cache():
    """
    Delete all operators compiled on demand in the current cache directory. Generally used to make sure there are
    no stale operators in the cache when testing and debugging.  Operators shipped in ``prebuilt_directory`` are
    content-addressed by source text and compiler flags and are left alone.
    """
    if not os.path.isdir(cache_directory):
        return
    for filename in os.listdir(cache_directory):
        if filename[0] == 'f':
            os.remove(os.path.join(cache_directory, filename))


def hip_compiler_available():
    return os.path.exists(hipcc) or shutil.which(hipcc) is not None


def _gpu_present():
    try:
        import torch
        return bool(torch.cuda.is_available())
    except Exception:  # pragma: no cover - torch missing or broken
        return False


def __getattr__(name):
    # ``hip_enabled`` tells whether a HIP device is usable in this process.  It is resolved on first use because
    # importing torch is slow; ``cuda_enabled`` is the reference's spelling of the same question (local.py:52-63).
    if name in ('hip_enabled', 'cuda_enabled'):
        value = _gpu_present()
        globals()['hip_enabled'] = value
        globals()['cuda_enabled'] = value
        return value
    raise AttributeError('module %r has no attribute %r' % (__name__, name))
