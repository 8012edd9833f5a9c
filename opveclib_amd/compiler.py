"""
Compile-and-cache layer: generated HIP source -> operator shared library.

Counterpart of ``_make_generic_cuda`` in the reference (opveclib/operator.py:2065-2096: write the source into the
cache directory, run the device compiler, reuse the library when it already exists).  Libraries are named by the
hash of their source text, the compiler flags and the device support header, so a change to any of them selects a
new file.  Lookup order: the package's prebuilt directory, then the per-user cache; a miss compiles into the
per-user cache (or into the prebuilt directory while ``prebuild_mode`` is on).
"""

import hashlib
import os
import subprocess
import threading

from . import local
from .local import logger

#: hipcc flags for operator libraries.  Contraction of a*b+c into fma is off so that results match code compiled
#: without fused multiply-add; packed fp32 instructions are disabled.
HIPCC_FLAGS = ('--offload-arch=' + local.gpu_arch, '-O3', '-std=c++17', '-fPIC', '-shared',
               '-ffp-contract=off', '-fno-fast-math',
               '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
               '-Wno-unused-value', '-Wno-unused-variable')

#: while True, operators are compiled into the package's prebuilt directory
prebuild_mode = False
#: while True, operators are compiled even when a built library exists (the "does it build" check)
force_rebuild = False

_header_paths = [os.path.join(local.csrc_directory, name) for name in ('ovl_device.h', 'ovl_math.h', 'ovl_fast_math.h', 'ovl_wave_scan.h')]
_lock = threading.Lock()
_header_cache = []


def _header_text():
    if not _header_cache:
        text = ''
        for path in _header_paths:
            with open(path, 'r') as f:
                text += f.read()
        _header_cache.append(text)
    return _header_cache[0]


def library_name(source):
    digest = hashlib.sha224()
    digest.update(source.encode('utf-8'))
    digest.update(' '.join(HIPCC_FLAGS).encode('utf-8'))
    digest.update(_header_text().encode('utf-8'))
    return 'f' + digest.hexdigest() + '_generic_hip.so'


def find_library(source):
    """Path of an already built library for ``source`` or None."""
    name = library_name(source)
    for directory in (local.prebuilt_directory, local.cache_directory):
        path = os.path.join(directory, name)
        if os.path.exists(path):
            return path
    return None


def build_library(source):
    """Return the path of the operator library for ``source``, compiling it when no cached copy exists."""
    found = find_library(source)
    if found is not None and not force_rebuild:
        return found

    directory = local.prebuilt_directory if prebuild_mode else local.ensure_cache_directory()
    os.makedirs(directory, exist_ok=True)
    name = library_name(source)
    so_path = os.path.join(directory, name)
    src_path = so_path[:-3] + '.hip'
    # Concurrent builders of the same library each compile into a private temporary file and rename it into place;
    # the rename is atomic, so readers only ever see complete libraries.
    logger.debug('Compiling HIP operator ' + name)
    tag = '.tmp.%d.%d' % (os.getpid(), threading.get_ident())
    tmp_src = src_path + tag
    with open(tmp_src, 'w') as f:
        f.write(source)
    os.replace(tmp_src, src_path)
    tmp_path = so_path + tag
    cmd = [local.hipcc] + list(HIPCC_FLAGS) + ['-I' + local.csrc_directory, src_path, '-o', tmp_path]
    try:
        subprocess.check_output(cmd, stderr=subprocess.STDOUT, universal_newlines=True)
    except subprocess.CalledProcessError as exception:
        logger.error('hipcc error: ' + exception.output)
        raise RuntimeError('hipcc failed for ' + src_path + ':\n' + exception.output)
    os.replace(tmp_path, so_path)
    return so_path
