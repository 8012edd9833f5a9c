"""Builds the native test libraries of this directory with hipcc (cross-compiles for gfx950 without a GPU)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(os.path.dirname(HERE)), 'opveclib_amd', 'csrc')
LIBRARY = os.path.join(HERE, 'libexhaustive_math.so')
HAND_WRITTEN = os.path.join(HERE, 'libhand_written_add.so')


def _tanh_body():
    """The text of tanhf_ from the product header, so the test compiles a second copy with IEEE divisions."""
    text = open(os.path.join(CSRC, 'ovl_math.h')).read()
    start = text.index('OVL_HD float tanhf_(float x) {')
    end = text.index('\n}\n', start) + 3
    return text[start:end]


def build():
    root = os.path.dirname(os.path.dirname(HERE))
    if root not in sys.path:
        sys.path.insert(0, root)
    from opveclib_amd.compiler import HIPCC_FLAGS
    from opveclib_amd import local
    include = os.path.join(HERE, '_generated')
    os.makedirs(include, exist_ok=True)
    with open(os.path.join(include, 'tanh_body.inc'), 'w') as f:
        f.write(_tanh_body())
    cmd = [local.hipcc] + list(HIPCC_FLAGS) + ['-I', CSRC, '-I', include, '-pthread',
                                                os.path.join(HERE, 'exhaustive_math.hip'), '-o', LIBRARY]
    subprocess.check_call(cmd)
    subprocess.check_call([local.hipcc] + list(HIPCC_FLAGS) + ['-I', CSRC, os.path.join(HERE, 'hand_written_add.hip'),
                                                            '-o', HAND_WRITTEN])
    return LIBRARY


if __name__ == '__main__':
    print(build())
