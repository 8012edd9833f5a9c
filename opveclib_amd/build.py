"""
Build step for the package's native code: ``python -m opveclib_amd.build`` compiles the C-ABI launcher
(csrc/ovl_launch.cpp -> csrc/libovl_launch.so) the hand-written LSTM cell kernels (csrc/ovl_lstm.hip -> csrc/libovl_lstm.so)
and the hand-written row scans (csrc/ovl_scan.hip -> csrc/libovl_scan.so) with hipcc.  Generated operators are compiled on demand and cached;
``python -m opveclib_amd.build --check`` additionally compiles one small operator to verify the toolchain.
"""

import sys


def build_all(force=True, check=False):
    from . import launcher, lstm_cell, row_scan
    path = launcher.build(force=force)
    lstm_cell.build(force=force)
    row_scan.build(force=force)
    if check:
        import numpy as np
        from . import runtime
        from .stdops import add
        a = np.zeros(8, dtype=np.float32)
        runtime.build_operator(add(a, a).expression_dag)
    return path


if __name__ == '__main__':
    print(build_all(force=True, check='--check' in sys.argv))
