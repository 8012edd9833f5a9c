"""
A 2-D indexed operator: an integer-driven gather combined with a transposed scatter.

Worker (i, j) of an [M, N] workgroup reads ``a[i, j]`` and ``b_flat[(i*stride + j) % b_flat.size]`` and writes
``alpha*a[i, j] + b_flat[...]`` to ``out[j, i]``.  The index arithmetic is carried out in the position's uint32, like
the computed store index of the reference's README.rst:40-60 and the 2-D index arithmetic of its pad/crop test
operators (opveclib/test/test_operator_merge.py:118-163).
"""

import opveclib_amd as ovl


@ovl.operator()
def gather_transpose(a, b_flat, alpha=None, stride=None):
    assert a.rank == 2
    assert b_flat.rank == 1
    assert a.dtype == b_flat.dtype
    rows, cols = a.shape

    out = ovl.output([cols, rows], a.dtype)
    pos = ovl.position_in([rows, cols])
    i = pos[0]
    j = pos[1]

    gathered = b_flat[(i * stride + j) % b_flat.size]
    out[j, i] = alpha * a[i, j] + gathered
    return out
