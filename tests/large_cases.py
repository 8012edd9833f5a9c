"""
Operators at the largest sizes the path supports: workgroups just below 2^32 workers (positions are 32-bit, as in the
reference: opveclib/expression.py:582-608), tensors beyond 2^31 and 2^32 elements (flat indices are 64-bit:
expression.py:859-973).  Data-movement and integer operators only, so that PyTorch on the GPU is an independent,
bit-exact reference at sizes the CPU oracle would need minutes for.

`cases(make)` yields (name, operator output, reference function); `make(shape, dtype)` supplies the tensors: shape-only
placeholders when the kernels are compiled ahead of time, device tensors in the GPU test.
"""
import numpy as np

import opveclib_amd as ovl
from opveclib_amd import stdops
from opveclib_amd.examples import shift_cyclic, cumsum, gather_transpose


@ovl.operator()
def reverse(x):
    """out[n - 1 - p] = x[p]: nothing to vectorise on 1-byte elements, one worker per thread."""
    pos = ovl.position_in(x.shape)
    out = ovl.output_like(x)
    out[(x.shape[0] - 1) - pos[0]] = x[pos]
    return out


@ovl.operator()
def channels_last(x):
    """[N, C, H, W] stored as [N, H, W, C]: unit stride along a workgroup dimension that is not one of the last two."""
    n, c, h, w = x.shape
    out = ovl.output([n, h, w, c], x.dtype)
    pos = ovl.position_in(x.shape)
    out[pos[0], pos[2], pos[3], pos[1]] = x[pos]
    return out


@ovl.operator()
def row_sum(x):
    rows, cols = x.shape
    out = ovl.output([rows], x.dtype)
    r = ovl.position_in([rows])[0]
    acc = ovl.variable(0, x.dtype)
    for j in ovl.arange(cols):
        acc <<= acc + x[r, j]
    out[r] = acc
    return out


@ovl.operator()
def column_sum(x):
    rows, cols = x.shape
    out = ovl.output([cols], x.dtype)
    c = ovl.position_in([cols])[0]
    acc = ovl.variable(0, x.dtype)
    for i in ovl.arange(rows):
        acc <<= acc + x[i, c]
    out[c] = acc
    return out


@ovl.operator()
def running_dot(a, b):
    """out[r, i] = sum of a[r, k] * b[r, k] over k <= i: a row scan whose body reads two inputs."""
    rows, cols = a.shape
    out = ovl.output_like(a)
    r = ovl.position_in([rows])[0]
    acc = ovl.variable(a[r, 0] * b[r, 0], a.dtype)
    out[r, 0] = acc
    for i in ovl.arange(1, cols):
        acc <<= acc + a[r, i] * b[r, i]
        out[r, i] = acc
    return out


def placeholder(shape, dtype):
    """An array of the given shape that owns one element (every stride is zero): enough to trace an operator."""
    shape = shape if isinstance(shape, tuple) else (shape,)
    return np.lib.stride_tricks.as_strided(np.zeros(1, dtype), shape=shape, strides=(0,) * len(shape))


def cases(make):
    import torch

    n = 2 ** 32 - 3       # 2^24 workgroups of 256 one-worker threads would be 2^32 threads: the kernel strides
    x = make(n, np.uint8)
    yield 'reverse uint8 [2^32 - 3]', reverse(x), lambda: torch.flip(x, [0])

    n = 2 ** 32 - 256     # sixteen workers per thread
    a, b = make(n, np.uint8), make(n, np.uint8)
    yield 'add uint8 [2^32 - 256]', stdops.add(a, b), lambda: a + b

    n = 2 ** 31 + 2 ** 20     # byte offsets beyond 2^33
    a, b = make(n, np.float32), make(n, np.float32)
    yield 'add float32 [2^31 + 2^20]', stdops.add(a, b), lambda: a + b

    n = 2 ** 31 + 4
    a = make(n, np.float32)
    yield 'shift_cyclic float32 [2^31 + 4]', shift_cyclic(a), lambda: torch.roll(a, 1)

    a = make((131088, 32832), np.int32)     # 2^32 + 2^23.3 elements, 131088 workers
    yield 'cumsum int32 [131088, 32832]', cumsum(a, axis=1), lambda: torch.cumsum(a, 1, dtype=torch.int32)

    a = make((70, 2 ** 21 + 64), np.int32)  # more than two million lines along the scanned axis
    yield 'cumsum int32 [70, 2^21 + 64] along axis 0', cumsum(a, axis=0), lambda: torch.cumsum(a, 0, dtype=torch.int32)

    a = make((3000, 70001), np.int32)       # rows that are neither whole groups of 64 columns nor 16-byte aligned
    yield 'cumsum int32 [3000, 70001]', cumsum(a, axis=1), lambda: torch.cumsum(a, 1, dtype=torch.int32)

    a = make((48, 256, 168, 168), np.int32)   # the tile template over dimensions 1 and 3, 2016 batches
    yield 'channels_last int32 [48, 256, 168, 168]', channels_last(a), lambda: a.permute(0, 2, 3, 1).contiguous()

    a = make((8192, 70001), np.int32)       # row reduction: wide groups, narrow groups and a partial group
    yield 'row_sum int32 [8192, 70001]', row_sum(a), lambda: torch.sum(a, 1, dtype=torch.int32)

    a = make((70001, 4100), np.int32)       # column reduction with a last strip that is not full
    yield 'column_sum int32 [70001, 4100]', column_sum(a), lambda: torch.sum(a, 0, dtype=torch.int32)

    a, b = make((3000, 70001), np.int32), make((3000, 70001), np.int32)     # a scan over two inputs
    yield 'running_dot int32 [3000, 70001]', running_dot(a, b), lambda: torch.cumsum(a * b, 1, dtype=torch.int32)

    rows, cols = 65536, 32768 + 256         # 2^31 + 2^24 workers, transposed store
    a, flat = make((rows, cols), np.float32), make(rows * cols, np.float32)

    def gathered_and_transposed():
        out = torch.empty((cols, rows), dtype=torch.float32, device=a.device)
        j = torch.arange(cols, device=a.device, dtype=torch.int64)[None, :]
        for r0 in range(0, rows, 4096):
            i = torch.arange(r0, r0 + 4096, device=a.device, dtype=torch.int64)[:, None]
            index = ((i * 7919 + j) & 0xffffffff) % (rows * cols)
            out[:, r0:r0 + 4096] = (0.5 * a[r0:r0 + 4096] + flat[index]).T
        return out
    yield 'gather_transpose float32 [65536, 33024]', gather_transpose(a, flat, alpha=0.5, stride=7919), \
        gathered_and_transposed


def operators_to_build():
    for _name, out, _ref in cases(placeholder):
        yield (out if hasattr(out, 'parent') else out[0]).parent.expression_dag
