"""
Operator DAGs the fusion optimizer must leave alone, evaluated on the CPU oracle unfused (the operators as written)
and fused (through the product's optimizer): the results must be equal.
"""
import numpy as np

import opveclib_amd as ovl
import oracle
from opveclib_amd import workloads


@ovl.operator()
def scatter_by(x, idx):
    """out[idx[p]] = x[p]"""
    out = ovl.output_like(x)
    pos = ovl.position_in(x.shape)
    out[ovl.cast(idx[pos], ovl.uint32)] = x[pos]
    return out


@ovl.operator()
def gather_by(t, idx):
    """out[p] = t[idx[p]]"""
    out = ovl.output_like(t)
    pos = ovl.position_in(t.shape)
    out[pos] = t[ovl.cast(idx[pos], ovl.uint32)]
    return out


def test_scatter_and_gather_through_different_index_tensors_are_not_merged():
    """Input numbers are local to an operator: both index tensors are 'input 1', of equal type, yet different
    tensors.  Merging on that would turn the gather into a read of the worker's own value."""
    n = 16
    x = np.arange(10, 10 + n).astype(np.float32)
    idx1 = np.roll(np.arange(n), 3).astype(np.int32)
    idx2 = np.roll(np.arange(n), -2).astype(np.int32)
    out = gather_by(scatter_by(x, idx1), idx2)
    assert len(workloads.fused_operators([out[0]])) == 2
    unfused = oracle.evaluate(out, opt_level=0)
    fused = oracle.evaluate(out, opt_level=3)
    expected = np.empty(n, np.float32)
    expected[idx1] = x
    expected = expected[idx2]
    assert np.array_equal(unfused, expected)
    assert np.array_equal(fused, expected)


def test_indices_read_from_one_tensor_are_not_merged_either():
    """With one index tensor the store need not be one-to-one: the element a consumer reads may have been written by
    another worker, which a merged kernel cannot see."""
    n = 16
    x = np.arange(n).astype(np.float32)
    idx = (np.arange(n) // 2 * 2).astype(np.int32)        # pairs of workers store to the same element
    out = gather_by(scatter_by(x, idx), idx)
    assert len(workloads.fused_operators([out[0]])) == 2
