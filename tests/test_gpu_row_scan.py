"""
The hand-written row scans (include/ovl_scan.h) on the GPU: the same bits as numpy's strictly sequential
cumsum / cumprod (which is what the reference's accumulate operator computes, examples/test_accumulate.py:63-76), as
the CPU oracle and as the generated operator, on shapes that take the lane-skewed kernel with deep and shallow request
bursts, the one-lane-per-row kernel (ragged column counts, unaligned views) and the benchmark's full sizes.
"""
import numpy as np
import pytest
import torch

import opveclib_amd as ovl
import oracle
from opveclib_amd import row_scan
from opveclib_amd.examples import cumsum, cumprod

pytestmark = pytest.mark.gpu

SHAPES = [(48, 1024), (7, 256), (5, 64), (3, 192), (515, 64), (259, 128), (4, 70, 128), (5, 70), (7, 3), (1, 1),
          (2, 4096), (4096,), (6, 1536), (1027, 512), (3, 5, 2048),
          # rows whose number of 64-column groups is not a multiple of the request burst: 1, 2 and 3 groups over
          (9, 320), (70, 384), (33, 448), (130, 16448),
          # rows that are not whole groups, rows that do not start on 16-byte boundaries
          (50, 1000), (7, 333), (100, 16383), (3, 4, 131)]


def _data(rng, shape, dtype, kind):
    if kind == 'sum':
        return rng.standard_normal(shape).astype(dtype)
    return (0.9 + 0.2 * rng.random(shape)).astype(dtype)


@pytest.mark.parametrize('dtype', [np.float32, np.float64])
@pytest.mark.parametrize('shape', SHAPES, ids=[str(s) for s in SHAPES])
def test_equal_to_sequential_accumulation(shape, dtype):
    rng = np.random.default_rng(len(shape) * 100 + shape[-1])
    for kind, fn, ref_fn in (('sum', row_scan.cumsum, np.cumsum), ('product', row_scan.cumprod, np.cumprod)):
        x = _data(rng, shape, dtype, kind)
        got = fn(torch.from_numpy(x).cuda()).cpu().numpy()
        ref = ref_fn(x, axis=-1, dtype=dtype)           # numpy accumulates strictly left to right
        assert got.dtype == ref.dtype and got.shape == ref.shape
        assert np.array_equal(got, ref), '%s %s %s: %d elements differ' % (kind, shape, np.dtype(dtype).name,
                                                                           int((got != ref).sum()))


def test_equal_to_the_oracle_with_special_values():
    x = np.random.default_rng(5).standard_normal((6, 128)).astype(np.float32)
    x[1, 5] = np.inf
    x[2, 9] = np.nan
    x[3, 0] = -0.0
    x[4, 17] = 3.0e38
    x[4, 18] = 3.0e38
    for op, fn in ((cumsum, row_scan.cumsum), (cumprod, row_scan.cumprod)):
        ref = oracle.evaluate(op(x, axis=1))
        got = fn(torch.from_numpy(x).cuda()).cpu().numpy()
        assert np.array_equal(got, ref, equal_nan=True)
        assert np.array_equal(np.signbit(got[~np.isnan(ref)]), np.signbit(ref[~np.isnan(ref)]))


def test_unaligned_views_take_the_row_per_lane_kernel():
    x = np.random.default_rng(6).standard_normal((9, 64)).astype(np.float32)
    backing = torch.zeros(x.size + 1, device='cuda')
    view = backing[1:].view(x.shape)
    view.copy_(torch.from_numpy(x))
    assert view.data_ptr() % 16 != 0
    assert np.array_equal(row_scan.cumsum(view).cpu().numpy(), np.cumsum(x, axis=1, dtype=np.float32))


def test_full_sizes_equal_the_generated_operators():
    g = torch.Generator(device='cuda')
    g.manual_seed(3)
    xs = torch.randn((4096, 16384), device='cuda', generator=g)
    assert torch.equal(row_scan.cumsum(xs), ovl.evaluate(cumsum(xs, axis=1)))
    xp = 0.99 + 0.02 * torch.rand((4096, 16384), device='cuda', generator=g)
    assert torch.equal(row_scan.cumprod(xp), ovl.evaluate(cumprod(xp, axis=1)))
    xd = torch.randn((1024, 16384), device='cuda', generator=g, dtype=torch.float64)
    assert torch.equal(row_scan.cumsum(xd), ovl.evaluate(cumsum(xd, axis=1)))


REASSOCIATED_SHAPES = [(48, 1024), (7, 256), (3, 4100), (515, 64), (4, 70, 128), (2, 16384), (5, 70), (1, 4), (4096,)]


@pytest.mark.parametrize('dtype', [np.float32, np.float64])
@pytest.mark.parametrize('shape', REASSOCIATED_SHAPES, ids=[str(s) for s in REASSOCIATED_SHAPES])
def test_reassociated_scans_agree_with_the_sequential_ones_to_rounding(shape, dtype):
    """The tree-shaped wavefront scan: not the reference's bits, but the same numbers up to rounding.  Positive
    data, so that the relative error of the running values is meaningful."""
    rng = np.random.default_rng(7)
    eps = np.finfo(dtype).eps
    for kind, fn, ref_fn in (('sum', row_scan.cumsum, np.cumsum), ('product', row_scan.cumprod, np.cumprod)):
        x = (0.9 + 0.2 * rng.random(shape)).astype(dtype)
        got = fn(torch.from_numpy(x).cuda(), reassociate=True).cpu().numpy()
        ref = ref_fn(x.astype(np.float64), axis=-1)
        assert got.dtype == x.dtype and got.shape == x.shape
        assert np.array_equal(got[..., 0], x[..., 0])
        # a product of n factors carries up to n roundings whatever the order; sums of positive terms far fewer
        bound = eps * (shape[-1] if kind == 'product' else 8 * max(1.0, np.log2(shape[-1])))
        assert np.max(np.abs(got - ref) / np.abs(ref)) <= bound, kind


def test_reassociated_scans_at_full_size_and_their_distance_from_the_sequential_result():
    g = torch.Generator(device='cuda')
    g.manual_seed(3)
    xs = torch.randn((4096, 16384), device='cuda', generator=g)
    seq, tree = row_scan.cumsum(xs), row_scan.cumsum(xs, reassociate=True)
    # sums of N(0, 1) values wander through zero: compare on the scale of the running sum's spread
    assert float((seq - tree).abs().max()) <= 1e-5 * float(seq.abs().max())
    xd = torch.randn((1024, 16384), device='cuda', generator=g, dtype=torch.float64)
    seq, tree = row_scan.cumsum(xd), row_scan.cumsum(xd, reassociate=True)
    assert float((seq - tree).abs().max()) <= 1e-13 * float(seq.abs().max())
    xp = (0.99 + 0.02 * torch.rand((1024, 16384), device='cuda', generator=g, dtype=torch.float64))
    seq, tree = row_scan.cumprod(xp), row_scan.cumprod(xp, reassociate=True)
    assert float(((seq - tree) / seq).abs().max()) <= 1e-11


@pytest.mark.parametrize('lines', [4, 8, 16])
@pytest.mark.parametrize('shape', [(1000, 200), (517, 37), (3, 5), (2048, 64)], ids=str)
def test_strip_copy_measurement_aid_moves_exactly_the_tensor(shape, lines):
    """ovl_strip_copy_f64 (include/ovl_scan.h): mode 3 copies the tensor, mode 2 writes every element's row index,
    mode 1 writes nothing; nothing outside the tensor is touched (guard values either side)."""
    lib = row_scan.library()
    rows, cols = shape
    g = torch.Generator(device='cuda')
    g.manual_seed(11)
    x = torch.randn(shape, device='cuda', generator=g, dtype=torch.float64)
    guard = 64
    for mode in (3, 2, 1):
        buffer = torch.full((rows * cols + 2 * guard,), -7.0, device='cuda', dtype=torch.float64)
        out = buffer[guard:guard + rows * cols].view(rows, cols)
        status = lib.ovl_strip_copy_f64(x.data_ptr(), rows, cols, out.data_ptr(), lines, mode, None)
        assert status == 0, lib.ovl_scan_last_error()
        torch.cuda.synchronize()
        assert bool((buffer[:guard] == -7.0).all()) and bool((buffer[guard + rows * cols:] == -7.0).all())
        if mode == 3:
            assert torch.equal(out, x)
        elif mode == 2:
            want = torch.arange(rows, device='cuda', dtype=torch.float64)[:, None].expand(rows, cols)
            assert torch.equal(out, want)
        else:
            assert bool((out == -7.0).all())
