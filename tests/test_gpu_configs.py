"""
The five benchmark configurations at their full sizes on the GPU.  The oracle is too slow for whole tensors of this
size, so each test combines an oracle comparison on a slice (all five operators act independently on rows or
elements, so the oracle on a row slice equals the slice of the full result) with a size-independent property that
covers every element.
"""
import numpy as np
import pytest

import opveclib_amd as ovl
import oracle
from opveclib_amd import stdops
from opveclib_amd.examples import shift_cyclic, expm1, log1p, cumsum, cumprod, gather_transpose
from opveclib_amd.lstm import lstm, lstm_grad
from tests import cases

pytestmark = pytest.mark.gpu


def test_c1_shift_expm1_log1p_full():
    import torch
    x = cases.uniform(np.random.default_rng(0), -0.9, 0.9, 1 << 20)
    shifted = ovl.evaluate(shift_cyclic(x))
    assert np.array_equal(shifted, np.roll(x, 1))                       # closed form, bit-exact
    got = ovl.evaluate(log1p(expm1(shift_cyclic(x))))
    ref = oracle.evaluate(log1p(expm1(shift_cyclic(x))))
    assert np.array_equal(got, ref)                                     # composite, bit-exact
    assert np.allclose(got, np.roll(x, 1), rtol=0, atol=2e-6)           # log1p(expm1(x)) == x up to rounding


def test_c2_chain_full():
    import torch
    rng = np.random.default_rng(2)
    a = cases.uniform(rng, -1, 1, (8192, 8192))
    b = cases.uniform(rng, -1, 1, (8192, 8192))
    s = np.array([1.0001], np.float32)
    ta, tb, ts = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(s).cuda()
    y = ovl.evaluate(cases.chain8(ta, tb, ts)[-1])
    assert y.shape == (8192, 8192) and y.dtype == torch.float32
    rows = np.r_[0:24, 4095:4105, 8180:8192]
    ref = oracle.evaluate(cases.chain8(np.ascontiguousarray(a[rows]), np.ascontiguousarray(b[rows]), s)[-1])
    assert np.array_equal(y[torch.from_numpy(rows).cuda()].cpu().numpy(), ref)
    # every element: finite, non-negative, and equal to |sigmoid(tanh((a+b)*s)) - b| up to float32 rounding
    assert bool(torch.isfinite(y).all()) and bool((y >= 0).all())
    approx = (torch.sigmoid(torch.tanh((ta.double() + tb.double()) * float(s[0]))) - tb.double()).abs()
    assert float((y.double() - approx).abs().max()) < 1e-6
    # fusing changes nothing: the unfused evaluation of a column block is bitwise identical
    blk = slice(0, 512)
    unfused = ovl.evaluate(cases.chain8(ta[blk].contiguous(), tb[blk].contiguous(), ts)[-1], opt_level=0)
    assert torch.equal(unfused, y[blk])


@pytest.mark.parametrize('dtype, rows', [(np.float32, 4096), (np.float64, 1024)])
def test_c3_accumulate_full(dtype, rows):
    import torch
    rng = np.random.default_rng(3)
    x = rng.standard_normal((rows, 16384), dtype=dtype)
    p = cases.uniform(rng, 0.99, 1.01, (rows, 16384), dtype)
    tx, tp = torch.from_numpy(x).cuda(), torch.from_numpy(p).cuda()
    cs = ovl.evaluate(cumsum(tx, axis=1)).cpu().numpy()
    cp = ovl.evaluate(cumprod(tp, axis=1)).cpu().numpy()
    # numpy's accumulate is the same strictly sequential recurrence in the same dtype: bit-exact on every element
    assert np.array_equal(cs, np.cumsum(x, axis=1, dtype=dtype))
    assert np.array_equal(cp, np.cumprod(p, axis=1, dtype=dtype))
    sample = np.r_[0:3, rows - 2:rows]
    assert np.array_equal(cs[sample], oracle.evaluate(cumsum(np.ascontiguousarray(x[sample]), axis=1)))


def test_c4_lstm_full():
    import torch
    rng = np.random.default_rng(4)
    concat = rng.standard_normal((4096, 4096), dtype=np.float32)
    c = rng.standard_normal((4096, 1024), dtype=np.float32)
    dc = rng.standard_normal((4096, 1024), dtype=np.float32)
    dh = rng.standard_normal((4096, 1024), dtype=np.float32)
    t = [torch.from_numpy(v).cuda() for v in (concat, c, dc, dh)]
    new_c, new_h = ovl.evaluate(cases.all_outputs(lstm(t[0], t[1], forget_bias=1.0)))
    d_concat, d_c = ovl.evaluate(cases.all_outputs(lstm_grad(t[0], t[1], t[2], t[3], forget_bias=1.0)))
    rows = np.r_[0:8, 2048:2052, 4092:4096]
    sl = [np.ascontiguousarray(v[rows]) for v in (concat, c, dc, dh)]
    ref_c, ref_h = oracle.evaluate(cases.all_outputs(lstm(sl[0], sl[1], forget_bias=1.0)))
    ref_dx, ref_dc = oracle.evaluate(cases.all_outputs(lstm_grad(sl[0], sl[1], sl[2], sl[3], forget_bias=1.0)))
    idx = torch.from_numpy(rows).cuda()
    assert np.array_equal(new_c[idx].cpu().numpy(), ref_c)
    assert np.array_equal(new_h[idx].cpu().numpy(), ref_h)
    assert np.array_equal(d_concat[idx].cpu().numpy(), ref_dx)
    assert np.array_equal(d_c[idx].cpu().numpy(), ref_dc)
    # every element: the gradient agrees with autograd of the float64 closed form
    tc = t[0].double().requires_grad_(True)
    tcp = t[1].double().requires_grad_(True)
    i, j, f, o = torch.split(tc, 1024, dim=1)
    cc = tcp * torch.sigmoid(f + 1.0) + torch.sigmoid(i) * torch.tanh(j)
    hh = torch.tanh(cc) * torch.sigmoid(o)
    assert float((new_c.double() - cc.detach()).abs().max()) < 1e-5
    assert float((new_h.double() - hh.detach()).abs().max()) < 1e-5
    ((cc * t[2].double()).sum() + (hh * t[3].double()).sum()).backward()
    assert float((d_concat.double() - tc.grad).abs().max()) < 1e-4
    assert float((d_c.double() - tcp.grad).abs().max()) < 1e-4


def test_c5_gather_transpose_full():
    import torch
    n = 16384
    g = np.random.default_rng(5)                # inputs drawn on the host and copied once, as for the other configurations
    a = torch.from_numpy(g.standard_normal((n, n), dtype=np.float32)).cuda()
    b = torch.from_numpy(g.standard_normal(n * n, dtype=np.float32)).cuda()
    out = ovl.evaluate(gather_transpose(a, b, alpha=0.5, stride=7919))
    assert out.shape == (n, n)
    # every element, in row blocks to bound memory: out[j, i] == 0.5*a[i, j] + b[i*7919 + j] in float32
    j = torch.arange(n, device='cuda', dtype=torch.int64)
    for start in range(0, n, 2048):
        i = torch.arange(start, start + 2048, device='cuda', dtype=torch.int64)
        idx = (i[:, None] * 7919 + j[None, :]) % (n * n)
        expect = a[start:start + 2048] * 0.5 + b[idx]
        assert torch.equal(out[:, start:start + 2048].t(), expect)
    rows = 64
    small = oracle.evaluate(gather_transpose(a[:rows].cpu().numpy(), b[:rows * n].cpu().numpy(), alpha=0.5, stride=7919))
    small_gpu = ovl.evaluate(gather_transpose(a[:rows].contiguous(), b[:rows * n].contiguous(), alpha=0.5,
                                              stride=7919))
    assert np.array_equal(small_gpu.cpu().numpy(), small)


def test_reference_timing_cumsum_float64_along_axis_0():
    """The shape the reference times (opveclib/examples/test_perf_accumulate.py:35-47): float64 [10000, 1000] along
    axis 0, against numpy's sequential accumulate and against the oracle, every element."""
    from opveclib_amd import workloads
    x = np.random.default_rng(6).standard_normal(workloads.REFERENCE_CUMSUM_SHAPE)
    got = ovl.evaluate(cumsum(x, axis=0))
    assert np.array_equal(got, np.cumsum(x, axis=0))
    assert np.array_equal(got, oracle.evaluate(cumsum(x, axis=0)))


@pytest.mark.parametrize('units', [200, 650, 1500])
def test_reference_timing_lstm_cell_batch_20(units):
    """The cell sizes the reference's profiler runs (lstm/profile_lstm.py:41-51): batch 20 with 200, 650 and 1500
    units, forward and gradient, generated operators and hand-written run-time-shape kernels (650 units are not a
    multiple of the vector width: the scalar kernels) against the oracle, bit for bit."""
    import torch
    from opveclib_amd import lstm_cell, workloads
    batch = workloads.REFERENCE_LSTM_BATCH
    g = np.random.default_rng(6 + units)
    concat = g.standard_normal((batch, 4 * units), dtype=np.float32)
    c, dc, dh = (g.standard_normal((batch, units), dtype=np.float32) for _ in range(3))
    want_fwd = oracle.evaluate(cases.all_outputs(lstm(concat, c, forget_bias=1.0)))
    want_grad = oracle.evaluate(cases.all_outputs(lstm_grad(concat, c, dc, dh, forget_bias=1.0)))
    got_fwd = ovl.evaluate(cases.all_outputs(lstm(concat, c, forget_bias=1.0)))
    got_grad = ovl.evaluate(cases.all_outputs(lstm_grad(concat, c, dc, dh, forget_bias=1.0)))
    t = [torch.from_numpy(v).cuda() for v in (concat, c, dc, dh)]
    hand_fwd = lstm_cell.lstm_cell(t[0], t[1], 1.0)
    hand_grad = lstm_cell.lstm_cell_grad(t[0], t[1], t[2], t[3], 1.0)
    for got, hand, want in zip(list(got_fwd) + list(got_grad), list(hand_fwd) + list(hand_grad),
                               list(want_fwd) + list(want_grad)):
        assert np.array_equal(got, want)
        assert np.array_equal(hand.cpu().numpy(), want)
