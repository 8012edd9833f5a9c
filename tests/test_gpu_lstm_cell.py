"""
The hand-written LSTM cell kernels (include/ovl_lstm.h) on the GPU: same bits as the CPU oracle of the reference's
fused LSTM operator (lstm/lstm.py:32-105) and as the generated operator, for shapes that take the 128-bit path, the
scalar path (units not a multiple of 4, unaligned views) and the benchmark's full size.
"""
import numpy as np
import pytest
import torch

import opveclib_amd as ovl
import oracle
from opveclib_amd import lstm_cell
from opveclib_amd.lstm import lstm, lstm_grad
from tests import cases

pytestmark = pytest.mark.gpu


def _inputs(rng, batch, units, special=False):
    make = cases.special_values if special else (lambda r, shape: r.standard_normal(shape, dtype=np.float32))
    return (make(rng, (batch, 4 * units)), make(rng, (batch, units)),
            rng.standard_normal((batch, units), dtype=np.float32), rng.standard_normal((batch, units), dtype=np.float32))


def _same(got, ref):
    got = got.cpu().numpy()
    assert got.dtype == ref.dtype and got.shape == ref.shape
    equal = ((got == ref) & (np.signbit(got) == np.signbit(ref))) | (np.isnan(got) & np.isnan(ref))
    assert equal.all(), '%d of %d elements differ' % (int((~equal).sum()), equal.size)


@pytest.mark.parametrize('batch,units,special', [(32, 128, False), (7, 52, False), (5, 13, False), (3, 1, False),
                                                 (16, 64, True), (9, 7, True)])
def test_hand_written_cell_equals_the_oracle(batch, units, special):
    rng = np.random.default_rng(40 + units)
    concat, c, d_c, d_h = _inputs(rng, batch, units, special)
    for forget_bias in (1.0, 0.0, -0.37):
        ref_fwd = oracle.profile(cases.all_outputs(lstm(concat, c, forget_bias=forget_bias)), 1, 0)[0]
        ref_bwd = oracle.profile(lstm_grad(concat, c, d_c, d_h, forget_bias=forget_bias), 1, 0)[0]
        dev = [torch.from_numpy(x).cuda() for x in (concat, c, d_c, d_h)]
        new_c, new_h = lstm_cell.lstm_cell(dev[0], dev[1], forget_bias)
        _same(new_c, ref_fwd[0])
        _same(new_h, ref_fwd[1])
        d_concat, d_cell = lstm_cell.lstm_cell_grad(dev[0], dev[1], dev[2], dev[3], forget_bias)
        _same(d_concat, ref_bwd[0])
        _same(d_cell, ref_bwd[1])


def test_unaligned_views_take_the_scalar_path():
    rng = np.random.default_rng(41)
    concat, c, d_c, d_h = _inputs(rng, 6, 16)
    ref = oracle.profile(cases.all_outputs(lstm(concat, c, forget_bias=1.0)), 1, 0)[0]
    # a tensor that starts 4 bytes into an allocation: contiguous but not 16-byte aligned
    backing = torch.zeros(concat.size + 1, device='cuda')
    view = backing[1:].view(concat.shape)
    view.copy_(torch.from_numpy(concat))
    assert view.data_ptr() % 16 != 0
    new_c, new_h = lstm_cell.lstm_cell(view, torch.from_numpy(c).cuda(), 1.0)
    _same(new_c, ref[0])
    _same(new_h, ref[1])


def test_full_size_equals_the_generated_operator_in_both_math_modes():
    rng = np.random.default_rng(4)
    batch, units = 4096, 1024
    concat, c, d_c, d_h = [torch.from_numpy(x).cuda() for x in _inputs(rng, batch, units)]
    for mode in ('exact', 'fast'):
        gen_c, gen_h = ovl.evaluate(cases.all_outputs(lstm(concat, c, forget_bias=1.0)), math_mode=mode)
        new_c, new_h = lstm_cell.lstm_cell(concat, c, 1.0, math_mode=mode)
        assert torch.equal(new_c, gen_c) and torch.equal(new_h, gen_h)
        gen_dconcat, gen_dc = ovl.evaluate(lstm_grad(concat, c, d_c, d_h, forget_bias=1.0), math_mode=mode)
        d_concat, d_cell = lstm_cell.lstm_cell_grad(concat, c, d_c, d_h, 1.0, math_mode=mode)
        assert torch.equal(d_concat, gen_dconcat) and torch.equal(d_cell, gen_dc)


def test_autograd_through_the_hand_written_cell():
    rng = np.random.default_rng(42)
    concat_np, c_np, d_c, d_h = _inputs(rng, 8, 24)
    concat = torch.from_numpy(concat_np).cuda().requires_grad_()
    c = torch.from_numpy(c_np).cuda().requires_grad_()
    new_c, new_h = lstm_cell.lstm_cell_torch(concat, c, 1.0)
    w_c, w_h = torch.from_numpy(d_c).cuda(), torch.from_numpy(d_h).cuda()
    ((new_c * w_c).sum() + (new_h * w_h).sum()).backward()
    ref = lstm_cell.lstm_cell_grad(concat.detach(), c.detach(), w_c, w_h, 1.0)
    assert torch.equal(concat.grad, ref[0]) and torch.equal(c.grad, ref[1])
    # against PyTorch's own differentiation of the same formula in float64
    x = torch.from_numpy(concat_np).double().requires_grad_()
    cc = torch.from_numpy(c_np).double().requires_grad_()
    i, j, f, o = x.chunk(4, dim=1)
    nc = cc * torch.sigmoid(f + 1.0) + torch.sigmoid(i) * torch.tanh(j)
    nh = torch.tanh(nc) * torch.sigmoid(o)
    ((nc * torch.from_numpy(d_c).double()).sum() + (nh * torch.from_numpy(d_h).double()).sum()).backward()
    assert np.allclose(concat.grad.cpu().numpy(), x.grad.numpy(), rtol=2e-5, atol=2e-6)
    assert np.allclose(c.grad.cpu().numpy(), cc.grad.numpy(), rtol=2e-5, atol=2e-6)
