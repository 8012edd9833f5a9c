"""
`ovl.as_torch`: OVL operator graphs inside torch.autograd on the GPU.  Forward values and gradients are compared with
the same functions written in torch operations (the reference's gradient tests, restated against torch instead of
TensorFlow), fused and unfused evaluation must agree bit for bit, and leaves without a gradient path get None.
"""
import numpy as np
import pytest

import opveclib_amd as ovl
from tests import autograd_cases as ac

pytestmark = pytest.mark.gpu


def _run(case, opt_level):
    import torch
    leaves = case.leaves()
    rng = np.random.default_rng(12)

    def tensors():
        out = []
        for n, leaf in enumerate(leaves):
            t = torch.from_numpy(leaf).cuda()
            t.requires_grad_(n in case.differentiable)
            out.append(t)
        return out

    ovl_leaves = tensors()
    ovl_outs = ovl.as_torch(case.graph(*ovl_leaves), opt_level=opt_level)
    ovl_outs = ovl_outs if isinstance(ovl_outs, list) else [ovl_outs]
    ref_leaves = tensors()
    ref_outs = case.torch_graph(torch, *ref_leaves)
    assert len(ovl_outs) == len(ref_outs)
    grads_above = [torch.from_numpy(rng.random(tuple(o.shape)).astype(leaves[0].dtype)).cuda() for o in ref_outs]
    wanted = [n for n in range(len(leaves)) if n in case.differentiable]
    ovl_grads = torch.autograd.grad(ovl_outs, [ovl_leaves[n] for n in wanted], grads_above, allow_unused=True)
    ref_grads = torch.autograd.grad(ref_outs, [ref_leaves[n] for n in wanted], grads_above, allow_unused=True)
    return ovl_outs, ref_outs, ovl_grads, ref_grads


def _close(case, got, ref, what):
    import torch
    assert got.dtype == ref.dtype and got.shape == ref.shape, what
    if case.exact:
        assert torch.equal(got, ref), '%s %s: not bit-equal' % (case.name, what)
    else:
        scale = float(ref.abs().max()) or 1.0
        err = float((got.double() - ref.double()).abs().max())
        assert err <= case.rtol * scale, '%s %s: error %g > %g' % (case.name, what, err, case.rtol * scale)


@pytest.mark.parametrize('case', ac.CASES, ids=[c.name for c in ac.CASES])
def test_values_and_gradients_match_torch(case):
    import torch
    fused = _run(case, 3)
    for n, (got, ref) in enumerate(zip(fused[0], fused[1])):
        _close(case, got.detach(), ref.detach(), 'output %d' % n)
    for n, (got, ref) in enumerate(zip(fused[2], fused[3])):
        assert (got is None) == (ref is None)
        if got is not None:
            _close(case, got, ref, 'gradient %d' % n)
    # the optimizer changes nothing: unfused forward and backward give the same bits
    unfused = _run(case, 0)
    for got, ref in zip(fused[0] + list(fused[2]), unfused[0] + list(unfused[2])):
        if got is not None:
            assert torch.equal(got.detach(), ref.detach()), case.name + ': fused and unfused results differ'


def test_leaf_behind_an_operator_without_gradient():
    """Asking for the gradient raises; not asking for it (the leaf does not require grad) works."""
    import torch
    case = ac.NO_GRADIENT
    a, b = (torch.from_numpy(x).cuda().requires_grad_(True) for x in case.leaves())
    y = ovl.as_torch(case.graph(a, b))
    with pytest.raises(ValueError, match='no_gradient_scale'):
        torch.autograd.grad(y, [a, b], torch.ones_like(y), allow_unused=True)
    a = a.detach()
    y = ovl.as_torch(case.graph(a, b))
    gb, = torch.autograd.grad(y, [b], torch.ones_like(y))
    assert torch.equal(gb, 2 * a)


def test_backward_through_surrounding_torch_graph_and_numpy_constants():
    import torch
    rng = np.random.default_rng(3)
    x = torch.from_numpy(rng.random((16, 32))).cuda().requires_grad_(True)
    w = rng.random((16, 32))                                    # numpy leaf: a constant
    y = ovl.as_torch(ovl.stdops.mul(ovl.stdops.tanh(x * 2.0), w))
    loss = (y * y).sum()
    loss.backward()
    xr = x.detach().clone().requires_grad_(True)
    yr = torch.tanh(xr * 2.0) * torch.from_numpy(w).cuda()
    (yr * yr).sum().backward()
    assert torch.allclose(x.grad, xr.grad, rtol=1e-12, atol=1e-14)
    # nothing requires grad: plain evaluation, no graph
    z = ovl.as_torch(ovl.stdops.tanh(x.detach()))
    assert not z.requires_grad


def test_multi_output_with_one_output_unused():
    import torch
    a = torch.linspace(0, 1, 12, dtype=torch.float64).cuda().requires_grad_(True)
    b = torch.linspace(1, 2, 12, dtype=torch.float64).cuda().requires_grad_(True)
    y0, y1, y2 = ovl.as_torch(ac.fan_out(a, b))
    y1.sum().backward()                                          # y0 and y2 receive no gradient
    assert torch.equal(a.grad, torch.zeros_like(a))
    assert torch.equal(b.grad, torch.full_like(b, 3.0))
