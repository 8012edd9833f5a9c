"""
Operator DAGs recorded into a HIP graph: every replay, with the program's own eager work and synchronisations in
between and with changed inputs, must produce what the eager launches produce.
"""
import numpy as np
import pytest
import torch

import opveclib_amd as ovl
from opveclib_amd import stdops
from tests import cases

pytestmark = pytest.mark.gpu


_unfused_dag = cases.graph_capture_dag


@pytest.mark.parametrize('opt_level', [0, 3])
def test_replays_equal_eager_evaluation(opt_level):
    rng = np.random.default_rng(60 + opt_level)
    x = torch.from_numpy(rng.uniform(-0.5, 0.5, (48, 256)).astype(np.float32)).cuda()
    y = torch.from_numpy(rng.uniform(-0.5, 0.5, (48, 256)).astype(np.float32)).cuda()
    captured = ovl.CapturedDag(_unfused_dag(x, y), opt_level=opt_level)
    assert len(captured.kernels) >= 3
    assert captured.inputs[0].data_ptr() in (x.data_ptr(), y.data_ptr())
    for round_number in range(5):
        eager = [t.clone() for t in ovl.evaluate(_unfused_dag(x, y), opt_level=opt_level)]
        torch.cuda.synchronize()
        for t in captured.outputs:
            t.fill_(float('nan'))                                   # eager work between the replays
        got = captured.replay()
        torch.cuda.synchronize()
        for g, e in zip(got, eager):
            assert torch.equal(g, e), 'replay %d differs from the eager result' % round_number
        # new data for the next round, written into the graph's input buffers
        x.copy_(torch.from_numpy(rng.uniform(-0.5, 0.5, (48, 256)).astype(np.float32)))
        y.mul_(0.9)
    again = [t.clone() for t in captured.launch_eagerly()]
    assert all(torch.equal(a, b) for a, b in zip(again, captured.replay()))


def test_fast_mode_and_single_kernel_dag():
    x = torch.linspace(-3, 3, 4096, device='cuda')
    captured = ovl.CapturedDag(cases.graph_capture_single(x), math_mode='fast')
    assert len(captured.kernels) == 1
    eager = ovl.evaluate(cases.graph_capture_single(x), math_mode='fast')
    assert torch.equal(captured.replay()[0], eager)


def test_capture_rejects_inputs_that_are_not_static_device_buffers():
    x = torch.zeros(8, 64, device='cuda')
    with pytest.raises(TypeError):
        ovl.CapturedDag(stdops.add(x, np.zeros((8, 64), np.float32)))
    with pytest.raises(TypeError):
        ovl.CapturedDag(stdops.add(x.t()[:32].t(), x.t()[:32].t()))     # not contiguous
    with pytest.raises(ValueError):
        ovl.CapturedDag(stdops.add(x, x), math_mode='sloppy')
