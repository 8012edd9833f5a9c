"""
The largest sizes on the GPU (tests/large_cases.py): bit-equal to PyTorch's flip / add / roll / integer cumsum /
gather on the same device tensors, and the hand-written LSTM cell on 2^32 - 1 elements against itself on row blocks.
About 40 GiB of device memory for the generated operators, 115 GiB for the LSTM cell.
"""
import numpy as np
import pytest

import opveclib_amd as ovl
from tests import large_cases

pytestmark = pytest.mark.gpu


def _device_tensor(shape, dtype):
    import torch
    shape = shape if isinstance(shape, tuple) else (shape,)
    torch_dtype = getattr(torch, np.dtype(dtype).name)
    if np.dtype(dtype).kind in 'iu':
        info = np.iinfo(dtype)
        return torch.randint(max(info.min, -100), min(info.max, 100) + 1, shape, dtype=torch_dtype, device='cuda:0')
    return torch.randn(shape, dtype=torch_dtype, device='cuda:0')


def _need_free_device_memory(gib):
    import torch
    free, _total = torch.cuda.mem_get_info()
    if free < gib * 2 ** 30:
        pytest.skip('needs %d GiB of free device memory, %.0f GiB are free' % (gib, free / 2 ** 30))


def test_generated_operators_at_the_largest_sizes():
    import torch
    _need_free_device_memory(48)
    torch.manual_seed(11)
    names = []
    for name, out, reference in large_cases.cases(_device_tensor):
        print('large case:', name, flush=True)
        got = ovl.evaluate(out, opt_level=0)
        want = reference()
        assert got.dtype == want.dtype and got.shape == want.shape and torch.equal(got, want), name
        names.append(name)
        del got, want, out, reference
        torch.cuda.empty_cache()
    assert len(names) == 12


def test_hand_written_lstm_cell_on_2_to_32_minus_1_elements():
    """Three units per row: the scalar variant, whose index steps come within 2^28 of 2^32.  Rows are independent, so
    the result must equal the same function on blocks of rows (which stay far below that)."""
    import torch
    from opveclib_amd.lstm_cell import lstm_cell, lstm_cell_grad
    _need_free_device_memory(128)
    torch.manual_seed(12)
    batch, units, block = 1431655765, 3, 1 << 27
    assert batch * units == 2 ** 32 - 1
    concat = torch.randn((batch, 4 * units), dtype=torch.float32, device='cuda:0')
    c = torch.randn((batch, units), dtype=torch.float32, device='cuda:0')
    print('large case: lstm forward', flush=True)
    new_c, new_h = lstm_cell(concat, c, 1.0)
    for r0 in range(0, batch, block):
        r1 = min(batch, r0 + block)
        part_c, part_h = lstm_cell(concat[r0:r1], c[r0:r1], 1.0)
        assert torch.equal(part_c, new_c[r0:r1]) and torch.equal(part_h, new_h[r0:r1]), r0
        del part_c, part_h
    del new_c, new_h
    torch.cuda.empty_cache()
    d_new_c = torch.randn((batch, units), dtype=torch.float32, device='cuda:0')
    d_new_h = torch.randn((batch, units), dtype=torch.float32, device='cuda:0')
    print('large case: lstm gradient', flush=True)
    d_concat, d_c = lstm_cell_grad(concat, c, d_new_c, d_new_h, 1.0)
    for r0 in range(0, batch, block):
        r1 = min(batch, r0 + block)
        part_concat, part_c = lstm_cell_grad(concat[r0:r1], c[r0:r1], d_new_c[r0:r1], d_new_h[r0:r1], 1.0)
        assert torch.equal(part_concat, d_concat[r0:r1]) and torch.equal(part_c, d_c[r0:r1]), r0
        del part_concat, part_c
    del concat, c, d_new_c, d_new_h, d_concat, d_c
    torch.cuda.empty_cache()
