"""GPU behaviour of the runtime and the launcher boundary: tensor kinds, timing, poisoning, error reporting."""
import ctypes

import numpy as np
import pytest

import opveclib_amd as ovl
import oracle
from opveclib_amd import runtime, launcher, stdops
from opveclib_amd.examples import shift_cyclic, expm1
from tests import cases

pytestmark = pytest.mark.gpu


def test_numpy_in_numpy_out_and_torch_in_torch_out():
    import torch
    rng = np.random.default_rng(0)
    a = rng.standard_normal((16, 64), dtype=np.float32)
    b = rng.standard_normal((16, 64), dtype=np.float32)
    out = ovl.evaluate(stdops.add(a, b))
    assert isinstance(out, np.ndarray) and np.array_equal(out, a + b)
    ta, tb = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    tout = ovl.evaluate(stdops.add(ta, tb))
    assert isinstance(tout, torch.Tensor) and tout.is_cuda
    assert np.array_equal(tout.cpu().numpy(), a + b)
    mixed = ovl.evaluate(stdops.add(ta, b))
    assert isinstance(mixed, torch.Tensor)
    # several outputs come back as a list in request order
    s, d = ovl.evaluate([stdops.add(a, b), stdops.sub(a, b)])
    assert np.array_equal(s, a + b) and np.array_equal(d, a - b)


def test_views_and_non_contiguous_inputs():
    import torch
    base = torch.arange(4 * 70, dtype=torch.float32, device='cuda').reshape(4, 70)
    shifted = base[:, 1:65]                 # non-contiguous rows
    offset = base.reshape(-1)[1:257]        # contiguous but not 16-byte aligned
    assert offset.data_ptr() % 16 != 0
    out = ovl.evaluate(stdops.add(shifted, shifted))
    assert torch.equal(out, shifted + shifted)
    out = ovl.evaluate(stdops.add(offset, offset))
    assert torch.equal(out, offset + offset)


def test_profile_returns_times_per_operator():
    a = np.random.default_rng(1).standard_normal(1 << 14).astype(np.float32)
    outs, times = ovl.profile(expm1(shift_cyclic(a)), 'hip', 4, 0)
    assert len(outs) == 1 and len(times) == 2           # unfused: one kernel per operator
    for name, ms in times.items():
        assert name.startswith('f') and ms.shape == (4,) and ms.dtype == np.float64
        assert np.all(ms > 0) and np.all(ms < 100)
    ref = oracle.evaluate(expm1(shift_cyclic(a)))
    assert np.array_equal(outs[0], ref)
    _, fused_times = ovl.profile(stdops.mul(stdops.add(a, a), a), 'hip', 1, 3)
    assert len(fused_times) == 1
    _, unfused_times = ovl.profile(stdops.mul(stdops.add(a, a), a), 'hip', 1, 0)
    assert len(unfused_times) == 2          # times are keyed by operator hash: two distinct operators


def test_poison_marks_unwritten_elements():
    import torch

    @ovl.operator()
    def write_evens(x):
        out = ovl.output_like(x)
        pos = ovl.position_in(x.shape)
        with ovl.if_(pos[0] % 2 == 0):
            out[pos] = x[pos]
        return out

    runtime.poison_outputs = True
    try:
        x = torch.ones(64, dtype=torch.float32, device='cuda')
        out = ovl.evaluate(write_evens(x)).cpu().numpy()
    finally:
        runtime.poison_outputs = False
    assert np.all(out[0::2] == 1.0)
    assert np.all(out[1::2].view(np.uint32) == 0xFEFEFEFE)


def test_launcher_reports_argument_errors_on_device():
    import torch
    a = torch.zeros(256, dtype=torch.float32, device='cuda')
    compiled = runtime.load_operator(stdops.add(a, a).expression_dag)
    stream = torch.cuda.current_stream().cuda_stream
    out = torch.empty(256, dtype=torch.float32, device='cuda')
    wrong = torch.zeros(256, dtype=torch.float64, device='cuda')
    with pytest.raises(TypeError):
        compiled.check_inputs([a, wrong])
    params_in = launcher.tensor_array([(a.data_ptr(), 2, 256), (wrong.data_ptr(), 3, 256)])
    params_out = launcher.tensor_array([(out.data_ptr(), 2, 256)])
    with pytest.raises(launcher.LauncherError) as err:
        compiled.lib.launch(params_in, 2, params_out, 1, stream)
    assert err.value.code == launcher.OVL_EARGS
    # ovl_launch by symbol name gives the same result as the resolved entry point
    good_in = launcher.tensor_array([(a.data_ptr(), 2, 256), (a.data_ptr(), 2, 256)])
    L = launcher.library()
    assert L.ovl_launch(compiled.lib.handle, compiled.gen.entry.encode(), good_in, 2, params_out, 1, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, a + a)
    times = (ctypes.c_double * 3)()
    assert L.ovl_time(compiled.lib.fn, good_in, 2, params_out, 1, stream, 3, times) == 0
    assert all(t > 0 for t in times)


def test_launch_is_asynchronous_on_the_callers_stream():
    import torch
    side = torch.cuda.Stream()
    a = torch.full((1 << 20,), 2.0, dtype=torch.float32, device='cuda')
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        out = ovl.evaluate(stdops.mul(stdops.add(a, a), a))
    side.synchronize()
    assert torch.all(out == 8.0)


def test_hand_written_library_through_the_c_abi():
    """A library written by hand against include/ovl_launch.h (the reference's addgpu.cu test, restated): open it,
    resolve its entry point and launch it with the launcher; wrong argument lists come back as error code 1."""
    import os
    import torch
    from opveclib_amd import launcher
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'native', 'libhand_written_add.so')
    if not os.path.exists(path):
        from tests.native import build
        build.build()
    op = launcher.OperatorLibrary(path, 'hand_written_add_generic_hip')
    stream = torch.cuda.current_stream().cuda_stream
    for dtype, code in ((torch.float32, 2), (torch.float64, 3)):
        a = torch.randn(100003, device='cuda', dtype=dtype)
        b = torch.randn(100003, device='cuda', dtype=dtype)
        total, diff = torch.empty_like(a), torch.empty_like(a)
        ins = launcher.tensor_array([(a.data_ptr(), code, a.numel()), (b.data_ptr(), code, b.numel())])
        outs = launcher.tensor_array([(total.data_ptr(), code, a.numel()), (diff.data_ptr(), code, a.numel())])
        op.launch(ins, 2, outs, 2, stream)
        torch.cuda.synchronize()
        assert torch.equal(total, a + b) and torch.equal(diff, a - b)
        op.launch(ins, 2, outs, 1, stream)                      # the second output is optional
        times = op.time(ins, 2, outs, 1, stream, 3)
        assert len(times) == 3 and all(t > 0 for t in times)
    with pytest.raises(launcher.LauncherError) as err:
        op.launch(ins, 1, outs, 1, stream)                      # one input only
    assert err.value.code == 1
    mixed = launcher.tensor_array([(a.data_ptr(), 3, a.numel()), (b.data_ptr(), 2, b.numel())])
    with pytest.raises(launcher.LauncherError):
        op.launch(mixed, 2, outs, 1, stream)                    # dtypes disagree
    with pytest.raises(launcher.LauncherError) as err:
        launcher.OperatorLibrary(path, 'no_such_entry_point')
    assert err.value.code == 3


def test_concurrent_evaluation_from_several_threads_and_streams():
    """Four Python threads trace, load and launch different operator DAGs at the same time, each on a HIP stream of
    its own (default priority), ten rounds each: every result equals the oracle's (computed beforehand on the CPU)."""
    import threading
    import torch
    import oracle
    from tests import cases
    names = ['c2_chain', 'c4_lstm_grad', 'c5_variants', 'c1_shift_expm1_log1p']
    expected = {}
    for name in names:
        expected[name] = oracle.profile(cases.CASE_BY_NAME[name].outputs(), 1, 0)[0]
    large = dict((name, np.random.default_rng(k).standard_normal((3 << 20) + k).astype(np.float32))
                 for k, name in enumerate(names))
    failures = []
    start = threading.Barrier(len(names))

    def worker(name):
        try:
            case = cases.CASE_BY_NAME[name]
            stream = torch.cuda.Stream()
            start.wait(timeout=60)
            for _ in range(10):
                with torch.cuda.stream(stream):
                    got = ovl.evaluate(case.outputs(), opt_level=3)
                got = got if isinstance(got, list) else [got]
                for n, (g, r) in enumerate(zip(got, expected[name])):
                    cases.assert_matches(case, g, r, '%s output %d' % (name, n))
                # host arrays large enough for the page-locked staging buffers, which the threads share
                with torch.cuda.stream(stream):
                    big = ovl.evaluate(stdops.add(large[name], large[name]))
                assert np.array_equal(big, large[name] + large[name]), name + ': staged transfer'
        except Exception as exception:      # reported by the main thread
            failures.append((name, repr(exception)))

    threads = [threading.Thread(target=worker, args=(name,)) for name in names]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not any(t.is_alive() for t in threads)
    assert failures == []


def test_staged_host_transfers_round_trip():
    """Arrays below, at and above the staging threshold and the staging buffer size, five element types, two
    transfers back to back: what comes back equals what went in, and the device tensor equals PyTorch's own copy."""
    import torch
    from opveclib_amd import transfer
    device = torch.device('cuda', torch.cuda.current_device())
    rng = np.random.default_rng(1)
    chunk, least = transfer.CHUNK_BYTES, transfer.MIN_STAGED_BYTES
    for dtype in (np.float32, np.uint8, np.float64, np.uint16, np.int64):
        for nbytes in (1, least - 8, least, least + 8, chunk + 24, 2 * chunk, 3 * chunk + 8):
            n = max(1, nbytes // np.dtype(dtype).itemsize)
            x = rng.integers(0, 250, n).astype(dtype)
            t = transfer.to_device(x, torch, device)
            assert tuple(t.shape) == x.shape and torch.equal(t.cpu(), torch.from_numpy(x))
            back = transfer.to_host(t, torch)
            assert back.dtype == x.dtype and back.shape == x.shape and np.array_equal(back, x)
            y = x[:(n // 3) * 3].reshape(-1, 3) if n >= 3 else x.reshape(1, -1)
            assert np.array_equal(transfer.to_host(transfer.to_device(y, torch, device), torch), y)


def test_evaluate_on_large_host_arrays_uses_the_staged_path_and_matches_torch():
    import torch
    rng = np.random.default_rng(2)
    a = rng.standard_normal((4096, 4096)).astype(np.float32)      # 64 MiB each
    b = rng.standard_normal((4096, 4096)).astype(np.float32)
    got = ovl.evaluate(stdops.mul(stdops.add(a, b), a))
    assert isinstance(got, np.ndarray) and np.array_equal(got, (a + b) * a)
