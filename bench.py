#!/usr/bin/env python
"""
Benchmark of the generated-operator hot path on one MI355X.

Headline workload ("chain8"): the fused element-wise chain of eight OVL operators
(add, mul by scalar 1.0001, tanh, sigmoid, log1p, expm1, sub, abs) over two float32 [8192, 8192] inputs drawn
uniformly from [-1, 1] (numpy default_rng(2)); the optimizer fuses the eight operators into one kernel.  One step is
one launch of the fused kernel on inputs that are already resident in HBM.  The metric is the achieved HBM bandwidth
in GB/s counted on algorithmic bytes (each input element read once, each output element written once:
3 * 2^26 * 4 + 4 bytes per launch).

Defaults: 100 untimed warm-up launches, then 100 timed ones.  The warm-up is that long on purpose: under this kernel's
vector ALU load the GPU's power management lets the first ten launches slow down by a third and needs about sixty
launches (25 ms) to settle (measured series: 310, 310, 310, 347, 377 ... 428 ... 340 ... 307, 307, 307 us), so a short
warm-up times the transient rather than the kernel.  For the same reason the headline kernel is first launched until
its time is stable (at least 40 ms of launches, reported as config.clock_settling_launches_before_warmup), whatever
--warmup says; so is every workload under `others`.

The JSON line also carries
  roofline      algorithmic bytes / average kernel duration (HIP events recorded around every launch on the launch
                stream) against the 8 TB/s HBM peak,
  cpu_baseline  the CPU oracle (the reference-shaped generated C++ compiled with the reference's flags) timed on this
                machine's host cores on a row slice of the same workload,
  others        time, bandwidth and roofline fraction of the remaining configurations (shift+expm1+log1p, cumsum,
                cumprod, LSTM cell forward and gradient, gather+transposed scatter).
"""

import argparse
import json
import os
import sys
import time

_ROOT = os.path.dirname(os.path.abspath(__file__))
if _ROOT not in sys.path:
    sys.path.insert(0, _ROOT)

import numpy as np

HBM_PEAK_GBPS = 8000.0

# HBM bytes per launch of the chain8 kernel from rocprofv3 counters (FETCH_SIZE 262207.5, WRITE_SIZE 262144.0, each
# scaled by the same counter's reading for the copy kernel of known size: factors 1.99986 and 0.99909).
# Source: profiles/bench_all_kernels_hbm_traffic_counters.md
CHAIN8_TRAFFIC_BYTES = 805152370


class Spec(object):
    """Shape and dtype of a tensor, enough to trace an operator without allocating the tensor."""

    def __init__(self, shape, dtype=np.float32):
        self.shape = list(shape)
        self.dtype = np.dtype(dtype).type


# ----------------------------------------------------------------------------------------------------------------------
# workloads
# ----------------------------------------------------------------------------------------------------------------------
def chain8_outputs(a, b, s):
    from tests.cases import chain8
    return [chain8(a, b, s)[-1][0]]


def copy_outputs(x):
    """out[pos] = x[pos]: the plain copy kernel that calibrates the profiler's byte counters."""
    import opveclib_amd as ovl

    @ovl.operator()
    def copy(arg):
        pos = ovl.position_in(arg.shape)
        out = ovl.output_like(arg)
        out[pos] = arg[pos]
        return out

    return [copy(x)[0]]


def c1_outputs(x):
    from opveclib_amd.examples import shift_cyclic, expm1, log1p
    return [log1p(expm1(shift_cyclic(x)))[0]]


def cumsum_outputs(x):
    from opveclib_amd.examples import cumsum
    return [cumsum(x, axis=1)[0]]


def cumprod_outputs(x):
    from opveclib_amd.examples import cumprod
    return [cumprod(x, axis=1)[0]]


def lstm_outputs(concat, c):
    from opveclib_amd.lstm import lstm
    op = lstm(concat, c, forget_bias=1.0)
    return [op[0], op[1]]


def lstm_grad_outputs(concat, c, dc, dh):
    from opveclib_amd.lstm import lstm_grad
    op = lstm_grad(concat, c, dc, dh, forget_bias=1.0)
    return [op[0], op[1]]


def gather_outputs(a, b_flat):
    from opveclib_amd.examples import gather_transpose
    return [gather_transpose(a, b_flat, alpha=0.5, stride=7919)[0]]


def all_workload_outputs():
    """Operator outputs of every benchmark workload at full size, built from shape specs (used to compile ahead)."""
    f32, f64 = np.float32, np.float64
    yield chain8_outputs(Spec((8192, 8192)), Spec((8192, 8192)), Spec((1,)))
    yield chain8_outputs(Spec((2048, 8192)), Spec((2048, 8192)), Spec((1,)))
    yield copy_outputs(Spec((8192, 8192)))
    yield c1_outputs(Spec((1 << 20,)))
    yield cumsum_outputs(Spec((4096, 16384), f32))
    yield cumprod_outputs(Spec((4096, 16384), f32))
    yield cumsum_outputs(Spec((1024, 16384), f64))
    yield cumprod_outputs(Spec((1024, 16384), f64))
    yield lstm_outputs(Spec((4096, 4096)), Spec((4096, 1024)))
    yield lstm_grad_outputs(Spec((4096, 4096)), Spec((4096, 1024)), Spec((4096, 1024)), Spec((4096, 1024)))
    yield gather_outputs(Spec((16384, 16384)), Spec((16384 * 16384,)))
    # the bounded samples that are also run through the CPU oracle
    yield cumsum_outputs(Spec((512, 16384), f32))
    yield cumprod_outputs(Spec((512, 16384), f32))
    yield cumsum_outputs(Spec((256, 16384), f64))
    yield lstm_outputs(Spec((512, 4096)), Spec((512, 1024)))
    yield lstm_grad_outputs(Spec((512, 4096)), Spec((512, 1024)), Spec((512, 1024)), Spec((512, 1024)))
    yield gather_outputs(Spec((2048, 2048)), Spec((2048 * 2048,)))


def uniform(rng, lo, hi, shape, dtype=np.float32):
    return (lo + (hi - lo) * rng.random(shape, dtype=dtype)).astype(dtype)


# ----------------------------------------------------------------------------------------------------------------------
# measurement
# ----------------------------------------------------------------------------------------------------------------------
class Prepared(object):
    """A fused operator DAG with its device tensors, ready to be launched repeatedly."""

    def __init__(self, outputs, options=None):
        import torch
        from opveclib_amd import runtime
        from opveclib_amd.operator import _build_op_dag
        from opveclib_amd.fusion import _merge_op_dag
        op_dag = _build_op_dag(*outputs)
        self.dag, _ = _merge_op_dag(op_dag.proto_dag, None)
        self.device = torch.device('cuda', 0)
        self.leaves = [x if isinstance(x, torch.Tensor) else torch.from_numpy(np.ascontiguousarray(x)).to(self.device)
                       for x in op_dag.inputs]
        self.ops = [runtime.load_operator(op, options) for op in self.dag.operators]
        self.buffers = []
        self.steps = []
        for op_index, compiled in enumerate(self.ops):
            ins = []
            for ref in self.dag.references[op_index].input_refs:
                ins.append(self.leaves[ref.dag_input_index] if ref.is_leaf
                           else self.buffers[ref.op_index][ref.op_output_index])
            compiled.check_inputs(ins)
            outs = compiled.allocate_outputs(self.device)
            self.buffers.append(outs)
            self.steps.append((compiled, compiled.params(ins, compiled.input_types), len(ins),
                               compiled.params(outs, compiled.output_types), len(outs)))
        self.algorithmic_bytes = sum(c.gen.algorithmic_bytes for c in self.ops)
        self.kernels = [c.lib.info for c in self.ops]

    def launch(self, stream):
        for compiled, in_params, n_in, out_params, n_out in self.steps:
            compiled.lib.launch(in_params, n_in, out_params, n_out, stream)

    def results(self):
        return [self.buffers[ref.op_index][ref.op_output_index] for ref in self.dag.dag_outputs]


def settle(prepared, busy_ms=40.0, limit_ms=250.0, window=8, tolerance=0.02):
    """
    Launch until the GPU's clocks have settled under this kernel: for at least ``busy_ms`` of kernel time and until
    the last ``window`` launch times lie within ``tolerance`` of each other, at most ``limit_ms``.  Untimed
    conditioning before the warm-up; returns the number of launches it took.
    """
    import torch
    stream_obj = torch.cuda.current_stream()
    stream = stream_obj.cuda_stream
    recent = []
    total = 0.0
    launches = 0
    while total < limit_ms:
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream_obj)
        prepared.launch(stream)
        stop.record(stream_obj)
        stop.synchronize()
        elapsed = start.elapsed_time(stop)
        total += elapsed
        launches += 1
        recent = (recent + [elapsed])[-window:]
        if total >= busy_ms and len(recent) == window and max(recent) <= (1.0 + tolerance) * min(recent):
            break
    return launches


def measure(prepared, steps, warmup):
    """Returns (ms per step from the host clock around the timed region, mean ms per launch from HIP events)."""
    import torch
    stream_obj = torch.cuda.current_stream()
    stream = stream_obj.cuda_stream
    for _ in range(warmup):
        prepared.launch(stream)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record(stream_obj)
        prepared.launch(stream)
        stops[i].record(stream_obj)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    per_launch = [s.elapsed_time(e) for s, e in zip(starts, stops)]
    measure.last_median_ms = float(np.median(per_launch))
    return (t1 - t0) * 1e3 / steps, float(np.mean(per_launch)), float(np.min(per_launch))


class HandWrittenLstm(object):
    """The hand-written LSTM cell kernels (include/ovl_lstm.h) behind the interface settle() and measure() use."""

    def __init__(self, concat, c, dc=None, dh=None):
        import torch
        from opveclib_amd import lstm_cell
        self.lib = lstm_cell.library()
        self.batch, self.units = c.shape
        given = [concat, c] + ([dc, dh] if dc is not None else [])
        self.tensors = [torch.from_numpy(np.ascontiguousarray(t)).cuda() for t in given]
        concat, c = self.tensors[0], self.tensors[1]
        if dc is None:
            self.outputs = [torch.empty_like(c), torch.empty_like(c)]
            self.kernels = [{'kernel': 'lstm_forward_kernel<false, 4>'}]
        else:
            self.outputs = [torch.empty_like(concat), torch.empty_like(c)]
            self.kernels = [{'kernel': 'lstm_backward_kernel<false, 4>'}]
        self.algorithmic_bytes = sum(t.numel() * 4 for t in self.tensors + self.outputs)

    def launch(self, stream):
        pointers = [t.data_ptr() for t in self.tensors]
        outs = [t.data_ptr() for t in self.outputs]
        if len(self.tensors) == 2:
            code = self.lib.ovl_lstm_forward(pointers[0], pointers[1], 1.0, self.batch, self.units, 0,
                                             outs[0], outs[1], stream)
        else:
            code = self.lib.ovl_lstm_backward(pointers[0], pointers[1], pointers[2], pointers[3], 1.0, self.batch,
                                              self.units, 0, outs[0], outs[1], stream)
        if code != 0:
            raise RuntimeError(self.lib.ovl_lstm_last_error().decode())


class HandWrittenScan(object):
    """The hand-written row scan kernels (include/ovl_scan.h) behind the interface settle() and measure() use."""

    def __init__(self, x, entry):
        import torch
        from opveclib_amd import row_scan
        self.lib = row_scan.library()
        self.entry = getattr(self.lib, entry)
        self.x = torch.from_numpy(np.ascontiguousarray(x)).cuda()
        self.out = torch.empty_like(self.x)
        self.rows, self.cols = self.x.shape
        self.algorithmic_bytes = 2 * self.x.numel() * self.x.element_size()
        self.kernels = [{'kernel': 'reassociated_scan_kernel' if entry.endswith('_reassociated')
                         else 'skewed_scan_kernel'}]

    def launch(self, stream):
        if self.entry(self.x.data_ptr(), self.rows, self.cols, self.out.data_ptr(), stream) != 0:
            raise RuntimeError(self.lib.ovl_scan_last_error().decode())


def side_workload(name, outputs, steps, warmup, options=None):
    prepared = outputs if isinstance(outputs, (HandWrittenLstm, HandWrittenScan)) else Prepared(outputs, options)
    return _side_workload(name, prepared, steps, warmup)


def _side_workload(name, prepared, steps, warmup):
    settle(prepared)
    wall_ms, event_ms, min_ms = measure(prepared, steps, warmup)
    # the median launch: kernels of a few tens of microseconds see occasional launches delayed by the host
    median_ms = measure.last_median_ms
    gbps = prepared.algorithmic_bytes / (median_ms * 1e-3) / 1e9
    return {'workload': name, 'us': round(median_ms * 1e3, 2), 'mean_us': round(event_ms * 1e3, 2),
            'min_us': round(min_ms * 1e3, 2),
            'GB/s': round(gbps, 1), 'frac': round(gbps / HBM_PEAK_GBPS, 4),
            'algorithmic_bytes': prepared.algorithmic_bytes,
            'kernels': [k['kernel'] for k in prepared.kernels]}


def clocks_under_load(prepared, seconds=2.0, per_launch_ms=0.26):
    """Shader and memory clock (MHz) as rocm-smi reports them while a queue of launches of the workload runs: the
    median of three readings taken after the first second (the power management needs that long to settle under
    this kernel); None where the tool is missing or says nothing.  Outside every timed region."""
    import subprocess
    import torch
    stream = torch.cuda.current_stream(prepared.device).cuda_stream
    for _ in range(int(seconds * 1e3 / per_launch_ms)):
        prepared.launch(stream)
    readings = {'sclk_mhz': [], 'mclk_mhz': []}
    try:
        time.sleep(1.0)
        for _ in range(3):
            text = subprocess.run(['rocm-smi', '--showclocks', '--json'], stdout=subprocess.PIPE,
                                  stderr=subprocess.DEVNULL, universal_newlines=True, timeout=30).stdout
            card = next(iter(json.loads(text[text.index('{'):]).values()))
            for key, value in card.items():
                digits = ''.join(ch for ch in str(value) if ch.isdigit() or ch == '.')
                if digits and key.startswith('sclk clock speed'):
                    readings['sclk_mhz'].append(float(digits))
                elif digits and key.startswith('mclk clock speed'):
                    readings['mclk_mhz'].append(float(digits))
    except Exception:           # the figures are informational: a missing or talkative tool must not end the benchmark
        pass
    torch.cuda.synchronize(prepared.device)
    found = dict((k, sorted(v)[len(v) // 2]) for k, v in readings.items() if v)
    return found or None


def cpu_baseline(seed_arrays, rows, iters=3):
    """The CPU oracle on the first ``rows`` rows of the chain8 inputs, all host threads, best of ``iters``."""
    import oracle
    a, b, s = seed_arrays
    outs = chain8_outputs(np.ascontiguousarray(a[:rows]), np.ascontiguousarray(b[:rows]), s)
    threads = oracle.hardware_threads()
    _, times = oracle.profile(outs, profiling_iterations=iters, opt_level=3, num_threads=threads)
    ms = min(min(t) for t in times.values()) if len(times) == 1 else sum(min(t) for t in times.values())
    nbytes = 3 * rows * a.shape[1] * 4 + 4
    # the same generated C++ built with -O2, as a courtesy next to the reference's own flags (never `value`)
    _, times_o2 = oracle.profile(outs, profiling_iterations=iters, opt_level=3, num_threads=threads,
                                 extra_flags=('-O2',))
    ms_o2 = sum(min(t) for t in times_o2.values())
    return {'value': round(nbytes / (ms * 1e-3) / 1e9, 3), 'unit': 'GB/s', 'cores': threads, 'kind': 'port',
            'ms': round(ms, 2),
            'with_O2': {'value': round(nbytes / (ms_o2 * 1e-3) / 1e9, 3), 'unit': 'GB/s', 'ms': round(ms_o2, 2)},
            'sample': 'first %d of %d rows of the chain8 inputs; reference-shaped fused C++ (g++, no -O flag as in '
                      'the reference), std::thread block split, thread create/join inside the timed region, '
                      'best of %d' % (rows, a.shape[0], iters)}, outs


def cpu_reference(outputs, sample, iters=3):
    """
    The CPU oracle on a bounded sample of a configuration (operators as written, one generated C++ function per
    operator, the reference's compiler flags, all host threads, best of ``iters``), and whether the HIP path returns
    the same bits for the same inputs.
    """
    import oracle
    import opveclib_amd as ovl
    threads = oracle.hardware_threads()
    ref, times = oracle.profile(outputs, profiling_iterations=iters, opt_level=0, num_threads=threads)
    ms = sum(float(min(t)) for t in times.values())
    got = ovl.evaluate(outputs, opt_level=3)
    got = got if isinstance(got, list) else [got]
    same = all(g.dtype == r.dtype and g.shape == r.shape and
               np.array_equal(g, r, equal_nan=(r.dtype.kind == 'f')) for g, r in zip(got, ref))
    return {'ms': round(ms, 3), 'cores': threads, 'sample': sample, 'bit_exact': bool(same)}


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument('--gpus', type=int, default=1)
    parser.add_argument('--steps', type=int, default=100)
    parser.add_argument('--warmup', type=int, default=100)
    parser.add_argument('--no-others', action='store_true', help='skip the secondary configurations')
    parser.add_argument('--no-cpu', action='store_true',
                        help='skip what starts other programs: the CPU baseline (compiler) and the clock reading '
                             '(rocm-smi); for runs under a profiler')
    args = parser.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)' % args.gpus)

    import torch
    if not torch.cuda.is_available():
        sys.exit('bench.py needs a HIP device')
    import opveclib_amd  # noqa: F401

    rng = np.random.default_rng(2)
    shape = (8192, 8192)
    a = uniform(rng, -1, 1, shape)
    b = uniform(rng, -1, 1, shape)
    s = np.array([1.0001], np.float32)

    chain = Prepared(chain8_outputs(a, b, s))
    assert len(chain.ops) == 1, 'the 8-op chain must fuse into one kernel'
    settled_after = settle(chain)
    wall_ms, event_ms, min_ms = measure(chain, args.steps, args.warmup)
    nbytes = chain.algorithmic_bytes
    value = nbytes / (wall_ms * 1e-3) / 1e9
    achieved = nbytes / (event_ms * 1e-3) / 1e9

    result = {
        'metric': 'achieved HBM bandwidth on the fused 8-op chain (algorithmic bytes / time)',
        'value': round(value, 1), 'unit': 'GB/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': round(wall_ms, 4), 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': 'chain8: add, mul 1.0001, tanh, sigmoid, log1p, expm1, sub, abs fused into one kernel; '
                               'A, B float32 [8192, 8192] uniform[-1, 1], numpy default_rng(2)',
                   'algorithmic_bytes': nbytes, 'kernel': chain.kernels[0]['kernel'],
                   'pct_of_hbm_peak': round(100.0 * value / HBM_PEAK_GBPS, 2),
                   'clock_settling_launches_before_warmup': settled_after,
                   'clocks_under_load': None if args.no_cpu else clocks_under_load(chain)},
        'roofline': {'bound': 'hbm', 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBPS, 'unit': 'GB/s',
                     'frac': round(achieved / HBM_PEAK_GBPS, 4), 'traffic': CHAIN8_TRAFFIC_BYTES,
                     'kernel_us': round(event_ms * 1e3, 2), 'kernel_min_us': round(min_ms * 1e3, 2)},
    }

    if not args.no_cpu:
        rows = 2048
        base, cpu_outs = cpu_baseline((a, b, s), rows)
        result['cpu_baseline'] = base
        # the GPU result on the same rows must equal the oracle's bit for bit
        import oracle
        ref = oracle.evaluate(cpu_outs, opt_level=0)
        got = chain.results()[0][:rows].cpu().numpy()
        result['parity'] = {'rows_checked': rows, 'bit_exact': bool(np.array_equal(got, ref))}
    else:
        result['cpu_baseline'] = None

    if not args.no_others:
        others = []
        steps = max(5, min(args.steps, 20))
        # The optional 'fast' math mode (device math library, reciprocal-based division): not bit-compatible with the
        # reference, so it is reported beside the headline, with its distance from the exact result.
        fast = Prepared(chain8_outputs(chain.leaves[0], chain.leaves[1], chain.leaves[2]), {'math': 'fast'})
        settle(fast)
        _, fast_ms, fast_min = measure(fast, steps, args.warmup)
        exact_y, fast_y = chain.results()[0], fast.results()[0]
        err = (fast_y.double() - exact_y.double()).abs()
        ulps = (fast_y.view(torch.int32).long() - exact_y.view(torch.int32).long()).abs()
        fast_gbps = nbytes / (fast_ms * 1e-3) / 1e9
        others.append({'workload': "chain8 in the optional 'fast' math mode (not the parity path)",
                       'us': round(fast_ms * 1e3, 2), 'min_us': round(fast_min * 1e3, 2),
                       'GB/s': round(fast_gbps, 1), 'frac': round(fast_gbps / HBM_PEAK_GBPS, 4),
                       'algorithmic_bytes': nbytes, 'kernels': [k['kernel'] for k in fast.kernels],
                       'vs_exact': {'max_abs_err': float(err.max()), 'frac_bit_equal': float((ulps == 0).double().mean()),
                                    'frac_within_2ulp': float((ulps <= 2).double().mean())}})
        del fast, exact_y, fast_y, err, ulps
        others.append(side_workload('copy f32[8192,8192] (counter calibration, plain copy bandwidth)',
                                    copy_outputs(a), steps, args.warmup))
        g = np.random.default_rng(0)
        x1 = uniform(g, -0.9, 0.9, 1 << 20)
        others.append(side_workload('c1 shift_cyclic -> expm1 -> log1p, f32[2^20]', c1_outputs(x1), steps,
                                    args.warmup))
        if not args.no_cpu:
            others[-1]['cpu_reference'] = cpu_reference(c1_outputs(x1), 'the full 2^20 elements')
        del chain
        torch.cuda.empty_cache()
        g = np.random.default_rng(3)
        xs = g.standard_normal((4096, 16384), dtype=np.float32)
        others.append(side_workload('c3 cumsum f32[4096,16384] last axis', cumsum_outputs(xs), steps, args.warmup))
        if not args.no_cpu:
            others[-1]['cpu_reference'] = cpu_reference(cumsum_outputs(np.ascontiguousarray(xs[:512])),
                                                        'the first 512 rows')
        xp = uniform(g, 0.99, 1.01, (4096, 16384))
        others.append(side_workload('c3 cumprod f32[4096,16384] last axis', cumprod_outputs(xp), steps, args.warmup))
        if not args.no_cpu:
            others[-1]['cpu_reference'] = cpu_reference(cumprod_outputs(np.ascontiguousarray(xp[:512])),
                                                        'the first 512 rows')
        xd = g.standard_normal((1024, 16384))
        others.append(side_workload('c3 cumsum f64[1024,16384] last axis', cumsum_outputs(xd), steps, args.warmup))
        if not args.no_cpu:
            others[-1]['cpu_reference'] = cpu_reference(cumsum_outputs(np.ascontiguousarray(xd[:256])),
                                                        'the first 256 rows')
        others.append(side_workload('c3 cumsum f32[4096,16384], hand-written kernel (run-time shape, same bits)',
                                    HandWrittenScan(xs, 'ovl_cumsum_f32'), steps, args.warmup))
        others.append(side_workload('c3 cumsum f64[1024,16384], hand-written kernel (run-time shape, same bits)',
                                    HandWrittenScan(xd, 'ovl_cumsum_f64'), steps, args.warmup))
        # the tree-shaped wavefront scan: another association of the operands, so not the parity path; reported with
        # its distance from the sequential result
        for label, data, entry in (('f32[4096,16384]', xs, 'ovl_cumsum_f32'), ('f64[1024,16384]', xd, 'ovl_cumsum_f64')):
            tree = HandWrittenScan(data, entry + '_reassociated')
            others.append(side_workload('c3 cumsum %s, reassociating wavefront scan (not the parity path)' % label,
                                        tree, steps, args.warmup))
            sequential = HandWrittenScan(data, entry)
            sequential.launch(torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
            distance = (tree.out.double() - sequential.out.double()).abs()
            others[-1]['vs_sequential'] = {
                'max_abs_diff': float(distance.max()),
                'max_abs_diff_over_max_abs_value': float(distance.max() / sequential.out.double().abs().max()),
                'frac_bit_equal': float((tree.out == sequential.out).double().mean())}
            del tree, sequential, distance
        others.append(side_workload("c3 cumsum f32[4096,16384] in the optional 'fast' math mode (generated "
                                    "reassociating scan)", cumsum_outputs(xs), steps, args.warmup, {'math': 'fast'}))
        others.append(side_workload("c3 cumsum f64[1024,16384] in the optional 'fast' math mode (generated "
                                    "reassociating scan)", cumsum_outputs(xd), steps, args.warmup, {'math': 'fast'}))
        g = np.random.default_rng(4)
        concat = g.standard_normal((4096, 4096), dtype=np.float32)
        c = g.standard_normal((4096, 1024), dtype=np.float32)
        dh = g.standard_normal((4096, 1024), dtype=np.float32)
        dc = g.standard_normal((4096, 1024), dtype=np.float32)
        others.append(side_workload('c4 lstm cell forward [4096, 4x1024]', lstm_outputs(concat, c), steps,
                                    args.warmup))
        if not args.no_cpu:
            others[-1]['cpu_reference'] = cpu_reference(lstm_outputs(concat[:512], c[:512]), 'the first 512 rows')
        others.append(side_workload('c4 lstm cell gradient [4096, 4x1024]',
                                    lstm_grad_outputs(concat, c, dc, dh), steps, args.warmup))
        if not args.no_cpu:
            others[-1]['cpu_reference'] = cpu_reference(lstm_grad_outputs(concat[:512], c[:512], dc[:512], dh[:512]),
                                                        'the first 512 rows')
        others.append(side_workload('c4 lstm cell forward, hand-written kernel (run-time shape, same bits)',
                                    HandWrittenLstm(concat, c), steps, args.warmup))
        others.append(side_workload('c4 lstm cell gradient, hand-written kernel (run-time shape, same bits)',
                                    HandWrittenLstm(concat, c, dc, dh), steps, args.warmup))
        others.append(side_workload("c4 lstm cell forward in the optional 'fast' math mode", lstm_outputs(concat, c),
                                    steps, args.warmup, {'math': 'fast'}))
        others.append(side_workload("c4 lstm cell gradient in the optional 'fast' math mode",
                                    lstm_grad_outputs(concat, c, dc, dh), steps, args.warmup, {'math': 'fast'}))
        torch.cuda.empty_cache()
        g5 = torch.Generator(device='cuda')
        g5.manual_seed(5)
        a5 = torch.randn((16384, 16384), device='cuda', generator=g5)
        b5 = torch.randn((16384 * 16384,), device='cuda', generator=g5)
        others.append(side_workload('c5 gather + transposed scatter f32[16384,16384]', gather_outputs(a5, b5),
                                    max(3, steps // 4), 2))
        if not args.no_cpu:
            g = np.random.default_rng(5)
            a_small = g.standard_normal((2048, 2048), dtype=np.float32)
            b_small = g.standard_normal(2048 * 2048, dtype=np.float32)
            others[-1]['cpu_reference'] = cpu_reference(gather_outputs(a_small, b_small),
                                                        'the same operator on A, B float32 [2048, 2048]')
        result['others'] = others

    print(json.dumps(result))


if __name__ == '__main__':
    main()
