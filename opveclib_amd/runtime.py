"""
Execution of an operator DAG on the GPU: generate, compile (cached), load and enqueue each operator.

Counterpart of the per-operator loop of the reference's ``profile`` (opveclib/operator.py:2262-2335) with its CUDA
test harness (opveclib/testcudaop.cc:60-395).  Differences that matter for speed: tensors live in device memory for
the whole DAG (the reference copies every operator's inputs to the device and its outputs back, testcudaop.cc:85-183,
311-379), launches go to the current PyTorch HIP stream without synchronising, and compiled operators stay loaded.
PyTorch is used for device memory and streams only.
"""

import threading

import numpy as np

from . import language as lang
from . import compiler
from . import hipgen
from . import launcher
from . import transfer
from .expression import TensorType
from .operator import _op_hash

#: fill operator outputs with 0xFE bytes before each launch so unwritten elements are recognisable
#: (the reference's harness always does, testcudaop.cc:188-269); off by default because it costs a memset per output
poison_outputs = False

_lock = threading.Lock()
_generated = {}     # op hash -> (GeneratedOperator, library path)
_loaded = {}        # op hash -> CompiledOperator


def _io_types(op):
    ins = sorted((e for e in op.expressions if e.code == lang.INPUT), key=lambda e: e.io_index)
    outs = sorted((e for e in op.expressions if e.code == lang.OUTPUT), key=lambda e: e.io_index)
    return ([TensorType.from_proto(e.tensor_type) for e in ins],
            [TensorType.from_proto(e.tensor_type) for e in outs])


# Code generator options applied to every operator that is loaded without explicit options, e.g. {'template': 'map'}
# to force the general kernel template (see hipgen.generate).
codegen_options = {}


#: the operations whose code the 'ulp2' math mode can change (float32 only)
_MATH_SENSITIVE = (lang.EXP, lang.LOG, lang.TANH, lang.DIVIDE)


def effective_options(op, options):
    """``options`` without a 'ulp2' math mode that cannot change this operator's code (no float32 exp, log, tanh or
    division in it): such an operator is the 'exact' kernel, and is generated, compiled and cached as that."""
    if options and options.get('math') == 'ulp2' and not any(
            e.code in _MATH_SENSITIVE and e.dtype == lang.FLOAT32 for e in op.expressions):
        options = dict((k, v) for k, v in options.items() if k != 'math')
    return options or None


def build_operator(op, options=None):
    """Generate HIP for one operator and make sure its library exists on disk.  Needs hipcc, not a GPU.

    :return: (GeneratedOperator, library path)
    """
    options = effective_options(op, options)
    name = _op_hash(op)
    key = (name, repr(sorted((options or {}).items())))
    with _lock:
        if key in _generated:
            return _generated[key]
    gen = hipgen.generate(op, name, options)
    so_path = compiler.build_library(gen.source)
    with _lock:
        _generated[key] = (gen, so_path)
    return gen, so_path


class CompiledOperator(object):
    """A loaded operator: entry point plus the tensor types it expects."""

    def __init__(self, op, options=None):
        self.gen, self.so_path = build_operator(op, options)
        self.lib = launcher.OperatorLibrary(self.so_path, self.gen.entry, self.gen.info_symbol)
        self.input_types, self.output_types = _io_types(op)
        self.name = self.gen.name
        self.dag_name = op.name

    def params(self, tensors, types):
        triples = []
        for t, tt in zip(tensors, types):
            triples.append((t.data_ptr(), tt.dtype.proto_dtype, tt.size))
        return launcher.tensor_array(triples)

    def allocate_outputs(self, device):
        import torch
        return [torch.empty(tt.shape, dtype=tt.dtype.as_torch(), device=device) for tt in self.output_types]

    def check_inputs(self, tensors):
        if len(tensors) != len(self.input_types):
            raise TypeError('%s expects %d inputs, got %d' % (self.dag_name, len(self.input_types), len(tensors)))
        for n, (t, tt) in enumerate(zip(tensors, self.input_types)):
            if t.dtype != tt.dtype.as_torch() or t.numel() != tt.size:
                raise TypeError('input %d of %s: expected %s %s, got %s %s' % (
                    n, self.dag_name, tt.dtype, tt.shape, t.dtype, tuple(t.shape)))
            if not t.is_contiguous():
                raise TypeError('input %d of %s is not contiguous' % (n, self.dag_name))

    def launch(self, inputs, outputs, stream):
        """Enqueue on ``stream`` (a raw hipStream_t value); returns immediately."""
        in_params = self.params(inputs, self.input_types)
        out_params = self.params(outputs, self.output_types)
        if poison_outputs:
            launcher.check(launcher.library().ovl_poison(out_params, len(outputs), stream))
        self.lib.launch(in_params, len(inputs), out_params, len(outputs), stream)

    def time(self, inputs, outputs, stream, iters):
        in_params = self.params(inputs, self.input_types)
        out_params = self.params(outputs, self.output_types)
        if poison_outputs:
            launcher.check(launcher.library().ovl_poison(out_params, len(outputs), stream))
        return self.lib.time(in_params, len(inputs), out_params, len(outputs), stream, iters)


def load_operator(op, options=None):
    if codegen_options:
        options = dict(codegen_options, **(options or {}))
    options = effective_options(op, options)
    name = _op_hash(op)
    key = (name, repr(sorted((options or {}).items())))
    with _lock:
        if key in _loaded:
            return _loaded[key]
    compiled = CompiledOperator(op, options)
    with _lock:
        _loaded[key] = compiled
    return compiled


#: compiler processes run side by side when several operators of one DAG have no library yet
max_parallel_builds = 8


def _build_missing(operators, options):
    """
    Cold start: generate and compile, in parallel, every operator of the DAG that is neither loaded nor built.  One
    hipcc run takes 10-20 s, so an unfused eight operator DAG starts in the time of one compilation instead of eight
    (the reference compiles its operators one after the other, opveclib/operator.py:2262-2300).
    """
    if codegen_options:
        options = dict(codegen_options, **(options or {}))
    missing = {}
    for op in operators:
        name = _op_hash(op)
        option_key = repr(sorted((effective_options(op, options) or {}).items()))
        with _lock:
            known = (name, option_key) in _loaded or (name, option_key) in _generated
        if not known:
            missing[name] = op
    if len(missing) > 1:
        from concurrent.futures import ThreadPoolExecutor
        with ThreadPoolExecutor(max_workers=min(max_parallel_builds, len(missing))) as pool:
            list(pool.map(lambda op: build_operator(op, options), missing.values()))


def _require_gpu():
    import torch
    if not torch.cuda.is_available():
        raise RuntimeError('No HIP device is available: opveclib_amd operators only run on an AMD GPU (gfx950).')
    return torch


def _to_device(x, torch, device):
    """Contiguous, 16-byte aligned device tensor for a DAG input; returns (tensor, came_from_host_array)."""
    if isinstance(x, np.ndarray):
        return transfer.to_device(x, torch, device), True
    if isinstance(x, torch.Tensor):
        t = x.detach()
        if t.device.type != 'cuda':
            t = t.to(device)
        t = t.contiguous()
        if t.data_ptr() % 16 != 0:
            t = t.clone()       # a view into the middle of an allocation: vector loads need an aligned base
        return t, False
    return transfer.to_device(np.asarray(x), torch, device), True


def run_op_dag(dag, leaf_inputs, profiling_iterations=1, timed=True, options=None):
    """
    Run every operator of ``dag`` in order.

    :param dag: OperatorDAG message (already optimised if wanted)
    :param leaf_inputs: the DAG's input tensors (numpy arrays or torch tensors) in ``dag_input_index`` order
    :param timed: time each operator over ``profiling_iterations`` launches (synchronises); otherwise launch once
        asynchronously
    :return: (outputs in request order, {operator hash name: float64 array of milliseconds})
    """
    torch = _require_gpu()
    device = None
    for x in leaf_inputs:
        if isinstance(x, torch.Tensor) and x.device.type == 'cuda':
            device = x.device
            break
    if device is None:
        device = torch.device('cuda', torch.cuda.current_device())

    all_host = True
    leaves = []
    for x in leaf_inputs:
        t, from_host = _to_device(x, torch, device)
        all_host = all_host and from_host
        leaves.append(t)

    _build_missing(dag.operators, options)
    with torch.cuda.device(device):
        stream = torch.cuda.current_stream(device).cuda_stream
        buffers = []
        times = {}
        for op_index, op in enumerate(dag.operators):
            compiled = load_operator(op, options)
            inputs = []
            for ref in dag.references[op_index].input_refs:
                if ref.is_leaf:
                    inputs.append(leaves[ref.dag_input_index])
                else:
                    inputs.append(buffers[ref.op_index][ref.op_output_index])
            compiled.check_inputs(inputs)
            outputs = compiled.allocate_outputs(device)
            buffers.append(outputs)
            if timed:
                ms = compiled.time(inputs, outputs, stream, profiling_iterations)
                times[compiled.name] = np.array(ms, dtype=np.float64)
            else:
                compiled.launch(inputs, outputs, stream)

        results = [buffers[ref.op_index][ref.op_output_index] for ref in dag.dag_outputs]
        if all_host:
            results = [transfer.to_host(r, torch) for r in results]
    return results, times
