"""
Operator DAGs recorded into a HIP graph.

A DAG that stays unfused in several kernels (producers that permute data, scans, reductions between element-wise
stages) or that is evaluated again and again on buffers of one shape (a recurrent cell, an inner loop) pays a few
microseconds of launch latency per kernel and the Python cost of ``evaluate`` per call.  :class:`CapturedDag` does the
front-end work once - trace, fuse, generate, compile, load, allocate - records the launches into a HIP graph
(through ``torch.cuda.CUDAGraph``: PyTorch is used for the stream capture, the launches are the C-ABI launcher's) and
replays them with a single call.

The graph reads the DAG's leaf tensors and writes its output tensors at replay time: feed new data by copying into
the leaves (``captured.inputs[k].copy_(...)``), read results from ``captured.outputs``.  Nothing is allocated, copied
or cleared inside the captured region (in particular no memset nodes).
"""

from .operator import _build_op_dag, _normalise_output_list, get_math_mode, MATH_MODES


class CapturedDag(object):
    """
    :param output_list: an operator, an operator output, or a list of either.  Every leaf input of the DAG must be a
        contiguous torch tensor on one HIP device whose data pointer is 16-byte aligned; these tensors are the graph's
        input buffers.
    :param opt_level: operators are fused when opt_level >= 3
    :param math_mode: 'exact', 'ulp2' or 'fast'; None uses the current default
    """

    def __init__(self, output_list, opt_level=3, math_mode=None):
        import torch
        from . import runtime
        from .fusion import _merge_op_dag

        if math_mode is None:
            math_mode = get_math_mode()
        if math_mode not in MATH_MODES:
            raise ValueError('math_mode must be one of ' + str(MATH_MODES))
        options = None if math_mode == 'exact' else {'math': math_mode}
        runtime._require_gpu()

        op_dag = _build_op_dag(*_normalise_output_list(output_list))
        dag = op_dag.proto_dag
        if opt_level >= 3:
            dag, _ = _merge_op_dag(dag, None)

        device = None
        for n, leaf in enumerate(op_dag.inputs):
            if not isinstance(leaf, torch.Tensor) or leaf.device.type != 'cuda':
                raise TypeError('input %d of a captured DAG must be a torch tensor on a HIP device' % n)
            if device is not None and leaf.device != device:
                raise TypeError('the inputs of a captured DAG must live on one device')
            device = leaf.device
            if not leaf.is_contiguous() or leaf.data_ptr() % 16 != 0:
                raise TypeError('input %d of a captured DAG must be contiguous and 16-byte aligned' % n)
        if device is None:
            raise TypeError('a captured DAG needs at least one tensor input')
        self.inputs = [leaf.detach() for leaf in op_dag.inputs]
        self.device = device

        # everything that compiles, loads or allocates happens before the capture
        runtime._build_missing(dag.operators, options)
        buffers = []
        self._steps = []
        self.kernels = []
        for op_index, op in enumerate(dag.operators):
            compiled = runtime.load_operator(op, options)
            ins = []
            for ref in dag.references[op_index].input_refs:
                ins.append(self.inputs[ref.dag_input_index] if ref.is_leaf
                           else buffers[ref.op_index][ref.op_output_index])
            compiled.check_inputs(ins)
            outs = compiled.allocate_outputs(device)
            buffers.append(outs)
            self._steps.append((compiled, compiled.params(ins, compiled.input_types), len(ins),
                                compiled.params(outs, compiled.output_types), len(outs)))
            self.kernels.append(compiled.name)
        self._buffers = buffers
        self.outputs = [buffers[ref.op_index][ref.op_output_index] for ref in dag.dag_outputs]

        with torch.cuda.device(device):
            # one eager pass on a side stream first, as stream capture requires of work that has never run
            side = torch.cuda.Stream(device)
            side.wait_stream(torch.cuda.current_stream(device))
            with torch.cuda.stream(side):
                self._launch(side.cuda_stream)
            torch.cuda.current_stream(device).wait_stream(side)
            torch.cuda.synchronize(device)
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self._launch(torch.cuda.current_stream(device).cuda_stream)

    def _launch(self, stream):
        for compiled, in_params, n_in, out_params, n_out in self._steps:
            compiled.lib.launch(in_params, n_in, out_params, n_out, stream)

    def launch_eagerly(self):
        """The same launches, one by one on the current stream (for comparison with :meth:`replay`)."""
        import torch
        with torch.cuda.device(self.device):
            self._launch(torch.cuda.current_stream(self.device).cuda_stream)
        return self.outputs

    def replay(self):
        """Run the recorded DAG on the current contents of ``inputs``; returns ``outputs`` (not synchronised)."""
        self.graph.replay()
        return self.outputs
