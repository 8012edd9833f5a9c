"""
HIP code generator: expression DAG -> source text of one operator library for gfx950.

Counterpart of ``ExpressionDAG.generate`` in the reference (opveclib/expression.py:521-706), which returns C++ and
CUDA text built around a one-thread-per-worker template.  Here the DAG is analysed first
(:mod:`.analysis`) and the kernel is produced by the template that fits its access pattern:

* :mod:`.map_kernel` - vectorised map (any DAG; vector width 1 is the general fallback);
* :mod:`.tile_kernel` - rank-2 workgroups with transposed stores: LDS-tiled so reads and writes are both coalesced;
* :mod:`.rowscan_kernel` - loop-carried accumulation along the last tensor axis: order-preserving row scans
  (lane-skewed out of registers; lane-skewed or lane = row out of LDS, fed by dedicated data-moving wavefronts, with
  the results written by the scanning wavefront or recomputed by a second one) and the reassociating wavefront scan;
* :mod:`.colscan_kernel` - the same accumulation along another axis: rows streamed through LDS, lane-skewed over
  sixteen lanes per line for tensors with up to 32768 lines ('colskew'), lane = line beyond ('colscan').

Every library exports ``<name>_generic_hip(in, n_in, out, n_out, stream)``: it validates tensor counts, lengths,
dtypes (the reference's ``*err = 1`` checks, expression.py:621-646, 662-663) and pointer alignment, enqueues the
kernel on the stream and returns a status code; and ``<name>_info()`` returning a JSON description of the kernel.
"""

import json

from .. import language as lang
from .analysis import DagInfo, ITEMSIZE
from .body import CTYPE
from . import map_kernel
from .map_kernel import MAX_GRID      # upper bound of the launch grid; kernels loop beyond it
from . import tile_kernel
from . import rowscan_kernel
from . import colscan_kernel

#: bump when generated code changes for an unchanged DAG, so cached binaries are not reused
CODEGEN_VERSION = 43



class GeneratedOperator(object):
    def __init__(self, name, source, entry, info_symbol, kernel_name, launch, algorithmic_bytes):
        self.name = name
        self.source = source
        self.entry = entry
        self.info_symbol = info_symbol
        self.kernel_name = kernel_name
        self.launch = launch
        self.algorithmic_bytes = algorithmic_bytes


def _kernel_label(dag_name):
    label = ''.join(ch if ch.isalnum() else '_' for ch in dag_name)
    return label[:48] if label else 'op'


def algorithmic_bytes(info):
    """Compulsory traffic of one launch: every input element read once, every output element written once."""
    total = 0
    for node in list(info.inputs.values()) + list(info.outputs.values()):
        total += node.size * ITEMSIZE[node.dtype]
    return total


def generate(expression_dag, function_name, options=None):
    """
    :param expression_dag: serialised expression DAG of one operator
    :param function_name: unique name of the operator (its content hash)
    :param options: optional dict.  ``template``: 'auto' (default), 'map', 'transpose', 'rowscan', 'skewscan', 'fedscan', 'carryscan', 'treescan', 'rowreduce', 'colreduce', 'colscan' or 'colskew' restricts
        the choice of kernel template (a template that does not fit the DAG falls back to 'map'); ``vec`` forces the
        map template with that vector width, ``per_thread`` its vectors per thread (1 or 2); ``scan_movers`` the number of threads that only move data in the lane-skewed column scan (0: every wavefront scans and moves), ``scan_carry`` False keeps the results in its scanning wavefronts instead of recomputing them in finishing ones, ``scan_depth`` / ``scan_sets`` / ``scan_width`` / ``scan_interleave`` set the request burst (groups), the
        number of register sets, the 128-bit vectors per lane and phase and the rows per lane group of the lane-skewed scan; ``math``: 'exact'
        or 'fast'; ``if_conversion`` / ``value_ranges`` / ``cse``: False switches that transformation off; ``scan_rows`` / ``scan_chunk`` the LDS tile of the row scan, ``scan_batch`` the vectors per register set of its scanning wavefront; ``nt`` /
        ``scan_nt`` which vector accesses carry the non-temporal hint ('l' loads, 's' stores, 'ls', ''); ``grid_cap``
        the largest grid of the map and transpose templates (their kernels then stride over the rest)
    :return: a :class:`GeneratedOperator`
    """
    options = options or {}
    info = DagInfo(expression_dag)
    if info.num_workers >= 2 ** 32:
        # positions are 32-bit, as in the reference (worker_index is uint32, expression.py:582-608)
        raise ValueError('workgroup of %d workers: at most 2^32 - 1 are supported' % info.num_workers)
    info.math = options.get('math', 'exact')
    info.if_conversion = options.get('if_conversion', True)
    info.value_ranges = options.get('value_ranges', True)
    info.cse = options.get('cse', True)
    kernel_name = 'ovl_' + _kernel_label(info.name) + '_' + function_name[1:9]
    if info.math != 'exact':
        kernel_name += '_' + info.math         # so that profiles tell the math modes of one operator apart

    template = options.get('template', 'auto')
    tree = None
    if options.get('vec') is None and template in ('auto', 'treescan'):
        tree = rowscan_kernel.tree_plan(info)
        # integer sums, products and extrema are associative (sums and products modulo 2^n): the tree gives the
        # reference's bits; floating point ones only when the caller has given up the order
        if tree is not None and template == 'auto' and info.math != 'fast' and \
                tree[0].x.dtype in (lang.FLOAT32, lang.FLOAT64):
            tree = None
        if tree is not None and (tree[0].length % tree[0].vec != 0 or tree[0].rows > MAX_GRID):
            tree = None
        # one workgroup per row pays from about one full step (256 vectors) per row; shorter rows keep the lane-skewed
        # scan, which packs sixteen rows into a workgroup
        if tree is not None and template == 'auto' and tree[0].length < 256 * tree[0].vec:
            tree = None
    if tree is not None:
        # sums, products and running extrema whose order the caller has given up: the reassociating scan
        kernel_src, launch = rowscan_kernel.generate_tree(info, kernel_name, options.get('scan_ahead') or 8)
    elif options.get('vec') is None and template in ('auto', 'carryscan') and \
            rowscan_kernel.carry_plan(info, options.get('scan_width')) is not None and \
            (template == 'carryscan' or (rowscan_kernel.carry_plan(info)[0].vec == 2 and
                                         rowscan_kernel.carry_preferred(info))):
        # 8-byte elements run at the latency of their recurrence: with at most one workgroup per compute unit the
        # scanning wavefront does nothing but the recurrence, a second one recomputes and writes the results
        kernel_src, launch = rowscan_kernel.generate_carry(info, kernel_name, options.get('scan_width'))
    elif options.get('vec') is None and template in ('auto', 'fedscan') and \
            rowscan_kernel.fed_plan(info, options.get('scan_width'), options.get('scan_chunk')) is not None and \
            (template == 'fedscan' or rowscan_kernel.fed_plan(info)[0].vec == 2):
        # 8-byte elements run at the latency of their recurrence: the LDS-fed variant halves the hand-overs
        kernel_src, launch = rowscan_kernel.generate_fed(info, kernel_name, options.get('scan_width'),
                                                         options.get('scan_chunk'))
    elif options.get('vec') is None and template in ('auto', 'skewscan') and rowscan_kernel.skew_plan(info) is not None:
        kernel_src, launch = rowscan_kernel.generate_skewed(info, kernel_name, options.get('scan_depth'), options.get('scan_sets'), options.get('scan_nt', 's'),
                                                             options.get('scan_width'), options.get('scan_interleave'),
                                                             options.get('scan_split'))
    elif options.get('vec') is None and template in ('auto', 'rowscan') and rowscan_kernel.plan(info) is not None:
        kernel_src, launch = rowscan_kernel.generate(info, kernel_name, options.get('scan_rows'),
                                                     options.get('scan_chunk'), options.get('scan_batch'))
    elif options.get('vec') is None and template in ('auto', 'colskew') and colscan_kernel.plan(info) is not None and \
            (template == 'colskew' or (colscan_kernel.worthwhile(info, colscan_kernel.plan(info)) and
                                       colscan_kernel.prefers_skew(info, colscan_kernel.plan(info)))):
        kernel_src, launch = colscan_kernel.generate_skewed(info, kernel_name, options.get('scan_sets'),
                                                            options.get('scan_strip'), options.get('scan_width'),
                                                            options.get('scan_movers'), carry=options.get('scan_carry'),
                                                            nt=options.get('scan_nt'))
    elif options.get('vec') is None and template in ('auto', 'colscan') and \
            colscan_kernel.plan(info, options.get('scan_rows'), options.get('scan_batch'),
                                options.get('scan_sets')) is not None and \
            (template == 'colscan' or colscan_kernel.worthwhile(info, colscan_kernel.plan(info))):
        kernel_src, launch = colscan_kernel.generate(info, kernel_name, options.get('scan_rows'),
                                                     options.get('scan_batch'), options.get('scan_sets'))
    elif options.get('vec') is None and template in ('auto', 'rowreduce') and rowscan_kernel.reduce_plan(info) is not None:
        # a loop-carried state over the last axis with nothing stored inside the loop: a dot product, a sum
        kernel_src, launch = rowscan_kernel.generate_reduce(info, kernel_name, options.get('scan_depth'),
                                                            options.get('scan_width'), options.get('scan_sets'),
                                                            options.get('scan_nt', ''))
    elif options.get('vec') is None and template in ('auto', 'colreduce') and \
            colscan_kernel.reduce_plan(info, options.get('scan_rows'), options.get('scan_batch'),
                                       options.get('scan_sets')) is not None and \
            (template == 'colreduce' or colscan_kernel.worthwhile(info, colscan_kernel.reduce_plan(info))):
        # a loop-carried state over an axis that is not the last, nothing stored inside the loop: a column sum
        if options.get('scan_skew', True) and options.get('scan_rows') is None and options.get('scan_batch') is None and \
                colscan_kernel.prefers_skew(info, colscan_kernel.reduce_plan(info)):
            # few lines: sixteen lanes per line, as for the scans
            kernel_src, launch = colscan_kernel.generate_skewed(info, kernel_name, options.get('scan_sets'),
                                                                options.get('scan_strip'), options.get('scan_width'),
                                                                options.get('scan_movers'), reduce=True)
        else:
            kernel_src, launch = colscan_kernel.generate(info, kernel_name, options.get('scan_rows'),
                                                         options.get('scan_batch'), options.get('scan_sets'),
                                                         reduce=True)
    elif options.get('vec') is None and template in ('auto', 'transpose') and tile_kernel.applicable(info) is not None:
        kernel_src, launch = tile_kernel.generate(info, kernel_name, options.get('tile_i'), options.get('tile_j'),
                                                  options.get('nt'), options.get('tile_order'))
    else:
        kernel_src, launch = map_kernel.generate(info, kernel_name, options.get('vec'), options.get('nt'),
                                                 options.get('grid_cap'), options.get('per_thread'))

    num_inputs = len(info.inputs)
    num_outputs = len(info.outputs)
    entry = function_name + '_generic_hip'
    info_symbol = function_name + '_info'

    src = ['// Generated by opveclib_amd.hipgen (codegen %d) for operator "%s"' % (CODEGEN_VERSION, info.name),
           '#include "ovl_device.h"', '', kernel_src]

    src.append('extern "C" int ' + entry + '(const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out,'
               ' void* stream) {')
    src.append('    if (n_in != %du || n_out != %du) return OVL_EARGS;' % (num_inputs, num_outputs))
    call_args = []
    for kind, table in (('in', info.inputs), ('out', info.outputs)):
        for i in range(len(table)):
            node = table[i]
            src.append('    if (%s[%d].len != %dull || %s[%d].dtype != %d) return OVL_EARGS;' % (
                kind, i, node.size, kind, i, node.dtype))
            need = launch['align'].get((kind, i), 1)
            if need > 1:
                src.append('    if ((reinterpret_cast<uintptr_t>(%s[%d].data) & %du) != 0) return OVL_EALIGN;' % (
                    kind, i, need - 1))
            const = 'const ' if kind == 'in' else ''
            call_args.append('static_cast<%s%s*>(%s[%d].data)' % (const, CTYPE[node.dtype], kind, i))
    grid = launch['blocks_needed']
    if launch['template'] in ('map', 'transpose'):
        # these kernels stride over what the grid does not cover
        grid = min(grid, launch.get('grid_cap') or options.get('grid_cap') or MAX_GRID, MAX_GRID)
    elif grid > MAX_GRID:
        raise ValueError('%d workgroups: the %s template launches at most %d' % (grid, launch['template'], MAX_GRID))
    src.append('    uint32_t grid = %du;' % grid)
    src.append('    hipLaunchKernelGGL(%s, dim3(grid), dim3(%du), 0, static_cast<hipStream_t>(stream),' % (
        kernel_name, launch['block']))
    src.append('                       ' + ', '.join(call_args) + ');')
    src.append('    return hipPeekAtLastError() == hipSuccess ? OVL_OK : OVL_EHIP;')
    src.append('}')
    src.append('')

    nbytes = algorithmic_bytes(info)
    description = {
        'operator': info.name, 'kernel': kernel_name, 'template': launch['template'], 'vec': launch['vec'],
        'block': launch['block'], 'workers': info.num_workers, 'algorithmic_bytes': nbytes,
        'vector_loads': launch['vector_loads'], 'vector_stores': launch['vector_stores']}
    text = json.dumps(description, sort_keys=True).replace('\\', '\\\\').replace('"', '\\"')
    src.append('extern "C" const char* ' + info_symbol + '(void) { return "' + text + '"; }')

    return GeneratedOperator(function_name, '\n'.join(src) + '\n', entry, info_symbol, kernel_name, launch, nbytes)
