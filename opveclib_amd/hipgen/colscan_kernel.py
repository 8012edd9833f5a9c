"""
The column-scan kernel template: operators that walk an axis other than the last with a loop-carried accumulator
(``accumulate`` / ``cumsum`` / ``cumprod`` of the reference's opveclib/examples/test_accumulate.py:22-147 along axis 0
of a matrix is the shape its timing script runs, test_perf_accumulate.py:35-47).

The workgroup is the tensor's shape without the scanned axis: one worker per line along the axis, neighbouring
workers on neighbouring elements of the last dimension.  In the one-worker-per-thread template the lanes of a
wavefront are therefore coalesced, but every trip of the worker's loop waits for its own load: with few lines there
are few wavefronts, and each moves one row of a strip per memory latency (float64 [10000, 1000]: 16 wavefronts,
2.3 ms, 70 GB/s).  Here a 1024-thread workgroup owns a strip of 64 neighbouring lines and streams it through LDS in
chunks of rows with three rotating buffers, as the row scans do:

  * fifteen wavefronts move data: each instruction loads or stores one row of the strip (64 consecutive elements),
    and several chunks of loads are in flight per workgroup, as many as fit the registers (with two, a workgroup
    moved one chunk per memory latency: float64 [10000, 1000] 324 us; with four 191 us);
  * wavefront 0 runs the recurrence, lane = line, out of LDS and in place, several rows per 128-bit LDS access
    (the tile is stored line-major so that a lane's next rows are adjacent), through two register sets so that the
    latency of an LDS read is paid once per chunk.  Its results go back to LDS and out through the movers: when the
    scanning wavefront stored them to global memory itself, one instruction per row, float64 [10000, 1000] took
    423 us instead of 191 us.  A raised issue priority for it changed nothing.

With enough loads in flight the scanning wavefront sets the pace, about 45 clocks per row of 64 float64 lines, so a
tensor with few lines (1000 lines = 16 workgroups) stays far below the memory's rate while one with many
([4096, 4096]: 82 us, 3.3 TB/s) comes close to the row scans.

The arithmetic each line sees is exactly the worker's sequential recurrence: results equal the generic template's
(and numpy's accumulate) bit for bit.
"""

from .. import language as lang
from .analysis import ITEMSIZE
from .body import BodyEmitter, CTYPE

BLOCK = 1024                    # one scanning wavefront and fifteen that move data
WAVE = 64
MOVERS = BLOCK - WAVE
STRIP = WAVE                    # lines per workgroup
SETS = 8                        # most chunks of loads in flight per workgroup
SET_REGISTERS = 40              # registers of a mover thread that may hold loads in flight (1024 threads: 128 each)
LDS_BUDGET = 96 * 1024
#: (no upper limit on the number of lines: the one-worker-per-thread template waits for one load per trip of its loop
#: however many wavefronts there are: float32 [1000, 70000] 979 us against 192 us, [64, 4194304] 1728 against 460 us)
MAX_BLOCKS = (1 << 24) - 1
MIN_LENGTH = 64


class ColumnPlan(object):
    def __init__(self, loop_item, counter, length, outer, inner, x, out, per, rows_per_chunk, batch, sets):
        self.loop_item = loop_item
        self.counter = counter
        self.length = length            # extent of the scanned axis
        self.outer = outer              # product of the dimensions before it
        self.inner = inner              # product of the dimensions after it: the distance between rows
        self.x = x
        self.out = out
        self.per = per                  # rows per 128-bit LDS access
        self.rows_per_chunk = rows_per_chunk
        self.batch = batch              # LDS accesses per register set of the scanning wavefront
        self.sets = sets                # register sets of the movers = chunks of loads in flight
        self.reduce = False             # a reduction: nothing is stored inside the loop, `out` is None
        self.start = 1                  # first row the loop visits
        self.end_idx = None             # (reductions) the node that closes the loop


def plan(info, rows_per_chunk=None, batch=None, sets=None):
    """A ColumnPlan when the DAG is a scan along a non-last axis that this template can run, else None."""
    if len(info.inputs) != 1 or len(info.outputs) != 1:
        return None
    loops = [item for item in info.tree if item.kind == 'loop']
    if len(loops) != 1 or any(item.kind == 'if' for item in info.tree):
        return None
    loop = loops[0]
    # set-up of the first row (at most one store), then the loop, then nothing
    if info.tree[-1] is not loop:
        return None
    stores_before = [item for item in info.tree[:-1] if item.kind == 'stmt' and
                     info.nodes[item.node].code == lang.ASSIGN_TENSOR and
                     info.nodes[info.nodes[item.node].ops[0]].code == lang.OUTPUT]
    if len(stores_before) > 1:
        return None
    range_node = info.nodes[loop.node]
    counter = range_node.ops[0]
    if counter not in info.loop_counters:
        return None
    start, stop, step = (info._literal_int(o) for o in range_node.ops[1:])
    if start != 1 or step != 1 or stop is None or stop < 2:
        return None
    length = stop
    if any(inner.kind != 'stmt' for inner in loop.body):
        return None

    x = info.inputs[0]
    out = info.outputs[0]
    if x.dtype != out.dtype or list(x.shape) != list(out.shape) or x.dtype not in CTYPE:
        return None
    itemsize = ITEMSIZE[x.dtype]
    if itemsize not in (4, 8):
        return None
    shape = list(x.shape)
    rank = len(shape)
    if rank < 2 or len(info.workgroup_shape) != rank - 1:
        return None
    # the scanned axis: the workgroup is the tensor's shape without it
    axis = None
    for k in range(rank - 1):       # not the last axis: the row scans take that one
        if shape[k] == length and shape[:k] + shape[k + 1:] == list(info.workgroup_shape):
            axis = k
            break
    if axis is None:
        return None
    strides = [1] * rank
    for k in range(rank - 2, -1, -1):
        strides[k] = strides[k + 1] * shape[k + 1]
    inner = strides[axis]
    outer = 1
    for d in shape[:axis]:
        outer *= d
    # flat index of the worker's line at row i: sum of position components times the tensor's strides, plus i * inner
    base = {}
    for j, dim in enumerate(d for d in range(rank) if d != axis):
        if info.workgroup_shape[j] > 1:
            base[('p', j)] = strides[dim]
    in_loop = dict(base)
    in_loop[('v', counter)] = inner
    sig_first = (tuple(sorted(base.items())), 0)
    sig_loop = (tuple(sorted(in_loop.items())), 0)
    for node, tensor, aff in info.tensor_accesses():
        if aff is None:
            return None
        expect = sig_loop if info.in_loop[node.idx] else sig_first
        if aff.signature() != expect:
            return None
    per = 16 // itemsize
    rows_per_chunk = rows_per_chunk or 64
    batch = batch or 8
    while batch > 1 and (rows_per_chunk // per) % (2 * batch) != 0:
        batch //= 2
    if rows_per_chunk % per != 0 or (rows_per_chunk // per) % (2 * batch) != 0:
        return None
    if 3 * rows_per_chunk * STRIP * itemsize > LDS_BUDGET:
        return None
    p = ColumnPlan(loop, counter, length, outer, inner, x, out, per, rows_per_chunk, batch,
                   max(2, min(int(sets or SETS), 16)))
    p.sets_forced = sets is not None
    return p


def reduce_plan(info, rows_per_chunk=None, batch=None, sets=None):
    """A ColumnPlan (with ``reduce`` set) when the DAG is a reduction along a non-last axis of one input: a counted loop
    with a loop-carried state that reads ``x[.., i, ..]`` and stores nothing inside the loop; else None."""
    loops = [item for item in info.tree if item.kind == 'loop']
    if len(loops) != 1 or any(item.kind == 'if' for item in info.tree):
        return None
    loop = loops[0]
    if any(inner.kind != 'stmt' for inner in loop.body):
        return None
    range_node = info.nodes[loop.node]
    counter = range_node.ops[0]
    if counter not in info.loop_counters:
        return None
    start, stop, step = (info._literal_int(o) for o in range_node.ops[1:])
    if start not in (0, 1) or step != 1 or stop is None or stop < 2:
        return None
    length = stop
    closers = [n.idx for n in info.nodes if n.idx > loop.node and n.code == lang.ENDRANGE and not info.in_loop[n.idx]]
    if not closers:
        return None
    x = None
    in_loop_accesses = []
    for node, tensor, aff in info.tensor_accesses():
        if not info.in_loop[node.idx]:
            continue                    # before and after the loop: ordinary code of the line's lane
        if node.code != lang.READ_TENSOR or tensor.code != lang.INPUT or aff is None:
            return None
        if x is not None and tensor is not x:
            return None
        x = tensor
        in_loop_accesses.append(aff)
    if x is None or x.dtype not in CTYPE or ITEMSIZE[x.dtype] not in (4, 8):
        return None
    shape = list(x.shape)
    rank = len(shape)
    if rank < 2 or len(info.workgroup_shape) != rank - 1:
        return None
    axis = None
    for k in range(rank - 1):
        if shape[k] == length and shape[:k] + shape[k + 1:] == list(info.workgroup_shape):
            axis = k
            break
    if axis is None:
        return None
    strides = [1] * rank
    for k in range(rank - 2, -1, -1):
        strides[k] = strides[k + 1] * shape[k + 1]
    inner = strides[axis]
    outer = 1
    for d in shape[:axis]:
        outer *= d
    sig = {}
    for j, dim in enumerate(d for d in range(rank) if d != axis):
        if info.workgroup_shape[j] > 1:
            sig[('p', j)] = strides[dim]
    sig[('v', counter)] = inner
    sig_loop = (tuple(sorted(sig.items())), 0)
    if any(aff.signature() != sig_loop for aff in in_loop_accesses):
        return None
    per = 16 // ITEMSIZE[x.dtype]
    rows_per_chunk = rows_per_chunk or 64
    batch = batch or 8
    while batch > 1 and (rows_per_chunk // per) % (2 * batch) != 0:
        batch //= 2
    if rows_per_chunk % per != 0 or (rows_per_chunk // per) % (2 * batch) != 0:
        return None
    if 3 * rows_per_chunk * STRIP * ITEMSIZE[x.dtype] > LDS_BUDGET:
        return None
    p = ColumnPlan(loop, counter, length, outer, inner, x, None, per, rows_per_chunk, batch,
                   max(2, min(int(sets or SETS), 16)))
    p.sets_forced = sets is not None
    p.reduce = True
    p.start = start
    p.end_idx = min(closers)
    from .rowscan_kernel import _carried_state
    state = _carried_state(info, p)
    if not state or any(info.nodes[idx].dtype not in CTYPE for idx in state):
        return None
    return p


def worthwhile(info, p):
    """A long enough axis: there the one-worker-per-thread template is bound by the latency of its loads."""
    strips = (p.inner + STRIP - 1) // STRIP
    return p.length >= MIN_LENGTH and p.outer * strips <= MAX_BLOCKS


def generate(info, kernel_name, rows_per_chunk=None, batch=None, sets=None, reduce=False):
    p = (reduce_plan if reduce else plan)(info, rows_per_chunk, batch, sets)
    assert p is not None
    ctype = CTYPE[p.x.dtype]
    per, rc, batch = p.per, p.rows_per_chunk, p.batch
    reads_per_chunk = rc // per
    num_chunks = (p.length + rc - 1) // rc
    strips = (p.inner + STRIP - 1) // STRIP
    items = rc * STRIP                              # elements of a chunk
    ipt = (items + MOVERS - 1) // MOVERS            # elements each mover thread handles per chunk

    # position of a line: (o, c) -> the workgroup's components (the tensor's dimensions without the scanned axis)
    shape = list(p.x.shape)
    wg = list(info.workgroup_shape)
    rank = len(wg)
    wg_strides = [1] * rank
    for k in range(rank - 2, -1, -1):
        wg_strides[k] = wg_strides[k + 1] * wg[k + 1]
    pos_exprs = []
    for k in range(rank):
        expr = 'line'
        if k > 0:
            expr = '(line % ' + str(wg_strides[k - 1]) + 'u)'
        pos_exprs.append(expr + ' / ' + str(wg_strides[k]) + 'u')

    if p.reduce:
        # only the reads inside the loop come out of the tile; what stands before and after the loop is ordinary code
        emitter = BodyEmitter(info, pos_exprs,
                              read_hook=lambda node, tensor, idx: 'OVL_SCAN_IN' if info.in_loop[node.idx] else None,
                              store_hook=None)
    else:
        emitter = BodyEmitter(info, pos_exprs,
                              read_hook=lambda node, tensor, idx: 'OVL_SCAN_IN',
                              store_hook=lambda node, tensor, idx, value: 'OVL_SCAN_OUT(' + value + ');')
    tagged = emitter.emit_tagged()
    range_idx = p.loop_item.node
    end_idx = p.end_idx if p.reduce else max(i for i, _ in tagged)
    prologue = [t for i, t in tagged if i < range_idx]
    body = [t.strip() for i, t in tagged if range_idx < i < end_idx]
    epilogue = [t.strip() for i, t in tagged if i > end_idx]
    counter_name = 'e' + str(p.counter)
    counter_type = CTYPE[info.nodes[p.counter].dtype]

    vname = 'ovl_scan_vec'
    src = []
    a = src.append
    a('typedef %s %s __attribute__((ext_vector_type(%d)));' % (ctype, vname, per))
    a('struct ovl_scan_yes { static constexpr bool value = true; };')
    a('struct ovl_scan_no { static constexpr bool value = false; };')
    a('')
    a('extern "C" __global__ void __launch_bounds__(%d)' % BLOCK)
    if p.reduce:
        args = ['const %s* __restrict__ in%d' % (CTYPE[info.inputs[i].dtype], i) for i in range(len(info.inputs))]
        args += ['%s* __restrict__ out%d' % (CTYPE[info.outputs[i].dtype], i) for i in range(len(info.outputs))]
        a('%s(%s) {' % (kernel_name, ', '.join(args)))
    else:
        a('%s(const %s* __restrict__ in%d, %s* __restrict__ out%d) {' % (
            kernel_name, ctype, p.x.io_index, ctype, p.out.io_index))
    if info.uses_math_tables():
        a('    OVL_DECLARE_MATH_TABLES();')
    a('    // tile[buffer][rows / %d][line]: the %d consecutive rows of one line are one 128-bit word' % (per, per))
    a('    __shared__ __attribute__((aligned(16))) %s tile[3][%d][%d];' % (vname, reads_per_chunk, STRIP))
    a('    const uint32_t strip = blockIdx.x %% %du;' % strips)
    a('    const uint32_t o = blockIdx.x / %du;                 // index over the dimensions before the scanned axis' % strips)
    a('    const uint32_t c0 = strip * %du;                      // first line of the strip within its row' % STRIP)
    a('    const uint32_t lane = threadIdx.x %% %du;' % WAVE)
    a('    const uint64_t obase = (uint64_t)o * %dull + c0;      // element of row 0, first line of the strip' % (
        p.length * p.inner))
    a('    const %s* __restrict__ gin = in%d + obase;' % (ctype, p.x.io_index))
    if not p.reduce:
        a('    %s* __restrict__ gout = out%d + obase;' % (ctype, p.out.io_index))
    a('')
    a('    // Movers (threads 64 and up): a thread owns up to %d elements of each chunk, one row of the strip per' % ipt)
    a('    // wavefront and instruction (a wavefront covering %d rows of %d lines would write LDS without bank conflicts but' % (per, STRIP // per))
    a('    // was slower: float32 [10000, 1000] 258 us against 117 us).  An element that does not exist is redirected to')
    a('    // the strip\'s first element for loading and skipped when writing, so the loops are branch free.')
    a('    struct MoverRegs { %s v[%d]; };' % (ctype, ipt))
    a('    auto slot = [&](uint32_t k, uint32_t m, uint32_t i, uint32_t& r, uint32_t& c) -> bool {')
    a('        const uint32_t e = m + i * %du;' % MOVERS)
    a('        r = e / %du; c = e %% %du;' % (STRIP, STRIP))
    a('        return e < %du && k * %du + r < %du && c0 + c < %du;' % (items, rc, p.length, p.inner))
    a('    };')
    a('    auto issue_loads = [&](uint32_t k, uint32_t m, MoverRegs& regs) {')
    a('        #pragma unroll')
    a('        for (uint32_t i = 0; i < %du; ++i) {' % ipt)
    a('            uint32_t r, c;')
    a('            const bool real = slot(k, m, i, r, c);')
    a('            const uint64_t g = real ? (uint64_t)(k * %du + r) * %dull + c : 0ull;' % (rc, p.inner))
    a('            regs.v[i] = gin[g];')
    a('        }')
    a('    };')
    a('    auto lds_word = [&](uint32_t k, uint32_t r, uint32_t c) -> %s* {' % ctype)
    a('        return reinterpret_cast<%s*>(&tile[k %% 3u][r / %du][c]) + (r %% %du);' % (ctype, per, per))
    a('    };')
    a('    auto write_lds = [&](uint32_t k, uint32_t m, const MoverRegs& regs) {')
    a('        #pragma unroll')
    a('        for (uint32_t i = 0; i < %du; ++i) {' % ipt)
    a('            uint32_t r, c;')
    a('            if (slot(k, m, i, r, c)) *lds_word(k, r, c) = regs.v[i];')
    a('        }')
    a('    };')
    if not p.reduce:
        a('    auto store_chunk = [&](uint32_t k, uint32_t m) {')
        a('        #pragma unroll')
        a('        for (uint32_t i = 0; i < %du; ++i) {' % ipt)
        a('            uint32_t r, c;')
        a('            if (slot(k, m, i, r, c))')
        a('                __builtin_nontemporal_store(*lds_word(k, r, c), gout + (uint64_t)(k * %du + r) * %dull + c);' % (
            rc, p.inner))
        a('        }')
        a('    };')
    a('')
    sets = min(p.sets, max(2, num_chunks))
    if not p.sets_forced:
        # float64 [10000, 1000]: 8 sets spill (322 us), 4 sets 191 us
        sets = max(2, min(sets, SET_REGISTERS // (ipt * (ITEMSIZE[p.x.dtype] // 4))))
    a('    if (threadIdx.x >= %du) {' % WAVE)
    _emit_movers(a, sets, num_chunks, stores=not p.reduce)
    a('    } else {')
    a('        // The scanning wavefront: lane = line c0 + lane of the strip; a lane past the last line shadows it.')
    a('        const uint32_t c = (c0 + lane < %du) ? lane : %du - c0;' % (p.inner, p.inner - 1))
    a('        const uint32_t line = o * %du + c0 + c;' % p.inner)
    if p.reduce:
        a('        // the statements the worker runs before its loop')
        for stmt in prologue:
            a('        ' + stmt)
    else:
        a('        // first row: the statements the worker runs before its loop')
        a('        %s first_out;' % ctype)
        a('#define OVL_SCAN_IN (gin[c])')
        a('#define OVL_SCAN_OUT(value) first_out = (value)')
        for stmt in prologue:
            a('        ' + stmt)
        a('#undef OVL_SCAN_IN')
        a('#undef OVL_SCAN_OUT')
    a('#define OVL_SCAN_IN xv[u]')
    a('#define OVL_SCAN_OUT(value) xv[u] = (value)')
    a('#define OVL_SCAN_STEP(row) { %s = (%s)(row); %s }' % (counter_name, counter_type, ' '.join(body)))
    a('        %s set_a[%d], set_b[%d];' % (vname, batch, batch))
    a('        auto fetch = [&](%s (&set)[%d], const %s* from) {' % (vname, batch, vname))
    a('            #pragma unroll')
    a('            for (uint32_t v = 0; v < %du; ++v) set[v] = from[v * %du];' % (batch, STRIP))
    a('        };')
    a('        auto put_back = [&](const %s (&set)[%d], %s* to) {' % (vname, batch, vname))
    a('            #pragma unroll')
    a('            for (uint32_t v = 0; v < %du; ++v) to[v * %du] = set[v];' % (batch, STRIP))
    a('        };')
    a('        // the recurrence over one register set; the tensor\'s first row was done above')
    a('        auto run = [&](%s (&set)[%d], uint32_t row0, bool first, auto last_chunk) {' % (vname, batch))
    a('            #pragma unroll')
    a('            for (uint32_t v = 0; v < %du; ++v) {' % batch)
    a('                %s& xv = set[v];' % vname)
    a('                #pragma unroll')
    a('                for (uint32_t u = 0; u < %du; ++u) {' % per)
    if p.reduce:
        # (rows past the last one of the tensor hold copies of other rows: they must not reach the state; only the
        # last chunk has such rows, so only its instantiation tests for them)
        skip_first = 'v == 0u && u == 0u && first' if p.start == 1 else 'false'
        in_tensor = 'true' if p.length % rc == 0 else \
            '(!decltype(last_chunk)::value || row0 + v * %du + u < %du)' % (per, p.length)
        a('                    if (!(%s) && %s) OVL_SCAN_STEP(row0 + v * %du + u)' % (skip_first, in_tensor, per))
    else:
        a('                    if (v == 0u && u == 0u && first) xv[0] = first_out;')
        a('                    else OVL_SCAN_STEP(row0 + v * %du + u)' % per)
    a('                }')
    a('            }')
    a('        };')
    a('        __syncthreads();')
    a('        auto chunk = [&](uint32_t k, auto last_chunk) {')
    # (a reduction's lanes past the last line store what its owner stores: they read the owner's rows too)
    a('            %s* colp = &tile[k %% 3u][0][%s];' % (vname, 'c' if p.reduce else 'lane'))
    a('            fetch(set_a, colp);')
    a('            #pragma unroll 1')
    a('            for (uint32_t q = 0; q < %du; q += %du) {' % (reads_per_chunk, 2 * batch))
    a('                fetch(set_b, colp + (q + %du) * %du);' % (batch, STRIP))
    a('                run(set_a, k * %du + q * %du, k == 0u && q == 0u, last_chunk);' % (rc, per))
    if not p.reduce:
        a('                put_back(set_a, colp + q * %du);' % STRIP)
    a('                if (q + %du < %du) fetch(set_a, colp + (q + %du) * %du);' % (2 * batch, reads_per_chunk, 2 * batch, STRIP))
    a('                run(set_b, k * %du + (q + %du) * %du, false, last_chunk);' % (rc, batch, per))
    if not p.reduce:
        a('                put_back(set_b, colp + (q + %du) * %du);' % (batch, STRIP))
    a('            }')
    a('            __syncthreads();')
    a('        };')
    a('        #pragma unroll 1')
    a('        for (uint32_t k = 0; k < %du; ++k) chunk(k, ovl_scan_no());' % (num_chunks - 1))
    a('        chunk(%du, ovl_scan_yes());' % (num_chunks - 1))
    if p.reduce:
        a('        // the statements after the worker\'s loop, once per line')
        for stmt in epilogue:
            a('        ' + stmt)
    a('#undef OVL_SCAN_STEP')
    a('#undef OVL_SCAN_IN')
    a('#undef OVL_SCAN_OUT')
    a('    }')
    a('}')

    itemsize = ITEMSIZE[p.x.dtype]
    launch = {
        'template': 'colreduce' if p.reduce else 'colscan',
        'vec': 1,
        'block': BLOCK,
        'blocks_needed': p.outer * strips,
        'align': {('in', p.x.io_index): itemsize} if p.reduce else
                 {('in', p.x.io_index): itemsize, ('out', p.out.io_index): itemsize},
        'vector_loads': 1,
        'vector_stores': 1,
    }
    return '\n'.join(src) + '\n', launch


def _emit_movers(a, sets, num_chunks, stores=True):
    a('        const uint32_t m = threadIdx.x - %du;' % WAVE)
    a('        // %d register sets keep %d chunks of loads in flight: chunk j travels through set j %% %d, is requested' % (
        sets, sets, sets))
    a('        // %d steps before it is written to LDS (or before the first step), and is written one step before the' % sets)
    a('        // scanning wavefront needs it.')
    a('        MoverRegs sets[%d];' % sets)
    for j in range(min(sets, num_chunks)):
        a('        issue_loads(%du, m, sets[%d]);' % (j, j))
    a('        write_lds(0u, m, sets[0]);')
    if sets < num_chunks:
        a('        issue_loads(%du, m, sets[0]);' % sets)
    a('        __syncthreads();')
    a('        // step k: chunk k is being scanned; chunk k + 1 goes to LDS, its set is refilled, chunk k - 1 goes out')
    a('        auto step = [&](uint32_t k, MoverRegs& regs) {')
    a('            if (k + 1u < %du) write_lds(k + 1u, m, regs);' % num_chunks)
    a('            if (k + 1u + %du < %du) issue_loads(k + 1u + %du, m, regs);' % (sets, num_chunks, sets))
    if stores:
        a('            if (k >= 1u) store_chunk(k - 1u, m);')
    a('            __syncthreads();')
    a('        };')
    full = num_chunks // sets
    if full:
        a('        #pragma unroll 1')
        a('        for (uint32_t k0 = 0; k0 < %du; k0 += %du) {' % (full * sets, sets))
        for d in range(sets):
            a('            step(k0 + %du, sets[%d]);' % (d, (d + 1) % sets))
        a('        }')
    for k in range(full * sets, num_chunks):
        a('        step(%du, sets[%d]);' % (k, (k + 1) % sets))
    if stores:
        a('        store_chunk(%du, m);' % (num_chunks - 1))


# ---------------------------------------------------------------------------------------------------------------------
# The lane-skewed column scan: every wavefront of the workgroup scans.
#
# In the kernel above one wavefront runs the recurrence for the 64 lines of a strip, one LDS access per two or four
# rows, and sets the pace: about 45 clocks per row.  A tensor with few lines has few strips, and the order-preserving
# recurrence leaves no other parallelism between rows.  But a wavefront need not own 64 lines: here a wavefront owns
# four lines, sixteen lanes per line, and the rows of a chunk are spread over the sixteen lanes of a line as in the
# lane-skewed row scans (rowscan_kernel.py): lane `part` owns SEG consecutive rows, runs the recurrence over them from
# the state it holds and hands its final state to its right neighbour; after sixteen such phases the chunk is exact.
# A chunk of 16 * SEG rows then costs a wavefront sixteen times (SEG steps + one hand-over), and a workgroup is a strip
# of 8 to 64 lines (2 to 16 wavefronts), chosen so that the tensor gives a few hundred workgroups: the instructions a
# wavefront issues are sixteen times redundant, so the gain is there only while the wavefronts have SIMDs to
# themselves (sixteen wavefronts on one CU's four SIMDs scan a strip of 64 lines no faster than the kernel above).
# Moving data: the chunks ahead are loaded into registers (row-major, sixteen lanes read neighbouring lines of one
# row), written transposed into LDS (line-major, so that a lane's rows are adjacent, whole 128-bit words), and after
# the scan the results are read back and stored.  In strips of 16 lines and more the scanning wavefronts do this
# themselves between two chunks (two LDS buffers alternate, two barriers per chunk).  The narrowest strips belong to
# tensors with few lines, where most SIMDs are idle and the time is the length of one wavefront's instruction stream:
# there four more wavefronts of the workgroup do nothing but move data through three rotating buffers (one barrier per
# chunk) and the scanning wavefronts only read their segments, run the recurrence and write them back (float64
# [10000, 1000] 58 -> 40 us, float32 47 -> 33 us, float64 [5000, 300] 32 -> 23 us; in strips of 16 lines the extra
# wavefronts lose: float64 [4096, 4096] 41 -> 45 us).  For 8-byte elements the scanning wavefronts of those strips do
# not write results either: they publish the state that enters each lane's segment and as many finishing wavefronts
# recompute the segments (six buffers; see `generate_skewed`).  Strips narrower than a cache line are placed on the
# XCDs so that the strips that share lines share an L2.  With all of it float64 [10000, 1000] takes 36 us; a kernel
# that only copies the tensor in the same strips takes 31 us (`ovl_strip_copy_f64`, csrc/ovl_scan.hip), and the
# scanning wavefront's own instruction stream 23.5 us (sixteen phases of sixteen dependent float64 additions and a
# hand-over: 5.6 clocks per row).
# ---------------------------------------------------------------------------------------------------------------------
SKEW_GROUP = 16                 # lanes per line
SKEW_SEG_VECTORS = 2            # 128-bit vectors a lane owns per phase (32 bytes: 4 float64 or 8 float32 rows)
SKEW_SEG_VECTORS_NARROW = 8     # ... in strips of 8 lines
SKEW_SETS = 8                   # chunks of loads in flight per workgroup
SKEW_MOVERS = 256               # threads that only move data, in strips of at most ...
SKEW_MOVERS_MAX_STRIP = 8       # ... this many lines (128, 256 and 512 threads measured the same)


#: with more lines than this the strips of 64 lines of the kernel above already give every CU several workgroups
SKEW_MAX_LINES = 1 << 15


def skew_strip(info, p):
    """Lines per workgroup of the lane-skewed column scan: a power of two between 8 and 64 that gives about 256
    workgroups.  Measured on MI355X with every wavefront moving data, 32-byte segments and eight register sets,
    microseconds with strips of 4 / 8 / 16 / 32 / 64 lines (and the kernel above):
    float64 [10000, 1000] 85 / 79 / 91 / 141 / 257 (191); float32 [10000, 1000] 82 / 56 / 61 / 72 / 120 (117);
    float64 [5000, 300] 41 / 42 / 48 / 74 / 131 (97); float64 [4096, 4096] 177 / 70 / 41 / 61 / 108 (82);
    float32 [4096, 8192] 356 / 195 / 66 / 46 / 54 (77); float32 [1000, 16384] 182 / 105 / 36 / 26 / 23 (31);
    float64 [1000, 16384] 193 / 67 / 46 / 46 / 50 (43)."""
    lines = p.outer * p.inner
    strip = 8
    while strip < 64 and lines > 256 * strip:
        strip *= 2
    return strip


def prefers_skew(info, p):
    """Few enough lines that the lane-skewed kernel's small strips pay (see `skew_strip`)."""
    from .rowscan_kernel import _carried_state
    if p.outer * p.inner > SKEW_MAX_LINES:
        return False
    return all(info.nodes[idx].dtype in CTYPE for idx in _carried_state(info, p))


def generate_skewed(info, kernel_name, sets=None, strip=None, seg_vectors=None, movers=None, reduce=False, carry=None,
                    nt=None):
    from .rowscan_kernel import _carried_state
    p = (reduce_plan if reduce else plan)(info)
    assert p is not None
    STRIP = strip or skew_strip(info, p)            # lines per workgroup
    SCAN_THREADS = STRIP * SKEW_GROUP               # sixteen lanes per line
    ctype = CTYPE[p.x.dtype]
    per = p.per
    narrow = STRIP <= 8
    if seg_vectors is None:
        # the narrowest strips are chosen for tensors with few lines, whose time is the latency of the recurrence:
        # there a lane owns 128 bytes of rows, so that a hand-over is paid once per 16 (32) steps (float64
        # [10000, 1000] without separate movers: 79 us with 32 bytes, 65 with 64, 59 with 128; with wider strips the
        # longer segments lose: float64 [4096, 4096] 41 -> 45 us)
        seg_vectors = SKEW_SEG_VECTORS_NARROW if narrow else SKEW_SEG_VECTORS
    seg = seg_vectors * per                         # rows a lane owns per phase
    rc = SKEW_GROUP * seg                           # rows per chunk
    if movers is None:
        movers = SKEW_MOVERS if STRIP <= SKEW_MOVERS_MAX_STRIP else 0
    if movers and (movers % WAVE or movers % STRIP or (rc // per) % (movers // STRIP) or
                   SCAN_THREADS + movers > 1024):
        movers = 0
    if sets is None:
        # chunks of loads in flight.  With separate movers two are enough and more lose (float32 [10000, 1000]: 33 us
        # with two, 37 with four, 55 with eight: neighbouring strips share the cache lines of a row, and the further
        # the workgroups run ahead of each other the more often a line is fetched twice); without them the narrow
        # strips take four
        sets = 2 if movers else 4 if narrow else SKEW_SETS
    # With separate movers, a scan (not a reduction) of 8-byte elements also takes its results off the scanning
    # wavefronts: they keep none, publish the exact state that enters each lane's segment, and as many finishing
    # wavefronts recompute the segments from those states and write them to LDS (see `rowscan_kernel.generate_carry`:
    # a 128-bit LDS write costs the wavefront that issues it five steps of a float64 recurrence).  The scanning
    # wavefronts then also read the next chunk's segments during the phases of the current one.  Measured: float64
    # [10000, 1000] along axis 0 41.4 -> 38.5 us, [5000, 300] 23.5 -> 21.6; float32 [10000, 1000] 33.9 -> 34.3 (not
    # chosen there).  What is left is moving the data: a kernel that only copies the tensor in the same strips (one
    # workgroup per 8 lines, 64 bytes of every row) takes 36 us, one that only loads it 24 us; 16 lines per workgroup
    # copy in 45 us on half as many compute units and 4 lines (32 bytes per row) in 86 us.
    if carry is None:
        carry = per == 2
    carry = bool(carry and movers and not p.reduce and seg_vectors in (1, 2, 4, 8, 16, 32))
    FINISH_THREADS = SCAN_THREADS if carry else 0
    BLOCK = SCAN_THREADS + FINISH_THREADS + movers
    if BLOCK > 1024:
        carry, FINISH_THREADS, BLOCK = False, 0, SCAN_THREADS + movers
    MOVE = movers or BLOCK                          # threads that move data
    NBUF = 6 if carry else 3 if movers else 2
    seg_stride = seg + per                          # a segment and its padding vector (bank conflicts)
    line_stride = SKEW_GROUP * seg_stride + per     # a line and its padding vector
    num_chunks = (p.length + rc - 1) // rc
    strips = (p.inner + STRIP - 1) // STRIP
    rows_per_pass = MOVE // STRIP                   # vectors of a line covered by one load instruction of the movers
    ipt = rc // rows_per_pass                       # elements each thread moves per chunk
    vpt = ipt // per                                # ... as 128-bit vectors of consecutive rows of one line
    sets = max(2, min(int(sets or SKEW_SETS), 16, max(2, num_chunks)))
    lines_per_wave = WAVE // SKEW_GROUP

    wg = list(info.workgroup_shape)
    rank = len(wg)
    wg_strides = [1] * rank
    for k in range(rank - 2, -1, -1):
        wg_strides[k] = wg_strides[k + 1] * wg[k + 1]
    pos_exprs = []
    for k in range(rank):
        expr = 'line'
        if k > 0:
            expr = '(line % ' + str(wg_strides[k - 1]) + 'u)'
        pos_exprs.append(expr + ' / ' + str(wg_strides[k]) + 'u')
    if p.reduce:
        # only the reads inside the loop come out of the tile; what stands before and after the loop is ordinary code
        emitter = BodyEmitter(info, pos_exprs,
                              read_hook=lambda node, tensor, idx: 'OVL_SCAN_IN' if info.in_loop[node.idx] else None,
                              store_hook=None)
    else:
        emitter = BodyEmitter(info, pos_exprs,
                              read_hook=lambda node, tensor, idx: 'OVL_SCAN_IN',
                              store_hook=lambda node, tensor, idx, value: 'OVL_SCAN_OUT(' + value + ');')
    tagged = emitter.emit_tagged()
    range_idx = p.loop_item.node
    end_idx = p.end_idx if p.reduce else max(i for i, _ in tagged)
    prologue = [t for i, t in tagged if i < range_idx]
    body = [t.strip() for i, t in tagged if range_idx < i < end_idx]
    epilogue = [t.strip() for i, t in tagged if i > end_idx]
    counter_name = 'e' + str(p.counter)
    counter_type = CTYPE[info.nodes[p.counter].dtype]
    state = [('e' + str(idx), CTYPE[info.nodes[idx].dtype]) for idx in _carried_state(info, p)]

    vname = 'ovl_scan_vec'
    src = []
    a = src.append
    a('typedef %s %s __attribute__((ext_vector_type(%d)));' % (ctype, vname, per))
    a('struct ovl_scan_yes { static constexpr bool value = true; };')
    a('struct ovl_scan_no { static constexpr bool value = false; };')
    a('')
    a('extern "C" __global__ void __launch_bounds__(%d)' % BLOCK)
    if p.reduce:
        args = ['const %s* __restrict__ in%d' % (CTYPE[info.inputs[i].dtype], i) for i in range(len(info.inputs))]
        args += ['%s* __restrict__ out%d' % (CTYPE[info.outputs[i].dtype], i) for i in range(len(info.outputs))]
        a('%s(%s) {' % (kernel_name, ', '.join(args)))
    else:
        a('%s(const %s* __restrict__ in%d, %s* __restrict__ out%d) {' % (
            kernel_name, ctype, p.x.io_index, ctype, p.out.io_index))
    if info.uses_math_tables():
        a('    OVL_DECLARE_MATH_TABLES();')
    a('    // tile[buffer][line][row]: a line holds the %d rows of a chunk as 16 segments of %d rows, each followed by one' % (rc, seg))
    a('    // spare vector, and one more at its end')
    a('    __shared__ __attribute__((aligned(16))) %s tile[%d][%d][%d];' % (ctype, NBUF, STRIP, line_stride))
    if carry:
        for name, stype in state:
            a('    __shared__ %s entering_%s[%d][%d];' % (stype, name, NBUF, SCAN_THREADS))
    # A strip narrower than a 128-byte line shares the lines of every row with its neighbours.  Workgroups go to the
    # eight XCDs (each with its own L2) in turn, so the strips that share lines are given to workgroups a multiple of
    # 8 apart: they run on one XCD at the same time and a line is fetched from memory once.
    #  * Row pitch a multiple of 128 bytes: the same 128 / (strip bytes) strips share a line in every row; they go to
    #    one XCD, the next such group to the next XCD (the pieces an XCD reads are spread over the whole row).
    #  * Any other pitch: which neighbours share depends on the row (float64 rows of 1000 columns: even rows pair a
    #    strip with one side, odd rows with the other), so every XCD is given one contiguous range of strips.  float64
    #    [10000, 1000] in strips of 8 lines reads its input 2.0 times with neighbouring strips on neighbouring XCDs,
    #    1.55 times with pairs of strips per XCD, 1.07 times with ranges (38.5 -> 37.5 us; float32 34 -> 31 us).
    #    (With a pitch that is a multiple of 128 bytes ranges lose: an XCD then reads one narrow column of the tensor
    #    at a power-of-two pitch; float32 [4096, 2048] 18 -> 23 us.)
    share = max(1, 128 // (STRIP * ITEMSIZE[p.x.dtype]))
    total = p.outer * strips
    if share > 1 and (p.inner * ITEMSIZE[p.x.dtype]) % 128 == 0 and total >= 8 * share:
        whole = total // (8 * share) * (8 * share)
        a('    // workgroups b, b + 8, ... (one XCD) take the %d neighbouring strips that share the cache lines of every row' % share)
        a('    const uint32_t wg = blockIdx.x < %du' % whole)
        a('        ? blockIdx.x / %du * %du + blockIdx.x %% 8u * %du + blockIdx.x / 8u %% %du : blockIdx.x;' % (
            8 * share, 8 * share, share, share))
    elif share > 1 and total >= 16:
        q, r = divmod(total, 8)
        a('    // workgroups b, b + 8, b + 16, ... (one XCD) take a contiguous range of strips, which share cache lines')
        a('    const uint32_t xcd = blockIdx.x % 8u, slot = blockIdx.x / 8u;')
        a('    const uint32_t wg = xcd * %du + (xcd < %du ? xcd : %du) + slot;' % (q, r, r))
    else:
        a('    const uint32_t wg = blockIdx.x;')
    if nt is None:
        # Stores carry the non-temporal hint (the results are not read again), except where the same neighbouring strips
        # share every line: there plain stores let the L2 put a line's parts together before it is written back
        # (float64 [4096, 2048]: 29.0 -> 24.7 us).  Where the sharing neighbours change from row to row plain stores
        # bring the written bytes from 1.25 times the tensor to 1.0 but take 1 us longer (float64 [10000, 1000]:
        # 37.7 -> 38.9 us), so the hint stays.
        nt = '' if share > 1 and (p.inner * ITEMSIZE[p.x.dtype]) % 128 == 0 else 's'
    if not p.reduce:
        if 's' in nt:
            a('#define OVL_SCAN_STORE(value, address) __builtin_nontemporal_store(value, address)')
        else:
            a('#define OVL_SCAN_STORE(value, address) (*(address) = (value))')
    a('    const uint32_t strip = wg %% %du;' % strips)
    a('    const uint32_t o = wg / %du;                         // index over the dimensions before the scanned axis' % strips)
    a('    const uint32_t c0 = strip * %du;                      // first line of the strip within its row' % STRIP)
    a('    const uint64_t obase = (uint64_t)o * %dull + c0;      // element of row 0, first line of the strip' % (
        p.length * p.inner))
    a('    const %s* __restrict__ gin = in%d + obase;' % (ctype, p.x.io_index))
    if not p.reduce:
        a('    %s* __restrict__ gout = out%d + obase;' % (ctype, p.out.io_index))
    a('')
    if carry:
        # (A compute unit places the wavefronts of a workgroup on its four SIMDs in turn, wavefronts w and w + 4 share
        # one.  Which roles share a SIMD made no difference to the time: scanning with finishing, scanning with
        # moving, or the scanning wavefronts alone beside two wavefronts of movers.)
        a('    // Threads 0..%d scan, %d..%d finish, %d and up move data.' % (
            SCAN_THREADS - 1, SCAN_THREADS, SCAN_THREADS + FINISH_THREADS - 1, SCAN_THREADS + FINISH_THREADS))
        a('    const uint32_t vt = threadIdx.x;')
        a('    const bool is_mover = vt >= %du;' % (SCAN_THREADS + FINISH_THREADS))
        a('    const uint32_t mt = vt - %du;' % (SCAN_THREADS + FINISH_THREADS))
    elif movers:
        a('    // Threads %d and up move data, the others scan.' % SCAN_THREADS)
        a('    const bool is_mover = threadIdx.x >= %du;' % SCAN_THREADS)
        a('    const uint32_t mt = threadIdx.x - %du;' % SCAN_THREADS)
    else:
        a('    const uint32_t mt = threadIdx.x;')
    a('    // Moving data: thread mt owns line mt %% %d of vectors mt / %d, mt / %d + %d, ... of every chunk (%d elements).' % (
        STRIP, STRIP, STRIP, rows_per_pass, ipt))
    a('    // An element that does not exist (past the last row, past the last line) is replaced by the nearest one that')
    a('    // does: it is loaded, and later stored, a second time with the same value.  Without conditions around the')
    a('    // memory instructions the compiler can count them, and waits for the loads of exactly the chunk it needs while')
    a('    // those of the chunks after it stay in flight (with conditional stores it waited for all but the last dozen')
    a('    // requests: float64 [10000, 1000] 264 us).')
    a('    const uint32_t lines_here = (%du - c0 < %du) ? %du - c0 : %du;' % (p.inner, STRIP, p.inner, STRIP))
    a('    const uint32_t mc = (mt %% %du < lines_here) ? mt %% %du : lines_here - 1u;' % (STRIP, STRIP))
    a('    const uint32_t mv = mt / %du;                        // first of the vectors (%d consecutive rows) the thread owns' % (
        STRIP, per))
    a('    struct MoverRegs { %s v[%d]; };' % (vname, vpt))
    a('    auto chunk_row = [&](uint32_t k, uint32_t i, uint32_t u) -> uint32_t {     // clamped to the chunk\'s last row')
    a('        const uint32_t r = (mv + i * %du) * %du + u;' % (rows_per_pass, per))
    a('        const uint32_t rows_here = (%du - k * %du < %du) ? %du - k * %du : %du;' % (
        p.length, rc, rc, p.length, rc, rc))
    a('        return r < rows_here ? r : rows_here - 1u;')
    a('    };')
    a('    // (a thread writes and reads whole 128-bit words of LDS: lanes on neighbouring lines are %d words apart, an odd' % (
        line_stride // per))
    a('    // number, so eight of them cover all banks; 64-bit accesses at that stride ran into 8-way conflicts: 257 us)')
    a('    auto lds_at = [&](uint32_t k, uint32_t i) -> %s* {' % vname)
    a('        const uint32_t r = (mv + i * %du) * %du;' % (rows_per_pass, per))
    a('        return reinterpret_cast<%s*>(&tile[k %% %du][mc][(r / %du) * %du + r %% %du]);' % (vname, NBUF, seg, seg_stride, seg))
    a('    };')
    a('    auto issue_loads = [&](uint32_t k, MoverRegs& regs) {')
    a('        #pragma unroll')
    a('        for (uint32_t i = 0; i < %du; ++i) {' % vpt)
    a('            #pragma unroll')
    a('            for (uint32_t u = 0; u < %du; ++u)' % per)
    a('                regs.v[i][u] = gin[(uint64_t)(k * %du + chunk_row(k, i, u)) * %dull + mc];' % (rc, p.inner))
    a('        }')
    a('    };')
    a('    auto write_lds = [&](uint32_t k, const MoverRegs& regs) {')
    a('        #pragma unroll')
    a('        for (uint32_t i = 0; i < %du; ++i) *lds_at(k, i) = regs.v[i];' % vpt)
    a('    };')
    # The same for a chunk all of whose rows exist (every chunk but the last), without the clamps: byte offsets and
    # LDS positions of a thread's elements are computed once, a chunk's base address is uniform.  (With the clamps and
    # the 64-bit index arithmetic per element a moving wavefront issued some 250 vector instructions per chunk; a
    # wavefront that shares a SIMD with a scanning one costs it about four clocks per instruction.)
    a('    uint32_t element_offset[%d], lds_offset[%d];' % (vpt * per, vpt))
    a('    #pragma unroll')
    a('    for (uint32_t i = 0; i < %du; ++i) {' % vpt)
    a('        const uint32_t r = (mv + i * %du) * %du;' % (rows_per_pass, per))
    a('        lds_offset[i] = mc * %du + (r / %du) * %du + r %% %du;' % (line_stride, seg, seg_stride, seg))
    a('        #pragma unroll')
    a('        for (uint32_t u = 0; u < %du; ++u) element_offset[i * %du + u] = ((r + u) * %du + mc) * %du;' % (
        per, per, p.inner, ITEMSIZE[p.x.dtype]))
    a('    }')
    a('    auto issue_loads_full = [&](uint32_t k, MoverRegs& regs) {')
    a('        const char* base = reinterpret_cast<const char*>(gin + (uint64_t)k * %dull);' % (rc * p.inner))
    a('        #pragma unroll')
    a('        for (uint32_t i = 0; i < %du; ++i) {' % vpt)
    a('            #pragma unroll')
    a('            for (uint32_t u = 0; u < %du; ++u)' % per)
    a('                regs.v[i][u] = *reinterpret_cast<const %s*>(base + element_offset[i * %du + u]);' % (ctype, per))
    a('        }')
    a('    };')
    if not p.reduce:
        a('    auto store_chunk_full = [&](uint32_t k) {')
        a('        const %s* buffer = &tile[k %% %du][0][0];' % (ctype, NBUF))
        a('        char* base = reinterpret_cast<char*>(gout + (uint64_t)k * %dull);' % (rc * p.inner))
        a('        MoverRegs regs;')
        a('        #pragma unroll')
        a('        for (uint32_t i = 0; i < %du; ++i) regs.v[i] = *reinterpret_cast<const %s*>(buffer + lds_offset[i]);' % (
            vpt, vname))
        a('        #pragma unroll')
        a('        for (uint32_t i = 0; i < %du; ++i) {' % vpt)
        a('            #pragma unroll')
        a('            for (uint32_t u = 0; u < %du; ++u)' % per)
        a('                OVL_SCAN_STORE(regs.v[i][u], reinterpret_cast<%s*>(base + element_offset[i * %du + u]));' % (
            ctype, per))
        a('        }')
        a('    };')
    else:
        a('    auto store_chunk_full = [&](uint32_t) {};')
    if p.reduce:
        a('    auto store_chunk = [&](uint32_t) {};      // a reduction stores nothing per row')
    else:
        a('    auto store_chunk = [&](uint32_t k) {')
        a('        // (a row past the chunk\'s last one is stored as that last row once more: its value comes from the word that')
        a('        // holds the last row)')
        a('        const uint32_t last = ((%du - k * %du < %du) ? %du - k * %du : %du) - 1u;' % (
            p.length, rc, rc, p.length, rc, rc))
        a('        MoverRegs regs;')
        a('        #pragma unroll')
        a('        for (uint32_t i = 0; i < %du; ++i) {' % vpt)
        a('            const uint32_t word = mv + i * %du;' % rows_per_pass)
        a('            const uint32_t r = (word < last / %du ? word : last / %du) * %du;' % (per, per, per))
        a('            regs.v[i] = *reinterpret_cast<const %s*>(&tile[k %% %du][mc][(r / %du) * %du + r %% %du]);' % (
            vname, NBUF, seg, seg_stride, seg))
        a('        }')
        a('        #pragma unroll')
        a('        for (uint32_t i = 0; i < %du; ++i) {' % vpt)
        a('            %s of_last = regs.v[i][0];' % ctype)
        a('            #pragma unroll')
        a('            for (uint32_t u = 1; u < %du; ++u) of_last = (last %% %du == u) ? regs.v[i][u] : of_last;' % (per, per))
        a('            #pragma unroll')
        a('            for (uint32_t u = 0; u < %du; ++u) {' % per)
        a('                const uint32_t r = (mv + i * %du) * %du + u;' % (rows_per_pass, per))
        a('                OVL_SCAN_STORE(r <= last ? regs.v[i][u] : of_last,')
        a('                               gout + (uint64_t)(k * %du + (r <= last ? r : last)) * %dull + mc);' % (
            rc, p.inner))
        a('            }')
        a('        }')
        a('    };')
    a('')
    a('    // Scanning: wavefront w owns lines %d w ... %d w + %d of the strip, sixteen lanes each; lane `part` of a line owns' % (
        lines_per_wave, lines_per_wave, lines_per_wave - 1))
    a('    // rows [part * %d, part * %d + %d) of every chunk.  A line past the last one shadows it.' % (seg, seg, seg))
    a('    const uint32_t lane = threadIdx.x %% %du;' % WAVE)
    a('    const uint32_t part = lane %% %du;' % SKEW_GROUP)
    if carry:
        a('    // scanning and finishing threads map to lines alike')
        a('    const uint32_t st = vt %% %du;' % SCAN_THREADS)
        a('    const uint32_t sl = st / %du * %du + lane / %du;      // line of the strip' % (
            WAVE, lines_per_wave, SKEW_GROUP))
    else:
        a('    const uint32_t sl = threadIdx.x / %du * %du + lane / %du;      // line of the strip' % (
            WAVE, lines_per_wave, SKEW_GROUP))
    a('    const uint32_t c = (c0 + sl < %du) ? sl : %du - c0;' % (p.inner, p.inner - 1))
    a('    const uint32_t line = o * %du + c0 + c;' % p.inner)
    if p.reduce:
        a('    // the statements the worker runs before its loop, in every lane')
        for stmt in prologue:
            a('    ' + stmt)
    else:
        a('    // first row: the statements the worker runs before its loop, in every lane')
        a('    %s first_out;' % ctype)
        a('#define OVL_SCAN_IN (gin[c])')
        a('#define OVL_SCAN_OUT(value) first_out = (value)')
        for stmt in prologue:
            a('    ' + stmt)
        a('#undef OVL_SCAN_IN')
        a('#undef OVL_SCAN_OUT')
    for name, stype in state:
        a('    %s carry_%s = %s;' % (stype, name, name))
    a('#define OVL_SCAN_IN xv[u]')
    a('#define OVL_SCAN_OUT(value) ov[w][u] = (value)')
    a('#define OVL_SCAN_STEP(row) { %s = (%s)(row); %s }' % (counter_name, counter_type, ' '.join(body)))
    a('    // one chunk: in phase p every lane runs the recurrence over its rows from the state it holds and hands its')
    a('    // final state to its right neighbour; after phase p lanes 0..p are exact')
    a('    struct Segment { %s v[%d]; };' % (vname, seg_vectors))
    a('    auto fetch_segment = [&](uint32_t k, Segment& segment) {')
    # (a reduction's lanes past the last line store what its owner stores: they read the owner's rows too)
    a('        const %s* segp = &tile[k %% %du][%s][part * %du];' % (ctype, NBUF, 'c' if p.reduce else 'sl', seg_stride))
    a('        #pragma unroll')
    a('        for (uint32_t w = 0; w < %du; ++w) segment.v[w] = *reinterpret_cast<const %s*>(segp + w * %du);' % (
        seg_vectors, vname, per))
    a('    };')
    a('    auto scan_segment = [&](uint32_t k, const Segment& segment, auto last_chunk) {')
    if not p.reduce:
        a('        %s* segp = &tile[k %% %du][sl][part * %du];' % (ctype, NBUF, seg_stride))
        a('        %s ov[%d];' % (vname, seg_vectors))
    a('        const uint32_t row0 = k * %du + part * %du;' % (rc, seg))
    a('        const bool first_row = k == 0u && part == 0u;')
    a('        #pragma unroll')
    a('        for (uint32_t phase = 0; phase < %du; ++phase) {' % SKEW_GROUP)
    for name, _ in state:
        a('            %s = carry_%s;' % (name, name))
    a('            #pragma unroll')
    a('            for (uint32_t w = 0; w < %du; ++w) {' % seg_vectors)
    a('                const %s xv = segment.v[w];' % vname)
    a('                #pragma unroll')
    a('                for (uint32_t u = 0; u < %du; ++u) {' % per)
    if p.reduce:
        # (rows past the last one of the tensor hold copies of the last: they must not reach the state.  Only the last
        # chunk has such rows, and only when the axis is not a whole number of chunks: the test stands in that chunk's
        # instantiation alone.  In every step of every chunk it cost the recurrence more than the additions did: column
        # sums float64 [10000, 1000] 34.6 -> 31.6 us, float32 29.0 -> 26.9)
        skip_first = 'w == 0u && u == 0u && first_row' if p.start == 1 else 'false'
        in_tensor = 'true' if p.length % rc == 0 else \
            '(!decltype(last_chunk)::value || row0 + w * %du + u < %du)' % (per, p.length)
        a('                    if (!(%s) && %s) OVL_SCAN_STEP(row0 + w * %du + u)' % (skip_first, in_tensor, per))
    else:
        a('                    if (w == 0u && u == 0u && first_row) ov[0][0] = first_out;')
        a('                    else OVL_SCAN_STEP(row0 + w * %du + u)' % per)
    a('                }')
    a('            }')
    for name, _ in state:
        a('            carry_%s = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry_%s, %s);' % (name, name, name))
    a('        }')
    a('        // the last lane of the line finished the chunk: its state is the carry into the next one')
    for name, _ in state:
        a('        carry_%s = ovl_dpp_move<OVL_DPP_ROW_ROR1>(carry_%s, %s);' % (name, name, name))
    if not p.reduce:
        a('        #pragma unroll')
        a('        for (uint32_t w = 0; w < %du; ++w) *reinterpret_cast<%s*>(segp + w * %du) = ov[w];' % (
            seg_vectors, vname, per))
    a('    };')
    a('    auto scan_chunk = [&](uint32_t k, auto last_chunk) {')
    a('        Segment segment;')
    a('        fetch_segment(k, segment);')
    a('        scan_segment(k, segment, last_chunk);')
    a('    };')
    a('')
    a('    // %d register sets keep %d chunks of loads in flight: chunk j travels through set j %% %d' % (sets, sets, sets))
    a('    MoverRegs sets[%d];' % sets)
    full = num_chunks // sets
    if carry:
        n = num_chunks
        read_phases = min(8, seg_vectors)              # the phases in which the next chunk's segments are read
        reads_per_phase = seg_vectors // read_phases
        a('    // Six buffers rotate, one barrier per step.  Step s: the movers bring chunk s + 2 into LDS and take the')
        a('    // results of chunk s - 3 out; the scanning wavefronts run the recurrence over chunk s and read their segments')
        a('    // of chunk s + 1 meanwhile; the finishing wavefronts recompute chunk s - 2 from the states that enter its')
        a('    // segments.  Every thread passes the same %d barriers.' % (n + 3))
        a('    if (is_mover) {')
        for j in range(2):
            a('        issue_loads%s(%du, sets[%d]);' % ('_full' if j < n - 1 else '', min(j, n - 1), j % sets))
        # chunks 0 and 1 go to LDS before the first barrier; chunks 2 .. 1 + sets are requested behind them
        a('        write_lds(0u, sets[0]);')
        if n > 1:
            a('        write_lds(1u, sets[1 %% %du]);' % sets)
        for j in range(sets):
            if 2 + j < n:
                a('        issue_loads%s(%du, sets[%d]);' % ('_full' if 2 + j < n - 1 else '', 2 + j, (2 + j) % sets))
        a('        __syncthreads();')

        def emit_step(k):
            regs = 'sets[%d]' % ((k + 2) % sets)
            if k + 2 < n:
                a('        write_lds(%du, %s);' % (k + 2, regs))
            if k + 2 + sets < n:
                a('        issue_loads%s(%du, %s);' % ('_full' if k + 2 + sets < n - 1 else '', k + 2 + sets, regs))
            if k >= 3:
                a('        store_chunk_full(%du);' % (k - 3))
            a('        __syncthreads();')
        steps = n + 2                                   # steps 0 .. n + 1
        steady_first = ((3 + sets - 1) // sets + 1) * sets      # a multiple of `sets` past the first stores
        # steps [steady_first, steady_end) do all three things, on chunks all of whose rows exist
        steady_end = max(steady_first, n - 3 - sets)
        groups = (steady_end - steady_first) // sets
        for k in range(0, min(steady_first, steps)):
            emit_step(k)
        if groups:
            a('        #pragma unroll 1')
            a('        for (uint32_t k0 = %du; k0 < %du; k0 += %du) {' % (steady_first, steady_first + groups * sets, sets))
            for d in range(sets):
                a('            write_lds(k0 + %du, sets[%d]);' % (d + 2, (steady_first + d + 2) % sets))
                a('            issue_loads_full(k0 + %du, sets[%d]);' % (d + 2 + sets, (steady_first + d + 2) % sets))
                a('            store_chunk_full(k0 + %du - 3u);' % d)
                a('            __syncthreads();')
            a('        }')
        for k in range(max(steady_first + groups * sets, min(steady_first, steps)), steps):
            emit_step(k)
        a('        store_chunk(%du);' % (n - 1))
        a('    } else if (vt < %du) {' % SCAN_THREADS)
        a('        // scanning wavefronts: no results kept; the next chunk\'s segments arrive during the first eight phases')
        a('#undef OVL_SCAN_OUT')
        a('#define OVL_SCAN_OUT(value) (void)(value)')
        a('        Segment set_a, set_b;')
        a('        __syncthreads();')
        a('        fetch_segment(0u, set_a);')
        a('        auto scan_only = [&](uint32_t k, const Segment& segment, Segment& other, auto first_chunk) {')
        a('            const %s* ahead = &tile[(k + 1u) %% %du][sl][part * %du];' % (ctype, NBUF, seg_stride))
        a('            const uint32_t row0 = k * %du + part * %du;' % (rc, seg))
        a('            #pragma unroll')
        a('            for (uint32_t phase = 0; phase < %du; ++phase) {' % SKEW_GROUP)
        for name, _ in state:
            a('                %s = carry_%s;' % (name, name))
        a('                #pragma unroll')
        a('                for (uint32_t w = 0; w < %du; ++w) {' % seg_vectors)
        a('                    const %s xv = segment.v[w];' % vname)
        a('                    #pragma unroll')
        a('                    for (uint32_t u = 0; u < %du; ++u) {' % per)
        a('                        // (the first row is what the statements before the loop computed)')
        a('                        if (decltype(first_chunk)::value && w == 0u && u == 0u) { if (part != 0u) OVL_SCAN_STEP(row0) }')
        a('                        else OVL_SCAN_STEP(row0 + w * %du + u)' % per)
        a('                    }')
        a('                }')
        for name, _ in state:
            a('                carry_%s = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry_%s, %s);' % (name, name, name))
        a('                if (phase < %du) {' % read_phases)
        a('                    #pragma unroll')
        a('                    for (uint32_t j = 0; j < %du; ++j)' % reads_per_phase)
        a('                        other.v[phase * %du + j] = *reinterpret_cast<const %s*>(ahead + (phase * %du + j) * %du);' % (
            reads_per_phase, vname, reads_per_phase, per))
        a('                }')
        a('                __builtin_amdgcn_sched_barrier(0);')
        a('                if (phase == 8u) {')
        a('                    __syncthreads();')
        a('                    __builtin_amdgcn_sched_barrier(0);')
        a('                }')
        a('            }')
        a('            // lanes 1..15 hold their left neighbour\'s exact final state, lane 0 the state that entered the chunk')
        for name, _ in state:
            a('            entering_%s[k %% %du][st] = carry_%s;' % (name, NBUF, name))
        for name, _ in state:
            a('            carry_%s = ovl_dpp_move<OVL_DPP_ROW_ROR1>(carry_%s, %s);' % (name, name, name))
        a('            __builtin_amdgcn_sched_barrier(0);')
        a('        };')
        a('        scan_only(0u, set_a, set_b, ovl_scan_yes());')
        if n > 1:
            a('        uint32_t k = 1u;')
            a('        #pragma unroll 1')
            a('        for (; k + 1u < %du; k += 2u) {' % n)
            a('            scan_only(k, set_b, set_a, ovl_scan_no());')
            a('            scan_only(k + 1u, set_a, set_b, ovl_scan_no());')
            a('        }')
            a('        if (k < %du) scan_only(k, set_b, set_a, ovl_scan_no());' % n)
        a('        __syncthreads();')
        a('        __syncthreads();')
        a('#undef OVL_SCAN_OUT')
        a('#define OVL_SCAN_OUT(value) ov[w][u] = (value)')
        a('    } else {')
        a('        // finishing wavefronts: chunk s - 2 in step s, every segment once more from the state that enters it')
        a('        __syncthreads();')
        a('        __syncthreads();')
        a('        __syncthreads();')
        a('        #pragma unroll 1')
        a('        for (uint32_t s = 2u; s <= %du; ++s) {' % (n + 1))
        a('            const uint32_t k = s - 2u;')
        a('            Segment segment;')
        a('            fetch_segment(k, segment);')
        a('            %s* segp = &tile[k %% %du][sl][part * %du];' % (ctype, NBUF, seg_stride))
        a('            %s ov[%d];' % (vname, seg_vectors))
        a('            const uint32_t row0 = k * %du + part * %du;' % (rc, seg))
        for name, _ in state:
            a('            %s = entering_%s[k %% %du][st];' % (name, name, NBUF))
        a('            #pragma unroll')
        a('            for (uint32_t w = 0; w < %du; ++w) {' % seg_vectors)
        a('                const %s xv = segment.v[w];' % vname)
        a('                #pragma unroll')
        a('                for (uint32_t u = 0; u < %du; ++u) {' % per)
        a('                    if (w == 0u && u == 0u && row0 == 0u) ov[0][0] = first_out;')
        a('                    else OVL_SCAN_STEP(row0 + w * %du + u)' % per)
        a('                }')
        a('            }')
        a('            #pragma unroll')
        a('            for (uint32_t w = 0; w < %du; ++w) *reinterpret_cast<%s*>(segp + w * %du) = ov[w];' % (
            seg_vectors, vname, per))
        a('            __syncthreads();')
        a('        }')
        a('    }')
    elif movers:
        # Three buffers rotate: while chunk k is scanned in place, the movers bring chunk k + 1 into the next buffer and
        # take the results of chunk k - 1 out of the one before; one barrier per chunk.  (A fourth buffer, the movers one
        # chunk further ahead and the scanning wavefronts reading the segments of chunk k + 1 into a second register
        # set before they start on chunk k gained 0.4 us of 40 on float64 [10000, 1000]: not kept.  Movers two to six
        # chunks ahead of a reduction's scanning wavefronts lose 0.5 to 2 us of 32, like more chunks of loads in flight:
        # workgroups that drift apart no longer meet their neighbours' lines in the L2.)
        ahead = 1
        a('    if (threadIdx.x >= %du) {' % SCAN_THREADS)
        full_tag = lambda k: '_full' if k < num_chunks - 1 else ''
        for j in range(min(sets, num_chunks)):
            a('        issue_loads%s(%du, sets[%d]);' % (full_tag(j), j, j))
        for j in range(ahead):
            if j < num_chunks:
                a('        write_lds(%du, sets[%d]);' % (j, j % sets))
                if j + sets < num_chunks:
                    a('        issue_loads%s(%du, sets[%d]);' % (full_tag(j + sets), j + sets, j % sets))
            a('        __syncthreads();')
        # Step k: chunk k + ahead goes to LDS, its register set is refilled with chunk k + ahead + sets, chunk k - 1 goes
        # out.  The steps in which all three happen run in a loop without conditions; the first steps and the last ones
        # are written out.  (With the conditions inside the loop the compiler merges the paths that skip the loads and
        # stores into its count of outstanding requests and then waits for all of them before every write to LDS.
        # On float64 [10000, 1000] both forms take 40 us, because there the scanning wavefronts set the pace; the
        # loads in flight are what keeps the movers ahead of them.)
        def emit_step(k):
            regs = 'sets[%d]' % ((k + ahead) % sets)
            if k + ahead < num_chunks:
                a('        write_lds(%du, %s);' % (k + ahead, regs))
            if k + ahead + sets < num_chunks:
                a('        issue_loads%s(%du, %s);' % (full_tag(k + ahead + sets), k + ahead + sets, regs))
            if k >= 1:
                a('        store_chunk%s(%du);' % (full_tag(k - 1), k - 1))
            a('        __syncthreads();')
        # (the loop is entered after one full round of complete steps, so that the requests outstanding at its entry are
        # those outstanding at its end: otherwise the compiler counts with the fewer of the two)
        steady_first = 1 + sets
        # steps [steady_first, steady_end) are complete, on chunks all of whose rows exist
        steady_end = max(steady_first, num_chunks - ahead - sets - 1)
        groups = (steady_end - steady_first) // sets
        for k in range(0, min(steady_first, num_chunks)):
            emit_step(k)
        if groups:
            a('        #pragma unroll 1')
            a('        for (uint32_t k0 = %du; k0 < %du; k0 += %du) {' % (steady_first, steady_first + groups * sets, sets))
            for d in range(sets):
                a('            write_lds(k0 + %du, sets[%d]);' % (d + ahead, (steady_first + d + ahead) % sets))
                a('            issue_loads_full(k0 + %du, sets[%d]);' % (d + ahead + sets, (steady_first + d + ahead) % sets))
                a('            store_chunk_full(k0 + %du - 1u);' % d)
                a('            __syncthreads();')
            a('        }')
        for k in range(steady_first + groups * sets, num_chunks):
            emit_step(k)
        a('        store_chunk(%du);' % (num_chunks - 1))
        a('    } else {')
        a('        __syncthreads();')
        a('        #pragma unroll 1')
        a('        for (uint32_t k = 0; k < %du; ++k) {' % (num_chunks - 1))
        a('            scan_chunk(k, ovl_scan_no());')
        a('            __syncthreads();')
        a('        }')
        a('        scan_chunk(%du, ovl_scan_yes());' % (num_chunks - 1))
        a('        __syncthreads();')
        a('    }')
    else:
        for j in range(min(sets, num_chunks)):
            a('    issue_loads(%du, sets[%d]);' % (j, j))
        a('    write_lds(0u, sets[0]);')
        if sets < num_chunks:
            a('    issue_loads(%du, sets[0]);' % sets)
        a('    __syncthreads();')
        a('    // step k: chunk k is scanned in place; then its results go out while chunk k + 1 comes into the other buffer')
        a('    auto step = [&](uint32_t k, MoverRegs& regs, auto last_chunk) {')
        a('        scan_chunk(k, last_chunk);')
        a('        __syncthreads();')
        a('        store_chunk(k);')
        a('        if (k + 1u < %du) write_lds(k + 1u, regs);' % num_chunks)
        a('        if (k + 1u + %du < %du) issue_loads(k + 1u + %du, regs);' % (sets, num_chunks, sets))
        a('        __syncthreads();')
        a('    };')
        full = (num_chunks - 1) // sets                 # whole rounds of the register sets before the last chunk
        if full:
            a('    #pragma unroll 1')
            a('    for (uint32_t k0 = 0; k0 < %du; k0 += %du) {' % (full * sets, sets))
            for d in range(sets):
                a('        step(k0 + %du, sets[%d], ovl_scan_no());' % (d, (d + 1) % sets))
            a('    }')
        for k in range(full * sets, num_chunks):
            a('    step(%du, sets[%d], ovl_scan_%s());' % (k, (k + 1) % sets, 'yes' if k == num_chunks - 1 else 'no'))
    if p.reduce:
        a('    // the statements after the worker\'s loop, once per line: lane 0 of the line holds the final state')
        a('    if (threadIdx.x < %du && part == 0u) {' % SCAN_THREADS)
        for name, _ in state:
            a('        %s = carry_%s;' % (name, name))
        for stmt in epilogue:
            a('        ' + stmt)
        a('    }')
    a('#undef OVL_SCAN_STEP')
    if not p.reduce:
        a('#undef OVL_SCAN_STORE')
    a('#undef OVL_SCAN_IN')
    a('#undef OVL_SCAN_OUT')
    a('}')

    itemsize = ITEMSIZE[p.x.dtype]
    launch = {
        'template': 'colreduce' if p.reduce else 'colskew',
        'vec': 1,
        'block': BLOCK,
        'blocks_needed': p.outer * strips,
        'align': {('in', p.x.io_index): itemsize} if p.reduce else
                 {('in', p.x.io_index): itemsize, ('out', p.out.io_index): itemsize},
        'vector_loads': 1,
        'vector_stores': 1,
    }
    return '\n'.join(src) + '\n', launch
