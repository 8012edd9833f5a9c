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
#: the template pays when the map template would have too few wavefronts to hide the latency of its loads
MAX_WORKERS = 1 << 16
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


def worthwhile(info, p):
    """Few lines and a long axis: where the one-worker-per-thread template is bound by the latency of its loads."""
    return info.num_workers <= MAX_WORKERS and p.length >= MIN_LENGTH


def generate(info, kernel_name, rows_per_chunk=None, batch=None, sets=None):
    p = plan(info, rows_per_chunk, batch, sets)
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

    emitter = BodyEmitter(info, pos_exprs,
                          read_hook=lambda node, tensor, idx: 'OVL_SCAN_IN',
                          store_hook=lambda node, tensor, idx, value: 'OVL_SCAN_OUT(' + value + ');')
    tagged = emitter.emit_tagged()
    range_idx = p.loop_item.node
    end_idx = max(i for i, _ in tagged)
    prologue = [t for i, t in tagged if i < range_idx]
    body = [t.strip() for i, t in tagged if range_idx < i < end_idx]
    counter_name = 'e' + str(p.counter)
    counter_type = CTYPE[info.nodes[p.counter].dtype]

    vname = 'ovl_scan_vec'
    src = []
    a = src.append
    a('typedef %s %s __attribute__((ext_vector_type(%d)));' % (ctype, vname, per))
    a('')
    a('extern "C" __global__ void __launch_bounds__(%d)' % BLOCK)
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
    _emit_movers(a, sets, num_chunks)
    a('    } else {')
    a('        // The scanning wavefront: lane = line c0 + lane of the strip; a lane past the last line shadows it.')
    a('        const uint32_t c = (c0 + lane < %du) ? lane : %du - c0;' % (p.inner, p.inner - 1))
    a('        const uint32_t line = o * %du + c0 + c;' % p.inner)
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
    a('        auto run = [&](%s (&set)[%d], uint32_t row0, bool first) {' % (vname, batch))
    a('            #pragma unroll')
    a('            for (uint32_t v = 0; v < %du; ++v) {' % batch)
    a('                %s& xv = set[v];' % vname)
    a('                #pragma unroll')
    a('                for (uint32_t u = 0; u < %du; ++u) {' % per)
    a('                    if (v == 0u && u == 0u && first) xv[0] = first_out;')
    a('                    else OVL_SCAN_STEP(row0 + v * %du + u)' % per)
    a('                }')
    a('            }')
    a('        };')
    a('        __syncthreads();')
    a('        for (uint32_t k = 0; k < %du; ++k) {' % num_chunks)
    a('            %s* colp = &tile[k %% 3u][0][lane];' % vname)
    a('            fetch(set_a, colp);')
    a('            #pragma unroll 1')
    a('            for (uint32_t q = 0; q < %du; q += %du) {' % (reads_per_chunk, 2 * batch))
    a('                fetch(set_b, colp + (q + %du) * %du);' % (batch, STRIP))
    a('                run(set_a, k * %du + q * %du, k == 0u && q == 0u);' % (rc, per))
    a('                put_back(set_a, colp + q * %du);' % STRIP)
    a('                if (q + %du < %du) fetch(set_a, colp + (q + %du) * %du);' % (2 * batch, reads_per_chunk, 2 * batch, STRIP))
    a('                run(set_b, k * %du + (q + %du) * %du, false);' % (rc, batch, per))
    a('                put_back(set_b, colp + (q + %du) * %du);' % (batch, STRIP))
    a('            }')
    a('            __syncthreads();')
    a('        }')
    a('#undef OVL_SCAN_STEP')
    a('#undef OVL_SCAN_IN')
    a('#undef OVL_SCAN_OUT')
    a('    }')
    a('}')

    itemsize = ITEMSIZE[p.x.dtype]
    launch = {
        'template': 'colscan',
        'vec': 1,
        'block': BLOCK,
        'blocks_needed': p.outer * strips,
        'align': {('in', p.x.io_index): itemsize, ('out', p.out.io_index): itemsize},
        'vector_loads': 1,
        'vector_stores': 1,
    }
    return '\n'.join(src) + '\n', launch


def _emit_movers(a, sets, num_chunks):
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
    a('        store_chunk(%du, m);' % (num_chunks - 1))

