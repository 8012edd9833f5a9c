"""
The row-scan kernel template: operators that walk the last axis of a tensor with a loop-carried accumulator
(``accumulate`` / ``cumsum`` / ``cumprod`` of the reference's opveclib/examples/test_accumulate.py:22-147 along the last
axis).

The worker function is a strictly sequential recurrence per row (``acc = f(acc, x[row, i]); out[row, i] = acc`` for
i = 1 .. L-1), so the order of the floating point operations is part of the result and must be kept: lane = row.  In
the one-worker-per-thread template neighbouring lanes then read addresses a whole row apart.  Here a 256-thread
workgroup owns ``ROWS`` consecutive rows and streams them through LDS in chunks of ``CHUNK`` columns with three
rotating buffers:

  * wavefronts 1-3 move data: 128-bit coalesced loads of chunk k+1 from global memory into LDS, and 128-bit
    coalesced stores of the finished chunk k-1 from LDS to global memory;
  * wavefront 0 scans chunk k in place in LDS: lane r walks row r left to right, four (float32) or two (float64)
    columns per 128-bit LDS access, running the operator's own loop body for every column in order.

One workgroup barrier separates the chunks.  The arithmetic each row sees is exactly the worker's sequential
recurrence, so results equal the generic template's (and numpy's accumulate) bit for bit; all global traffic is
coalesced and every element is read and written once.
"""

import re

from .. import language as lang
from .analysis import ITEMSIZE
from .body import BodyEmitter, CTYPE

BLOCK = 256
WAVE = 64
MOVERS = BLOCK - WAVE
LDS_BUDGET = 128 * 1024
NUM_CU = 256


class ScanPlan(object):
    def __init__(self, loop_item, counter, length, rows, x, out, vec, rows_per_block, chunk):
        self.loop_item = loop_item
        self.counter = counter
        self.length = length
        self.rows = rows
        self.x = x
        self.out = out
        self.vec = vec
        self.rows_per_block = rows_per_block
        self.chunk = chunk


def plan(info, rows_per_block=None, chunk=None, need_chunk=True, multi=False):
    """A ScanPlan when the DAG is a last-axis row scan this template can run, else None.  ``need_chunk``: the LDS
    templates stream rows in chunks that divide them; the lane-skewed scan does not.  ``multi``: the body may read
    several inputs of the output's shape and type (a gated recurrence ``h = a[r, i] * h + x[r, i]``); the lane-skewed
    scan takes up to four, the other templates one."""
    forced_rows, forced_chunk = rows_per_block, chunk
    if not info.inputs or len(info.inputs) > (4 if multi else 1) or not info.outputs or \
            len(info.outputs) > (4 if multi else 1):
        return None
    loops = [item for item in info.tree if item.kind == 'loop']
    if len(loops) != 1 or any(item.kind == 'if' for item in info.tree):
        return None
    loop = loops[0]
    # the shape the scan generators rely on: what sets up the first column (at most one store), then the loop, then
    # nothing; anything else (a store after the loop, two stores before it) runs on the map template
    if info.tree[-1] is not loop:
        return None
    stores_before = [item for item in info.tree[:-1] if item.kind == 'stmt' and
                     info.nodes[item.node].code == lang.ASSIGN_TENSOR and
                     info.nodes[info.nodes[item.node].ops[0]].code == lang.OUTPUT]
    if len(stores_before) > len(info.outputs):
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
        return None                 # nested loops or conditionals inside the scan body: use the generic template

    rows = info.num_workers
    # row base = worker_index * length, expressed in the position components
    rank = len(info.workgroup_shape)
    stride = 1
    wg_stride = [1] * rank
    for k in range(rank - 2, -1, -1):
        stride *= info.workgroup_shape[k + 1]
        wg_stride[k] = stride
    base = dict((('p', k), length * wg_stride[k]) for k in range(rank) if info.workgroup_shape[k] > 1)
    in_loop = dict(base)
    in_loop[('v', counter)] = 1
    sig_first = (tuple(sorted(base.items())), 0)
    sig_loop = (tuple(sorted(in_loop.items())), 0)

    x = out = None
    xs = []
    outs = []
    for node, tensor, aff in info.tensor_accesses():
        if aff is None:
            return None
        expect = sig_loop if info.in_loop[node.idx] else sig_first
        if aff.signature() != expect:
            return None
        if node.code == lang.READ_TENSOR:
            if tensor not in xs:
                xs.append(tensor)
            x = xs[0]
        else:
            if tensor not in outs:
                outs.append(tensor)
            out = outs[0]
    if x is None or out is None or len(xs) != len(info.inputs):
        return None
    if any(t.code != lang.INPUT or t.dtype != out.dtype or t.size != rows * length for t in xs):
        return None
    if any(t.code != lang.OUTPUT or t.dtype != out.dtype or t.size != rows * length for t in outs):
        return None
    if len(outs) != len(info.outputs):
        return None
    # every output is stored exactly once inside the loop (a worker that only stores before its loop is a reduction
    # that writes one column: the scan templates would store registers nothing assigned over every column), and,
    # when there are several outputs, exactly once before it (column 0); a single output at most once before it
    for t in outs:
        for inside in (False, True):
            count = len([n for n, tensor, _ in info.tensor_accesses()
                         if n.code == lang.ASSIGN_TENSOR and tensor is t and bool(info.in_loop[n.idx]) == inside])
            if inside or len(outs) > 1:
                if count != 1:
                    return None
            elif count > 1:
                return None
    itemsize = ITEMSIZE[x.dtype]
    if itemsize not in (4, 8) or x.dtype not in CTYPE:
        return None
    vec = 16 // itemsize

    rows_per_block = forced_rows or max(1, min(WAVE, (rows + NUM_CU - 1) // NUM_CU))
    chunk = None
    for cand in ((forced_chunk,) if forced_chunk else (1024, 512, 256, 128, 64)):
        if length % cand == 0 and cand % (2 * vec) == 0 and \
                3 * rows_per_block * (cand + vec) * itemsize <= LDS_BUDGET:
            chunk = cand
            break
    if chunk is None and need_chunk:
        return None
    p = ScanPlan(loop, counter, length, rows, x, out, vec, rows_per_block, chunk)
    p.xs = xs           # every input the body reads, in the order of their first use; x is the first
    p.outs = outs       # every output the body stores, likewise; out is the first
    return p


def _emit_movers(src, p, ctype, vname, vec, chunk, rpb, num_chunks, lds_column=None):
    """
    Source of the data-moving wavefronts (threads 64..255) of the LDS-fed scans, up to and including their branch of
    the kernel: they stream chunks of ``chunk`` columns of the workgroup's ``rpb`` rows from global memory into three
    rotating LDS buffers ``tile[3][rpb][...]`` and the scanned chunks back, with coalesced 128-bit accesses, one
    barrier per chunk.  ``lds_column(text)`` maps the C expression of a column (a multiple of ``vec``) to the column
    of the LDS row that holds it (identity by default; the lane-skewed scanner pads its segments).
    """
    if lds_column is None:
        lds_column = lambda text: text
    vectors_per_row = chunk // vec
    tile_vectors = rpb * vectors_per_row
    vpt = (tile_vectors + MOVERS - 1) // MOVERS      # vectors each mover thread handles per chunk
    ragged_rows = p.rows % rpb != 0
    src.append('    // Movers (threads 64..255): every thread owns %d vectors of each chunk.  A vector that does not exist (past' % vpt)
    src.append('    // the tile, past the last row) is replaced by the nearest one that does: it is loaded, written to LDS and')
    src.append('    // later stored a second time with the same value.  No memory instruction sits under a condition, so the')
    src.append('    // compiler can count them and waits for the loads of exactly the chunk it needs while those of the chunks')
    src.append('    // after it stay in flight.')
    src.append('    struct MoverRegs { %s v[%d]; };' % (vname, vpt))
    if ragged_rows:
        src.append('    const uint32_t rows_here = (%du - row0 < %du) ? %du - row0 : %du;' % (p.rows, rpb, p.rows, rpb))
    src.append('    auto slot = [&](uint32_t m, uint32_t i, uint32_t& r, uint32_t& cv) {')
    src.append('        uint32_t v = m + i * %du;' % MOVERS)
    if vpt * MOVERS > tile_vectors:
        src.append('        v = v < %du ? v : %du;' % (tile_vectors, tile_vectors - 1))
    src.append('        r = v / %du; cv = (v %% %du) * %du;' % (vectors_per_row, vectors_per_row, vec))
    if ragged_rows:
        src.append('        r = r < rows_here ? r : rows_here - 1u;')
    src.append('    };')
    src.append('    auto issue_loads = [&](uint32_t k, uint32_t m, MoverRegs& regs) {')
    src.append('        #pragma unroll')
    src.append('        for (uint32_t i = 0; i < %du; ++i) {' % vpt)
    src.append('            uint32_t r, cv;')
    src.append('            slot(m, i, r, cv);')
    src.append('            const uint64_t g = (uint64_t)(row0 + r) * %dull + k * %du + cv;' % (p.length, chunk))
    # (plain loads: with the non-temporal hint on loads and stores the mixed stream runs a quarter slower)
    src.append('            regs.v[i] = *reinterpret_cast<const %s*>(gin + g);' % vname)
    src.append('        }')
    src.append('    };')
    src.append('    auto write_lds = [&](uint32_t k, uint32_t m, const MoverRegs& regs) {')
    src.append('        #pragma unroll')
    src.append('        for (uint32_t i = 0; i < %du; ++i) {' % vpt)
    src.append('            uint32_t r, cv;')
    src.append('            slot(m, i, r, cv);')
    src.append('            *reinterpret_cast<%s*>(&tile[k %% 3u][r][%s]) = regs.v[i];' % (vname, lds_column('cv')))
    src.append('        }')
    src.append('    };')
    src.append('    auto store_chunk = [&](uint32_t k, uint32_t m) {')
    src.append('        MoverRegs regs;')
    src.append('        #pragma unroll')
    src.append('        for (uint32_t i = 0; i < %du; ++i) {' % vpt)
    src.append('            uint32_t r, cv;')
    src.append('            slot(m, i, r, cv);')
    src.append('            regs.v[i] = *reinterpret_cast<const %s*>(&tile[k %% 3u][r][%s]);' % (vname, lds_column('cv')))
    src.append('        }')
    src.append('        #pragma unroll')
    src.append('        for (uint32_t i = 0; i < %du; ++i) {' % vpt)
    src.append('            uint32_t r, cv;')
    src.append('            slot(m, i, r, cv);')
    src.append('            const uint64_t g = (uint64_t)(row0 + r) * %dull + k * %du + cv;' % (p.length, chunk))
    src.append('            __builtin_nontemporal_store(regs.v[i], reinterpret_cast<%s*>(gout + g));' % vname)
    src.append('        }')
    src.append('    };')
    src.append('')
    src.append('    if (threadIdx.x >= %du) {' % WAVE)
    src.append('        const uint32_t m = threadIdx.x - %du;' % WAVE)
    src.append('        // Two register sets keep two chunks of loads in flight: chunk j travels through set j %% 2, is requested two')
    src.append('        // steps before it is written to LDS, and is written one step before the scanning wavefront needs it.')
    src.append('        MoverRegs sets[2];')
    sets = 2
    for j in range(min(sets, num_chunks)):
        src.append('        issue_loads(%du, m, sets[%d]);' % (j, j))
    src.append('        write_lds(0u, m, sets[0]);')
    if sets < num_chunks:
        src.append('        issue_loads(%du, m, sets[0]);' % sets)
    src.append('        __syncthreads();')

    # Step k: chunk k is being scanned; chunk k + 1 goes to LDS, its register set is refilled with chunk k + 3, chunk
    # k - 1 goes out.  The steps in which all three happen run in a loop without conditions, entered after one full
    # round of them (the compiler counts outstanding requests along the cheapest path into a join: with the first
    # and last steps' conditions inside the loop it waits for every outstanding request before each write to LDS).
    def emit_step(k):
        regs = 'sets[%d]' % ((k + 1) % sets)
        if k + 1 < num_chunks:
            src.append('        write_lds(%du, m, %s);' % (k + 1, regs))
        if k + 1 + sets < num_chunks:
            src.append('        issue_loads(%du, m, %s);' % (k + 1 + sets, regs))
        if k >= 1:
            src.append('        store_chunk(%du, m);' % (k - 1))
        src.append('        __syncthreads();')
    steady_first = 1 + sets
    steady_end = max(steady_first, num_chunks - 1 - sets)
    groups = (steady_end - steady_first) // sets
    for k in range(0, min(steady_first, num_chunks)):
        emit_step(k)
    if groups:
        src.append('        #pragma unroll 1')
        src.append('        for (uint32_t k0 = %du; k0 < %du; k0 += %du) {' % (steady_first, steady_first + groups * sets, sets))
        for d in range(sets):
            regs = 'sets[%d]' % ((steady_first + d + 1) % sets)
            src.append('            write_lds(k0 + %du, m, %s);' % (d + 1, regs))
            src.append('            issue_loads(k0 + %du, m, %s);' % (d + 1 + sets, regs))
            src.append('            store_chunk(k0 + %du - 1u, m);' % d)
            src.append('            __syncthreads();')
        src.append('        }')
    for k in range(steady_first + groups * sets, num_chunks):
        emit_step(k)
    src.append('        store_chunk(%du, m);' % (num_chunks - 1))


def generate(info, kernel_name, rows_per_block=None, chunk=None, batch=None):
    p = plan(info, rows_per_block, chunk)
    assert p is not None
    # vectors per register set of the scanning wavefront: two sets must fit a chunk a whole number of times
    batch = batch or 8
    while p.chunk % (2 * batch * p.vec) != 0:
        batch //= 2
    assert batch >= 1
    ctype = CTYPE[p.x.dtype]
    vec, chunk, rpb = p.vec, p.chunk, p.rows_per_block
    row_stride = chunk + vec        # keeps 128-bit alignment; lanes of the scanning wavefront fall in different banks
    num_chunks = p.length // chunk
    vectors_per_row = chunk // vec
    tile_vectors = rpb * vectors_per_row

    # position of a row: the workgroup is the tensor shape without the scanned axis
    rank = len(info.workgroup_shape)
    pos_exprs = []
    stride = 1
    strides = [1] * rank
    for k in range(rank - 2, -1, -1):
        stride *= info.workgroup_shape[k + 1]
        strides[k] = stride
    for k in range(rank):
        expr = 'row'
        if k > 0:
            expr = '(row % ' + str(strides[k - 1]) + 'u)'
        pos_exprs.append(expr + ' / ' + str(strides[k]) + 'u')

    emitter = BodyEmitter(info, pos_exprs,
                          read_hook=lambda node, tensor, idx: 'OVL_SCAN_IN',
                          store_hook=lambda node, tensor, idx, value: 'OVL_SCAN_OUT(' + value + ');')
    tagged = emitter.emit_tagged()
    range_idx = p.loop_item.node
    end_idx = max(i for i, _ in tagged)         # ENDRANGE is the last statement of a plan-conforming DAG
    prologue = [t for i, t in tagged if i < range_idx]
    body = [t.strip() for i, t in tagged if range_idx < i < end_idx]
    counter_name = 'e' + str(p.counter)
    counter_type = CTYPE[info.nodes[p.counter].dtype]

    src = []
    vname = 'ovl_scan_vec'
    src.append('typedef %s %s __attribute__((ext_vector_type(%d)));' % (ctype, vname, vec))
    src.append('')
    src.append('extern "C" __global__ void __launch_bounds__(%d)' % BLOCK)
    src.append('%s(const %s* __restrict__ in%d, %s* __restrict__ out%d) {' % (
        kernel_name, ctype, p.x.io_index, ctype, p.out.io_index))
    src.append('    __shared__ __attribute__((aligned(16))) %s tile[3][%d][%d];' % (ctype, rpb, row_stride))
    src.append('    const uint32_t row0 = blockIdx.x * %du;' % rpb)
    src.append('    const uint32_t lane = threadIdx.x %% %du;' % WAVE)
    src.append('    const %s* __restrict__ gin = in%d;' % (ctype, p.x.io_index))
    src.append('    %s* __restrict__ gout = out%d;' % (ctype, p.out.io_index))
    src.append('')
    _emit_movers(src, p, ctype, vname, vec, chunk, rpb, num_chunks)
    src.append('    } else {')
    src.append('        // The scanning wavefront: lane r owns row row0 + r; surplus lanes are switched off for the LDS accesses')
    src.append('        // (an LDS instruction costs by the lanes that take part).')
    src.append('        // The row travels through two register sets of %d vectors: while one set runs the recurrence, the' % batch)
    src.append('        // other is being read from LDS, so the latency of an LDS read is paid once per chunk and not once per')
    src.append('        // vector; what remains on the critical path is the recurrence itself.')
    src.append('        const uint32_t r = lane < %du ? lane : %du;' % (rpb, rpb - 1))
    src.append('        const uint32_t row = (row0 + r < %du) ? row0 + r : %du;' % (p.rows, p.rows - 1))
    src.append('        __syncthreads();')
    src.append('        %s* rowp = &tile[0][r][0];' % ctype)
    src.append('        %s set_a[%d], set_b[%d];' % (vname, batch, batch))
    src.append('        auto fetch = [&](%s (&set)[%d], const %s* from) {' % (vname, batch, ctype))
    src.append('            #pragma unroll')
    src.append('            for (uint32_t v = 0; v < %du; ++v) set[v] = *reinterpret_cast<const %s*>(from + v * %du);' % (
        batch, vname, vec))
    src.append('        };')
    src.append('        const bool owner = lane < %du;' % rpb)
    src.append('        auto put_back = [&](const %s (&set)[%d], %s* to) {' % (vname, batch, ctype))
    src.append('            #pragma unroll')
    src.append('            for (uint32_t v = 0; v < %du; ++v) *reinterpret_cast<%s*>(to + v * %du) = set[v];' % (
        batch, vname, vec))
    src.append('        };')
    src.append('        if (owner) fetch(set_a, rowp);')
    src.append('        // first column: the statements the worker runs before its loop')
    src.append('#define OVL_SCAN_IN set_a[0][0]')
    src.append('#define OVL_SCAN_OUT(value) set_a[0][0] = (value)')
    for stmt in prologue:
        src.append('        ' + stmt)
    src.append('#undef OVL_SCAN_IN')
    src.append('#undef OVL_SCAN_OUT')
    src.append('#define OVL_SCAN_IN xv[u]')
    src.append('#define OVL_SCAN_OUT(value) xv[u] = (value)')
    src.append('#define OVL_SCAN_STEP(column) { %s = (%s)(column); %s }' % (
        counter_name, counter_type, ' '.join(body)))
    src.append('        // the recurrence over one register set; `first` skips the row\'s first column, which is done above')
    src.append('        auto run = [&](%s (&set)[%d], uint32_t column0, bool first) {' % (vname, batch))
    src.append('            #pragma unroll')
    src.append('            for (uint32_t v = 0; v < %du; ++v) {' % batch)
    src.append('                %s& xv = set[v];' % vname)
    src.append('                #pragma unroll')
    src.append('                for (uint32_t u = 0; u < %du; ++u) {' % vec)
    src.append('                    if (v == 0u && u == 0u && first) continue;')
    src.append('                    OVL_SCAN_STEP(column0 + v * %du + u)' % vec)
    src.append('                }')
    src.append('            }')
    src.append('        };')
    src.append('        for (uint32_t k = 0; k < %du; ++k) {' % num_chunks)
    src.append('            rowp = &tile[k % 3u][r][0];')
    src.append('            if (owner) {')
    src.append('            if (k != 0u) fetch(set_a, rowp);')
    src.append('            #pragma unroll 1')
    src.append('            for (uint32_t c = 0; c < %du; c += %du) {' % (chunk, 2 * batch * vec))
    src.append('                fetch(set_b, rowp + c + %du);' % (batch * vec))
    src.append('                run(set_a, k * %du + c, k == 0u && c == 0u);' % chunk)
    src.append('                put_back(set_a, rowp + c);')
    src.append('                if (c + %du < %du) fetch(set_a, rowp + c + %du);' % (2 * batch * vec, chunk, 2 * batch * vec))
    src.append('                run(set_b, k * %du + c + %du, false);' % (chunk, batch * vec))
    src.append('                put_back(set_b, rowp + c + %du);' % (batch * vec))
    src.append('            }')
    src.append('            }')
    src.append('            __syncthreads();')
    src.append('        }')
    src.append('#undef OVL_SCAN_STEP')
    src.append('#undef OVL_SCAN_IN')
    src.append('#undef OVL_SCAN_OUT')
    src.append('    }')
    src.append('}')

    blocks = (p.rows + rpb - 1) // rpb
    launch = {
        'template': 'rowscan',
        'vec': vec,
        'block': BLOCK,
        'blocks_needed': blocks,
        'align': {('in', p.x.io_index): 16, ('out', p.out.io_index): 16},
        'vector_loads': 1,
        'vector_stores': 1,
    }
    return '\n'.join(src) + '\n', launch


# ---------------------------------------------------------------------------------------------------------------------
# The lane-skewed variant: no LDS, no barriers.
#
# Sixteen neighbouring lanes share one row; lane i of the group holds VEC consecutive columns of the current group of
# 16*VEC columns, loaded and stored as one 128-bit access, so a wavefront reads and writes 256-byte runs of four rows.
# The recurrence still runs strictly left to right: in phase p (p = 0..15) every lane runs the loop body over its own
# VEC columns starting from the carried state it currently holds, then hands its final state to its right neighbour
# (one DPP move per 32 bits of state).  Lane 0 starts from the true carry, so after phase p lanes 0..p hold exact
# results; a lane that is already exact recomputes the same values, a lane that is not yet exact computes values
# that are overwritten in a later phase.  After phase 15 all 16*VEC results are exact and lane 15's state is rotated
# to lane 0 as the carry into the next group.  Per column the wavefront issues one loop body plus 1/VEC state moves,
# against one loop body plus a 128-bit LDS read and write per VEC columns in the lane = row variant, and rows are
# spread over four times as many wavefronts.
# ---------------------------------------------------------------------------------------------------------------------

GROUP_LANES = 16
SKEW_MAX_BODY = 64


def _body_size(info):
    """Nodes inside the loop, without the 64-bit index arithmetic of the tensor accesses (the templates address
    the rows themselves, so those nodes leave no code): what is unrolled sixteen phases times a vector's elements."""
    return len([n for n in info.nodes if info.in_loop[n.idx] and n.dtype != lang.UINT64])


HEAVY_CODES = (lang.DIVIDE, lang.MODULO, lang.POW, lang.SQRT, lang.EXP, lang.LOG, lang.LOG10, lang.TANH, lang.SIN,
               lang.COS, lang.TAN, lang.SINH, lang.COSH, lang.ASIN, lang.ACOS, lang.ATAN, lang.ATAN2)


def _heavy_outside_recurrence(info, p):
    """True when the loop body computes something costly (a division, a transcendental function) that the carried
    state does not depend on: work for the outputs only, which need not be repeated in every phase of the skewed
    recurrence."""
    needed = set()
    stack = [n.idx for n in info.nodes if info.in_loop[n.idx] and n.code == lang.ASSIGN_VARIABLE and
             n.ops[0] != p.counter]
    while stack:
        idx = stack.pop()
        if idx in needed:
            continue
        needed.add(idx)
        stack.extend(info.nodes[idx].ops)
    return any(info.in_loop[n.idx] and n.idx not in needed and n.code in HEAVY_CODES for n in info.nodes)


def _carried_state(info, p):
    """Variables declared before the loop and assigned inside it (the loop counter excluded), in DAG order."""
    range_idx = p.loop_item.node
    state = []
    for node in info.nodes:
        if node.code == lang.ASSIGN_VARIABLE and info.in_loop[node.idx]:
            target = node.ops[0]
            if target < range_idx and target != p.counter and target not in state:
                state.append(target)
    return sorted(state)


def skew_plan(info):
    """The structural plan when the lane-skewed variant can run this DAG, else None."""
    # (a row need not be a whole number of groups of 16 * VEC columns, nor aligned: what is left after the last whole
    # group is scanned by one lane, and rows that do not start on 16-byte boundaries are moved with unaligned vectors)
    p = plan(info, need_chunk=False, multi=True)
    if p is None or p.length < GROUP_LANES * p.vec:
        return None
    if _body_size(info) > SKEW_MAX_BODY:
        return None
    for idx in _carried_state(info, p):
        if info.nodes[idx].dtype not in CTYPE:
            return None
    return p


# ---------------------------------------------------------------------------------------------------------------------
# The LDS-fed lane-skewed variant, for recurrences that run at their own latency (8-byte elements, few rows).
#
# The lane-skewed scan above pays a hand-over between neighbouring lanes once per VEC * width columns, and its width
# is limited by the memory pipeline: a lane that owns more than 32 consecutive bytes makes the wavefront's requests
# sparse (float64 [1024, 16384]: 75 us with 32 bytes per lane, 126 us with 64).  Here the requests are made by other
# wavefronts: three of the workgroup's four wavefronts stream the rows through LDS with dense 128-bit accesses (as in
# the lane = row variant), and the fourth runs the skewed recurrence out of LDS, where a lane can own a segment of any
# length at no cost: with 16 columns per lane and phase the hand-over is paid once per 16 additions.  Segments are
# padded by one vector in LDS so that the sixteen lanes of a group read and write without bank conflicts.
# Measured on MI355X, float64, against the lane-skewed scan: [1024, 16384] 60 us against 74, [512, 16384] 55 / 73,
# [2048, 16384] 111 / 119, [4096, 4096] 51 / 75, [8192, 2048] 51 / 69, [256, 65536] 203 / 279.  The recurrence alone
# (no memory traffic at all, segments in registers) takes 45 us for 16384 columns, fed from LDS 52 us.  float32,
# whose lane-skewed scan already runs at the speed of memory, loses with it (108 us against 85).
# ---------------------------------------------------------------------------------------------------------------------
FED_ROWS = WAVE // GROUP_LANES      # rows per workgroup: one group of sixteen lanes of the scanning wavefront each


def fed_plan(info, width=None, chunk=None):
    """(ScanPlan, width, chunk) when the LDS-fed lane-skewed variant can run this DAG, else None."""
    p = skew_plan(info)
    if p is None or len(p.xs) != 1 or len(p.outs) != 1 or p.length % (GROUP_LANES * p.vec) != 0:
        return None
    itemsize = ITEMSIZE[p.x.dtype]
    width = width or 8
    while width > 1 and p.length % (GROUP_LANES * p.vec * width) != 0:
        width //= 2
    group_cols = GROUP_LANES * p.vec * width
    if p.length % group_cols != 0:
        return None
    # (float64 [1024, 16384]: chunks of 512 and 1024 columns run alike; 512 lets two workgroups share a CU's LDS,
    # which is what tensors with more rows than CUs times four need)
    for cand in ((chunk,) if chunk else (512, 1024, 256, 128, 64)):
        padded = cand + (cand // (p.vec * width)) * p.vec
        if cand % group_cols == 0 and p.length % cand == 0 and 3 * FED_ROWS * padded * itemsize <= LDS_BUDGET:
            return p, width, cand
    return None


def generate_fed(info, kernel_name, width=None, chunk=None):
    p, width, chunk = fed_plan(info, width, chunk)
    ctype = CTYPE[p.x.dtype]
    vec = p.vec
    rpb = FED_ROWS
    seg = vec * width                       # columns a lane owns per group
    group_cols = GROUP_LANES * seg
    groups = chunk // group_cols            # groups per chunk
    num_chunks = p.length // chunk
    row_stride = chunk + (chunk // seg) * vec

    rank = len(info.workgroup_shape)
    pos_exprs = []
    stride = 1
    strides = [1] * rank
    for k in range(rank - 2, -1, -1):
        stride *= info.workgroup_shape[k + 1]
        strides[k] = stride
    for k in range(rank):
        expr = 'row'
        if k > 0:
            expr = '(row % ' + str(strides[k - 1]) + 'u)'
        pos_exprs.append(expr + ' / ' + str(strides[k]) + 'u')
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
    state = [('e' + str(idx), CTYPE[info.nodes[idx].dtype]) for idx in _carried_state(info, p)]

    vname = 'ovl_scan_vec'
    src = []
    src.append('typedef %s %s __attribute__((ext_vector_type(%d)));' % (ctype, vname, vec))
    src.append('')
    src.append('extern "C" __global__ void __launch_bounds__(%d)' % BLOCK)
    src.append('%s(const %s* __restrict__ in%d, %s* __restrict__ out%d) {' % (
        kernel_name, ctype, p.x.io_index, ctype, p.out.io_index))
    if info.uses_math_tables():
        src.append('    OVL_DECLARE_MATH_TABLES();')
    src.append('    __shared__ __attribute__((aligned(16))) %s tile[3][%d][%d];' % (ctype, rpb, row_stride))
    src.append('    const uint32_t row0 = blockIdx.x * %du;' % rpb)
    src.append('    const uint32_t lane = threadIdx.x %% %du;' % WAVE)
    src.append('    const %s* __restrict__ gin = in%d;' % (ctype, p.x.io_index))
    src.append('    %s* __restrict__ gout = out%d;' % (ctype, p.out.io_index))
    src.append('')
    # column cv of a chunk lives at cv + (cv / seg) * vec of the LDS row: every segment is followed by one spare vector
    _emit_movers(src, p, ctype, vname, vec, chunk, rpb, num_chunks,
                 lds_column=lambda cv: '%s + (%s / %du) * %du' % (cv, cv, seg, vec))
    src.append('    } else {')
    src.append('        // The scanning wavefront: sixteen lanes per row, lane `part` of a group owns columns')
    src.append('        // [part * %d, part * %d + %d) of every group of %d columns.  A group past the last row shadows it.' % (
        seg, seg, seg, group_cols))
    src.append('        const uint32_t part = lane %% %du;' % GROUP_LANES)
    src.append('        const uint32_t q = lane / %du;' % GROUP_LANES)
    src.append('        const uint32_t row = (row0 + q < %du) ? row0 + q : %du;' % (p.rows, p.rows - 1))
    src.append('        // first column: the statements the worker runs before its loop, in every lane')
    src.append('        %s first_out;' % ctype)
    src.append('#define OVL_SCAN_IN (in%d[(uint64_t)row * %dull])' % (p.x.io_index, p.length))
    src.append('#define OVL_SCAN_OUT(value) first_out = (value)')
    for stmt in prologue:
        src.append('        ' + stmt)
    src.append('#undef OVL_SCAN_IN')
    src.append('#undef OVL_SCAN_OUT')
    for name, stype in state:
        src.append('        %s carry_%s = %s;' % (stype, name, name))
    src.append('#define OVL_SCAN_IN xv[u]')
    src.append('#define OVL_SCAN_OUT(value) ov[w][u] = (value)')
    src.append('#define OVL_SCAN_STEP(column) { %s = (%s)(column); %s }' % (
        counter_name, counter_type, ' '.join(body)))
    src.append('        %s set_a[%d], set_b[%d];' % (vname, width, width))
    src.append('        auto fetch = [&](%s (&set)[%d], const %s* from) {' % (vname, width, ctype))
    src.append('            #pragma unroll')
    src.append('            for (uint32_t w = 0; w < %du; ++w) set[w] = *reinterpret_cast<const %s*>(from + w * %du);' % (
        width, vname, vec))
    src.append('        };')
    src.append('        // one group: in phase p every lane runs the recurrence over its segment from the state it holds and')
    src.append('        // hands its final state to its right neighbour; after phase p lanes 0..p are exact')
    src.append('        auto run = [&](%s (&set)[%d], %s* to, uint32_t column0, bool first_group) {' % (vname, width, ctype))
    src.append('            %s ov[%d];' % (vname, width))
    src.append('            const uint32_t col0 = column0 + part * %du;' % seg)
    src.append('            const bool first_column = first_group && part == 0u;')
    src.append('            #pragma unroll')
    src.append('            for (uint32_t phase = 0; phase < %du; ++phase) {' % GROUP_LANES)
    for name, _ in state:
        src.append('                %s = carry_%s;' % (name, name))
    src.append('                #pragma unroll')
    src.append('                for (uint32_t w = 0; w < %du; ++w) {' % width)
    src.append('                    const %s xv = set[w];' % vname)
    src.append('                    #pragma unroll')
    src.append('                    for (uint32_t u = 0; u < %du; ++u) {' % vec)
    src.append('                        if (w == 0u && u == 0u && first_column) ov[0][0] = first_out;')
    src.append('                        else OVL_SCAN_STEP(col0 + w * %du + u)' % vec)
    src.append('                    }')
    src.append('                }')
    for name, _ in state:
        src.append('                carry_%s = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry_%s, %s);' % (name, name, name))
    src.append('            }')
    src.append('            // the last lane of the group finished the group: its state is the carry into the next one')
    for name, _ in state:
        src.append('            carry_%s = ovl_dpp_move<OVL_DPP_ROW_ROR1>(carry_%s, %s);' % (name, name, name))
    src.append('            #pragma unroll')
    src.append('            for (uint32_t w = 0; w < %du; ++w) *reinterpret_cast<%s*>(to + w * %du) = ov[w];' % (
        width, vname, vec))
    src.append('        };')
    src.append('        __syncthreads();')
    src.append('        for (uint32_t k = 0; k < %du; ++k) {' % num_chunks)
    src.append('            %s* segp = &tile[k %% 3u][q][part * %du];' % (ctype, seg + vec))
    src.append('            fetch(set_a, segp);')
    src.append('            #pragma unroll 1')
    src.append('            for (uint32_t g = 0; g < %du; g += 2u) {' % groups)
    src.append('                %s* here = segp + g * %du;' % (ctype, GROUP_LANES * (seg + vec)))
    src.append('                if (g + 1u < %du) fetch(set_b, here + %du);' % (groups, GROUP_LANES * (seg + vec)))
    src.append('                run(set_a, here, k * %du + g * %du, k == 0u && g == 0u);' % (chunk, group_cols))
    src.append('                if (g + 2u < %du) fetch(set_a, here + %du);' % (groups, 2 * GROUP_LANES * (seg + vec)))
    src.append('                if (g + 1u < %du) run(set_b, here + %du, k * %du + (g + 1u) * %du, false);' % (
        groups, GROUP_LANES * (seg + vec), chunk, group_cols))
    src.append('            }')
    src.append('            __syncthreads();')
    src.append('        }')
    src.append('#undef OVL_SCAN_STEP')
    src.append('#undef OVL_SCAN_IN')
    src.append('#undef OVL_SCAN_OUT')
    src.append('    }')
    src.append('}')

    launch = {
        'template': 'fedscan',
        'vec': vec,
        'block': BLOCK,
        'blocks_needed': (p.rows + rpb - 1) // rpb,
        'align': {('in', p.x.io_index): 16, ('out', p.out.io_index): 16},
        'vector_loads': 1,
        'vector_stores': 1,
    }
    return '\n'.join(src) + '\n', launch


# ---------------------------------------------------------------------------------------------------------------------
# The LDS-fed lane-skewed variant whose scanning wavefront keeps no results ('carryscan'), for tensors that give every
# compute unit at most one workgroup.
#
# A scan of float64 rows runs at the latency of its recurrence (a dependent float64 addition issues every 5 clocks),
# and in the variant above the scanning wavefront also writes every result to LDS: a 128-bit LDS write costs the
# wavefront that issues it about 25 clocks, five steps of the recurrence, a read about 5.  Here the scanning wavefront
# only reads: after the sixteenth phase of a chunk every lane holds the exact state that enters its segment, and that
# state is all it writes (one value per lane and carried variable).  A second wavefront, the finisher, runs the loop
# body once more over every segment from its entering state - the same operations in the same order, hence the same
# bits - and writes the results over the inputs in LDS; a third stores them, two more load.  The workgroup streams its
# four rows through six rotating LDS buffers in chunks of 16 * seg columns, one barrier per chunk; chunk c is written
# to LDS in step c - 2, read by the scanning wavefront in step c - 1, scanned in step c, finished in step c + 2 and
# stored in step c + 3.  float64 [1024, 16384]: 47 us against 58; the 105 KiB of LDS allow one workgroup per compute
# unit, so tensors with more workgroups than compute units stay with the variant above unless they fill whole rounds
# with long rows.
# ---------------------------------------------------------------------------------------------------------------------
CARRY_BUFFERS = 6
CARRY_AHEAD = 4          # chunks of loads a loading thread keeps in flight
CARRY_LOADER_WAVES = 2
CARRY_BLOCK = (3 + CARRY_LOADER_WAVES) * WAVE
CARRY_SYNC_PHASE = 8     # the scanning wavefront's LDS reads of a step fill the phases before this one


def carry_plan(info, width=None):
    """(ScanPlan, width) when the variant without results in the scanning wavefront can run this DAG, else None."""
    p = skew_plan(info)
    if p is None or len(p.xs) != 1 or len(p.outs) != 1:
        return None
    itemsize = ITEMSIZE[p.x.dtype]
    width = width or 32 // p.vec
    while width >= CARRY_SYNC_PHASE and p.length % (GROUP_LANES * p.vec * width) != 0:
        width //= 2
    # the scanning wavefront reads width vectors in CARRY_SYNC_PHASE phases; the movers own whole vectors
    if width < CARRY_SYNC_PHASE or width % CARRY_SYNC_PHASE != 0 or p.length % (GROUP_LANES * p.vec * width) != 0:
        return None
    chunk_vectors = FED_ROWS * GROUP_LANES * width
    if chunk_vectors % (CARRY_LOADER_WAVES * WAVE) != 0:
        return None
    padded = GROUP_LANES * (p.vec * width + p.vec)
    if CARRY_BUFFERS * FED_ROWS * padded * itemsize > LDS_BUDGET:
        return None
    return p, width


def carry_preferred(info):
    """True when 'auto' should take the variant without results in the scanning wavefront: its workgroups fit in one
    round over the compute units, or fill their rounds and have rows long enough to pay for the start of the pipeline
    in each (measured, float64: [1024, 16384] 47 us against 58, [2048, 16384] 94 / 97, [256, 65536] 154 / 192, but
    [4096, 4096] 59 / 41, [1500, 8192] 49 / 34, [16384, 512] 59 / 31)."""
    planned = carry_plan(info)
    if planned is None:
        return False
    p, width = planned
    groups = (p.rows + FED_ROWS - 1) // FED_ROWS
    rounds = (groups + NUM_CU - 1) // NUM_CU
    chunks = p.length // (GROUP_LANES * p.vec * width)
    return groups <= NUM_CU or (10 * groups >= 9 * rounds * NUM_CU and chunks >= 24)


def generate_carry(info, kernel_name, width=None):
    p, width = carry_plan(info, width)
    ctype = CTYPE[p.x.dtype]
    vec = p.vec
    rpb = FED_ROWS
    seg = vec * width                       # columns a lane owns per chunk
    chunk = GROUP_LANES * seg
    num_chunks = p.length // chunk
    padded_seg = seg + vec
    row_stride = GROUP_LANES * padded_seg
    chunk_vectors = rpb * chunk // vec
    per_loader = chunk_vectors // (CARRY_LOADER_WAVES * WAVE)
    per_storer = chunk_vectors // WAVE
    reads_per_phase = width // CARRY_SYNC_PHASE

    rank = len(info.workgroup_shape)
    pos_exprs = []
    stride = 1
    strides = [1] * rank
    for k in range(rank - 2, -1, -1):
        stride *= info.workgroup_shape[k + 1]
        strides[k] = stride
    for k in range(rank):
        expr = 'row'
        if k > 0:
            expr = '(row % ' + str(strides[k - 1]) + 'u)'
        pos_exprs.append(expr + ' / ' + str(strides[k]) + 'u')
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
    state = [('e' + str(idx), CTYPE[info.nodes[idx].dtype]) for idx in _carried_state(info, p)]

    vname = 'ovl_scan_vec'
    src = []
    a = src.append
    a('typedef %s %s __attribute__((ext_vector_type(%d)));' % (ctype, vname, vec))
    a('struct ovl_scan_yes { static constexpr bool value = true; };')
    a('struct ovl_scan_no { static constexpr bool value = false; };')
    a('')
    a('extern "C" __global__ void __launch_bounds__(%d)' % CARRY_BLOCK)
    a('%s(const %s* __restrict__ in%d, %s* __restrict__ out%d) {' % (
        kernel_name, ctype, p.x.io_index, ctype, p.out.io_index))
    if info.uses_math_tables():
        a('    OVL_DECLARE_MATH_TABLES();')
    a('    __shared__ __attribute__((aligned(16))) %s tile[%d][%d][%d];' % (ctype, CARRY_BUFFERS, rpb, row_stride))
    for name, stype in state:
        a('    __shared__ %s entering_%s[%d][%d];' % (stype, name, CARRY_BUFFERS, WAVE))
    a('    const uint32_t row0 = blockIdx.x * %du;' % rpb)
    a('    const uint32_t wave = threadIdx.x / %du, lane = threadIdx.x %% %du;' % (WAVE, WAVE))
    a('    const %s* __restrict__ gin = in%d;' % (ctype, p.x.io_index))
    a('    %s* __restrict__ gout = out%d;' % (ctype, p.out.io_index))
    a('    // Every wavefront passes the same %d barriers: one after the first two chunks are in LDS, then one at the end' % (num_chunks + 3))
    a('    // of each of the steps 0 .. %d.' % (num_chunks + 1))
    a('    if (wave < 2u) {')
    a('        // Scanning wavefront (0) and finisher (1): sixteen lanes per row, lane `part` of a group owns columns')
    a('        // [part * %d, part * %d + %d) of every chunk of %d columns.  A group past the last row shadows it.' % (
        seg, seg, seg, chunk))
    a('        const uint32_t part = lane %% %du;' % GROUP_LANES)
    a('        const uint32_t q = lane / %du;' % GROUP_LANES)
    a('        const uint32_t row = (row0 + q < %du) ? row0 + q : %du;' % (p.rows, p.rows - 1))
    a('        %s* const mine = &tile[0][q][part * %du];' % (ctype, padded_seg))
    a('        // first column: the statements the worker runs before its loop, in every lane')
    a('        %s first_out;' % ctype)
    a('#define OVL_SCAN_IN (in%d[(uint64_t)row * %dull])' % (p.x.io_index, p.length))
    a('#define OVL_SCAN_OUT(value) first_out = (value)')
    for stmt in prologue:
        a('        ' + stmt)
    a('#undef OVL_SCAN_IN')
    a('#undef OVL_SCAN_OUT')
    a('#define OVL_SCAN_IN xv[u]')
    a('#define OVL_SCAN_STEP(column) { %s = (%s)(column); %s }' % (counter_name, counter_type, ' '.join(body)))
    a('        if (wave == 0u) {')
    for name, stype in state:
        a('            %s carry_%s = %s;' % (stype, name, name))
    a('#define OVL_SCAN_OUT(value) (void)(value)')
    a('            %s set_a[%d], set_b[%d];' % (vname, width, width))
    a('            __syncthreads();')
    a('            #pragma unroll')
    a('            for (uint32_t w = 0; w < %du; ++w) set_a[w] = *reinterpret_cast<const %s*>(mine + w * %du);' % (
        width, vname, vec))
    a('            uint32_t next = 1u, slot = 0u;        // buffer of the chunk after this one; this chunk\'s slot')
    a('            // One chunk: in phase p every lane runs the recurrence over its segment from the state it holds and hands')
    a('            // its final state to its right neighbour; after phase p lanes 0..p are exact.  Meanwhile the segments of')
    a('            // the next chunk arrive in the other register set.  The results are not kept.')
    a('            auto scan_chunk = [&](const %s (&set)[%d], %s (&other)[%d], uint32_t column0, auto first_chunk) {' % (
        vname, width, vname, width))
    a('                const %s* ahead = mine + next * %du;' % (ctype, rpb * row_stride))
    a('                const uint32_t col0 = column0 + part * %du;' % seg)
    a('                #pragma unroll')
    a('                for (uint32_t phase = 0; phase < %du; ++phase) {' % GROUP_LANES)
    for name, _ in state:
        a('                    %s = carry_%s;' % (name, name))
    a('                    #pragma unroll')
    a('                    for (uint32_t w = 0; w < %du; ++w) {' % width)
    a('                        const %s xv = set[w];' % vname)
    a('                        #pragma unroll')
    a('                        for (uint32_t u = 0; u < %du; ++u) {' % vec)
    a('                            // (the row\'s first column is what the statements before the loop computed)')
    a('                            if (decltype(first_chunk)::value && w == 0u && u == 0u) { if (part != 0u) OVL_SCAN_STEP(col0) }')
    a('                            else OVL_SCAN_STEP(col0 + w * %du + u)' % vec)
    a('                        }')
    a('                    }')
    for name, _ in state:
        a('                    carry_%s = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry_%s, %s);' % (name, name, name))
    a('                    if (phase < %du) {' % CARRY_SYNC_PHASE)
    a('                        #pragma unroll')
    a('                        for (uint32_t j = 0; j < %du; ++j)' % reads_per_phase)
    a('                            other[phase * %du + j] = *reinterpret_cast<const %s*>(ahead + (phase * %du + j) * %du);' % (
        reads_per_phase, vname, reads_per_phase, vec))
    a('                    }')
    a('                    // (the fences keep each read in its phase and the barrier in its place)')
    a('                    __builtin_amdgcn_sched_barrier(0);')
    a('                    if (phase == %du) {' % CARRY_SYNC_PHASE)
    a('                        __syncthreads();')
    a('                        __builtin_amdgcn_sched_barrier(0);')
    a('                    }')
    a('                }')
    a('                // lanes 1..15 now hold their left neighbour\'s exact final state, lane 0 the state that entered the')
    a('                // chunk: what enters each lane\'s segment')
    for name, _ in state:
        a('                entering_%s[slot][lane] = carry_%s;' % (name, name))
    a('                // the last lane finished the chunk: its state is the carry into the next one')
    for name, _ in state:
        a('                carry_%s = ovl_dpp_move<OVL_DPP_ROW_ROR1>(carry_%s, %s);' % (name, name, name))
    a('                next = next + 1u == %du ? 0u : next + 1u;' % CARRY_BUFFERS)
    a('                slot = slot + 1u == %du ? 0u : slot + 1u;' % CARRY_BUFFERS)
    a('                __builtin_amdgcn_sched_barrier(0);')
    a('            };')
    a('            scan_chunk(set_a, set_b, 0u, ovl_scan_yes());')
    if num_chunks > 1:
        a('            uint32_t g = 1u;')
        a('            #pragma unroll 1')
        a('            for (; g + 1u < %du; g += 2u) {' % num_chunks)
        a('                scan_chunk(set_b, set_a, g * %du, ovl_scan_no());' % chunk)
        a('                scan_chunk(set_a, set_b, (g + 1u) * %du, ovl_scan_no());' % chunk)
        a('            }')
        a('            if (g < %du) scan_chunk(set_b, set_a, g * %du, ovl_scan_no());' % (num_chunks, chunk))
    a('            __syncthreads();       // the last two steps: the others finish and store')
    a('            __syncthreads();')
    a('#undef OVL_SCAN_OUT')
    a('        } else {')
    a('            // The finisher: chunk s - 2 in step s, every segment once more from the state that enters it.')
    a('#define OVL_SCAN_OUT(value) v[w][u] = (value)')
    a('            __syncthreads();')
    a('            __syncthreads();')
    a('            __syncthreads();')
    a('            for (uint32_t s = 2u; s <= %du; ++s) {' % (num_chunks + 1))
    a('                const uint32_t buffer = (s - 2u) %% %du;' % CARRY_BUFFERS)
    a('                %s* here = mine + buffer * %du;' % (ctype, rpb * row_stride))
    a('                const uint32_t col0 = (s - 2u) * %du + part * %du;' % (chunk, seg))
    a('                %s v[%d];' % (vname, width))
    a('                #pragma unroll')
    a('                for (uint32_t w = 0; w < %du; ++w) v[w] = *reinterpret_cast<const %s*>(here + w * %du);' % (
        width, vname, vec))
    for name, _ in state:
        a('                %s = entering_%s[buffer][lane];' % (name, name))
    a('                #pragma unroll')
    a('                for (uint32_t w = 0; w < %du; ++w) {' % width)
    a('                    const %s xv = v[w];' % vname)
    a('                    #pragma unroll')
    a('                    for (uint32_t u = 0; u < %du; ++u) {' % vec)
    a('                        if (w == 0u && u == 0u && col0 == 0u) v[0][0] = first_out;')
    a('                        else OVL_SCAN_STEP(col0 + w * %du + u)' % vec)
    a('                    }')
    a('                }')
    a('                #pragma unroll')
    a('                for (uint32_t w = 0; w < %du; ++w) *reinterpret_cast<%s*>(here + w * %du) = v[w];' % (width, vname, vec))
    a('                __syncthreads();')
    a('            }')
    a('#undef OVL_SCAN_OUT')
    a('        }')
    a('#undef OVL_SCAN_STEP')
    a('#undef OVL_SCAN_IN')
    a('    } else {')
    a('        // Storer (wavefront 2) and loaders: thread m of its kind owns vectors m, m + <threads of the kind>, ... of')
    a('        // every chunk.  A loader\'s vector past the last row is a second copy of the last row\'s; the storer skips it.')
    a('        auto place = [&](uint32_t v, uint64_t& global_offset, uint32_t& lds_offset, bool& exists) {')
    a('            const uint32_t r = v / %du, c = (v %% %du) * %du;' % (chunk // vec, chunk // vec, vec))
    a('            exists = row0 + r < %du;' % p.rows)
    a('            global_offset = (uint64_t)(exists ? row0 + r : %du) * %dull + c;' % (p.rows - 1, p.length))
    a('            lds_offset = r * %du + c + (c / %du) * %du;' % (row_stride, seg, vec))
    a('        };')
    a('        if (wave == 2u) {')
    a('            uint64_t global_offset[%d];' % per_storer)
    a('            uint32_t lds_offset[%d];' % per_storer)
    a('            bool exists[%d];' % per_storer)
    a('            #pragma unroll')
    a('            for (uint32_t i = 0; i < %du; ++i) place(lane + i * %du, global_offset[i], lds_offset[i], exists[i]);' % (
        per_storer, WAVE))
    a('            auto store_chunk = [&](uint32_t c) {')
    a('                const %s* buffer = &tile[c %% %du][0][0];' % (ctype, CARRY_BUFFERS))
    a('                %s regs[%d];' % (vname, per_storer))
    a('                #pragma unroll')
    a('                for (uint32_t i = 0; i < %du; ++i) regs[i] = *reinterpret_cast<const %s*>(buffer + lds_offset[i]);' % (
        per_storer, vname))
    a('                #pragma unroll')
    a('                for (uint32_t i = 0; i < %du; ++i)' % per_storer)
    a('                    if (exists[i])')
    a('                        __builtin_nontemporal_store(regs[i], reinterpret_cast<%s*>(gout + global_offset[i] + c * %du));' % (
        vname, chunk))
    a('            };')
    a('            __syncthreads();')
    a('            __syncthreads();')
    a('            __syncthreads();')
    a('            __syncthreads();')
    a('            for (uint32_t s = 3u; s <= %du; ++s) {' % (num_chunks + 1))
    a('                store_chunk(s - 3u);')
    a('                __syncthreads();')
    a('            }')
    a('            store_chunk(%du);' % (num_chunks - 1))
    a('        } else {')
    a('            const uint32_t m = threadIdx.x - %du;' % (3 * WAVE))
    a('            uint64_t global_offset[%d];' % per_loader)
    a('            uint32_t lds_offset[%d];' % per_loader)
    a('            #pragma unroll')
    a('            for (uint32_t i = 0; i < %du; ++i) {' % per_loader)
    a('                bool exists;')
    a('                place(m + i * %du, global_offset[i], lds_offset[i], exists);' % (CARRY_LOADER_WAVES * WAVE))
    a('            }')
    a('            // Plain loads (with the non-temporal hint on loads and stores the mixed stream runs a quarter slower).  A')
    a('            // chunk past the end of the row is requested as the last chunk once more and lands in a buffer that')
    a('            // nobody reads any more: the steps are free of conditions and the counts of requests in flight exact.')
    a('            auto request = [&](uint32_t c, %s (&regs)[%d]) {' % (vname, per_loader))
    a('                const uint32_t cc = c < %du ? c : %du;' % (num_chunks, num_chunks - 1))
    a('                #pragma unroll')
    a('                for (uint32_t i = 0; i < %du; ++i)' % per_loader)
    a('                    regs[i] = *reinterpret_cast<const %s*>(gin + global_offset[i] + cc * %du);' % (vname, chunk))
    a('            };')
    a('            auto to_lds = [&](uint32_t c, const %s (&regs)[%d]) {' % (vname, per_loader))
    a('                %s* buffer = &tile[c %% %du][0][0];' % (ctype, CARRY_BUFFERS))
    a('                #pragma unroll')
    a('                for (uint32_t i = 0; i < %du; ++i) *reinterpret_cast<%s*>(buffer + lds_offset[i]) = regs[i];' % (
        per_loader, vname))
    a('            };')
    a('            %s set[%d][%d];' % (vname, CARRY_AHEAD, per_loader))
    a('            {')
    a('                %s first[2][%d];' % (vname, per_loader))
    a('                request(0u, first[0]);')
    a('                request(1u, first[1]);')
    for k in range(CARRY_AHEAD):
        a('                request(%du, set[%d]);' % (2 + k, (2 + k) % CARRY_AHEAD))
    a('                to_lds(0u, first[0]);')
    a('                to_lds(1u, first[1]);')
    a('            }')
    a('            __syncthreads();')
    a('            // step s: chunk s + 2 goes to LDS from the register set requested %d steps ago, which is then requested' % CARRY_AHEAD)
    a('            // again with chunk s + %d' % (2 + CARRY_AHEAD))
    a('            auto step = [&](uint32_t s, %s (&regs)[%d]) {' % (vname, per_loader))
    a('                to_lds(s + 2u, regs);')
    a('                request(s + %du, regs);' % (2 + CARRY_AHEAD))
    a('                __syncthreads();')
    a('            };')
    steps = num_chunks + 2
    whole = steps // CARRY_AHEAD
    if whole:
        a('            #pragma unroll 1')
        a('            for (uint32_t s = 0u; s < %du; s += %du) {' % (whole * CARRY_AHEAD, CARRY_AHEAD))
        for k in range(CARRY_AHEAD):
            a('                step(s + %du, set[%d]);' % (k, (2 + k) % CARRY_AHEAD))
        a('            }')
    for s_ in range(whole * CARRY_AHEAD, steps):
        a('            step(%du, set[%d]);' % (s_, (2 + s_) % CARRY_AHEAD))
    a('        }')
    a('    }')
    a('}')

    launch = {
        'template': 'carryscan',
        'vec': vec,
        'block': CARRY_BLOCK,
        'blocks_needed': (p.rows + rpb - 1) // rpb,
        'align': {('in', p.x.io_index): 16, ('out', p.out.io_index): 16},
        'vector_loads': 1,
        'vector_stores': 1,
    }
    return '\n'.join(src) + '\n', launch


# ---------------------------------------------------------------------------------------------------------------------
# Row reductions: a worker that walks the last axis of its inputs with a loop-carried state and stores nothing inside the
# loop (a dot product, a sum, a norm, a running extremum: the reference's opveclib/test/test_dot_product.py:27-45).
#
# In the one-worker-per-thread template the lanes of a wavefront read addresses a whole row apart (float32
# [4096, 16384]: 1.9 ms for a row sum).  The order of a floating point reduction is part of its result, so the rows are
# walked exactly as in the lane-skewed scan above: sixteen lanes per row, a lane owns VEC * width consecutive columns of
# a group, runs the loop body over them from the state it holds and hands its state to its right neighbour; after
# sixteen phases the group is done and the last lane's state is the carry into the next.  There is nothing to store
# per column; the statements after the loop run once per row, in the lane that holds the final state.
# ---------------------------------------------------------------------------------------------------------------------
class ReducePlan(object):
    def __init__(self, loop_item, end_idx, counter, start, length, rows, tensors, vec):
        self.loop_item = loop_item
        self.end_idx = end_idx          # the node that closes the loop
        self.counter = counter
        self.start = start              # first column the loop visits: 0, or 1 when the worker sets up with column 0
        self.length = length            # row length of the tensors read in the loop
        self.rows = rows
        self.tensors = tensors          # the INPUT nodes read in the loop
        self.vec = vec


def reduce_plan(info):
    """A ReducePlan when the DAG is a reduction along the last axis that `generate_reduce` can run, else None."""
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
    if start not in (0, 1) or step != 1 or stop is None:
        return None
    length = stop
    closers = [n.idx for n in info.nodes if n.idx > loop.node and n.code == lang.ENDRANGE and not info.in_loop[n.idx]]
    if not closers:
        return None
    end_idx = min(closers)

    rows = info.num_workers
    rank = len(info.workgroup_shape)
    stride = 1
    wg_stride = [1] * rank
    for k in range(rank - 2, -1, -1):
        stride *= info.workgroup_shape[k + 1]
        wg_stride[k] = stride
    def layout_of(aff):
        """(elements between the rows of two consecutive workers, offset of column 0) of an access that walks a
        row with the loop counter: a matrix row (row stride = its row length, or more for a slice of wider rows) or
        one vector that every worker reads (row stride 0)."""
        if aff is None or aff.coeff(('v', counter)) != 1:
            return None
        row_stride = None
        for sym, c in aff.coeffs.items():
            if sym == ('v', counter):
                continue
            if sym[0] != 'p':
                return None
            k = sym[1]
            if info.workgroup_shape[k] == 1:
                continue
            if c % wg_stride[k] != 0 or (row_stride is not None and c // wg_stride[k] != row_stride):
                return None
            row_stride = c // wg_stride[k]
        moving = [k for k in range(rank) if info.workgroup_shape[k] > 1]
        if row_stride is None:
            row_stride = 0
        elif any(aff.coeff(('p', k)) != row_stride * wg_stride[k] for k in moving):
            return None
        if row_stride < 0 or aff.const < 0:
            return None
        return row_stride, aff.const

    tensors = []
    layouts = {}
    for node, tensor, aff in info.tensor_accesses():
        if not info.in_loop[node.idx]:
            continue                    # before and after the loop: ordinary code of one lane
        if node.code != lang.READ_TENSOR or tensor.code != lang.INPUT or tensor.dtype not in CTYPE:
            return None
        layout = layout_of(aff)
        if layout is None or layouts.setdefault(tensor.idx, layout) != layout:
            return None
        if aff.lo < 0 or aff.hi >= tensor.size:
            return None
        if tensor not in tensors:
            tensors.append(tensor)
    if all(layouts[t.idx][0] == 0 for t in tensors):
        return None                     # no worker reads a row of its own
    if not tensors or len(tensors) > 4:
        return None
    itemsize = ITEMSIZE[tensors[0].dtype]
    if itemsize not in (4, 8) or any(ITEMSIZE[t.dtype] != itemsize for t in tensors):
        return None
    vec = 16 // itemsize
    # (short rows stay with one worker per thread: float32 [100000, 100] 18 us there, 26 us here)
    if length < 4 * GROUP_LANES * vec:
        return None
    if _body_size(info) > SKEW_MAX_BODY:
        return None
    p = ReducePlan(loop, end_idx, counter, start, length, rows, tensors, vec)
    p.layouts = layouts
    state = _carried_state(info, p)
    if not state or any(info.nodes[idx].dtype not in CTYPE for idx in state):
        return None
    return p


def generate_reduce(info, kernel_name, depth=None, width=None, sets=None, nt=''):
    p = reduce_plan(info)
    assert p is not None
    vec = p.vec
    itemsize = 16 // vec
    # width = 128-bit vectors per lane and phase.  With nothing to store, a reduction gains from wider lanes than a scan
    # does: the hand-over between lanes comes once per VEC * width columns (measured on MI355X, [4096, 16384] float32,
    # widths 1 / 2 / 4 / 8: row sum 58 / 46 / 44 / 45 us, dot product 98 / 93 / 91 / 104 us; float64 [1024, 16384] row
    # sum 94 / 66 / 52 / 61 us).  The columns after the last whole group are walked by one lane, so a width is taken
    # only if it leaves few of them.
    if width is None:
        width = 4
    while width > 1 and p.length < GROUP_LANES * vec * width:
        width //= 2
    group_cols = GROUP_LANES * vec * width
    num_groups = p.length // group_cols
    tail_cols = p.length % group_cols
    # What the wide groups leave over goes through the same lanes in groups of one vector per lane, requested at the
    # start like the rest, and the fewer than 16 * VEC columns after those as one more such group in which the
    # columns past the end of the row are skipped (their loads read the row's last element instead).  A walk of one
    # lane over the columns left over costs more: float32 [4096, 16448], 64 columns left over by groups of 256,
    # 56 us that way against 44 us for 16384 columns.
    small = GROUP_LANES * vec
    narrow0 = num_groups * group_cols           # first column of the narrow groups
    narrow_groups = 0
    if width > 1:
        narrow_groups = tail_cols // small
        tail_cols -= narrow_groups * small
    tail0 = narrow0 + narrow_groups * small     # first column walked by one lane
    # rows that start wherever the one before ends: vectors in memory are then only aligned like their elements
    aligned = dict((t.idx, (p.layouts[t.idx][0] * itemsize) % 16 == 0 and (p.layouts[t.idx][1] * itemsize) % 16 == 0)
                   for t in p.tensors)
    depth = max(1, min(depth or (2 if width == 4 else max(1, 4 // width)), num_groups))
    rows_per_wave = WAVE // GROUP_LANES
    waves = BLOCK // WAVE
    rows_per_block = rows_per_wave * waves

    rank = len(info.workgroup_shape)
    pos_exprs = []
    stride = 1
    strides = [1] * rank
    for k in range(rank - 2, -1, -1):
        stride *= info.workgroup_shape[k + 1]
        strides[k] = stride
    for k in range(rank):
        expr = 'row'
        if k > 0:
            expr = '(row % ' + str(strides[k - 1]) + 'u)'
        pos_exprs.append(expr + ' / ' + str(strides[k]) + 'u')
    loop_tensors = dict((t.idx, t) for t in p.tensors)

    def read_hook(node, tensor, index_name):
        if info.in_loop[node.idx] and tensor.idx in loop_tensors:
            return 'OVL_REDUCE_IN%d' % tensor.io_index
        return None
    emitter = BodyEmitter(info, pos_exprs, read_hook=read_hook, store_hook=None)
    tagged = emitter.emit_tagged()
    range_idx = p.loop_item.node
    prologue = [t for i, t in tagged if i < range_idx]
    body = [t.strip() for i, t in tagged if range_idx < i < p.end_idx]
    epilogue = [t for i, t in tagged if i > p.end_idx]
    counter_name = 'e' + str(p.counter)
    counter_type = CTYPE[info.nodes[p.counter].dtype]
    state = [('e' + str(idx), CTYPE[info.nodes[idx].dtype]) for idx in _carried_state(info, p)]

    src = []
    vnames = {}
    for t in p.tensors:
        ctype = CTYPE[t.dtype]
        if ctype not in vnames:
            vname = 'ovl_reduce_' + ctype.replace(' ', '_') + 'x%d' % vec
            vnames[ctype] = vname
            src.append('typedef %s %s __attribute__((ext_vector_type(%d)));' % (ctype, vname, vec))
            src.append('typedef %s %s_u __attribute__((aligned(%d)));' % (vname, vname, itemsize))
    src.append('')
    args = ['const %s* __restrict__ in%d' % (CTYPE[info.inputs[i].dtype], i) for i in range(len(info.inputs))]
    args += ['%s* __restrict__ out%d' % (CTYPE[info.outputs[i].dtype], i) for i in range(len(info.outputs))]
    src.append('extern "C" __global__ void __launch_bounds__(%d)' % BLOCK)
    src.append('%s(%s) {' % (kernel_name, ', '.join(args)))
    if info.uses_math_tables():
        src.append('    OVL_DECLARE_MATH_TABLES();')
    src.append('    const uint32_t lane = threadIdx.x %% %du;' % WAVE)
    src.append('    const uint32_t part = lane %% %du;              // which columns of a group this lane holds' % GROUP_LANES)
    src.append('    // A wavefront wholly past the last row leaves; single lanes past it shadow the last row instead (all lanes')
    src.append('    // must stay active for the lane-to-lane moves): they load, compute and store exactly what its owners do.')
    src.append('    if ((blockIdx.x * %du + threadIdx.x / %du) * %du >= %du) return;' % (waves, WAVE, rows_per_wave, p.rows))
    src.append('    const uint32_t row_raw = (blockIdx.x * %du + threadIdx.x / %du) * %du + lane / %du;' % (
        waves, WAVE, rows_per_wave, GROUP_LANES))
    src.append('    const uint32_t row = row_raw < %du ? row_raw : %du;' % (p.rows, p.rows - 1))
    for t in p.tensors:
        src.append('    const %s* __restrict__ gin%d = in%d + (uint64_t)row * %dull + %dull + part * %du;' % (
            CTYPE[t.dtype], t.io_index, t.io_index, p.layouts[t.idx][0], p.layouts[t.idx][1], vec * width))
        if narrow_groups:
            src.append('    const %s* __restrict__ gs%d = in%d + (uint64_t)row * %dull + %dull + part * %du;' % (
                CTYPE[t.dtype], t.io_index, t.io_index, p.layouts[t.idx][0], p.layouts[t.idx][1] + narrow0, vec))
        if tail_cols:
            src.append('    const %s* __restrict__ grow%d = in%d + (uint64_t)row * %dull + %dull;' % (
                CTYPE[t.dtype], t.io_index, t.io_index, p.layouts[t.idx][0], p.layouts[t.idx][1]))
    batch = depth
    num_batches = num_groups // batch
    tail = num_groups % batch
    batch_cols = batch * group_cols

    def request_partial():
        # element by element: a vector may cross the end of the row, and of the tensor
        for t in p.tensors:
            src.append('        #pragma unroll')
            src.append('        for (uint32_t u = 0; u < %du; ++u) {' % vec)
            src.append('            const uint32_t column = %du + part * %du + u;' % (tail0, vec))
            src.append('            q%d_z[0][0][u] = grow%d[column < %du ? column : %du];' % (
                t.io_index, t.io_index, p.length, p.length - 1))
            src.append('        }')

    def request(k, batch_expr, nb, suffix, narrow=False):
        for t in p.tensors:
            vname = vnames[CTYPE[t.dtype]]
            mname = vname if aligned[t.idx] and (not narrow or (narrow0 * itemsize) % 16 == 0) else vname + '_u'
            load = '__builtin_nontemporal_load' if 'l' in nt else '*'
            src.append('        #pragma unroll')
            src.append('        for (uint32_t j = 0; j < %du; ++j)' % nb)
            if narrow:
                src.append('            q%d%s[j][0] = %s(reinterpret_cast<const %s*>(gs%d + j * %du));' % (
                    t.io_index, suffix, load, mname, t.io_index, small))
                continue
            src.append('            #pragma unroll')
            src.append('            for (uint32_t w = 0; w < %du; ++w)' % width)
            src.append('                q%d%s[j][w] = %s(reinterpret_cast<const %s*>(gin%d + (%s) * %du + j * %du + w * %du));' % (
                t.io_index, suffix, load, mname, t.io_index, batch_expr, batch_cols, group_cols, vec))

    def process(suffix, batch_expr, refill_expr, nb, narrow=False, partial=False):
        src.append('        {')
        src.append('        const uint32_t b = %s;' % batch_expr)
        src.append('        #pragma unroll')
        src.append('        for (uint32_t j = 0; j < %du; ++j) {' % nb)
        if partial:
            src.append('            const uint32_t col0 = %du + part * %du;' % (tail0, vec))
        elif narrow:
            src.append('            const uint32_t col0 = %du + j * %du + part * %du;' % (narrow0, small, vec))
        else:
            src.append('            const uint32_t col0 = b * %du + j * %du + part * %du;' % (batch_cols, group_cols, vec * width))
        src.append('            #pragma unroll')
        src.append('            for (uint32_t phase = 0; phase < %du; ++phase) {' % GROUP_LANES)
        for name, _ in state:
            src.append('                %s = carry_%s;' % (name, name))
        src.append('                #pragma unroll')
        src.append('                for (uint32_t w = 0; w < %du; ++w) {' % (1 if narrow else width))
        for t in p.tensors:
            src.append('                    const %s xv%d = q%d%s[j][w];' % (
                vnames[CTYPE[t.dtype]], t.io_index, t.io_index, suffix))
        src.append('                    #pragma unroll')
        src.append('                    for (uint32_t u = 0; u < %du; ++u) {' % vec)
        if p.start == 1:
            src.append('                        if (col0 + w * %du + u == 0u) continue;     // column 0: done before the loop' % vec)
        if partial:
            src.append('                        if (col0 + u >= %du) continue;              // past the end of the row' % p.length)
        src.append('                        OVL_REDUCE_STEP(col0 + w * %du + u)' % vec)
        src.append('                    }')
        src.append('                }')
        for name, _ in state:
            src.append('                carry_%s = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry_%s, %s);' % (name, name, name))
        src.append('            }')
        src.append('            // the last lane of the group finished the group: its state is the carry into the next one')
        for name, _ in state:
            src.append('            carry_%s = ovl_dpp_move<OVL_DPP_ROW_ROR1>(carry_%s, %s);' % (name, name, name))
        src.append('        }')
        if refill_expr is not None:
            src.append('        __builtin_amdgcn_sched_barrier(0);')
            request(None, refill_expr, nb, suffix)
            src.append('        __builtin_amdgcn_sched_barrier(0);')
        src.append('        }')

    sets = max(2, min(sets or 2, num_batches)) if num_batches > 1 else 1
    src.append('    // %d register sets of %d groups each per tensor: one is consumed while the other is in flight' % (sets, batch))
    for t in p.tensors:
        vname = vnames[CTYPE[t.dtype]]
        src.append('    %s %s;' % (vname, ', '.join('q%d_%d[%d][%d]' % (t.io_index, k, batch, width) for k in range(sets))))
        if tail:
            src.append('    %s q%d_t[%d][%d];       // the groups that end the row, requested now and held until then' % (
                vname, t.io_index, tail, width))
        if narrow_groups:
            src.append('    %s q%d_s[%d][1];       // ... and the groups of one vector per lane after those' % (
                vname, t.io_index, narrow_groups))
        if tail_cols:
            src.append('    %s q%d_z[1][1];        // ... and the columns after the last whole group' % (vname, t.io_index))
    src.append('    {')
    for k in range(sets):
        request(k, '%du' % k, batch, '_%d' % k)
    if tail:
        request(None, '%du' % num_batches, tail, '_t')
    if narrow_groups:
        request(None, '0u', narrow_groups, '_s', narrow=True)
    if tail_cols:
        request_partial()
    src.append('    }')
    src.append('    // the statements the worker runs before its loop, in every lane')
    for stmt in prologue:
        src.append('    ' + stmt)
    for name, stype in state:
        src.append('    %s carry_%s = %s;' % (stype, name, name))
    for t in p.tensors:
        src.append('#define OVL_REDUCE_IN%d xv%d[u]' % (t.io_index, t.io_index))
    src.append('#define OVL_REDUCE_STEP(column) { %s = (%s)(column); %s }' % (counter_name, counter_type, ' '.join(body)))
    rounds = num_batches // sets
    last = num_batches - 1
    if rounds:
        src.append('    #pragma unroll 1')
        src.append('    for (uint32_t b0 = 0; b0 < %du; b0 += %du) {' % (rounds * sets, sets))
        # past the end a set is refilled with the last batch again, which keeps the loop free of branches
        for k in range(sets):
            process('_%d' % k, 'b0 + %du' % k, '(b0 + %du < %du ? b0 + %du : %du)' % (k + sets, num_batches, k + sets, last), batch)
        src.append('    }')
    for k in range(num_batches % sets):
        src.append('    {')
        process('_%d' % k, '%du' % (rounds * sets + k), None, batch)
        src.append('    }')
    if tail:
        src.append('    {')
        process('_t', '%du' % num_batches, None, tail)
        src.append('    }')
    if narrow_groups:
        src.append('    {')
        process('_s', '0u', None, narrow_groups, narrow=True)
        src.append('    }')
    if tail_cols:
        src.append('    {')
        process('_z', '0u', None, 1, narrow=True, partial=True)
        src.append('    }')
    src.append('    // Lane 0 of the row holds the state that leaves the last group: it runs the statements that follow the')
    src.append('    // worker\'s loop.')
    src.append('    if (part == 0u) {')
    for name, _ in state:
        src.append('        %s = carry_%s;' % (name, name))
    for stmt in epilogue:
        src.append('        ' + stmt.strip())
    src.append('    }')
    for t in p.tensors:
        src.append('#undef OVL_REDUCE_IN%d' % t.io_index)
    src.append('#undef OVL_REDUCE_STEP')
    src.append('}')

    launch = {
        'template': 'rowreduce',
        'vec': vec,
        'block': BLOCK,
        'blocks_needed': (p.rows + rows_per_block - 1) // rows_per_block,
        'align': dict((('in', t.io_index), 16 if aligned[t.idx] else itemsize) for t in p.tensors),
        'vector_loads': len(p.tensors),
        'vector_stores': 0,
    }
    return '\n'.join(src) + '\n', launch


TREE_OPS = (lang.ADD, lang.MULTIPLY, lang.MIN, lang.MAX)


def tree_plan(info):
    """
    (ScanPlan, operation code) when the DAG is exactly ``acc = x[., 0]; out[., 0] = acc; for i in 1..n-1:
    acc = op(acc, x[., i]); out[., i] = acc`` with op one of +, *, min, max: the scans whose operands may be
    associated as a tree when the caller gives up the sequential order (math mode 'fast').  Else None.
    """
    p = plan(info)
    if p is None:
        return None
    state = _carried_state(info, p)
    if len(state) != 1:
        return None
    s = state[0]
    if info.nodes[s].dtype != p.x.dtype:
        return None
    loads = {False: [], True: []}
    assigns = {False: [], True: []}
    stores = {False: [], True: []}
    for node in info.nodes:
        inside = bool(info.in_loop[node.idx])
        if node.code == lang.READ_TENSOR and info.nodes[node.ops[0]].code == lang.INPUT:
            loads[inside].append(node)
        elif node.code == lang.ASSIGN_VARIABLE and node.ops[0] != p.counter:
            assigns[inside].append(node)
        elif node.code == lang.ASSIGN_TENSOR:
            stores[inside].append(node)
    for inside in (False, True):
        if len(loads[inside]) != 1 or len(assigns[inside]) != 1 or len(stores[inside]) != 1:
            return None
        assign, store = assigns[inside][0], stores[inside][0]
        if assign.ops[0] != s or store.ops[2] != s or store.idx < assign.idx:
            return None
    if assigns[False][0].ops[1] != loads[False][0].idx:         # acc = x[., 0]
        return None
    update = info.nodes[assigns[True][0].ops[1]]                # acc = op(acc, x[., i]) in either operand order
    if update.code not in TREE_OPS or sorted(update.ops) != sorted([s, loads[True][0].idx]):
        return None
    return p, update.code


def _tree_unit(code, dtype):
    """C text of the value u with op(u, x) == x for every x (for the sum -0, which also keeps the sign of a zero)."""
    floating = dtype in (lang.FLOAT32, lang.FLOAT64)
    if code == lang.ADD:
        return '-0.0' if floating else '0'
    if code == lang.MULTIPLY:
        return '1'
    limits = {lang.INT32: ('INT32_MIN', 'INT32_MAX'), lang.INT64: ('INT64_MIN', 'INT64_MAX'),
              lang.UINT32: ('0u', 'UINT32_MAX'), lang.UINT64: ('0ull', 'UINT64_MAX')}
    if floating:
        lowest, highest = '(-__builtin_inf())', '__builtin_inf()'
    else:
        lowest, highest = limits[dtype]
    return highest if code == lang.MIN else lowest


def generate_tree(info, kernel_name, ahead=8):
    """
    The reassociating row scan: one workgroup per row, the row in steps of 256 vectors.  Every thread scans its own
    128-bit vector, the threads' totals are scanned over the wavefront with lane-to-lane moves, the four wavefront
    totals go through a double-buffered LDS array (one barrier per step), the total of the steps before travels in a
    register; ``ahead`` steps of loads stay in flight.  The kernel runs at the speed of memory, but associates the
    operands as a tree: its results differ from the sequential recurrence by rounding, so it is only chosen in the
    'fast' math mode.
    """
    from .body import binary_text
    p, code = tree_plan(info)
    ctype = CTYPE[p.x.dtype]
    vec = p.vec
    if p.length % vec != 0:
        raise ValueError('the reassociating scan needs rows of whole vectors')
    step_cols = BLOCK * vec
    steps = (p.length + step_cols - 1) // step_cols
    ahead = max(1, min(ahead, steps))
    unit = '(%s)(%s)' % (ctype, _tree_unit(code, p.x.dtype))
    src = []
    src.append('typedef %s ovl_scan_vec __attribute__((ext_vector_type(%d)));' % (ctype, vec))
    unsigned = {lang.INT32: 'uint32_t', lang.INT64: 'uint64_t'}.get(p.x.dtype)
    if unsigned is not None and code in (lang.ADD, lang.MULTIPLY):
        # partial sums and products of a tree may pass the limits of a signed type where the sequential order does
        # not: formed in the unsigned type (arithmetic modulo 2^n, always defined) they end in the same bits
        text = '(%s)(%s)' % (ctype, binary_text(code, p.x.dtype, '(%s)(a)' % unsigned, '(%s)(b)' % unsigned))
        src.append('#define OVL_TREE_OP(a, b) (%s)' % text)
    else:
        src.append('#define OVL_TREE_OP(a, b) (%s)' % binary_text(code, p.x.dtype, 'a', 'b'))
    src.append('')
    src.append('extern "C" __global__ void __launch_bounds__(%d)' % BLOCK)
    src.append('%s(const %s* __restrict__ in%d, %s* __restrict__ out%d) {' % (
        kernel_name, ctype, p.x.io_index, ctype, p.out.io_index))
    src.append('    __shared__ %s wave_totals[2][%d];' % (ctype, BLOCK // WAVE))
    src.append('    const uint32_t lane = threadIdx.x %% %du, wave = threadIdx.x / %du;' % (WAVE, WAVE))
    src.append('    const %s* __restrict__ in_row = in%d + (uint64_t)blockIdx.x * %dull;' % (ctype, p.x.io_index, p.length))
    src.append('    %s* __restrict__ out_row = out%d + (uint64_t)blockIdx.x * %dull;' % (ctype, p.out.io_index, p.length))
    src.append('    const %s unit = %s;' % (ctype, unit))
    src.append('    auto combine = [](%s a, %s b) -> %s { return OVL_TREE_OP(a, b); };' % (ctype, ctype, ctype))
    src.append('    // a vector past the end of the row holds the unit and is not stored')
    src.append('    auto fetch = [&](uint32_t step) -> ovl_scan_vec {')
    src.append('        const uint32_t col = step * %du + threadIdx.x * %du;' % (step_cols, vec))
    src.append('        ovl_scan_vec r;')
    src.append('        if (step < %du && col < %du) r = *reinterpret_cast<const ovl_scan_vec*>(in_row + col);' % (steps, p.length))
    src.append('        else')
    src.append('            #pragma unroll')
    src.append('            for (uint32_t u = 0; u < %du; ++u) r[u] = unit;' % vec)
    src.append('        return r;')
    src.append('    };')
    src.append('    %s carry = unit;' % ctype)
    src.append('    uint32_t buffer = 0;')
    src.append('    // %d steps of loads are always in flight: a register is refilled as soon as its vector has been taken' % ahead)
    src.append('    ovl_scan_vec v[%d];' % ahead)
    src.append('    #pragma unroll')
    src.append('    for (uint32_t a = 0; a < %du; ++a) v[a] = fetch(a);' % ahead)
    src.append('    for (uint32_t s0 = 0; s0 < %du; s0 += %du) {' % (steps, ahead))
    src.append('        #pragma unroll')
    src.append('        for (uint32_t a = 0; a < %du; ++a) {' % ahead)
    src.append('            if (s0 + a >= %du) break;        // uniform over the workgroup' % steps)
    src.append('            const uint32_t col = (s0 + a) * %du + threadIdx.x * %du;' % (step_cols, vec))
    src.append('            ovl_scan_vec mine = v[a];')
    src.append('            v[a] = fetch(s0 + a + %du);' % ahead)
    src.append('            #pragma unroll')
    src.append('            for (uint32_t u = 1; u < %du; ++u) mine[u] = combine(mine[u - 1], mine[u]);' % vec)
    src.append('            const %s inclusive = ovl_wave_inclusive_scan(mine[%d], unit, combine);' % (ctype, vec - 1))
    src.append('            const %s before_me = ovl_wave_shift_up(inclusive, unit);      // total of the lanes below' % ctype)
    src.append('            if (lane == %du) wave_totals[buffer][wave] = inclusive;' % (WAVE - 1))
    src.append('            __syncthreads();')
    src.append('            %s base = carry, all = carry;' % ctype)
    src.append('            #pragma unroll')
    src.append('            for (uint32_t w = 0; w < %du; ++w) {' % (BLOCK // WAVE))
    src.append('                const %s t = wave_totals[buffer][w];' % ctype)
    src.append('                if (w < wave) base = combine(base, t);')
    src.append('                all = combine(all, t);')
    src.append('            }')
    src.append('            base = combine(base, before_me);')
    src.append('            #pragma unroll')
    src.append('            for (uint32_t u = 0; u < %du; ++u) mine[u] = combine(base, mine[u]);' % vec)
    src.append('            if (col < %du) __builtin_nontemporal_store(mine, reinterpret_cast<ovl_scan_vec*>(out_row + col));' % p.length)
    src.append('            carry = all;')
    src.append('            // the next step writes the other buffer; this one is written again only behind another barrier')
    src.append('            buffer ^= 1u;')
    src.append('        }')
    src.append('    }')
    src.append('}')
    src.append('#undef OVL_TREE_OP')
    launch = {
        'template': 'treescan',
        'vec': vec,
        'block': BLOCK,
        'blocks_needed': p.rows,
        'align': {('in', p.x.io_index): 16, ('out', p.out.io_index): 16},
        'vector_loads': 1,
        'vector_stores': 1,
    }
    return '\n'.join(src) + '\n', launch


def _default_interleave(rows, vec):
    """Rows per lane group of the lane-skewed scan when the caller does not say."""
    return 1


def _for_slot(text, slot):
    """The per-row names of a source fragment renamed for the row with number ``slot`` of a lane group (slot 0 keeps
    the plain names): expression variables e<N> and their carries, position, row, the row's pointers, register sets,
    output vectors and the step macro."""
    if slot == 0:
        return text
    suffix = '_r%d' % slot
    text = re.sub(r'\b(carry_e\d+|e\d+|position|row_raw|row|gin\d*|gout\d*|grow\d*|orow\d*|q\d+|qt\d*|qz\d*|ov\d*|xv\d*|first_out\d*|OVL_SCAN_STEP_DRY|OVL_SCAN_STEP)\b',
                  lambda m: m.group(1) + suffix, text)
    return text


def generate_skewed(info, kernel_name, depth=None, sets=None, nt='s', width=None, interleave=None, split=None):
    p = skew_plan(info)
    assert p is not None
    ctype = CTYPE[p.x.dtype]
    vec = p.vec
    # width = 128-bit vectors per lane and phase: a lane owns vec * width consecutive columns of a group, so the
    # hand-over to the neighbouring lane (a move and its wait states on the critical path of the recurrence) comes
    # once per vec * width columns
    # (measured on MI355X: float64 [1024, 16384] 104 us with one vector per phase, 76 us with two, 126 us with four,
    # whose 64-byte stride between lanes wastes the memory pipeline; float32 [4096, 16384], which runs at the speed of
    # memory, 85 us with one and 111 us with two)
    if width is None:
        width = 2 if vec == 2 else 1
    while width > 1 and (p.length < GROUP_LANES * vec * width or
                         (p.length % (GROUP_LANES * vec) == 0 and p.length % (GROUP_LANES * vec * width) != 0)):
        width //= 2
    group_cols = GROUP_LANES * vec * width
    num_groups = p.length // group_cols
    tail_cols = p.length % group_cols           # columns after the last whole group: scanned by one lane per row
    aligned = (p.length * ITEMSIZE[p.x.dtype]) % 16 == 0
    # interleave = rows per group of sixteen lanes.  With few rows there are fewer wavefronts than SIMDs and each runs
    # at the latency of its one recurrence; a lane group that carries two rows has two independent recurrences whose
    # additions and hand-overs fill each other's wait states.
    if interleave is None:
        interleave = _default_interleave(p.rows, vec)
    interleave = max(1, min(int(interleave), 4))
    slots = list(range(interleave))
    rows_per_wave = (WAVE // GROUP_LANES) * interleave
    waves = BLOCK // WAVE
    rows_per_block = rows_per_wave * waves
    if depth is None:
        # measured on MI355X: request bursts of 1 KiB per row are the fastest
        depth = max(1, 4 // width)
    # (a row whose number of groups is not a multiple of the burst ends in one shorter burst; before, the burst was
    # halved until it divided the row, and float32 [4096, 16448], 257 groups, took 177 us against 85 us for 16384)
    depth = max(1, min(depth, num_groups))

    rank = len(info.workgroup_shape)
    pos_exprs = []
    stride = 1
    strides = [1] * rank
    for k in range(rank - 2, -1, -1):
        stride *= info.workgroup_shape[k + 1]
        strides[k] = stride
    for k in range(rank):
        expr = 'row'
        if k > 0:
            expr = '(row % ' + str(strides[k - 1]) + 'u)'
        pos_exprs.append(expr + ' / ' + str(strides[k]) + 'u')

    # the inputs the body reads, numbered in the order of their first use: each has its pointer, register sets and
    # vector of the moment under a name with that number (the first without one)
    # Costly work that only the outputs need: the sixteen phases then run with the stores dropped (the compiler removes
    # what only they used), and one more pass over the lane's columns, from the carried state that is exact by then,
    # computes and stores the outputs (float32 [2048, 8192], c = f * c + i * g, h = o * tanh(c): 968 -> 313 us).
    split = _heavy_outside_recurrence(info, p) if split is None else bool(split)
    number = dict((t.idx, k) for k, t in enumerate(p.xs))
    out_number = dict((t.idx, k) for k, t in enumerate(p.outs))
    tag = lambda k: '' if k == 0 else str(k)

    def set_name(regs, k):
        if k == 0:
            return regs
        return 'qt%d' % k if regs == 'qt' else 'q%d' % (int(regs[1:]) + 10 * k)

    emitter = BodyEmitter(info, pos_exprs,
                          read_hook=lambda node, tensor, idx: 'OVL_SCAN_IN_T%d' % number[tensor.idx],
                          store_hook=lambda node, tensor, idx, value: 'OVL_SCAN_OUT_T%d(' % out_number[tensor.idx] + value + ');')
    tagged = emitter.emit_tagged()
    range_idx = p.loop_item.node
    end_idx = max(i for i, _ in tagged)
    prologue = [t for i, t in tagged if i < range_idx]
    body = [t.strip() for i, t in tagged if range_idx < i < end_idx]
    counter_name = 'e' + str(p.counter)
    counter_type = CTYPE[info.nodes[p.counter].dtype]
    state = [('e' + str(idx), CTYPE[info.nodes[idx].dtype]) for idx in _carried_state(info, p)]

    vname = 'ovl_scan_vec'
    src = []

    def emit(lines, per_row=True):
        """Append source lines: once, or once per row of the lane group with that row's names."""
        for slot in (slots if per_row else [0]):
            for line in lines:
                src.append(_for_slot(line, slot))

    src.append('typedef %s %s __attribute__((ext_vector_type(%d)));' % (ctype, vname, vec))
    mname = vname
    if not aligned:
        # rows start wherever the one before ends: vectors in memory are only aligned like their elements
        mname = vname + '_u'
        src.append('typedef %s %s __attribute__((aligned(%d)));' % (vname, mname, ITEMSIZE[p.x.dtype]))
    src.append('')
    src.append('extern "C" __global__ void __launch_bounds__(%d)' % BLOCK)
    src.append('%s(%s, %s) {' % (
        kernel_name, ', '.join('const %s* __restrict__ in%d' % (CTYPE[info.inputs[i].dtype], i) for i in range(len(info.inputs))),
        ', '.join('%s* __restrict__ out%d' % (CTYPE[info.outputs[i].dtype], i) for i in range(len(info.outputs)))))
    if info.uses_math_tables():
        src.append('    OVL_DECLARE_MATH_TABLES();')
    src.append('    const uint32_t lane = threadIdx.x %% %du;' % WAVE)
    src.append('    const uint32_t part = lane %% %du;              // which VEC columns of a group this lane holds' % GROUP_LANES)
    src.append('    // A wavefront wholly past the last row leaves; single lanes past it shadow the last row instead (all lanes')
    src.append('    // must stay active for the lane-to-lane moves): they load, compute and store exactly what its owners do.')
    src.append('    if ((blockIdx.x * %du + threadIdx.x / %du) * %du >= %du) return;' % (waves, WAVE, rows_per_wave, p.rows))
    for slot in slots:
        if interleave == 1:
            raw = '(blockIdx.x * %du + threadIdx.x / %du) * %du + lane / %du' % (waves, WAVE, rows_per_wave, GROUP_LANES)
        else:
            raw = '(blockIdx.x * %du + threadIdx.x / %du) * %du + (lane / %du) * %du + %du' % (
                waves, WAVE, rows_per_wave, GROUP_LANES, interleave, slot)
        src.append(_for_slot('    const uint32_t row_raw = %s;' % raw, slot))
    emit(['    const uint32_t row = row_raw < %du ? row_raw : %du;' % (p.rows, p.rows - 1)] +
         ['    const %s* __restrict__ gin%s = in%d + (uint64_t)row * %dull + part * %du;' % (
             ctype, tag(k), t.io_index, p.length, vec * width) for k, t in enumerate(p.xs)] +
         ['    %s* __restrict__ gout%s = out%d + (uint64_t)row * %dull + part * %du;' % (
             ctype, tag(k), t.io_index, p.length, vec * width) for k, t in enumerate(p.outs)] +
         (['    const %s* __restrict__ grow%s = in%d + (uint64_t)row * %dull;' % (ctype, tag(k), t.io_index, p.length)
           for k, t in enumerate(p.xs)] +
          ['    %s* __restrict__ orow%s = out%d + (uint64_t)row * %dull;' % (ctype, tag(k), t.io_index, p.length)
           for k, t in enumerate(p.outs)]
          if tail_cols else []))
    # measured on MI355X (float32 [4096, 16384]): non-temporal stores with plain loads 85 us, hint on both 100 us,
    # on the loads only 90 us, on neither 102 us
    batch = depth
    num_batches = num_groups // batch
    tail = num_groups % batch               # groups of the shorter burst that ends the row
    batch_cols = batch * group_cols

    def request(regs, batch_expr, nb=None):
        """All loads of one batch (of nb groups), back to back: every row is read in runs of batch * 256 bytes."""
        nb = nb or batch
        for k in range(len(p.xs)):
            lines = ['        #pragma unroll',
                     '        for (uint32_t j = 0; j < %du; ++j)' % nb,
                     '            #pragma unroll',
                     '            for (uint32_t w = 0; w < %du; ++w)' % width]
            if 'l' in nt:
                lines.append('                %s[j][w] = __builtin_nontemporal_load(reinterpret_cast<const %s*>(gin%s + (%s) * %du + j * %du + w * %du));' % (
                    set_name(regs, k), mname, tag(k), batch_expr, batch_cols, group_cols, vec))
            else:
                lines.append('                %s[j][w] = *(reinterpret_cast<const %s*>(gin%s + (%s) * %du + j * %du + w * %du));' % (
                    set_name(regs, k), mname, tag(k), batch_expr, batch_cols, group_cols, vec))
            emit(lines)

    def process(regs, batch_expr, refill_expr, nb=None):
        nb = nb or batch
        src.append('        {')
        src.append('        const uint32_t b = %s;' % batch_expr)
        emit(['        %s ov%s[%d][%d];' % (vname, tag(k), nb, width) for k in range(len(p.outs))])
        src.append('        #pragma unroll')
        src.append('        for (uint32_t j = 0; j < %du; ++j) {' % nb)
        src.append('            const uint32_t col0 = b * %du + j * %du + part * %du;' % (batch_cols, group_cols, vec * width))
        src.append('            const bool first_column = (j == 0u) && (b == 0u) && (part == 0u);')
        src.append('            #pragma unroll')
        src.append('            for (uint32_t phase = 0; phase < %du; ++phase) {' % GROUP_LANES)
        # the rows of a lane group advance column by column, side by side: their recurrences are independent, and in
        # this order the additions and hand-overs of one row fill the wait states of the other
        emit(['                %s = carry_%s;' % (name, name) for name, _ in state])
        src.append('                #pragma unroll')
        src.append('                for (uint32_t w = 0; w < %du; ++w) {' % width)
        emit(['                    const %s xv%s = %s[j][w];' % (vname, tag(k), set_name(regs, k)) for k in range(len(p.xs))])
        src.append('                    #pragma unroll')
        src.append('                    for (uint32_t u = 0; u < %du; ++u) {' % vec)
        if split:
            emit(['                        if (w == 0u && u == 0u && first_column) continue;',
                  '                        OVL_SCAN_STEP_DRY(col0 + w * %du + u)' % vec])
        else:
            emit(['                        if (w == 0u && u == 0u && first_column) { %s }' % ' '.join(
                      'ov%s[j][0][0] = first_out%s;' % (tag(k), tag(k)) for k in range(len(p.outs))),
                  '                        else OVL_SCAN_STEP(col0 + w * %du + u)' % vec])
        src.append('                    }')
        src.append('                }')
        emit(['                carry_%s = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry_%s, %s);' % (name, name, name)
              for name, _ in state])
        src.append('            }')
        if split:
            # every lane's carried state is exact now: one pass that computes and keeps the outputs
            emit(['            %s = carry_%s;' % (name, name) for name, _ in state])
            src.append('            #pragma unroll')
            src.append('            for (uint32_t w = 0; w < %du; ++w) {' % width)
            emit(['                const %s xv%s = %s[j][w];' % (vname, tag(k), set_name(regs, k)) for k in range(len(p.xs))])
            src.append('                #pragma unroll')
            src.append('                for (uint32_t u = 0; u < %du; ++u) {' % vec)
            emit(['                    if (w == 0u && u == 0u && first_column) { %s }' % ' '.join(
                      'ov%s[j][0][0] = first_out%s;' % (tag(k), tag(k)) for k in range(len(p.outs))),
                  '                    else OVL_SCAN_STEP(col0 + w * %du + u)' % vec])
            src.append('                }')
            src.append('            }')
        src.append('            // the last lane of the group finished the group: its state is the carry into the next one')
        emit(['            carry_%s = ovl_dpp_move<OVL_DPP_ROW_ROR1>(carry_%s, %s);' % (name, name, name)
              for name, _ in state])
        src.append('        }')
        src.append('        // The scheduling fences keep the memory traffic of a batch together, after its arithmetic: runs of')
        src.append('        // batch * 256 bytes per row, and no load is moved ahead of the last use of the registers it fills.')
        src.append('        __builtin_amdgcn_sched_barrier(0);')
        for k in range(len(p.outs)):
            lines = ['        #pragma unroll',
                     '        for (uint32_t j = 0; j < %du; ++j)' % nb,
                     '            #pragma unroll',
                     '            for (uint32_t w = 0; w < %du; ++w)' % width]
            if 's' in nt:
                lines.append('                __builtin_nontemporal_store(ov%s[j][w], reinterpret_cast<%s*>(gout%s + b * %du + j * %du + w * %du));' % (
                    tag(k), mname, tag(k), batch_cols, group_cols, vec))
            else:
                lines.append('                *(reinterpret_cast<%s*>(gout%s + b * %du + j * %du + w * %du)) = ov%s[j][w];' % (
                    mname, tag(k), batch_cols, group_cols, vec, tag(k)))
            emit(lines)
        if refill_expr is not None:
            request(regs, refill_expr)
        src.append('        __builtin_amdgcn_sched_barrier(0);')
        src.append('        }')

    sets = max(2, min(sets or 2, num_batches)) if num_batches > 1 else 1
    src.append('    // %d register sets of %d groups each: one is consumed while the others are in flight' % (sets, batch))
    emit(['    %s %s;' % (vname, ', '.join('%s[%d][%d]' % (set_name('q%d' % k, t), batch, width) for k in range(sets)))
          for t in range(len(p.xs))])
    if tail:
        src.append('    // ... and the %d groups that end the row, requested now and held until the end' % tail)
        emit(['    %s %s[%d][%d];' % (vname, set_name('qt', t), tail, width) for t in range(len(p.xs))])
    tail0 = num_groups * group_cols
    if tail_cols:
        src.append('    // ... and the columns after the last whole group, element by element (a vector may cross the end of')
        src.append('    // the row): they run as one more group in which the columns past the end are skipped')
        emit(['    %s qz%s[%d];' % (vname, tag(t), width) for t in range(len(p.xs))])
    src.append('    {')
    for k in range(sets if num_batches else 0):
        request('q%d' % k, '%du' % k)
    if tail:
        request('qt', '%du' % num_batches, tail)
    if tail_cols:
        for k in range(len(p.xs)):
            emit(['        #pragma unroll',
                  '        for (uint32_t w = 0; w < %du; ++w)' % width,
                  '            #pragma unroll',
                  '            for (uint32_t u = 0; u < %du; ++u) {' % vec,
                  '                const uint32_t column = %du + part * %du + w * %du + u;' % (tail0, vec * width, vec),
                  '                qz%s[w][u] = grow%s[column < %du ? column : %du];' % (tag(k), tag(k), p.length, p.length - 1),
                  '            }'])
    src.append('    }')
    src.append('    // first column: the statements the worker runs before its loop, in every lane')
    for slot in slots:
        emit_one = lambda lines: src.extend(_for_slot(line, slot) for line in lines)
        emit_one(['    %s first_out%s;' % (ctype, tag(k)) for k in range(len(p.outs))])
        for k, t in enumerate(p.xs):
            src.append('#define OVL_SCAN_IN_T%d (in%d[(uint64_t)%s * %dull])' % (
                k, t.io_index, _for_slot('row', slot), p.length))
        for k in range(len(p.outs)):
            src.append('#define OVL_SCAN_OUT_T%d(value) %s = (value)' % (k, _for_slot('first_out' + tag(k), slot)))
        emit_one(['    ' + stmt for stmt in prologue])
        for k in range(len(p.xs)):
            src.append('#undef OVL_SCAN_IN_T%d' % k)
        for k in range(len(p.outs)):
            src.append('#undef OVL_SCAN_OUT_T%d' % k)
        emit_one(['    %s carry_%s = %s;' % (stype, name, name) for name, stype in state])
    for slot in slots:
        # (the output vector is named in the step macro itself, so that every row writes its own)
        src.append(_for_slot('#define OVL_SCAN_STEP(column) { %s = (%s)(column); %s }' % (
            counter_name, counter_type, ' '.join(body)), slot).replace(
                'OVL_SCAN_OUT_T', 'OVL_SCAN_OUT_R%d_T' % slot).replace('OVL_SCAN_IN', 'OVL_SCAN_IN_R%d' % slot))
        if split:
            src.append(_for_slot('#define OVL_SCAN_STEP_DRY(column) { %s = (%s)(column); %s }' % (
                counter_name, counter_type, ' '.join(body)), slot).replace(
                    'OVL_SCAN_OUT_T', 'OVL_SCAN_DROP_T').replace('OVL_SCAN_IN', 'OVL_SCAN_IN_R%d' % slot))
        for k in range(len(p.xs)):
            src.append('#define OVL_SCAN_IN_R%d_T%d %s[u]' % (slot, k, _for_slot('xv' + tag(k), slot)))
        for k in range(len(p.outs)):
            src.append('#define OVL_SCAN_OUT_R%d_T%d(value) %s[j][w][u] = (value)' % (
                slot, k, _for_slot('ov' + tag(k), slot)))
            if split and slot == 0:
                src.append('#define OVL_SCAN_DROP_T%d(value) (void)(value)' % k)
    rounds = num_batches // sets
    last = num_batches - 1
    if rounds:
        src.append('    #pragma unroll 1')
        src.append('    for (uint32_t b0 = 0; b0 < %du; b0 += %du) {' % (rounds * sets, sets))
        # past the end a set is refilled with the last batch again, which keeps the loop free of branches
        for k in range(sets):
            process('q%d' % k, 'b0 + %du' % k, '(b0 + %du < %du ? b0 + %du : %du)' % (k + sets, num_batches, k + sets, last))
        src.append('    }')
    for k in range(num_batches % sets):
        src.append('    {')
        process('q%d' % k, '%du' % (rounds * sets + k), None)
        src.append('    }')
    if tail:
        src.append('    {')
        process('qt', '%du' % num_batches, None, tail)
        src.append('    }')
    if tail_cols:
        # The columns after the last whole group (fewer than one lane group's worth): one more group of one vector per
        # lane in which the columns past the end of the row are skipped, stored element by element.  (A walk of one
        # lane over these columns waits for every load in turn: 0.2 us per column.)
        src.append('    {')
        emit(['        %s ov%s[1][%d];' % (vname, tag(k), width) for k in range(len(p.outs))])
        src.append('        const uint32_t col0 = %du + part * %du;' % (tail0, vec * width))
        src.append('        const uint32_t j = 0u;')
        src.append('        #pragma unroll')
        src.append('        for (uint32_t phase = 0; phase < %du; ++phase) {' % GROUP_LANES)
        emit(['            %s = carry_%s;' % (name, name) for name, _ in state])
        src.append('            #pragma unroll')
        src.append('            for (uint32_t w = 0; w < %du; ++w) {' % width)
        emit(['                const %s xv%s = qz%s[w];' % (vname, tag(k), tag(k)) for k in range(len(p.xs))])
        src.append('                #pragma unroll')
        src.append('                for (uint32_t u = 0; u < %du; ++u) {' % vec)
        src.append('                    if (col0 + w * %du + u >= %du) continue;' % (vec, p.length))
        emit(['                    %s(col0 + w * %du + u)' % ('OVL_SCAN_STEP_DRY' if split else 'OVL_SCAN_STEP', vec)])
        src.append('                }')
        src.append('            }')
        emit(['            carry_%s = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry_%s, %s);' % (name, name, name)
              for name, _ in state])
        src.append('        }')
        if split:
            emit(['        %s = carry_%s;' % (name, name) for name, _ in state])
            src.append('        #pragma unroll')
            src.append('        for (uint32_t w = 0; w < %du; ++w) {' % width)
            emit(['            const %s xv%s = qz%s[w];' % (vname, tag(k), tag(k)) for k in range(len(p.xs))])
            src.append('            #pragma unroll')
            src.append('            for (uint32_t u = 0; u < %du; ++u) {' % vec)
            src.append('                if (col0 + w * %du + u >= %du) continue;' % (vec, p.length))
            emit(['                OVL_SCAN_STEP(col0 + w * %du + u)' % vec])
            src.append('            }')
            src.append('        }')
        for k in range(len(p.outs)):
            emit(['        #pragma unroll',
                  '        for (uint32_t w = 0; w < %du; ++w)' % width,
                  '            #pragma unroll',
                  '            for (uint32_t u = 0; u < %du; ++u)' % vec,
                  '                if (col0 + w * %du + u < %du) orow%s[col0 + w * %du + u] = ov%s[0][w][u];' % (
                      vec, p.length, tag(k), vec, tag(k))])
        src.append('    }')
    for slot in slots:
        src.append('#undef %s' % _for_slot('OVL_SCAN_STEP', slot))
        if split:
            src.append('#undef %s' % _for_slot('OVL_SCAN_STEP_DRY', slot))
        for k in range(len(p.outs)):
            src.append('#undef OVL_SCAN_OUT_R%d_T%d' % (slot, k))
            if split and slot == 0:
                src.append('#undef OVL_SCAN_DROP_T%d' % k)
        for k in range(len(p.xs)):
            src.append('#undef OVL_SCAN_IN_R%d_T%d' % (slot, k))
    src.append('}')

    row_align = 16 if aligned else ITEMSIZE[p.x.dtype]
    launch = {
        'template': 'skewscan',
        'vec': vec,
        'block': BLOCK,
        'blocks_needed': (p.rows + rows_per_block - 1) // rows_per_block,
        'align': dict([(('in', t.io_index), row_align) for t in p.xs] +
                      [(('out', t.io_index), row_align) for t in p.outs]),
        'vector_loads': len(p.xs),
        'vector_stores': len(p.outs),
    }
    return '\n'.join(src) + '\n', launch
