"""
The map kernel template: one thread processes VEC consecutive workers along the last workgroup dimension.

Replaces the reference's one-thread-per-worker CUDA template (opveclib/expression.py:595-609, launched with 32
threads per block, expression.py:696-698 and operator.py:30).  For gfx950 the template

* gives each thread VEC workers that are neighbours along the last workgroup dimension, so that every tensor access
  whose flat index is ``base(outer position) + last position + constant`` becomes one aligned vector load or store of
  up to 16 bytes per thread, fully coalesced across the 64 lanes of a wavefront;
* hoists those loads to the top of the thread's iteration (all loads in flight before the arithmetic starts) and
  buffers the stores in registers until the end of the iteration;
* launches one 256-thread workgroup (four wavefronts) per 256 vectors, in address order, so that at any time the
  whole chip streams through one neighbourhood of each tensor (measured on MI355X: 6.85 TB/s for a three-stream
  float32 add, against 5.3 TB/s for a grid-stride loop over 8 workgroups per CU); the vector stores or the vector
  loads carry the non-temporal hint, whichever was measured to be faster for the kernel's mix of streams;
* keeps every other access (gathers, scatters, accesses inside loops or behind non-exhaustive conditions) as the
  scalar access the worker function asked for.

With VEC = 1 it is the fully general fallback for any DAG.
"""

from .. import language as lang
from .analysis import ITEMSIZE
from .body import BodyEmitter, CTYPE

BLOCK = 256
# largest grid the generated entry points launch: 2^24 - 1 workgroups of 256 threads keep the number of threads of a
# launch, and with it gridDim.x * 256 inside the kernels, below 2^32
MAX_GRID = (1 << 24) - 1
SCALAR_TABLE_GRID = 4096        # workgroups of a one-element-per-thread kernel that copies the math tables


class Access(object):
    """A group of identical tensor accesses (same tensor, same affine index) realised as one vector."""

    def __init__(self, tensor, aff, reg):
        self.tensor = tensor
        self.aff = aff
        self.reg = reg


def _index_expr(aff, pos_names, wide):
    """C expression of an affine index in the position variables of lane 0."""
    ctype = 'uint64_t' if wide else 'uint32_t'
    terms = []
    if aff.const != 0 or not aff.coeffs:
        terms.append('(' + ctype + ')' + str(aff.const) + ('ull' if wide else 'u'))
    for (kind, k), c in sorted(aff.coeffs.items()):
        assert kind == 'p'
        term = '(' + ctype + ')' + pos_names[k]
        if c != 1:
            term = term + ' * (' + ctype + ')' + str(c) + ('ull' if wide else 'u')
        terms.append(term)
    return ' + '.join(terms)


def choose_vec(info):
    """Largest power-of-two vector width (elements) usable for this DAG, and the accesses it vectorises."""
    last = len(info.workgroup_shape) - 1
    extent = info.workgroup_shape[last]
    accesses = info.tensor_accesses()
    widest = 1
    for _, tensor, _ in accesses:
        widest = max(widest, ITEMSIZE[tensor.dtype])
    vec = max(1, 16 // widest)
    while vec > 1:
        if extent % vec == 0 and any(_is_vector_access(info, node, tensor, aff, vec)
                                     for node, tensor, aff in accesses):
            break
        vec //= 2
    return vec


def _is_vector_access(info, node, tensor, aff, vec):
    if aff is None or not aff.only_position():
        return False
    last = len(info.workgroup_shape) - 1
    if aff.coeff(('p', last)) != 1:
        return False
    if aff.const % vec != 0:
        return False
    for sym, c in aff.coeffs.items():
        if sym != ('p', last) and c % vec != 0:
            return False
    if aff.lo < 0 or aff.hi >= tensor.size:
        return False            # cannot prove every lane in bounds for every worker
    if info.in_loop[node.idx]:
        return False
    return True


def contiguous_unaligned(info, node, tensor, aff, vec):
    """Unit stride along the last workgroup dimension, but the vector's first element may sit at any element
    offset (e.g. a gather row that starts at i*7919): one 128-bit load with element alignment instead of VEC loads."""
    if aff is None or not aff.only_position() or info.in_loop[node.idx]:
        return False
    last = len(info.workgroup_shape) - 1
    if aff.coeff(('p', last)) != 1:
        return False
    if aff.lo < 0 or aff.hi >= tensor.size:
        return False
    return not _is_vector_access(info, node, tensor, aff, vec)


#: several vectors per thread are chosen only while the grid keeps this many workgroups (eight per compute unit)
MIN_BLOCKS_PER_THREAD_VECTORS = 2048


def _arithmetic_weight(info):
    """Rough count of expensive float operations per worker (transcendental calls and divisions)."""
    heavy = (lang.EXP, lang.LOG, lang.TANH, lang.DIVIDE, lang.SIN, lang.COS, lang.TAN, lang.POW, lang.SQRT,
             lang.SINH, lang.COSH, lang.ASIN, lang.ACOS, lang.ATAN, lang.ATAN2, lang.LOG10)
    return sum(1 for n in info.nodes if n.code in heavy and n.dtype in (lang.FLOAT32, lang.FLOAT64))


def generate(info, kernel_name, vec=None, nt=None, grid_cap=None, per_thread=None):
    """
    :param per_thread: vectors per thread (None chooses 1, 2 or 4).  The vectors, 256 apart so that every request of a
        wavefront stays one contiguous run, are requested together before the arithmetic of any: a wavefront then
        has several times the bytes in flight while it waits and the workgroup's set-up (math tables, barrier) is paid
        once for that much more work.  Measured on MI355X, interleaved runs: the 8-op chain in the 'ulp2' math mode,
        where arithmetic and memory time are about equal, 148.7 -> 142.4 us with two, and in steady state at the
        power limit 138.3 -> 133.1 us with four instead of two (eight: 138.3, sixteen: 162); the same chain in the
        'exact' mode, which is bound by arithmetic alone, 252 -> 255 us; the LSTM cell with its five to seven load
        streams 27.8 -> 30.4 us (forward) and 36.2 -> 39.9 us (gradient).  So it is chosen for bodies with few
        streams and some arithmetic, outside the 'exact' mode.
    :return: (kernel source text, launch description dict) for the map template.
    """
    rank = len(info.workgroup_shape)
    last = rank - 1
    if vec is None:
        vec = choose_vec(info)
    if info.workgroup_shape[last] % vec != 0:
        raise ValueError('vector width does not divide the last workgroup dimension')

    accesses = info.tensor_accesses()
    loads = {}      # (input node idx, signature) -> Access
    unaligned = {}  # same, for loads that are contiguous but only element aligned
    stores = {}     # (output node idx, signature) -> Access
    store_keys = []
    for node, tensor, aff in accesses:
        if vec > 1 and _is_vector_access(info, node, tensor, aff, vec):
            key = (tensor.idx, aff.signature())
            if node.code == lang.READ_TENSOR:
                if key not in loads:
                    loads[key] = Access(tensor, aff, 'ld%d' % len(loads))
            else:
                store_keys.append(key)
        elif vec > 1 and node.code == lang.READ_TENSOR and contiguous_unaligned(info, node, tensor, aff, vec):
            key = (tensor.idx, aff.signature())
            if key not in unaligned:
                unaligned[key] = Access(tensor, aff, 'lu%d' % len(unaligned))
    certain = info.definitely_stores(store_keys)
    bufferable = info.bufferable_outputs(
        lambda node, tensor, aff: vec > 1 and (tensor.idx, aff.signature()) in certain and
        _is_vector_access(info, node, tensor, aff, vec))
    for node, tensor, aff in accesses:
        if node.code == lang.ASSIGN_TENSOR and aff is not None and tensor.idx in bufferable:
            key = (tensor.idx, aff.signature())
            if key in certain and key not in stores and vec > 1 and _is_vector_access(info, node, tensor, aff, vec):
                stores[key] = Access(tensor, aff, 'st%d' % len(stores))

    # Non-temporal hints, measured on MI355X (every element is touched exactly once in all of these):
    #   copy, 1 load : 1 store             hint on the stores 75 us, on neither 84
    #   three-operand add, 2 : 1           hint on the loads 116 us, on both 124, on the stores 135, on neither 138
    #   LSTM cell forward, 5 : 2           stores 26.5 us, both 27.2, neither 27.2, loads 29.7
    #   LSTM cell gradient, 7 : 5          stores 36.4 us, neither 38.1, loads 40.5, both 41.7
    # so: on the stores when there are at least as many stores as loads or many load streams, on the loads when two
    # or three load streams feed fewer stores.
    if nt is None:
        streams = len(loads) + len(unaligned)
        nt = 's' if (streams <= len(stores) or streams >= 4) else 'l'
    load_fn = 'OVL_LOAD_NT' if 'l' in nt else 'OVL_LOAD_PLAIN'
    store_fn = 'OVL_STORE_NT' if 's' in nt else 'OVL_STORE_PLAIN'

    def read_hook(node, tensor, index_name):
        aff = info.affine[node.ops[1]]
        if aff is not None:
            acc = loads.get((tensor.idx, aff.signature())) or unaligned.get((tensor.idx, aff.signature()))
            if acc is not None and not info.in_loop[node.idx]:
                return acc.reg + '[lane]'
        return None

    def store_hook(node, tensor, index_name, value_name):
        aff = info.affine[node.ops[1]]
        if aff is not None:
            acc = stores.get((tensor.idx, aff.signature()))
            if acc is not None and not info.in_loop[node.idx]:
                return acc.reg + '[lane] = ' + value_name + ';'
        return None

    num_vectors = info.num_workers // vec
    single_grid = (num_vectors + BLOCK - 1) // BLOCK <= min(grid_cap or MAX_GRID, MAX_GRID)
    if per_thread is None:
        few_streams = len(loads) + len(unaligned) + len(stores) <= 3
        per_thread = 4 if (vec > 1 and few_streams and _arithmetic_weight(info) >= 4 and
                           getattr(info, 'math', 'exact') != 'exact') else 1
        # (a small tensor keeps one vector per thread: its time is latency, and fewer, longer threads only add to it.
        # The reference's README pipeline on 2^20 floats in the 'ulp2' mode: 10 us with four vectors per thread and
        # 256 workgroups, 6 us with one and 1024)
        while per_thread > 1 and (num_vectors % (BLOCK * per_thread) != 0 or
                                  num_vectors // (BLOCK * per_thread) < MIN_BLOCKS_PER_THREAD_VECTORS):
            per_thread //= 2
    if per_thread > 1 and not (single_grid and num_vectors % (BLOCK * per_thread) == 0 and
                               not any(info.in_loop.values())):
        per_thread = 1
    # names of the registers of one of the thread's vectors: '' for a single vector, else '_0', '_1', ...
    reps = [''] if per_thread == 1 else ['_%d' % r for r in range(per_thread)]

    def hooks(sfx):
        def read_rep(node, tensor, index_name):
            text = read_hook(node, tensor, index_name)
            return text.replace('[lane]', sfx + '[lane]') if text else text

        def store_rep(node, tensor, index_name, value_name):
            text = store_hook(node, tensor, index_name, value_name)
            return text.replace('[lane] = ', sfx + '[lane] = ', 1) if text else text
        return read_rep, store_rep

    def names_of(sfx):
        return ['p%d%s' % (k, sfx) for k in range(rank)]

    bodies = {}
    for sfx in reps:
        lane_position = names_of(sfx)
        if vec > 1:
            lane_position[last] = lane_position[last] + ' + lane'
        read_rep, store_rep = hooks(sfx)
        bodies[sfx] = BodyEmitter(info, lane_position, read_rep, store_rep).emit()
    pos_names = names_of(reps[0])

    args = []
    for i in range(len(info.inputs)):
        args.append('const ' + CTYPE[info.inputs[i].dtype] + '* __restrict__ in' + str(i))
    for i in range(len(info.outputs)):
        args.append(CTYPE[info.outputs[i].dtype] + '* __restrict__ out' + str(i))

    src = []
    vec_types = {}
    for acc in list(loads.values()) + list(stores.values()) + list(unaligned.values()):
        ctype = CTYPE[acc.tensor.dtype]
        vec_types[ctype] = ('ovl_' + ctype.replace(' ', '_') + 'x' + str(vec), ITEMSIZE[acc.tensor.dtype])
    for ctype, (vname, itemsize) in sorted(vec_types.items()):
        src.append('typedef ' + ctype + ' ' + vname + ' __attribute__((ext_vector_type(' + str(vec) + ')));')
        src.append('typedef ' + vname + ' ' + vname + '_u __attribute__((aligned(' + str(itemsize) + ')));')
    vec_types = dict((k, v[0]) for k, v in vec_types.items())
    src.append('')
    src.append('extern "C" __global__ void __launch_bounds__(%d)' % BLOCK)
    src.append(kernel_name + '(' + ', '.join(args) + ') {')
    blocks_needed = (num_vectors + BLOCK * per_thread - 1) // (BLOCK * per_thread)
    # One element per thread (a last dimension that is not a multiple of the vector width) and the LDS math tables: a
    # workgroup that covers 256 elements would copy the tables for 256 elements' worth of work.  Such kernels get a
    # grid of SCALAR_TABLE_GRID workgroups that stride over the tensor (the 8-op chain on float32 [8191, 8191]: 'ulp2'
    # 284 -> 159 us, 'exact' 318 -> 266 us; with four elements per thread and more the single pass is the faster one).
    if grid_cap is None and vec == 1 and info.uses_math_tables() and blocks_needed > SCALAR_TABLE_GRID:
        grid_cap = SCALAR_TABLE_GRID
    # When the grid covers every vector (always, unless the workgroup has more than 2^32 - 256 workers at VEC = 1 or
    # the caller caps the grid) a thread runs its vectors without a loop.  Kernels that use the LDS math tables then
    # request their operands first and copy the tables (with the barrier that implies) while they are in flight,
    # instead of waiting for the tables before the first request.
    covers = blocks_needed <= min(grid_cap or MAX_GRID, MAX_GRID)
    single_pass = info.uses_math_tables() and covers
    src.append('    const uint32_t num_vectors = %du;' % num_vectors)
    if per_thread > 1:
        # the grid covers the vectors exactly: no idle threads
        src.append('    const uint32_t v = blockIdx.x * %du + threadIdx.x;' % (BLOCK * per_thread))
        src.append('    {')
    elif single_pass:
        src.append('    const uint32_t v_raw = blockIdx.x * %du + threadIdx.x;' % BLOCK)
        src.append('    const bool active = v_raw < num_vectors;')
        src.append('    // idle threads of the last workgroup request vector 0 and store nothing')
        src.append('    const uint32_t v = active ? v_raw : 0u;')
        src.append('    {')
    elif covers:
        src.append('    const uint32_t v = blockIdx.x * %du + threadIdx.x;' % BLOCK)
        src.append('    if (v < num_vectors) {')
    else:
        if info.uses_math_tables():
            src.append('    OVL_DECLARE_MATH_TABLES();')
        src.append('    // v + stride may pass 2^32: the step is taken only while it stays below num_vectors')
        src.append('    const uint32_t stride = gridDim.x * %du;' % BLOCK)
        src.append('    for (uint32_t v = blockIdx.x * %du + threadIdx.x; v < num_vectors;' % BLOCK)
        src.append('         v = (num_vectors - v > stride) ? v + stride : num_vectors) {')
    # position of the first worker of each of this thread's vectors
    block = 1
    blocks = [1] * rank
    for k in range(rank - 2, -1, -1):
        block *= info.workgroup_shape[k + 1]
        blocks[k] = block
    for r, sfx in enumerate(reps):
        names = names_of(sfx)
        src.append('        const uint32_t worker0%s = (v + %du) * %du;' % (sfx, r * BLOCK, vec))
        for k in range(rank):
            expr = 'worker0' + sfx
            if k > 0:
                expr = '(worker0' + sfx + ' % ' + str(blocks[k - 1]) + 'u)'
            src.append('        const uint32_t %s = %s / %du;' % (names[k], expr, blocks[k]))
    for sfx in reps:
        names = names_of(sfx)
        for acc in loads.values():
            vname = vec_types[CTYPE[acc.tensor.dtype]]
            wide = acc.aff.hi >= 2 ** 32
            src.append('        const %s %s = %s(reinterpret_cast<const %s*>(in%d + (%s)));' % (
                vname, acc.reg + sfx, load_fn, vname, acc.tensor.io_index, _index_expr(acc.aff, names, wide)))
        for acc in unaligned.values():
            vname = vec_types[CTYPE[acc.tensor.dtype]]
            wide = acc.aff.hi >= 2 ** 32
            src.append('        const %s %s = *reinterpret_cast<const %s_u*>(in%d + (%s));' % (
                vname, acc.reg + sfx, vname, acc.tensor.io_index, _index_expr(acc.aff, names, wide)))
    if single_pass:
        src.append('        OVL_DECLARE_MATH_TABLES();')
        if per_thread == 1:
            src.append('        if (active) {')
    for sfx in reps:
        names = names_of(sfx)
        src.append('        {')
        for acc in stores.values():
            src.append('        %s %s;' % (vec_types[CTYPE[acc.tensor.dtype]], acc.reg + sfx))
        if vec > 1:
            src.append('        #pragma unroll')
            src.append('        for (uint32_t lane = 0; lane < %du; ++lane) {' % vec)
        else:
            src.append('        {')
        for stmt in bodies[sfx]:
            src.append('            ' + stmt)
        src.append('        }')
        for acc in stores.values():
            vname = vec_types[CTYPE[acc.tensor.dtype]]
            wide = acc.aff.hi >= 2 ** 32
            src.append('        %s(%s, reinterpret_cast<%s*>(out%d + (%s)));' % (
                store_fn, acc.reg + sfx, vname, acc.tensor.io_index, _index_expr(acc.aff, names, wide)))
        src.append('        }')
    if single_pass and per_thread == 1:
        src.append('        }')
    src.append('    }')
    src.append('}')

    align = {}
    for acc in loads.values():
        key = ('in', acc.tensor.io_index)
        align[key] = max(align.get(key, 1), vec * ITEMSIZE[acc.tensor.dtype])
    for acc in stores.values():
        key = ('out', acc.tensor.io_index)
        align[key] = max(align.get(key, 1), vec * ITEMSIZE[acc.tensor.dtype])

    launch = {
        'template': 'map',
        'vec': vec,
        'per_thread': per_thread,
        'block': BLOCK,
        'blocks_needed': blocks_needed,
        'grid_cap': grid_cap,
        'align': align,
        'vector_loads': len(loads) + len(unaligned),
        'vector_stores': len(stores),
    }
    return '\n'.join(src) + '\n', launch
