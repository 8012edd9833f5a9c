"""
The tile kernel template: a workgroup of rank two or more whose operator stores one or more outputs with its last two
dimensions transposed (the dimensions before them are batches: one grid of tiles after the other; a batched transpose
float32 [64, 2048, 2048] takes 362 us with it, 2473 us with one worker per thread).

A worker at (i, j) that writes ``out[j, i]`` makes neighbouring workers along j (the lanes of a wavefront in the
one-worker-per-thread template of the reference, opveclib/expression.py:602-608) store to addresses a whole output
row apart: every lane of every store instruction touches a different cache line.  This template gives one 256-thread
workgroup a TILE_I x TILE_J block of workers (32 x 256 for 4-byte elements):

  phase 1  threads walk the tile row by row, VEC consecutive j per thread, exactly like the map kernel (aligned or
           dword-aligned 128-bit loads along j, register-buffered 128-bit stores for outputs that are contiguous along
           j); values of transposed outputs are written into an LDS tile at [j][i] (row length TILE_I+1 words, which
           spreads the column-wise writes and the row-wise reads over the LDS banks);
  phase 2  after a barrier the threads walk the LDS tile the other way, VEC consecutive i per thread, and store
           128-bit vectors that are contiguous along i, so a wavefront writes whole 128-byte lines of the output rows.

The worker body is the same statement sequence as in every other template; only where a store lands changes.
"""

from .. import language as lang
from .analysis import ITEMSIZE
from .body import BodyEmitter, CTYPE
from .map_kernel import Access, _index_expr, _is_vector_access, contiguous_unaligned

BLOCK = 256
TILE_I_BYTES = 128        # extent of a tile along the workgroup dimension before the last, in bytes of the widest element
TILE_J_BYTES = 1024       # extent along the last dimension
MIN_TILE_EXTENT = 8       # tiles shrink to the workgroup's extents down to this many workers a side


def _tile_dim(info, aff):
    """The workgroup dimension (not the last) along which this store has unit stride, or None."""
    if aff is None:
        return None
    rank = len(info.workgroup_shape)
    for k in range(rank - 2, -1, -1):
        if info.workgroup_shape[k] > 1 and aff.coeff(('p', k)) == 1:
            return k
    return None


def _is_transposed_store(info, node, tensor, aff, vec, dim):
    """out[.., p_last*C + p_dim + c] with dim a workgroup dimension before the last: unit stride along it, vector
    aligned (the other dimensions are batch dimensions: any multiple of the vector width)."""
    if aff is None or not aff.only_position() or info.in_loop[node.idx]:
        return False
    rank = len(info.workgroup_shape)
    if dim is None or aff.coeff(('p', dim)) != 1:
        return False
    c_last = aff.coeff(('p', rank - 1))
    if c_last == 0 or c_last % vec != 0 or aff.const % vec != 0:
        return False
    for sym, c in aff.coeffs.items():
        if sym not in (('p', dim), ('p', rank - 1)) and c % vec != 0:
            return False
    if aff.lo < 0 or aff.hi >= tensor.size:
        return False
    return True


def _plan(info):
    """(vector width, dimension that the tile spans beside the last), or None if the template does not fit.  The
    dimension is the one along which the first position-indexed store outside loops has unit stride: [N, C, H, W]
    stored as [N, H, W, C] takes C, a transposition of the last two dimensions takes the one before the last."""
    rank = len(info.workgroup_shape)
    if rank < 2:
        return None
    accesses = info.tensor_accesses()
    stores = [(n, t, a) for n, t, a in accesses if n.code == lang.ASSIGN_TENSOR]
    dim = None
    for n, t, a in stores:
        if a is not None and a.only_position() and not info.in_loop[n.idx] and a.coeff(('p', rank - 1)) != 1:
            dim = _tile_dim(info, a)
            if dim is not None:
                break
    if dim is None:
        return None
    rows, cols = info.workgroup_shape[dim], info.workgroup_shape[-1]
    widest = 1
    for _, tensor, _ in accesses:
        widest = max(widest, ITEMSIZE[tensor.dtype])
    # the widest vectors that divide both extents: one element per access still goes through the tile, since what the
    # template is for is the coalescing of the transposed stores (float32 [16383, 16385]: 1391 us with one worker per
    # thread and stores a row apart)
    vec = max(1, 16 // widest)
    while vec > 1 and (rows % vec != 0 or cols % vec != 0):
        vec //= 2
    return vec, dim


def applicable(info):
    """Vector width if the tile template fits this DAG, else None."""
    planned = _plan(info)
    if planned is None:
        return None
    vec, dim = planned
    accesses = info.tensor_accesses()
    stores = [(n, t, a) for n, t, a in accesses if n.code == lang.ASSIGN_TENSOR]
    keys = [(t.idx, a.signature()) for n, t, a in stores if _is_transposed_store(info, n, t, a, vec, dim)]
    if not keys:
        return None
    certain = info.definitely_stores(keys)
    bufferable = info.bufferable_outputs(
        lambda node, tensor, aff: (tensor.idx, aff.signature()) in certain and
        _is_transposed_store(info, node, tensor, aff, vec, dim))
    certain = set(key for key in certain if key[0] in bufferable)
    if not certain:
        return None
    # all transposed outputs share one element width so one tile geometry serves them all
    return vec


def generate(info, kernel_name, tile_i=None, tile_j=None, nt=None, tile_order=None):
    nt_given = nt is not None
    nt = 'ls' if nt is None else nt
    load_fn = 'OVL_LOAD_NT' if 'l' in nt else 'OVL_LOAD_PLAIN'
    store_fn = 'OVL_STORE_NT' if 's' in nt else 'OVL_STORE_PLAIN'
    assert applicable(info) is not None
    vec, dim = _plan(info)
    # Measured on MI355X (float32 [16384, 16384], gather + transposed store): 32 x 256 workers per tile, i.e. one
    # 128-byte line per transposed output row and 1 KiB runs along j, runs at the speed of a plain copy (480 us against
    # 570 us for 64 x 64 and 549 us for 128 x 128).
    rank = len(info.workgroup_shape)
    # the two dimensions that a tile spans; the others are batches
    rows, cols = info.workgroup_shape[dim], info.workgroup_shape[-1]
    batch_dims = [k for k in range(rank - 1) if k != dim]
    batches = 1
    for k in batch_dims:
        batches *= info.workgroup_shape[k]
    pi, pj = 'p%d' % dim, 'p%d' % (rank - 1)
    pos_names = ['p%d' % k for k in range(rank)]
    accesses = info.tensor_accesses()
    widest = max(ITEMSIZE[tensor.dtype] for _, tensor, _ in accesses)
    tile_i = tile_i or TILE_I_BYTES // widest
    while tile_i // 2 >= max(rows, vec, MIN_TILE_EXTENT):     # short tile dimensions: no rows of idle threads
        tile_i //= 2
    # Narrower vectors, shorter tiles: a thread then has fewer bytes in flight, and the smaller tile lets more
    # workgroups share a compute unit's LDS (float32 [8191, 8191], one element per access: 209 us with 32 x 256
    # workers, 133 us with 32 x 128; [16382, 16386], two per access: 539 -> 492 us).
    full_vec = max(1, 16 // widest)
    tile_j = tile_j or max(TILE_J_BYTES // widest * vec // full_vec, TILE_J_BYTES // 2 // widest)
    while tile_j // 2 >= max(cols, vec, MIN_TILE_EXTENT):
        tile_j //= 2

    loads = {}
    unaligned = {}
    stores = {}
    tstores = {}
    store_keys = []
    tkeys = []
    for node, tensor, aff in accesses:
        if node.code == lang.READ_TENSOR:
            if _is_vector_access(info, node, tensor, aff, vec):
                key = (tensor.idx, aff.signature())
                loads.setdefault(key, Access(tensor, aff, 'ld%d' % len(loads)))
            elif contiguous_unaligned(info, node, tensor, aff, vec):
                key = (tensor.idx, aff.signature())
                unaligned.setdefault(key, Access(tensor, aff, 'lu%d' % len(unaligned)))
        else:
            if _is_vector_access(info, node, tensor, aff, vec):
                store_keys.append((tensor.idx, aff.signature()))
            elif _is_transposed_store(info, node, tensor, aff, vec, dim):
                tkeys.append((tensor.idx, aff.signature()))
    certain = info.definitely_stores(store_keys + tkeys)
    bufferable = info.bufferable_outputs(
        lambda node, tensor, aff: (tensor.idx, aff.signature()) in certain and
        (_is_vector_access(info, node, tensor, aff, vec) or _is_transposed_store(info, node, tensor, aff, vec, dim)))
    for node, tensor, aff in accesses:
        if node.code != lang.ASSIGN_TENSOR or aff is None or tensor.idx not in bufferable:
            continue
        key = (tensor.idx, aff.signature())
        if key not in certain:
            continue
        if key in store_keys and key not in stores:
            stores[key] = Access(tensor, aff, 'st%d' % len(stores))
        elif key in tkeys and key not in tstores:
            tstores[key] = Access(tensor, aff, 'tile%d' % len(tstores))

    def read_hook(node, tensor, index_name):
        aff = info.affine[node.ops[1]]
        if aff is not None and not info.in_loop[node.idx]:
            acc = loads.get((tensor.idx, aff.signature())) or unaligned.get((tensor.idx, aff.signature()))
            if acc is not None:
                return acc.reg + '[lane]'
        return None

    def store_hook(node, tensor, index_name, value_name):
        aff = info.affine[node.ops[1]]
        if aff is not None and not info.in_loop[node.idx]:
            key = (tensor.idx, aff.signature())
            if key in stores:
                return stores[key].reg + '[lane] = ' + value_name + ';'
            if key in tstores:
                return tstores[key].reg + '[tj + lane][ti] = ' + value_name + ';'
        return None

    body = BodyEmitter(info, pos_names[:-1] + [pj + ' + lane'], read_hook, store_hook, register_stores=False).emit()

    threads_per_row = tile_j // vec             # phase 1: a tile row is tile_j workers along j
    rows_per_pass = BLOCK // threads_per_row
    threads_per_col = tile_i // vec             # phase 2: a row of the LDS tile is tile_i workers along i
    cols_per_pass = BLOCK // threads_per_col
    tiles_i = (rows + tile_i - 1) // tile_i
    tiles_j = (cols + tile_j - 1) // tile_j

    args = []
    for i in range(len(info.inputs)):
        args.append('const ' + CTYPE[info.inputs[i].dtype] + '* __restrict__ in' + str(i))
    for i in range(len(info.outputs)):
        args.append(CTYPE[info.outputs[i].dtype] + '* __restrict__ out' + str(i))

    src = []
    vec_types = {}
    for acc in list(loads.values()) + list(stores.values()) + list(tstores.values()) + list(unaligned.values()):
        ctype = CTYPE[acc.tensor.dtype]
        vec_types[ctype] = ('ovl_' + ctype.replace(' ', '_') + 'x' + str(vec), ITEMSIZE[acc.tensor.dtype])
    for ctype, (vname, itemsize) in sorted(vec_types.items()):
        src.append('typedef ' + ctype + ' ' + vname + ' __attribute__((ext_vector_type(' + str(vec) + ')));')
        src.append('typedef ' + vname + ' ' + vname + '_u __attribute__((aligned(' + str(itemsize) + ')));')
    vec_types = dict((k, v[0]) for k, v in vec_types.items())
    src.append('')
    src.append('extern "C" __global__ void __launch_bounds__(%d)' % BLOCK)
    src.append(kernel_name + '(' + ', '.join(args) + ') {')
    if info.uses_math_tables():
        src.append('    OVL_DECLARE_MATH_TABLES();')
    for acc in tstores.values():
        src.append('    __shared__ %s %s[%d][%d];' % (CTYPE[acc.tensor.dtype], acc.reg, tile_j, tile_i + 1))
    misaligned = any((acc.aff.coeff(('p', rank - 1)) * ITEMSIZE[acc.tensor.dtype]) % 128 != 0
                     for acc in tstores.values())
    blocks_needed = batches * tiles_i * tiles_j
    stripes = batches * tiles_j                 # a stripe: the tiles_i tiles that follow one another along i
    order = tile_order or ('xcd' if misaligned else 'plain')
    src.append('    const uint32_t num_tiles = %du;' % blocks_needed)
    src.append('    for (uint32_t tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {')
    if order == 'xcd':
        # Transposed output rows that are not whole 128-byte lines: two tiles that follow one another along i share
        # the line their runs meet in (see phase 2).  Workgroups go to the eight XCDs in turn, each with an L2 of its
        # own, so the tiles are numbered 64 stripes abreast (the stripes left over eight abreast, and what is then
        # left side by side): the two that share lines are a multiple of eight workgroups apart, on one XCD and at
        # work at the same time, and the line leaves that L2 whole.  float32 [16380, 16388], 65 tiles along j:
        # 783 -> 467 us.  (A workgroup that takes its neighbour's tile itself a moment later is too late:
        # [16380, 16384] 447 -> 766 us; eight abreast throughout reads shorter runs of each row: 447 -> 532 us.)
        segments = []           # (first tile, first stripe, stripes abreast, groups)
        first_tile, first_stripe = 0, 0
        for abreast in (64, 8, 1):
            left = stripes - first_stripe
            if abreast == 1:
                abreast = left
            if left == 0 or left < abreast:
                continue
            groups = left // abreast
            segments.append((first_tile, first_stripe, abreast, groups))
            first_tile += groups * abreast * tiles_i
            first_stripe += groups * abreast
        src.append('        uint32_t stripe, along_i;')
        for k, (first_tile, first_stripe, abreast, groups) in enumerate(segments):
            last = k == len(segments) - 1
            head = '        ' + ('' if k == 0 else '} else ') + \
                ('{' if last and k > 0 else 'if (tile < %du) {' % (first_tile + groups * abreast * tiles_i) if not last
                 else '{')
            src.append(head)
            src.append('            const uint32_t t = tile - %du;' % first_tile)
            src.append('            stripe = %du + t / %du * %du + t %% %du;' % (
                first_stripe, abreast * tiles_i, abreast, abreast))
            src.append('            along_i = t %% %du / %du;' % (abreast * tiles_i, abreast))
        src.append('        }')
    else:
        src.append('        const uint32_t stripe = tile / %du * %du + tile %% %du;' % (tiles_i * tiles_j, tiles_j, tiles_j))
        src.append('        const uint32_t along_i = tile / %du %% %du;' % (tiles_j, tiles_i))
    src.append('        const uint32_t i0 = along_i * %du;' % tile_i)
    src.append('        const uint32_t j0 = (stripe %% %du) * %du;' % (tiles_j, tile_j))
    # the dimensions beside the tile's two: one tile grid after the other
    stride = tiles_j
    for k in reversed(batch_dims):
        src.append('        const uint32_t p%d = stripe / %du %% %du;' % (k, stride, info.workgroup_shape[k]))
        stride *= info.workgroup_shape[k]
    src.append('        const uint32_t tj = (threadIdx.x %% %du) * %du;' % (threads_per_row, vec))
    src.append('        #pragma unroll 1')
    src.append('        for (uint32_t ti = threadIdx.x / %du; ti < %du; ti += %du) {' % (
        threads_per_row, tile_i, rows_per_pass))
    src.append('            const uint32_t %s = i0 + ti;' % pi)
    src.append('            const uint32_t %s = j0 + tj;' % pj)
    src.append('            if (%s < %du && %s < %du) {' % (pi, rows, pj, cols))
    for acc in loads.values():
        vname = vec_types[CTYPE[acc.tensor.dtype]]
        wide = acc.aff.hi >= 2 ** 32
        src.append('                const %s %s = %s(reinterpret_cast<const %s*>(in%d + (%s)));'
                   % (vname, acc.reg, load_fn, vname, acc.tensor.io_index, _index_expr(acc.aff, pos_names, wide)))
    for acc in unaligned.values():
        vname = vec_types[CTYPE[acc.tensor.dtype]]
        wide = acc.aff.hi >= 2 ** 32
        src.append('                const %s %s = *reinterpret_cast<const %s_u*>(in%d + (%s));' % (
            vname, acc.reg, vname, acc.tensor.io_index, _index_expr(acc.aff, pos_names, wide)))
    for acc in stores.values():
        src.append('                %s %s;' % (vec_types[CTYPE[acc.tensor.dtype]], acc.reg))
    src.append('                #pragma unroll')
    src.append('                for (uint32_t lane = 0; lane < %du; ++lane) {' % vec)
    for stmt in body:
        src.append('                    ' + stmt)
    src.append('                }')
    for acc in stores.values():
        vname = vec_types[CTYPE[acc.tensor.dtype]]
        wide = acc.aff.hi >= 2 ** 32
        src.append('                %s(%s, reinterpret_cast<%s*>(out%d + (%s)));' % (
            store_fn, acc.reg, vname, acc.tensor.io_index, _index_expr(acc.aff, pos_names, wide)))
    src.append('            }')
    src.append('        }')
    src.append('        __syncthreads();')
    # phase 2: rows of the LDS tile are runs along i.  A transposed output row that is not a whole number of 128-byte
    # lines long puts the runs a tile stores across line boundaries, and the rest of each line belongs to the tile's
    # neighbour along i; with the non-temporal hint the two parts reach memory as partial lines (float32
    # [16380, 16384]: 1085 us against 484 us for [16384, 16384]), without it they meet in the L2 (603 us; giving the
    # two neighbours to workgroups on one XCD at the same time made it slower, 744 us).  For whole lines the hint is
    # the faster form (484 against 494 us).
    tstore_fn = store_fn
    if not nt_given and misaligned:
        tstore_fn = 'OVL_STORE_PLAIN'
    src.append('        const uint32_t oi = (threadIdx.x %% %du) * %du;' % (threads_per_col, vec))
    src.append('        #pragma unroll 1')
    src.append('        for (uint32_t oj = threadIdx.x / %du; oj < %du; oj += %du) {' % (
        threads_per_col, tile_j, cols_per_pass))
    src.append('            const uint32_t %s = i0 + oi;' % pi)
    src.append('            const uint32_t %s = j0 + oj;' % pj)
    src.append('            if (%s < %du && %s < %du) {' % (pi, rows, pj, cols))
    for acc in tstores.values():
        vname = vec_types[CTYPE[acc.tensor.dtype]]
        wide = acc.aff.hi >= 2 ** 32
        src.append('                %s v_%s;' % (vname, acc.reg))
        src.append('                #pragma unroll')
        src.append('                for (uint32_t lane = 0; lane < %du; ++lane) v_%s[lane] = %s[oj][oi + lane];' % (
            vec, acc.reg, acc.reg))
        src.append('                %s(v_%s, reinterpret_cast<%s*>(out%d + (%s)));' % (
            tstore_fn, acc.reg, vname, acc.tensor.io_index, _index_expr(acc.aff, pos_names, wide)))
    src.append('            }')
    src.append('        }')
    src.append('        __syncthreads();')
    src.append('    }')
    src.append('}')

    align = {}
    for acc in loads.values():
        key = ('in', acc.tensor.io_index)
        align[key] = max(align.get(key, 1), vec * ITEMSIZE[acc.tensor.dtype])
    for acc in list(stores.values()) + list(tstores.values()):
        key = ('out', acc.tensor.io_index)
        align[key] = max(align.get(key, 1), vec * ITEMSIZE[acc.tensor.dtype])

    launch = {
        'template': 'transpose',
        'vec': vec,
        'block': BLOCK,
        'blocks_needed': blocks_needed,
        'align': align,
        'vector_loads': len(loads) + len(unaligned),
        'vector_stores': len(stores) + len(tstores),
    }
    return '\n'.join(src) + '\n', launch
