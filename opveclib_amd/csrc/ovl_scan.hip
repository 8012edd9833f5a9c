// Hand-written order-preserving row scans (running sum and product along the last axis) for gfx950 behind the C ABI
// of include/ovl_scan.h.
//
// The recurrence of the reference's accumulate operator (opveclib/examples/test_accumulate.py:63-76) is kept exactly:
// out[r, 0] = x[r, 0], out[r, i] = f(out[r, i-1], x[r, i]) in the tensor's own type, left to right.  Floating point
// addition and multiplication are not associative, so a tree-shaped wavefront scan would give other bits; what is
// parallel here is the rows (four per wavefront) and the movement of data.
//
// Lane-skewed scan: sixteen neighbouring lanes share one row.  Lane p of the group owns RUN = VEC * WIDTH consecutive
// columns of the current group of 16 * RUN columns, loaded and stored as WIDTH 128-bit accesses.  In phase 0..15 every
// lane runs the recurrence over its own run starting from the carried state it holds, then hands its final state to
// its right neighbour (a DPP row_shr:1 move; lane 0 keeps the true carry).  After phase p lanes 0..p hold exact
// results: a lane that is already exact recomputes the same values, a lane that is not yet exact computes values that
// a later phase overwrites.  After phase 15 the group is exact and lane 15's state is rotated to lane 0 (row_ror:1)
// as the carry into the next group.  Global accesses are issued in bursts of DEPTH groups into two register sets, so
// one burst is in flight while the other is consumed.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string>
#include <type_traits>

#include "ovl_device.h"
#include "ovl_scan.h"

// ovl_device.h carries the status codes generated operators return; this one (ovl_status in ovl_launch.h) is the
// launcher's own
#define OVL_EINVAL 6

// steps of loads the reassociating scan keeps in flight per thread
#ifndef OVL_SCAN_AHEAD
#define OVL_SCAN_AHEAD 8
#endif

namespace {

thread_local std::string g_last_error;

int fail(int code, const std::string& detail) {
    g_last_error = detail;
    return code;
}

constexpr uint32_t BLOCK = 256, WAVE = 64, GROUP = 16;
constexpr uint32_t ROWS_PER_WAVE = WAVE / GROUP, ROWS_PER_BLOCK = ROWS_PER_WAVE * (BLOCK / WAVE);

// `start` is the value s with f(s, x) == x bit for bit for every x, signed zeros and infinities included (-0 for the
// sum: +0 would turn a leading -0 into +0).  Starting the recurrence from it makes column 0 an ordinary step, with no
// special case on the critical path: out[r, 0] = f(start, x[r, 0]) = x[r, 0].
struct op_sum {
    template <typename T> static __device__ __forceinline__ T apply(T a, T b) { return a + b; }
    template <typename T> static __device__ __forceinline__ T start() { return (T)-0.0; }
};
struct op_product {
    template <typename T> static __device__ __forceinline__ T apply(T a, T b) { return a * b; }
    template <typename T> static __device__ __forceinline__ T start() { return (T)1.0; }
};

template <typename T, int VEC> struct vec_of { typedef T type __attribute__((ext_vector_type(VEC))); };

// A vector as it lies in memory: on a 16-byte boundary, or (ALIGNED = false) only aligned like its elements.  (The
// alignment is stated on a typedef at the place of the access: as a template argument it would be dropped.)
template <bool ALIGNED, typename V, typename T>
static __device__ __forceinline__ V load_vector(const T* p) {
    if constexpr (ALIGNED) {
        return *reinterpret_cast<const V*>(p);
    } else {
        typedef V unaligned __attribute__((aligned(alignof(T))));
        return *reinterpret_cast<const unaligned*>(p);
    }
}
template <bool ALIGNED, typename V, typename T>
static __device__ __forceinline__ void store_vector(V value, T* p) {
    if constexpr (ALIGNED) {
        __builtin_nontemporal_store(value, reinterpret_cast<V*>(p));
    } else {
        typedef V unaligned __attribute__((aligned(alignof(T))));
        __builtin_nontemporal_store(value, reinterpret_cast<unaligned*>(p));
    }
}

// cols must be at least DEPTH groups of 16 * VEC * WIDTH columns (scan() chooses DEPTH = 1 for shorter rows).  A row
// whose number of groups is not a multiple of DEPTH ends in up to DEPTH - 1 single groups, requested at the start and
// held in registers until then.  The columns after the last whole group (fewer than one group's worth) run as one more,
// partial group across all sixteen lanes: every lane loads its columns element by element with the index clamped to
// the row's last column, skips the columns past the end in the recurrence, and stores its columns element by element.
// ALIGNED: every row of x and out starts on a 16-byte boundary; otherwise vectors are moved with the alignment of
// their elements.
template <typename T, typename OP, int VEC, int WIDTH, int DEPTH, bool ALIGNED>
__global__ void __launch_bounds__(BLOCK)
skewed_scan_kernel(const T* __restrict__ x, T* __restrict__ out, uint32_t rows, uint32_t cols) {
    typedef typename vec_of<T, VEC>::type vec;
    constexpr uint32_t RUN = VEC * WIDTH, GROUP_COLS = GROUP * RUN, BATCH_COLS = GROUP_COLS * DEPTH;
    const uint32_t lane = threadIdx.x % WAVE;
    const uint32_t part = lane % GROUP;
    const uint32_t first_row = (blockIdx.x * (BLOCK / WAVE) + threadIdx.x / WAVE) * ROWS_PER_WAVE;
    // A wavefront wholly past the last row leaves; single lanes past it shadow the last row instead (all lanes must
    // stay active for the lane-to-lane moves): they load, compute and store exactly what its owners do.
    if (first_row >= rows) return;
    const uint32_t row_raw = first_row + lane / GROUP;
    const uint32_t row = row_raw < rows ? row_raw : rows - 1u;
    const T* __restrict__ gin = x + (uint64_t)row * cols + part * RUN;
    T* __restrict__ gout = out + (uint64_t)row * cols + part * RUN;
    const uint32_t num_batches = cols / BATCH_COLS;
    const uint32_t last_batch = num_batches - 1u;
    const uint32_t num_groups = cols / GROUP_COLS;
    const uint32_t tail = num_groups - num_batches * (uint32_t)DEPTH;      // 0 ... DEPTH - 1 groups after the batches
    constexpr uint32_t TAIL_MAX = DEPTH > 1 ? DEPTH - 1 : 1;

    vec q[2][DEPTH][WIDTH];
    // (a tail group that does not exist is requested as the row's last group once more and never used)
    vec qt[TAIL_MAX][WIDTH];
    if constexpr (DEPTH > 1) {
#pragma unroll
        for (uint32_t j = 0; j < TAIL_MAX; ++j) {
            const uint32_t g = num_batches * (uint32_t)DEPTH + j < num_groups ? num_batches * (uint32_t)DEPTH + j : num_groups - 1u;
#pragma unroll
            for (uint32_t w = 0; w < (uint32_t)WIDTH; ++w)
                qt[j][w] = load_vector<ALIGNED, vec>(gin + (uint64_t)g * GROUP_COLS + w * VEC);
        }
    }
#pragma unroll
    for (uint32_t s = 0; s < 2u; ++s) {
        const uint32_t b = s < num_batches ? s : last_batch;
#pragma unroll
        for (uint32_t j = 0; j < (uint32_t)DEPTH; ++j)
#pragma unroll
            for (uint32_t w = 0; w < (uint32_t)WIDTH; ++w)
                q[s][j][w] = load_vector<ALIGNED, vec>(gin + (uint64_t)b * BATCH_COLS + j * GROUP_COLS + w * VEC);
    }
    // ... and the columns after the last whole group, element by element (a vector may cross the end of the row; a
    // column past it is read as the row's last element and never used)
    const T* __restrict__ grow = gin - part * (uint32_t)(VEC * WIDTH);
    T* __restrict__ orow = gout - part * (uint32_t)(VEC * WIDTH);
    const uint32_t tail0 = num_groups * GROUP_COLS;
    vec qz[WIDTH];
#pragma unroll
    for (uint32_t w = 0; w < (uint32_t)WIDTH; ++w) {
#pragma unroll
        for (uint32_t u = 0; u < (uint32_t)VEC; ++u) {
            const uint32_t column = tail0 + part * (uint32_t)(VEC * WIDTH) + w * VEC + u;
            qz[w][u] = grow[column < cols ? column : cols - 1u];
        }
    }
    T carry = OP::template start<T>();

    // One group: in phase p every lane runs the recurrence over its columns from the carried state it holds and hands
    // its final state to its right neighbour; after the last phase all lanes are exact and the last lane's state goes
    // round to lane 0.
    auto scan_group = [&](const vec (&in)[WIDTH], vec (&ov)[WIDTH]) {
        T acc = carry;
#pragma unroll
        for (uint32_t phase = 0; phase < GROUP; ++phase) {
            acc = carry;
#pragma unroll
            for (uint32_t w = 0; w < (uint32_t)WIDTH; ++w) {
#pragma unroll
                for (uint32_t u = 0; u < (uint32_t)VEC; ++u) {
                    acc = OP::apply(acc, in[w][u]);
                    ov[w][u] = acc;
                }
            }
            carry = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry, acc);
        }
        carry = ovl_dpp_move<OVL_DPP_ROW_ROR1>(carry, acc);
    };

    // One batch: scan the DEPTH groups held in register set s, store them, refill the set with batch b + 2.
    auto process = [&](auto set, uint32_t b) {
        constexpr uint32_t s = decltype(set)::value;
        vec ov[DEPTH][WIDTH];
#pragma unroll
        for (uint32_t j = 0; j < (uint32_t)DEPTH; ++j) scan_group(q[s][j], ov[j]);
        // The scheduling fences keep the memory traffic of a batch together, after its arithmetic, and no load is
        // moved ahead of the last use of the registers it fills.
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (uint32_t j = 0; j < (uint32_t)DEPTH; ++j)
#pragma unroll
            for (uint32_t w = 0; w < (uint32_t)WIDTH; ++w)
                store_vector<ALIGNED, vec>(ov[j][w], gout + (uint64_t)b * BATCH_COLS + j * GROUP_COLS + w * VEC);
        // past the end a set is refilled with the last batch again, which keeps the loop free of branches
        const uint32_t next = b + 2u < num_batches ? b + 2u : last_batch;
#pragma unroll
        for (uint32_t j = 0; j < (uint32_t)DEPTH; ++j)
#pragma unroll
            for (uint32_t w = 0; w < (uint32_t)WIDTH; ++w)
                q[s][j][w] = load_vector<ALIGNED, vec>(gin + (uint64_t)next * BATCH_COLS + j * GROUP_COLS + w * VEC);
        __builtin_amdgcn_sched_barrier(0);
    };
    typedef std::integral_constant<uint32_t, 0> set0;
    typedef std::integral_constant<uint32_t, 1> set1;

    // straight-line pairs of batches (the wait counters of the loads in flight stay exact), then the odd one
    uint32_t b0 = 0;
#pragma unroll 1
    for (; b0 + 1u < num_batches; b0 += 2u) {
        process(set0(), b0);
        process(set1(), b0 + 1u);
    }
    if (b0 < num_batches) process(set0(), b0);
    if constexpr (DEPTH > 1) {
        // the single groups that end the row (the same number in every wavefront: the branches are uniform)
#pragma unroll
        for (uint32_t j = 0; j < TAIL_MAX; ++j) {
            if (j < tail) {
                vec ov[WIDTH];
                scan_group(qt[j], ov);
#pragma unroll
                for (uint32_t w = 0; w < (uint32_t)WIDTH; ++w)
                    store_vector<ALIGNED, vec>(ov[w], gout + (uint64_t)(num_batches * (uint32_t)DEPTH + j) * GROUP_COLS + w * VEC);
            }
        }
    }
    // The columns after the last whole group (fewer than one group's worth) run as one more group in which the
    // columns past the end of the row are skipped; they are stored element by element.  (A walk of one lane over them
    // waits for each load in turn.)
    if (tail0 < cols) {
        const uint32_t col0 = tail0 + part * (uint32_t)(VEC * WIDTH);
        vec ov[WIDTH] = {};
        T acc = carry;
#pragma unroll
        for (uint32_t phase = 0; phase < GROUP; ++phase) {
            acc = carry;
#pragma unroll
            for (uint32_t w = 0; w < (uint32_t)WIDTH; ++w) {
#pragma unroll
                for (uint32_t u = 0; u < (uint32_t)VEC; ++u) {
                    if (col0 + w * VEC + u >= cols) continue;
                    acc = OP::apply(acc, qz[w][u]);
                    ov[w][u] = acc;
                }
            }
            carry = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry, acc);
        }
#pragma unroll
        for (uint32_t w = 0; w < (uint32_t)WIDTH; ++w)
#pragma unroll
            for (uint32_t u = 0; u < (uint32_t)VEC; ++u)
                if (col0 + w * VEC + u < cols) orow[col0 + w * VEC + u] = ov[w][u];
    }
}

// LDS-fed lane-skewed scan, for 8-byte elements: a scan of float64 rows runs at the latency of its recurrence, and in
// the kernel above the hand-over between lanes is paid once per RUN columns, where RUN is limited by the shape of the
// memory requests (a lane that owns more than 32 consecutive bytes makes the wavefront's requests sparse).  Here the
// requests are made by other wavefronts: wavefronts 1-3 of the workgroup stream its four rows through three rotating
// LDS buffers of FED_CHUNK columns with dense 128-bit accesses (two chunks of loads in flight in registers), and
// wavefront 0 runs the skewed recurrence out of LDS and in place, sixteen lanes per row, each lane owning FED_SEG
// consecutive columns of every group of 16 * FED_SEG: the hand-over is paid once per FED_SEG additions.  Segments are
// padded by one vector in LDS so that the sixteen lanes of a group read and write without bank conflicts.
// cols must be a multiple of FED_CHUNK; x and out 16-byte aligned.  float64 [1024, 16384]: 59 us against 83 us.
constexpr uint32_t FED_SEG = 16, FED_GROUP_COLS = GROUP * FED_SEG, FED_CHUNK = 2 * FED_GROUP_COLS;

template <typename T, typename OP>
__global__ void __launch_bounds__(BLOCK)
fed_scan_kernel(const T* __restrict__ x, T* __restrict__ out, uint32_t rows, uint32_t cols) {
    constexpr uint32_t VEC = 16 / sizeof(T);
    typedef typename vec_of<T, VEC>::type vec;
    constexpr uint32_t W = FED_SEG / VEC;                          // vectors per lane and phase
    constexpr uint32_t PADDED_SEG = FED_SEG + VEC;                 // a segment and its padding
    constexpr uint32_t ROW_STRIDE = FED_CHUNK / FED_SEG * PADDED_SEG;
    constexpr uint32_t MOVERS = BLOCK - WAVE;
    constexpr uint32_t CHUNK_VECS = ROWS_PER_WAVE * FED_CHUNK / VEC;       // vectors of a chunk of the four rows
    constexpr uint32_t PER_MOVER = (CHUNK_VECS + MOVERS - 1) / MOVERS;
    __shared__ __attribute__((aligned(16))) T tile[3][ROWS_PER_WAVE][ROW_STRIDE];

    const uint32_t row0 = blockIdx.x * ROWS_PER_WAVE;
    const uint32_t num_chunks = cols / FED_CHUNK;

    // Movers: thread m owns vectors m, m + 192, ... of every chunk.  A vector that does not exist (past the chunk or
    // past the last row) is redirected to an existing one for loading and skipped when writing, so the loops are
    // free of branches and all loads of a chunk are in flight together.
    struct mover_regs { vec v[PER_MOVER]; };
    auto slot = [&](uint32_t m, uint32_t i, uint32_t& r, uint32_t& c) -> bool {
        const uint32_t v = m + i * MOVERS;
        r = v / (FED_CHUNK / VEC);
        c = (v % (FED_CHUNK / VEC)) * VEC;
        return v < CHUNK_VECS && row0 + r < rows;
    };
    auto lds_at = [&](uint32_t k, uint32_t r, uint32_t c) -> vec* {
        return reinterpret_cast<vec*>(&tile[k % 3u][r][c + (c / FED_SEG) * VEC]);
    };
    auto issue_loads = [&](uint32_t k, uint32_t m, mover_regs& regs) {
#pragma unroll
        for (uint32_t i = 0; i < PER_MOVER; ++i) {
            uint32_t r, c;
            if (!slot(m, i, r, c)) { r = 0; c = 0; }
            // (plain loads: with the non-temporal hint on loads and stores the mixed stream runs a quarter slower)
            regs.v[i] = *reinterpret_cast<const vec*>(x + (uint64_t)(row0 + r) * cols + (uint64_t)k * FED_CHUNK + c);
        }
    };
    auto write_lds = [&](uint32_t k, uint32_t m, const mover_regs& regs) {
#pragma unroll
        for (uint32_t i = 0; i < PER_MOVER; ++i) {
            uint32_t r, c;
            if (slot(m, i, r, c)) *lds_at(k, r, c) = regs.v[i];
        }
    };
    auto store_chunk = [&](uint32_t k, uint32_t m) {
        mover_regs regs;
#pragma unroll
        for (uint32_t i = 0; i < PER_MOVER; ++i) {
            uint32_t r, c;
            if (!slot(m, i, r, c)) { r = 0; c = 0; }
            regs.v[i] = *lds_at(k, r, c);
        }
#pragma unroll
        for (uint32_t i = 0; i < PER_MOVER; ++i) {
            uint32_t r, c;
            if (slot(m, i, r, c))
                __builtin_nontemporal_store(regs.v[i], reinterpret_cast<vec*>(
                    out + (uint64_t)(row0 + r) * cols + (uint64_t)k * FED_CHUNK + c));
        }
    };

    if (threadIdx.x >= WAVE) {
        const uint32_t m = threadIdx.x - WAVE;
        // chunk 0 and the even chunks travel through set_a, the odd ones through set_b: while chunk k is scanned,
        // chunk k + 1 goes to LDS from the set requested two steps ago and chunk k + 3 is requested into that set
        mover_regs set_a, set_b;
        issue_loads(0u, m, set_a);
        write_lds(0u, m, set_a);
        if (1u < num_chunks) issue_loads(1u, m, set_b);
        if (2u < num_chunks) issue_loads(2u, m, set_a);
        __syncthreads();
        auto step = [&](uint32_t k, mover_regs& regs) {
            if (k + 1u < num_chunks) write_lds(k + 1u, m, regs);
            if (k + 3u < num_chunks) issue_loads(k + 3u, m, regs);
            if (k >= 1u) store_chunk(k - 1u, m);
            __syncthreads();
        };
        uint32_t k = 0;
#pragma unroll 1
        for (; k + 1u < num_chunks; k += 2u) {
            step(k, set_b);
            step(k + 1u, set_a);
        }
        if (k < num_chunks) step(k, set_b);
        store_chunk(num_chunks - 1u, m);
    } else {
        // The scanning wavefront.  A group of lanes whose row does not exist works on whatever its part of the tile
        // holds: nobody stores it.
        const uint32_t lane = threadIdx.x;
        const uint32_t part = lane % GROUP, q = lane / GROUP;
        T carry = OP::template start<T>();
        vec set_a[W], set_b[W];
        auto fetch = [&](vec (&set)[W], const T* from) {
#pragma unroll
            for (uint32_t w = 0; w < W; ++w) set[w] = *reinterpret_cast<const vec*>(from + w * VEC);
        };
        // one group of 16 * FED_SEG columns: in phase p every lane runs the recurrence over its segment from the
        // state it holds and hands its final state to its right neighbour; after phase p lanes 0..p are exact
        auto run = [&](vec (&set)[W], T* to) {
            vec ov[W];
            T acc = carry;
#pragma unroll
            for (uint32_t phase = 0; phase < GROUP; ++phase) {
                acc = carry;
#pragma unroll
                for (uint32_t w = 0; w < W; ++w) {
#pragma unroll
                    for (uint32_t u = 0; u < VEC; ++u) {
                        acc = OP::apply(acc, set[w][u]);
                        ov[w][u] = acc;
                    }
                }
                carry = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry, acc);
            }
            carry = ovl_dpp_move<OVL_DPP_ROW_ROR1>(carry, acc);
#pragma unroll
            for (uint32_t w = 0; w < W; ++w) *reinterpret_cast<vec*>(to + w * VEC) = ov[w];
        };
        constexpr uint32_t GROUP_STRIDE = GROUP * PADDED_SEG;         // distance between a lane's segments of two groups
        __syncthreads();
        for (uint32_t k = 0; k < num_chunks; ++k) {
            T* here = &tile[k % 3u][q][part * PADDED_SEG];
            fetch(set_a, here);
            fetch(set_b, here + GROUP_STRIDE);
            run(set_a, here);
            run(set_b, here + GROUP_STRIDE);
            __syncthreads();
        }
    }
}

// The same with the results taken off the scanning wavefront, for tensors that give every compute unit at most one
// workgroup: a scan of float64 rows runs at the latency of its recurrence (a dependent float64 addition issues every
// 5 clocks), so everything that is not an addition is taken off the wavefront that runs it.  A workgroup of five wavefronts owns four rows and streams them through six rotating LDS buffers in
// chunks of CARRY_CHUNK = 16 * CARRY_SEG columns, one workgroup barrier per chunk:
//
//   loaders (wavefronts 3, 4)  global memory -> registers (CARRY_AHEAD chunks of requests in flight) -> LDS
//   scanner (wavefront 0)      reads its segments of the next chunk from LDS while it runs the skewed recurrence over
//                              the current one: sixteen lanes per row, lane p owns CARRY_SEG consecutive columns, sixteen
//                              phases of CARRY_SEG dependent operations and one hand-over (DPP row_shr:1) each.  It keeps
//                              no results: after the last phase every lane holds the exact state that enters its
//                              segment, and that one value per lane is all it writes to LDS (a 128-bit LDS write costs
//                              the issuing wavefront about 25 clocks, five operations of the recurrence; a read 5)
//   finisher (wavefront 1)     recomputes every segment from its exact entering state, one pass of CARRY_SEG operations
//                              in the same order, hence the same bits, and writes the results over the inputs in LDS
//   storer (wavefront 2)       LDS -> global memory
//
// Chunk c is written to LDS in step c - 2, read by the scanner in step c - 1, scanned in step c, finished in step
// c + 2 and stored in step c + 3; its buffer is written again in step c + 4.  Segments are padded by one vector in LDS
// so that the sixteen lanes of a group read and write without bank conflicts.  cols must be a multiple of CARRY_CHUNK;
// x and out 16-byte aligned.  The workgroup holds 105 KiB of LDS, one workgroup per compute unit: float64 [1024, 16384]
// 47 us against 58 us for the kernel above, [256, 65536] 154 against 192; with more workgroups than compute units the
// kernel above, three workgroups of which share a compute unit, is the faster one ([4096, 4096] 46 against 59 us).
constexpr uint32_t CARRY_SEG = 32, CARRY_CHUNK = GROUP * CARRY_SEG, CARRY_BUFFERS = 6, CARRY_AHEAD = 4, CARRY_LOADER_WAVES = 2;
constexpr uint32_t CARRY_BLOCK = (3 + CARRY_LOADER_WAVES) * WAVE;
// the phase of a group after which the scanner meets the others at the barrier: its LDS reads of the step are done
constexpr uint32_t CARRY_SYNC_PHASE = 8;

template <typename T, typename OP>
__global__ void __launch_bounds__(CARRY_BLOCK)
carry_scan_kernel(const T* __restrict__ x, T* __restrict__ out, uint32_t rows, uint32_t cols) {
    constexpr uint32_t VEC = 16 / sizeof(T);
    typedef typename vec_of<T, VEC>::type vec;
    constexpr uint32_t W = CARRY_SEG / VEC;                          // vectors per lane and chunk
    constexpr uint32_t PADDED_SEG = CARRY_SEG + VEC;                 // a segment and its padding
    constexpr uint32_t ROW_STRIDE = GROUP * PADDED_SEG;
    constexpr uint32_t CHUNK_VECS = ROWS_PER_WAVE * CARRY_CHUNK / VEC;       // vectors of a chunk of the four rows
    constexpr uint32_t READS_PER_PHASE = W / CARRY_SYNC_PHASE;
    static_assert(READS_PER_PHASE * CARRY_SYNC_PHASE == W, "the scanner's reads of a chunk fill the phases before the barrier");
    __shared__ __attribute__((aligned(16))) T tile[CARRY_BUFFERS][ROWS_PER_WAVE][ROW_STRIDE];
    __shared__ T entering[CARRY_BUFFERS][WAVE];

    const uint32_t row0 = blockIdx.x * ROWS_PER_WAVE;
    const uint32_t n = cols / CARRY_CHUNK;                           // chunks, and steps 0 .. n + 2
    const uint32_t wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    // Every wavefront passes the same n + 3 barriers: one after the first two chunks are in LDS, then one at the end
    // of each of the steps 0 .. n + 1.

    if (wave == 0) {
        // A group of lanes whose row does not exist works on what the loaders put there (a copy of the last row):
        // nobody stores it.
        const uint32_t part = lane % GROUP, q = lane / GROUP;
        T* mine = &tile[0][q][part * PADDED_SEG];
        constexpr uint32_t BUFFER = ROWS_PER_WAVE * ROW_STRIDE;
        T carry = OP::template start<T>();
        vec in[2][W];
        __syncthreads();
#pragma unroll
        for (uint32_t w = 0; w < W; ++w) in[0][w] = *reinterpret_cast<const vec*>(mine + w * VEC);
        uint32_t next = 1, slot = 0;                               // buffer of the chunk after this one; this chunk's slot
        // one chunk out of register set `cur`, in step g: in phase p every lane runs the recurrence over its segment
        // from the state it holds and hands its final state to its right neighbour; after phase p lanes 0 .. p are
        // exact.  Meanwhile the segments of chunk g + 1 arrive in the other register set.
        auto scan_chunk = [&](auto cur_c) {
            constexpr uint32_t cur = decltype(cur_c)::value, nxt = cur ^ 1u;
            const T* ahead = mine + next * BUFFER;
            T acc = carry;
#pragma unroll
            for (uint32_t phase = 0; phase < GROUP; ++phase) {
                acc = carry;
#pragma unroll
                for (uint32_t w = 0; w < W; ++w)
#pragma unroll
                    for (uint32_t u = 0; u < VEC; ++u) acc = OP::apply(acc, in[cur][w][u]);
                carry = ovl_dpp_move<OVL_DPP_ROW_SHR1>(carry, acc);
                if (phase < CARRY_SYNC_PHASE) {
#pragma unroll
                    for (uint32_t j = 0; j < READS_PER_PHASE; ++j) {
                        const uint32_t w = phase * READS_PER_PHASE + j;
                        in[nxt][w] = *reinterpret_cast<const vec*>(ahead + w * VEC);
                    }
                }
                // (the fences keep each read in its phase and the barrier in its place)
                __builtin_amdgcn_sched_barrier(0);
                if (phase == CARRY_SYNC_PHASE) {
                    __syncthreads();
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // lanes 1 .. 15 now hold their left neighbour's exact final state, lane 0 the state that entered the
            // chunk: what enters each lane's segment
            entering[slot][lane] = carry;
            // the last lane finished the chunk: its state is the carry into the next one
            carry = ovl_dpp_move<OVL_DPP_ROW_ROR1>(carry, acc);
            next = next + 1u == CARRY_BUFFERS ? 0u : next + 1u;
            slot = slot + 1u == CARRY_BUFFERS ? 0u : slot + 1u;
            __builtin_amdgcn_sched_barrier(0);
        };
        typedef std::integral_constant<uint32_t, 0> set0;
        typedef std::integral_constant<uint32_t, 1> set1;
        uint32_t g = 0;
#pragma unroll 1
        for (; g + 1u < n; g += 2u) {
            scan_chunk(set0());
            scan_chunk(set1());
        }
        if (g < n) scan_chunk(set0());
        __syncthreads();                                           // steps n and n + 1: the others finish and store
        __syncthreads();
    } else if (wave == 1) {
        // The finisher: chunk s - 2 in step s.
        const uint32_t part = lane % GROUP, q = lane / GROUP;
        __syncthreads();
        __syncthreads();
        __syncthreads();
        for (uint32_t s = 2; s <= n + 1u; ++s) {
            const uint32_t buffer = (s - 2u) % CARRY_BUFFERS;
            T* mine = &tile[buffer][q][part * PADDED_SEG];
            vec v[W];
#pragma unroll
            for (uint32_t w = 0; w < W; ++w) v[w] = *reinterpret_cast<const vec*>(mine + w * VEC);
            T acc = entering[buffer][lane];
#pragma unroll
            for (uint32_t w = 0; w < W; ++w)
#pragma unroll
                for (uint32_t u = 0; u < VEC; ++u) {
                    acc = OP::apply(acc, v[w][u]);
                    v[w][u] = acc;
                }
#pragma unroll
            for (uint32_t w = 0; w < W; ++w) *reinterpret_cast<vec*>(mine + w * VEC) = v[w];
            __syncthreads();
        }
    } else {
        // Loaders and storer: thread m of `movers` owns vectors m, m + movers, ... of every chunk.  A loader's vector
        // past the last row is a second copy of the last row's; the storer skips it.
        const bool storer = wave == 2;
        constexpr uint32_t LOADERS = CARRY_LOADER_WAVES * WAVE;
        constexpr uint32_t PER_LOADER = CHUNK_VECS / LOADERS, PER_STORER = CHUNK_VECS / WAVE;
        static_assert(PER_LOADER * LOADERS == CHUNK_VECS && PER_STORER * WAVE == CHUNK_VECS, "whole vectors per thread");
        auto place = [&](uint32_t v, uint32_t& global_offset, uint32_t& lds_offset, bool& exists) {
            const uint32_t r = v / (CARRY_CHUNK / VEC), c = (v % (CARRY_CHUNK / VEC)) * VEC;
            exists = row0 + r < rows;
            global_offset = (exists ? row0 + r : rows - 1u) * cols + c;           // rows * cols < 2^32
            lds_offset = r * ROW_STRIDE + c + (c / CARRY_SEG) * VEC;
        };
        if (storer) {
            uint32_t global_offset[PER_STORER], lds_offset[PER_STORER];
            bool exists[PER_STORER];
#pragma unroll
            for (uint32_t i = 0; i < PER_STORER; ++i) place(lane + i * WAVE, global_offset[i], lds_offset[i], exists[i]);
            auto store_chunk = [&](uint32_t c) {
                const T* buffer = &tile[c % CARRY_BUFFERS][0][0];
                vec regs[PER_STORER];
#pragma unroll
                for (uint32_t i = 0; i < PER_STORER; ++i) regs[i] = *reinterpret_cast<const vec*>(buffer + lds_offset[i]);
#pragma unroll
                for (uint32_t i = 0; i < PER_STORER; ++i)
                    if (exists[i])
                        __builtin_nontemporal_store(regs[i], reinterpret_cast<vec*>(out + global_offset[i] + c * CARRY_CHUNK));
            };
            __syncthreads();
            __syncthreads();
            __syncthreads();
            __syncthreads();
            for (uint32_t s = 3; s <= n + 1u; ++s) {
                store_chunk(s - 3u);
                __syncthreads();
            }
            store_chunk(n - 1u);                                   // step n + 2
        } else {
            const uint32_t m = threadIdx.x - 3u * WAVE;
            uint32_t global_offset[PER_LOADER], lds_offset[PER_LOADER];
#pragma unroll
            for (uint32_t i = 0; i < PER_LOADER; ++i) {
                bool exists;
                place(m + i * LOADERS, global_offset[i], lds_offset[i], exists);
            }
            // Plain loads: with the non-temporal hint on both sides the mixed stream of reads and writes runs a
            // quarter slower.  A chunk past the end of the row is requested as the last chunk once more and lands in
            // a buffer that nobody reads any more, so the steps are free of conditions and the compiler's counts of
            // the requests in flight stay exact.
            auto request = [&](uint32_t c, vec (&regs)[PER_LOADER]) {
                const uint32_t cc = c < n ? c : n - 1u;
#pragma unroll
                for (uint32_t i = 0; i < PER_LOADER; ++i)
                    regs[i] = *reinterpret_cast<const vec*>(x + global_offset[i] + cc * CARRY_CHUNK);
            };
            auto to_lds = [&](uint32_t c, const vec (&regs)[PER_LOADER]) {
                T* buffer = &tile[c % CARRY_BUFFERS][0][0];
#pragma unroll
                for (uint32_t i = 0; i < PER_LOADER; ++i) *reinterpret_cast<vec*>(buffer + lds_offset[i]) = regs[i];
            };
            vec set[CARRY_AHEAD][PER_LOADER];
            {
                vec first[2][PER_LOADER];
                request(0u, first[0]);
                request(1u, first[1]);
#pragma unroll
                for (uint32_t a = 0; a < CARRY_AHEAD; ++a) request(2u + a, set[(2u + a) % CARRY_AHEAD]);
                to_lds(0u, first[0]);
                to_lds(1u, first[1]);
            }
            __syncthreads();
            // step s: chunk s + 2 goes to LDS from the register set requested CARRY_AHEAD steps ago, which is then
            // requested again with chunk s + 2 + CARRY_AHEAD
            auto step = [&](uint32_t s, vec (&regs)[PER_LOADER]) {
                to_lds(s + 2u, regs);
                request(s + 2u + CARRY_AHEAD, regs);
                __syncthreads();
            };
            uint32_t s = 0;
#pragma unroll 1
            for (; s + CARRY_AHEAD <= n + 2u; s += CARRY_AHEAD) {
#pragma unroll
                for (uint32_t a = 0; a < CARRY_AHEAD; ++a) step(s + a, set[(2u + a) % CARRY_AHEAD]);
            }
#pragma unroll
            for (uint32_t a = 0; a < CARRY_AHEAD; ++a)
                if (s + a <= n + 1u) step(s + a, set[(2u + a) % CARRY_AHEAD]);
        }
    }
}

// Rows shorter than one group of the kernels above: one lane per row.
template <typename T, typename OP>
__global__ void __launch_bounds__(BLOCK)
row_per_lane_scan_kernel(const T* __restrict__ x, T* __restrict__ out, uint32_t rows, uint32_t cols) {
    const uint32_t row = blockIdx.x * BLOCK + threadIdx.x;     // the grid has at most 2^24 - 1 workgroups
    if (row >= rows) return;
    const T* in_row = x + (uint64_t)row * cols;
    T* out_row = out + (uint64_t)row * cols;
    T acc = in_row[0];
    out_row[0] = acc;
    for (uint32_t i = 1; i < cols; ++i) {
        acc = OP::apply(acc, in_row[i]);
        out_row[i] = acc;
    }
}

template <typename T, typename OP>
int scan(const char* who, const T* x, uint32_t rows, uint32_t cols, T* out, void* hip_stream) {
    if (x == nullptr || out == nullptr) return fail(OVL_EINVAL, std::string(who) + ": null tensor");
    if (rows == 0 || cols == 0) return fail(OVL_EINVAL, std::string(who) + ": rows and cols must be positive");
    if ((uint64_t)rows * cols >= (1ull << 32)) return fail(OVL_EINVAL, std::string(who) + ": rows * cols must be below 2^32");
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    // measured on MI355X: one 128-bit vector per lane and phase for 4-byte elements (the scan runs at the speed of
    // memory), two for 8-byte elements (it runs at the latency of the recurrence, and the hand-over is paid half as
    // often); request bursts of 1 KiB per row
    constexpr int VEC = 16 / sizeof(T), WIDTH = sizeof(T) == 8 ? 2 : 1, DEPTH = 4 / WIDTH;
    constexpr uint32_t GROUP_COLS = GROUP * VEC * WIDTH;
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    const bool rows_aligned = aligned && cols % VEC == 0;      // every row starts on a 16-byte boundary
    const dim3 block(BLOCK);
    bool fed = false;
    if constexpr (sizeof(T) == 8) {
        // 8-byte elements: the recurrence sets the pace, and the LDS-fed kernels pay fewer hand-overs
        if (aligned && cols % FED_CHUNK == 0) {
            fed = true;
            const uint32_t groups = (rows + ROWS_PER_WAVE - 1) / ROWS_PER_WAVE;
            // the kernel whose scanning wavefront keeps no results runs one workgroup per compute unit: it is chosen
            // when the workgroups fit in one round, or fill their rounds and have rows long enough to pay for the
            // start of its pipeline in each
            const uint32_t rounds = (groups + OVL_NUM_CU - 1) / OVL_NUM_CU;
            const bool one_round = groups <= OVL_NUM_CU;
            const bool full_rounds = 10u * groups >= 9u * rounds * OVL_NUM_CU && cols / CARRY_CHUNK >= 24u;
            if (cols % CARRY_CHUNK == 0 && (one_round || full_rounds))
                hipLaunchKernelGGL((carry_scan_kernel<T, OP>), dim3(groups), dim3(CARRY_BLOCK), 0, stream, x, out, rows, cols);
            else
                hipLaunchKernelGGL((fed_scan_kernel<T, OP>), dim3(groups), block, 0, stream, x, out, rows, cols);
        }
    }
    if (fed) {
    } else if (cols >= GROUP_COLS) {
        const dim3 grid((rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK);
        // (rows of fewer than DEPTH groups: one group per request)
        if (cols >= GROUP_COLS * DEPTH) {
            if (rows_aligned)
                hipLaunchKernelGGL((skewed_scan_kernel<T, OP, VEC, WIDTH, DEPTH, true>), grid, block, 0, stream, x, out, rows, cols);
            else
                hipLaunchKernelGGL((skewed_scan_kernel<T, OP, VEC, WIDTH, DEPTH, false>), grid, block, 0, stream, x, out, rows, cols);
        } else {
            if (rows_aligned)
                hipLaunchKernelGGL((skewed_scan_kernel<T, OP, VEC, WIDTH, 1, true>), grid, block, 0, stream, x, out, rows, cols);
            else
                hipLaunchKernelGGL((skewed_scan_kernel<T, OP, VEC, WIDTH, 1, false>), grid, block, 0, stream, x, out, rows, cols);
        }
    } else {
        // (a launch has fewer than 2^32 threads)
        if (rows > 0xffffffffu - BLOCK)
            return fail(OVL_EINVAL, std::string(who) + ": more than 2^32 - 257 rows");
        const dim3 grid((rows + BLOCK - 1) / BLOCK);
        hipLaunchKernelGGL((row_per_lane_scan_kernel<T, OP>), grid, block, 0, stream, x, out, rows, cols);
    }
    const hipError_t err = hipPeekAtLastError();
    if (err != hipSuccess) {
        (void)hipGetLastError();
        return fail(OVL_EHIP, std::string(who) + ": " + hipGetErrorString(err));
    }
    return OVL_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// The reassociating scan (ovl_*_reassociated): one workgroup per row, the row taken in steps of 256 vectors.  Every
// thread scans its own 128-bit vector, the threads' totals are scanned across the wavefront with six lane-to-lane
// steps (a tree, hence another association of the operands than the sequential recurrence), the four wavefront totals go through LDS, and the running total of the steps before is
// carried in a register.  Data moves exactly once in coalesced 128-bit accesses, several steps of loads in flight, so
// the kernel runs at the speed of memory whatever the latency of one addition; the price is the bits: results differ
// from the sequential recurrence by rounding (the distance is reported by the tests and the benchmark).
template <typename T, typename OP, int VEC, int AHEAD>
__global__ void __launch_bounds__(BLOCK)
reassociated_scan_kernel(const T* __restrict__ x, T* __restrict__ out, uint32_t cols) {
    typedef typename vec_of<T, VEC>::type vec;
    __shared__ T wave_totals[2][BLOCK / WAVE];
    const uint32_t lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const T* __restrict__ in_row = x + (uint64_t)blockIdx.x * cols;
    T* __restrict__ out_row = out + (uint64_t)blockIdx.x * cols;
    const uint32_t step_cols = BLOCK * VEC;
    const uint32_t steps = (cols + step_cols - 1u) / step_cols;
    T carry = OP::template start<T>();
    uint32_t buffer = 0;
    // a vector past the end of the row holds the value that leaves its neighbours unchanged and is not stored
    auto fetch = [&](uint32_t step) -> vec {
        const uint32_t col = step * step_cols + threadIdx.x * VEC;
        vec r;
        if (step < steps && col < cols) r = *reinterpret_cast<const vec*>(in_row + col);
        else
#pragma unroll
            for (uint32_t u = 0; u < (uint32_t)VEC; ++u) r[u] = OP::template start<T>();
        return r;
    };
    // AHEAD steps of loads are always in flight: a register is refilled as soon as its vector has been taken
    vec v[AHEAD];
#pragma unroll
    for (uint32_t a = 0; a < (uint32_t)AHEAD; ++a) v[a] = fetch(a);
    for (uint32_t s0 = 0; s0 < steps; s0 += AHEAD) {
#pragma unroll
        for (uint32_t a = 0; a < (uint32_t)AHEAD; ++a) {
            if (s0 + a >= steps) break;         // uniform over the workgroup
            const uint32_t col = (s0 + a) * step_cols + threadIdx.x * VEC;
            vec mine = v[a];
            v[a] = fetch(s0 + a + AHEAD);
#pragma unroll
            for (uint32_t u = 1; u < (uint32_t)VEC; ++u) mine[u] = OP::apply(mine[u - 1], mine[u]);
            // inclusive scan of the threads' totals over the wavefront
            const T unit = OP::template start<T>();
            const T inclusive = ovl_wave_inclusive_scan(mine[VEC - 1], unit, [](T a, T b) { return OP::apply(a, b); });
            const T before_me = ovl_wave_shift_up(inclusive, unit);     // total of the lanes below this one
            if (lane == WAVE - 1u) wave_totals[buffer][wave] = inclusive;
            __syncthreads();
            T base = carry, all = carry;
#pragma unroll
            for (uint32_t w = 0; w < BLOCK / WAVE; ++w) {
                const T t = wave_totals[buffer][w];
                if (w < wave) base = OP::apply(base, t);
                all = OP::apply(all, t);
            }
            base = OP::apply(base, before_me);
#pragma unroll
            for (uint32_t u = 0; u < (uint32_t)VEC; ++u) mine[u] = OP::apply(base, mine[u]);
            if (col < cols) __builtin_nontemporal_store(mine, reinterpret_cast<vec*>(out_row + col));
            carry = all;
            // the next step writes the other buffer: a thread can only get there after every thread has passed this
            // step's barrier, and can only write this buffer again after the next barrier, behind all reads of it
            buffer ^= 1u;
        }
    }
}

template <typename T, typename OP>
int reassociated_scan(const char* who, const T* x, uint32_t rows, uint32_t cols, T* out, void* hip_stream) {
    if (x == nullptr || out == nullptr) return fail(OVL_EINVAL, std::string(who) + ": null tensor");
    if (rows == 0 || cols == 0) return fail(OVL_EINVAL, std::string(who) + ": rows and cols must be positive");
    if ((uint64_t)rows * cols >= (1ull << 32)) return fail(OVL_EINVAL, std::string(who) + ": rows * cols must be below 2^32");
    constexpr int VEC = 16 / sizeof(T), AHEAD = OVL_SCAN_AHEAD;
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
    // rows of whole, aligned vectors only; anything else takes the order-preserving kernels
    // (column indices of the last, partial step must not wrap: rows that long also go the other way)
    if (!aligned || cols % VEC != 0 || rows >= (1u << 24) || cols > 0xffffffffu - 16u * BLOCK)
        return scan<T, OP>(who, x, rows, cols, out, hip_stream);
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    hipLaunchKernelGGL((reassociated_scan_kernel<T, OP, VEC, AHEAD>), dim3(rows), dim3(BLOCK), 0, stream, x, out, cols);
    const hipError_t err = hipPeekAtLastError();
    if (err != hipSuccess) {
        (void)hipGetLastError();
        return fail(OVL_EHIP, std::string(who) + ": " + hipGetErrorString(err));
    }
    return OVL_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// Measurement aid: what moving a [rows, cols] float64 tensor costs when one workgroup owns a strip of LINES neighbouring
// lines (columns) and walks down the rows, as the kernels that scan along the first axis do (hipgen/colscan_kernel.py).
// Every load instruction of a wavefront reads 64 / LINES rows, LINES * 8 bytes of each; eight rows per thread are in
// flight.  MODE 1 only loads (the values are added up and the sum is stored where no run reaches), 2 only stores
// (the row index), 3 copies.
// ---------------------------------------------------------------------------------------------------------------------
constexpr int STRIP_THREADS = 256, STRIP_IN_FLIGHT = 8;

template <int LINES, int MODE>
__global__ __launch_bounds__(STRIP_THREADS) void strip_copy_kernel(const double* __restrict__ x, double* __restrict__ out,
                                                                   uint32_t rows, uint32_t cols) {
    constexpr uint32_t ROWS_PER_PASS = STRIP_THREADS / LINES, ROWS_PER_STEP = ROWS_PER_PASS * STRIP_IN_FLIGHT;
    // Strips narrower than a 128-byte line share lines with their neighbours; as in the generated scans, the
    // workgroups of one XCD (every eighth) take the strips that share: groups of SHARE neighbours when every row
    // starts on a line boundary, else one contiguous range per XCD.
    constexpr uint32_t SHARE = 128 / (LINES * 8) > 1 ? 128 / (LINES * 8) : 1;
    const uint32_t total = gridDim.x;
    uint32_t strip = blockIdx.x;
    if (SHARE > 1 && (cols * 8u) % 128u == 0u && total >= 8u * SHARE) {
        const uint32_t whole = total / (8u * SHARE) * (8u * SHARE);
        if (blockIdx.x < whole)
            strip = blockIdx.x / (8u * SHARE) * (8u * SHARE) + blockIdx.x % 8u * SHARE + blockIdx.x / 8u % SHARE;
    } else if (SHARE > 1 && total >= 16u) {
        const uint32_t q = total / 8u, r = total % 8u, xcd = blockIdx.x % 8u;
        strip = xcd * q + (xcd < r ? xcd : r) + blockIdx.x / 8u;
    }
    uint32_t c = strip * LINES + threadIdx.x % LINES;
    const bool line_exists = c < cols;
    if (!line_exists) c = cols - 1u;          // a thread past the last line loads that line once more and stores nothing
    const uint32_t r0 = threadIdx.x / LINES;
    const double* p = x + (uint64_t)r0 * cols + c;
    double* q = out + (uint64_t)r0 * cols + c;
    const uint64_t pass_stride = (uint64_t)ROWS_PER_PASS * cols;
    double sum = 0.0;
    uint32_t base = 0;
    // steps all of whose rows exist: no conditions around the loads
    for (; base + ROWS_PER_STEP <= rows; base += ROWS_PER_STEP) {
        double v[STRIP_IN_FLIGHT];
        #pragma unroll
        for (uint32_t u = 0; u < STRIP_IN_FLIGHT; ++u) v[u] = (MODE & 1) ? p[u * pass_stride] : (double)(base + u * ROWS_PER_PASS + r0);
        if (MODE & 2) {
            if (line_exists) {
                #pragma unroll
                for (uint32_t u = 0; u < STRIP_IN_FLIGHT; ++u) __builtin_nontemporal_store(v[u], &q[u * pass_stride]);
            }
        } else {
            #pragma unroll
            for (uint32_t u = 0; u < STRIP_IN_FLIGHT; ++u) sum += v[u];
        }
        p += STRIP_IN_FLIGHT * pass_stride;
        q += STRIP_IN_FLIGHT * pass_stride;
    }
    // the last rows
    for (uint32_t r = base + r0; r < rows; r += ROWS_PER_PASS) {
        const double v = (MODE & 1) ? x[(uint64_t)r * cols + c] : (double)r;
        if (MODE & 2) {
            if (line_exists) __builtin_nontemporal_store(v, &out[(uint64_t)r * cols + c]);
        } else {
            sum += v;
        }
    }
    if (!(MODE & 2) && sum == -1.2345e300) out[0] = sum;
}

template <int LINES>
void launch_strip_copy(int mode, const double* x, double* out, uint32_t rows, uint32_t cols, hipStream_t stream) {
    const dim3 grid((cols + LINES - 1) / LINES), block(STRIP_THREADS);
    if (mode == 1) hipLaunchKernelGGL((strip_copy_kernel<LINES, 1>), grid, block, 0, stream, x, out, rows, cols);
    else if (mode == 2) hipLaunchKernelGGL((strip_copy_kernel<LINES, 2>), grid, block, 0, stream, x, out, rows, cols);
    else hipLaunchKernelGGL((strip_copy_kernel<LINES, 3>), grid, block, 0, stream, x, out, rows, cols);
}

}  // namespace

extern "C" {

const char* ovl_scan_last_error(void) { return g_last_error.c_str(); }

int ovl_strip_copy_f64(const double* x, uint32_t rows, uint32_t cols, double* out, uint32_t lines, uint32_t mode,
                       void* hip_stream) {
    const char* who = "ovl_strip_copy_f64";
    if (x == nullptr || out == nullptr) return fail(OVL_EINVAL, std::string(who) + ": null tensor");
    if (rows == 0 || cols == 0) return fail(OVL_EINVAL, std::string(who) + ": rows and cols must be positive");
    if ((uint64_t)rows * cols >= (1ull << 32)) return fail(OVL_EINVAL, std::string(who) + ": rows * cols must be below 2^32");
    if (mode < 1 || mode > 3) return fail(OVL_EINVAL, std::string(who) + ": mode is 1 (load), 2 (store) or 3 (copy)");
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    if (lines == 4) launch_strip_copy<4>((int)mode, x, out, rows, cols, stream);
    else if (lines == 8) launch_strip_copy<8>((int)mode, x, out, rows, cols, stream);
    else if (lines == 16) launch_strip_copy<16>((int)mode, x, out, rows, cols, stream);
    else return fail(OVL_EINVAL, std::string(who) + ": 4, 8 or 16 lines per workgroup");
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess) return fail(OVL_EHIP, std::string(who) + ": " + hipGetErrorString(err));
    return OVL_OK;
}

int ovl_cumsum_f32_reassociated(const float* x, uint32_t rows, uint32_t cols, float* out, void* hip_stream) {
    return reassociated_scan<float, op_sum>("ovl_cumsum_f32_reassociated", x, rows, cols, out, hip_stream);
}

int ovl_cumprod_f32_reassociated(const float* x, uint32_t rows, uint32_t cols, float* out, void* hip_stream) {
    return reassociated_scan<float, op_product>("ovl_cumprod_f32_reassociated", x, rows, cols, out, hip_stream);
}

int ovl_cumsum_f64_reassociated(const double* x, uint32_t rows, uint32_t cols, double* out, void* hip_stream) {
    return reassociated_scan<double, op_sum>("ovl_cumsum_f64_reassociated", x, rows, cols, out, hip_stream);
}

int ovl_cumprod_f64_reassociated(const double* x, uint32_t rows, uint32_t cols, double* out, void* hip_stream) {
    return reassociated_scan<double, op_product>("ovl_cumprod_f64_reassociated", x, rows, cols, out, hip_stream);
}

int ovl_cumsum_f32(const float* x, uint32_t rows, uint32_t cols, float* out, void* hip_stream) {
    return scan<float, op_sum>("ovl_cumsum_f32", x, rows, cols, out, hip_stream);
}

int ovl_cumprod_f32(const float* x, uint32_t rows, uint32_t cols, float* out, void* hip_stream) {
    return scan<float, op_product>("ovl_cumprod_f32", x, rows, cols, out, hip_stream);
}

int ovl_cumsum_f64(const double* x, uint32_t rows, uint32_t cols, double* out, void* hip_stream) {
    return scan<double, op_sum>("ovl_cumsum_f64", x, rows, cols, out, hip_stream);
}

int ovl_cumprod_f64(const double* x, uint32_t rows, uint32_t cols, double* out, void* hip_stream) {
    return scan<double, op_product>("ovl_cumprod_f64", x, rows, cols, out, hip_stream);
}

}  // extern "C"
