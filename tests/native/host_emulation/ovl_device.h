// Test infrastructure: a stand-in for opveclib_amd/csrc/ovl_device.h (and for the HIP runtime header it includes) that
// lets the generated operator sources compile as plain C++ for the host and run there, one host thread per GPU thread
// of a workgroup, workgroups one after the other:
//
//   * blockIdx / threadIdx / gridDim / blockDim, __syncthreads (a barrier over the threads of the workgroup),
//     __shared__ (one static copy, as there is one workgroup at a time), hipLaunchKernelGGL;
//   * the lane-to-lane moves of the scan kernels (ovl_dpp_move) through a table shared by the 64 threads of a wavefront;
//   * the float32 exp / log / tanh of ovl_math.h in their host build, IEEE division where the device uses its
//     reciprocal based sequences (both are compared with IEEE division exhaustively on the GPU);
//   * every other math function from the host C library, which is also what the oracle calls.
//
// The host threads of a wavefront do not run in lockstep: a kernel that relies on all lanes finishing one instruction
// before any starts the next (beyond __syncthreads and the lane moves) cannot be run this way.
//
// Built with -fsanitize=address on buffers of exactly the tensors' sizes, a run shows every out-of-bounds access of a
// kernel without a GPU; its results are compared with the oracle's by tests/test_host_emulation.py.  Never part of the
// product: nothing in the package includes or loads it.
#ifndef OVL_DEVICE_H_
#define OVL_DEVICE_H_

#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <functional>
#include <thread>
#include <vector>

#include "ovl_math.h"

typedef struct ovl_tensor {
    void*    data;
    int32_t  dtype;
    uint64_t len;
} ovl_tensor;

#define OVL_NUM_CU 256u
#define OVL_OK 0
#define OVL_EARGS 1
#define OVL_EHIP 4
#define OVL_EALIGN 5

#define __global__
#define __device__
#define __forceinline__ inline
#define __launch_bounds__(n)
#define __shared__ static

struct dim3 {
    uint32_t x, y, z;
    dim3(uint32_t x_ = 1, uint32_t y_ = 1, uint32_t z_ = 1) : x(x_), y(y_), z(z_) {}
};
static thread_local dim3 blockIdx, threadIdx;
static dim3 gridDim, blockDim;
typedef void* hipStream_t;
typedef int hipError_t;
enum { hipSuccess = 0 };
static inline hipError_t hipPeekAtLastError() { return hipSuccess; }
static inline hipError_t hipGetLastError() { return hipSuccess; }
static inline const char* hipGetErrorString(hipError_t) { return "no error"; }

static pthread_barrier_t ovl_emulated_block_barrier;
static pthread_barrier_t ovl_emulated_wave_barrier[16];
static uint64_t ovl_emulated_lane_values[1024];

static inline void __syncthreads() { pthread_barrier_wait(&ovl_emulated_block_barrier); }
#define __builtin_amdgcn_sched_barrier(mask) ((void)0)

// One host thread per GPU thread of a workgroup; the workgroups of the grid run one after the other.  A thread that
// returns from the kernel early still takes part in the barrier that ends the workgroup.
static inline void ovl_emulate_launch(dim3 grid, dim3 block, const std::function<void()>& kernel) {
    gridDim = grid;
    blockDim = block;
    const uint32_t waves = (block.x + 63u) / 64u;
    if (block.x > 1024u || block.y != 1 || block.z != 1 || grid.y != 1 || grid.z != 1) abort();
    pthread_barrier_init(&ovl_emulated_block_barrier, nullptr, block.x);
    for (uint32_t w = 0; w < waves; ++w) {
        const uint32_t lanes = (w + 1u) * 64u <= block.x ? 64u : block.x - w * 64u;
        pthread_barrier_init(&ovl_emulated_wave_barrier[w], nullptr, lanes);
    }
    pthread_barrier_t block_done;
    pthread_barrier_init(&block_done, nullptr, block.x);
    std::vector<std::thread> threads;
    for (uint32_t t = 0; t < block.x; ++t)
        threads.emplace_back([&, t]() {
            threadIdx = dim3(t);
            for (uint32_t b = 0; b < grid.x; ++b) {
                blockIdx = dim3(b);
                kernel();
                pthread_barrier_wait(&block_done);
            }
        });
    for (auto& thread : threads) thread.join();
    pthread_barrier_destroy(&block_done);
    pthread_barrier_destroy(&ovl_emulated_block_barrier);
    for (uint32_t w = 0; w < waves; ++w) pthread_barrier_destroy(&ovl_emulated_wave_barrier[w]);
}
#define hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, ...) \
    ovl_emulate_launch((grid), (block), [=]() { kernel(__VA_ARGS__); })

static inline int8_t ovl_abs_8(int8_t x) { return (x < 0) ? -x : x; }
static inline int16_t ovl_abs_16(int16_t x) { return (x < 0) ? -x : x; }

#define OVL_LOAD_NT(ptr) __builtin_nontemporal_load(ptr)
#define OVL_LOAD_PLAIN(ptr) (*(ptr))
#define OVL_STORE_NT(value, ptr) __builtin_nontemporal_store(value, ptr)
#define OVL_STORE_PLAIN(value, ptr) (*(ptr) = (value))

// Lane i of every row of 16 lanes receives the value of lane i - 1; lane 0 of the row keeps `old` (row_shr:1) or
// receives lane 15 (row_ror:1).  All 64 threads of the wavefront arrive here together, as its lanes do on the device.
#define OVL_DPP_ROW_SHR1 0x111
#define OVL_DPP_ROW_ROR1 0x121
template <int CTRL, typename T>
static inline T ovl_dpp_move(T old, T src) {
    static_assert(sizeof(T) <= 8, "lane moves carry at most 8 bytes");
    const uint32_t t = threadIdx.x, wave = t / 64u, in_row = t % 16u;
    uint64_t bits = 0;
    memcpy(&bits, &src, sizeof(T));
    ovl_emulated_lane_values[t] = bits;
    pthread_barrier_wait(&ovl_emulated_wave_barrier[wave]);
    T result = old;
    if (in_row != 0u) memcpy(&result, &ovl_emulated_lane_values[t - 1u], sizeof(T));
    else if (CTRL == OVL_DPP_ROW_ROR1) memcpy(&result, &ovl_emulated_lane_values[t + 15u], sizeof(T));
    pthread_barrier_wait(&ovl_emulated_wave_barrier[wave]);
    return result;
}

// The lane-move builtin for 32-bit values with the patterns the hand-written scans use: row_shr:n (0x110 + n),
// row_ror:1 (0x121), wave_shr:1 (0x138), row_bcast:15 (0x142), row_bcast:31 (0x143).  Rows of 16 lanes whose bit is
// clear in row_mask, and lanes the pattern gives no source, receive `old`.
static inline int ovl_emulated_update_dpp(int old, int src, int ctrl, int row_mask) {
    const uint32_t t = threadIdx.x, wave = t / 64u, lane = t % 64u, row = lane / 16u, in_row = lane % 16u;
    ovl_emulated_lane_values[t] = (uint32_t)src;
    pthread_barrier_wait(&ovl_emulated_wave_barrier[wave]);
    int from = -1;
    if (ctrl > 0x110 && ctrl <= 0x11f) { if (in_row >= (uint32_t)(ctrl - 0x110)) from = (int)lane - (ctrl - 0x110); }
    else if (ctrl == 0x121) from = (int)(row * 16u + (in_row + 15u) % 16u);
    else if (ctrl == 0x138) { if (lane > 0u) from = (int)lane - 1; }
    else if (ctrl == 0x142) { if (row > 0u) from = (int)(row * 16u) - 1; }
    else if (ctrl == 0x143) { if (row > 1u) from = 31; }
    else abort();
    int result = old;
    if (from >= 0 && ((row_mask >> row) & 1)) result = (int)(uint32_t)ovl_emulated_lane_values[wave * 64u + (uint32_t)from];
    pthread_barrier_wait(&ovl_emulated_wave_barrier[wave]);
    return result;
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, row_mask, bank_mask, bound_ctrl) \
    ovl_emulated_update_dpp((old), (src), (ctrl), (row_mask))
#include "ovl_wave_scan.h"

// __shfl_up: lane i receives the value of lane i - delta of its wavefront; lanes below delta keep their own.
template <typename T>
static inline T __shfl_up(T value, unsigned delta, int width = 64) {
    static_assert(sizeof(T) <= 8, "shuffles carry at most 8 bytes");
    (void)width;
    const uint32_t t = threadIdx.x, wave = t / 64u, lane = t % 64u;
    uint64_t bits = 0;
    memcpy(&bits, &value, sizeof(T));
    ovl_emulated_lane_values[t] = bits;
    pthread_barrier_wait(&ovl_emulated_wave_barrier[wave]);
    T result = value;
    if (lane >= delta) memcpy(&result, &ovl_emulated_lane_values[t - delta], sizeof(T));
    pthread_barrier_wait(&ovl_emulated_wave_barrier[wave]);
    return result;
}

#define ovl_expf(x) ovl_math::expf_<true>((x), ovl_exp_tab)
#define ovl_logf(x) ovl_math::logf_((x), ovl_log_tab)
#define ovl_tanhf(x) ovl_math::tanhf_(x)
#define ovl_recipf(x) (1.0f / (x))
#define ovl_expf_inrange(x) ovl_math::expf_<false>((x), ovl_exp_tab)
#define ovl_logf_inrange(x) ovl_math::logf_inrange_<false>((x), ovl_log_tab)
#define ovl_logf_inrange_nan(x) ovl_math::logf_inrange_<true>((x), ovl_log_tab)
#define ovl_recipf_inrange(x) (1.0f / (x))
#define ovl_divf_inrange(a, b) ((a) / (b))
#define ovl_atan2f(a, b) atan2f((a), (b))

// The 'fast' math mode is built on device instructions; sources that also instantiate it (the hand-written LSTM
// cell) compile against the exact routines here, and the emulation tests never select it.
#define ovl_fast_expf(x) ovl_expf(x)
#define ovl_fast_tanhf(x) ovl_tanhf(x)
#define ovl_fast_divf(a, b) ((a) / (b))

#define OVL_DECLARE_MATH_TABLES()                                   \
    const uint64_t* const ovl_exp_tab = ovl_math::exp2f_tab;        \
    const ovl_math::logf_entry* const ovl_log_tab = ovl_math::logf_tab

#endif  // OVL_DEVICE_H_
