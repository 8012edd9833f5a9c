// Test infrastructure: exhaustive checks of the device float32 math over all 2^32 argument bit patterns.
//
//   ovl_exh_against_host   device expf / logf / tanhf / reciprocal (opveclib_amd/csrc/ovl_math.h, as generated kernels
//                          call them) against the host C library's expf / logf / tanhf / (1.0f / x) on this machine
//                          (function 4 evaluates the device math library's own expf instead: a self-test of the
//                          checker, which must report differences for it)
//   ovl_exh_ulp_in_range   the once-rounded log1p / expm1 of the 'ulp2' math mode (and their shorter forms for narrow
//                          argument ranges) against the reference's formulas for them evaluated with the host C
//                          library, on every float of a range of bit patterns
//   ovl_exh_tanh_division  device tanhf with its shortened divisions against the same code with IEEE divisions
//   ovl_exh_in_range       the variants without a rare-argument block (expf, logf, reciprocal, division) against the
//                          full routines / the '/' operator, on every argument the code generator may hand them
//
// Built by tests/native/build.py into tests/native/libexhaustive_math.so; called through ctypes by
// tests/test_gpu_math_exhaustive.py.  Plain C ABI: returns 0 on success, a HIP error code otherwise.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <thread>
#include <vector>

#include "ovl_device.h"

// a second copy of tanhf_ with IEEE divisions, for the division check
namespace ovl_ieee {
using namespace ovl_math;
#undef OVL_TANH_DIV
#define OVL_TANH_DIV(a, b) ((a) / (b))
#define tanhf_ tanhf_ieee_
#include "tanh_body.inc"
#undef tanhf_
}  // namespace ovl_ieee

namespace {

enum { FN_EXP = 0, FN_LOG = 1, FN_TANH = 2, FN_RECIP = 3, FN_DEVICE_LIBRARY_EXP = 4,
       FN_FAST_EXP = 5, FN_FAST_LOG = 6, FN_FAST_TANH = 7, FN_FAST_RECIP = 8,
       FN_LOG1P_DIRECT = 9, FN_EXPM1_DIRECT = 10, FN_SIGMOID_ULP2 = 11, FN_LOG1P_UNIT = 12, FN_EXPM1_SMALL = 13,
       FN_SIGMOID_SMALL = 14 };

__global__ void __launch_bounds__(256) eval_kernel(int fn, uint32_t first, uint32_t count, float* __restrict__ out) {
    OVL_DECLARE_MATH_TABLES();
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
        const float x = __builtin_bit_cast(float, first + i);
        float y;
        if (fn == FN_EXP) y = ovl_expf(x);
        else if (fn == FN_LOG) y = ovl_logf(x);
        else if (fn == FN_TANH) y = ovl_tanhf(x);
        else if (fn == FN_RECIP) y = ovl_recipf(x);
        else if (fn == FN_FAST_EXP) y = ovl_fast_expf(x);
        else if (fn == FN_FAST_LOG) y = ovl_fast_logf(x);
        else if (fn == FN_FAST_TANH) y = ovl_fast_tanhf(x);
        else if (fn == FN_FAST_RECIP) y = ovl_fast_divf(1.0f, x);
        else if (fn == FN_LOG1P_DIRECT) y = ovl_log1p_direct_nan(x);
        else if (fn == FN_EXPM1_DIRECT) y = ovl_expm1_direct(x);
        else if (fn == FN_SIGMOID_ULP2) y = ovl_sigmoid_ulp2(x);
        else if (fn == FN_LOG1P_UNIT) y = ovl_log1p_unit(x);
        else if (fn == FN_EXPM1_SMALL) y = ovl_expm1_small(x);
        else if (fn == FN_SIGMOID_SMALL) y = ovl_sigmoid_small(x);
        else y = expf(x);            // the device math library's own expf: differs from the host's in the last place
        out[i] = y;
    }
}

__global__ void __launch_bounds__(256) tanh_division_kernel(unsigned long long* __restrict__ mismatches,
                                                            uint32_t* __restrict__ first_bad) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    unsigned long long bad = 0;
    for (uint64_t u = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; u < (1ull << 32); u += stride) {
        const float x = __builtin_bit_cast(float, (uint32_t)u);
        const float a = ovl_math::tanhf_(x), b = ovl_ieee::tanhf_ieee_(x);
        const bool same = __builtin_bit_cast(uint32_t, a) == __builtin_bit_cast(uint32_t, b) || (a != a && b != b);
        if (!same) {
            ++bad;
            atomicMin(first_bad, (uint32_t)u);
        }
    }
    if (bad) atomicAdd(mismatches, bad);
}

enum { IN_RANGE_EXP = 0, IN_RANGE_LOG = 1, IN_RANGE_RECIP = 2, IN_RANGE_DIV = 3 };

__device__ __forceinline__ uint64_t mix64(uint64_t z) {        // splitmix64 finaliser
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ bool same_bits(float a, float b) {
    return __builtin_bit_cast(uint32_t, a) == __builtin_bit_cast(uint32_t, b) || (a != a && b != b);
}

// which = exp / log / reciprocal: all 2^32 bit patterns, those outside the variant's domain skipped (NaN stays in).
// which = division: 2^32 operand pairs drawn from the variant's domain (|a| in [2^-100, 2^120], |b| in
// [2^-120, 2^120], |a / b| in [2^-120, 2^90]; every 16th pair has an all-ones or all-zeros significand).
__global__ void __launch_bounds__(256) in_range_kernel(int which, unsigned long long* __restrict__ mismatches,
                                                       unsigned long long* __restrict__ compared,
                                                       uint32_t* __restrict__ first_bad) {
    OVL_DECLARE_MATH_TABLES();
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    unsigned long long bad = 0, done = 0;
    for (uint64_t u = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; u < (1ull << 32); u += stride) {
        const uint32_t bits = (uint32_t)u;
        const float x = __builtin_bit_cast(float, bits);
        const float ax = __builtin_fabsf(x);
        bool same = true, use = false;
        if (which == IN_RANGE_EXP) {
            use = ax < 88.0f || x != x;
            if (use) same = same_bits(ovl_expf_inrange(x), ovl_expf(x));
        } else if (which == IN_RANGE_LOG) {
            const bool normal = x >= 0x1p-126f && x < __builtin_inff();
            use = normal || x != x;
            if (use) same = same_bits(ovl_logf_inrange_nan(x), ovl_logf(x));
            if (normal) same = same && same_bits(ovl_logf_inrange(x), ovl_logf(x));
        } else if (which == IN_RANGE_RECIP) {
            use = (ax >= 0x1p-125f && ax <= 0x1p125f) || x != x;
            if (use) same = same_bits(ovl_recipf_inrange(x), 1.0f / x);
        } else {
            const uint64_t h = mix64(u);
            const int ea = -100 + (int)((h >> 48) % 220u);                      // 2^ea <= |a| < 2^(ea+1)
            const int eb = -120 + (int)((h >> 56) % 240u + ((h >> 40) & 0xffu) % 240u) % 240;
            uint32_t ma = (uint32_t)h & 0x7fffffu, mb = (uint32_t)(h >> 23) & 0x7fffffu;
            if ((u & 15u) == 0) {
                ma = (h & (1ull << 46)) ? 0x7fffffu : 0u;
                mb = (h & (1ull << 47)) ? 0x7fffffu : 0u;
            }
            const uint32_t sa = (uint32_t)(h >> 62) & 1u, sb = (uint32_t)(h >> 63) & 1u;
            const float a = __builtin_bit_cast(float, (sa << 31) | ((uint32_t)(ea + 127) << 23) | ma);
            const float b = __builtin_bit_cast(float, (sb << 31) | ((uint32_t)(eb + 127) << 23) | mb);
            use = (ea - eb) <= 88 && (ea - eb) >= -119 && (ea < 120 || ma == 0u) && (eb < 120 || mb == 0u);
            if (use) same = same_bits(ovl_divf_inrange(a, b), a / b);
        }
        if (use) ++done;
        if (!same) {
            ++bad;
            atomicMin(first_bad, bits);
        }
    }
    if (bad) atomicAdd(mismatches, bad);
    atomicAdd(compared, done);
}

// The reference's log1p and expm1 operators (opveclib/examples/test_log1p.py:22-61, test_expm1.py:22-62) as the
// generated C++ evaluates them: every operation in float, exp and log from the host C library.
float host_log1p_formula(float x) {
    volatile float u = 1.0f + x;
    volatile float d = u - 1.0f;
    if (isinf(x) && x > 0.0f) return x;
    if (d == 0.0f) return x;
    volatile float l = logf(u);
    volatile float p = l * x;
    return p / d;
}

float host_expm1_formula(float x) {
    volatile float e = expf(x);
    if (isinf(x) && x > 0.0f) return x;
    if (e == 1.0f) return x;
    volatile float em = e - 1.0f;
    if (em == -1.0f) return -1.0f;
    volatile float p = em * x;
    volatile float l = logf(e);
    return p / l;
}

// The reference's sigmoid (opveclib/stdops/math.py:93): 1 / (1 + exp(-x)) in float.
float host_sigmoid_formula(float x) {
    volatile float e = expf(-x);
    volatile float s = 1.0f + e;
    volatile float one = 1.0f;
    return one / s;
}

float host_value(int fn, float x) {
    if (fn == FN_SIGMOID_ULP2 || fn == FN_SIGMOID_SMALL) return host_sigmoid_formula(x);
    if (fn == FN_LOG1P_DIRECT || fn == FN_LOG1P_UNIT) return host_log1p_formula(x);
    if (fn == FN_EXPM1_DIRECT || fn == FN_EXPM1_SMALL) return host_expm1_formula(x);
    if (fn == FN_EXP || fn == FN_DEVICE_LIBRARY_EXP || fn == FN_FAST_EXP) return expf(x);
    if (fn == FN_LOG || fn == FN_FAST_LOG) return logf(x);
    if (fn == FN_TANH || fn == FN_FAST_TANH) return tanhf(x);
    volatile float one = 1.0f;          // keep the division at run time
    return one / x;
}

}  // namespace

extern "C" int ovl_exh_tanh_division(uint64_t* mismatches, uint32_t* first_bad) {
    unsigned long long* d_count = nullptr;
    uint32_t* d_first = nullptr;
    hipError_t err = hipMalloc(&d_count, sizeof(unsigned long long));
    if (err != hipSuccess) return (int)err;
    err = hipMalloc(&d_first, sizeof(uint32_t));
    if (err != hipSuccess) return (int)err;
    unsigned long long zero = 0;
    uint32_t all = 0xffffffffu;
    hipMemcpy(d_count, &zero, sizeof(zero), hipMemcpyHostToDevice);
    hipMemcpy(d_first, &all, sizeof(all), hipMemcpyHostToDevice);
    hipLaunchKernelGGL(tanh_division_kernel, dim3(4096), dim3(256), 0, 0, d_count, d_first);
    err = hipDeviceSynchronize();
    unsigned long long h = 0;
    hipMemcpy(&h, d_count, sizeof(h), hipMemcpyDeviceToHost);
    hipMemcpy(first_bad, d_first, sizeof(uint32_t), hipMemcpyDeviceToHost);
    *mismatches = h;
    hipFree(d_count);
    hipFree(d_first);
    return (int)err;
}

extern "C" int ovl_exh_in_range(int which, uint64_t* mismatches, uint64_t* compared, uint32_t* first_bad) {
    unsigned long long* d_counts = nullptr;
    uint32_t* d_first = nullptr;
    hipError_t err = hipMalloc(&d_counts, 2 * sizeof(unsigned long long));
    if (err != hipSuccess) return (int)err;
    err = hipMalloc(&d_first, sizeof(uint32_t));
    if (err != hipSuccess) { hipFree(d_counts); return (int)err; }
    unsigned long long zero[2] = {0, 0};
    uint32_t all = 0xffffffffu;
    hipMemcpy(d_counts, zero, sizeof(zero), hipMemcpyHostToDevice);
    hipMemcpy(d_first, &all, sizeof(all), hipMemcpyHostToDevice);
    hipLaunchKernelGGL(in_range_kernel, dim3(4096), dim3(256), 0, 0, which, d_counts, d_counts + 1, d_first);
    err = hipDeviceSynchronize();
    unsigned long long h[2] = {0, 0};
    hipMemcpy(h, d_counts, sizeof(h), hipMemcpyDeviceToHost);
    hipMemcpy(first_bad, d_first, sizeof(uint32_t), hipMemcpyDeviceToHost);
    *mismatches = h[0];
    *compared = h[1];
    hipFree(d_counts);
    hipFree(d_first);
    return (int)err;
}

// Compare fn over the bit patterns first, first + step, ... (count of them) with the host C library.
// step = 1 and count = 2^32 is the exhaustive run.  threads = host threads used for the host side.
static int against_host(int fn, uint64_t count, uint32_t step, uint32_t threads, uint64_t* mismatches,
                        uint32_t* first_bad, uint64_t* beyond_two_ulp, uint32_t* max_ulp, uint32_t* worst_bits,
                        uint64_t first_pattern = 0, uint64_t end_pattern = 1ull << 32);

extern "C" int ovl_exh_against_host(int fn, uint64_t count, uint32_t step, uint32_t threads, uint64_t* mismatches,
                                    uint32_t* first_bad) {
    uint64_t beyond = 0;
    uint32_t max_ulp = 0, worst = 0;
    return against_host(fn, count, step, threads, mismatches, first_bad, &beyond, &max_ulp, &worst);
}

// The same comparison reporting distances in units in the last place: the number of arguments whose results lie more
// than two units apart, the largest distance and an argument where it occurs.
extern "C" int ovl_exh_ulp_against_host(int fn, uint64_t count, uint32_t step, uint32_t threads,
                                        uint64_t* mismatches, uint64_t* beyond_two_ulp, uint32_t* max_ulp,
                                        uint32_t* worst_bits) {
    uint32_t first = 0;
    return against_host(fn, count, step, threads, mismatches, &first, beyond_two_ulp, max_ulp, worst_bits);
}

static int64_t ordered(uint32_t bits) {       // float bit pattern -> integer that grows with the value
    return (bits & 0x80000000u) ? -(int64_t)(bits & 0x7fffffffu) : (int64_t)bits;
}

// Every float whose bit pattern lies in [first_bits, last_bits] (a range of one sign: consecutive patterns are
// consecutive floats): fn against its host counterpart, distances in units in the last place.
extern "C" int ovl_exh_ulp_in_range(int fn, uint32_t first_bits, uint32_t last_bits, uint32_t threads,
                                    uint64_t* compared, uint64_t* mismatches, uint64_t* beyond_two_ulp,
                                    uint32_t* max_ulp, uint32_t* worst_bits) {
    uint32_t first = 0;
    *compared = (uint64_t)last_bits - first_bits + 1;
    return against_host(fn, 1ull << 32, 1, threads, mismatches, &first, beyond_two_ulp, max_ulp, worst_bits,
                        first_bits, (uint64_t)last_bits + 1);
}

static int against_host(int fn, uint64_t count, uint32_t step, uint32_t threads, uint64_t* mismatches,
                        uint32_t* first_bad, uint64_t* beyond_two_ulp, uint32_t* max_ulp, uint32_t* worst_bits,
                        uint64_t first_pattern, uint64_t end_pattern) {
    const uint32_t chunk = 1u << 26;
    float* d_out = nullptr;
    float* h_out = nullptr;
    hipError_t err = hipMalloc(&d_out, (size_t)chunk * sizeof(float));
    if (err != hipSuccess) return (int)err;
    err = hipHostMalloc(&h_out, (size_t)chunk * sizeof(float), hipHostMallocDefault);
    if (err != hipSuccess) { hipFree(d_out); return (int)err; }
    uint64_t total_bad = 0, total_far = 0;
    uint32_t lowest = 0xffffffffu, largest = 0, largest_at = 0;
    if (threads == 0) threads = 1;
    // with step > 1 the device still evaluates whole chunks; the host then samples every step-th pattern
    for (uint64_t base = first_pattern & ~(uint64_t)(chunk - 1); base < end_pattern && base / step < count;
         base += chunk) {
        hipLaunchKernelGGL(eval_kernel, dim3(2048), dim3(256), 0, 0, fn, (uint32_t)base, chunk, d_out);
        err = hipMemcpy(h_out, d_out, (size_t)chunk * sizeof(float), hipMemcpyDeviceToHost);
        if (err != hipSuccess) break;
        std::vector<uint64_t> bad(threads, 0), far(threads, 0);
        std::vector<uint32_t> low(threads, 0xffffffffu), worst(threads, 0), worst_at(threads, 0);
        std::vector<std::thread> pool;
        for (uint32_t t = 0; t < threads; ++t) {
            pool.emplace_back([&, t]() {
                const uint32_t begin = (uint32_t)((uint64_t)chunk * t / threads);
                const uint32_t end = (uint32_t)((uint64_t)chunk * (t + 1) / threads);
                uint32_t i = begin + (step - (base + begin) % step) % step;
                for (; i < end; i += step) {
                    const uint32_t bits = (uint32_t)base + i;
                    if (bits < first_pattern || bits >= end_pattern) continue;
                    float x;
                    memcpy(&x, &bits, 4);
                    const float want = host_value(fn, x);
                    const float got = h_out[i];
                    uint32_t wb, gb;
                    memcpy(&wb, &want, 4);
                    memcpy(&gb, &got, 4);
                    if (wb != gb && !(want != want && got != got)) {
                        ++bad[t];
                        if (bits < low[t]) low[t] = bits;
                        int64_t d = ordered(wb) - ordered(gb);
                        if (d < 0) d = -d;
                        if (want != want || got != got || d > 0x7fffffff) d = 0x7fffffff;   // NaN against a number
                        if (d > 2) ++far[t];
                        if ((uint32_t)d > worst[t]) { worst[t] = (uint32_t)d; worst_at[t] = bits; }
                    }
                }
            });
        }
        for (auto& th : pool) th.join();
        for (uint32_t t = 0; t < threads; ++t) {
            total_bad += bad[t];
            total_far += far[t];
            if (low[t] < lowest) lowest = low[t];
            if (worst[t] > largest) { largest = worst[t]; largest_at = worst_at[t]; }
        }
    }
    hipFree(d_out);
    hipHostFree(h_out);
    *mismatches = total_bad;
    *first_bad = lowest;
    *beyond_two_ulp = total_far;
    *max_ulp = largest;
    *worst_bits = largest_at;
    return (int)err;
}
