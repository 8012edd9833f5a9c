// Device-side support code included by every generated operator.
//
// Holds what the reference's generated CUDA text carries inline (integer abs helpers,
// opveclib/expression.py:598-600) plus the parameter struct of the launcher ABI and the scalar math entry points the
// body emitter calls.
#ifndef OVL_DEVICE_H_
#define OVL_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <float.h>

#include "ovl_math.h"
#include "ovl_fast_math.h"
#include "ovl_wave_scan.h"

// Same layout as ovl_tensor in include/ovl_launch.h.
typedef struct ovl_tensor {
    void*    data;
    int32_t  dtype;
    uint64_t len;
} ovl_tensor;

// MI355X: 256 compute units in 8 XCDs.
#define OVL_NUM_CU 256u

// status codes shared with the launcher
#define OVL_OK 0
#define OVL_EARGS 1
#define OVL_EHIP 4
#define OVL_EALIGN 5

__device__ __forceinline__ int8_t ovl_abs_8(int8_t x) { return (x < 0) ? -x : x; }
__device__ __forceinline__ int16_t ovl_abs_16(int16_t x) { return (x < 0) ? -x : x; }

// Vector accesses with and without the non-temporal (streaming) hint; the code generator picks per template.
#define OVL_LOAD_NT(ptr) __builtin_nontemporal_load(ptr)
#define OVL_LOAD_PLAIN(ptr) (*(ptr))
#define OVL_STORE_NT(value, ptr) __builtin_nontemporal_store(value, ptr)
#define OVL_STORE_PLAIN(value, ptr) (*(ptr) = (value))

// Lane-to-lane moves inside a wavefront (data-parallel-primitive modifiers of the vector ALU).
//   OVL_DPP_ROW_SHR1: lane i of every 16-lane row receives the value of lane i-1; lane 0 of the row keeps `old`
//   OVL_DPP_ROW_ROR1: lane i receives lane i-1, lane 0 of the row receives lane 15
#define OVL_DPP_ROW_SHR1 0x111
#define OVL_DPP_ROW_ROR1 0x121
template <int CTRL, typename T>
__device__ __forceinline__ T ovl_dpp_move(T old, T src) {
    if constexpr (sizeof(T) == 8) {
        const uint64_t o = __builtin_bit_cast(uint64_t, old), s = __builtin_bit_cast(uint64_t, src);
        const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp((int)(uint32_t)o, (int)(uint32_t)s, CTRL, 0xf, 0xf, false);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp((int)(uint32_t)(o >> 32), (int)(uint32_t)(s >> 32),
                                                                  CTRL, 0xf, 0xf, false);
        return __builtin_bit_cast(T, ((uint64_t)hi << 32) | lo);
    } else if constexpr (sizeof(T) == 4) {
        return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old),
                                                                 __builtin_bit_cast(int, src), CTRL, 0xf, 0xf, false));
    } else {
        return (T)__builtin_amdgcn_update_dpp((int)old, (int)src, CTRL, 0xf, 0xf, false);
    }
}

// float32 transcendental entry points used by generated code: bit-compatible with the host C library's
// expf/logf/tanhf (see ovl_math.h).  ovl_exp_tab / ovl_log_tab name the lookup tables in scope: kernels that call
// exp or log declare them with OVL_DECLARE_MATH_TABLES at their top, pointing at copies in LDS, together with
// ovl_f64, the routines' float64 constants held in scalar registers.
#define ovl_expf(x) ovl_math::expf_<true>((x), ovl_exp_tab, ovl_f64)
#define ovl_logf(x) ovl_math::logf_((x), ovl_log_tab, ovl_f64)
#define ovl_tanhf(x) ovl_math::tanhf_(x)
#define ovl_recipf(x) ovl_math::recipf_<true>(x)
// Variants for arguments that the code generator has proved to lie where the routine's common path is valid
// (hipgen/ranges.py): no rare-argument block.
#define ovl_expf_inrange(x) ovl_math::expf_<false>((x), ovl_exp_tab, ovl_f64)
#define ovl_logf_inrange(x) ovl_math::logf_inrange_<false>((x), ovl_log_tab, ovl_f64)
#define ovl_logf_inrange_nan(x) ovl_math::logf_inrange_<true>((x), ovl_log_tab, ovl_f64)
#define ovl_recipf_inrange(x) ovl_math::recipf_<false>(x)
#define ovl_divf_inrange(a, b) ovl_math::divf_inrange_((a), (b))

// atan2 in float32 through the device library's double precision routine, rounded once.  The device library's own
// float routine is up to three units in the last place away from the host C library's atan2f (measured on a million
// operand pairs); the rounded double precision value is the correctly rounded result except in the rarest cases and
// therefore within one unit of any faithful atan2f.
__device__ __forceinline__ float ovl_atan2f(float a, float b) { return (float)atan2((double)a, (double)b); }

// Once-rounded log(1 + x) and exp(x) - 1 on their checked domains, which the 'ulp2' math mode puts in place of the
// reference's formulas for them (hipgen/accuracy.py).
#define ovl_log1p_direct(x) ovl_math::log1p_direct_<false>((x), ovl_log_tab, ovl_f64)
#define ovl_log1p_direct_nan(x) ovl_math::log1p_direct_<true>((x), ovl_log_tab, ovl_f64)
#define ovl_expm1_direct(x) ovl_math::expm1_direct_((x), ovl_exp_tab, ovl_f64)
// The same for arguments whose value range is known to be narrow: 2^-4 <= x < 1 resp. 2^-12 <= x <= 0.68.
#define ovl_log1p_unit(x) ovl_math::log1p_unit_((x), ovl_log_unit_tab, ovl_f64)
#define ovl_expm1_small(x) ovl_math::expm1_small_((x), ovl_exp_plain_tab, ovl_f64)

// The logistic function 1 / (1 + exp(-x)) for -16 <= x <= 64 (NaN propagates): hardware-based exp, the sum and the
// correctly rounded reciprocal.  On that domain it is within two units in the last place of the same formula evaluated
// with the host C library's expf (below -16 the exponential passes 2^24, where adding 1 rounds, and the distance can
// reach 4); compared over every float32 argument of the domain by tests/test_gpu_math_exhaustive.py.
#define ovl_sigmoid_ulp2(x) ovl_math::recipf_<false>(1.0f + ovl_fast::expf_<false>(-(x)))
// The same for -1 <= x <= 64: there exp(-x) <= e, and the rounding of the product x * log2(e) (which the routine above
// carries along in a second term) moves the result by less than the bound leaves room for: four instructions fewer.
// Also compared with the formula on every float32 argument of its domain.
#define ovl_sigmoid_small(x) ovl_math::recipf_<false>(1.0f + __builtin_amdgcn_exp2f((x) * -0x1.715476p+0f))

// Entry points of the optional 'fast' math mode (ovl_fast_math.h).
#define ovl_fast_expf(x) ovl_fast::expf_<true>(x)
#define ovl_fast_logf(x) ovl_fast::logf_<true>(x)
#define ovl_fast_tanhf(x) ovl_fast::tanhf_(x)
#define ovl_fast_divf(a, b) ovl_fast::divf_<true>((a), (b))
#define ovl_fast_expf_inrange(x) ovl_fast::expf_<false>(x)
#define ovl_fast_logf_inrange(x) ovl_fast::logf_<false>(x)
#define ovl_fast_divf_inrange(a, b) ovl_fast::divf_<false>((a), (b))

#define OVL_DECLARE_MATH_TABLES()                                              \
    __shared__ ovl_math::lds_tables ovl_lds_tables;                            \
    ovl_math::load_tables(ovl_lds_tables);                                     \
    const uint64_t* const ovl_exp_tab = ovl_lds_tables.exp2f;                  \
    const ovl_math::logf_entry* const ovl_log_tab = ovl_lds_tables.logf;       \
    const uint64_t* const ovl_exp_plain_tab = ovl_lds_tables.exp2_plain;       \
    const ovl_math::logf_entry* const ovl_log_unit_tab = ovl_lds_tables.log_unit; \
    const ovl_math::f64_constants ovl_f64 = ovl_math::pinned_constants()

#endif  // OVL_DEVICE_H_
