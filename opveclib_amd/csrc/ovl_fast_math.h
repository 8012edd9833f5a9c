// Float32 routines of the optional 'fast' math mode (device only).
//
// Built on the hardware's exp2 / log2 / reciprocal instructions (each accurate to one unit in the last place), with
// the common path written without conditions and rare arguments (results in the subnormal range, overflow, zero or
// negative logarithm arguments, infinities) handed to the device math library inside a wave-uniform block.  Not
// bit-compatible with the host C library: tests/test_gpu_math_exhaustive.py measures the distance from the host's
// expf / logf / tanhf / division over all 2^32 arguments (at most 2 units in the last place for each routine).
#ifndef OVL_FAST_MATH_H_
#define OVL_FAST_MATH_H_

#include "ovl_math.h"

namespace ovl_fast {

// exp(x) = 2^(x * log2 e).  The product is formed to about 48 bits (p + e1); 2^p comes from the hardware and the
// factor 2^e1 ~ 1 + e1 ln 2 is applied with one fused multiply-add.
// (CHECKED = false in this file: the caller knows that no argument needs the rare-argument block; NaN propagates
// through the common path of every routine.)
template <bool CHECKED = true>
__device__ __forceinline__ float expf_(float x) {
    const float log2e = 0x1.715476p+0f, log2e_lo = 0x1.4ae0cp-26f, ln2 = 0x1.62e43p-1f;
    const float p = x * log2e;
    float e1 = __builtin_fmaf(x, log2e, -p);
    e1 = __builtin_fmaf(x, log2e_lo, e1);
    const float r = __builtin_amdgcn_exp2f(p);
    float result = __builtin_fmaf(r, e1 * ln2, r);
    // |x| >= 87: the result may be subnormal, zero or infinite (or x is NaN)
    const bool special = !(__builtin_fabsf(x) < 87.0f);
    if (CHECKED && OVL_ANY(special)) {
        OVL_RARE();
        result = special ? expf(x) : result;
    }
    return result;
}

// log(x) = log2(x) * ln 2 with the product carried to about 48 bits.
template <bool CHECKED = true>
__device__ __forceinline__ float logf_(float x) {
    const float ln2 = 0x1.62e430p-1f, ln2_lo = -0x1.05c610p-29f;
    const float l = __builtin_amdgcn_logf(x);
    const float r = l * ln2;
    float result = r + __builtin_fmaf(l, ln2_lo, __builtin_fmaf(l, ln2, -r));
    // subnormal, zero, negative, infinite or NaN arguments
    const bool special = !(x >= 0x1p-126f && x < __builtin_inff());
    if (CHECKED && OVL_ANY(special)) {
        OVL_RARE();
        result = special ? logf(x) : result;
    }
    return result;
}

// tanh(x): an odd polynomial below 0.6, 1 - 2 / (exp(2|x|) + 1) above.  Large arguments give exactly 1 through the
// clamped exponential, tiny ones give x through the polynomial, NaN propagates: no rare-argument block is needed.
__device__ __forceinline__ float tanhf_(float x) {
    const float ax = __builtin_fabsf(x);
    const float u = ax * ax;
    float p = -5.883233056e-03f;
    p = __builtin_fmaf(p, u, 2.078514762e-02f);
    p = __builtin_fmaf(p, u, -5.378039939e-02f);
    p = __builtin_fmaf(p, u, 1.333188030e-01f);
    p = __builtin_fmaf(p, u, -3.333329618e-01f);
    const float small = __builtin_fmaf(ax * u, p, ax);
    // exp(2|x|), with the rounding error of the product 2|x| log2(e) put back in (as in expf_)
    // (arguments above 10, where tanh rounds to 1, are clamped so that the exponential stays finite)
    const float c = 0x1.715476p+1f;
    // (one median-of-three instruction instead of a compare and a select; for NaN it gives a number, and the
    // selection below then takes the polynomial's NaN)
    const float ac = __builtin_amdgcn_fmed3f(ax, 0.0f, 10.0f);
    const float e2 = ac * c;
    float t = __builtin_amdgcn_exp2f(e2);
    t = __builtin_fmaf(t, __builtin_fmaf(ac, c, -e2) * 0x1.62e43p-1f, t);
    const float big = __builtin_fmaf(-2.0f, __builtin_amdgcn_rcpf(t + 1.0f), 1.0f);
    const float z = ax >= 0.6f ? big : small;
    return __builtin_copysignf(z, x);
}

// a / b: hardware reciprocal, product and one residual correction.
template <bool CHECKED = true>
__device__ __forceinline__ float divf_(float a, float b) {
    const float r = __builtin_amdgcn_rcpf(b);
    const float q = a * r;
    float result = __builtin_fmaf(__builtin_fmaf(-b, q, a), r, q);
    // divisors outside [2^-126, 2^126), quotients in or near the subnormal range, infinities and NaN
    const float ab = __builtin_fabsf(b), aq = __builtin_fabsf(q);
    // (a zero dividend needs nothing special: the quotient is a correctly signed zero)
    const bool special = !(ab >= 0x1p-126f && ab < 0x1p126f && ((aq >= 0x1p-100f && aq < __builtin_inff()) || a == 0.0f));
    if (CHECKED && OVL_ANY(special)) {
        OVL_RARE();
        result = special ? a / b : result;
    }
    return result;
}

}  // namespace ovl_fast

#endif  // OVL_FAST_MATH_H_
