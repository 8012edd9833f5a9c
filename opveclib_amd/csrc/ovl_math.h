// float32 transcendental functions for generated operators: exp, log, expm1, tanh.
//
// Generated operators must reproduce, on the GPU, what the reference's generated C++ computes with the host C
// library (opveclib/expression.py:1430-1456 maps EXP/LOG/TANH on float32 to expf/logf/tanhf).  Differences of one
// unit in the last place between two correct math libraries are amplified without bound by later cancellation
// (x - y with x close to y), so these routines follow the algorithms of the C library that the reference path runs
// on (GNU libc 2.35, x86-64, processors with FMA):
//
//   expf, logf   table driven, evaluated in double precision (Arm Optimized Routines' single precision exp/log:
//                exp(x) = 2^(k/32) * P3(r) with a 32 entry table of 2^(i/32); log(x) = log(c_i) + k*ln2 + P3(z/c_i - 1)
//                with a 16 entry table of (1/c_i, log c_i)).  The x86-64 build of the library selects a variant
//                compiled with fused multiply-add; the places where a multiply feeds an add are therefore fused
//                here too (fma), everywhere else products are rounded separately.
//   expm1f       FreeBSD msun / fdlibm single precision expm1: argument reduction by k*ln2 (two part ln2), a
//                degree 5 rational correction in float arithmetic, scaling by 2^k through the exponent field.
//   tanhf        fdlibm single precision tanh on top of expm1f: -t/(t+2) with t = expm1f(-2|x|) for |x| < 1,
//                1 - 2/(t+2) with t = expm1f(2|x|) for 1 <= |x| < 22, +-1 beyond.
//
// The file compiles as plain C++ for the host as well (no HIP headers needed), which is how the routines are checked
// against the host C library over all 2^32 float arguments.  All arithmetic must be compiled without contraction
// (-ffp-contract=off); fused operations are spelled out with __builtin_fma.
//
// Third-party notices.  The algorithms, lookup tables and polynomial coefficients of expf_ / logf_ (and of the
// once-rounded expm1 / log1p built on them) come from Arm Optimized Routines (math/expf.c, math/logf.c,
// math/exp2f_data.c, math/logf_data.c), which the GNU C library adopted:
//
//   Copyright (c) 2017-2018, Arm Limited.
//   SPDX-License-Identifier: MIT
//
//   Permission is hereby granted, free of charge, to any person obtaining a copy of this software and associated
//   documentation files (the "Software"), to deal in the Software without restriction, including without limitation
//   the rights to use, copy, modify, merge, publish, distribute, sublicense, and/or sell copies of the Software, and
//   to permit persons to whom the Software is furnished to do so, subject to the following conditions:
//
//   The above copyright notice and this permission notice shall be included in all copies or substantial portions of
//   the Software.
//
//   THE SOFTWARE IS PROVIDED "AS IS", WITHOUT WARRANTY OF ANY KIND, EXPRESS OR IMPLIED, INCLUDING BUT NOT LIMITED TO
//   THE WARRANTIES OF MERCHANTABILITY, FITNESS FOR A PARTICULAR PURPOSE AND NONINFRINGEMENT.  IN NO EVENT SHALL THE
//   AUTHORS OR COPYRIGHT HOLDERS BE LIABLE FOR ANY CLAIM, DAMAGES OR OTHER LIABILITY, WHETHER IN AN ACTION OF
//   CONTRACT, TORT OR OTHERWISE, ARISING FROM, OUT OF OR IN CONNECTION WITH THE SOFTWARE OR THE USE OR OTHER DEALINGS
//   IN THE SOFTWARE.
//
// expm1f_ and the tanh routines follow fdlibm's s_expm1f.c and s_tanhf.c (constants and evaluation order):
//
//   ====================================================
//   Copyright (C) 1993 by Sun Microsystems, Inc. All rights reserved.
//
//   Developed at SunPro, a Sun Microsystems, Inc. business.
//   Permission to use, copy, modify, and distribute this
//   software is freely granted, provided that this notice
//   is preserved.
//   ====================================================
#ifndef OVL_MATH_H_
#define OVL_MATH_H_

#include <stdint.h>

#if defined(__HIPCC__)
#define OVL_HD __device__ __forceinline__
#define OVL_TABLE static __device__ const
// True when the condition holds in any lane of the wavefront: a wave-uniform value, so `if (OVL_ANY(c))` is a scalar
// branch around a block that every lane executes or skips together.  The functions below compute their common path
// unconditionally and repair rare arguments (NaN, infinities, overflow, subnormals) inside such blocks with per-lane
// selects: no execution-mask juggling on the common path, and identical calls in one kernel can be merged by the
// compiler because the common path is not nested in a condition.
#define OVL_ANY(cond) (__builtin_amdgcn_ballot_w64(cond) != 0)
// True when the condition holds in every active lane of the wavefront (also wave-uniform).
#define OVL_ALL(cond) (__builtin_amdgcn_ballot_w64(!(cond)) == 0)
// OVL_RARE() as first statement of such a block keeps the compiler from turning the block into unconditional code
// with selects, which it does when it judges the block cheap.  That is welcome for the few selects of the routines in
// this file (measured: faster without the marker) and unwelcome for blocks that call a library routine
// (ovl_fast_math.h).
#define OVL_RARE() asm volatile("; rare arguments")
#else
#define OVL_HD static inline
#define OVL_TABLE static const
#define OVL_ANY(cond) (cond)
#define OVL_ALL(cond) (cond)
#define OVL_RARE() ((void)0)
#endif

// Every multiply-add site can be switched between fused (bit set) and separately rounded (bit clear); the default
// mask is the combination that reproduces the host C library bit for bit.
#ifndef OVL_MATH_FMA_SITES
#define OVL_MATH_FMA_SITES 0xffffffffu
#endif
#define OVL_MADD(site, a, b, c) \
    (((OVL_MATH_FMA_SITES >> (site)) & 1u) ? __builtin_fma((a), (b), (c)) : ((a) * (b) + (c)))

namespace ovl_math {

OVL_HD uint32_t as_u32(float f) { return __builtin_bit_cast(uint32_t, f); }
OVL_HD float as_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
OVL_HD uint64_t as_u64(double f) { return __builtin_bit_cast(uint64_t, f); }
OVL_HD double as_f64(uint64_t u) { return __builtin_bit_cast(double, u); }

// The float64 constants of the table-driven routines below.  A float64 operand cannot be written into a vector
// instruction as a literal, so the compiler moves each half into a scalar register first, and in straight-line code
// it does that again at every use: a kernel with twelve inlined exponentials issued 116 scalar moves per wavefront
// for their five constants, a tenth of all its instructions.  Kernels therefore set the constants up once
// (pinned_constants: the values pass through an empty assembly statement, after which the compiler cannot recreate
// them and keeps them in scalar registers) and hand them to every call.
struct f64_constants {
    double InvLn2N, Shift, C0, C1, C2;      // expf: N / ln 2, 1.5 * 2^52, the polynomial of 2^(r/N)
    double Ln2, A0, A1, A2;                 // logf: ln 2, the polynomial of log1p(r)
};
#define OVL_F64_CONSTANTS {                                                                      \
    0x1.71547652b82fep+0 * OVL_EXP2F_N, 0x1.8p+52,                                                 \
    0x1.c6af84b912394p-5 / OVL_EXP2F_N / OVL_EXP2F_N / OVL_EXP2F_N,                               \
    0x1.ebfce50fac4f3p-3 / OVL_EXP2F_N / OVL_EXP2F_N, 0x1.62e42ff0c52d6p-1 / OVL_EXP2F_N,          \
    0x1.62e42fefa39efp-1, -0x1.00ea348b88334p-2, 0x1.5575b0be00b6ap-2, -0x1.ffffef20a4123p-2 }

// ---------------------------------------------------------------------------------------------------------------------
// expf
// ---------------------------------------------------------------------------------------------------------------------
#define OVL_EXP2F_TABLE_BITS 5
#define OVL_EXP2F_N (1 << OVL_EXP2F_TABLE_BITS)

// tab[i] = bits(2^(i/32)) - (i << 47): adding k << 47 puts k/32's integer part into the exponent field
#define OVL_EXP2F_TABLE { \
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull, \
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull, \
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull, \
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull, \
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull, \
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull, \
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull, \
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull }

OVL_TABLE uint64_t exp2f_tab[OVL_EXP2F_N] = OVL_EXP2F_TABLE;

OVL_HD uint32_t top12(float x) { return as_u32(x) >> 20; }

// CHECKED = false leaves out the repair of |x| >= 88 and NaN: for callers that know -88 < x < 88 (NaN still gives
// NaN, through the polynomial in r).
template <bool CHECKED = true>
OVL_HD float expf_(float x, const uint64_t* tab = exp2f_tab, const f64_constants& f64 = f64_constants OVL_F64_CONSTANTS) {
    const double InvLn2N = f64.InvLn2N, Shift = f64.Shift, C0 = f64.C0, C1 = f64.C1, C2 = f64.C2;

    double xd = (double)x;
    uint32_t abstop = top12(x) & 0x7ff;
    // x*N/Ln2 = k + r with r in [-1/2, 1/2] and int k
    double kd = OVL_MADD(0, InvLn2N, xd, Shift);
    uint64_t ki = as_u64(kd);
    kd -= Shift;
    double r = OVL_MADD(1, InvLn2N, xd, -kd);
    // exp(x) = 2^(k/N) * 2^(r/N) ~= s * (C0*r^3 + C1*r^2 + C2*r + 1)
    uint64_t t = tab[ki % OVL_EXP2F_N];
    t += ki << (52 - OVL_EXP2F_TABLE_BITS);
    double s = as_f64(t);
    double z2 = OVL_MADD(2, C0, r, C1);
    double r2 = r * r;
    double y = OVL_MADD(3, C2, r, 1.0);
    y = OVL_MADD(4, z2, r2, y);
    y = y * s;
    float result = (float)y;
    const bool special = abstop >= top12(88.0f);        // |x| >= 88 or x is NaN
    if (CHECKED && OVL_ANY(special)) {
        float fixed = result;                                               // 88 <= |x| below the thresholds: as computed
        if (x < -0x1.9fe368p6f) fixed = 0.0f;                               // underflow, also -inf
        if (x > 0x1.62e42ep6f) fixed = __builtin_inff();                    // overflow, also +inf
        if (x != x) fixed = x + x;                                          // NaN
        result = special ? fixed : result;
    }
    return result;
}

// exp(x) - 1 for callers that know 2^-12 <= x <= 64, rounded once: the double precision value that expf_ forms before
// its final conversion, minus one in the same fused multiply-add that applies the scale (so it costs what expf_
// costs).  That value is within 2^-31 of exp(x) - 1, far below half a float32 unit in the last place for x >= 2^-12:
// the result is the correctly rounded expm1(x) except where exp(x) - 1 lies that close to a rounding boundary.  Used
// by the code generator's 'ulp2' math mode in place of the reference's expm1 formula
// (e - 1) * x / log(e), e = exp(x) (opveclib/examples/test_expm1.py:22-62), from which it is at most two units in the
// last place away on that domain (compared over every float32 argument of the domain).
OVL_HD float expm1_direct_(float x, const uint64_t* tab = exp2f_tab,
                           const f64_constants& f64 = f64_constants OVL_F64_CONSTANTS) {
    const double InvLn2N = f64.InvLn2N, Shift = f64.Shift, C0 = f64.C0, C1 = f64.C1, C2 = f64.C2;
    double xd = (double)x;
    double kd = __builtin_fma(InvLn2N, xd, Shift);
    uint64_t ki = as_u64(kd);
    kd -= Shift;
    double r = __builtin_fma(InvLn2N, xd, -kd);
    uint64_t t = tab[ki % OVL_EXP2F_N];
    t += ki << (52 - OVL_EXP2F_TABLE_BITS);
    double s = as_f64(t);
    double z2 = __builtin_fma(C0, r, C1);
    double r2 = r * r;
    double y = __builtin_fma(C2, r, 1.0);
    y = __builtin_fma(z2, r2, y);
    return (float)__builtin_fma(y, s, -1.0);
}

// exp(x) - 1 for 2^-12 <= x <= 0.68, where the scaled argument x * 32 / ln 2 rounds to 0 ... 31: the same arithmetic as
// expm1_direct_, but the table entry is 2^(i/32) itself and needs no exponent added.  On the device `plain` is that
// table (a copy in LDS, built from exp2f_tab when the tables are loaded); on the host the entry is computed here.
// NaN gives NaN; the index is masked, so an argument outside the domain reads inside the table (and gets a wrong
// value: the code generator uses the routine only where the value range of the argument lies in the domain).
OVL_HD float expm1_small_(float x, const uint64_t* plain = nullptr,
                          const f64_constants& f64 = f64_constants OVL_F64_CONSTANTS) {
    const double InvLn2N = f64.InvLn2N, Shift = f64.Shift, C0 = f64.C0, C1 = f64.C1, C2 = f64.C2;
    double xd = (double)x;
    double kd = __builtin_fma(InvLn2N, xd, Shift);
    const uint32_t i = (uint32_t)as_u64(kd) % OVL_EXP2F_N;
    kd -= Shift;
    double r = __builtin_fma(InvLn2N, xd, -kd);
#if defined(__HIP_DEVICE_COMPILE__)
    const uint64_t t = plain[i];
#else
    const uint64_t t = plain ? plain[i] : exp2f_tab[i] + ((uint64_t)i << (52 - OVL_EXP2F_TABLE_BITS));
#endif
    double s = as_f64(t);
    double z2 = __builtin_fma(C0, r, C1);
    double r2 = r * r;
    double y = __builtin_fma(C2, r, 1.0);
    y = __builtin_fma(z2, r2, y);
    return (float)__builtin_fma(y, s, -1.0);
}

// ---------------------------------------------------------------------------------------------------------------------
// logf
// ---------------------------------------------------------------------------------------------------------------------
#define OVL_LOGF_TABLE_BITS 4
#define OVL_LOGF_N (1 << OVL_LOGF_TABLE_BITS)

struct logf_entry { double invc, logc; };

#define OVL_LOGF_TABLE { \
    { 0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2 }, \
    { 0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2 }, \
    { 0x1.49539f0f010bp+0, -0x1.01eae7f513a67p-2 }, \
    { 0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3 }, \
    { 0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3 }, \
    { 0x1.25e227b0b8eap+0, -0x1.1aa2bc79c81p-3 }, \
    { 0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4 }, \
    { 0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4 }, \
    { 0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5 }, \
    { 0x1p+0, 0x0p+0 }, \
    { 0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5 }, \
    { 0x1.ca4b31f026aap-1, 0x1.c5e53aa362eb4p-4 }, \
    { 0x1.b2036576afce6p-1, 0x1.526e57720db08p-3 }, \
    { 0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3 }, \
    { 0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2 }, \
    { 0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2 } }

OVL_TABLE logf_entry logf_tab[OVL_LOGF_N] = OVL_LOGF_TABLE;

// For arguments in [1, 2): entry i belongs to [1 + i/16, 1 + (i+1)/16), c = 1 + (2 i + 1)/32 is its centre,
// { 1/c, log(c) } rounded to double.
#define OVL_LOG_UNIT_TABLE { \
    { 0x1.f07c1f07c1f08p-1, 0x1.f829b0e783300p-6 }, \
    { 0x1.d41d41d41d41dp-1, 0x1.6f0d28ae56b4cp-4 }, \
    { 0x1.bacf914c1bad0p-1, 0x1.29552f81ff523p-3 }, \
    { 0x1.a41a41a41a41ap-1, 0x1.9525a9cf456b4p-3 }, \
    { 0x1.8f9c18f9c18fap-1, 0x1.fb9186d5e3e2bp-3 }, \
    { 0x1.7d05f417d05f4p-1, 0x1.2e8e2bae11d31p-2 }, \
    { 0x1.6c16c16c16c17p-1, 0x1.5d1bdbf5809cap-2 }, \
    { 0x1.5c9882b931057p-1, 0x1.89a3386c1425bp-2 }, \
    { 0x1.4e5e0a72f0539p-1, 0x1.b44f77bcc8f63p-2 }, \
    { 0x1.4141414141414p-1, 0x1.dd46a04c1c4a1p-2 }, \
    { 0x1.3521cfb2b78c1p-1, 0x1.02552a5a5d0ffp-1 }, \
    { 0x1.29e4129e4129ep-1, 0x1.154c3d2f4d5eap-1 }, \
    { 0x1.1f7047dc11f70p-1, 0x1.2795e1289b11bp-1 }, \
    { 0x1.15b1e5f75270dp-1, 0x1.393e0d3562a1ap-1 }, \
    { 0x1.0c9714fbcda3bp-1, 0x1.4a4f85db03ebbp-1 }, \
    { 0x1.0410410410410p-1, 0x1.5ad404c359f2dp-1 } }

OVL_TABLE logf_entry log_unit_tab[OVL_LOGF_N] = OVL_LOG_UNIT_TABLE;

#if defined(__HIPCC__)
// Copies of the lookup tables in LDS.  Table lookups are per-lane gathers; served from LDS they cost a few cycles,
// while gathers from global memory occupy the vector memory pipeline that the kernel needs for streaming its tensors.
struct lds_tables {
    uint64_t exp2f[OVL_EXP2F_N];
    logf_entry logf[OVL_LOGF_N];
    uint64_t exp2_plain[OVL_EXP2F_N];       // bits of 2^(i/32): exp2f[i] with the exponent part of i/32 put back
    logf_entry log_unit[OVL_LOGF_N];
};

// The float64 constants in scalar registers for the rest of the kernel (see f64_constants).
__device__ __forceinline__ f64_constants pinned_constants() {
    f64_constants k = OVL_F64_CONSTANTS;
    // (an instruction reads at most one scalar operand: the second constant of Shift + InvLn2N * x, C1 + C0 * r and
    // A2 + A1 * r lives in vector registers)
    asm volatile("" : "+s"(k.InvLn2N), "+v"(k.Shift), "+s"(k.C0), "+v"(k.C1), "+s"(k.C2),
                      "+s"(k.Ln2), "+s"(k.A0), "+s"(k.A1), "+v"(k.A2));
    return k;
}

// Must be called by every thread of the workgroup before any divergent control flow.
__device__ __forceinline__ void load_tables(lds_tables& t) {
    if (threadIdx.x < OVL_EXP2F_N) {
        const uint64_t entry = exp2f_tab[threadIdx.x];
        t.exp2f[threadIdx.x] = entry;
        t.exp2_plain[threadIdx.x] = entry + ((uint64_t)threadIdx.x << (52 - OVL_EXP2F_TABLE_BITS));
    }
    if (threadIdx.x < OVL_LOGF_N) {
        t.logf[threadIdx.x] = logf_tab[threadIdx.x];
        t.log_unit[threadIdx.x] = log_unit_tab[threadIdx.x];
    }
    __syncthreads();
}
#endif

OVL_HD float logf_main_(uint32_t ix, const logf_entry* tab, const f64_constants& f64) {
    const double Ln2 = f64.Ln2, A0 = f64.A0, A1 = f64.A1, A2 = f64.A2;
    const uint32_t Off = 0x3f330000;
    // x = 2^k z; z in [Off, 2*Off) is exact; the range is split into N subintervals, c is near the centre of z's
    uint32_t tmp = ix - Off;
    int i = (tmp >> (23 - OVL_LOGF_TABLE_BITS)) % OVL_LOGF_N;
    int k = (int32_t)tmp >> 23;
    uint32_t iz = ix - (tmp & (0x1ffu << 23));
    double invc = tab[i].invc;
    double logc = tab[i].logc;
    double z = (double)as_f32(iz);
    // log(x) = log1p(z/c-1) + log(c) + k*Ln2
    double r = OVL_MADD(8, z, invc, -1.0);
    double y0 = OVL_MADD(9, (double)k, Ln2, logc);
    double r2 = r * r;
    double y = OVL_MADD(10, A1, r, A2);
    y = OVL_MADD(11, A0, r2, y);
    y = OVL_MADD(12, y, r2, y0 + r);
    return (float)y;
}

// logf_inrange_: for callers that know x is a positive normal number or, with MAYBE_NAN, possibly NaN.  The common
// path works on the bits of x and would turn NaN into a number; adding x * 0 (+0 for every number) puts the NaN back.
template <bool MAYBE_NAN>
OVL_HD float logf_inrange_(float x, const logf_entry* tab = logf_tab,
                           const f64_constants& f64 = f64_constants OVL_F64_CONSTANTS) {
    float result = logf_main_(as_u32(x), tab, f64);
    if (MAYBE_NAN) result = __builtin_fmaf(x, 0.0f, result);
    return result;
}

OVL_HD float logf_(float x, const logf_entry* tab = logf_tab, const f64_constants& f64 = f64_constants OVL_F64_CONSTANTS) {
    uint32_t ix = as_u32(x);
    // log(1) needs no special case in round-to-nearest: the table entry around 1 has invc = 1 and logc = 0, so the
    // common path returns +0 (the exhaustive comparison with the host library covers it)
    float result = logf_main_(ix, tab, f64);
    const bool special = ix - 0x00800000 >= 0x7f800000 - 0x00800000;    // x < 0x1p-126 or inf or nan
    if (OVL_ANY(special)) {
        // subnormal arguments are normalised and evaluated again
        uint32_t scaled = as_u32(x * 0x1p23f) - (23u << 23);
        float fixed = logf_main_(scaled, tab, f64);
        if ((ix & 0x80000000) || ix * 2 >= 0xff000000) fixed = __builtin_nanf("");
        if (ix == 0x7f800000) fixed = x;
        if (ix * 2 == 0) fixed = -__builtin_inff();
        result = special ? fixed : result;
    }
    return result;
}

// log(1 + x) for callers that know 2^-10 <= x <= 2^64, rounded once: u = 1 + x is exact in double precision, and the
// table and polynomial of logf_main_ are applied to the double u instead of a float (the table index and the exponent
// come from the same bits, which sit in the upper word of a double).  The polynomial is within 2^-31 of log(u), so the
// result is the correctly rounded log1p(x) except within that distance of a rounding boundary.  Used by the code
// generator's 'ulp2' math mode in place of the reference's log1p formula log(u) * x / (u - 1), u = 1 + x rounded to
// float (opveclib/examples/test_log1p.py:22-61), from which it is at most two units in the last place away on that
// domain (compared over every float32 argument of the domain).
// The common path works on the bits of u and would turn NaN into a number; with MAYBE_NAN, adding x * 0 (+-0 for every
// number) puts the NaN back.
template <bool MAYBE_NAN>
OVL_HD float log1p_direct_(float x, const logf_entry* tab = logf_tab,
                           const f64_constants& f64 = f64_constants OVL_F64_CONSTANTS) {
    const double Ln2 = f64.Ln2, A0 = f64.A0, A1 = f64.A1, A2 = f64.A2;
    const uint32_t Off = 0x3fe66000;            // upper word of 0.69921875, the lower end of the table's range
    const double u = 1.0 + (double)x;
    const uint64_t iu = as_u64(u);
    const uint32_t tmp = (uint32_t)(iu >> 32) - Off;
    const int i = (tmp >> (20 - OVL_LOGF_TABLE_BITS)) % OVL_LOGF_N;
    const int k = (int32_t)tmp >> 20;
    const double z = as_f64(iu - ((uint64_t)(tmp & 0xfff00000u) << 32));
    const double invc = tab[i].invc;
    const double logc = tab[i].logc;
    double r = __builtin_fma(z, invc, -1.0);
    double y0 = __builtin_fma((double)k, Ln2, logc);
    double r2 = r * r;
    double y = __builtin_fma(A1, r, A2);
    y = __builtin_fma(A0, r2, y);
    y = __builtin_fma(y, r2, y0 + r);
    float result = (float)y;
    if (MAYBE_NAN) result = __builtin_fmaf(x, 0.0f, result);
    return result;
}

// log(1 + x) for 2^-4 <= x < 1: u = 1 + x (exact in double precision) lies in [1, 2), so its exponent is known, the
// table is indexed by the top four fraction bits of u itself and neither the exponent's share k * ln 2 nor the
// re-centring of u is needed.  Same polynomial as logf_; |u / c - 1| <= 1/33.  NaN gives NaN (u is used as it is).
// The lower end of the domain keeps log(c) + log1p(u / c - 1) away from cancellation.
OVL_HD float log1p_unit_(float x, const logf_entry* tab = log_unit_tab,
                         const f64_constants& f64 = f64_constants OVL_F64_CONSTANTS) {
    const double A0 = f64.A0, A1 = f64.A1, A2 = f64.A2;
    const double u = 1.0 + (double)x;
    const uint32_t i = ((uint32_t)(as_u64(u) >> 32) >> (20 - OVL_LOGF_TABLE_BITS)) % OVL_LOGF_N;
    const double invc = tab[i].invc;
    const double logc = tab[i].logc;
    double r = __builtin_fma(u, invc, -1.0);
    double r2 = r * r;
    double y = __builtin_fma(A1, r, A2);
    y = __builtin_fma(A0, r2, y);
    y = __builtin_fma(y, r2, logc + r);
    return (float)y;
}

// ---------------------------------------------------------------------------------------------------------------------
// expm1f and tanhf (float arithmetic throughout)
// ---------------------------------------------------------------------------------------------------------------------
OVL_HD float expm1f_(float x) {
    const float one = 1.0f, huge = 1.0e+30f, tiny = 1.0e-30f;
    const float o_threshold = 8.8721679688e+01f;    // 0x42b17180
    const float ln2_hi = 6.9313812256e-01f;         // 0x3f317180
    const float ln2_lo = 9.0580006145e-06f;         // 0x3717f7d1
    const float invln2 = 1.4426950216e+00f;         // 0x3fb8aa3b
    const float Q1 = -3.3333335072e-02f;            // 0xbd088889
    const float Q2 = 1.5873016091e-03f;             // 0x3ad00d01
    const float Q3 = -7.9365076090e-05f;            // 0xb8a670cd
    const float Q4 = 4.0082177293e-06f;             // 0x36867e54
    const float Q5 = -2.0109921195e-07f;            // 0xb457edbb

    float y, hi, lo, c = 0.0f, t, e, hxs, hfx, r1;
    int32_t k;
    uint32_t hx = as_u32(x);
    uint32_t xsb = hx & 0x80000000u;    // sign bit of x
    hx &= 0x7fffffffu;                  // bits of |x|

    // filter out huge and non-finite argument
    if (hx >= 0x4195b844u) {            // |x| >= 27*ln2
        if (hx >= 0x42b17218u) {        // |x| >= 88.721...
            if (hx > 0x7f800000u) return x + x;                         // NaN
            if (hx == 0x7f800000u) return (xsb == 0) ? x : -1.0f;       // exp(+-inf) - 1 = {inf, -1}
            if (x > o_threshold) return huge * huge;                    // overflow
        }
        if (xsb != 0) return tiny - one;                                // x < -27*ln2: -1 (inexact)
    }

    // argument reduction
    if (hx > 0x3eb17218u) {             // |x| > 0.5 ln2
        if (hx < 0x3F851592u) {         // and |x| < 1.5 ln2
            if (xsb == 0) { hi = x - ln2_hi; lo = ln2_lo; k = 1; }
            else { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = (int32_t)(invln2 * x + ((xsb == 0) ? 0.5f : -0.5f));
            t = (float)k;
            hi = x - t * ln2_hi;        // t*ln2_hi is exact here
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x33000000u) {      // |x| < 2**-25: return x
        t = huge + x;
        return x - (t - (huge + x));
    } else {
        k = 0;
    }

    // x is now in primary range
    hfx = 0.5f * x;
    hxs = x * hfx;
    r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    t = 3.0f - r1 * hfx;
    e = hxs * ((r1 - t) / (6.0f - x * t));
    if (k == 0) return x - (x * e - hxs);       // c is 0
    e = (x * (e - c) - c);
    e -= hxs;
    if (k == -1) return 0.5f * (x - e) - 0.5f;
    if (k == 1) {
        if (x < -0.25f) return -2.0f * (e - (x + 0.5f));
        return one + 2.0f * (x - e);
    }
    if (k <= -2 || k > 56) {            // suffice to return exp(x)-1
        y = one - (e - x);
        y = as_f32(as_u32(y) + ((uint32_t)k << 23));    // add k to y's exponent
        return y - one;
    }
    if (k < 23) {
        t = as_f32(0x3f800000u - (0x1000000u >> k));    // t = 1 - 2^-k
        y = t - (e - x);
        y = as_f32(as_u32(y) + ((uint32_t)k << 23));
    } else {
        t = as_f32((uint32_t)(0x7f - k) << 23);          // 2^-k
        y = x - (e + t);
        y += one;
        y = as_f32(as_u32(y) + ((uint32_t)k << 23));
    }
    return y;
}

// tanh in terms of expm1, arranged as straight-line code.  For 2^-55 <= |x| < 22 fdlibm evaluates
//     |x| >= 1:  1 - 2/(t+2)  with t = expm1( 2|x|),     |x| < 1:  -t/(t+2)  with t = expm1(-2|x|),
// so expm1 only ever sees arguments in (-2, -2^-54] or [2, 44).  On that domain its overflow/infinity filter does
// nothing, its |a| < 2^-25 shortcut returns what the k = 0 path returns, and k = 1 cannot occur; what remains is one
// argument reduction, one polynomial and five short result formulas.  All of them are evaluated and the lane's own
// one is selected, which costs less on a wavefront than branching five ways; every selected value is produced by
// exactly the operations fdlibm performs for that case, so results are unchanged (checked against the host C
// library over all 2^32 arguments).
// The two quotients inside tanh.  On the device the IEEE division (scaling, reciprocal, three refinements, fix-up:
// about 14 issue slots) is replaced by reciprocal, product and one residual correction (7 slots).  That shortcut is
// not correctly rounded for arbitrary operands, but for the operands tanh produces it returns the same bits: the
// results of tanhf_ with it and with IEEE division were compared on MI355X over all 2^32 arguments, zero differences
// (the generated test library tests/native/exhaustive_math.hip repeats that comparison).
#if defined(__HIPCC__) && !defined(OVL_TANH_DIV)
OVL_HD float tanh_div_(float a, float b) {
    const float r = __builtin_amdgcn_rcpf(b);
    const float q = a * r;
    return __builtin_fmaf(__builtin_fmaf(-b, q, a), r, q);
}
#define OVL_TANH_DIV(a, b) tanh_div_((a), (b))
#endif
#ifndef OVL_TANH_DIV
#define OVL_TANH_DIV(a, b) ((a) / (b))
#endif
OVL_HD float tanhf_general_(float x) {
    const float one = 1.0f, two = 2.0f, tiny = 1.0e-30f;
    const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f;
    const float Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f;
    const float Q4 = 4.0082177293e-06f, Q5 = -2.0109921195e-07f;

    uint32_t jx = as_u32(x);
    uint32_t ix = jx & 0x7fffffffu;
    bool negative = (jx & 0x80000000u) != 0;


    float ax = as_f32(ix);
    bool big = ix >= 0x3f800000u;                   // |x| >= 1
    float a = big ? two * ax : -two * ax;           // argument of expm1
    uint32_t ha = as_u32(two * ax);                 // bits of |a|

    // argument reduction a = k*ln2 + xr (+ correction c); k = 0 leaves a untouched
    int32_t kg = (int32_t)(invln2 * a + (big ? 0.5f : -0.5f));
#if defined(OVL_TANH_FDLIBM_K)
    int32_t k = (ha > 0x3eb17218u) ? ((ha < 0x3F851592u) ? -1 : kg) : 0;
#else
    // fdlibm sets k = 0 for |a| <= 0.5 ln2 and k = -+1 for |a| < 1.5 ln2 without computing it; the rounded quotient
    // gives the same k for every argument tanh passes on (checked over all 2^32 arguments against the host library)
    int32_t k = kg;
#endif
    float t = (float)k;
    float hi = a - t * ln2_hi;
    float lo = t * ln2_lo;
    float xr = hi - lo;
    float c = (hi - xr) - lo;

    float hfx = 0.5f * xr;
    float hxs = xr * hfx;
    float r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    float t3 = 3.0f - r1 * hfx;
    float e = hxs * OVL_TANH_DIV(r1 - t3, 6.0f - xr * t3);

    float e2 = xr * (e - c) - c;
    e2 -= hxs;
    float d = e2 - xr;
    // k == 0: fdlibm returns xr - (xr*e - hxs); c is zero then, so e2 is that same xr*e - hxs and the result is -d
    float res0 = -d;
    float resm1 = 0.5f * (-d) - 0.5f;               // k == -1: 0.5*(xr-e2) - 0.5
    // k <= -2 or k > 56: (1 - d) * 2^k - 1;  3 <= k < 23: ((1 - 2^-k) - d) * 2^k;  23 <= k <= 56: ((xr-(e2+2^-k))+1) * 2^k
    bool tail_a = (k <= -2) || (k > 56);
    bool tail_b = (k >= 0) && (k < 23);
    uint32_t ks = (uint32_t)k & 31u;
    float base = tail_b ? as_f32(0x3f800000u - (0x1000000u >> ks)) : one;
    float y = base - d;
    float yc = (xr - (e2 + as_f32((uint32_t)(0x7f - k) << 23))) + one;
    y = (tail_a || tail_b) ? y : yc;
    y = as_f32(as_u32(y) + ((uint32_t)k << 23));    // add k to y's exponent
    float resk = tail_a ? y - one : y;
    float em1 = (k == 0) ? res0 : ((k == -1) ? resm1 : resk);

    float q = OVL_TANH_DIV(big ? two : -em1, em1 + two);
    float z = big ? one - q : q;
    float result = as_f32(as_u32(z) | (jx & 0x80000000u));      // z >= +0: give it the sign of x
    const bool special = ix >= 0x41b00000u || ix < 0x24000000u;     // |x| >= 22 (or inf, NaN), |x| < 2**-55 (or zero)
    if (OVL_ANY(special)) {
        float fixed = x * (one + x);                                                // tiny
        if (ix == 0) fixed = x;
        if (ix >= 0x41b00000u) fixed = negative ? -(one - tiny) : (one - tiny);
        if (ix >= 0x7f800000u) fixed = negative ? one / x - one : one / x + one;    // +-1 for infinities, NaN for NaN
        result = special ? fixed : result;
    }
    return result;
}

// tanhf_: the routine generated code calls.  For |x| < 7.5 the quotient k of the argument reduction can only
// be 0, -1, -2 or -3 (|x| < 1) or 3 .. 22 (|x| >= 1), so of fdlibm's result formulas only four remain and the one for
// |x| >= 1 is chosen by the comparison that is needed anyway; every other argument (NaN, infinities, large
// magnitudes) goes to tanhf_general_ inside a block that is entered only if some lane of the wavefront needs it.
// Same operations on the same operands as tanhf_general_ for the arguments it keeps, hence the same bits (compared
// with the host library over all 2^32 arguments, on the host and on the GPU).
OVL_HD float tanhf_(float x) {
    const float one = 1.0f, two = 2.0f;
    const float ln2_hi = 6.9313812256e-01f, ln2_lo = 9.0580006145e-06f, invln2 = 1.4426950216e+00f;
    const float Q1 = -3.3333335072e-02f, Q2 = 1.5873016091e-03f, Q3 = -7.9365076090e-05f;
    const float Q4 = 4.0082177293e-06f, Q5 = -2.0109921195e-07f;

    uint32_t jx = as_u32(x);
    uint32_t ix = jx & 0x7fffffffu;
    float ax = as_f32(ix);
    bool big = ix >= 0x3f800000u;                   // |x| >= 1
    float a = big ? two * ax : -two * ax;           // argument of expm1
    int32_t k = (int32_t)(invln2 * a + (big ? 0.5f : -0.5f));
    float t = (float)k;
    float hi = a - t * ln2_hi;
    float lo = t * ln2_lo;
    float xr = hi - lo;
    float c = (hi - xr) - lo;

    float hfx = 0.5f * xr;
    float hxs = xr * hfx;
    float r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    float t3 = 3.0f - r1 * hfx;
    float e = hxs * OVL_TANH_DIV(r1 - t3, 6.0f - xr * t3);

    float e2 = xr * (e - c) - c;
    e2 -= hxs;
    float d = e2 - xr;
    float res0 = -d;                                // k == 0
    float resm1 = 0.5f * (-d) - 0.5f;               // k == -1
    // k <= -2: (1 - d) * 2^k - 1;  3 <= k < 23: ((1 - 2^-k) - d) * 2^k
    uint32_t ks = (uint32_t)k & 31u;
    float base = big ? as_f32(0x3f800000u - (0x1000000u >> ks)) : one;
    float y = base - d;
    y = as_f32(as_u32(y) + ((uint32_t)k << 23));    // add k to y's exponent
    float small_em1 = (k == 0) ? res0 : ((k == -1) ? resm1 : y - one);
    float em1 = big ? y : small_em1;

    float q = OVL_TANH_DIV(big ? two : -em1, em1 + two);
    float z = big ? one - q : q;
    float result = as_f32(as_u32(z) | (jx & 0x80000000u));      // z >= +0: give it the sign of x
    // (zero and tiny arguments need no special case: with k == 0 the formulas above return x itself, as fdlibm's
    // x * (1 + x) does)
    const bool special = ix >= 0x40f00000u;         // |x| >= 7.5, infinities, NaN
    if (OVL_ANY(special)) {
        OVL_RARE();
        result = special ? tanhf_general_(x) : result;
    }
    return result;
}

#if defined(__HIPCC__)
// 1.0f / b.  Hardware reciprocal plus one Newton refinement is the correctly rounded reciprocal for every divisor
// with 2^-126 <= |b| < 2^126 (compared with IEEE division on MI355X over all 2^32 divisors: the only differences are
// subnormal divisors and divisors of 2^126 and above, whose reciprocals are subnormal); those, zeros, infinities and
// NaN take the IEEE division.
// CHECKED = false: for callers that know 2^-126 <= |b| < 2^126 (or NaN, which propagates).
template <bool CHECKED = true>
OVL_HD float recipf_(float b) {
    float r = __builtin_amdgcn_rcpf(b);
    r = __builtin_fmaf(__builtin_fmaf(-b, r, 1.0f), r, r);
    const float ab = __builtin_fabsf(b);
    const bool special = !(ab >= 0x1p-126f && ab < 0x1p126f);
    if (CHECKED && OVL_ANY(special)) r = special ? 1.0f / b : r;
    return r;
}

// a / b for operands whose quotient needs none of the IEEE division's operand scaling and no fix-up: both normal and
// nonzero, |b| <= 2^120, 2^-120 <= |a / b| <= 2^90 (NaN propagates).  These are the operations the device's division
// sequence performs between its scaling and fix-up instructions (reciprocal, two refinements of it, quotient, three
// residual corrections), which leave operands in that range untouched; the result is the correctly rounded quotient
// (tests/native/exhaustive_math.hip compares it with the '/' operator on 2^32 operand pairs).
OVL_HD float divf_inrange_(float a, float b) {
    float r = __builtin_amdgcn_rcpf(b);
    r = __builtin_fmaf(__builtin_fmaf(-b, r, 1.0f), r, r);
    float q = a * r;
    q = __builtin_fmaf(__builtin_fmaf(-b, q, a), r, q);
    return __builtin_fmaf(__builtin_fmaf(-b, q, a), r, q);
}
#endif

}  // namespace ovl_math

#endif  // OVL_MATH_H_
