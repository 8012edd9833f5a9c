// Hand-written LSTM cell and gradient kernels for gfx950 behind the C ABI of include/ovl_lstm.h.
//
// The arithmetic is the reference's fused LSTM operator (lstm/lstm.py:14-105) statement for statement: float32
// throughout, products and sums rounded separately (the file is compiled without contraction), sigmoid as
// 1 / (1 + exp(-x)), the sigmoid derivative e / ((1 + e) * (1 + e)) only for -50 < x < 50.  exp, tanh, the reciprocal
// and the division are the routines generated operators use (ovl_math.h: the host C library's bits; ovl_fast_math.h
// with fast_math), so the results equal those of the generated operator for the same shape bit for bit.
//
// Work layout: the cell is a map over [batch, units].  One thread owns VEC = 4 consecutive units of one batch row:
// four 128-bit loads fetch its slices of the gates i, j, f, o, which lie `units` floats apart in the row of `concat`,
// one more fetches c; results leave as 128-bit stores.  A wavefront therefore reads five and writes two (gradient:
// reads seven, writes five) 1 KiB runs.  Rows whose length is not a multiple of 4, or unaligned tensors, take the
// same kernel with VEC = 1.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string>

#include "ovl_device.h"
#include "ovl_index_div.h"
#include "ovl_lstm.h"

// ovl_device.h carries the status codes generated operators return; this one (ovl_status in ovl_launch.h) is the
// launcher's own
#define OVL_EINVAL 6

namespace {

thread_local std::string g_last_error;

int fail(int code, const std::string& detail) {
    g_last_error = detail;
    return code;
}

constexpr uint32_t BLOCK = 256;
constexpr uint32_t MAX_GRID = 1u << 20;     // the kernels stride over the rest

template <int VEC> struct vec_of;
template <> struct vec_of<1> { typedef float type; };
template <> struct vec_of<4> { typedef float type __attribute__((ext_vector_type(4))); };

template <int VEC>
__device__ __forceinline__ float lane_of(const typename vec_of<VEC>::type& v, int u) {
    if constexpr (VEC == 1) return v; else return v[u];
}

template <int VEC>
__device__ __forceinline__ void set_lane(typename vec_of<VEC>::type& v, int u, float x) {
    if constexpr (VEC == 1) v = x; else v[u] = x;
}

// The scalar functions of lstm/lstm.py:14-29.  The math tables (LDS copies) are those declared by the kernel.
#define LSTM_EXP(x) (FAST ? ovl_fast_expf(x) : ovl_expf(x))
#define LSTM_TANH(x) (FAST ? ovl_fast_tanhf(x) : ovl_tanhf(x))
#define LSTM_DIV(a, b) (FAST ? ovl_fast_divf((a), (b)) : ((a) / (b)))
#define LSTM_SIG_FROM_EXP(e) ovl_recipf(1.0f + (e))                 /* sig(x) = 1 / (1 + exp(-x)) */
#define LSTM_SIG_GRAD(x, e) sig_grad_<FAST>((x), (e))

// sig_grad(x) with e = exp(-x) (lstm/lstm.py:18-24): the quotient is formed for every lane and selected, as the
// generated operator does after turning the conditional into a select.
template <bool FAST>
__device__ __forceinline__ float sig_grad_(float x, float e) {
    const float q = LSTM_DIV(e, (1.0f + e) * (1.0f + e));
    return (x > -50.0f && x < 50.0f) ? q : 0.0f;
}

// Plain loads and non-temporal stores: measured fastest for these kernels' five to seven load streams
// (forward 26.5 us against 27.2 with the hint on the loads too, gradient 36.4 against 41.7).
template <typename V>
__device__ __forceinline__ V load_vec(const float* p) {
    return *reinterpret_cast<const V*>(p);
}

template <bool FAST, int VEC>
__global__ void __launch_bounds__(BLOCK)
lstm_forward_kernel(const float* __restrict__ concat, const float* __restrict__ c, float forget_bias,
                    uint32_t units, index_divisor vectors_per_row, uint32_t num_vectors,
                    float* __restrict__ new_c, float* __restrict__ new_h) {
    typedef typename vec_of<VEC>::type vec;
    OVL_DECLARE_MATH_TABLES();
    // v + stride may pass 2^32 (scalar variant on more than 2^32 - 2^28 elements): step only while it stays in range
    const uint32_t stride = gridDim.x * BLOCK;
    for (uint32_t v = blockIdx.x * BLOCK + threadIdx.x; v < num_vectors;
         v = (num_vectors - v > stride) ? v + stride : num_vectors) {
        const uint32_t row = divide(v, vectors_per_row);
        const uint32_t elem = (v - row * vectors_per_row.divisor) * VEC;
        const float* gates = concat + (uint64_t)row * 4u * units + elem;
        const uint64_t at = (uint64_t)row * units + elem;
        const vec vi = load_vec<vec>(gates);
        const vec vj = load_vec<vec>(gates + units);
        const vec vf = load_vec<vec>(gates + (uint64_t)2 * units);
        const vec vo = load_vec<vec>(gates + (uint64_t)3 * units);
        const vec vc = load_vec<vec>(c + at);
        vec out_c, out_h;
#pragma unroll
        for (int u = 0; u < VEC; ++u) {
            const float i = lane_of<VEC>(vi, u), j = lane_of<VEC>(vj, u), f = lane_of<VEC>(vf, u);
            const float o = lane_of<VEC>(vo, u), c_cur = lane_of<VEC>(vc, u);
            const float fb = f + forget_bias;
            const float sig_f = LSTM_SIG_FROM_EXP(LSTM_EXP(-fb));
            const float sig_i = LSTM_SIG_FROM_EXP(LSTM_EXP(-i));
            const float new_c_cur = c_cur * sig_f + sig_i * LSTM_TANH(j);
            const float sig_o = LSTM_SIG_FROM_EXP(LSTM_EXP(-o));
            set_lane<VEC>(out_c, u, new_c_cur);
            set_lane<VEC>(out_h, u, LSTM_TANH(new_c_cur) * sig_o);
        }
        __builtin_nontemporal_store(out_c, reinterpret_cast<vec*>(new_c + at));
        __builtin_nontemporal_store(out_h, reinterpret_cast<vec*>(new_h + at));
    }
}

template <bool FAST, int VEC>
__global__ void __launch_bounds__(BLOCK)
lstm_backward_kernel(const float* __restrict__ concat, const float* __restrict__ c,
                     const float* __restrict__ d_new_c, const float* __restrict__ d_new_h, float forget_bias,
                     uint32_t units, index_divisor vectors_per_row, uint32_t num_vectors,
                     float* __restrict__ d_concat, float* __restrict__ d_c) {
    typedef typename vec_of<VEC>::type vec;
    OVL_DECLARE_MATH_TABLES();
    // v + stride may pass 2^32 (scalar variant on more than 2^32 - 2^28 elements): step only while it stays in range
    const uint32_t stride = gridDim.x * BLOCK;
    for (uint32_t v = blockIdx.x * BLOCK + threadIdx.x; v < num_vectors;
         v = (num_vectors - v > stride) ? v + stride : num_vectors) {
        const uint32_t row = divide(v, vectors_per_row);
        const uint32_t elem = (v - row * vectors_per_row.divisor) * VEC;
        const uint64_t gate_at = (uint64_t)row * 4u * units + elem;
        const uint64_t at = (uint64_t)row * units + elem;
        const float* gates = concat + gate_at;
        const vec vi = load_vec<vec>(gates);
        const vec vj = load_vec<vec>(gates + units);
        const vec vf = load_vec<vec>(gates + (uint64_t)2 * units);
        const vec vo = load_vec<vec>(gates + (uint64_t)3 * units);
        const vec vc = load_vec<vec>(c + at);
        const vec vdc = load_vec<vec>(d_new_c + at);
        const vec vdh = load_vec<vec>(d_new_h + at);
        vec out_i, out_j, out_f, out_o, out_c;
#pragma unroll
        for (int u = 0; u < VEC; ++u) {
            const float i = lane_of<VEC>(vi, u), j = lane_of<VEC>(vj, u), f = lane_of<VEC>(vf, u);
            const float o = lane_of<VEC>(vo, u), c_cur = lane_of<VEC>(vc, u);
            const float d_new_c_cur = lane_of<VEC>(vdc, u), d_new_h_cur = lane_of<VEC>(vdh, u);
            const float fb = f + forget_bias;
            const float e_f = LSTM_EXP(-fb), e_i = LSTM_EXP(-i), e_o = LSTM_EXP(-o);
            const float sig_f = LSTM_SIG_FROM_EXP(e_f), sig_i = LSTM_SIG_FROM_EXP(e_i), sig_o = LSTM_SIG_FROM_EXP(e_o);
            const float tanh_j = LSTM_TANH(j);
            const float new_c_cur = c_cur * sig_f + sig_i * tanh_j;
            const float tanh_c = LSTM_TANH(new_c_cur);
            const float back_ch = d_new_c_cur + (1.0f - tanh_c * tanh_c) * sig_o * d_new_h_cur;
            set_lane<VEC>(out_i, u, tanh_j * LSTM_SIG_GRAD(i, e_i) * back_ch);
            set_lane<VEC>(out_j, u, sig_i * (1.0f - tanh_j * tanh_j) * back_ch);
            set_lane<VEC>(out_f, u, c_cur * LSTM_SIG_GRAD(fb, e_f) * back_ch);
            set_lane<VEC>(out_c, u, sig_f * back_ch);
            set_lane<VEC>(out_o, u, tanh_c * LSTM_SIG_GRAD(o, e_o) * d_new_h_cur);
        }
        float* grads = d_concat + gate_at;
        __builtin_nontemporal_store(out_i, reinterpret_cast<vec*>(grads));
        __builtin_nontemporal_store(out_j, reinterpret_cast<vec*>(grads + units));
        __builtin_nontemporal_store(out_f, reinterpret_cast<vec*>(grads + (uint64_t)2 * units));
        __builtin_nontemporal_store(out_o, reinterpret_cast<vec*>(grads + (uint64_t)3 * units));
        __builtin_nontemporal_store(out_c, reinterpret_cast<vec*>(d_c + at));
    }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Number of workers must fit the 32-bit indices of the kernels (the generated operators have the same limit).
int check_shape(const char* who, uint32_t batch, uint32_t units) {
    if (batch == 0 || units == 0) return fail(OVL_EINVAL, std::string(who) + ": batch and units must be positive");
    if ((uint64_t)batch * units >= (1ull << 32))
        return fail(OVL_EINVAL, std::string(who) + ": batch * units must be below 2^32");
    return OVL_OK;
}

int after_launch(const char* who) {
    const hipError_t err = hipPeekAtLastError();
    if (err != hipSuccess) {
        (void)hipGetLastError();
        return fail(OVL_EHIP, std::string(who) + ": " + hipGetErrorString(err));
    }
    return OVL_OK;
}

}  // namespace

extern "C" {

const char* ovl_lstm_last_error(void) { return g_last_error.c_str(); }

int ovl_lstm_forward(const float* concat, const float* c, float forget_bias, uint32_t batch, uint32_t units,
                     int32_t fast_math, float* new_c, float* new_h, void* hip_stream) {
    if (concat == nullptr || c == nullptr || new_c == nullptr || new_h == nullptr)
        return fail(OVL_EINVAL, "ovl_lstm_forward: null tensor");
    const int rc = check_shape("ovl_lstm_forward", batch, units);
    if (rc != OVL_OK) return rc;
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const bool wide = units % 4u == 0 && aligned16(concat) && aligned16(c) && aligned16(new_c) && aligned16(new_h);
    const uint32_t vec = wide ? 4u : 1u;
    const index_divisor per_row = make_divisor(units / vec);
    const uint32_t total = batch * per_row.divisor;
    const uint64_t blocks = ((uint64_t)total + BLOCK - 1) / BLOCK;
    const dim3 grid(blocks < MAX_GRID ? (uint32_t)blocks : MAX_GRID), block(BLOCK);
#define OVL_LSTM_LAUNCH(FAST, VEC)                                                                           \
    hipLaunchKernelGGL((lstm_forward_kernel<FAST, VEC>), grid, block, 0, stream, concat, c, forget_bias,    \
                       units, per_row, total, new_c, new_h)
    if (fast_math) { if (wide) OVL_LSTM_LAUNCH(true, 4); else OVL_LSTM_LAUNCH(true, 1); }
    else { if (wide) OVL_LSTM_LAUNCH(false, 4); else OVL_LSTM_LAUNCH(false, 1); }
#undef OVL_LSTM_LAUNCH
    return after_launch("ovl_lstm_forward");
}

int ovl_lstm_backward(const float* concat, const float* c, const float* d_new_c, const float* d_new_h,
                      float forget_bias, uint32_t batch, uint32_t units, int32_t fast_math,
                      float* d_concat, float* d_c, void* hip_stream) {
    if (concat == nullptr || c == nullptr || d_new_c == nullptr || d_new_h == nullptr || d_concat == nullptr ||
        d_c == nullptr)
        return fail(OVL_EINVAL, "ovl_lstm_backward: null tensor");
    const int rc = check_shape("ovl_lstm_backward", batch, units);
    if (rc != OVL_OK) return rc;
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    const bool wide = units % 4u == 0 && aligned16(concat) && aligned16(c) && aligned16(d_new_c) &&
                      aligned16(d_new_h) && aligned16(d_concat) && aligned16(d_c);
    const uint32_t vec = wide ? 4u : 1u;
    const index_divisor per_row = make_divisor(units / vec);
    const uint32_t total = batch * per_row.divisor;
    const uint64_t blocks = ((uint64_t)total + BLOCK - 1) / BLOCK;
    const dim3 grid(blocks < MAX_GRID ? (uint32_t)blocks : MAX_GRID), block(BLOCK);
#define OVL_LSTM_LAUNCH(FAST, VEC)                                                                           \
    hipLaunchKernelGGL((lstm_backward_kernel<FAST, VEC>), grid, block, 0, stream, concat, c, d_new_c,       \
                       d_new_h, forget_bias, units, per_row, total, d_concat, d_c)
    if (fast_math) { if (wide) OVL_LSTM_LAUNCH(true, 4); else OVL_LSTM_LAUNCH(true, 1); }
    else { if (wide) OVL_LSTM_LAUNCH(false, 4); else OVL_LSTM_LAUNCH(false, 1); }
#undef OVL_LSTM_LAUNCH
    return after_launch("ovl_lstm_backward");
}

}  // extern "C"
