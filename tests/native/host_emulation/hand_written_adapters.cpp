// Test infrastructure: the run-time-shape entry points of include/ovl_lstm.h and include/ovl_scan.h behind the
// (inputs, outputs) calling convention of main.cpp in this directory, for host emulation of the hand-written kernels.
// The last input of every adapter is a uint32 array {dim0, dim1, skew}: with skew = 1 every tensor starts one element
// into its buffer (the buffers then hold one element more), which takes the kernels' unaligned variants.
#include "ovl_device.h"
#include "ovl_lstm.h"
#include "ovl_scan.h"

namespace {
struct shape_args { uint32_t dim0, dim1, skew; };
shape_args shape_of(const ovl_tensor& t) {
    const uint32_t* p = static_cast<const uint32_t*>(t.data);
    return shape_args{p[0], p[1], p[2]};
}
template <typename T> T* at(const ovl_tensor& t, uint32_t skew) { return static_cast<T*>(t.data) + skew; }
}  // namespace

extern "C" int emu_lstm_forward(const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* stream) {
    if (n_in != 4 || n_out != 2) return OVL_EARGS;
    const shape_args s = shape_of(in[3]);
    const float forget_bias = *static_cast<const float*>(in[2].data);
    return ovl_lstm_forward(at<const float>(in[0], s.skew), at<const float>(in[1], s.skew), forget_bias, s.dim0, s.dim1, 0,
                            at<float>(out[0], s.skew), at<float>(out[1], s.skew), stream);
}

extern "C" int emu_lstm_backward(const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* stream) {
    if (n_in != 6 || n_out != 2) return OVL_EARGS;
    const shape_args s = shape_of(in[5]);
    const float forget_bias = *static_cast<const float*>(in[4].data);
    return ovl_lstm_backward(at<const float>(in[0], s.skew), at<const float>(in[1], s.skew),
                             at<const float>(in[2], s.skew), at<const float>(in[3], s.skew), forget_bias, s.dim0, s.dim1,
                             0, at<float>(out[0], s.skew), at<float>(out[1], s.skew), stream);
}

#define OVL_EMU_SCAN(name, type)                                                                                  \
    extern "C" int emu_##name(const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* stream) { \
        if (n_in != 2 || n_out != 1) return OVL_EARGS;                                                             \
        const shape_args s = shape_of(in[1]);                                                                      \
        return ovl_##name(at<const type>(in[0], s.skew), s.dim0, s.dim1, at<type>(out[0], s.skew), stream);        \
    }
OVL_EMU_SCAN(cumsum_f32, float)
OVL_EMU_SCAN(cumprod_f32, float)
OVL_EMU_SCAN(cumsum_f64, double)
OVL_EMU_SCAN(cumprod_f64, double)
OVL_EMU_SCAN(cumsum_f32_reassociated, float)
OVL_EMU_SCAN(cumprod_f32_reassociated, float)
OVL_EMU_SCAN(cumsum_f64_reassociated, double)
OVL_EMU_SCAN(cumprod_f64_reassociated, double)

// One program serves every adapter: the environment variable OVL_EMU_FUNCTION names the one to run.
extern "C" int emu_dispatch(const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* stream) {
    typedef int (*adapter)(const ovl_tensor*, uint32_t, ovl_tensor*, uint32_t, void*);
    static const struct { const char* name; adapter fn; } table[] = {
        {"emu_lstm_forward", emu_lstm_forward}, {"emu_lstm_backward", emu_lstm_backward},
        {"emu_cumsum_f32", emu_cumsum_f32}, {"emu_cumprod_f32", emu_cumprod_f32},
        {"emu_cumsum_f64", emu_cumsum_f64}, {"emu_cumprod_f64", emu_cumprod_f64},
        {"emu_cumsum_f32_reassociated", emu_cumsum_f32_reassociated},
        {"emu_cumprod_f32_reassociated", emu_cumprod_f32_reassociated},
        {"emu_cumsum_f64_reassociated", emu_cumsum_f64_reassociated},
        {"emu_cumprod_f64_reassociated", emu_cumprod_f64_reassociated}};
    const char* wanted = getenv("OVL_EMU_FUNCTION");
    for (const auto& entry : table)
        if (wanted != nullptr && strcmp(wanted, entry.name) == 0) return entry.fn(in, n_in, out, n_out, stream);
    fprintf(stderr, "OVL_EMU_FUNCTION names no adapter\n");
    return OVL_EARGS;
}
