// Test infrastructure: an operator library written by hand against the launcher's C ABI, not produced by the code
// generator - the counterpart of the reference's test operator opveclib/test/addgpu.cu (loaded there through the
// DynamicLib op, opveclib/test/test_dynamiclib_addgpu.py).  It shows that the boundary is the ABI of
// include/ovl_launch.h and nothing else: any library exporting entry points of this signature can be launched.
//
//   out0 = in0 + in1      (float32 or float64, equal lengths)
//   out1 = in0 - in1      (optional second output)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ovl_device.h"

namespace {

template <typename T>
__global__ void __launch_bounds__(256) add_sub_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                      T* __restrict__ sum, T* __restrict__ diff, uint64_t n) {
    const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        sum[i] = a[i] + b[i];
        if (diff != nullptr) diff[i] = a[i] - b[i];
    }
}

template <typename T>
int launch(const ovl_tensor* in, ovl_tensor* out, uint32_t n_out, hipStream_t stream) {
    const uint64_t n = in[0].len;
    if (n == 0) return OVL_OK;
    const uint32_t grid = (uint32_t)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
    hipLaunchKernelGGL(add_sub_kernel<T>, dim3(grid), dim3(256), 0, stream, static_cast<const T*>(in[0].data),
                       static_cast<const T*>(in[1].data), static_cast<T*>(out[0].data),
                       n_out > 1 ? static_cast<T*>(out[1].data) : nullptr, n);
    return hipPeekAtLastError() == hipSuccess ? OVL_OK : OVL_EHIP;
}

}  // namespace

extern "C" int hand_written_add_generic_hip(const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out,
                                            void* stream) {
    if (n_in != 2 || n_out < 1 || n_out > 2) return OVL_EARGS;
    for (uint32_t k = 0; k < n_out; ++k)
        if (out[k].len != in[0].len || out[k].dtype != in[0].dtype) return OVL_EARGS;
    if (in[1].len != in[0].len || in[1].dtype != in[0].dtype) return OVL_EARGS;
    if (in[0].dtype == 2) return launch<float>(in, out, n_out, static_cast<hipStream_t>(stream));     // FLOAT32
    if (in[0].dtype == 3) return launch<double>(in, out, n_out, static_cast<hipStream_t>(stream));    // FLOAT64
    return OVL_EARGS;
}
