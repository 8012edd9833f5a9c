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

// float32 transcendental entry points used by generated code: bit-compatible with the host C library's
// expf/logf/tanhf (see ovl_math.h)
__device__ __forceinline__ float ovl_expf(float x) { return ovl_math::expf_(x); }
__device__ __forceinline__ float ovl_logf(float x) { return ovl_math::logf_(x); }
__device__ __forceinline__ float ovl_tanhf(float x) { return ovl_math::tanhf_(x); }

#endif  // OVL_DEVICE_H_
