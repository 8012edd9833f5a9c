/*
 * C ABI of the OVL operator launcher for AMD GPUs (libovl_launch.so).
 *
 * The launcher loads operator libraries that the HIP code generator produced with hipcc and enqueues their kernels
 * on a caller-supplied HIP stream.  It replaces the reference's native launch layer:
 *
 *   reference interface                                                     replaced by
 *   ----------------------------------------------------------------------  ---------------------------------
 *   struct TensorParam {void* data; DType dtype; size_t len;}               ovl_tensor
 *       opveclib/testcop.cc:28-32, testcudaop.cc:52-56;
 *       Python twin _TensorParam, opveclib/operator.py:128-131
 *   InputParameter / TypedInput<T> / OutputParameter / TypedOutput<T>       ovl_tensor (dtype checked by the
 *       opveclib/dynamiclibop.h:25-94                                       generated entry point)
 *   testCUDAOperator(libPath, funcName, in, nIn, out, nOut, tpb, ms, it)    ovl_lib_open + ovl_launch / ovl_time
 *       opveclib/testcudaop.cc:60-66 (dlopen 276-290, timed loop 294-304)
 *   DynamicLibLaunch<GPUDevice>: dlopen + dlsym + enqueue on d.stream()     ovl_lib_open + ovl_lib_sym +
 *       opveclib/dynamiclibop.cc:129-176                                    ovl_launch_fn
 *   generated  <f>_generic_cuda(inputs, outputs, CUstream, tpb, err*)       ovl_entry_fn (symbol <f>_generic_hip)
 *       opveclib/expression.py:686-698
 *
 * Conventions
 *   - All tensor memory is owned by the caller and must be device accessible; the launcher never allocates, frees
 *     or copies tensor memory.  `len` counts elements, not bytes.
 *   - ovl_launch / ovl_launch_fn only enqueue work on `hip_stream` (a hipStream_t; NULL is the default stream) and
 *     return without synchronising.  ovl_time synchronises the stream around every timed launch.
 *   - Every function returns 0 on success or one of the OVL_E* codes; nothing calls exit() or throws.
 *   - Functions are thread safe; a handle may be shared between threads.  Handles stay valid until ovl_lib_close.
 */
#ifndef OVL_LAUNCH_H_
#define OVL_LAUNCH_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Data type codes: the DType enum of the operator IR (opveclib/language.proto:16-37). */
enum ovl_dtype {
    OVL_UNDEFINED_TYPE = 0,
    OVL_FLOAT16 = 1, OVL_FLOAT32 = 2, OVL_FLOAT64 = 3,
    OVL_INT8 = 4, OVL_INT16 = 5, OVL_INT32 = 6, OVL_INT64 = 7,
    OVL_UINT8 = 8, OVL_UINT16 = 9, OVL_UINT32 = 10, OVL_UINT64 = 11
};

/* One flat, C-ordered tensor argument. */
typedef struct ovl_tensor {
    void*    data;   /* device pointer */
    int32_t  dtype;  /* enum ovl_dtype */
    uint64_t len;    /* number of elements */
} ovl_tensor;

/* Error codes. 1 keeps the meaning of the reference's `*err = 1` (expression.py:622, 639, 662-663). */
enum ovl_status {
    OVL_OK = 0,
    OVL_EARGS = 1,       /* wrong number of tensors, wrong element count or wrong dtype for this operator */
    OVL_EOPEN = 2,       /* operator library could not be opened */
    OVL_ESYMBOL = 3,     /* entry point not found in the operator library */
    OVL_EHIP = 4,        /* the HIP runtime reported an error (see ovl_last_error) */
    OVL_EALIGN = 5,      /* a tensor pointer is not aligned for the kernel's vector accesses (16 bytes) */
    OVL_EINVAL = 6       /* invalid argument to the launcher itself (null pointer, zero iterations, ...) */
};

/* Signature of every generated operator entry point `<name>_generic_hip`: validates its arguments, enqueues the
 * operator's kernel(s) on `stream`, returns an ovl_status.  `stream` is a hipStream_t passed as void*. */
typedef int (*ovl_entry_fn)(const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* stream);

/* Open an operator library built by the code generator.  *handle receives an opaque handle. */
int ovl_lib_open(const char* so_path, void** handle);

/* Resolve an entry point of an open library. */
int ovl_lib_sym(void* handle, const char* symbol, ovl_entry_fn* fn);

/* Close a library handle.  Kernels already enqueued keep running; do not close while launches are being issued. */
int ovl_lib_close(void* handle);

/* Enqueue operator `symbol` of an open library on `hip_stream`. */
int ovl_launch(void* handle, const char* symbol,
               const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* hip_stream);

/* Enqueue an already resolved entry point (avoids the symbol lookup in tight loops). */
int ovl_launch_fn(ovl_entry_fn fn,
                  const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* hip_stream);

/* Launch `iters` times, timing each launch with HIP events recorded on `hip_stream` (device time between the two
 * events, in milliseconds, written to ms_per_iter[0..iters-1]).  Synchronises the stream. */
int ovl_time(ovl_entry_fn fn,
             const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* hip_stream,
             uint32_t iters, double* ms_per_iter);

/* Fill every output tensor with 0xFE bytes on `hip_stream`, so elements an operator fails to write are
 * recognisable (the reference's harness does the same: testcudaop.cc:188-269, testcop.cc:105-113). */
int ovl_poison(ovl_tensor* out, uint32_t n_out, void* hip_stream);

/* Size in bytes of one element of `dtype`, 0 for an unknown code. */
uint32_t ovl_dtype_size(int32_t dtype);

/* Static description of a status code. */
const char* ovl_strerror(int code);

/* Detail of the most recent failure on the calling thread (empty string if none). */
const char* ovl_last_error(void);

/* Launcher ABI version; bumped when this header changes incompatibly. */
uint32_t ovl_abi_version(void);

#ifdef __cplusplus
}
#endif

#endif  /* OVL_LAUNCH_H_ */
