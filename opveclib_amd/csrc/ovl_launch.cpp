// C-ABI launcher for generated HIP operators (declared in include/ovl_launch.h).
//
// Native successor of the reference's launch layer: the dlopen/dlsym/launch/timing parts of
// opveclib/testcudaop.cc:276-304 and opveclib/dynamiclibop.cc:129-176.  Unlike testcudaop.cc it owns no device
// memory and creates neither context nor stream: tensors and the stream come from the caller (PyTorch in this
// package), so an operator launch is asynchronous and allocation free.
//
// Build: hipcc -O2 -fPIC -shared -std=c++17 -I include opveclib_amd/csrc/ovl_launch.cpp
//              -o opveclib_amd/csrc/libovl_launch.so -ldl

#include "ovl_launch.h"

#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>

namespace {

thread_local std::string g_last_error;

int fail(int code, const std::string& detail) {
    g_last_error = detail;
    return code;
}

int hip_fail(hipError_t err, const char* what) {
    return fail(OVL_EHIP, std::string(what) + ": " + hipGetErrorString(err));
}

struct Library {
    void* dl;
    std::string path;
};

}  // namespace

extern "C" {

uint32_t ovl_abi_version(void) { return 1; }

uint32_t ovl_dtype_size(int32_t dtype) {
    switch (dtype) {
        case OVL_FLOAT16: case OVL_INT16: case OVL_UINT16: return 2;
        case OVL_FLOAT32: case OVL_INT32: case OVL_UINT32: return 4;
        case OVL_FLOAT64: case OVL_INT64: case OVL_UINT64: return 8;
        case OVL_INT8: case OVL_UINT8: return 1;
        default: return 0;
    }
}

const char* ovl_strerror(int code) {
    switch (code) {
        case OVL_OK: return "success";
        case OVL_EARGS: return "operator argument count, length or dtype mismatch";
        case OVL_EOPEN: return "cannot open operator library";
        case OVL_ESYMBOL: return "operator entry point not found";
        case OVL_EHIP: return "HIP runtime error";
        case OVL_EALIGN: return "tensor pointer not aligned for vector access";
        case OVL_EINVAL: return "invalid launcher argument";
        default: return "unknown error code";
    }
}

const char* ovl_last_error(void) { return g_last_error.c_str(); }

int ovl_lib_open(const char* so_path, void** handle) {
    if (so_path == nullptr || handle == nullptr) return fail(OVL_EINVAL, "ovl_lib_open: null argument");
    *handle = nullptr;
    void* dl = dlopen(so_path, RTLD_NOW | RTLD_LOCAL);
    if (dl == nullptr) {
        const char* why = dlerror();
        return fail(OVL_EOPEN, std::string(so_path) + ": " + (why ? why : "dlopen failed"));
    }
    *handle = new Library{dl, so_path};
    return OVL_OK;
}

int ovl_lib_sym(void* handle, const char* symbol, ovl_entry_fn* fn) {
    if (handle == nullptr || symbol == nullptr || fn == nullptr)
        return fail(OVL_EINVAL, "ovl_lib_sym: null argument");
    Library* lib = static_cast<Library*>(handle);
    dlerror();
    void* sym = dlsym(lib->dl, symbol);
    if (sym == nullptr) {
        *fn = nullptr;
        return fail(OVL_ESYMBOL, std::string(symbol) + " not found in " + lib->path);
    }
    *fn = reinterpret_cast<ovl_entry_fn>(sym);
    return OVL_OK;
}

int ovl_lib_close(void* handle) {
    if (handle == nullptr) return fail(OVL_EINVAL, "ovl_lib_close: null handle");
    Library* lib = static_cast<Library*>(handle);
    int rc = dlclose(lib->dl);
    delete lib;
    if (rc != 0) return fail(OVL_EOPEN, "dlclose failed");
    return OVL_OK;
}

int ovl_launch_fn(ovl_entry_fn fn, const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out,
                  void* hip_stream) {
    if (fn == nullptr) return fail(OVL_EINVAL, "ovl_launch_fn: null entry point");
    if ((n_in > 0 && in == nullptr) || (n_out > 0 && out == nullptr))
        return fail(OVL_EINVAL, "ovl_launch_fn: null tensor list");
    int rc = fn(in, n_in, out, n_out, hip_stream);
    if (rc != OVL_OK) {
        if (rc == OVL_EHIP) {
            hipError_t err = hipGetLastError();
            return hip_fail(err, "kernel launch");
        }
        return fail(rc, ovl_strerror(rc));
    }
    return OVL_OK;
}

int ovl_launch(void* handle, const char* symbol, const ovl_tensor* in, uint32_t n_in, ovl_tensor* out,
               uint32_t n_out, void* hip_stream) {
    ovl_entry_fn fn = nullptr;
    int rc = ovl_lib_sym(handle, symbol, &fn);
    if (rc != OVL_OK) return rc;
    return ovl_launch_fn(fn, in, n_in, out, n_out, hip_stream);
}

int ovl_time(ovl_entry_fn fn, const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out,
             void* hip_stream, uint32_t iters, double* ms_per_iter) {
    if (iters == 0 || ms_per_iter == nullptr) return fail(OVL_EINVAL, "ovl_time: no iterations or null result");
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    hipEvent_t start = nullptr, stop = nullptr;
    hipError_t err = hipEventCreate(&start);
    if (err != hipSuccess) return hip_fail(err, "hipEventCreate");
    err = hipEventCreate(&stop);
    if (err != hipSuccess) {
        hipEventDestroy(start);
        return hip_fail(err, "hipEventCreate");
    }
    int rc = OVL_OK;
    for (uint32_t i = 0; i < iters && rc == OVL_OK; ++i) {
        err = hipStreamSynchronize(stream);
        if (err != hipSuccess) { rc = hip_fail(err, "hipStreamSynchronize"); break; }
        err = hipEventRecord(start, stream);
        if (err != hipSuccess) { rc = hip_fail(err, "hipEventRecord"); break; }
        rc = ovl_launch_fn(fn, in, n_in, out, n_out, hip_stream);
        if (rc != OVL_OK) break;
        err = hipEventRecord(stop, stream);
        if (err != hipSuccess) { rc = hip_fail(err, "hipEventRecord"); break; }
        err = hipEventSynchronize(stop);
        if (err != hipSuccess) { rc = hip_fail(err, "hipEventSynchronize"); break; }
        float ms = 0.0f;
        err = hipEventElapsedTime(&ms, start, stop);
        if (err != hipSuccess) { rc = hip_fail(err, "hipEventElapsedTime"); break; }
        ms_per_iter[i] = static_cast<double>(ms);
    }
    hipEventDestroy(start);
    hipEventDestroy(stop);
    return rc;
}

int ovl_poison(ovl_tensor* out, uint32_t n_out, void* hip_stream) {
    if (n_out > 0 && out == nullptr) return fail(OVL_EINVAL, "ovl_poison: null tensor list");
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    for (uint32_t i = 0; i < n_out; ++i) {
        uint32_t width = ovl_dtype_size(out[i].dtype);
        if (width == 0) return fail(OVL_EARGS, "ovl_poison: unknown dtype");
        hipError_t err = hipMemsetAsync(out[i].data, 0xFE, static_cast<size_t>(width) * out[i].len, stream);
        if (err != hipSuccess) return hip_fail(err, "hipMemsetAsync");
    }
    return OVL_OK;
}

}  // extern "C"
