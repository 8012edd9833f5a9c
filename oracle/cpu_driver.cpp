// TEST ORACLE - not part of the product.  Only tests, the smoke check and the benchmark's CPU-baseline leg use it.
//
// Host driver for operators emitted by oracle/cpp_emitter.py.  It restates the reference's ctypes test harness
// opveclib/testcop.cc:36-226 without TensorFlow's thread pool:
//   * output buffers are poisoned with 0xFE bytes before the run (testcop.cc:105-113),
//   * the operator library is dlopen'ed and the entry point looked up by name (testcop.cc:183-195),
//   * every profiling iteration creates num_threads threads, calls the entry once per thread with
//     (num_threads, thread_index) and joins them; thread creation and join are inside the timed region
//     (testcop.cc:204-219),
//   * num_threads defaults to std::thread::hardware_concurrency() (testcop.cc:198),
//   * a non-zero error word from the operator is returned to the caller (testcop.cc:221-225).
// Unlike the reference the result of dlsym is checked (the reference tests the dlopen handle twice,
// testcop.cc:190-195).
//
// Build: g++ -O2 -fPIC -shared -std=c++11 -pthread oracle/cpu_driver.cpp -o oracle/libovl_cpu_driver.so -ldl

#include <dlfcn.h>
#include <stdint.h>
#include <string.h>

#include <chrono>
#include <iostream>
#include <thread>
#include <vector>

typedef struct { void* data; int32_t dtype; uint64_t len; } ovl_tensor;

typedef void (*cpu_op_fn)(const ovl_tensor* inputs, uint32_t num_inputs, ovl_tensor* outputs, uint32_t num_outputs,
                          uint32_t num_threads, uint32_t thread_index, uint16_t* err);

static size_t dtype_size(int32_t dtype) {
    switch (dtype) {
        case 1: return 2;            // FLOAT16
        case 2: return 4;            // FLOAT32
        case 3: return 8;            // FLOAT64
        case 4: case 8: return 1;    // INT8, UINT8
        case 5: case 9: return 2;    // INT16, UINT16
        case 6: case 10: return 4;   // INT32, UINT32
        case 7: case 11: return 8;   // INT64, UINT64
        default: return 0;
    }
}

extern "C" unsigned int ovl_cpu_hardware_threads() { return std::thread::hardware_concurrency(); }

// Returns 0 on success, the operator's error word (1 = argument count/length/dtype mismatch), 2 when the library
// cannot be opened, 3 when the symbol is missing, 5 for an unknown dtype.
extern "C" int32_t ovl_cpu_run(const char* lib_path, const char* func_name,
                               const ovl_tensor* inputs, uint32_t num_inputs,
                               ovl_tensor* outputs, uint32_t num_outputs,
                               uint32_t num_threads, double* ms_per_iter, uint32_t iters) {
    for (uint32_t i = 0; i < num_outputs; ++i) {
        size_t bytes = dtype_size(outputs[i].dtype);
        if (bytes == 0) {
            std::cerr << "***ERROR - unsupported output type. " << outputs[i].dtype << '\n';
            return 5;
        }
        memset(outputs[i].data, 0xFE, bytes * outputs[i].len);
    }

    void* handle = dlopen(lib_path, RTLD_LAZY);
    if (handle == nullptr) {
        std::cerr << "***ERROR - Unable to find operator library " << lib_path << ": " << dlerror() << '\n';
        return 2;
    }
    cpu_op_fn func = reinterpret_cast<cpu_op_fn>(dlsym(handle, func_name));
    if (func == nullptr) {
        std::cerr << "***ERROR - Unable to find operator function " << func_name << '\n';
        return 3;
    }

    if (num_threads == 0) num_threads = std::thread::hardware_concurrency();
    if (num_threads == 0) num_threads = 1;

    uint16_t err = 0;
    for (uint32_t iter = 0; iter < iters; ++iter) {
        auto t1 = std::chrono::high_resolution_clock::now();
        {
            std::vector<std::thread> pool;
            pool.reserve(num_threads);
            for (uint32_t thread = 0; thread < num_threads; ++thread) {
                pool.emplace_back(func, inputs, num_inputs, outputs, num_outputs, num_threads, thread, &err);
            }
            for (auto& t : pool) t.join();
        }
        auto t2 = std::chrono::high_resolution_clock::now();
        std::chrono::duration<double, std::milli> dt = t2 - t1;
        if (ms_per_iter != nullptr) ms_per_iter[iter] = dt.count();
    }

    if (err != 0)
        std::cerr << "***ERROR - Generated operator function execution error code: " << err << '\n';
    return err;
}
