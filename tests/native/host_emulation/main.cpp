// Test infrastructure: runs one generated operator entry point on the host (see ovl_device.h in this directory).
//   usage: <program> n_in n_out  { dtype itemsize len path } for every input, then for every output
// Inputs are read from their files into buffers of exactly len * itemsize bytes, outputs are filled with 0xFE bytes,
// handed to the entry point and written to their files.  Exit status: 0, or 10 + the entry point's status.
#include "ovl_device.h"

#ifndef OVL_ENTRY
#error "compile with -DOVL_ENTRY=<entry point of the generated operator>"
#endif
extern "C" int OVL_ENTRY(const ovl_tensor* in, uint32_t n_in, ovl_tensor* out, uint32_t n_out, void* stream);

int main(int argc, char** argv) {
    if (argc < 3) return 2;
    const uint32_t n_in = (uint32_t)atoi(argv[1]), n_out = (uint32_t)atoi(argv[2]);
    if (argc != 3 + 4 * (int)(n_in + n_out)) return 2;
    std::vector<ovl_tensor> tensors(n_in + n_out);
    std::vector<size_t> bytes(n_in + n_out);
    for (uint32_t k = 0; k < n_in + n_out; ++k) {
        char** a = argv + 3 + 4 * k;
        tensors[k].dtype = atoi(a[0]);
        tensors[k].len = strtoull(a[2], nullptr, 10);
        bytes[k] = (size_t)tensors[k].len * (size_t)atoi(a[1]);
        if (posix_memalign(&tensors[k].data, 16, bytes[k]) != 0) return 3;
        if (k < n_in) {
            FILE* f = fopen(a[3], "rb");
            if (f == nullptr || fread(tensors[k].data, 1, bytes[k], f) != bytes[k]) return 4;
            fclose(f);
        } else {
            memset(tensors[k].data, 0xFE, bytes[k]);
        }
    }
    const int rc = OVL_ENTRY(tensors.data(), n_in, tensors.data() + n_in, n_out, nullptr);
    if (rc != 0) { fprintf(stderr, "entry point returned %d\n", rc); return 10 + rc; }
    for (uint32_t k = n_in; k < n_in + n_out; ++k) {
        FILE* f = fopen(argv[3 + 4 * k + 3], "wb");
        if (f == nullptr || fwrite(tensors[k].data, 1, bytes[k], f) != bytes[k]) return 5;
        fclose(f);
    }
    for (auto& t : tensors) free(t.data);
    return 0;
}
