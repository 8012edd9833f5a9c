"""
The invariant-divisor index division of the hand-written kernels (opveclib_amd/csrc/ovl_index_div.h) compiled for the
host and compared with the `/` operator: every divisor and dividend near the powers of two and the ends of the 32-bit
range (where a wrong magic number or shift shows first), plus a seeded random sweep.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), 'opveclib_amd', 'csrc')

PROGRAM = r'''
#include <stdio.h>
#include <stdint.h>
#include <vector>
#include "ovl_index_div.h"
int main() {
    std::vector<uint32_t> edge;
    for (int b = 0; b < 32; ++b)
        for (int64_t off = -3; off <= 3; ++off) {
            int64_t v = (1ll << b) + off;
            if (v >= 0 && v < (1ll << 32)) edge.push_back((uint32_t)v);
        }
    for (uint32_t k = 0; k < 8; ++k) edge.push_back(0xffffffffu - k);
    const uint32_t odd[] = {3, 5, 7, 10, 641, 1000, 7919, 65521, 1000003, 16777213, 0x7fffffffu, 0xfffffffbu};
    for (uint32_t v : odd) edge.push_back(v);
    unsigned long long checked = 0, bad = 0;
    for (uint32_t d : edge) {
        if (d == 0) continue;
        const index_divisor div = make_divisor(d);
        for (uint32_t n : edge) { ++checked; if (divide(n, div) != n / d) ++bad; }
        // multiples of the divisor and their neighbours
        for (uint64_t q = 1; q * d < (1ull << 32); q = q * 3 + 1)
            for (int64_t off = -1; off <= 1; ++off) {
                const int64_t n = (int64_t)(q * d) + off;
                if (n >= 0 && n < (1ll << 32)) { ++checked; if (divide((uint32_t)n, div) != (uint32_t)n / d) ++bad; }
            }
    }
    uint64_t state = 88172645463325252ull;
    for (int i = 0; i < 2000000; ++i) {
        state ^= state << 13; state ^= state >> 7; state ^= state << 17;
        uint32_t d = (uint32_t)(state >> 32) >> ((uint32_t)state % 32u), n = (uint32_t)(state * 2654435761u >> 16);
        if (d == 0) d = 1;
        ++checked;
        if (divide(n, make_divisor(d)) != n / d) ++bad;
    }
    printf("%llu %llu\n", checked, bad);
    return 0;
}
'''


def test_invariant_division_equals_the_division_operator(tmp_path):
    src = tmp_path / 'index_div.cpp'
    src.write_text(PROGRAM)
    exe = tmp_path / 'index_div'
    subprocess.check_call(['g++', '-O2', '-std=c++14', '-I' + CSRC, str(src), '-o', str(exe)])
    checked, bad = (int(v) for v in subprocess.check_output([str(exe)], universal_newlines=True).split())
    assert checked > 2000000 and bad == 0
