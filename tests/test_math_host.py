"""
The device math header compiled for the host: its float32 exp, log, expm1 and tanh must return, bit for bit, what
the host C library returns (the reference's generated C++ calls expf/logf/tanhf, opveclib/expression.py:1439-1441).
The same source text is what the GPU kernels compile, so agreement here plus IEEE arithmetic on the device gives
agreement on the device; the GPU parity tests confirm it end to end.

The sweep below covers every 4099th float bit pattern (about one million arguments per function, all exponents,
both signs, subnormals, infinities and NaNs); the full 2^32 sweep of all four functions was run once with the same
program (step 1) and found no mismatch.  Over all 2^32 arguments a build with the fused multiply-adds switched off
differs from the C library for exactly two arguments of expf (bit patterns 0x4202422f and 0xc27c65d9) and for none of
logf; the second test checks those two arguments, so a change of the fused/unfused choice is caught.
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), 'opveclib_amd', 'csrc')

PROGRAM = r'''
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "ovl_math.h"
typedef float (*fn)(float);
static float g_exp(float x) { return expf(x); }
static float g_log(float x) { return logf(x); }
static float g_expm1(float x) { return expm1f(x); }
static float g_tanh(float x) { return tanhf(x); }
static float o_exp(float x) { return ovl_math::expf_(x); }
static float o_log(float x) { return ovl_math::logf_(x); }
static float o_expm1(float x) { return ovl_math::expm1f_(x); }
static float o_tanh(float x) { return ovl_math::tanhf_(x); }
int main(int argc, char** argv) {
    const char* names[4] = {"exp", "log", "expm1", "tanh"};
    fn libm[4] = {g_exp, g_log, g_expm1, g_tanh};
    fn ours[4] = {o_exp, o_log, o_expm1, o_tanh};
    if (argc > 2) {
        // compare expf at the given bit patterns: prints 1 per argument when equal to the C library, else 0
        for (int i = 2; i < argc; ++i) {
            uint32_t b = (uint32_t)strtoul(argv[i], 0, 16); float x; memcpy(&x, &b, 4);
            float a = expf(x), c = ovl_math::expf_(x);
            printf("%d\n", memcmp(&a, &c, 4) == 0 ? 1 : 0);
        }
        return 0;
    }
    unsigned long long step = strtoull(argv[1], 0, 10);
    for (int f = 0; f < 4; ++f) {
        unsigned long long bad = 0, total = 0;
        for (unsigned long long u = 0; u < (1ull << 32); u += step) {
            uint32_t b = (uint32_t)u; float x; memcpy(&x, &b, 4);
            float a = libm[f](x), c = ours[f](x);
            uint32_t ua, uc; memcpy(&ua, &a, 4); memcpy(&uc, &c, 4);
            ++total;
            if (ua != uc && !(a != a && c != c)) ++bad;
        }
        printf("%s %llu %llu\n", names[f], bad, total);
    }
    return 0;
}
'''


def build(tmp_path, extra_flags):
    src = tmp_path / 'sweep.cpp'
    src.write_text(PROGRAM)
    exe = tmp_path / ('sweep' + '_'.join(extra_flags).replace('=', '_').replace('-', ''))
    subprocess.check_call(['g++', '-O2', '-ffp-contract=off', '-mfma', '-std=c++17', '-I' + CSRC] + extra_flags +
                          [str(src), '-o', str(exe)])
    return exe


def build_and_run(tmp_path, extra_flags, step):
    exe = build(tmp_path, extra_flags)
    out = subprocess.check_output([str(exe), str(step)], universal_newlines=True)
    result = {}
    for line in out.strip().splitlines():
        name, bad, total = line.split()
        result[name] = (int(bad), int(total))
    return result


def test_matches_host_libm_bit_for_bit(tmp_path):
    result = build_and_run(tmp_path, [], 4099)
    for name in ('exp', 'log', 'expm1', 'tanh'):
        bad, total = result[name]
        assert total > 1000000
        assert bad == 0, '%s: %d of %d arguments differ from the host C library' % (name, bad, total)


def test_fused_sites_matter_at_the_two_known_arguments(tmp_path):
    points = ['4202422f', 'c27c65d9']
    fused = subprocess.check_output([str(build(tmp_path, [])), '0'] + points, universal_newlines=True).split()
    assert fused == ['1', '1']
    unfused = subprocess.check_output([str(build(tmp_path, ['-DOVL_MATH_FMA_SITES=0u'])), '0'] + points,
                                      universal_newlines=True).split()
    assert unfused == ['0', '0']
