// Host build of the device's exact Mish arithmetic (tennis_amd/csrc/tsx_mish.hpp, the very header the kernels
// compile) swept against the C library's chain as the reference's operators evaluate it
// (src/kernels/cpu/softplus.cpp:30-39, tanh.cpp:14-23, mul): counts of floats whose bits differ.
// Built by tests/test_mish_host.py with g++ -O2 -ffp-contract=off -fopenmp.
#include <cmath>
#include <cstdint>
#include <cstring>

#include "tsx_mish.hpp"

static inline uint32_t bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float host_softplus(float x) { return float(std::log(double(std::exp(x)) + 1.)); }
static inline float host_tanh(float y) { return 2.f * (1.f / (1.f + std::exp(-(2.f * y)))) - 1.f; }

// Every `stride`-th float bit pattern from `first` on whose magnitude is below `limit`; out = {checked, mish,
// softplus, tanh, expf} mismatches (NaN results compare as equal when both are NaN).
extern "C" void mish_sweep(uint32_t first, uint32_t stride, float limit, long long *out) {
    long long total = 0, bad_mish = 0, bad_sp = 0, bad_tanh = 0, bad_exp = 0;
#pragma omp parallel for reduction(+ : total, bad_mish, bad_sp, bad_tanh, bad_exp) schedule(static)
    for (long long b = first; b < (1LL << 32); b += stride) {
        const uint32_t u = uint32_t(b);
        float x;
        memcpy(&x, &u, 4);
        if (!(std::fabs(x) < limit)) continue;
        ++total;
        const float sp = host_softplus(x);
        bad_exp += bits(tsx::expf_host(x)) != bits(std::exp(x));
        bad_sp += bits(tsx::softplus_value(x)) != bits(sp);
        bad_tanh += bits(tsx::tanh_value(x)) != bits(host_tanh(x));
        bad_mish += bits(tsx::mish_value(x)) != bits(x * host_tanh(sp));
    }
    out[0] = total, out[1] = bad_mish, out[2] = bad_sp, out[3] = bad_tanh, out[4] = bad_exp;
}

extern "C" void mish_values(const float *x, long long count, float *mish, float *softplus, float *tanh_, float *expf_) {
    for (long long i = 0; i < count; ++i) {
        mish[i] = tsx::mish_value(x[i]);
        softplus[i] = tsx::softplus_value(x[i]);
        tanh_[i] = tsx::tanh_value(x[i]);
        expf_[i] = tsx::expf_host(x[i]);
    }
}
