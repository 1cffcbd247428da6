// Mish as TenniS graphs compose it -- mul(x, tanh(softplus(x))) -- in the host's arithmetic:
//   softplus(x) = float(log(double(expf(x)) + 1.0))          src/kernels/cpu/softplus.cpp:30-39
//   tanh(y)     = 2 * (1 / (1 + expf(-(2 y)))) - 1 in float  src/kernels/cpu/tanh.cpp:14-23
// The host's expf and log are its C library's (glibc 2.35 on the reference's x86-64 build).  Here expf is restated
// operation for operation and log is evaluated far beyond float precision, so every rounded intermediate of the
// chain, and with it the result, is the host's bit for bit.
//
// This header compiles for the device (hipcc) and, unchanged, for the host (g++ -ffp-contract=off): the host build
// exists so that a dense sweep over the floats can hold these very functions against the C library's chain without
// a GPU.  Everything is written with explicit fused multiply-adds and otherwise plain IEEE operations; the build
// must not contract or reassociate (-ffp-contract=off, no fast-math).
#pragma once
#include <cstdint>

#ifdef __HIPCC__
#define TSX_MISH_FN __device__ __forceinline__
#define TSX_MISH_MEMBER __device__ __forceinline__
#define TSX_MISH_TABLE static __device__ const
#else
#define TSX_MISH_FN static inline
#define TSX_MISH_MEMBER inline
#define TSX_MISH_TABLE static const
#endif

namespace tsx {

// 2^(i/32) as doubles, less i << 47 (the table of glibc's expf, sysdeps/ieee754/flt-32/e_exp2f_data.c)
TSX_MISH_TABLE uint64_t exp2f_table[32] = {
    0x3ff0000000000000ULL, 0x3fefd9b0d3158574ULL, 0x3fefb5586cf9890fULL, 0x3fef9301d0125b51ULL,
    0x3fef72b83c7d517bULL, 0x3fef54873168b9aaULL, 0x3fef387a6e756238ULL, 0x3fef1e9df51fdee1ULL,
    0x3fef06fe0a31b715ULL, 0x3feef1a7373aa9cbULL, 0x3feedea64c123422ULL, 0x3feece086061892dULL,
    0x3feebfdad5362a27ULL, 0x3feeb42b569d4f82ULL, 0x3feeab07dd485429ULL, 0x3feea47eb03a5585ULL,
    0x3feea09e667f3bcdULL, 0x3fee9f75e8ec5f74ULL, 0x3feea11473eb0187ULL, 0x3feea589994cce13ULL,
    0x3feeace5422aa0dbULL, 0x3feeb737b0cdc5e5ULL, 0x3feec49182a3f090ULL, 0x3feed503b23e255dULL,
    0x3feee89f995ad3adULL, 0x3feeff76f2fb5e47ULL, 0x3fef199bdd85529cULL, 0x3fef3720dcef9069ULL,
    0x3fef5818dcfba487ULL, 0x3fef7c97337b9b5fULL, 0x3fefa4afa2a490daULL, 0x3fefd0765b6e4540ULL,
};

#ifdef __HIPCC__
TSX_MISH_FN float div_rn(float a, float b) { return __fdiv_rn(a, b); }   // IEEE division whatever the build's default
#else
TSX_MISH_FN float div_rn(float a, float b) { return a / b; }
#endif
// where expf_host finds 2^(i/32): this table in memory, or whatever holds a copy of it (on the device, the lanes of
// the wavefront)
struct Exp2fTableInMemory {
    TSX_MISH_MEMBER uint64_t operator()(uint64_t i) const { return exp2f_table[i]; }
};

TSX_MISH_FN double f64_of_bits(uint64_t u) { double d; __builtin_memcpy(&d, &u, 8); return d; }
TSX_MISH_FN uint64_t bits_of_f64(double d) { uint64_t u; __builtin_memcpy(&u, &d, 8); return u; }

// The host's expf: x * 32 / ln2 = k + r, e^x = 2^(k/32) * (1 + r ln2/32 + ...) as a cubic in r, all in double, the
// product rounded to float once (glibc sysdeps/ieee754/flt-32/e_expf.c, the build with fused multiply-adds).  Its
// early returns -- inf, 0, the largest and smallest finite results beyond |x| of 88 -- come out of the same
// arithmetic on the clamped argument: the double result overflows or underflows the float conversion as the host's
// special cases say.  NaN -> NaN.
template <class Table = Exp2fTableInMemory>
TSX_MISH_FN float expf_host(float x, const Table &table = Table()) {
    const double xd = double(__builtin_fminf(__builtin_fmaxf(x, -150.f), 89.f));
    const double z = 0x1.71547652b82fep+5 * xd;          // x * 32 / ln2
    double kd = z + 0x1.8p+52;                           // the integer nearest to z, in the low mantissa bits
    const uint64_t ki = bits_of_f64(kd);
    kd -= 0x1.8p+52;
    const double r = z - kd;
    const double s = f64_of_bits(table(ki & 31) + (ki << 47));
    const double c = __builtin_fma(0x1.c6af84b912394p-5 / 32768.0, r, 0x1.ebfce50fac4f3p-3 / 1024.0);
    const double r2 = r * r;
    double y = __builtin_fma(0x1.62e42ff0c52d6p-1 / 32.0, r, 1.0);
    y = __builtin_fma(c, r2, y);
    const float e = float(y * s);
    return x != x ? x : e;
}

// log(s) for a finite double s >= 1, to well under 2^-50 relative: s = 2^k m with m in [sqrt(1/2), sqrt(2)),
// log m = 2 atanh(z), z = (m - 1) / (m + 1), as a series in z^2.  Rounded to float it is what the host's log gives
// rounded to float: both are far inside half a float ulp of the exact value.
TSX_MISH_FN double log_precise(double s) {
    const uint64_t ix = bits_of_f64(s);
    const int64_t k = int64_t(ix - 0x3fe6a09e667f3bcdULL) >> 52;
    const double m = f64_of_bits(ix - (uint64_t(k) << 52));
    const double f = m - 1.0;
    const double z = f / (2.0 + f);
    const double w = z * z;
    double p = 1.0 / 23;
    p = __builtin_fma(p, w, 1.0 / 21);
    p = __builtin_fma(p, w, 1.0 / 19);
    p = __builtin_fma(p, w, 1.0 / 17);
    p = __builtin_fma(p, w, 1.0 / 15);
    p = __builtin_fma(p, w, 1.0 / 13);
    p = __builtin_fma(p, w, 1.0 / 11);
    p = __builtin_fma(p, w, 1.0 / 9);
    p = __builtin_fma(p, w, 1.0 / 7);
    p = __builtin_fma(p, w, 1.0 / 5);
    p = __builtin_fma(p, w, 1.0 / 3);
    const double zz = z + z;
    const double lm = __builtin_fma(zz * w, p, zz);
    const double kd = double(k);
    return __builtin_fma(kd, 0x1.62e42fefa38p-1, __builtin_fma(kd, 0x1.ef35793c7673p-45, lm));   // k ln2, ln2 in two parts
}

// cpu::Softplus (src/kernels/cpu/softplus.cpp:30-39): float(log(double(expf(x)) + 1.0))
template <class Table = Exp2fTableInMemory>
TSX_MISH_FN float softplus_value(float x, const Table &table = Table()) {
    const double s = double(expf_host(x, table)) + 1.0;
    return s < __builtin_inf() ? float(log_precise(s)) : float(s);   // +inf and NaN pass through
}

// cpu::Tanh (src/kernels/cpu/tanh.cpp:14-23): T(2) * (T(1) / (T(1) + exp(-(T(2) * x)))) - T(1) in float
template <class Table = Exp2fTableInMemory>
TSX_MISH_FN float tanh_value(float y, const Table &table = Table()) {
    const float u = expf_host(-(2.f * y), table);
    const float q = div_rn(1.f, 1.f + u);
    return __builtin_fmaf(2.f, q, -1.f);   // 2q is exact: one rounding, fused or not
}

template <class Table = Exp2fTableInMemory>
TSX_MISH_FN float mish_value(float x, const Table &table = Table()) {
    return x * tanh_value(softplus_value(x, table), table);
}

}  // namespace tsx
