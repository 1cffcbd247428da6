// Shared host/device helpers of the gfx950 kernels behind include/tsx_hip.h.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <type_traits>

#include "tsx_hip.h"

namespace tsx {

// Thread-local message behind tsx_last_error().
char *error_buffer();
int fail(int code, const char *fmt, ...);

inline int check_hip(hipError_t e, const char *what) {
    if (e == hipSuccess) return 0;
    return fail(int(e), "%s: %s", what, hipGetErrorString(e));
}

#define TSX_HIP(expr)                                        \
    do {                                                     \
        int _rc = ::tsx::check_hip((expr), #expr);           \
        if (_rc) return _rc;                                 \
    } while (0)

#define TSX_REQUIRE(cond, ...)                               \
    do {                                                     \
        if (!(cond)) return ::tsx::fail(TSX_E_INVALID, __VA_ARGS__); \
    } while (0)

// Launch check: the reference checks the runtime right after every launch and ejects
// (include/kernels/gpu/gpu_kernel.h:13-19); here the error code goes back over the C ABI.
#define TSX_LAUNCH_CHECK(name) TSX_HIP(hipGetLastError())

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// Output extent of a convolution (include/backend/common_function.h:30-40).
inline int conv_out(int in, int pad_a, int pad_b, int k, int stride, int dilation) {
    return (in + pad_a + pad_b - (dilation * (k - 1) + 1)) / stride + 1;
}

// ---------------------------------------------------------------------------
// Device-side scalar semantics shared by the quantize kernel and fused epilogues.
// ---------------------------------------------------------------------------
#ifdef __HIPCC__

// Compile-time loop: register arrays are only ever indexed by constants, which keeps them
// in VGPRs (loop-indexed arrays, and arrays of HIP's uint4/float4 structs, can end up in
// scratch memory).
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// q = clamp(round(v), -128, 127) with the reference's x86 conversion behaviour:
// NaN and |v| >= 2^31 convert to INT_MIN, i.e. -128 after the clamp
// (src/kernels/cpu/quantize.cpp:15-29,83-96).
__device__ __forceinline__ int quantize_value(float v, bool half_even) {
    // rintf = round half to even (_mm256_cvtps_epi32).  round() = half away from zero, computed as
    // trunc(v + copysign(0.5 - 2^-25, v)): the addend is the float below 0.5, so 0.49999997 stays 0 while
    // every x.5 still reaches the next integer (the sum rounds up to it); equal to roundf(v) for
    // |v| < 2^23 and, like it, far outside the clamp beyond (three instructions instead of roundf's six;
    // this runs once per element in the staging kernel, which is bound by its arithmetic).
    const float away = __builtin_truncf(v + __builtin_copysignf(0.49999997f, v));
    const float r = half_even ? __builtin_rintf(v) : away;
    // selects, not branches: this runs once per output element in the epilogues
    const float c = __builtin_amdgcn_fmed3f(r, -128.f, 127.f);   // the clamp as one instruction; NaN is overridden below
    const bool in_range = __builtin_fabsf(v) < 2147483648.0f;   // false for NaN as well
    return in_range ? int(c) : -128;
}

// Byte SEL of `word` := quantize_value(v, half_even) + 128 (offset binary; the caller XORs the finished word with
// 0x80808080): the conversion instruction saturates to [0, 255] and packs, so clamp, conversion and packing are one
// instruction.  r + 128 is exact wherever the clamp does not apply anyway; NaN and |v| >= 2^31 give byte 0 = -128, the
// reference's INT_MIN after its clamp, as in quantize_value.
template <int SEL>
__device__ __forceinline__ uint32_t quantize_pack(float v, bool half_even, uint32_t word) {
    const float away = __builtin_truncf(v + __builtin_copysignf(0.49999997f, v));
    const float r = half_even ? __builtin_rintf(v) : away;
    const bool in_range = __builtin_fabsf(v) < 2147483648.0f;   // false for NaN as well
    return __builtin_amdgcn_cvt_pk_u8_f32(in_range ? __fadd_rn(r, 128.f) : 0.f, SEL, word);
}

// relu / leaky_relu of element `in_body` (= linear index < 4*floor(count/4) of the whole
// tensor): SIMD body vs scalar tail of src/kernels/cpu/relu.cpp:30-52 and
// leaky_relu.cpp:41-66.  Body: max(x,0) returns +0 for -0 and NaN; the leaky form is one
// fused multiply-add in the reference's FMA build.  Tail: std::max / ternary.
// none / relu / leaky_relu only: for kernels that unroll the call many times -- the Mish branch below is a few hundred
// instructions (double-precision log), and dozens of inlined copies of it put the taken branches of the cheap
// activations an instruction-cache miss apart.
__device__ __forceinline__ float apply_act_basic(float v, int act, float slope, bool in_body) {
    if (act == TSX_ACT_RELU) {
        return in_body ? (v > 0.f ? v : 0.f) : (v < 0.f ? 0.f : v);
    }
    if (act == TSX_ACT_LEAKY_RELU) {
        if (in_body) {
            const float mx = v > 0.f ? v : 0.f;
            const float mn = v < 0.f ? v : 0.f;
            return __builtin_fmaf(slope, mn, mx);
        }
        return v > 0.f ? v : __fmul_rn(v, slope);
    }
    return v;
}

// cpu::Softplus (src/kernels/cpu/softplus.cpp:30-39): float(log(double(expf(x)) + 1.0)).  The host goes through double
// only to round log(1 + e) to float well; here log1pf does that in single precision (within an ulp or two of the
// correctly rounded value) at a fraction of the cost -- a double-precision logarithm per element made the Mish
// epilogue, not memory or the MFMAs, the bound of every Mish layer.  expf / log1pf are this device's library
// routines in either form, so Mish values agree with the host's to a few ulp, not bit for bit.
__device__ __forceinline__ float softplus_value(float x) { return log1pf(expf(x)); }

// e^x for the Mish epilogue: the hardware's 2^a (v_exp_f32, 1 ulp) on a = x * log2(e) carried in two floats, so that
// the product's rounding does not reach the result: 2^(ah + al) = 2^ah * (1 + al ln2 + ...).  About 1.5 ulp, no range
// handling: arguments are below 89 in magnitude where the result matters (see mish_value).
__device__ __forceinline__ float mish_exp(float x) {
    const float ah = __fmul_rn(x, 1.4426950216293335f);
    const float al = __builtin_fmaf(x, 1.925963033500011e-08f, __builtin_fmaf(x, 1.4426950216293335f, -ah));
    const float e = __builtin_amdgcn_exp2f(ah);
    return __builtin_fmaf(e, __fmul_rn(al, 0.6931471824645996f), e);
}

// Mish as TenniS graphs compose it, x * tanh(softplus(x)) with softplus = float(log(double(expf(x)) + 1.0))
// (src/kernels/cpu/softplus.cpp:30-39) and tanh(y) = 2 * (1 / (1 + expf(-2y))) - 1 in float
// (src/kernels/cpu/tanh.cpp:14-23): the same chain of rounded intermediates -- e, softplus, expf(-2 softplus), the
// quotient, 2q - 1, the product -- each within an ulp or two of the host's, evaluated on the hardware's exp2 / log2 /
// reciprocal instead of the library routines: ~45 issue slots against ~160 (two expf, a log1pf and an IEEE division
// with all their range handling), which was what bounded every Mish layer.
//   softplus: s = 1 + e with its rounding error c kept (two-sum), log(s) = log2(s) ln2 (constant in two floats) + c / s;
//             for e below 2^-24 this is e itself, as log1p gives.
//   quotient: reciprocal with one Newton step (correctly rounded but for rare ties).
// Limits as the host's: x large -> x, x very negative -> -0 or 0, NaN -> NaN.
__device__ __forceinline__ float mish_value(float x) {
    const float e = mish_exp(fminf(x, 88.f));              // beyond 88 the host's expf overflows to inf and tanh gives 1: so does this
    const float hi = fmaxf(e, 1.f), lo = fminf(e, 1.f);
    const float s = __fadd_rn(hi, lo);
    const float c = __fsub_rn(lo, __fsub_rn(s, hi));       // s + c = 1 + e exactly
    const float l2 = __builtin_amdgcn_logf(s);             // log2(s), 1 ulp
    const float rs = __builtin_amdgcn_rcpf(s);
    const float sp = __builtin_fmaf(l2, 0.6931471824645996f, __builtin_fmaf(l2, -1.9046542121259336e-09f, __fmul_rn(c, rs)));
    const float u = mish_exp(__fmul_rn(-2.f, sp));
    const float d = __fadd_rn(1.f, u);
    const float r0 = __builtin_amdgcn_rcpf(d);
    const float q = __builtin_fmaf(r0, __builtin_fmaf(-d, r0, 1.f), r0);
    const float t = __builtin_fmaf(2.f, q, -1.f);          // 2q is exact: one rounding, as fl(fl(2q) - 1)
    return __fmul_rn(x, t);
}

// Mish for the epilogues of the int8 convolution kernels, where the activation's arithmetic, not memory or the MFMAs,
// bounds a layer (the 608x608 and 304x304 layers of a YOLOv4-shaped backbone spend more issue slots on the epilogue
// than the VALUs have in the time the layer's bytes take): one exponential and one reciprocal at the hardware's 1 ulp,
//     tanh(softplus(x)) = w / (w + 2) = 1 - 2 / (w + 2),  w = e (e + 2),  e = e^x = 2^(x log2 e),
// 14 issue slots.  1 - 2r with r = 1 / (w + 2) in (0, 0.5] has the shape of the host's tanh, 2 * (1 / (1 + u)) - 1
// (src/kernels/cpu/tanh.cpp:14-23): an absolute error of about 1e-7 in the quotient, so about 1e-7 |x| in the result
// (relative 1e-7 for positive x; at most 2e-6 absolute for negative x, where Mish itself is small), against a bar of
// 1e-4 relative + 1e-5 absolute -- and, like the host's, exactly 0 (-0 for the product) once x is below about -17,
// where w + 2 rounds to 2.  NaN -> NaN, +-inf as the host's.
__device__ __forceinline__ float mish_short(float x) {
    const float e = __builtin_amdgcn_exp2f(__fmul_rn(fminf(x, 30.f), 1.4426950216293335f));   // beyond 30 the quotient is 1
    const float d = __builtin_fmaf(e, __fadd_rn(e, 2.f), 2.f);
    const float t = __builtin_fmaf(-2.f, __builtin_amdgcn_rcpf(d), 1.f);
    return __fmul_rn(x, t);
}

// apply_act for the int8 convolution epilogues: Mish in its short form (every path of those kernels -- fragment-wise
// and per element -- goes through this one, so an element's value does not depend on the tile it falls into)
__device__ __forceinline__ float apply_act_conv_i8(float v, int act, float slope, bool in_body) {
    if (act != TSX_ACT_MISH) return apply_act_basic(v, act, slope, in_body);
    return mish_short(v);
}

__device__ __forceinline__ float apply_act(float v, int act, float slope, bool in_body) {
    if (act != TSX_ACT_MISH) return apply_act_basic(v, act, slope, in_body);
    return mish_value(v);
}

#endif  // __HIPCC__

}  // namespace tsx
