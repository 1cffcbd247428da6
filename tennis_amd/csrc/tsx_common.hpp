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

__device__ __forceinline__ float apply_act(float v, int act, float slope, bool in_body) {
    if (act != TSX_ACT_MISH) return apply_act_basic(v, act, slope, in_body);
    {
        // x * tanh(softplus(x)) as TenniS graphs compose it: softplus = float(log(double(expf(x)) + 1.0))
        // (src/kernels/cpu/softplus.cpp:30-39), tanh = 2 * (1 / (1 + expf(-2y))) - 1 in float
        // (src/kernels/cpu/tanh.cpp:14-23), then mul.  Same formulas; expf/log are this device's
        // library routines, so results agree with the host's to a few ulp, not bit for bit.
        const float sp = float(log(double(expf(v)) + 1.0));
        const float t = __fsub_rn(__fmul_rn(2.f, __fdiv_rn(1.f, __fadd_rn(1.f, expf(-__fmul_rn(2.f, sp))))), 1.f);
        return __fmul_rn(v, t);
    }
}

#endif  // __HIPCC__

}  // namespace tsx
