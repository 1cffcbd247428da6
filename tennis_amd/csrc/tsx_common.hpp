// Shared host/device helpers of the gfx950 kernels behind include/tsx_hip.h.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <type_traits>

#include "tsx_hip.h"
#include "tsx_mish.hpp"

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

// Mish, softplus and tanh in the host's arithmetic: tsx_mish.hpp (shared with the CPU build that pins them)
// The fast form for layers bound by the activation's arithmetic (the 608x608 and 304x304 layers of a YOLOv4-shaped
// backbone spend more issue slots on an exact Mish than the VALUs have in the time the layer's bytes take): one
// exponential and one reciprocal at the hardware's 1 ulp,
//     tanh(softplus(x)) = w / (w + 2) = 1 - 2 / (w + 2),  w = e (e + 2),  e = e^x = 2^(x log2 e),
// 14 issue slots.  1 - 2r with r = 1 / (w + 2) in (0, 0.5] has the shape of the host's tanh: an absolute error of about
// 1e-7 in the quotient, so about 1e-7 |x| in the result (at most 2e-6 absolute for negative x, where Mish itself is
// small) -- and, like the host's, exactly 0 (-0 for the product) once x is below about -17, where w + 2 rounds to 2.
// NaN -> NaN, +-inf as the host's.  A requantized int8 value differs from the exact form's in about one of a million.
// Opt-in (TSX_ACT_MISH_FAST); TSX_ACT_MISH is the exact form, mish_value.
__device__ __forceinline__ float mish_short(float x) {
    const float e = __builtin_amdgcn_exp2f(__fmul_rn(fminf(x, 30.f), 1.4426950216293335f));   // beyond 30 the quotient is 1
    const float d = __builtin_fmaf(e, __fadd_rn(e, 2.f), 2.f);
    const float t = __builtin_fmaf(-2.f, __builtin_amdgcn_rcpf(d), 1.f);
    return __fmul_rn(x, t);
}

// The activation of every epilogue: none / relu / leaky_relu / Mish (exact) / Mish (fast).  One function for all
// kernels and all their paths, so an element's value never depends on the kernel or tile it falls into, and a fused
// node gives what the separate operators give.
__device__ __forceinline__ float apply_act(float v, int act, float slope, bool in_body) {
    if (act == TSX_ACT_MISH) return mish_value(v);
    if (act == TSX_ACT_MISH_FAST) return mish_short(v);
    return apply_act_basic(v, act, slope, in_body);
}
// The 2^(i/32) table of the host's expf held by the wavefront itself: lane l keeps entry l % 32 in two registers, and
// a lane's look-up is two cross-lane reads (ds_bpermute) instead of a gather from memory -- twice per Mish value, in
// the middle of its dependent chain.  Every lane must be active where it is used.
struct Exp2fTableInLanes {
    int lo, hi;
    __device__ __forceinline__ explicit Exp2fTableInLanes(int lane) {
        const uint64_t mine = exp2f_table[lane & 31];
        lo = int(uint32_t(mine));
        hi = int(uint32_t(mine >> 32));
    }
    __device__ __forceinline__ uint64_t operator()(uint64_t i) const {
        const int addr = int(i) * 4;
        return uint64_t(uint32_t(__builtin_amdgcn_ds_bpermute(addr, lo))) |
               (uint64_t(uint32_t(__builtin_amdgcn_ds_bpermute(addr, hi))) << 32);
    }
};

// The exact Mish of the 16 values of an accumulator fragment, two values per turn of a loop that stays a loop: each
// value's chain holds a dozen double-precision temporaries and twenty constants, and sixteen chains unrolled side by
// side would push a kernel that keeps its accumulators and operands in registers into scratch memory; two give the
// scheduler something to put into the other's latencies.  The loop counter is uniform: the values are reached by
// register indexing.
__device__ __forceinline__ void mish_fragment(float (&v)[16]) {
    typedef float v16f __attribute__((ext_vector_type(16)));
    v16f t;
#pragma unroll
    for (int r = 0; r < 16; ++r) t[r] = v[r];
    if (__builtin_amdgcn_ballot_w64(true) == ~0ull) {
        const Exp2fTableInLanes table(int(threadIdx.x));
#pragma clang loop unroll(disable)
        for (int r = 0; r < 16; r += 2) {
            const float a = mish_value(t[r], table), b = mish_value(t[r + 1], table);
            t[r] = a;
            t[r + 1] = b;
        }
    } else {
#pragma clang loop unroll(disable)
        for (int r = 0; r < 16; ++r) t[r] = mish_value(t[r]);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) v[r] = t[r];
}

// The exact Mish where only a requantized int8 value leaves the kernel: round((mish(x) [+ add]) * scale) has to be
// the exact form's, the float in between does not.  mish_short is within 5.21 * 2^-24 |x| of mish_value for every
// float x (all 2^32 inputs compared on the device, tests/test_gpu_yolo.py), so wherever the short form's product
// lies further from a rounding boundary k + 1/2 than that bound (taken as 8 * 2^-24 |x scale|, plus 2^-21 of the
// product for the two float roundings behind the activation) both forms round to the same integer.  The few values
// that lie closer -- about one in ten thousand -- are evaluated again by the exact chain, a wavefront at a time and
// only where a lane asks.  Values in v: pre-activation in, mish out (exact where it matters).
__device__ __forceinline__ void mish_fragment_for_rounding(float (&v)[16], const float (&add)[16], bool with_add, float scale) {
    typedef float v16f __attribute__((ext_vector_type(16)));
    v16f x, m;
    unsigned near = 0;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        x[r] = v[r];
        m[r] = mish_short(v[r]);
        const float sum = with_add ? __fadd_rn(m[r], add[r]) : m[r];
        const float a = __builtin_fabsf(__fmul_rn(sum, scale));
        const float dist = __builtin_fabsf(__fsub_rn(__fsub_rn(a, __builtin_floorf(a)), 0.5f));
        const float margin = __builtin_fmaf(__builtin_fabsf(__fmul_rn(v[r], scale)), 0x1p-21f, __builtin_fmaf(a, 0x1p-21f, 1e-30f));
        near |= dist > margin ? 0u : 1u << r;      // NaN and infinity: near
    }
    if (__builtin_amdgcn_ballot_w64(near != 0) != 0) {
#pragma clang loop unroll(disable)
        for (int r = 0; r < 16; ++r)
            if ((near >> r) & 1u) m[r] = mish_value(x[r]);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) v[r] = m[r];
}

__device__ __forceinline__ float apply_act_conv_i8(float v, int act, float slope, bool in_body) {
    return apply_act(v, act, slope, in_body);
}
// ... for kernel instantiations that layers with the exact Mish are never routed to
__device__ __forceinline__ float apply_act_without_exact_mish(float v, int act, float slope, bool in_body) {
    if (act == TSX_ACT_MISH_FAST) return mish_short(v);
    return apply_act_basic(v, act, slope, in_body);
}

#endif  // __HIPCC__

}  // namespace tsx
