// Stand-alone HBM-bound epilogue operators (4 B read + 4 B written per element), for graphs
// that keep add_bias / relu / leaky_relu as separate nodes:
//   cpu::AddBias    src/kernels/cpu/add_bias.cpp:47-85      y = x + b[c]
//   cpu::ReLU       src/kernels/cpu/relu.cpp:30-52          SIMD body max(x,0), scalar tail std::max
//   cpu::LeakyReLU  src/kernels/cpu/leaky_relu.cpp:41-66    body fma(scale, min(x,0), max(x,0)), tail x>0?x:x*scale
//   cpu::Add        src/kernels/cpu/add.cpp                 y = a + b on equal shapes (a residual join), optionally
//                                                           followed by the activation operator in the same pass
//   cpu::Mul        src/kernels/cpu/mul.cpp                 y = a * b, equal shapes or broadcast
//   cpu::Softplus   src/kernels/cpu/softplus.cpp:30-39      y = float(log(double(expf(x)) + 1.0))
//   cpu::Tanh       src/kernels/cpu/tanh.cpp:14-23          y = 2 * (1 / (1 + expf(-2x))) - 1 in float
// (softplus, tanh and mul are the nodes TenniS graphs compose Mish from; expf / log are this device's library
// routines, so those two agree with the host's to a few ulp, not bit for bit)
// Each lane handles 4 consecutive elements (16-byte accesses) in a grid-stride loop.
#include "tsx_common.hpp"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

// MODE 0: add_bias (layout [pre][channels][inner]); 1: relu; 2: leaky_relu; 3: add (second operand in `bias`) + act;
// 4: mish; 5: softplus; 6: tanh; 7: mul (second operand in `bias`)
template <int MODE>
__global__ __launch_bounds__(256) void elementwise_kernel(const float *__restrict__ x, int64_t count,
                                                         const float *__restrict__ bias, int channels, int64_t inner,
                                                         float slope, int64_t body, float *__restrict__ out, bool vec,
                                                         int act) {
    const int64_t stride = int64_t(gridDim.x) * blockDim.x * 4;
    for (int64_t base = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) * 4; base < count; base += stride) {
        float v[4];
        const bool full = vec && base + 4 <= count;
        float u[4] = {0.f, 0.f, 0.f, 0.f};
        if (full) {
            const v4f in = *reinterpret_cast<const v4f *>(x + base);
            v[0] = in[0]; v[1] = in[1]; v[2] = in[2]; v[3] = in[3];
            if (MODE == 3 || MODE == 7) {
                const v4f in2 = *reinterpret_cast<const v4f *>(bias + base);
                u[0] = in2[0]; u[1] = in2[1]; u[2] = in2[2]; u[3] = in2[3];
            }
        } else {
            for (int j = 0; j < 4; ++j) v[j] = base + j < count ? x[base + j] : 0.f;
            if (MODE == 3 || MODE == 7)
                for (int j = 0; j < 4; ++j) u[j] = base + j < count ? bias[base + j] : 0.f;
        }
        // add_bias: a lane's four elements share their channel when the inner extent is a multiple of 4 (one
        // division instead of four; 32-bit where the tensor allows it)
        const bool one_channel = MODE == 0 && full && (inner & 3) == 0;
        float lane_bias = 0.f;
        if (one_channel)
            lane_bias = bias[count < (int64_t(1) << 32) ? int((unsigned(base) / unsigned(inner)) % unsigned(channels))
                                                        : int((base / inner) % channels)];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t i = base + j;
            if (MODE == 0) {
                if (one_channel) v[j] = __fadd_rn(v[j], lane_bias);
                else if (i < count) v[j] = __fadd_rn(v[j], bias[(i / inner) % channels]);
            } else if (MODE == 3) {
                v[j] = tsx::apply_act(__fadd_rn(v[j], u[j]), act, slope, i < body);
            } else if (MODE == 4) {
                v[j] = tsx::apply_act(v[j], TSX_ACT_MISH, 0.f, true);
            } else if (MODE == 5) {
                v[j] = tsx::softplus_value(v[j]);
            } else if (MODE == 6) {
                v[j] = tsx::tanh_value(v[j]);
            } else if (MODE == 7) {
                v[j] = __fmul_rn(v[j], u[j]);
            } else {
                v[j] = tsx::apply_act(v[j], MODE == 1 ? TSX_ACT_RELU : TSX_ACT_LEAKY_RELU, slope, i < body);
            }
        }
        if (full) {
            v4f o = {v[0], v[1], v[2], v[3]};
            *reinterpret_cast<v4f *>(out + base) = o;
        } else {
            for (int j = 0; j < 4; ++j)
                if (base + j < count) out[base + j] = v[j];
        }
    }
}

template <int MODE>
int launch(const float *x, int64_t count, const float *bias, int channels, int64_t inner, float slope, float *out,
           void *stream, int act = TSX_ACT_NONE) {
    if (count == 0) return 0;
    TSX_REQUIRE(x && out, "elementwise: null pointer");
    const bool vec = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                     ((MODE != 3 && MODE != 7) || reinterpret_cast<uintptr_t>(bias) % 16 == 0);
    int64_t blocks = tsx::ceil_div(tsx::ceil_div(count, 4), 256);
    if (blocks > 256 * 8) blocks = 256 * 8;
    hipLaunchKernelGGL(elementwise_kernel<MODE>, dim3(unsigned(blocks)), dim3(256), 0, tsx::as_stream(stream), x, count,
                       bias, channels, inner, slope, count / 4 * 4, out, vec, act);
    TSX_LAUNCH_CHECK("elementwise_kernel");
    return 0;
}

// batch_norm / batch_scale / fused_batch_norm on [pre][channels][inner] (src/kernels/cpu/batch_norm.cpp:61-105,
// batch_scale.cpp:57-97, fused_batch_norm.cpp:70-125), 4 elements per lane.  The reference's arithmetic, rounding
// for rounding: 1 / sqrt(var + eps) with the sum in float, root and quotient in double, rounded to float once;
// (x - mean) * that; x * scale + bias as ONE fused multiply-add (its FMA build contracts the 4-wide body and the
// scalar tail alike).  NORM: 0 = batch_scale, 1 = batch_norm, 2 = fused_batch_norm.
template <int NORM>
__global__ __launch_bounds__(256) void channel_affine_kernel(const float *__restrict__ x, int64_t count, int channels,
                                                            int64_t inner, const float *__restrict__ mean,
                                                            const float *__restrict__ variance,
                                                            const float *__restrict__ scale, const float *__restrict__ bias,
                                                            float epsilon, float *__restrict__ out, bool vec) {
    auto apply = [&](float v, int c) -> float {
        if (NORM != 0) {
            const float sum = __fadd_rn(variance[c], epsilon);
            const float inv = float(1.0 / sqrt(double(sum)));
            v = __fmul_rn(__fsub_rn(v, mean[c]), inv);
        }
        if (NORM != 1) v = __builtin_fmaf(v, scale[c], bias[c]);
        return v;
    };
    const int64_t stride = int64_t(gridDim.x) * blockDim.x * 4;
    for (int64_t base = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) * 4; base < count; base += stride) {
        if (vec && base + 4 <= count) {
            const v4f in = *reinterpret_cast<const v4f *>(x + base);
            v4f o;
            if ((inner & 3) == 0) {   // the lane's four elements share their channel
                const int c = count < (int64_t(1) << 32) ? int((unsigned(base) / unsigned(inner)) % unsigned(channels))
                                                         : int((base / inner) % channels);
                float m = 0.f, inv = 0.f, sc = 0.f, bi = 0.f;
                if (NORM != 0) {
                    m = mean[c];
                    inv = float(1.0 / sqrt(double(__fadd_rn(variance[c], epsilon))));
                }
                if (NORM != 1) {
                    sc = scale[c];
                    bi = bias[c];
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float v = in[j];
                    if (NORM != 0) v = __fmul_rn(__fsub_rn(v, m), inv);
                    if (NORM != 1) v = __builtin_fmaf(v, sc, bi);
                    o[j] = v;
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] = apply(in[j], int(((base + j) / inner) % channels));
            }
            *reinterpret_cast<v4f *>(out + base) = o;
        } else {
            for (int j = 0; j < 4; ++j)
                if (base + j < count) out[base + j] = apply(x[base + j], int(((base + j) / inner) % channels));
        }
    }
}

template <int NORM>
int launch_affine(const char *who, const float *x, int64_t pre, int channels, int64_t inner, const float *mean,
                  const float *variance, const float *scale, const float *bias, float epsilon, float *out, void *stream) {
    TSX_REQUIRE(pre >= 0 && channels > 0 && inner > 0, "%s: bad extent", who);
    TSX_REQUIRE((NORM == 0 || (mean && variance)) && (NORM == 1 || (scale && bias)), "%s: null parameter vector", who);
    const int64_t count = pre * channels * inner;
    if (count == 0) return 0;
    TSX_REQUIRE(x && out, "%s: null pointer", who);
    const bool vec = reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    int64_t blocks = tsx::ceil_div(tsx::ceil_div(count, 4), 256);
    if (blocks > 256 * 8) blocks = 256 * 8;
    hipLaunchKernelGGL(channel_affine_kernel<NORM>, dim3(unsigned(blocks)), dim3(256), 0, tsx::as_stream(stream), x, count,
                       channels, inner, mean, variance, scale, bias, epsilon, out, vec);
    TSX_LAUNCH_CHECK("channel_affine_kernel");
    return 0;
}

// out = lhs + rhs (MUL: lhs * rhs) with numpy-style broadcasting over up to 8 aligned axes (an extent of 1 repeats).
// One lane per output element; an operand's stride is 0 on the axes it is broadcast along.
struct BroadcastGeom {
    int out_shape[8];   // right-aligned; leading unused axes have extent 1
    int64_t lhs_stride[8], rhs_stride[8];
};

template <bool MUL>
__global__ __launch_bounds__(256) void broadcast_kernel(const float *__restrict__ lhs, const float *__restrict__ rhs,
                                                           BroadcastGeom g, int64_t count, float *__restrict__ out) {
    const int64_t stride = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride) {
        int64_t rest = i, lo = 0, ro = 0;
#pragma unroll
        for (int d = 7; d >= 0; --d) {
            const int64_t q = rest / g.out_shape[d];
            const int c = int(rest - q * g.out_shape[d]);
            rest = q;
            lo += c * g.lhs_stride[d];
            ro += c * g.rhs_stride[d];
        }
        out[i] = MUL ? __fmul_rn(lhs[lo], rhs[ro]) : __fadd_rn(lhs[lo], rhs[ro]);
    }
}

template <bool MUL>
int launch_broadcast(const char *who, const float *lhs_dev, const int32_t *lhs_shape, const float *rhs_dev, const int32_t *rhs_shape,
                     int32_t dims, float *out_dev, void *stream) {
    TSX_REQUIRE(dims >= 1 && dims <= 8 && lhs_shape && rhs_shape, "%s: 1..8 axes, got %d", who, dims);
    BroadcastGeom g{};
    for (int d = 0; d < 8; ++d) g.out_shape[d] = 1;
    int64_t count = 1, ls = 1, rs = 1;
    for (int d = dims - 1; d >= 0; --d) {
        const int l = lhs_shape[d], r = rhs_shape[d];
        TSX_REQUIRE(l >= 0 && r >= 0 && (l == r || l == 1 || r == 1), "%s: axis %d: %d vs %d", who, d, l, r);
        const int slot = d + 8 - dims;
        g.out_shape[slot] = l == 1 ? r : l;
        g.lhs_stride[slot] = l == 1 ? 0 : ls;
        g.rhs_stride[slot] = r == 1 ? 0 : rs;
        ls *= l;
        rs *= r;
        count *= g.out_shape[slot];
    }
    if (count == 0) return 0;
    TSX_REQUIRE(lhs_dev && rhs_dev && out_dev, "%s: null pointer", who);
    const int64_t blocks = (count + 255) / 256;
    hipLaunchKernelGGL(broadcast_kernel<MUL>, dim3(unsigned(blocks < 8192 ? blocks : 8192)), dim3(256), 0, tsx::as_stream(stream),
                       lhs_dev, rhs_dev, g, count, out_dev);
    TSX_LAUNCH_CHECK("broadcast_kernel");
    return 0;
}

}  // namespace

extern "C" {

int tsx_add_bias_f32(const float *x_dev, int64_t pre, int32_t channels, int64_t inner, const float *bias_dev,
                     float *out_dev, void *stream) {
    TSX_REQUIRE(pre >= 0 && channels > 0 && inner > 0 && bias_dev, "add_bias: bad argument");
    return launch<0>(x_dev, pre * channels * inner, bias_dev, channels, inner, 0.f, out_dev, stream);
}

int tsx_batch_norm_f32(const float *x_dev, int64_t pre, int32_t channels, int64_t inner, const float *mean_dev,
                       const float *variance_dev, float epsilon, float *out_dev, void *stream) {
    return launch_affine<1>("batch_norm", x_dev, pre, channels, inner, mean_dev, variance_dev, nullptr, nullptr, epsilon,
                            out_dev, stream);
}

int tsx_batch_scale_f32(const float *x_dev, int64_t pre, int32_t channels, int64_t inner, const float *scale_dev,
                        const float *bias_dev, float *out_dev, void *stream) {
    return launch_affine<0>("batch_scale", x_dev, pre, channels, inner, nullptr, nullptr, scale_dev, bias_dev, 0.f, out_dev,
                            stream);
}

int tsx_fused_batch_norm_f32(const float *x_dev, int64_t pre, int32_t channels, int64_t inner, const float *mean_dev,
                             const float *variance_dev, const float *scale_dev, const float *bias_dev, float epsilon,
                             float *out_dev, void *stream) {
    return launch_affine<2>("fused_batch_norm", x_dev, pre, channels, inner, mean_dev, variance_dev, scale_dev, bias_dev,
                            epsilon, out_dev, stream);
}

int tsx_relu_f32(const float *x_dev, int64_t count, float *out_dev, void *stream) {
    TSX_REQUIRE(count >= 0, "relu: negative count");
    return launch<1>(x_dev, count, nullptr, 1, 1, 0.f, out_dev, stream);
}

int tsx_leaky_relu_f32(const float *x_dev, int64_t count, float scale, float *out_dev, void *stream) {
    TSX_REQUIRE(count >= 0, "leaky_relu: negative count");
    return launch<2>(x_dev, count, nullptr, 1, 1, scale, out_dev, stream);
}

int tsx_add_f32(const float *a_dev, const float *b_dev, int64_t count, int32_t act, float slope, float *out_dev,
                void *stream) {
    TSX_REQUIRE(count >= 0 && (count == 0 || b_dev), "add: bad argument");
    TSX_REQUIRE(act >= TSX_ACT_NONE && act <= TSX_ACT_MISH_FAST, "add: unknown activation %d", act);
    return launch<3>(a_dev, count, b_dev, 1, 1, slope, out_dev, stream, act);
}

int tsx_add_broadcast_f32(const float *lhs_dev, const int32_t *lhs_shape, const float *rhs_dev, const int32_t *rhs_shape,
                          int32_t dims, float *out_dev, void *stream) {
    return launch_broadcast<false>("add_broadcast", lhs_dev, lhs_shape, rhs_dev, rhs_shape, dims, out_dev, stream);
}

int tsx_mul_f32(const float *a_dev, const float *b_dev, int64_t count, float *out_dev, void *stream) {
    TSX_REQUIRE(count >= 0 && (count == 0 || b_dev), "mul: bad argument");
    return launch<7>(a_dev, count, b_dev, 1, 1, 0.f, out_dev, stream);
}

int tsx_mul_broadcast_f32(const float *lhs_dev, const int32_t *lhs_shape, const float *rhs_dev, const int32_t *rhs_shape,
                          int32_t dims, float *out_dev, void *stream) {
    return launch_broadcast<true>("mul_broadcast", lhs_dev, lhs_shape, rhs_dev, rhs_shape, dims, out_dev, stream);
}

int tsx_softplus_f32(const float *x_dev, int64_t count, float *out_dev, void *stream) {
    TSX_REQUIRE(count >= 0, "softplus: negative count");
    return launch<5>(x_dev, count, nullptr, 1, 1, 0.f, out_dev, stream);
}

int tsx_tanh_f32(const float *x_dev, int64_t count, float *out_dev, void *stream) {
    TSX_REQUIRE(count >= 0, "tanh: negative count");
    return launch<6>(x_dev, count, nullptr, 1, 1, 0.f, out_dev, stream);
}

int tsx_mish_f32(const float *x_dev, int64_t count, float *out_dev, void *stream) {
    TSX_REQUIRE(count >= 0, "mish: negative count");
    return launch<4>(x_dev, count, nullptr, 1, 1, 0.f, out_dev, stream);
}

}  // extern "C"
