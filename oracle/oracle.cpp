// TEST INFRASTRUCTURE ONLY -- a CPU restatement of the TenniS reference's
// convolution hot path, used as the parity checker for the HIP kernels and as
// the "port" CPU baseline.  Nothing in the shipped product path (tennis_amd/,
// include/) links, loads or calls this file; only tests/, __graft_entry__.smoke()
// and bench.py's cpu_baseline leg do.
//
// Every function cites the reference file:line it restates (paths relative to
// the TenniS tree).  How each one is pinned (tests/test_oracle_*.py):
//   orc_quantize_f32      known-answer vectors of both rounding paths + compiled reference
//   orc_im2col_*          brute-force index formula on tiny inputs + compiled reference (via conv)
//   orc_gemm_i8           numpy int64 matmul (exact integers) + compiled reference
//   orc_conv2d_quantized  brute-force integer conv + closed-form float(acc)*dq + compiled reference
//   orc_add_bias/relu/leaky_relu  closed forms incl. signed-zero cases + compiled reference
//   orc_epilogue / orc_conv2d_i8_fused / orc_gemm_i8_dequant   composition of the above
//   orc_gemm_f32 / orc_conv2d_f32 / orc_inner_prod_f32  fp64 brute force (tolerance) +
//                         compiled reference (bit-exact, remainder paths included)
//   orc_winograd_f63 / orc_winograd_f23  fp64 direct conv (tolerance) + compiled reference (bit-exact)
//   orc_depthwise_conv2d_f32   fp64 brute force (tolerance) + compiled reference depthwise_conv2d (bit-exact on its
//                         general path, tolerance on its 3x3 SIMD paths)
//   orc_resize_nearest_f32     index closed form + compiled reference resize2d (bit-exact: a copy)
//   orc_softplus/tanh/mish     closed forms in fp64 (tolerance) + compiled reference softplus, tanh, mul (bit-exact)
//   orc_add_f32 / orc_pooling2d_f32      numpy closed forms (max / mean of clipped windows) + compiled
//                         reference operators add, pooling2d, global_pooling2d (bit-exact)
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>
#include <immintrin.h>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

int g_threads = 1;

inline int out_size(int in, int pad_a, int pad_b, int k, int stride, int dilation) {
    // include/backend/common_function.h:30-40 (integer division inside std::floor)
    return (in + pad_a + pad_b - (dilation * (k - 1) + 1)) / stride + 1;
}

// x86 float->int32 conversions return INT_MIN ("integer indefinite") for NaN and
// out-of-range inputs; both of the reference's paths go through such a conversion.
inline int32_t cvt_rne(float v) { return _mm_cvtss_si32(_mm_set_ss(v)); }   // _mm256_cvtps_epi32 per lane
inline int32_t cvt_trunc(float v) { return _mm_cvttss_si32(_mm_set_ss(v)); } // int32_t(float)

inline int8_t clamp_i8(int32_t v) {
    // src/kernels/cpu/quantize.cpp:15-20
    if (v > 127) return 127;
    if (v < -128) return -128;
    return int8_t(v);
}

inline int8_t quant_half_away(float v) {
    // src/kernels/cpu/quantize.cpp:23-29: int32_t(round(src)) then clamp
    return clamp_i8(cvt_trunc(std::round(v)));
}

inline int8_t quant_rne(float v) {
    // src/kernels/cpu/quantize.cpp:83-96 via simd_avx_def.h:273-275
    return clamp_i8(cvt_rne(v));
}

inline float relu_body(float v) {
    // _mm_max_ps(x, 0): returns the second operand when x is NaN or both are zero
    // (src/kernels/cpu/relu.cpp:39-46)
    return v > 0.f ? v : 0.f;
}

inline float relu_tail(float v) {
    // std::max(val, 0.f) == (val < 0.f) ? 0.f : val  (src/kernels/cpu/relu.cpp:47-51)
    return v < 0.f ? 0.f : v;
}

inline float min_body(float v) { return v < 0.f ? v : 0.f; }  // _mm_min_ps(x, 0)

}  // namespace

extern "C" {

void orc_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int orc_get_max_threads() {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

// ---------------------------------------------------------------------------
// quantize: src/kernels/cpu/quantize.cpp:70-125 (+ base_quantize.cpp:26: len(scales)==x.sizes()[0])
//   nscales == 1: first 8*floor(count/8) elements round-half-even, tail half-away;
//   nscales  > 1: group g owns the next ceil(count/nscales) elements, all half-away.
// ---------------------------------------------------------------------------
void orc_quantize_f32(const float *x, int64_t count, const float *scales, int nscales, int8_t *out) {
    if (nscales == 1) {
        const float s = scales[0];
        const int64_t bulk = (count >> 3) << 3;
#pragma omp parallel for num_threads(g_threads)
        for (int64_t i = 0; i < bulk; ++i) out[i] = quant_rne(x[i] * s);
        for (int64_t i = bulk; i < count; ++i) out[i] = quant_half_away(x[i] * s);
        return;
    }
    const int64_t loop = int64_t(std::ceil(float(count) / float(nscales)));
    int64_t index = 0;
    for (int g = 0; g < nscales; ++g) {
        const float s = scales[g];
        for (int64_t left = loop; index < count && left; --left, ++index) out[index] = quant_half_away(x[index] * s);
    }
}

// ---------------------------------------------------------------------------
// im2col: src/kernels/cpu/im2col.cpp:37-111
//   col[(c*KH+kh)*KW+kw][ho*Wo+wo] = im[c][ho*sh-pt+kh*dh][wo*sw-pl+kw*dw] or padding_value
// ---------------------------------------------------------------------------
#define ORC_IM2COL(NAME, T)                                                                               \
    void NAME(const T *im, int c, int h, int w, int kh, int kw, int pt, int pb, int pl, int pr, int sh,  \
              int sw, int dh, int dw, T *col, T padding_value) {                                         \
        const int ho = out_size(h, pt, pb, kh, sh, dh), wo = out_size(w, pl, pr, kw, sw, dw);            \
        _Pragma("omp parallel for num_threads(g_threads)") for (int ch = 0; ch < c; ++ch) {              \
            T *dst = col + int64_t(ch) * kh * kw * ho * wo;                                              \
            const T *src = im + int64_t(ch) * h * w;                                                     \
            for (int r = 0; r < kh; ++r)                                                                  \
                for (int s = 0; s < kw; ++s)                                                              \
                    for (int y = 0; y < ho; ++y) {                                                        \
                        const int iy = y * sh - pt + r * dh;                                              \
                        for (int xo = 0; xo < wo; ++xo) {                                                 \
                            const int ix = xo * sw - pl + s * dw;                                         \
                            const bool in = iy >= 0 && iy < h && ix >= 0 && ix < w;                       \
                            *dst++ = in ? src[iy * w + ix] : padding_value;                               \
                        }                                                                                 \
                    }                                                                                     \
        }                                                                                                 \
    }
ORC_IM2COL(orc_im2col_i8, int8_t)
ORC_IM2COL(orc_im2col_f32, float)

// ---------------------------------------------------------------------------
// int8 GEMM, int32 accumulate: src/kernels/cpu/math_cpu.cpp:30-46,143-210,238-244
//   C[M][N] = A[M][K] * B[K][N], row-major, alpha=1, beta=0.  Integer sums are
//   order-independent, so the restatement may pick any loop order:
//   faithful != 0 : the reference's order -- one strided dot per output, single thread;
//   faithful == 0 : i-k-j order, OpenMP over rows (same integers, far faster).
// ---------------------------------------------------------------------------
void orc_gemm_i8(int m, int n, int k, const int8_t *a, const int8_t *b, int32_t *c, int faithful) {
    if (faithful) {
        for (int i = 0; i < m; ++i)
            for (int j = 0; j < n; ++j) {
                int32_t sum = 0;
                const int8_t *x = a + int64_t(i) * k;
                const int8_t *y = b + j;
                for (int kk = 0; kk < k; ++kk, y += n) sum += int32_t(x[kk]) * int32_t(*y);
                c[int64_t(i) * n + j] = sum;
            }
        return;
    }
#pragma omp parallel for num_threads(g_threads)
    for (int i = 0; i < m; ++i) {
        int32_t *row = c + int64_t(i) * n;
        std::memset(row, 0, sizeof(int32_t) * size_t(n));
        for (int kk = 0; kk < k; ++kk) {
            const int32_t av = a[int64_t(i) * k + kk];
            if (av == 0) continue;
            const int8_t *br = b + int64_t(kk) * n;
            for (int j = 0; j < n; ++j) row[j] += av * int32_t(br[j]);
        }
    }
}

// ---------------------------------------------------------------------------
// conv2d_quantized: src/kernels/cpu/quantized/conv2d_quantized_core.cpp:18-126
//   per image: im2col<int8> (skipped for 1x1/s1/p0), int8 GEMM into an INT32
//   scratch, then out = float(acc) * dq[c].  acc_out (optional) receives the int32
//   accumulators.  The reference's dequant loop is only correct single-threaded;
//   this is its single-threaded result.
// ---------------------------------------------------------------------------
void orc_conv2d_quantized(const int8_t *x, int n, int c, int h, int w, const int8_t *wt, int cout, int kh,
                          int kw, int pt, int pb, int pl, int pr, int sh, int sw, int dh, int dw,
                          float padding_value, const float *dq, float *out, int32_t *acc_out, int faithful) {
    const int ho = out_size(h, pt, pb, kh, sh, dh), wo = out_size(w, pl, pr, kw, sw, dw);
    const int hw = ho * wo, kdim = c * kh * kw;
    const bool is_1x1 = sh == 1 && sw == 1 && kh == 1 && kw == 1 && !pt && !pb && !pl && !pr;
    std::vector<int8_t> col(is_1x1 ? 0 : size_t(kdim) * hw);
    std::vector<int32_t> acc_local;
    int32_t *acc = acc_out;
    if (!acc) {
        acc_local.resize(size_t(n) * cout * hw);
        acc = acc_local.data();
    }
    for (int i = 0; i < n; ++i) {
        const int8_t *xi = x + int64_t(i) * c * h * w;
        const int8_t *bmat = xi;
        if (!is_1x1) {
            orc_im2col_i8(xi, c, h, w, kh, kw, pt, pb, pl, pr, sh, sw, dh, dw, col.data(), int8_t(padding_value));
            bmat = col.data();
        }
        orc_gemm_i8(cout, hw, kdim, wt, bmat, acc + int64_t(i) * cout * hw, faithful);
    }
    if (out) {
        const int64_t total = int64_t(n) * cout * hw;
#pragma omp parallel for num_threads(g_threads)
        for (int64_t idx = 0; idx < total; ++idx) out[idx] = float(acc[idx]) * dq[(idx / hw) % cout];
    }
}

// ---------------------------------------------------------------------------
// add_bias / relu / leaky_relu: src/kernels/cpu/add_bias.cpp:47-85, relu.cpp:30-52,
// leaky_relu.cpp:41-66.  relu/leaky use a 4-wide SIMD body over the first
// 4*floor(count/4) elements of the whole tensor and a scalar tail; the two differ in
// the sign of zero and in NaN handling, which is restated here.
// ---------------------------------------------------------------------------
void orc_add_bias_f32(const float *x, int64_t pre, int channels, int64_t inner, const float *bias, float *out) {
    const int64_t total = pre * channels * inner;
#pragma omp parallel for num_threads(g_threads)
    for (int64_t i = 0; i < total; ++i) out[i] = x[i] + bias[(i / inner) % channels];
}

// ---------------------------------------------------------------------------
// batch_norm / batch_scale / fused_batch_norm on fp32, layout [pre][channels][inner]:
// src/kernels/cpu/batch_norm.cpp:61-105, batch_scale.cpp:57-97, fused_batch_norm.cpp:70-125.
// The reciprocal standard deviation is float(1) / sqrt(var + float(eps)) with the sum in float and the
// unqualified sqrt taking it as a double: root and quotient are computed in double and rounded to float once.
// x * scale + bias is one fused multiply-add in the reference's FMA build, in its 4-wide body and in its
// scalar tail alike (gcc contracts both); (x - mean) * inv has nothing to contract.
// ---------------------------------------------------------------------------
static inline float inv_std(float variance, float epsilon) {
    const float sum = variance + epsilon;
    return float(1.0 / std::sqrt(double(sum)));
}

void orc_batch_norm_f32(const float *x, int64_t pre, int channels, int64_t inner, const float *mean,
                        const float *variance, float epsilon, float *out) {
    const int64_t total = pre * channels * inner;
#pragma omp parallel for num_threads(g_threads)
    for (int64_t i = 0; i < total; ++i) {
        const int c = int((i / inner) % channels);
        out[i] = (x[i] - mean[c]) * inv_std(variance[c], epsilon);
    }
}

void orc_batch_scale_f32(const float *x, int64_t pre, int channels, int64_t inner, const float *scale,
                         const float *bias, float *out) {
    const int64_t total = pre * channels * inner;
#pragma omp parallel for num_threads(g_threads)
    for (int64_t i = 0; i < total; ++i) {
        const int c = int((i / inner) % channels);
        out[i] = std::fmaf(x[i], scale[c], bias[c]);
    }
}

void orc_fused_batch_norm_f32(const float *x, int64_t pre, int channels, int64_t inner, const float *mean,
                              const float *variance, const float *scale, const float *bias, float epsilon, float *out) {
    const int64_t total = pre * channels * inner;
#pragma omp parallel for num_threads(g_threads)
    for (int64_t i = 0; i < total; ++i) {
        const int c = int((i / inner) % channels);
        const float t = (x[i] - mean[c]) * inv_std(variance[c], epsilon);
        out[i] = std::fmaf(t, scale[c], bias[c]);
    }
}

void orc_relu_f32(const float *x, int64_t count, float *out) {
    const int64_t body = count / 4 * 4;
#pragma omp parallel for num_threads(g_threads)
    for (int64_t i = 0; i < count; ++i) out[i] = i < body ? relu_body(x[i]) : relu_tail(x[i]);
}

void orc_leaky_relu_f32(const float *x, int64_t count, float scale, float *out) {
    const int64_t body = count / 4 * 4;
#pragma omp parallel for num_threads(g_threads)
    for (int64_t i = 0; i < count; ++i) {
        const float v = x[i];
        if (i < body) {
            // max(x,0) + scale*min(x,0).  The reference's AVX2/FMA build contracts the
            // intrinsic multiply and add into one fused multiply-add (gcc -O3 -mfma,
            // default -ffp-contract=fast); it shows when scale*x underflows: the
            // result keeps the sign of x (-0.0) instead of 0 + (-0.0) = +0.0.
            out[i] = std::fmaf(scale, min_body(v), relu_body(v));
        } else {
            out[i] = v > 0.f ? v : v * scale;
        }
    }
}

// ---------------------------------------------------------------------------
// Fused epilogue = the reference's operator chain applied to the fp32 tensor
//   y0 = float(acc) * dq[c]                 (conv2d_quantized_core.cpp:81-106)
//   y1 = y0 + bias[c]     if bias           (add_bias.cpp:47-85)
//   y2 = act(y1)          act: 0 none, 1 relu, 2 leaky_relu(slope)
//   q  = quantize(y2)     if q_out          (quantize.cpp:70-125; requant for the next layer)
// Each step is a separately rounded fp32 operation, exactly as separate operators.
// Layout [pre][channels][inner] (NCHW: pre=N, inner=H*W; GEMM rows: channels=N, inner=1).
// ---------------------------------------------------------------------------
void orc_epilogue(const int32_t *acc, int64_t pre, int channels, int64_t inner, const float *dq,
                  const float *row_scale, const float *bias, int act, float slope, float *out_f32,
                  const float *q_scales, int n_qscales, int8_t *q_out) {
    const int64_t total = pre * channels * inner;
    std::vector<float> tmp(out_f32 ? 0 : size_t(total));
    float *y = out_f32 ? out_f32 : tmp.data();
#pragma omp parallel for num_threads(g_threads)
    for (int64_t i = 0; i < total; ++i) {
        const int ch = int((i / inner) % channels);
        volatile float v = float(acc[i]) * dq[ch];
        if (row_scale) v = v * row_scale[i / (inner * channels)];
        if (bias) v = v + bias[ch];
        y[i] = v;
    }
    if (act == 1) orc_relu_f32(y, total, y);
    if (act == 2) orc_leaky_relu_f32(y, total, slope, y);
    if (q_out) orc_quantize_f32(y, total, q_scales, n_qscales, q_out);
}

// conv2d_quantized -> add_bias -> relu/leaky -> (quantize) as one call.
void orc_conv2d_i8_fused(const int8_t *x, int n, int c, int h, int w, const int8_t *wt, int cout, int kh, int kw,
                         int pt, int pb, int pl, int pr, int sh, int sw, int dh, int dw, float padding_value,
                         const float *dq, const float *bias, int act, float slope, float *out_f32,
                         const float *q_scales, int n_qscales, int8_t *q_out) {
    const int ho = out_size(h, pt, pb, kh, sh, dh), wo = out_size(w, pl, pr, kw, sw, dw);
    std::vector<int32_t> acc(size_t(n) * cout * ho * wo);
    orc_conv2d_quantized(x, n, c, h, w, wt, cout, kh, kw, pt, pb, pl, pr, sh, sw, dh, dw, padding_value, dq,
                         nullptr, acc.data(), 0);
    orc_epilogue(acc.data(), n, cout, int64_t(ho) * wo, dq, nullptr, bias, act, slope, out_f32, q_scales,
                 n_qscales, q_out);
}

// Quantized inner product (no reference operator; defined by composition of
// math<int8,int32>::gemm, the conv2d_quantized dequant form, a broadcast mul and add_bias):
//   out[m][n] = ((float(acc[m][n]) * dq_w[n]) * dq_a[m]) + bias[n]
void orc_gemm_i8_dequant(int m, int n, int k, const int8_t *a, const int8_t *b, const float *dq_w,
                         const float *dq_a, const float *bias, float *out, int32_t *acc_out) {
    std::vector<int32_t> acc_local;
    int32_t *acc = acc_out;
    if (!acc) {
        acc_local.resize(size_t(m) * n);
        acc = acc_local.data();
    }
    orc_gemm_i8(m, n, k, a, b, acc, 0);
    orc_epilogue(acc, m, n, 1, dq_w, dq_a, bias, 0, 0.f, out, nullptr, 0, nullptr);
}

// ---------------------------------------------------------------------------
// fp32 GEMM: src/kernels/cpu/math_cpu.cpp:247-292 (pack8_A), :338-373 (pack8_B),
// :386-700 (kernel_8x8), :717-743.  Packing only permutes storage; the arithmetic
// per output element C[i][j] (8-row blocks i < M8, 8-col blocks j < N8) is:
//   i <  M8, j <  N8 : one FMA chain, k ascending, from 0
//   i <  M8, j >= N8 : 4 interleaved FMA chains (k mod 4), (s0+s1),(s2+s3), 0+s01, +s23, then FMA tail
//   i >= M8, j <  N8 : one FMA chain, k ascending
//   i >= M8, j >= N8 : 4 interleaved FMA chains, horizontal sum, then scalar tail
// ---------------------------------------------------------------------------
static float hsum4(const float s[4]) {
    // ts::sum(simd<T,4>): a[0] + a[1] + a[2] + a[3], left to right (include/kernels/common/simd.h:54-59)
    return ((s[0] + s[1]) + s[2]) + s[3];
}

void orc_gemm_f32(int m, int n, int k, const float *a, const float *b, float *c) {
    const int m8 = m / 8 * 8, n8 = n / 8 * 8, k4 = k / 4 * 4;
#pragma omp parallel for num_threads(g_threads)
    for (int i = 0; i < m; ++i) {
        const float *ar = a + int64_t(i) * k;
        for (int j = 0; j < n; ++j) {
            float r;
            if (j < n8) {
                float acc = 0.f;
                for (int kk = 0; kk < k; ++kk) acc = std::fmaf(b[int64_t(kk) * n + j], ar[kk], acc);
                r = acc;
            } else if (i < m8) {
                float s[4] = {0.f, 0.f, 0.f, 0.f};
                for (int kk = 0; kk < k4; ++kk) s[kk & 3] = std::fmaf(ar[kk], b[int64_t(kk) * n + j], s[kk & 3]);
                volatile float s01 = s[0] + s[1];
                volatile float s23 = s[2] + s[3];
                float acc = 0.f;
                acc += s01;
                acc += s23;
                for (int kk = k4; kk < k; ++kk) acc = std::fmaf(ar[kk], b[int64_t(kk) * n + j], acc);
                r = acc;
            } else {
                float s[4] = {0.f, 0.f, 0.f, 0.f};
                for (int kk = 0; kk < k4; ++kk) s[kk & 3] = std::fmaf(ar[kk], b[int64_t(kk) * n + j], s[kk & 3]);
                float acc = hsum4(s);
                for (int kk = k4; kk < k; ++kk) acc = std::fmaf(ar[kk], b[int64_t(kk) * n + j], acc);
                r = acc;
            }
            c[int64_t(i) * n + j] = r;
        }
    }
}

// fp32 conv2d: src/kernels/cpu/conv2d_core.cpp:17-119 -- per image im2col + the GEMM above
// with M=Cout, N=Ho*Wo, K=Cin*KH*KW.
void orc_conv2d_f32(const float *x, int n, int c, int h, int w, const float *wt, int cout, int kh, int kw,
                    int pt, int pb, int pl, int pr, int sh, int sw, int dh, int dw, float padding_value,
                    float *out) {
    const int ho = out_size(h, pt, pb, kh, sh, dh), wo = out_size(w, pl, pr, kw, sw, dw);
    const int hw = ho * wo, kdim = c * kh * kw;
    const bool is_1x1 = sh == 1 && sw == 1 && kh == 1 && kw == 1 && !pt && !pb && !pl && !pr;
    std::vector<float> col(is_1x1 ? 0 : size_t(kdim) * hw);
    for (int i = 0; i < n; ++i) {
        const float *xi = x + int64_t(i) * c * h * w;
        const float *bmat = xi;
        if (!is_1x1) {
            orc_im2col_f32(xi, c, h, w, kh, kw, pt, pb, pl, pr, sh, sw, dh, dw, col.data(), padding_value);
            bmat = col.data();
        }
        orc_gemm_f32(cout, hw, kdim, wt, bmat, out + int64_t(i) * cout * hw);
    }
}

// inner_prod: src/backend/base/base_inner_prod.cpp:26-93, src/kernels/cpu/inner_prod.cpp:19-74
//   out[M][N] = lhs[M][K] * rhs (rhs is [K][N], or [N][K] when transpose) through the GEMM above.
void orc_inner_prod_f32(const float *lhs, int m, int k, const float *rhs, int n, int transpose, float *out) {
    if (!transpose) {
        orc_gemm_f32(m, n, k, lhs, rhs, out);
        return;
    }
    std::vector<float> t(size_t(k) * n);
    for (int j = 0; j < n; ++j)
        for (int kk = 0; kk < k; ++kk) t[size_t(kk) * n + j] = rhs[size_t(j) * k + kk];
    orc_gemm_f32(m, n, k, lhs, t.data(), out);
}

// ---------------------------------------------------------------------------
// Winograd F(6,3): src/kernels/cpu/winograd_algorithm.cpp:504-947 with the padding rule
// of src/kernels/common/function.cpp:14-78 (output rounded up to a multiple of 6, input
// padded bottom/right with padding_value to out_padded+2, result cut back).
//   U = G g G^T (kernel, :504-566), V = B^T d B (input, :607-699), M_t = U_t V_t (64 GEMMs
//   Cout x Cin x tiles through the fp32 GEMM above, :917-936), Y = A^T M A (:738-833).
// The reference writes the transforms as plain float expressions and is built with gcc -O3 -mfma,
// whose default -ffp-contract=fast turns a*b+c patterns into fused multiply-adds; that choice
// is part of the reference's numerics (F(6,3) amplifies single roundings to ~1e-5).  The fused
// forms are written out explicitly here -- in `a*c1 - b*c2 [+ ...]` gcc fuses the FIRST product
// and rounds the second -- and this file is compiled with -ffp-contract=off, so the result no
// longer depends on the compiler.  Checked bit for bit against the compiled reference.
// ---------------------------------------------------------------------------
static void wino_f63_kernel(const float *g, float u[64]) {
    static const float G[8][3] = {{1.0f, 0.0f, 0.0f},
                                  {-2.f / 9, -2.f / 9, -2.f / 9},
                                  {-2.f / 9, 2.f / 9, -2.f / 9},
                                  {1.f / 90, 1.f / 45, 2.f / 45},
                                  {1.f / 90, -1.f / 45, 2.f / 45},
                                  {1.f / 45, 1.f / 90, 1.f / 180},
                                  {1.f / 45, -1.f / 90, 1.f / 180},
                                  {0.0f, 0.0f, 1.0f}};
    float tmp[3][8];
    for (int i = 0; i < 8; ++i)
        for (int r = 0; r < 3; ++r)
            tmp[r][i] = std::fmaf(g[r * 3 + 2], G[i][2], std::fmaf(g[r * 3 + 0], G[i][0], g[r * 3 + 1] * G[i][1]));
    for (int i = 0; i < 8; ++i)
        for (int j = 0; j < 8; ++j) u[i * 8 + j] = std::fmaf(tmp[2][j], G[i][2], std::fmaf(tmp[0][j], G[i][0], tmp[1][j] * G[i][1]));
}

static inline void wino_f63_bt(const float i0[8], float o[8]) {
    o[0] = std::fmaf(i0[4] - i0[2], 5.25f, i0[0] - i0[6]);
    o[7] = std::fmaf(i0[3] - i0[5], 5.25f, i0[7] - i0[1]);
    float tmp12_a = std::fmaf(-i0[4], 4.25f, i0[2] + i0[6]);
    float tmp12_b = std::fmaf(-i0[3], 4.25f, i0[1] + i0[5]);
    o[1] = tmp12_a + tmp12_b;
    o[2] = tmp12_a - tmp12_b;
    float tmp34_a = std::fmaf(-i0[4], 1.25f, std::fmaf(i0[2], 0.25f, i0[6]));
    float tmp34_b = std::fmaf(i0[5], 2.f, std::fmaf(i0[1], 0.5f, -(i0[3] * 2.5f)));
    o[3] = tmp34_a + tmp34_b;
    o[4] = tmp34_a - tmp34_b;
    float tmp56_a = std::fmaf(std::fmaf(-i0[4], 1.25f, i0[2]), 4.f, i0[6]);
    float tmp56_b = std::fmaf(i0[5], 0.5f, std::fmaf(i0[1], 2.f, -(i0[3] * 2.5f)));
    o[5] = tmp56_a + tmp56_b;
    o[6] = tmp56_a - tmp56_b;
}

static inline void wino_f63_bt_col(const float d[8], float o[8]) {
    o[0] = std::fmaf(d[4] - d[2], 5.25f, d[0] - d[6]);
    o[7] = std::fmaf(d[3] - d[5], 5.25f, d[7] - d[1]);
    float tmp12_a = std::fmaf(-d[4], 4.25f, d[2] + d[6]);
    float tmp12_b = std::fmaf(-d[3], 4.25f, d[1]) + d[5];
    o[1] = tmp12_a + tmp12_b;
    o[2] = tmp12_a - tmp12_b;
    float tmp34_a = std::fmaf(-d[4], 1.25f, std::fmaf(d[2], 0.25f, d[6]));
    float tmp34_b = std::fmaf(d[5], 2.f, std::fmaf(d[1], 0.5f, -(d[3] * 2.5f)));
    o[3] = tmp34_a + tmp34_b;
    o[4] = tmp34_a - tmp34_b;
    float tmp56_a = std::fmaf(std::fmaf(-d[4], 1.25f, d[2]), 4.f, d[6]);
    float tmp56_b = std::fmaf(d[5], 0.5f, std::fmaf(d[1], 2.f, -(d[3] * 2.5f)));
    o[5] = tmp56_a + tmp56_b;
    o[6] = tmp56_a - tmp56_b;
}

static inline void wino_f63_at(const float t[8], float o[6]) {
    float re0 = t[1] + t[2];
    float re1 = t[1] - t[2];
    float re2 = t[3] + t[4];
    float re3 = t[3] - t[4];
    float re4 = t[5] + t[6];
    float re5 = t[5] - t[6];
    o[0] = t[0] + re0 + re2 + re4 * 32.f;
    o[1] = re1 + re3 + re3 + re5 * 16.f;
    o[2] = re0 + re2 * 4 + re4 * 8.f;
    o[3] = re1 + re3 * 8 + re5 * 4.f;
    o[4] = re0 + re2 * 16 + re4 + re4;
    o[5] = re1 + re3 * 32 + re5 + t[7];
}

void orc_winograd_f63(const float *x, int n, int c, int h, int w, const float *wt, int cout, int pt, int pb,
                      int pl, int pr, float padding_value, float *out) {
    const int ho = h + pt + pb - 2, wo = w + pl + pr - 2;
    const int hop = (ho + 5) / 6 * 6, wop = (wo + 5) / 6 * 6;
    const int hip = hop + 2, wip = wop + 2;
    const int th = hop / 6, tw = wop / 6, tiles = th * tw;

    // U: [64][Cout][Cin]
    std::vector<float> u(size_t(64) * cout * c);
#pragma omp parallel for num_threads(g_threads)
    for (int p = 0; p < cout; ++p)
        for (int q = 0; q < c; ++q) {
            float tmp[64];
            wino_f63_kernel(wt + (int64_t(p) * c + q) * 9, tmp);
            for (int t = 0; t < 64; ++t) u[(size_t(t) * cout + p) * c + q] = tmp[t];
        }

    std::vector<float> xp(size_t(c) * hip * wip);
    std::vector<float> v(size_t(64) * c * tiles);
    std::vector<float> mm(size_t(64) * cout * tiles);
    std::vector<float> yp(size_t(cout) * hop * wop);
    for (int img = 0; img < n; ++img) {
        // pad2d (src/kernels/cpu/pad2d_algorithm.cpp:89-160): top/left = conv padding, rest to fit
        std::fill(xp.begin(), xp.end(), padding_value);
        for (int ch = 0; ch < c; ++ch)
            for (int y = 0; y < h; ++y)
                std::memcpy(&xp[(size_t(ch) * hip + y + pt) * wip + pl], x + ((int64_t(img) * c + ch) * h + y) * w,
                            sizeof(float) * size_t(w));
        // V: [64][Cin][tiles]
#pragma omp parallel for num_threads(g_threads)
        for (int ch = 0; ch < c; ++ch)
            for (int ty = 0; ty < th; ++ty)
                for (int tx = 0; tx < tw; ++tx) {
                    const float *src = &xp[(size_t(ch) * hip + ty * 6) * wip + tx * 6];
                    float db[8][8];
                    for (int i = 0; i < 8; ++i) wino_f63_bt(src + size_t(i) * wip, db[i]);
                    const int tile = ty * tw + tx;
                    for (int i = 0; i < 8; ++i) {
                        float colv[8], o[8];
                        for (int r = 0; r < 8; ++r) colv[r] = db[r][i];
                        wino_f63_bt_col(colv, o);
                        // out_at[(8*r + i) * stride]: row r of B^T applied down the column
                        for (int r = 0; r < 8; ++r) v[(size_t(r * 8 + i) * c + ch) * tiles + tile] = o[r];
                    }
                }
        // 64 GEMMs: M_t[Cout][tiles] = U_t[Cout][Cin] * V_t[Cin][tiles]
        for (int t = 0; t < 64; ++t)
            orc_gemm_f32(cout, tiles, c, &u[size_t(t) * cout * c], &v[size_t(t) * c * tiles],
                         &mm[size_t(t) * cout * tiles]);
        // Y = A^T M A per tile
#pragma omp parallel for num_threads(g_threads)
        for (int p = 0; p < cout; ++p)
            for (int ty = 0; ty < th; ++ty)
                for (int tx = 0; tx < tw; ++tx) {
                    const int tile = ty * tw + tx;
                    float tmpa[8][6];
                    for (int i = 0; i < 8; ++i) {
                        float t8[8];
                        for (int j = 0; j < 8; ++j) t8[j] = mm[(size_t(i * 8 + j) * cout + p) * tiles + tile];
                        wino_f63_at(t8, tmpa[i]);
                    }
                    for (int i = 0; i < 6; ++i) {
                        float t8[8], o[6];
                        for (int r = 0; r < 8; ++r) t8[r] = tmpa[r][i];
                        wino_f63_at(t8, o);
                        for (int r = 0; r < 6; ++r) yp[(size_t(p) * hop + ty * 6 + r) * wop + tx * 6 + i] = o[r];
                    }
                }
        // cut2d back to the true output size
        for (int p = 0; p < cout; ++p)
            for (int y = 0; y < ho; ++y)
                std::memcpy(out + ((int64_t(img) * cout + p) * ho + y) * wo, &yp[(size_t(p) * hop + y) * wop],
                            sizeof(float) * size_t(wo));
    }
}

// ---------------------------------------------------------------------------
// Winograd F(2,3): src/kernels/cpu/winograd_algorithm.cpp:57-459, the 4x4-tile twin of F(6,3)
// (output rounded up to a multiple of 2, 16 GEMMs).  B^T and A^T hold only 0/+-1, so those
// transforms are sums and differences written exactly as the reference groups them; the kernel
// transform G (4x3, entries 0, 1, +-1/2) has the same a*g0 + b*g1 + c*g2 shape as F(6,3)'s and
// is contracted by the reference's build the same way.
// ---------------------------------------------------------------------------
static void wino_f23_kernel(const float *g, float u[16]) {
    static const float G[4][3] = {{1.f, 0.f, 0.f}, {0.5f, 0.5f, 0.5f}, {0.5f, -0.5f, 0.5f}, {0.f, 0.f, 1.f}};
    float tmp[3][4];
    for (int i = 0; i < 4; ++i)
        for (int r = 0; r < 3; ++r)
            tmp[r][i] = std::fmaf(g[r * 3 + 2], G[i][2], std::fmaf(g[r * 3 + 0], G[i][0], g[r * 3 + 1] * G[i][1]));
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 4; ++j) u[i * 4 + j] = std::fmaf(tmp[2][j], G[i][2], std::fmaf(tmp[0][j], G[i][0], tmp[1][j] * G[i][1]));
}

void orc_winograd_f23(const float *x, int n, int c, int h, int w, const float *wt, int cout, int pt, int pb,
                      int pl, int pr, float padding_value, float *out) {
    const int ho = h + pt + pb - 2, wo = w + pl + pr - 2;
    const int hop = (ho + 1) / 2 * 2, wop = (wo + 1) / 2 * 2;
    const int hip = hop + 2, wip = wop + 2;
    const int th = hop / 2, tw = wop / 2, tiles = th * tw;

    std::vector<float> u(size_t(16) * cout * c);   // [16][Cout][Cin]
#pragma omp parallel for num_threads(g_threads)
    for (int p = 0; p < cout; ++p)
        for (int q = 0; q < c; ++q) {
            float tmp[16];
            wino_f23_kernel(wt + (int64_t(p) * c + q) * 9, tmp);
            for (int t = 0; t < 16; ++t) u[(size_t(t) * cout + p) * c + q] = tmp[t];
        }

    std::vector<float> xp(size_t(c) * hip * wip);
    std::vector<float> v(size_t(16) * c * tiles);
    std::vector<float> mm(size_t(16) * cout * tiles);
    std::vector<float> yp(size_t(cout) * hop * wop);
    for (int img = 0; img < n; ++img) {
        std::fill(xp.begin(), xp.end(), padding_value);
        for (int ch = 0; ch < c; ++ch)
            for (int y = 0; y < h; ++y)
                std::memcpy(&xp[(size_t(ch) * hip + y + pt) * wip + pl], x + ((int64_t(img) * c + ch) * h + y) * w,
                            sizeof(float) * size_t(w));
        // V = B^T d B (:181-243): rows first as (i_a -+ i_b), then the column combination
#pragma omp parallel for num_threads(g_threads)
        for (int ch = 0; ch < c; ++ch)
            for (int ty = 0; ty < th; ++ty)
                for (int tx = 0; tx < tw; ++tx) {
                    const float *i0 = &xp[(size_t(ch) * hip + ty * 2) * wip + tx * 2];
                    const float *i1 = i0 + wip, *i2 = i1 + wip, *i3 = i2 + wip;
                    float r[4][4];   // r[k][j]: row combination k at column j
                    for (int j = 0; j < 4; ++j) {
                        r[0][j] = i0[j] - i2[j];
                        r[1][j] = i1[j] + i2[j];
                        r[2][j] = i2[j] - i1[j];
                        r[3][j] = i1[j] - i3[j];
                    }
                    const int tile = ty * tw + tx;
                    for (int k = 0; k < 4; ++k) {
                        const float t[4] = {r[k][0] - r[k][2], r[k][1] + r[k][2], r[k][2] - r[k][1], r[k][1] - r[k][3]};
                        for (int j = 0; j < 4; ++j) v[(size_t(k * 4 + j) * c + ch) * tiles + tile] = t[j];
                    }
                }
        for (int t = 0; t < 16; ++t)
            orc_gemm_f32(cout, tiles, c, &u[size_t(t) * cout * c], &v[size_t(t) * c * tiles],
                         &mm[size_t(t) * cout * tiles]);
        // Y = A^T M A (:262-330)
#pragma omp parallel for num_threads(g_threads)
        for (int p = 0; p < cout; ++p)
            for (int ty = 0; ty < th; ++ty)
                for (int tx = 0; tx < tw; ++tx) {
                    const int tile = ty * tw + tx;
                    float m[16], a[8];
                    for (int t = 0; t < 16; ++t) m[t] = mm[(size_t(t) * cout + p) * tiles + tile];
                    for (int k = 0; k < 4; ++k) {
                        a[2 * k] = m[4 * k] + m[4 * k + 1] + m[4 * k + 2];
                        a[2 * k + 1] = m[4 * k + 1] - m[4 * k + 2] - m[4 * k + 3];
                    }
                    float *o = &yp[(size_t(p) * hop + ty * 2) * wop + tx * 2];
                    o[0] = a[0] + a[2] + a[4];
                    o[1] = a[1] + a[3] + a[5];
                    o[wop] = a[2] - a[4] - a[6];
                    o[wop + 1] = a[3] - a[5] - a[7];
                }
        for (int p = 0; p < cout; ++p)
            for (int y = 0; y < ho; ++y)
                std::memcpy(out + ((int64_t(img) * cout + p) * ho + y) * wo, &yp[(size_t(p) * hop + y) * wop],
                            sizeof(float) * size_t(wo));
    }
}

// ---------------------------------------------------------------------------
// Glue operators between convolutions in whole networks.
// ---------------------------------------------------------------------------

// cpu::Add on equal shapes (src/kernels/cpu/add.cpp: x = lhs + rhs per element).
void orc_add_f32(const float *a, const float *b, int64_t count, float *out) {
#pragma omp parallel for num_threads(g_threads)
    for (int64_t i = 0; i < count; ++i) out[i] = a[i] + b[i];
}

// cpu::Pooling2DCore (src/kernels/cpu/pooling2d_core.cpp:48-186), NCHW fp32.  Output size is the
// caller's (pooling2d_forward, include/backend/common_function.h:14-20: ceil).  The window is
// clipped to the image; MAX (type 0) starts from the first valid element; AVG (type 1) sums the
// valid elements in row-major order in fp32 and divides by their count (BLACK padding, white = 0)
// or by kh*kw (WHITE padding, white = 1).  planes = N*C.
void orc_pooling2d_f32(const float *x, int64_t planes, int h, int w, int type, int pt, int pl, int kh, int kw, int sh,
                       int sw, int white, float *out, int ho, int wo) {
#pragma omp parallel for num_threads(g_threads)
    for (int64_t pc = 0; pc < planes; ++pc) {
        const float *in = x + pc * h * w;
        float *o = out + pc * ho * wo;
        for (int oh = 0; oh < ho; ++oh) {
            int hs = oh * sh - pt;
            const int he = std::min(hs + kh, h);
            hs = std::max(hs, 0);
            for (int ow = 0; ow < wo; ++ow) {
                int ws = ow * sw - pl;
                const int we = std::min(ws + kw, w);
                ws = std::max(ws, 0);
                if (type == 0) {
                    float m = in[hs * w + ws];
                    for (int ih = hs; ih < he; ++ih)
                        for (int iw = ws; iw < we; ++iw)
                            if (in[ih * w + iw] > m) m = in[ih * w + iw];
                    o[oh * wo + ow] = m;
                } else {
                    float sum = 0.f;
                    int count = 0;
                    for (int ih = hs; ih < he; ++ih)
                        for (int iw = ws; iw < we; ++iw) {
                            sum += in[ih * w + iw];
                            ++count;
                        }
                    if (white) o[oh * wo + ow] = sum / float(kh * kw);
                    else o[oh * wo + ow] = count == 0 ? 0.f : sum / float(count);
                }
            }
        }
    }
}

// cpu::DepthwiseConv2dAlgorithm<float>::depthwise_general
// (src/kernels/cpu/depthwise_conv2d_algorithm.cpp:44-85): one filter per channel (multiplier 1),
// value += w * x over (kh, kw) in order, padding contributing w * padding_value; the reference's
// FMA build contracts each step to one fused multiply-add.  Its 3x3 stride-1/2 SIMD paths sum the
// same terms in another order and agree with this to fp32 rounding (tolerance, not bits).
void orc_depthwise_conv2d_f32(const float *x, int n, int c, int h, int w, const float *wt, int kh, int kw, int pt,
                              int pb, int pl, int pr, int sh, int sw, int dh, int dw, float padding_value, float *out) {
    // conv2d_forward (include/backend/common_function.h:30-40)
    const int ho = (h + pt + pb - (dh * (kh - 1) + 1)) / sh + 1, wo = (w + pl + pr - (dw * (kw - 1) + 1)) / sw + 1;
#pragma omp parallel for collapse(2) num_threads(g_threads)
    for (int ni = 0; ni < n; ++ni)
        for (int ci = 0; ci < c; ++ci) {
            const float *in = x + (int64_t(ni) * c + ci) * h * w;
            const float *k = wt + int64_t(ci) * kh * kw;
            float *o = out + (int64_t(ni) * c + ci) * ho * wo;
            for (int oh = 0; oh < ho; ++oh)
                for (int ow = 0; ow < wo; ++ow) {
                    float value = 0.f;
                    for (int i = 0; i < kh; ++i)
                        for (int j = 0; j < kw; ++j) {
                            const int hi = -pt + oh * sh + i * dh, wi = -pl + ow * sw + j * dw;
                            const float v = (hi >= 0 && hi < h && wi >= 0 && wi < w) ? in[hi * w + wi] : padding_value;
                            value = std::fmaf(k[i * kw + j], v, value);
                        }
                    o[oh * wo + ow] = value;
                }
        }
}

// Nearest-neighbour resize of [planes][h][w] (src/kernels/cpu/resize2d.cpp:186-215): source index
// round(scale * d + scale/2 - 0.5) in double, scale = src/dst, clamped to the image.
void orc_resize_nearest_f32(const float *x, int64_t planes, int h, int w, float *out, int ho, int wo) {
    const double sx = double(w) / wo, sy = double(h) / ho;
    const double bx = sx / 2 - 0.5, by = sy / 2 - 0.5;
#pragma omp parallel for num_threads(g_threads)
    for (int64_t p = 0; p < planes; ++p)
        for (int y = 0; y < ho; ++y)
            for (int xd = 0; xd < wo; ++xd) {
                int xs = int(std::round(sx * xd + bx)), ys = int(std::round(sy * y + by));
                xs = xs >= 0 ? xs : 0;
                xs = xs < w - 1 ? xs : w - 1;
                ys = ys >= 0 ? ys : 0;
                ys = ys < h - 1 ? ys : h - 1;
                out[(p * ho + y) * wo + xd] = (h == ho && w == wo) ? x[(p * h + y) * w + xd] : x[(p * h + ys) * w + xs];
            }
}

// Mish as TenniS graphs compose it: x * tanh(softplus(x)) with
//   softplus  y = float(log(double(expf(x)) + 1.0))        src/kernels/cpu/softplus.cpp:30-39
//   tanh      2 * (1 / (1 + expf(-2y))) - 1 in float         src/kernels/cpu/tanh.cpp:14-23
//   mul       x * t                                          src/kernels/cpu/mul.cpp
void orc_softplus_f32(const float *x, int64_t count, float *out) {
    for (int64_t i = 0; i < count; ++i) out[i] = static_cast<float>(std::log(std::exp(x[i]) + 1.));
}
void orc_tanh_f32(const float *x, int64_t count, float *out) {
    for (int64_t i = 0; i < count; ++i) out[i] = 2.f * (1.f / (1.f + std::exp(-(2.f * x[i])))) - 1.f;
}
void orc_mish_f32(const float *x, int64_t count, float *out) {
    for (int64_t i = 0; i < count; ++i) {
        const float sp = static_cast<float>(std::log(std::exp(x[i]) + 1.));
        const float t = 2.f * (1.f / (1.f + std::exp(-(2.f * sp)))) - 1.f;
        out[i] = x[i] * t;
    }
}

}  // extern "C"
