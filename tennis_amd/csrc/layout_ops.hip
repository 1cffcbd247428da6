// Copies between convolutions of detection-style graphs (HBM-bound: every byte read and written once):
//   concat on the channel axis     cpu::Concat   src/kernels/cpu/concat.cpp
//   nearest-neighbour resize       cpu::Resize2D src/kernels/cpu/resize2d.cpp:186-215
//   depthwise convolution          cpu::DepthwiseConv2D src/kernels/cpu/depthwise_conv2d_algorithm.cpp:44-85
#include "tsx_common.hpp"

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

// dst[n][c_offset + c][inner] = src[n][c][inner]; rows of c_src*inner floats are contiguous on both sides
__global__ __launch_bounds__(256) void concat_channels_kernel(const float *__restrict__ src, int64_t n, int64_t row,
                                                             float *__restrict__ dst, int64_t dst_row, int64_t dst_off,
                                                             bool vec) {
    const int64_t per = vec ? row / 4 : row;
    const int64_t total = n * per;
    for (int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; id < total; id += int64_t(gridDim.x) * blockDim.x) {
        const int64_t ni = id / per, e = id - ni * per;
        if (vec)
            *reinterpret_cast<v4f *>(dst + ni * dst_row + dst_off + e * 4) = *reinterpret_cast<const v4f *>(src + ni * row + e * 4);
        else
            dst[ni * dst_row + dst_off + e] = src[ni * row + e];
    }
}

__global__ __launch_bounds__(256) void resize_nearest_kernel(const float *__restrict__ x, int64_t planes, int h, int w,
                                                            float *__restrict__ out, int ho, int wo) {
    const int64_t total = planes * ho * wo;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int xd = int(id % wo);
    const int yd = int((id / wo) % ho);
    const int64_t p = id / wo / ho;
    int xs = xd, ys = yd;
    if (!(h == ho && w == wo)) {
        const double sx = double(w) / wo, sy = double(h) / ho;
        xs = int(round(sx * xd + (sx / 2 - 0.5)));
        ys = int(round(sy * yd + (sy / 2 - 0.5)));
        xs = xs >= 0 ? xs : 0;
        xs = xs < w - 1 ? xs : w - 1;
        ys = ys >= 0 ? ys : 0;
        ys = ys < h - 1 ? ys : h - 1;
    }
    out[id] = x[(p * h + ys) * w + xs];
}

struct DwGeom {
    int n, c, h, w, ho, wo, kh, kw, pt, pl, sh, sw, dh, dw;
    float padding_value;
};

// One lane per output element, adjacent lanes along W; value = fma(w, x, value) over (kh, kw) in the
// reference's order, padding taps contributing w * padding_value.
__global__ __launch_bounds__(256) void depthwise_kernel(const float *__restrict__ x, const float *__restrict__ wt, DwGeom g,
                                                       const float *__restrict__ bias, int act, float slope,
                                                       int64_t act_body, float *__restrict__ out) {
    const int64_t total = int64_t(g.n) * g.c * g.ho * g.wo;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int ow = int(id % g.wo);
    const int oh = int((id / g.wo) % g.ho);
    const int64_t pc = id / g.wo / g.ho;
    const int ci = int(pc % g.c);
    const float *in = x + pc * g.h * g.w;
    const float *k = wt + int64_t(ci) * g.kh * g.kw;
    float value = 0.f;
    for (int i = 0; i < g.kh; ++i)
        for (int j = 0; j < g.kw; ++j) {
            const int hi = -g.pt + oh * g.sh + i * g.dh, wi = -g.pl + ow * g.sw + j * g.dw;
            const float v = (hi >= 0 && hi < g.h && wi >= 0 && wi < g.w) ? in[hi * g.w + wi] : g.padding_value;
            value = __builtin_fmaf(k[i * g.kw + j], v, value);
        }
    if (bias) value = __fadd_rn(value, bias[ci]);
    out[id] = tsx::apply_act(value, act, slope, id < act_body);
}

}  // namespace

extern "C" {

int tsx_concat_channels_f32(const float *src_dev, int64_t n, int32_t c_src, int64_t inner, float *dst_dev, int32_t c_dst,
                            int32_t c_offset, void *stream) {
    TSX_REQUIRE(src_dev && dst_dev, "concat: null pointer");
    TSX_REQUIRE(n > 0 && c_src > 0 && inner > 0 && c_offset >= 0 && c_offset + c_src <= c_dst, "concat: channels [%d, %d) do not fit %d",
                c_offset, c_offset + c_src, c_dst);
    const int64_t row = int64_t(c_src) * inner, dst_row = int64_t(c_dst) * inner, dst_off = int64_t(c_offset) * inner;
    const bool vec = row % 4 == 0 && dst_row % 4 == 0 && dst_off % 4 == 0 && reinterpret_cast<uintptr_t>(src_dev) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(dst_dev) % 16 == 0;
    int64_t blocks = tsx::ceil_div(n * (vec ? row / 4 : row), 256);
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL(concat_channels_kernel, dim3(unsigned(blocks)), dim3(256), 0, tsx::as_stream(stream), src_dev, n, row,
                       dst_dev, dst_row, dst_off, vec);
    TSX_LAUNCH_CHECK("concat_channels_kernel");
    return 0;
}

int tsx_resize_nearest_f32(const float *x_dev, int64_t planes, int32_t h, int32_t w, float *out_dev, int32_t out_h,
                           int32_t out_w, void *stream) {
    TSX_REQUIRE(x_dev && out_dev, "resize_nearest: null pointer");
    TSX_REQUIRE(planes > 0 && h > 0 && w > 0 && out_h > 0 && out_w > 0, "resize_nearest: non-positive extent");
    const int64_t total = planes * out_h * out_w;
    TSX_REQUIRE(tsx::ceil_div(total, 256) < (int64_t(1) << 31), "resize_nearest: tensor too large");
    hipLaunchKernelGGL(resize_nearest_kernel, dim3(unsigned(tsx::ceil_div(total, 256))), dim3(256), 0, tsx::as_stream(stream),
                       x_dev, planes, h, w, out_dev, out_h, out_w);
    TSX_LAUNCH_CHECK("resize_nearest_kernel");
    return 0;
}

int tsx_depthwise_conv2d_f32(const tsx_conv2d_geom *g, const float *x_dev, const float *w_dev, float padding_value,
                             const float *bias_dev, int32_t act, float slope, float *out_dev, void *stream) {
    TSX_REQUIRE(g && x_dev && w_dev && out_dev, "depthwise_conv2d: null argument");
    TSX_REQUIRE(g->n > 0 && g->c > 0 && g->h > 0 && g->w > 0 && g->kh > 0 && g->kw > 0, "depthwise_conv2d: non-positive extent");
    TSX_REQUIRE(g->cout == g->c, "depthwise_conv2d: one filter per channel (cout %d != c %d)", g->cout, g->c);
    TSX_REQUIRE(g->stride_h > 0 && g->stride_w > 0 && g->dilation_h > 0 && g->dilation_w > 0,
                "depthwise_conv2d: stride and dilation must be positive");
    TSX_REQUIRE(act >= TSX_ACT_NONE && act <= TSX_ACT_MISH, "depthwise_conv2d: unknown activation %d", act);
    const int ho = tsx::conv_out(g->h, g->pad_top, g->pad_bottom, g->kh, g->stride_h, g->dilation_h);
    const int wo = tsx::conv_out(g->w, g->pad_left, g->pad_right, g->kw, g->stride_w, g->dilation_w);
    TSX_REQUIRE(ho > 0 && wo > 0, "depthwise_conv2d: empty output %dx%d", ho, wo);
    DwGeom d{g->n, g->c, g->h, g->w, ho, wo, g->kh, g->kw, g->pad_top, g->pad_left, g->stride_h, g->stride_w,
             g->dilation_h, g->dilation_w, padding_value};
    const int64_t total = int64_t(g->n) * g->c * ho * wo;
    TSX_REQUIRE(tsx::ceil_div(total, 256) < (int64_t(1) << 31), "depthwise_conv2d: tensor too large");
    hipLaunchKernelGGL(depthwise_kernel, dim3(unsigned(tsx::ceil_div(total, 256))), dim3(256), 0, tsx::as_stream(stream), x_dev,
                       w_dev, d, bias_dev, act, slope, total / 4 * 4, out_dev);
    TSX_LAUNCH_CHECK("depthwise_kernel");
    return 0;
}

}  // extern "C"
