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
    // blockIdx.y walks the batch, blockIdx.x one image's row: no division per element
    const int64_t per = vec ? row / 4 : row;
    for (int64_t ni = blockIdx.y; ni < n; ni += gridDim.y)
    for (int64_t e = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; e < per; e += int64_t(gridDim.x) * blockDim.x) {
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
    int xd, yd;
    int64_t p;
    if (total <= 0xffffffffll) {   // 32-bit divisions where the element count allows: this kernel is bound by its arithmetic
        const uint32_t id32 = uint32_t(id), r = id32 / uint32_t(wo), p32 = r / uint32_t(ho);
        xd = int(id32 - r * uint32_t(wo));
        yd = int(r - p32 * uint32_t(ho));
        p = p32;
    } else {
        xd = int(id % wo);
        yd = int((id / wo) % ho);
        p = id / wo / ho;
    }
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

// One lane per DW_RUN consecutive outputs of a row, adjacent lanes along W then H inside one (n, c) plane
// (blockIdx.x), so a wavefront reads and writes contiguous runs of the plane; per output
// value = fma(w, x, value) over (kh, kw) in the reference's order, padding taps contributing
// w * padding_value.  K3 = a 3x3 kernel at stride 1, dilation 1 (the usual depthwise layer): the taps are
// unrolled, the nine weights sit in registers and a lane loads each input row's DW_RUN + 2 columns once for
// its DW_RUN outputs instead of three per output.  K3V = the same with padding 1 on both sides of a row whose
// length is a multiple of 4: a lane's four centre columns are one aligned 16-byte load (a wavefront reads whole
// cache lines; scalar loads at a 16-byte lane stride fetch every line four times over) and the two columns
// beside them come from the neighbouring lanes' registers.
constexpr int DW_RUN = 4;
enum { DW_GENERIC = 0, DW_K3 = 1, DW_K3V = 2 };

template <int MODE>
__global__ __launch_bounds__(256) void depthwise_kernel(const float *__restrict__ x, const float *__restrict__ wt, DwGeom g,
                                                       const float *__restrict__ bias, int act, float slope,
                                                       int64_t act_body, float *__restrict__ out) {
    const int runs = (g.wo + DW_RUN - 1) / DW_RUN;        // runs per output row
    const int lin = blockIdx.y * 256 + threadIdx.x;
    const int oh = lin / runs;
    if (oh >= g.ho) return;   // whole rows only: a lane that stays has both row neighbours beside it
    const int ow0 = (lin - oh * runs) * DW_RUN;
    const int64_t pc = blockIdx.x;
    const int ci = int(pc % g.c);
    const float *in = x + pc * g.h * g.w;
    const float *k = wt + int64_t(ci) * g.kh * g.kw;
    float value[DW_RUN];
#pragma unroll
    for (int t = 0; t < DW_RUN; ++t) value[t] = 0.f;
    if (MODE == DW_K3V) {
        float kk[9];
#pragma unroll
        for (int i = 0; i < 9; ++i) kk[i] = k[i];
        const int lane = threadIdx.x % 64;
        const bool first = ow0 == 0, last = ow0 + DW_RUN == g.w;   // the row's first / last run (w == wo here)
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int hi = oh - g.pt + i;
            const bool row_in = hi >= 0 && hi < g.h;
            const float *row = in + min(max(hi, 0), g.h - 1) * g.w;
            const float4 c4 = *reinterpret_cast<const float4 *>(row + ow0);
            // column ow0 - 1 is the previous lane's last value, column ow0 + 4 the next lane's first one (same row
            // unless this is the row's first / last run); the wavefront's edge lanes load theirs
            float left = __shfl_up(c4.w, 1), right = __shfl_down(c4.x, 1);
            if (lane == 0 && !first) left = row[ow0 - 1];
            if (lane == 63 && !last) right = row[ow0 + DW_RUN];
            float v[DW_RUN + 2] = {left, c4.x, c4.y, c4.z, c4.w, right};
            if (first) v[0] = g.padding_value;
            if (last) v[DW_RUN + 1] = g.padding_value;
            if (!row_in) {
#pragma unroll
                for (int c = 0; c < DW_RUN + 2; ++c) v[c] = g.padding_value;
            }
#pragma unroll
            for (int j = 0; j < 3; ++j)
#pragma unroll
                for (int t = 0; t < DW_RUN; ++t) value[t] = __builtin_fmaf(kk[i * 3 + j], v[t + j], value[t]);
        }
    } else if (MODE == DW_K3) {
        float kk[9];
#pragma unroll
        for (int i = 0; i < 9; ++i) kk[i] = k[i];
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            const int hi = oh - g.pt + i;
            const bool row_in = hi >= 0 && hi < g.h;
            const float *row = in + min(max(hi, 0), g.h - 1) * g.w;
            // unconditional loads from clamped addresses, then a select: the loads of a lane are all in flight
            // at once instead of one branch (and one memory round trip) after the other
            float v[DW_RUN + 2];
#pragma unroll
            for (int c = 0; c < DW_RUN + 2; ++c) {
                const int wi = ow0 - g.pl + c;
                const float loaded = row[min(max(wi, 0), g.w - 1)];
                v[c] = (row_in && wi >= 0 && wi < g.w) ? loaded : g.padding_value;
            }
#pragma unroll
            for (int j = 0; j < 3; ++j)
#pragma unroll
                for (int t = 0; t < DW_RUN; ++t) value[t] = __builtin_fmaf(kk[i * 3 + j], v[t + j], value[t]);
        }
    } else {
        for (int i = 0; i < g.kh; ++i)
            for (int j = 0; j < g.kw; ++j) {
                const float kv = k[i * g.kw + j];
                const int hi = -g.pt + oh * g.sh + i * g.dh;
                const float *row = in + min(max(hi, 0), g.h - 1) * g.w;
                float v[DW_RUN];
#pragma unroll
                for (int t = 0; t < DW_RUN; ++t) {
                    const int wi = -g.pl + (ow0 + t) * g.sw + j * g.dw;
                    const float loaded = row[min(max(wi, 0), g.w - 1)];
                    v[t] = (hi >= 0 && hi < g.h && wi >= 0 && wi < g.w) ? loaded : g.padding_value;
                }
#pragma unroll
                for (int t = 0; t < DW_RUN; ++t) value[t] = __builtin_fmaf(kv, v[t], value[t]);
            }
    }
    const int64_t id0 = (pc * g.ho + oh) * g.wo + ow0;
    const float b = bias ? bias[ci] : 0.f;
    float r[DW_RUN];
#pragma unroll
    for (int t = 0; t < DW_RUN; ++t) {
        const float v = bias ? __fadd_rn(value[t], b) : value[t];
        r[t] = tsx::apply_act(v, act, slope, id0 + t < act_body);
    }
    if (ow0 + DW_RUN <= g.wo && (id0 & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        *reinterpret_cast<float4 *>(out + id0) = make_float4(r[0], r[1], r[2], r[3]);
    } else {
#pragma unroll
        for (int t = 0; t < DW_RUN; ++t)
            if (ow0 + t < g.wo) out[id0 + t] = r[t];
    }
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
    int64_t blocks = tsx::ceil_div(vec ? row / 4 : row, 256);
    if (blocks > 256 * 16) blocks = 256 * 16;
    const unsigned batch_blocks = unsigned(n < 65535 ? n : 65535);
    hipLaunchKernelGGL(concat_channels_kernel, dim3(unsigned(blocks), batch_blocks), dim3(256), 0, tsx::as_stream(stream), src_dev, n, row,
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
    TSX_REQUIRE(act >= TSX_ACT_NONE && act <= TSX_ACT_MISH_FAST, "depthwise_conv2d: unknown activation %d", act);
    const int ho = tsx::conv_out(g->h, g->pad_top, g->pad_bottom, g->kh, g->stride_h, g->dilation_h);
    const int wo = tsx::conv_out(g->w, g->pad_left, g->pad_right, g->kw, g->stride_w, g->dilation_w);
    TSX_REQUIRE(ho > 0 && wo > 0, "depthwise_conv2d: empty output %dx%d", ho, wo);
    DwGeom d{g->n, g->c, g->h, g->w, ho, wo, g->kh, g->kw, g->pad_top, g->pad_left, g->stride_h, g->stride_w,
             g->dilation_h, g->dilation_w, padding_value};
    const int64_t total = int64_t(g->n) * g->c * ho * wo;
    const int64_t planes = int64_t(g->n) * g->c;
    const int64_t lanes_per_plane = int64_t(ho) * ((wo + DW_RUN - 1) / DW_RUN);
    TSX_REQUIRE(planes < (int64_t(1) << 31) && tsx::ceil_div(lanes_per_plane, 256) <= 65535 && int64_t(g->h) * g->w < (int64_t(1) << 31),
                "depthwise_conv2d: tensor too large");
    const dim3 grid(unsigned(planes), unsigned(tsx::ceil_div(lanes_per_plane, 256)));
    const bool k3 = g->kh == 3 && g->kw == 3 && g->stride_h == 1 && g->stride_w == 1 && g->dilation_h == 1 && g->dilation_w == 1;
    const bool k3v = k3 && g->pad_left == 1 && wo == g->w && g->w % 4 == 0 && reinterpret_cast<uintptr_t>(x_dev) % 16 == 0;
    if (k3v)
        hipLaunchKernelGGL(depthwise_kernel<DW_K3V>, grid, dim3(256), 0, tsx::as_stream(stream), x_dev, w_dev, d, bias_dev, act,
                           slope, total / 4 * 4, out_dev);
    else if (k3)
        hipLaunchKernelGGL(depthwise_kernel<DW_K3>, grid, dim3(256), 0, tsx::as_stream(stream), x_dev, w_dev, d, bias_dev, act,
                           slope, total / 4 * 4, out_dev);
    else
        hipLaunchKernelGGL(depthwise_kernel<DW_GENERIC>, grid, dim3(256), 0, tsx::as_stream(stream), x_dev, w_dev, d, bias_dev, act,
                           slope, total / 4 * 4, out_dev);
    TSX_LAUNCH_CHECK("depthwise_kernel");
    return 0;
}

}  // extern "C"
