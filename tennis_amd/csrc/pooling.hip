// 2-D pooling, NCHW fp32: cpu::Pooling2DCore (src/kernels/cpu/pooling2d_core.cpp:48-186) and, with the
// window set to the whole map, base::GlobalPooling2D (src/backend/base/base_global_pooling2d.cpp:58-79).
// HBM-bound: each input element is read once per window that covers it (served by L2 for overlapping
// windows), each output written once.
//
// Semantics kept from the reference: the window is clipped to the image (padding never contributes);
// MAX starts from the first valid element and replaces it on `>`; AVG sums the valid elements in
// row-major order in fp32 and divides by their count (BLACK padding) or by kh*kw (WHITE padding).
// One lane per output element, adjacent lanes along W; one lane's sequential sum is the reference's.
#include "tsx_common.hpp"

namespace {

struct PoolGeom {
    int64_t planes;
    int h, w, ho, wo, type, pad_top, pad_left, kh, kw, sh, sw, white;
};

__global__ __launch_bounds__(256) void pooling2d_kernel(const float *__restrict__ x, PoolGeom g, float *__restrict__ out) {
    const int64_t total = g.planes * g.ho * g.wo;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int ow = int(id % g.wo);
    const int oh = int((id / g.wo) % g.ho);
    const int64_t pc = id / g.wo / g.ho;
    const float *in = x + pc * g.h * g.w;
    int hs = oh * g.sh - g.pad_top, ws = ow * g.sw - g.pad_left;
    const int he = min(hs + g.kh, g.h), we = min(ws + g.kw, g.w);
    hs = max(hs, 0);
    ws = max(ws, 0);
    float r;
    if (g.type == 0) {
        // the reference reads the first element unconditionally; a window with no valid element
        // cannot occur for a shape its own size rule produces, and is reported as 0 here
        float m = (hs < he && ws < we) ? in[hs * g.w + ws] : 0.f;
        for (int ih = hs; ih < he; ++ih)
            for (int iw = ws; iw < we; ++iw) {
                const float v = in[ih * g.w + iw];
                if (v > m) m = v;
            }
        r = m;
    } else {
        float sum = 0.f;
        int count = 0;
        for (int ih = hs; ih < he; ++ih)
            for (int iw = ws; iw < we; ++iw) {
                sum = __fadd_rn(sum, in[ih * g.w + iw]);
                ++count;
            }
        if (g.white) r = __fdiv_rn(sum, float(g.kh * g.kw));
        else r = count == 0 ? 0.f : __fdiv_rn(sum, float(count));
    }
    out[id] = r;
}

// Global pooling of large maps: one wavefront per plane would change the summation order, so the
// sequential order is kept and parallelism comes from the N*C planes (32 x 2048 at the end of a
// ResNet-50-shaped network).

}  // namespace

extern "C" {

int tsx_pooling2d_out_size(int32_t h, int32_t w, int32_t kh, int32_t kw, int32_t pad_top, int32_t pad_bottom,
                           int32_t pad_left, int32_t pad_right, int32_t stride_h, int32_t stride_w, int32_t *out_h,
                           int32_t *out_w) {
    TSX_REQUIRE(out_h && out_w && stride_h > 0 && stride_w > 0 && kh > 0 && kw > 0, "pooling2d_out_size: bad argument");
    // pooling2d_forward (include/backend/common_function.h:14-20): ceil of an fp32 quotient
    *out_h = int32_t(ceilf(float(h + pad_top + pad_bottom - kh) / float(stride_h) + 1.f));
    *out_w = int32_t(ceilf(float(w + pad_left + pad_right - kw) / float(stride_w) + 1.f));
    return 0;
}

int tsx_pooling2d_f32(const float *x_dev, int64_t planes, int32_t h, int32_t w, int32_t type, int32_t pad_top,
                      int32_t pad_left, int32_t kh, int32_t kw, int32_t stride_h, int32_t stride_w, int32_t white_padding,
                      float *out_dev, int32_t out_h, int32_t out_w, void *stream) {
    TSX_REQUIRE(x_dev && out_dev, "pooling2d: null pointer");
    TSX_REQUIRE(planes > 0 && h > 0 && w > 0 && out_h > 0 && out_w > 0 && kh > 0 && kw > 0 && stride_h > 0 && stride_w > 0,
                "pooling2d: non-positive extent");
    TSX_REQUIRE(type == 0 || type == 1, "pooling2d: type must be 0 (max) or 1 (avg)");
    TSX_REQUIRE(pad_top >= 0 && pad_left >= 0, "pooling2d: negative padding");
    // every window must hold at least one element's row/column start inside the map (the reference
    // reads in[hs][ws] unconditionally for MAX)
    TSX_REQUIRE((int64_t(out_h) - 1) * stride_h - pad_top < h && (int64_t(out_w) - 1) * stride_w - pad_left < w,
                "pooling2d: output %dx%d has windows outside the %dx%d map", out_h, out_w, h, w);
    PoolGeom g{planes, h, w, out_h, out_w, type, pad_top, pad_left, kh, kw, stride_h, stride_w, white_padding ? 1 : 0};
    const int64_t total = planes * out_h * out_w;
    TSX_REQUIRE(tsx::ceil_div(total, 256) < (int64_t(1) << 31), "pooling2d: tensor too large");
    hipLaunchKernelGGL(pooling2d_kernel, dim3(unsigned(tsx::ceil_div(total, 256))), dim3(256), 0, tsx::as_stream(stream),
                       x_dev, g, out_dev);
    TSX_LAUNCH_CHECK("pooling2d_kernel");
    return 0;
}

}  // extern "C"
