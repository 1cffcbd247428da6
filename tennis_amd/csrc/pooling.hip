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

#include <algorithm>

namespace {

struct PoolGeom {
    int64_t planes;
    int h, w, ho, wo, type, pad_top, pad_left, kh, kw, sh, sw, white;
};

// KH, KW > 0: a window of that size, unrolled -- every element is loaded from a clamped address before the
// first comparison or addition, so a lane's loads are in flight together (the runtime-sized loop below waits
// for each element in turn: one memory round trip per window element).  KH == 0: any window size.
template <int KH, int KW>
__global__ __launch_bounds__(256) void pooling2d_kernel(const float *__restrict__ x, PoolGeom g, float *__restrict__ out) {
    const int64_t total = g.planes * g.ho * g.wo;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    int ow, oh;
    int64_t pc;
    if (total < (int64_t(1) << 32)) {   // 32-bit divisions: a 64-bit one costs more than the window's loads
        const unsigned u = unsigned(id), row = u / unsigned(g.wo);
        ow = int(u - row * unsigned(g.wo));
        pc = row / unsigned(g.ho);
        oh = int(row - unsigned(pc) * unsigned(g.ho));
    } else {
        ow = int(id % g.wo);
        oh = int((id / g.wo) % g.ho);
        pc = id / g.wo / g.ho;
    }
    const float *in = x + pc * g.h * g.w;
    int hs = oh * g.sh - g.pad_top, ws = ow * g.sw - g.pad_left;
    const int he = min(hs + g.kh, g.h), we = min(ws + g.kw, g.w);
    hs = max(hs, 0);
    ws = max(ws, 0);
    float r;
    if (KH > 0) {
        const int h0 = oh * g.sh - g.pad_top, w0 = ow * g.sw - g.pad_left;
        float v[KH > 0 ? KH * KW : 1];
#pragma unroll
        for (int i = 0; i < KH; ++i)
#pragma unroll
            for (int j = 0; j < KW; ++j)
                v[i * KW + j] = in[min(max(h0 + i, 0), g.h - 1) * g.w + min(max(w0 + j, 0), g.w - 1)];
        // the valid elements in row-major order, as the reference walks them
        float m = 0.f, sum = 0.f;
        int count = 0;
#pragma unroll
        for (int i = 0; i < KH; ++i)
#pragma unroll
            for (int j = 0; j < KW; ++j) {
                const bool ok = h0 + i >= 0 && h0 + i < g.h && w0 + j >= 0 && w0 + j < g.w;
                const float e = v[i * KW + j];
                if (ok) {
                    if (count == 0 || e > m) m = e;    // MAX starts from the first valid element, replaces on `>`
                    sum = __fadd_rn(sum, e);
                    ++count;
                }
            }
        if (g.type == 0) r = m;
        else if (g.white) r = __fdiv_rn(sum, float(KH * KW));
        else r = count == 0 ? 0.f : __fdiv_rn(sum, float(count));
    } else if (g.type == 0) {
        // the reference reads the first element unconditionally; the launcher admits no MAX window
        // without a valid element
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

// MAX pooling between two quantized convolutions, on int8 in the pixel-major staged layout
// [n][hs][ws][cp] on both sides.  quantize is monotone non-decreasing for a positive scale, so
// quantize(max(window)) == max(quantize(window)) element for element: pooling the producer's
// requantized int8 output gives the bytes that pooling2d(fp32) -> quantize would, with a quarter of
// the traffic and no layout pass in between.  One lane = 16 channels of one output pixel.
typedef short s2v __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t max_i8x4(uint32_t a, uint32_t b) {
    // signed bytes compared as the high bytes of 16-bit lanes: odd bytes in place, even bytes shifted up
    const uint32_t m = 0xff00ff00u;
    const s2v hi = __builtin_elementwise_max(__builtin_bit_cast(s2v, a & m), __builtin_bit_cast(s2v, b & m));
    const s2v lo = __builtin_elementwise_max(__builtin_bit_cast(s2v, (a << 8) & m), __builtin_bit_cast(s2v, (b << 8) & m));
    return __builtin_bit_cast(uint32_t, hi) | (__builtin_bit_cast(uint32_t, lo) >> 8);
}

struct PoolStagedGeom {
    int n, h, w, ho, wo, pad_top, pad_left, kh, kw, sh, sw;
    int s_hs, s_ws, s_cp, s_pt, s_pl;   // source buffer
    int d_hs, d_ws, d_cp, d_pt, d_pl;   // destination buffer
    int cb;                             // channels handled: the map's, rounded up to whole 64-channel blocks
};

// KH, KW > 0: a window of that size with every load issued before the first comparison -- rows and columns outside the
// map are clamped into it, which repeats elements the window holds anyway (max does not mind) -- where the
// runtime-sized loop (KH = 0) waits for each 16-byte element in turn.
template <int KH, int KW>
__global__ __launch_bounds__(256) void max_pooling2d_i8_staged_kernel(const int8_t *__restrict__ src, PoolStagedGeom g,
                                                                     int8_t *__restrict__ dst) {
    const int chunks = g.cb / 16;
    const int64_t total = int64_t(g.n) * g.ho * g.wo * chunks;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    int chunk, ow, oh, ni;
    if (total <= 0xffffffffll) {   // 32-bit divisions where the lane count allows
        const uint32_t id32 = uint32_t(id), r1 = id32 / uint32_t(chunks), r2 = r1 / uint32_t(g.wo), r3 = r2 / uint32_t(g.ho);
        chunk = int(id32 - r1 * uint32_t(chunks));
        ow = int(r1 - r2 * uint32_t(g.wo));
        oh = int(r2 - r3 * uint32_t(g.ho));
        ni = int(r3);
    } else {
        chunk = int(id % chunks);
        int64_t rest = id / chunks;
        ow = int(rest % g.wo);
        rest /= g.wo;
        oh = int(rest % g.ho);
        ni = int(rest / g.ho);
    }
    v4i r = {0, 0, 0, 0};   // channels the source does not have stay zero (channel padding)
    if (chunk * 16 < min(g.s_cp, g.cb)) {
        int hs = oh * g.sh - g.pad_top, ws = ow * g.sw - g.pad_left;
        const int he = min(hs + g.kh, g.h), we = min(ws + g.kw, g.w);
        hs = max(hs, 0);
        ws = max(ws, 0);
        const int8_t *base = src + ((int64_t(ni) * g.s_hs + g.s_pt) * g.s_ws + g.s_pl) * g.s_cp + chunk * 16;
        if (KH > 0) {
            v4i v[KH > 0 ? KH * KW : 1];
#pragma unroll
            for (int i = 0; i < KH; ++i)
#pragma unroll
                for (int j = 0; j < KW; ++j)
                    v[i * KW + j] = *reinterpret_cast<const v4i *>(
                        base + (int64_t(min(hs + i, he - 1)) * g.s_ws + min(ws + j, we - 1)) * g.s_cp);
            r = v[0];
#pragma unroll
            for (int t = 1; t < KH * KW; ++t)
#pragma unroll
                for (int k = 0; k < 4; ++k) r[k] = int(max_i8x4(uint32_t(r[k]), uint32_t(v[t][k])));
        } else {
            r = *reinterpret_cast<const v4i *>(base + (int64_t(hs) * g.s_ws + ws) * g.s_cp);   // the first valid element
            for (int ih = hs; ih < he; ++ih)
                for (int iw = ws; iw < we; ++iw) {
                    const v4i v = *reinterpret_cast<const v4i *>(base + (int64_t(ih) * g.s_ws + iw) * g.s_cp);
#pragma unroll
                    for (int k = 0; k < 4; ++k) r[k] = int(max_i8x4(uint32_t(r[k]), uint32_t(v[k])));
                }
        }
    }
    *reinterpret_cast<v4i *>(dst + ((int64_t(ni) * g.d_hs + oh + g.d_pt) * g.d_ws + ow + g.d_pl) * g.d_cp + chunk * 16) = r;
}

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
    // The ceil-mode size rule can give a last window that starts behind the map (9 rows, pads 1+2, 3 rows at
    // stride 2: the sixth window starts at row 9).  The reference's average of no element is 0
    // (src/kernels/cpu/pooling2d_core.cpp:131-134, 179), which the kernel reproduces; its MAX reads
    // in[hs][ws] unconditionally (:69), i.e. behind the plane -- there is no value to match, so that is refused.
    TSX_REQUIRE(type == 1 || ((int64_t(out_h) - 1) * stride_h - pad_top < h && (int64_t(out_w) - 1) * stride_w - pad_left < w),
                "pooling2d: max pooling output %dx%d has windows outside the %dx%d map", out_h, out_w, h, w);
    PoolGeom g{planes, h, w, out_h, out_w, type, pad_top, pad_left, kh, kw, stride_h, stride_w, white_padding ? 1 : 0};
    const int64_t total = planes * out_h * out_w;
    TSX_REQUIRE(tsx::ceil_div(total, 256) < (int64_t(1) << 31), "pooling2d: tensor too large");
    const dim3 grid(unsigned(tsx::ceil_div(total, 256)));
    if (kh == 3 && kw == 3)
        hipLaunchKernelGGL((pooling2d_kernel<3, 3>), grid, dim3(256), 0, tsx::as_stream(stream), x_dev, g, out_dev);
    else if (kh == 2 && kw == 2)
        hipLaunchKernelGGL((pooling2d_kernel<2, 2>), grid, dim3(256), 0, tsx::as_stream(stream), x_dev, g, out_dev);
    else if (kh == 5 && kw == 5)
        hipLaunchKernelGGL((pooling2d_kernel<5, 5>), grid, dim3(256), 0, tsx::as_stream(stream), x_dev, g, out_dev);
    else
        hipLaunchKernelGGL((pooling2d_kernel<0, 0>), grid, dim3(256), 0, tsx::as_stream(stream), x_dev, g, out_dev);
    TSX_LAUNCH_CHECK("pooling2d_kernel");
    return 0;
}

int tsx_max_pooling2d_i8_staged(const tsx_staged_map *src, const tsx_staged_map *dst, int32_t kh, int32_t kw, int32_t pad_top,
                                int32_t pad_left, int32_t stride_h, int32_t stride_w, void *stream) {
    TSX_REQUIRE(src && dst && src->data && dst->data, "max_pooling2d_i8_staged: null pointer");
    for (const tsx_staged_map *m : {src, dst}) {
        TSX_REQUIRE(m->n > 0 && m->h > 0 && m->w > 0 && m->c > 0 && m->cp >= m->c && m->cp % 64 == 0 && m->pad_top >= 0 &&
                        m->pad_left >= 0 && m->h + m->pad_top <= m->hs && m->w + m->pad_left <= m->ws,
                    "max_pooling2d_i8_staged: map %dx%dx%d does not fit [%d][%d][%d] at (%d,%d)", m->h, m->w, m->c, m->hs,
                    m->ws, m->cp, m->pad_top, m->pad_left);
        TSX_REQUIRE(reinterpret_cast<uintptr_t>(m->data) % 16 == 0, "max_pooling2d_i8_staged: buffers must be 16-byte aligned");
        // whole 64-channel blocks are read and written: a map that is a run of channels inside a wider buffer must
        // consist of whole blocks, or its last block would reach into the neighbouring run
        TSX_REQUIRE(m->cp == tsx::round_up(m->c, 64) || m->c % 64 == 0,
                    "max_pooling2d_i8_staged: %d channels inside a pitch of %d are not whole 64-channel blocks", m->c, m->cp);
    }
    TSX_REQUIRE(src->n == dst->n && src->c == dst->c, "max_pooling2d_i8_staged: batch / channels differ");
    // padding smaller than the window: together with the next check every window holds a valid element
    TSX_REQUIRE(kh > 0 && kw > 0 && stride_h > 0 && stride_w > 0 && pad_top >= 0 && pad_left >= 0 && pad_top < kh && pad_left < kw,
                "max_pooling2d_i8_staged: bad window");
    TSX_REQUIRE((int64_t(dst->h) - 1) * stride_h - pad_top < src->h && (int64_t(dst->w) - 1) * stride_w - pad_left < src->w,
                "max_pooling2d_i8_staged: output %dx%d has windows outside the %dx%d map", dst->h, dst->w, src->h, src->w);
    PoolStagedGeom g{src->n, src->h, src->w, dst->h, dst->w, pad_top, pad_left, kh, kw, stride_h, stride_w,
                     src->hs, src->ws, src->cp, src->pad_top, src->pad_left,
                     dst->hs, dst->ws, dst->cp, dst->pad_top, dst->pad_left,
                     int(std::min<int64_t>(dst->cp, tsx::round_up(dst->c, 64)))};
    const int64_t total = int64_t(dst->n) * dst->h * dst->w * (g.cb / 16);
    TSX_REQUIRE(tsx::ceil_div(total, 256) < (int64_t(1) << 31), "max_pooling2d_i8_staged: tensor too large");
    const dim3 grid(unsigned(tsx::ceil_div(total, 256)));
    const int8_t *s8 = static_cast<const int8_t *>(src->data);
    int8_t *d8 = static_cast<int8_t *>(dst->data);
    if (kh == 3 && kw == 3)
        hipLaunchKernelGGL((max_pooling2d_i8_staged_kernel<3, 3>), grid, dim3(256), 0, tsx::as_stream(stream), s8, g, d8);
    else if (kh == 5 && kw == 5)
        hipLaunchKernelGGL((max_pooling2d_i8_staged_kernel<5, 5>), grid, dim3(256), 0, tsx::as_stream(stream), s8, g, d8);
    else
        hipLaunchKernelGGL((max_pooling2d_i8_staged_kernel<0, 0>), grid, dim3(256), 0, tsx::as_stream(stream), s8, g, d8);
    TSX_LAUNCH_CHECK("max_pooling2d_i8_staged_kernel");
    return 0;
}

}  // extern "C"
