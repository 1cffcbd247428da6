// Error plumbing and device queries of the C ABI (include/tsx_hip.h).
#include "tsx_common.hpp"

namespace tsx {

char *error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

}  // namespace tsx

extern "C" {


const char *tsx_last_error(void) { return tsx::error_buffer(); }

int tsx_version(void) { return 100; }

int tsx_device_cu_count(void) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    return cus;
}

int tsx_conv2d_out_size(const tsx_conv2d_geom *g, int32_t *out_h, int32_t *out_w) {
    TSX_REQUIRE(g && out_h && out_w, "null argument");
    TSX_REQUIRE(g->stride_h > 0 && g->stride_w > 0 && g->dilation_h > 0 && g->dilation_w > 0 && g->kh > 0 && g->kw > 0,
                "stride, dilation and kernel size must be positive");
    *out_h = tsx::conv_out(g->h, g->pad_top, g->pad_bottom, g->kh, g->stride_h, g->dilation_h);
    *out_w = tsx::conv_out(g->w, g->pad_left, g->pad_right, g->kw, g->stride_w, g->dilation_w);
    return 0;
}

}  // extern "C"

#ifdef TSX_MEASUREMENT_AIDS
#include "tsx_aids.h"
namespace {

typedef int probe_v4i __attribute__((ext_vector_type(4)));
typedef int probe_v16i __attribute__((ext_vector_type(16)));

// Register-only MFMA loop: 8 independent 32x32 accumulators, operands read once from memory.
// What it sustains is the ceiling any i8 contraction kernel can reach on this part with this
// operand data; the rate depends on the data (clocks drop under the power of random operands).
__global__ __launch_bounds__(256) void probe_mfma_i8_kernel(const probe_v4i *__restrict__ src, int iters,
                                                           int32_t *__restrict__ sink) {
    probe_v16i acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0;
    probe_v4i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i] = src[threadIdx.x + 256 * i];
        b[i] = src[threadIdx.x + 256 * (i + 4)];
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i % 4], b[(i + it) % 4], acc[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[i][r];
    if (s == 0x7fffffff) sink[0] = s;   // keeps the loop alive; practically never taken
}

}  // namespace

extern "C" int tsx_probe_mfma_i8(const void *operands_dev, int32_t iters, int32_t blocks, int32_t *sink_dev, void *stream) {
    TSX_REQUIRE(operands_dev && sink_dev && iters > 0 && blocks > 0, "probe_mfma_i8: bad argument");
    TSX_REQUIRE(reinterpret_cast<uintptr_t>(operands_dev) % 16 == 0, "probe_mfma_i8: operands must be 16-byte aligned");
    hipLaunchKernelGGL(probe_mfma_i8_kernel, dim3(unsigned(blocks)), dim3(256), 0, tsx::as_stream(stream),
                       static_cast<const probe_v4i *>(operands_dev), iters, sink_dev);
    TSX_LAUNCH_CHECK("probe_mfma_i8_kernel");
    return 0;
}
#endif  // TSX_MEASUREMENT_AIDS
