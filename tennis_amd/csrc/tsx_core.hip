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
