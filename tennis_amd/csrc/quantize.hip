// quantize: fp32 -> int8 with the reference's two rounding paths.
// Restates cpu::Quantize (src/kernels/cpu/quantize.cpp:70-125) for gfx950.
//
// HBM-bound: 4 B read + 1 B written per element.  Each lane converts 16 consecutive
// elements (4 x 16-byte loads, one 16-byte store), so a wavefront reads 4 KiB and writes
// 1 KiB contiguous per iteration.
#include "tsx_common.hpp"
#include <cmath>

namespace {

using tsx::quantize_value;

// Element i belongs to scale group i / group_len (group_len = ceil(count / n_scales));
// with one scale the first bulk8 = 8*floor(count/8) elements round half to even.
__device__ __forceinline__ int quantize_at(float x, int64_t i, const float *__restrict__ scales, int n_scales,
                                           int64_t group_len, int64_t bulk8) {
    const float s = n_scales == 1 ? scales[0] : scales[i / group_len];
    return quantize_value(__fmul_rn(x, s), n_scales == 1 && i < bulk8);
}

__global__ __launch_bounds__(256) void quantize_f32_i8_kernel(const float *__restrict__ x, int64_t count,
                                                             const float *__restrict__ scales, int n_scales,
                                                             int64_t group_len, int64_t bulk8,
                                                             int8_t *__restrict__ out, bool aligned) {
    const int64_t stride = int64_t(gridDim.x) * blockDim.x * 16;
    for (int64_t base = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) * 16; base < count; base += stride) {
        if (aligned && base + 16 <= count) {
            const float4 *src = reinterpret_cast<const float4 *>(x + base);
            uint32_t packed[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float4 f = src[v];
                const float e[4] = {f.x, f.y, f.z, f.w};
                uint32_t word = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int q = quantize_at(e[j], base + v * 4 + j, scales, n_scales, group_len, bulk8);
                    word |= uint32_t(q & 0xff) << (8 * j);
                }
                packed[v] = word;
            }
            *reinterpret_cast<uint4 *>(out + base) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        } else {
            for (int j = 0; j < 16 && base + j < count; ++j)
                out[base + j] = int8_t(quantize_at(x[base + j], base + j, scales, n_scales, group_len, bulk8));
        }
    }
}

}  // namespace

extern "C" int tsx_quantize_f32_i8(const float *x_dev, int64_t count, const float *scales_dev, int32_t n_scales,
                                   int8_t *out_dev, void *stream) {
    TSX_REQUIRE(count >= 0 && n_scales >= 1, "quantize: count %lld, n_scales %d", (long long)count, n_scales);
    if (count == 0) return 0;
    TSX_REQUIRE(x_dev && scales_dev && out_dev, "quantize: null pointer");
    // Same expression as the reference (quantize.cpp:110), float rounding of count included.
    const int64_t group_len = int64_t(std::ceil(static_cast<float>(count) / static_cast<float>(n_scales)));
    const int64_t bulk8 = (count >> 3) << 3;
    const bool aligned = (reinterpret_cast<uintptr_t>(x_dev) % 16 == 0) && (reinterpret_cast<uintptr_t>(out_dev) % 16 == 0);
    const int64_t chunks = tsx::ceil_div(count, 16);
    int64_t blocks = tsx::ceil_div(chunks, 256);
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL(quantize_f32_i8_kernel, dim3(unsigned(blocks)), dim3(256), 0, tsx::as_stream(stream), x_dev,
                       count, scales_dev, n_scales, group_len, bulk8, out_dev, aligned);
    TSX_LAUNCH_CHECK("quantize_f32_i8_kernel");
    return 0;
}
