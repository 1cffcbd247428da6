// quantize: fp32 -> int8 with the reference's two rounding paths.
// Restates cpu::Quantize (src/kernels/cpu/quantize.cpp:70-125) for gfx950.
//
// HBM-bound: 4 B read + 1 B written per element.
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

// A wavefront converts chunks of 1024 consecutive elements: four rounds of one aligned 16-byte load per lane
// (the wavefront reads 1 KiB contiguous per round) and one 4-byte store per lane and round.  The scale group
// is looked up once per chunk when the chunk lies inside one group (groups are whole images or rows: nearly
// always), else per element.
constexpr int Q_CHUNK = 1024;

__global__ __launch_bounds__(256) void quantize_f32_i8_kernel(const float *__restrict__ x, int64_t count,
                                                             const float *__restrict__ scales, int n_scales,
                                                             int64_t group_len, int64_t bulk8,
                                                             int8_t *__restrict__ out, bool aligned) {
    const int lane = threadIdx.x % 64;
    const int64_t wave = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) / 64;
    const int64_t stride = int64_t(gridDim.x) * (blockDim.x / 64) * Q_CHUNK;
    for (int64_t chunk = wave * Q_CHUNK; chunk < count; chunk += stride) {
        if (aligned && chunk + Q_CHUNK <= count) {
            const int64_t g0 = n_scales == 1 ? 0 : chunk / group_len;
            const bool uniform = n_scales == 1 || (chunk + Q_CHUNK - 1) / group_len == g0;
            const float s0 = scales[g0];
            const bool even = n_scales == 1 && chunk + Q_CHUNK <= bulk8;   // the whole chunk rounds half to even
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int64_t base = chunk + v * 256 + lane * 4;
                const float4 f = *reinterpret_cast<const float4 *>(x + base);
                const float e[4] = {f.x, f.y, f.z, f.w};
                uint32_t word = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    int q;
                    if (uniform && (even || n_scales != 1)) q = quantize_value(__fmul_rn(e[j], s0), even);
                    else q = quantize_at(e[j], base + j, scales, n_scales, group_len, bulk8);
                    word |= uint32_t(q & 0xff) << (8 * j);
                }
                *reinterpret_cast<uint32_t *>(out + base) = word;
            }
        } else {
            for (int64_t i = chunk + lane; i < chunk + Q_CHUNK && i < count; i += 64)
                out[i] = int8_t(quantize_at(x[i], i, scales, n_scales, group_len, bulk8));
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
    int64_t blocks = tsx::ceil_div(tsx::ceil_div(count, Q_CHUNK), 4);   // four wavefronts per block
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL(quantize_f32_i8_kernel, dim3(unsigned(blocks)), dim3(256), 0, tsx::as_stream(stream), x_dev,
                       count, scales_dev, n_scales, group_len, bulk8, out_dev, aligned);
    TSX_LAUNCH_CHECK("quantize_f32_i8_kernel");
    return 0;
}
