// Winograd F(6x6, 3x3) and F(2x2, 3x3) fp32 convolution, restating
// Conv2dWinogradAlgorithm<float>::winograd_f63 / winograd_f23
// (src/kernels/cpu/winograd_algorithm.cpp:504-947 / :57-459) with the padding rule of
// KernelCommonFunc::in_out_pad_and_fix_size (src/kernels/common/function.cpp:14-78).
// F(6,3) is described below; F(2,3) is its twin with 4x4 patches (stride 2), 16 GEMMs and
// transforms made of sums and differences only.
//
//   U = G g G^T      kernel transform, once per weight tensor          -> u[64][Cout][Cin]
//   V = B^T d B      input transform of every 8x8 patch (stride 6)      -> v[N][64][Cin][tiles]
//   M_t = U_t V_t    64 independent GEMMs (Cout x Cin x tiles) per image -> m[N][64][Cout][tiles]
//   Y = A^T M A      output transform, cut to the true output size       -> out NCHW
//
// F(6,3) in fp32 amplifies single roundings to ~1e-5 of an O(1) output, the same size as the
// parity tolerance, so this path reproduces the reference's arithmetic exactly instead of merely
// approximating it:
//   * every transform uses the reference's factoring AND its fused multiply-adds: the reference
//     is built with gcc -O3 -mfma, whose default contraction fuses a*b+c patterns (in
//     a*c1 - b*c2 it fuses the first product and rounds the second); those FMAs are written
//     out explicitly here and the file is compiled with -ffp-contract=off;
//   * the 64 small GEMMs accumulate like the reference's pack8/kernel_8x8 micro-kernel
//     (src/kernels/cpu/math_cpu.cpp:386-700): one k-ascending FMA chain per output, and for
//     columns beyond the last full block of 8 four interleaved chains combined as
//     (s0+s1), (s2+s3), 0+s01, +s23.  They run on the vector ALUs -- the work is 4.4x smaller
//     than the direct convolution and the fp32 MFMA would change the summation order.
// All kernels here are memory/latency-bound elementwise or small-GEMM kernels.
#include "tsx_common.hpp"

#include <atomic>

namespace tsx {
namespace {

// ---------------------------------------------------------------- transforms (explicit FMAs)

__device__ __forceinline__ void bt_row(const float *i0, float *o) {
    // winograd_algorithm.cpp:640-663 (first pass over the rows of the patch)
    o[0] = fmaf(i0[4] - i0[2], 5.25f, i0[0] - i0[6]);
    o[7] = fmaf(i0[3] - i0[5], 5.25f, i0[7] - i0[1]);
    const float tmp12_a = fmaf(-i0[4], 4.25f, i0[2] + i0[6]);
    const float tmp12_b = fmaf(-i0[3], 4.25f, i0[1] + i0[5]);
    o[1] = tmp12_a + tmp12_b;
    o[2] = tmp12_a - tmp12_b;
    const float tmp34_a = fmaf(-i0[4], 1.25f, fmaf(i0[2], 0.25f, i0[6]));
    const float tmp34_b = fmaf(i0[5], 2.f, fmaf(i0[1], 0.5f, -(i0[3] * 2.5f)));
    o[3] = tmp34_a + tmp34_b;
    o[4] = tmp34_a - tmp34_b;
    const float tmp56_a = fmaf(fmaf(-i0[4], 1.25f, i0[2]), 4.f, i0[6]);
    const float tmp56_b = fmaf(i0[5], 0.5f, fmaf(i0[1], 2.f, -(i0[3] * 2.5f)));
    o[5] = tmp56_a + tmp56_b;
    o[6] = tmp56_a - tmp56_b;
}

__device__ __forceinline__ void bt_col(const float *d, float *o) {
    // winograd_algorithm.cpp:668-692 (second pass; tmp12_b's operand order differs from the first)
    o[0] = fmaf(d[4] - d[2], 5.25f, d[0] - d[6]);
    o[7] = fmaf(d[3] - d[5], 5.25f, d[7] - d[1]);
    const float tmp12_a = fmaf(-d[4], 4.25f, d[2] + d[6]);
    const float tmp12_b = fmaf(-d[3], 4.25f, d[1]) + d[5];
    o[1] = tmp12_a + tmp12_b;
    o[2] = tmp12_a - tmp12_b;
    const float tmp34_a = fmaf(-d[4], 1.25f, fmaf(d[2], 0.25f, d[6]));
    const float tmp34_b = fmaf(d[5], 2.f, fmaf(d[1], 0.5f, -(d[3] * 2.5f)));
    o[3] = tmp34_a + tmp34_b;
    o[4] = tmp34_a - tmp34_b;
    const float tmp56_a = fmaf(fmaf(-d[4], 1.25f, d[2]), 4.f, d[6]);
    const float tmp56_b = fmaf(d[5], 0.5f, fmaf(d[1], 2.f, -(d[3] * 2.5f)));
    o[5] = tmp56_a + tmp56_b;
    o[6] = tmp56_a - tmp56_b;
}

__device__ __forceinline__ void at_pass(const float *t, float *o) {
    // winograd_algorithm.cpp:775-795 / :808-830; every multiplier is a power of two, so fused
    // and unfused forms round identically -- only the left-to-right order of the sums matters.
    const float re0 = t[1] + t[2];
    const float re1 = t[1] - t[2];
    const float re2 = t[3] + t[4];
    const float re3 = t[3] - t[4];
    const float re4 = t[5] + t[6];
    const float re5 = t[5] - t[6];
    o[0] = t[0] + re0 + re2 + re4 * 32.f;
    o[1] = re1 + re3 + re3 + re5 * 16.f;
    o[2] = re0 + re2 * 4 + re4 * 8.f;
    o[3] = re1 + re3 * 8 + re5 * 4.f;
    o[4] = re0 + re2 * 16 + re4 + re4;
    o[5] = re1 + re3 * 32 + re5 + t[7];
}

// U[t = i*8+j][cout][cin] = (G g G^T)[i][j]  (winograd_algorithm.cpp:504-566, before its pack8_A)
__global__ __launch_bounds__(256) void wino_kernel_transform_kernel(const float *__restrict__ w, int cout, int cin,
                                                                   float *__restrict__ u) {
    const int id = blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= cout * cin) return;
    const float G[8][3] = {{1.0f, 0.0f, 0.0f},
                           {-2.f / 9, -2.f / 9, -2.f / 9},
                           {-2.f / 9, 2.f / 9, -2.f / 9},
                           {1.f / 90, 1.f / 45, 2.f / 45},
                           {1.f / 90, -1.f / 45, 2.f / 45},
                           {1.f / 45, 1.f / 90, 1.f / 180},
                           {1.f / 45, -1.f / 90, 1.f / 180},
                           {0.0f, 0.0f, 1.0f}};
    float g[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) g[i] = w[int64_t(id) * 9 + i];
    float tmp[3][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 3; ++r)
            tmp[r][i] = fmaf(g[r * 3 + 2], G[i][2], fmaf(g[r * 3 + 0], G[i][0], g[r * 3 + 1] * G[i][1]));
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j)
            u[int64_t(i * 8 + j) * cout * cin + id] =
                fmaf(tmp[2][j], G[i][2], fmaf(tmp[0][j], G[i][0], tmp[1][j] * G[i][1]));
}

struct WinoGeom {
    int n, c, h, w, cout, ho, wo, pad_top, pad_left, th, tw, tiles;
    float padding_value;
};

// One thread per (image, channel, tile); adjacent lanes take adjacent tiles, so the 64 stores of a
// lane (stride Cin*tiles) are coalesced across the wavefront.
__global__ __launch_bounds__(256) void wino_input_transform_kernel(const float *__restrict__ x, WinoGeom g,
                                                                  float *__restrict__ v) {
    const int64_t total = int64_t(g.n) * g.c * g.tiles;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int tile = int(id % g.tiles);
    const int ch = int((id / g.tiles) % g.c);
    const int img = int(id / g.tiles / g.c);
    const int ty = tile / g.tw, tx = tile - ty * g.tw;
    const float *src = x + (int64_t(img) * g.c + ch) * g.h * g.w;
    float db[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float row[8];
        const int hh = ty * 6 + i - g.pad_top;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int ww = tx * 6 + j - g.pad_left;
            // outside the tensor: the conv padding and the bottom/right fill both use padding_value
            row[j] = (hh >= 0 && hh < g.h && ww >= 0 && ww < g.w) ? src[hh * g.w + ww] : g.padding_value;
        }
        bt_row(row, db[i]);
    }
    float *dst = v + (int64_t(img) * 64 * g.c + ch) * g.tiles + tile;
    const int64_t stride = int64_t(g.c) * g.tiles;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float col[8], o[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) col[r] = db[r][i];
        bt_col(col, o);
#pragma unroll
        for (int r = 0; r < 8; ++r) dst[(r * 8 + i) * stride] = o[r];
    }
}

// C[b][m][n] = A[b % a_batches][m][k] * B[b][k][n] in the reference's accumulation order
// (math_cpu.cpp:386-700 as restated by the CPU oracle): m8/n8 = extents rounded down to 8.
// Columns below n8 are one fused-multiply-add chain in ascending k per output; the columns from n8 on sum four
// interleaved partial chains first.  Two kernels: the tiled one for the columns below n8, this one (one lane per
// output, columns j0..n) for the rest.
__global__ __launch_bounds__(256) void gemm_f32_seq_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                          float *__restrict__ c, int m, int n, int k, int batches,
                                                          int a_batches, int j0) {
    const int cols = n - j0;
    const int64_t total = int64_t(batches) * m * cols;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int j = j0 + int(id % cols);
    const int i = int((id / cols) % m);
    const int bt = int(id / cols / m);
    const float *ar = a + (int64_t(bt % a_batches) * m + i) * k;
    const float *bc = b + int64_t(bt) * k * n + j;
    const int m8 = m / 8 * 8, n8 = n / 8 * 8, k4 = k / 4 * 4;
    float r;
    if (j < n8) {
        float acc = 0.f;
        for (int kk = 0; kk < k; ++kk) acc = fmaf(bc[int64_t(kk) * n], ar[kk], acc);
        r = acc;
    } else {
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
        for (int kk = 0; kk < k4; kk += 4) {
            s0 = fmaf(ar[kk + 0], bc[int64_t(kk + 0) * n], s0);
            s1 = fmaf(ar[kk + 1], bc[int64_t(kk + 1) * n], s1);
            s2 = fmaf(ar[kk + 2], bc[int64_t(kk + 2) * n], s2);
            s3 = fmaf(ar[kk + 3], bc[int64_t(kk + 3) * n], s3);
        }
        float acc;
        if (i < m8) {
            const float s01 = s0 + s1, s23 = s2 + s3;
            acc = 0.f + s01;
            acc = acc + s23;
        } else {
            acc = ((s0 + s1) + s2) + s3;
        }
        for (int kk = k4; kk < k; ++kk) acc = fmaf(ar[kk], bc[int64_t(kk) * n], acc);
        r = acc;
    }
    c[(int64_t(bt) * m + i) * n + j] = r;
}

// The columns below n8: every output is the same chain acc = fma(B[k][j], A[i][k], acc) over ascending k, so a
// lane can hold a 4 x 4 block of outputs and feed 16 chains from 4 values of A and 4 of B per k -- an eighth of
// the loads of one lane per output, the same bits.  VEC: k and n multiples of 4 and 16-byte aligned operands, so
// A is read four k at a time and B four columns at a time as 16-byte loads.  Lanes run along the column blocks.
template <bool VEC>
__global__ __launch_bounds__(256) void gemm_f32_seq_tiled_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                                float *__restrict__ c, int m, int n, int k, int batches,
                                                                int a_batches, int n8) {
    const int jb = n8 / 4, ib = (m + 3) / 4;
    const int64_t total = int64_t(batches) * ib * jb;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int j = int(id % jb) * 4;
    const int i = int((id / jb) % ib) * 4;
    const int bt = int(id / jb / ib);
    const float *ab = a + int64_t(bt % a_batches) * m * k;
    const float *bc = b + int64_t(bt) * k * n + j;
    const float *ar[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) ar[r] = ab + int64_t(min(i + r, m - 1)) * k;   // rows past m: computed, not stored
    float acc[4][4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[r][q] = 0.f;
    int kk = 0;
    if (VEC) {
        for (; kk + 4 <= k; kk += 4) {
            float4 av[4], bv[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) av[r] = *reinterpret_cast<const float4 *>(ar[r] + kk);
#pragma unroll
            for (int t = 0; t < 4; ++t) bv[t] = *reinterpret_cast<const float4 *>(bc + int64_t(kk + t) * n);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float av_t = t == 0 ? av[r].x : t == 1 ? av[r].y : t == 2 ? av[r].z : av[r].w;
                    acc[r][0] = fmaf(bv[t].x, av_t, acc[r][0]);
                    acc[r][1] = fmaf(bv[t].y, av_t, acc[r][1]);
                    acc[r][2] = fmaf(bv[t].z, av_t, acc[r][2]);
                    acc[r][3] = fmaf(bv[t].w, av_t, acc[r][3]);
                }
            }
        }
    }
    for (; kk < k; ++kk) {
        float bv[4], av[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) bv[q] = bc[int64_t(kk) * n + q];
#pragma unroll
        for (int r = 0; r < 4; ++r) av[r] = ar[r][kk];
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[r][q] = fmaf(bv[q], av[r], acc[r][q]);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (i + r >= m) break;
        float *dst = c + (int64_t(bt) * m + i + r) * n + j;
        if (VEC) *reinterpret_cast<float4 *>(dst) = make_float4(acc[r][0], acc[r][1], acc[r][2], acc[r][3]);
        else {
#pragma unroll
            for (int q = 0; q < 4; ++q) dst[q] = acc[r][q];
        }
    }
}

// Both parts of the sequential-order GEMM on `stream`.
int launch_gemm_f32_seq(const float *a, const float *b, float *c, int m, int n, int k, int batches, int a_batches,
                        hipStream_t stream) {
    const int n8 = n / 8 * 8;
    if (n8 > 0) {
        const int64_t threads = int64_t(batches) * ((m + 3) / 4) * (n8 / 4);
        const bool vec = k % 4 == 0 && n % 4 == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(b) % 16 == 0 && reinterpret_cast<uintptr_t>(c) % 16 == 0;
        const dim3 grid(unsigned(ceil_div(threads, 256)));
        if (vec) hipLaunchKernelGGL(gemm_f32_seq_tiled_kernel<true>, grid, dim3(256), 0, stream, a, b, c, m, n, k, batches, a_batches, n8);
        else hipLaunchKernelGGL(gemm_f32_seq_tiled_kernel<false>, grid, dim3(256), 0, stream, a, b, c, m, n, k, batches, a_batches, n8);
        TSX_LAUNCH_CHECK("gemm_f32_seq_tiled_kernel");
    }
    if (n8 < n) {
        const int64_t threads = int64_t(batches) * m * (n - n8);
        hipLaunchKernelGGL(gemm_f32_seq_kernel, dim3(unsigned(ceil_div(threads, 256))), dim3(256), 0, stream, a, b, c, m, n, k,
                           batches, a_batches, n8);
        TSX_LAUNCH_CHECK("gemm_f32_seq_kernel");
    }
    return 0;
}

// One thread per (image, cout, tile): Y = A^T M A, cut to the true output, then the optional
// add_bias / activation that follow the convolution in the graph.
// MISH: whether the activation may be Mish (see apply_act_basic for why that is a compile-time matter here)
template <bool MISH>
__global__ __launch_bounds__(256) void wino_output_transform_kernel(const float *__restrict__ mm, WinoGeom g,
                                                                   const float *__restrict__ bias, int act,
                                                                   float slope, int64_t act_body,
                                                                   float *__restrict__ out) {
    const int64_t total = int64_t(g.n) * g.cout * g.tiles;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int tile = int(id % g.tiles);
    const int co = int((id / g.tiles) % g.cout);
    const int img = int(id / g.tiles / g.cout);
    const int ty = tile / g.tw, tx = tile - ty * g.tw;
    const float *src = mm + (int64_t(img) * 64 * g.cout + co) * g.tiles + tile;
    const int64_t stride = int64_t(g.cout) * g.tiles;
    float tmpa[8][6];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float t8[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) t8[j] = src[(i * 8 + j) * stride];
        at_pass(t8, tmpa[i]);
    }
    const float bv = bias ? bias[co] : 0.f;
    float *dst = out + (int64_t(img) * g.cout + co) * g.ho * g.wo;
#pragma unroll
    for (int i = 0; i < 6; ++i) {
        float t8[8], o[6];
#pragma unroll
        for (int r = 0; r < 8; ++r) t8[r] = tmpa[r][i];
        at_pass(t8, o);
        const int ww = tx * 6 + i;
#pragma unroll
        for (int r = 0; r < 6; ++r) {
            const int hh = ty * 6 + r;
            if (hh < g.ho && ww < g.wo) {
                float val = o[r];
                if (bias) val = __fadd_rn(val, bv);
                const int64_t idx = (int64_t(img) * g.cout + co) * g.ho * g.wo + hh * g.wo + ww;
                dst[hh * g.wo + ww] = MISH ? apply_act(val, act, slope, idx < act_body) : apply_act_basic(val, act, slope, idx < act_body);
            }
        }
    }
}

// ---------------------------------------------------------------- F(6,3), fast path
// The same algorithm on the fp32 MFMA, for callers that hold the path to its floating-point tolerance rather than
// to its bits (the MFMA sums the channel products in another order than the reference's FMA chains): the input
// transform kernel above, then ONE kernel for the 64 frequency GEMMs and the output transform -- M never exists in
// memory.  A workgroup owns 16 tiles x 16 output channels and all 64 frequencies; wavefront w multiplies
// frequencies 16w .. 16w+15 on v_mfma_f32_16x16x4_f32 with both operands loaded from global memory (L2: U and V
// are a few MB) straight into the MFMA operand registers, four 16-channel blocks in flight: lane l holds
// U_f[cout l%16][4 consecutive channels of group l/16] as one 16-byte load and V_f[those channels][tile l%16]; the
// four MFMAs of a block take the channels group by group (a sum does not care which k a step carries).
// Accumulator register r of lane l is output channel 4*(l/16) + r, tile l%16.  The 64 products of every (output
// channel, tile) then go through LDS to one thread, which applies A^T M A, bias and activation and stores the 6x6
// outputs.
constexpr int WF_TILES = 16, WF_COUT = 16;
constexpr int WF_DEPTH = 4;   // ring of 16-channel blocks per wavefront: WF_DEPTH - 1 in flight

typedef float wf_v4f __attribute__((ext_vector_type(4)));

// BLOCKS = C / 16 when C is 64, 128 or 256 (then the whole walk over frequencies and channel blocks is unrolled
// around a 16-slot ring, 15 blocks in flight: with one wavefront per SIMD nothing else hides an L2 round trip),
// 0 for any other channel count (rounds of WF_DEPTH blocks per frequency).
template <int BLOCKS, bool MISH>
__global__ __launch_bounds__(256) void wino_f63_gemm_output_kernel(const float *__restrict__ v, const float *__restrict__ u,
                                                                  WinoGeom g, const float *__restrict__ bias, int act, float slope,
                                                                  int64_t act_body, float *__restrict__ out) {
    __shared__ float ms[64 * WF_COUT * WF_TILES];           // M[f][cout][tile]
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int total_tiles = g.n * g.tiles;
    const int t0 = blockIdx.x * WF_TILES, co0 = blockIdx.y * WF_COUT;
    // operand rows / columns of this lane (beyond the edge: the last one again; computed, never stored)
    const int a_co = min(co0 + lane % 16, g.cout - 1);
    const int b_t = min(t0 + lane % 16, total_tiles - 1);
    const int b_img = b_t / g.tiles, b_tile = b_t - b_img * g.tiles;
    const int kgrp = (lane / 16) * 4;
    const bool a_vec = g.c % 4 == 0 && reinterpret_cast<uintptr_t>(u) % 16 == 0;
    wf_v4f acc[16];
#pragma unroll
    for (int f = 0; f < 16; ++f) acc[f] = wf_v4f{0.f, 0.f, 0.f, 0.f};
    if constexpr (BLOCKS > 0) {
        constexpr int RING = 16, STEPS = 16 * BLOCKS;
        float av[RING][4], bv[RING][4];
        auto load = [&](auto stepc) __attribute__((always_inline)) {
            constexpr int step = decltype(stepc)::value;
            constexpr int s = step % RING;
            const int f = wave * 16 + step / BLOCKS, k0 = (step % BLOCKS) * 16 + kgrp;
            const wf_v4f t = *reinterpret_cast<const wf_v4f *>(u + (int64_t(f) * g.cout + a_co) * g.c + k0);
            static_for<0, 4>([&](auto ic) { av[s][decltype(ic)::value] = t[decltype(ic)::value]; });
            const float *bp = v + ((int64_t(b_img) * 64 + f) * g.c + k0) * g.tiles + b_tile;
            static_for<0, 4>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                bv[s][i] = bp[int64_t(i) * g.tiles];
            });
        };
        static_for<0, RING - 1>([&](auto sc) { load(sc); });
        static_for<0, STEPS>([&](auto stepc) {
            constexpr int step = decltype(stepc)::value;
            if constexpr (step + RING - 1 < STEPS) load(std::integral_constant<int, step + RING - 1>{});
            static_for<0, 4>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                acc[step / BLOCKS] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[step % RING][i], bv[step % RING][i], acc[step / BLOCKS], 0, 0, 0);
            });
        });
    } else {
    // 16-channel blocks per frequency, rounded up to whole rounds of the ring (blocks beyond C multiply zeros)
    const int blocks = (g.c + 16 * WF_DEPTH - 1) / (16 * WF_DEPTH) * WF_DEPTH;
    const int steps = 16 * blocks;            // (frequency, block) pairs of this wavefront, frequency-major

    float av[WF_DEPTH][4], bv[WF_DEPTH][4];
    // unconditional loads from clamped addresses; what lies beyond C is zeroed where the block is used
    auto load = [&](auto slot, int step) __attribute__((always_inline)) {
        constexpr int s = decltype(slot)::value;
        if (step >= steps) step = steps - 1;
        const int f = wave * 16 + step / blocks, k0 = (step % blocks) * 16 + kgrp;
        const float *ap = u + (int64_t(f) * g.cout + a_co) * g.c;
        const float *bp = v + ((int64_t(b_img) * 64 + f) * g.c) * g.tiles + b_tile;
        if (a_vec) {
            const wf_v4f t = *reinterpret_cast<const wf_v4f *>(ap + max(0, min(k0, g.c - 4)));
            static_for<0, 4>([&](auto ic) { av[s][decltype(ic)::value] = t[decltype(ic)::value]; });
        } else {
            static_for<0, 4>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                av[s][i] = ap[min(k0 + i, g.c - 1)];
            });
        }
        static_for<0, 4>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            bv[s][i] = bp[int64_t(min(k0 + i, g.c - 1)) * g.tiles];
        });
    };

    static_for<0, WF_DEPTH - 1>([&](auto sc) { load(sc, decltype(sc)::value); });
    int step = 0;
    static_for<0, 16>([&](auto fc) {
        constexpr int fl = decltype(fc)::value;
        for (int blk = 0; blk < blocks; blk += WF_DEPTH) {
            static_for<0, WF_DEPTH>([&](auto uc) {
                constexpr int uu = decltype(uc)::value;       // = step % WF_DEPTH: every frequency starts a round
                load(std::integral_constant<int, (uu + WF_DEPTH - 1) % WF_DEPTH>{}, step + WF_DEPTH - 1);
                const int k0 = (blk + uu) * 16 + kgrp;
                static_for<0, 4>([&](auto ic) {
                    constexpr int i = decltype(ic)::value;
                    const bool ok = k0 + i < g.c;
                    acc[fl] = __builtin_amdgcn_mfma_f32_16x16x4f32(ok ? av[uu][i] : 0.f, ok ? bv[uu][i] : 0.f, acc[fl], 0, 0, 0);
                });
                ++step;
            });
        }
    });
    }

    // ---- M[f][cout][tile] into LDS, then one thread per (cout, tile)
#pragma unroll
    for (int fl = 0; fl < 16; ++fl) {
        const int f = wave * 16 + fl;
#pragma unroll
        for (int r = 0; r < 4; ++r) ms[(f * WF_COUT + 4 * (lane / 16) + r) * WF_TILES + lane % 16] = acc[fl][r];
    }
    __syncthreads();
    const int co = co0 + tid / WF_TILES;
    const int my_t = t0 + tid % WF_TILES;
    if (my_t >= total_tiles || co >= g.cout) return;
    const int my_img = my_t / g.tiles, my_tile = my_t - my_img * g.tiles;
    const int my_ty = my_tile / g.tw, my_tx = my_tile - my_ty * g.tw;
    float tmpa[8][6];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float t8[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) t8[j] = ms[((i * 8 + j) * WF_COUT + tid / WF_TILES) * WF_TILES + tid % WF_TILES];
        at_pass(t8, tmpa[i]);
    }
    const float bvv = bias ? bias[co] : 0.f;
    const int64_t plane = (int64_t(my_img) * g.cout + co) * g.ho * g.wo;
#pragma unroll
    for (int i = 0; i < 6; ++i) {
        float t8[8], o[6];
#pragma unroll
        for (int r = 0; r < 8; ++r) t8[r] = tmpa[r][i];
        at_pass(t8, o);
        const int ww = my_tx * 6 + i;
#pragma unroll
        for (int r = 0; r < 6; ++r) {
            const int hh = my_ty * 6 + r;
            if (hh < g.ho && ww < g.wo) {
                float val = o[r];
                if (bias) val = __fadd_rn(val, bvv);
                const int64_t idx = plane + hh * g.wo + ww;
                out[idx] = MISH ? apply_act(val, act, slope, idx < act_body) : apply_act_basic(val, act, slope, idx < act_body);
            }
        }
    }
}

// ---------------------------------------------------------------- F(2,3)

// U[t = i*4+j][cout][cin] = (G g G^T)[i][j], G = {1,0,0; 1/2,1/2,1/2; 1/2,-1/2,1/2; 0,0,1}
// (winograd_algorithm.cpp:57-105, before its pack8_A); same contraction as the F(6,3) transform.
__global__ __launch_bounds__(256) void wino23_kernel_transform_kernel(const float *__restrict__ w, int cout, int cin,
                                                                     float *__restrict__ u) {
    const int id = blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= cout * cin) return;
    const float G[4][3] = {{1.f, 0.f, 0.f}, {0.5f, 0.5f, 0.5f}, {0.5f, -0.5f, 0.5f}, {0.f, 0.f, 1.f}};
    float g[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) g[i] = w[int64_t(id) * 9 + i];
    float tmp[3][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 3; ++r)
            tmp[r][i] = fmaf(g[r * 3 + 2], G[i][2], fmaf(g[r * 3 + 0], G[i][0], g[r * 3 + 1] * G[i][1]));
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            u[int64_t(i * 4 + j) * cout * cin + id] =
                fmaf(tmp[2][j], G[i][2], fmaf(tmp[0][j], G[i][0], tmp[1][j] * G[i][1]));
}

// V = B^T d B (winograd_algorithm.cpp:181-243): row combinations (i0-i2, i1+i2, i2-i1, i1-i3) first,
// then the same combination across columns, in the reference's grouping.
__global__ __launch_bounds__(256) void wino23_input_transform_kernel(const float *__restrict__ x, WinoGeom g,
                                                                    float *__restrict__ v) {
    const int64_t total = int64_t(g.n) * g.c * g.tiles;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int tile = int(id % g.tiles);
    const int ch = int((id / g.tiles) % g.c);
    const int img = int(id / g.tiles / g.c);
    const int ty = tile / g.tw, tx = tile - ty * g.tw;
    const float *src = x + (int64_t(img) * g.c + ch) * g.h * g.w;
    float d[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int hh = ty * 2 + i - g.pad_top;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int ww = tx * 2 + j - g.pad_left;
            d[i][j] = (hh >= 0 && hh < g.h && ww >= 0 && ww < g.w) ? src[hh * g.w + ww] : g.padding_value;
        }
    }
    float *dst = v + (int64_t(img) * 16 * g.c + ch) * g.tiles + tile;
    const int64_t stride = int64_t(g.c) * g.tiles;
    float r[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        r[0][j] = d[0][j] - d[2][j];
        r[1][j] = d[1][j] + d[2][j];
        r[2][j] = d[2][j] - d[1][j];
        r[3][j] = d[1][j] - d[3][j];
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        dst[(k * 4 + 0) * stride] = r[k][0] - r[k][2];
        dst[(k * 4 + 1) * stride] = r[k][1] + r[k][2];
        dst[(k * 4 + 2) * stride] = r[k][2] - r[k][1];
        dst[(k * 4 + 3) * stride] = r[k][1] - r[k][3];
    }
}

// Y = A^T M A (winograd_algorithm.cpp:262-330), cut to the true output, + optional bias / activation.
template <bool MISH>
__global__ __launch_bounds__(256) void wino23_output_transform_kernel(const float *__restrict__ mm, WinoGeom g,
                                                                     const float *__restrict__ bias, int act,
                                                                     float slope, int64_t act_body,
                                                                     float *__restrict__ out) {
    const int64_t total = int64_t(g.n) * g.cout * g.tiles;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int tile = int(id % g.tiles);
    const int co = int((id / g.tiles) % g.cout);
    const int img = int(id / g.tiles / g.cout);
    const int ty = tile / g.tw, tx = tile - ty * g.tw;
    const float *src = mm + (int64_t(img) * 16 * g.cout + co) * g.tiles + tile;
    const int64_t stride = int64_t(g.cout) * g.tiles;
    float m[16], a[8], o[4];
#pragma unroll
    for (int t = 0; t < 16; ++t) m[t] = src[t * stride];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        a[2 * k] = m[4 * k] + m[4 * k + 1] + m[4 * k + 2];
        a[2 * k + 1] = m[4 * k + 1] - m[4 * k + 2] - m[4 * k + 3];
    }
    o[0] = a[0] + a[2] + a[4];
    o[1] = a[1] + a[3] + a[5];
    o[2] = a[2] - a[4] - a[6];
    o[3] = a[3] - a[5] - a[7];
    const float bv = bias ? bias[co] : 0.f;
    const int64_t plane = (int64_t(img) * g.cout + co) * g.ho * g.wo;
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int hh = ty * 2 + r, ww = tx * 2 + i;
            if (hh < g.ho && ww < g.wo) {
                float val = o[r * 2 + i];
                if (bias) val = __fadd_rn(val, bv);
                const int64_t idx = plane + hh * g.wo + ww;
                out[idx] = MISH ? apply_act(val, act, slope, idx < act_body) : apply_act_basic(val, act, slope, idx < act_body);
            }
        }
}

int make_geom(const tsx_conv2d_geom *q, float padding_value, WinoGeom *g, int tile = 6) {
    TSX_REQUIRE(q, "winograd: null geometry");
    TSX_REQUIRE(q->kh == 3 && q->kw == 3 && q->stride_h == 1 && q->stride_w == 1 && q->dilation_h == 1 &&
                    q->dilation_w == 1,
                "winograd: needs a 3x3 kernel with stride 1 and dilation 1");
    TSX_REQUIRE(q->n > 0 && q->c > 0 && q->h > 0 && q->w > 0 && q->cout > 0, "winograd: non-positive extent");
    TSX_REQUIRE(q->pad_top >= 0 && q->pad_bottom >= 0 && q->pad_left >= 0 && q->pad_right >= 0,
                "winograd: negative padding is not supported");
    g->n = q->n;
    g->c = q->c;
    g->h = q->h;
    g->w = q->w;
    g->cout = q->cout;
    g->ho = q->h + q->pad_top + q->pad_bottom - 2;
    g->wo = q->w + q->pad_left + q->pad_right - 2;
    TSX_REQUIRE(g->ho > 0 && g->wo > 0, "winograd: empty output %dx%d", g->ho, g->wo);
    g->pad_top = q->pad_top;
    g->pad_left = q->pad_left;
    g->th = (g->ho + tile - 1) / tile;
    g->tw = (g->wo + tile - 1) / tile;
    g->tiles = g->th * g->tw;
    g->padding_value = padding_value;
    return 0;
}

}  // namespace
}  // namespace tsx

extern "C" {

size_t tsx_winograd_f63_kernel_bytes(int32_t cout, int32_t cin) {
    if (cout <= 0 || cin <= 0) return 0;
    return size_t(64) * size_t(cout) * size_t(cin) * sizeof(float);
}

int tsx_winograd_f63_transform_kernel(int32_t cout, int32_t cin, const float *w_oihw_dev, float *u_dev, void *stream) {
    TSX_REQUIRE(cout > 0 && cin > 0 && w_oihw_dev && u_dev, "winograd_f63_transform_kernel: bad argument");
    const int total = cout * cin;
    hipLaunchKernelGGL(tsx::wino_kernel_transform_kernel, dim3(unsigned(tsx::ceil_div(total, 256))), dim3(256), 0,
                       tsx::as_stream(stream), w_oihw_dev, cout, cin, u_dev);
    TSX_LAUNCH_CHECK("wino_kernel_transform_kernel");
    return 0;
}

size_t tsx_winograd_f63_workspace_bytes(const tsx_conv2d_geom *q) {
    tsx::WinoGeom g;
    if (tsx::make_geom(q, 0.f, &g)) return 0;
    return size_t(g.n) * 64 * g.tiles * (size_t(g.c) + size_t(g.cout)) * sizeof(float);
}

int tsx_conv2d_winograd_f63_nchw(const tsx_conv2d_geom *q, const float *x_dev, const float *u_dev, float padding_value,
                                 const float *bias_dev, int32_t act, float slope, float *out_dev, void *workspace_dev,
                                 size_t workspace_bytes, void *stream_) {
    tsx::WinoGeom g;
    int rc = tsx::make_geom(q, padding_value, &g);
    if (rc) return rc;
    TSX_REQUIRE(x_dev && u_dev && out_dev, "winograd: null argument");
    TSX_REQUIRE(act >= TSX_ACT_NONE && act <= TSX_ACT_MISH_FAST, "winograd: unknown activation %d", act);
    const size_t need = tsx_winograd_f63_workspace_bytes(q);
    if (!workspace_dev || workspace_bytes < need)
        return tsx::fail(TSX_E_WORKSPACE, "winograd: workspace %zu < %zu bytes", workspace_bytes, need);
    hipStream_t stream = tsx::as_stream(stream_);
    float *v = static_cast<float *>(workspace_dev);
    float *mm = v + size_t(g.n) * 64 * g.c * g.tiles;

    const int64_t in_threads = int64_t(g.n) * g.c * g.tiles;
    hipLaunchKernelGGL(tsx::wino_input_transform_kernel, dim3(unsigned(tsx::ceil_div(in_threads, 256))), dim3(256), 0,
                       stream, x_dev, g, v);
    TSX_LAUNCH_CHECK("wino_input_transform_kernel");

    const int batches = g.n * 64;
    if (int rc = tsx::launch_gemm_f32_seq(u_dev, v, mm, g.cout, g.tiles, g.c, batches, 64, stream)) return rc;

    const int64_t out_threads = int64_t(g.n) * g.cout * g.tiles;
    const int64_t count = int64_t(g.n) * g.cout * g.ho * g.wo;
    if (act >= TSX_ACT_MISH)
        hipLaunchKernelGGL(tsx::wino_output_transform_kernel<true>, dim3(unsigned(tsx::ceil_div(out_threads, 256))), dim3(256), 0,
                           stream, mm, g, bias_dev, act, slope, count / 4 * 4, out_dev);
    else
        hipLaunchKernelGGL(tsx::wino_output_transform_kernel<false>, dim3(unsigned(tsx::ceil_div(out_threads, 256))), dim3(256), 0,
                           stream, mm, g, bias_dev, act, slope, count / 4 * 4, out_dev);
    TSX_LAUNCH_CHECK("wino_output_transform_kernel");
    return 0;
}

size_t tsx_winograd_f63_fast_workspace_bytes(const tsx_conv2d_geom *q) {
    tsx::WinoGeom g;
    if (tsx::make_geom(q, 0.f, &g)) return 0;
    return size_t(g.n) * 64 * g.tiles * size_t(g.c) * sizeof(float);
}

int tsx_conv2d_winograd_f63_fast_nchw(const tsx_conv2d_geom *q, const float *x_dev, const float *u_dev, float padding_value,
                                      const float *bias_dev, int32_t act, float slope, float *out_dev, void *workspace_dev,
                                      size_t workspace_bytes, void *stream_) {
    tsx::WinoGeom g;
    int rc = tsx::make_geom(q, padding_value, &g);
    if (rc) return rc;
    TSX_REQUIRE(x_dev && u_dev && out_dev, "winograd: null argument");
    TSX_REQUIRE(act >= TSX_ACT_NONE && act <= TSX_ACT_MISH_FAST, "winograd: unknown activation %d", act);
    const size_t need = tsx_winograd_f63_fast_workspace_bytes(q);
    if (!workspace_dev || workspace_bytes < need)
        return tsx::fail(TSX_E_WORKSPACE, "winograd: workspace %zu < %zu bytes", workspace_bytes, need);
    const int64_t total_tiles = int64_t(g.n) * g.tiles;
    TSX_REQUIRE(total_tiles < (int64_t(1) << 31) - tsx::WF_TILES, "winograd: too many tiles");
    hipStream_t stream = tsx::as_stream(stream_);
    float *v = static_cast<float *>(workspace_dev);
    const int64_t in_threads = int64_t(g.n) * g.c * g.tiles;
    hipLaunchKernelGGL(tsx::wino_input_transform_kernel, dim3(unsigned(tsx::ceil_div(in_threads, 256))), dim3(256), 0,
                       stream, x_dev, g, v);
    TSX_LAUNCH_CHECK("wino_input_transform_kernel");
    const int64_t count = int64_t(g.n) * g.cout * g.ho * g.wo;
    const dim3 grid(unsigned(tsx::ceil_div(total_tiles, int64_t(tsx::WF_TILES))), unsigned(tsx::ceil_div(g.cout, tsx::WF_COUT)));
    const bool aligned = reinterpret_cast<uintptr_t>(u_dev) % 16 == 0;
    const int blocks = aligned && (g.c == 64 || g.c == 128 || g.c == 256) ? g.c / 16 : 0;
    const bool mish = act >= TSX_ACT_MISH;
#define TSX_WF_LAUNCH(B, M)                                                                                         \
    hipLaunchKernelGGL((tsx::wino_f63_gemm_output_kernel<B, M>), grid, dim3(256), 0, stream, v, u_dev, g, bias_dev, act, \
                       slope, count / 4 * 4, out_dev)
    if (blocks == 4) { if (mish) TSX_WF_LAUNCH(4, true); else TSX_WF_LAUNCH(4, false); }
    else if (blocks == 8) { if (mish) TSX_WF_LAUNCH(8, true); else TSX_WF_LAUNCH(8, false); }
    else if (blocks == 16) { if (mish) TSX_WF_LAUNCH(16, true); else TSX_WF_LAUNCH(16, false); }
    else { if (mish) TSX_WF_LAUNCH(0, true); else TSX_WF_LAUNCH(0, false); }
#undef TSX_WF_LAUNCH
    TSX_LAUNCH_CHECK("wino_f63_gemm_output_kernel");
    return 0;
}

size_t tsx_winograd_f23_kernel_bytes(int32_t cout, int32_t cin) {
    if (cout <= 0 || cin <= 0) return 0;
    return size_t(16) * size_t(cout) * size_t(cin) * sizeof(float);
}

int tsx_winograd_f23_transform_kernel(int32_t cout, int32_t cin, const float *w_oihw_dev, float *u_dev, void *stream) {
    TSX_REQUIRE(cout > 0 && cin > 0 && w_oihw_dev && u_dev, "winograd_f23_transform_kernel: bad argument");
    const int total = cout * cin;
    hipLaunchKernelGGL(tsx::wino23_kernel_transform_kernel, dim3(unsigned(tsx::ceil_div(total, 256))), dim3(256), 0,
                       tsx::as_stream(stream), w_oihw_dev, cout, cin, u_dev);
    TSX_LAUNCH_CHECK("wino23_kernel_transform_kernel");
    return 0;
}

size_t tsx_winograd_f23_workspace_bytes(const tsx_conv2d_geom *q) {
    tsx::WinoGeom g;
    if (tsx::make_geom(q, 0.f, &g, 2)) return 0;
    return size_t(g.n) * 16 * g.tiles * (size_t(g.c) + size_t(g.cout)) * sizeof(float);
}

int tsx_conv2d_winograd_f23_nchw(const tsx_conv2d_geom *q, const float *x_dev, const float *u_dev, float padding_value,
                                 const float *bias_dev, int32_t act, float slope, float *out_dev, void *workspace_dev,
                                 size_t workspace_bytes, void *stream_) {
    tsx::WinoGeom g;
    int rc = tsx::make_geom(q, padding_value, &g, 2);
    if (rc) return rc;
    TSX_REQUIRE(x_dev && u_dev && out_dev, "winograd_f23: null argument");
    TSX_REQUIRE(act >= TSX_ACT_NONE && act <= TSX_ACT_MISH_FAST, "winograd_f23: unknown activation %d", act);
    const size_t need = tsx_winograd_f23_workspace_bytes(q);
    if (!workspace_dev || workspace_bytes < need)
        return tsx::fail(TSX_E_WORKSPACE, "winograd_f23: workspace %zu < %zu bytes", workspace_bytes, need);
    hipStream_t stream = tsx::as_stream(stream_);
    float *v = static_cast<float *>(workspace_dev);
    float *mm = v + size_t(g.n) * 16 * g.c * g.tiles;

    const int64_t in_threads = int64_t(g.n) * g.c * g.tiles;
    hipLaunchKernelGGL(tsx::wino23_input_transform_kernel, dim3(unsigned(tsx::ceil_div(in_threads, 256))), dim3(256), 0,
                       stream, x_dev, g, v);
    TSX_LAUNCH_CHECK("wino23_input_transform_kernel");

    const int batches = g.n * 16;
    if (int rc = tsx::launch_gemm_f32_seq(u_dev, v, mm, g.cout, g.tiles, g.c, batches, 16, stream)) return rc;

    const int64_t out_threads = int64_t(g.n) * g.cout * g.tiles;
    const int64_t count = int64_t(g.n) * g.cout * g.ho * g.wo;
    if (act >= TSX_ACT_MISH)
        hipLaunchKernelGGL(tsx::wino23_output_transform_kernel<true>, dim3(unsigned(tsx::ceil_div(out_threads, 256))), dim3(256), 0,
                           stream, mm, g, bias_dev, act, slope, count / 4 * 4, out_dev);
    else
        hipLaunchKernelGGL(tsx::wino23_output_transform_kernel<false>, dim3(unsigned(tsx::ceil_div(out_threads, 256))), dim3(256), 0,
                           stream, mm, g, bias_dev, act, slope, count / 4 * 4, out_dev);
    TSX_LAUNCH_CHECK("wino23_output_transform_kernel");
    return 0;
}

}  // extern "C"
