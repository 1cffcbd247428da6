// fp32 GEMM-shaped kernels on the gfx950 fp32 MFMA (v_mfma_f32_32x32x2_f32):
//   * conv2d as implicit im2col-GEMM straight from NCHW (no col buffer), standing in for
//     cpu::Conv2DCore::conv2d (src/kernels/cpu/conv2d_core.cpp:17-119: im2col_cpu + pack8 +
//     kernel_8x8 of src/kernels/cpu/math_cpu.cpp:386-743);
//   * inner_prod, standing in for cpu::InnerProd (src/kernels/cpu/inner_prod.cpp:19-74);
//   * the strided-batch GEMM used by the Winograd path.
// One kernel, three ways of fetching the B operand.  C[m][n] = sum_k A[m][k] * B[k][n] with
// A row-major [M][K] (OIHW weights are exactly that with K = Cin*KH*KW), accumulated in the
// MFMA's fp32 accumulators; the summation order differs from the reference's sequential FMA
// chain, which the parity tolerance (1e-4 relative / 1e-5 absolute) covers.
//
// Tiling: a workgroup of 4 wavefronts owns a (32*WM) x (32*WN) output tile; K is consumed in
// chunks of 32 staged through LDS (A padded to 33 floats per row, both operand reads
// conflict-free); with WK > 1 the wavefronts split each chunk's K range and reduce through
// LDS at the end -- that is what fills the machine for small problems such as a single
// 64-channel 56x56 layer.
//
// MFMA layout (32x32x2 f32): lane l supplies A[row l%32][k l/32] and B[k l/32][col l%32];
// accumulator register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32.
#include "gemm_f32.hpp"

namespace tsx {
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int KC = 32;          // K per staged chunk
constexpr int THREADS = 256;

constexpr int MAX_SLOTS = 8;    // B elements a thread fetches per chunk (KC * BN / THREADS at BN = 64)

// B operand = implicit im2col of an NCHW tensor (src/kernels/cpu/im2col.cpp:37-111).
struct ConvLoader {
    const float *x;
    int c, h, w, kh, kw, pad_top, pad_left, stride_h, stride_w, dil_h, dil_w, wo, howo;
    float padding_value;
    // per-thread column state
    const float *img;
    int h0, w0;
    bool col_ok;
    __device__ __forceinline__ void set_column(int col, int ncols) {
        col_ok = col < ncols;
        const int cc = col_ok ? col : 0;
        const int n = cc / howo;
        const int r = cc - n * howo;
        const int ho = r / wo, wo_ = r - ho * wo;
        img = x + int64_t(n) * c * h * w;
        h0 = ho * stride_h - pad_top;
        w0 = wo_ * stride_w - pad_left;
    }
    // A thread fetches the same few rows k of every staged chunk, KC further each time: row k is kept as
    // (input channel, tap) and stepped, so the K loop has no division (tap -> kernel row / column is a
    // multiply-shift, exact for the tap counts of any real kernel).
    int slot_ci[MAX_SLOTS], slot_tap[MAX_SLOTS], slot_k[MAX_SLOTS];
    __device__ __forceinline__ void init_slot(int i, int k) {
        const int khw = kh * kw;
        slot_k[i] = k;
        slot_ci[i] = k / khw;
        slot_tap[i] = k - slot_ci[i] * khw;
    }
    __device__ __forceinline__ void advance_slot(int i, int step) {
        const int khw = kh * kw;
        slot_k[i] += step;
        slot_ci[i] += step / khw;
        slot_tap[i] += step % khw;
        if (slot_tap[i] >= khw) {
            slot_tap[i] -= khw;
            ++slot_ci[i];
        }
    }
    __device__ __forceinline__ float load_slot(int i, int kdim) const {
        if (!col_ok || slot_k[i] >= kdim) return 0.f;
        const int inv_kw = (65536 + kw - 1) / kw;
        const int r = (slot_tap[i] * inv_kw) >> 16, s = slot_tap[i] - r * kw;
        const int hh = h0 + r * dil_h, ww = w0 + s * dil_w;
        if (hh < 0 || hh >= h || ww < 0 || ww >= w) return padding_value;
        return img[(int64_t(slot_ci[i]) * h + hh) * w + ww];
    }
};

// B operand = plain matrix: element (k, n) at b[k*ld_k + n*ld_n] (+ batch stride).
struct MatLoader {
    const float *b;
    int64_t ld_k, ld_n;
    const float *colp;
    bool col_ok;
    __device__ __forceinline__ void set_column(int col, int ncols) {
        col_ok = col < ncols;
        colp = b + int64_t(col_ok ? col : 0) * ld_n;
    }
    int slot_k[MAX_SLOTS];
    __device__ __forceinline__ void init_slot(int i, int k) { slot_k[i] = k; }
    __device__ __forceinline__ void advance_slot(int i, int step) { slot_k[i] += step; }
    __device__ __forceinline__ float load_slot(int i, int kdim) const {
        if (!col_ok || slot_k[i] >= kdim) return 0.f;
        return colp[int64_t(slot_k[i]) * ld_k];
    }
};

struct GemmArgs {
    const float *a;       // [M][K] row-major (+ batch stride)
    float *c;             // output
    int m, n, k;
    int64_t a_batch, b_batch, c_batch;
    // output index of (row, col): conv: ((col / howo) * m + row) * howo + col % howo ; matrix: row*n + col
    int howo;             // 0 for plain matrix output
    const float *bias;    // [M] or nullptr  (cpu::AddBias, add_bias.cpp:47-85)
    int act;              // TSX_ACT_*
    float slope;
    int64_t act_body;     // elements of the output inside the activation's SIMD body
};

template <class Loader, int WM, int WN, int WK>
__global__ __launch_bounds__(THREADS) void gemm_f32_kernel(GemmArgs g, Loader ld) {
    static_assert(WM * WN * WK == 4, "four wavefronts per workgroup");
    constexpr int BM = 32 * WM, BN = 32 * WN;
    constexpr int A_PER = BM * KC / THREADS, B_PER = KC * BN / THREADS;
    constexpr int KW_ = KC / WK;                    // K range of one wavefront inside a chunk
    __shared__ float as[BM][KC + 1];
    __shared__ float bs[KC][BN];
    __shared__ float red[WK > 1 ? (WK - 1) * BM * BN : 1];

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wk = wave % WK, wn = (wave / WK) % WN, wm = wave / (WK * WN);
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int batch = blockIdx.z;
    const float *a = g.a + batch * g.a_batch;
    if constexpr (std::is_same<Loader, MatLoader>::value) ld.b += batch * g.b_batch;

    static_assert(B_PER <= MAX_SLOTS, "more B elements per thread than loader slots");
    ld.set_column(n0 + tid % BN, g.n);
    const int b_krow = tid / BN;                    // this thread's first k row of the B tile
    static_for<0, B_PER>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        ld.init_slot(i, b_krow + i * (THREADS / BN));
    });

    v16f acc;
    static_for<0, 16>([&](auto rc) { acc[decltype(rc)::value] = 0.f; });

    float a_reg[A_PER], b_reg[B_PER];
    auto load_chunk = [&](int k0) __attribute__((always_inline)) {
        static_for<0, A_PER>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int idx = tid + i * THREADS;
            const int mm = idx / KC, kk = idx % KC;
            const bool ok = m0 + mm < g.m && k0 + kk < g.k;
            a_reg[i] = ok ? a[int64_t(m0 + mm) * g.k + k0 + kk] : 0.f;
        });
        static_for<0, B_PER>([&](auto ic) {      // chunks are fetched in ascending order: the slots step with them
            constexpr int i = decltype(ic)::value;
            b_reg[i] = ld.load_slot(i, g.k);
            ld.advance_slot(i, KC);
        });
    };
    auto store_chunk = [&]() __attribute__((always_inline)) {
        static_for<0, A_PER>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int idx = tid + i * THREADS;
            as[idx / KC][idx % KC] = a_reg[i];
        });
        static_for<0, B_PER>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            bs[b_krow + i * (THREADS / BN)][tid % BN] = b_reg[i];
        });
    };

    load_chunk(0);
    for (int k0 = 0; k0 < g.k; k0 += KC) {
        __syncthreads();            // previous chunk fully consumed
        store_chunk();
        __syncthreads();
        if (k0 + KC < g.k) load_chunk(k0 + KC);     // in flight during the MFMAs
        const int row = wm * 32 + lane % 32, col = wn * 32 + lane % 32;
        static_for<0, KW_ / 2>([&](auto sc) {
            constexpr int s = decltype(sc)::value;
            const int kk = wk * KW_ + s * 2 + lane / 32;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as[row][kk], bs[kk][col], acc, 0, 0, 0);
        });
    }

    // reduce the K split: wavefronts wk > 0 hand their partial tile to wk == 0
    if constexpr (WK > 1) {
        __syncthreads();
        if (wk > 0) {
            static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                const int rr = wm * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4), cc = wn * 32 + lane % 32;
                red[((wk - 1) * BM + rr) * BN + cc] = acc[r];
            });
        }
        __syncthreads();
        if (wk > 0) return;
        static_for<0, WK - 1>([&](auto wc) {
            constexpr int w = decltype(wc)::value;
            static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                const int rr = wm * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4), cc = wn * 32 + lane % 32;
                acc[r] += red[(w * BM + rr) * BN + cc];
            });
        });
    }

    const int col = n0 + wn * 32 + lane % 32;
    if (col >= g.n) return;
    int64_t col_base;
    int64_t row_stride;
    if (g.howo > 0) {
        const int n = col / g.howo;
        col_base = int64_t(n) * g.m * g.howo + (col - n * g.howo);
        row_stride = g.howo;
    } else {
        col_base = col;
        row_stride = g.n;
    }
    float *c = g.c + batch * g.c_batch;
    static_for<0, 16>([&](auto rc) {
        constexpr int r = decltype(rc)::value;
        const int row = m0 + wm * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
        if (row < g.m) {
            const int64_t idx = col_base + int64_t(row) * row_stride;
            float v = acc[r];
            if (g.bias) v = __fadd_rn(v, g.bias[row]);
            c[idx] = apply_act_basic(v, g.act, g.slope, idx < g.act_body);   // the entry points take none / relu / leaky_relu
        }
    });
}

// inner_prod with few rows (a classifier behind a batch of 32: M = 32, K = 2048, N = 1000).  The tiled kernel
// above gives such a problem 32 workgroups that each walk all of K chunk by chunk, one global round trip per
// chunk.  Here a workgroup owns a 16 x 16 output tile on v_mfma_f32_16x16x4_f32, its eight wavefronts take an
// eighth of K each, operands go from global memory straight into the MFMA operand registers (no LDS staging)
// with seven 16-deep K blocks in flight per wavefront (the right operand streams from HBM once: what bounds the
// kernel is how many bytes are in flight), and the eighths are summed through LDS in a fixed order
// (results do not depend on timing).  Lane l holds A[row l%16][4 consecutive k of group l/16] as one 16-byte
// load, and B[those k][col l%16]; the four MFMAs of a block take k group by group -- the sum over k does not
// care which k an MFMA step carries.  Accumulator register r of lane l is row 4*(l/16) + r, column l%16.
typedef float v4f __attribute__((ext_vector_type(4)));

struct SkinnyArgs {
    const float *a, *b;
    float *c;
    int m, n, k;
    int64_t ld_k, ld_n;   // element (k, n) of the right operand at b[k*ld_k + n*ld_n]
};

constexpr int SK_DEPTH = 8;   // ring of K blocks (16 k each) per wavefront: SK_DEPTH - 1 in flight
constexpr int SK_WAVES = 8;

__global__ __launch_bounds__(64 * SK_WAVES) void inner_prod_skinny_kernel(SkinnyArgs g) {
    __shared__ float part[SK_WAVES - 1][256];
    const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    const int row = min(int(blockIdx.y) * 16 + lane % 16, g.m - 1);      // rows / columns beyond the edge repeat the
    const int col = min(int(blockIdx.x) * 16 + lane % 16, g.n - 1);      // last one: computed, never stored
    const int kgrp = (lane / 16) * 4;
    const int blocks = (g.k + 15) / 16;
    const int per_wave = (blocks + SK_WAVES - 1) / SK_WAVES;
    const int b0 = wave * per_wave, b1 = min(blocks, b0 + per_wave);
    const float *ap = g.a + int64_t(row) * g.k;
    const float *bp = g.b + int64_t(col) * g.ld_n;
    const bool a_vec = g.k % 4 == 0 && reinterpret_cast<uintptr_t>(g.a) % 16 == 0;

    float av[SK_DEPTH][4], bv[SK_DEPTH][4];
    // Unconditional loads from clamped addresses (a load behind a branch is waited for before the next one is
    // issued); what lies beyond K or beyond this wavefront's range is zeroed where the block is USED, so that
    // nothing between a load and its use seven blocks later needs the loaded value.
    auto load = [&](auto slot, int blk) __attribute__((always_inline)) {
        constexpr int s = decltype(slot)::value;
        const int k0 = blk * 16 + kgrp;
        if (a_vec) {
            const v4f t = *reinterpret_cast<const v4f *>(ap + max(0, min(k0, g.k - 4)));
            static_for<0, 4>([&](auto ic) { av[s][decltype(ic)::value] = t[decltype(ic)::value]; });
        } else {
            static_for<0, 4>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                av[s][i] = ap[min(k0 + i, g.k - 1)];
            });
        }
        static_for<0, 4>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            bv[s][i] = bp[int64_t(min(k0 + i, g.k - 1)) * g.ld_k];
        });
    };

    v4f acc = {0.f, 0.f, 0.f, 0.f};
    static_for<0, SK_DEPTH - 1>([&](auto sc) { load(sc, b0 + decltype(sc)::value); });
    for (int blk = b0; blk < b1; blk += SK_DEPTH) {
        // all SK_DEPTH blocks of this round inside the wavefront's range and inside K: no masking
        const bool whole = blk + SK_DEPTH <= b1 && (blk + SK_DEPTH) * 16 <= g.k;
        static_for<0, SK_DEPTH>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            load(std::integral_constant<int, (u + SK_DEPTH - 1) % SK_DEPTH>{}, blk + u + SK_DEPTH - 1);
            const int k0 = (blk + u) * 16 + kgrp;
            const bool live = blk + u < b1;
            static_for<0, 4>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                // with K % 4 == 0 the clamped 16-byte load is the lane's own four values whenever any of them is inside K
                const bool ok = whole || (live && k0 + i < g.k);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ok ? av[u][i] : 0.f, ok ? bv[u][i] : 0.f, acc, 0, 0, 0);
            });
        });
    }

    if (wave > 0) {
        static_for<0, 4>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            part[wave - 1][r * 64 + lane] = acc[r];
        });
    }
    __syncthreads();
    if (wave > 0) return;
    const int orow = int(blockIdx.y) * 16 + 4 * (lane / 16), ocol = int(blockIdx.x) * 16 + lane % 16;
    static_for<0, 4>([&](auto rc) {
        constexpr int r = decltype(rc)::value;
        float v = acc[r];
        static_for<0, SK_WAVES - 1>([&](auto wc) { v += part[decltype(wc)::value][r * 64 + lane]; });
        if (orow + r < g.m && ocol < g.n) g.c[int64_t(orow + r) * g.n + ocol] = v;
    });
}

template <class Loader>
int launch(const GemmArgs &g, const Loader &ld, int batches, hipStream_t stream) {
    // Big problems: 64x64 tiles, no K split.  Small ones (fewer tiles than SIMDs): 32x32 tiles
    // with the four wavefronts splitting K, so a single small layer still spreads over the chip.
    const int64_t tiles64 = ceil_div(g.m, 64) * ceil_div(g.n, 64) * batches;
    if (tiles64 >= 512 || g.k < 4 * KC) {
        dim3 grid(unsigned(ceil_div(g.n, 64)), unsigned(ceil_div(g.m, 64)), unsigned(batches));
        hipLaunchKernelGGL((gemm_f32_kernel<Loader, 2, 2, 1>), grid, dim3(THREADS), 0, stream, g, ld);
    } else {
        dim3 grid(unsigned(ceil_div(g.n, 32)), unsigned(ceil_div(g.m, 32)), unsigned(batches));
        hipLaunchKernelGGL((gemm_f32_kernel<Loader, 1, 1, 4>), grid, dim3(THREADS), 0, stream, g, ld);
    }
    TSX_LAUNCH_CHECK("gemm_f32_kernel");
    return 0;
}

}  // namespace

int gemm_f32_batched(const float *a, int64_t a_batch, const float *b, int64_t ld_k, int64_t ld_n, int64_t b_batch,
                     float *c, int64_t c_batch, int m, int n, int k, int batches, hipStream_t stream) {
    GemmArgs g{};
    g.a = a;
    g.c = c;
    g.m = m;
    g.n = n;
    g.k = k;
    g.a_batch = a_batch;
    g.b_batch = b_batch;
    g.c_batch = c_batch;
    g.howo = 0;
    g.act = TSX_ACT_NONE;
    MatLoader ld{};
    ld.b = b;
    ld.ld_k = ld_k;
    ld.ld_n = ld_n;
    return launch(g, ld, batches, stream);
}

}  // namespace tsx

extern "C" {

int tsx_conv2d_f32_nchw(const tsx_conv2d_geom *geo, const float *x_dev, const float *w_oihw_dev, float padding_value,
                        const float *bias_dev, int32_t act, float slope, float *out_dev, void *stream) {
    TSX_REQUIRE(geo && x_dev && w_oihw_dev && out_dev, "conv2d_f32: null argument");
    TSX_REQUIRE(geo->n > 0 && geo->c > 0 && geo->h > 0 && geo->w > 0 && geo->cout > 0 && geo->kh > 0 && geo->kw > 0,
                "conv2d_f32: non-positive extent");
    TSX_REQUIRE(geo->stride_h > 0 && geo->stride_w > 0 && geo->dilation_h > 0 && geo->dilation_w > 0,
                "conv2d_f32: stride and dilation must be positive");
    TSX_REQUIRE(act >= TSX_ACT_NONE && act <= TSX_ACT_LEAKY_RELU, "conv2d_f32: unknown activation %d", act);
    const int ho = tsx::conv_out(geo->h, geo->pad_top, geo->pad_bottom, geo->kh, geo->stride_h, geo->dilation_h);
    const int wo = tsx::conv_out(geo->w, geo->pad_left, geo->pad_right, geo->kw, geo->stride_w, geo->dilation_w);
    TSX_REQUIRE(ho > 0 && wo > 0, "conv2d_f32: empty output %dx%d", ho, wo);
    const int64_t cols = int64_t(geo->n) * ho * wo;
    TSX_REQUIRE(cols < (int64_t(1) << 31), "conv2d_f32: too many output positions");
    tsx::GemmArgs g{};
    g.a = w_oihw_dev;
    g.c = out_dev;
    g.m = geo->cout;
    g.n = int(cols);
    g.k = geo->c * geo->kh * geo->kw;
    g.howo = ho * wo;
    g.bias = bias_dev;
    g.act = act;
    g.slope = slope;
    g.act_body = (cols * geo->cout) / 4 * 4;
    tsx::ConvLoader ld{};
    ld.x = x_dev;
    ld.c = geo->c;
    ld.h = geo->h;
    ld.w = geo->w;
    ld.kh = geo->kh;
    ld.kw = geo->kw;
    ld.pad_top = geo->pad_top;
    ld.pad_left = geo->pad_left;
    ld.stride_h = geo->stride_h;
    ld.stride_w = geo->stride_w;
    ld.dil_h = geo->dilation_h;
    ld.dil_w = geo->dilation_w;
    ld.wo = wo;
    ld.howo = ho * wo;
    ld.padding_value = padding_value;
    return tsx::launch(g, ld, 1, tsx::as_stream(stream));
}

int tsx_inner_prod_f32(int32_t m, int32_t n, int32_t k, const float *lhs_dev, const float *rhs_dev, int32_t transpose,
                       float *out_dev, void *stream) {
    TSX_REQUIRE(m > 0 && n > 0 && k > 0, "inner_prod_f32: non-positive extent");
    TSX_REQUIRE(lhs_dev && rhs_dev && out_dev, "inner_prod_f32: null argument");
    if (m <= 64 && k >= 256) {
        // few rows: the tiled kernel would run on m/32 * n/32 workgroups, each walking all of K
        tsx::SkinnyArgs s{lhs_dev, rhs_dev, out_dev, m, n, k, transpose ? 1 : int64_t(n), transpose ? int64_t(k) : 1};
        hipLaunchKernelGGL(tsx::inner_prod_skinny_kernel, dim3(unsigned(tsx::ceil_div(n, 16)), unsigned(tsx::ceil_div(m, 16))),
                           dim3(64 * tsx::SK_WAVES), 0, tsx::as_stream(stream), s);
        TSX_LAUNCH_CHECK("inner_prod_skinny_kernel");
        return 0;
    }
    tsx::GemmArgs g{};
    g.a = lhs_dev;
    g.c = out_dev;
    g.m = m;
    g.n = n;
    g.k = k;
    g.howo = 0;
    g.bias = nullptr;
    g.act = TSX_ACT_NONE;
    tsx::MatLoader ld{};
    ld.b = rhs_dev;
    ld.ld_k = transpose ? 1 : n;   // rhs [k][n], or [n][k] when transposed
    ld.ld_n = transpose ? k : 1;
    return tsx::launch(g, ld, 1, tsx::as_stream(stream));
}

}  // extern "C"
