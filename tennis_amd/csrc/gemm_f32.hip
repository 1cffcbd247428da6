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

#include <algorithm>
#include <atomic>
#include <cstdlib>

namespace tsx {
namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int KC = 32;          // K per staged chunk
constexpr int THREADS = 256;

constexpr int MAX_SLOTS = 16;   // B elements a thread fetches per chunk (KC * BN / THREADS at BN = 64; 16 in the register-fed kernel)

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
    // The same in two steps, for loads that are issued unconditionally and resolved later: the address to read
    // (any valid one when the element is padding or beyond the matrix), whether the loaded value is the element,
    // and whether the element exists at all (else it is 0; an existing element outside the map is padding_value).
    __device__ __forceinline__ const float *slot_address(int i, int kdim, bool &inside, bool &valid) const {
        valid = col_ok && slot_k[i] < kdim;
        const int inv_kw = (65536 + kw - 1) / kw;
        const int r = (slot_tap[i] * inv_kw) >> 16, s = slot_tap[i] - r * kw;
        const int hh = h0 + r * dil_h, ww = w0 + s * dil_w;
        inside = valid && hh >= 0 && hh < h && ww >= 0 && ww < w;
        return inside ? img + (int64_t(slot_ci[i]) * h + hh) * w + ww : x;
    }
    __device__ __forceinline__ float fill_value() const { return padding_value; }
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
    __device__ __forceinline__ const float *slot_address(int i, int kdim, bool &inside, bool &valid) const {
        valid = inside = col_ok && slot_k[i] < kdim;
        return inside ? colp + int64_t(slot_k[i]) * ld_k : b;
    }
    __device__ __forceinline__ float fill_value() const { return 0.f; }
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

// A 32 x 32 accumulator tile's bias values and its stores.  Lane l holds rows row0 + 8 (r / 4) + 4 (l / 32) + r % 4
// (r = 0 .. 15) of column l % 32.  The sixteen bias values are requested in one go, well before they are added (a
// load inside the store loop would cost a memory round trip per row); rows beyond m read the last row's.
__device__ __forceinline__ void tile_bias_load(const GemmArgs &g, int row0, int lane, float (&bias)[16]) {
    if (g.bias) {
        static_for<0, 16>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            bias[r] = g.bias[min(row0 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4), g.m - 1)];
        });
    } else {
        static_for<0, 16>([&](auto rc) { bias[decltype(rc)::value] = 0.f; });
    }
}

__device__ __forceinline__ void tile_store(const GemmArgs &g, float *c, const v16f &acc, const float (&bias)[16], int row0,
                                           int lane, int64_t col_base, int64_t row_stride) {
    const bool with_bias = g.bias != nullptr;
    static_for<0, 16>([&](auto rc) {
        constexpr int r = decltype(rc)::value;
        const int row = row0 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
        if (row < g.m) {
            const int64_t idx = col_base + int64_t(row) * row_stride;
            float v = acc[r];
            if (with_bias) v = __fadd_rn(v, bias[r]);
            c[idx] = apply_act_basic(v, g.act, g.slope, idx < g.act_body);   // the entry points take none / relu / leaky_relu
        }
    });
}


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
    // bias values row by row: requesting the sixteen at once (as the small-problem kernels below do) costs this
    // kernel, whose register budget is the K loop's, a wavefront of occupancy, and its layers are large
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

// Small problems (a single 64-channel 56x56 layer: 196 tiles of 32 x 32): the staged kernel above walks K chunk by
// chunk with one global round trip per chunk and nothing else on the CU to hide it.  Here the operands go from
// global memory straight into the MFMA operand registers -- no LDS staging, no barrier in the loop -- and the eight
// wavefronts of a workgroup take the 32-deep K chunks of one 32 x 32 tile in turn (chunk c goes to wavefront c % 8),
// each with the next chunk's 20 loads in flight while it multiplies the current one; their partial tiles are summed
// through LDS in a fixed order (results do not depend on timing).  Which k an MFMA step carries is free as long as
// both operands agree: lane l (half hf = l / 32) takes k = hf * 16 + j of the chunk at step j, so its A operands are
// four 16-byte loads of its row and its B operands 16 gathers that are contiguous across the 32 lanes of a half.
// Needs 16-byte aligned rows of A (K a multiple of 4).
constexpr int KS_WAVES = 8;

template <class Loader>
__global__ __launch_bounds__(64 * KS_WAVES) void gemm_f32_regfed_kernel(GemmArgs g, Loader ld) {
    typedef float v4f_ __attribute__((ext_vector_type(4)));
    __shared__ float red[KS_WAVES - 1][16][64];
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int hf = lane / 32;
    const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const int batch = blockIdx.z;
    const float *a = g.a + batch * g.a_batch;
    if constexpr (std::is_same<Loader, MatLoader>::value) ld.b += batch * g.b_batch;
    ld.set_column(n0 + lane % 32, g.n);
    const int arow = min(m0 + lane % 32, g.m - 1);          // rows beyond m are loaded from the last row and never stored
    const float *arowp = a + int64_t(arow) * g.k + hf * 16;
    static_for<0, 16>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        ld.init_slot(i, wave * KC + hf * 16 + i);
    });
    const int chunks = (g.k + KC - 1) / KC;

    v16f acc;
    static_for<0, 16>([&](auto rc) { acc[decltype(rc)::value] = 0.f; });
    constexpr int NBUF = 2;      // chunks in flight per wavefront
    v4f_ a_reg[NBUF][4];
    float b_reg[NBUF][16];
    unsigned b_mask[NBUF];       // bit i: slot i's loaded value is the element; bit 16 + i: the element exists
    const float fill = ld.fill_value();
    auto load_chunk = [&](auto bufc, int c) __attribute__((always_inline)) {
        constexpr int buf = decltype(bufc)::value;
        const int k0 = c * KC + hf * 16;
        static_for<0, 4>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            // K is a multiple of 4: a group of four k is inside K or wholly beyond it (then the row's first group)
            a_reg[buf][i] = *reinterpret_cast<const v4f_ *>(k0 + 4 * i < g.k ? arowp + int64_t(c) * KC + 4 * i : arowp - hf * 16);
        });
        // every load issued without a branch around it; what a padding or out-of-range element reads is replaced
        // when the chunk is multiplied
        unsigned mask = 0;
        static_for<0, 16>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            bool inside, valid;
            const float *ptr = ld.slot_address(i, g.k, inside, valid);
            b_reg[buf][i] = *ptr;
            mask |= (inside ? 1u << i : 0u) | (valid ? 1u << (16 + i) : 0u);
            ld.advance_slot(i, KC * KS_WAVES);
        });
        b_mask[buf] = mask;
    };
    auto multiply = [&](auto bufc, int c) __attribute__((always_inline)) {
        constexpr int buf = decltype(bufc)::value;
        const int k0 = c * KC + hf * 16;
        const unsigned mask = b_mask[buf];
        static_for<0, 16>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const float bv = (mask >> j) & 1u ? b_reg[buf][j] : ((mask >> (16 + j)) & 1u ? fill : 0.f);
            const float av = k0 + j < g.k ? a_reg[buf][j / 4][j % 4] : 0.f;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
        });
    };
    // chunk c of this wavefront's sequence lives in buffer (its ordinal % NBUF); NBUF - 1 chunks ahead are in flight
    int c = wave;
    static_for<0, NBUF - 1>([&](auto bc) {
        if (c + decltype(bc)::value * KS_WAVES < chunks) load_chunk(bc, c + decltype(bc)::value * KS_WAVES);
    });
    while (c < chunks) {
        bool done = false;
        static_for<0, NBUF>([&](auto bc) {
            constexpr int b_ = decltype(bc)::value;
            if (!done) {
                if (c + (NBUF - 1) * KS_WAVES < chunks)
                    load_chunk(std::integral_constant<int, (b_ + NBUF - 1) % NBUF>{}, c + (NBUF - 1) * KS_WAVES);
                multiply(bc, c);
                c += KS_WAVES;
                done = c >= chunks;
            }
        });
    }

    float bias[16];
    if (wave > 0) {
        static_for<0, 16>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            red[wave - 1][r][lane] = acc[r];
        });
    } else {
        tile_bias_load(g, m0, lane, bias);
    }
    __syncthreads();
    if (wave > 0) return;
    static_for<0, KS_WAVES - 1>([&](auto wc) {
        constexpr int w = decltype(wc)::value;
        static_for<0, 16>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            acc[r] += red[w][r][lane];
        });
    });

    const int col = n0 + lane % 32;
    if (col >= g.n) return;
    int64_t col_base, row_stride;
    if (g.howo > 0) {
        const int n = col / g.howo;
        col_base = int64_t(n) * g.m * g.howo + (col - n * g.howo);
        row_stride = g.howo;
    } else {
        col_base = col;
        row_stride = g.n;
    }
    tile_store(g, g.c + batch * g.c_batch, acc, bias, m0, lane, col_base, row_stride);
}

// A single small 3x3 layer (BASELINE config 1: 1 x 64 x 56 x 56, 64 output channels: 196 tiles of 32 x 32, under one
// per CU) is bound by what the kernels above do per element of B: the im2col gather computes an address, two
// bounds and a padding select per element per K chunk, and walks K in dependent round trips.  This kernel orders K
// as the layer is laid out -- (input channel, tap) -- and gives every lane ONE input channel per MFMA step: lane l of
// a wavefront supplies output position l % 32 and, at step (t, tap), channel 2 (wave + 8 t) + l / 32.  A lane's nine
// taps of a channel are nine fixed byte offsets, and which of them fall into the padding depends on the lane's
// position only: both are computed once, and every load of B is "uniform channel base + the lane's tap offset".
// The eight wavefronts of a workgroup take the channel pairs of one 32 x 32 tile in turn and issue ALL their B loads
// (T pairs x 9 taps, one register each) and all their 16-byte pieces of the tile's 32 rows of A before waiting for
// any; A goes through LDS transposed ([k][row]: a lane reading its own row from global memory would touch 64 cache
// lines per instruction).  One round trip to memory in all, then T x 9 MFMAs per wavefront with A read from LDS, and
// the partial tiles summed through LDS in a fixed order.  T = channel pairs per wavefront: 4 (up to 64 input
// channels) or 2 (up to 32).  Tensors under 4 GiB (32-bit byte offsets), channels a multiple of 4 (rows of A are
// read in 16-byte pieces).
constexpr int SMALL_PITCH = 33;      // floats between consecutive k of the A tile in LDS (32 rows + 1)

template <int T>
__global__ __launch_bounds__(64 * KS_WAVES) void conv3x3_f32_small_kernel(GemmArgs g, ConvLoader ld) {
    typedef float v4f_ __attribute__((ext_vector_type(4)));
    constexpr int TAPS = 9;
    extern __shared__ __attribute__((aligned(16))) float lds_f[];   // A: K x SMALL_PITCH; then the partial tiles
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int hf = lane / 32;
    const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const int K = g.k;
    // the loader's fields as scalars of their own (the struct also carries the other kernels' per-thread state)
    const float *const x = ld.x;
    const int C = ld.c, H = ld.h, W = ld.w, dil_h = ld.dil_h, dil_w = ld.dil_w, howo = ld.howo, wo_ = ld.wo;
    const int stride_h = ld.stride_h, stride_w = ld.stride_w, pad_top = ld.pad_top, pad_left = ld.pad_left;
    const float padding_value = ld.padding_value;
    const float *const a_base = g.a;
    const int M = g.m, N = g.n;

    // ---- B: this lane's position, its base offset and which taps lie inside the map
    const int col = n0 + lane % 32;
    const bool col_ok = col < N;
    const int cc = col_ok ? col : 0;
    const int img_n = cc / howo, rpos = cc - img_n * howo;
    const int oh = rpos / wo_, ow = rpos - oh * wo_;
    const int h0 = oh * stride_h - pad_top, w0 = ow * stride_w - pad_left;
    // Byte offsets of the lane's nine taps from the first channel of its pair (32 bits: the launcher admits tensors
    // under 4 GiB only); a tap in the padding points at the channel's first pixel and its value is replaced below.
    // With them every load below is "uniform base + the lane's offset", no address arithmetic per load.
    const unsigned plane4 = unsigned(H * W) * 4u;
    const unsigned lane_base = (unsigned(img_n) * unsigned(C) + unsigned(hf)) * plane4;
    const int pos_off = h0 * W + w0;          // may be negative: only used where the tap is inside
    unsigned inside = 0;                      // bit tap: the tap's pixel exists
    unsigned b_off[TAPS];
    static_for<0, TAPS>([&](auto jc) {
        constexpr int j = decltype(jc)::value, r = j / 3, q = j % 3;
        const int hh = h0 + r * dil_h, ww = w0 + q * dil_w;
        const bool in = col_ok & (unsigned(hh) < unsigned(H)) & (unsigned(ww) < unsigned(W));
        inside |= unsigned(in) << j;
        b_off[j] = lane_base + (in ? unsigned(pos_off + r * dil_h * W + q * dil_w) * 4u : 0u);
    });
    float b_reg[T][TAPS];
    static_for<0, T>([&](auto tc) {
        constexpr int t = decltype(tc)::value;
        const int pair = wave + KS_WAVES * t;                 // channels 2 pair, 2 pair + 1 (c is even)
        const char *chan = reinterpret_cast<const char *>(x) + (2 * pair < C ? size_t(2 * pair) * plane4 : size_t(0));
        static_for<0, TAPS>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            b_reg[t][j] = *reinterpret_cast<const float *>(chan + b_off[j]);     // resolved below
        });
    });

    // ---- A: rows m0 .. m0 + 31, all of K, into LDS as [k][SMALL_PITCH] (rows beyond m: the last row, never stored).
    // A wavefront's load covers 8 rows x 128 bytes (8 whole cache lines); its four stores then go to banks
    // 4 (lane % 8) + lane / 8 (+ j): no two lanes of a half wavefront share one, and the MFMA loop's reads (32
    // consecutive rows of one k) share none either.
    // All of a wavefront's pieces are requested before the first is stored: one round trip, not one per piece.
    {
        constexpr int PIECES = (4 * ((T * 36 + 7) / 8) + KS_WAVES - 1) / KS_WAVES;   // per wavefront, at most (K <= 144 T)
        const int k4s = K / 4, groups = (k4s + 7) / 8;  // 16-byte pieces per row; groups of 8 pieces
        const int kk = lane % 8, rr = lane / 8;
        v4f_ piece[PIECES];
        static_for<0, PIECES>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int item = wave + KS_WAVES * i;
            const int row = 8 * (item % 4) + rr, k4 = min(8 * (item / 4) + kk, k4s - 1);
            const unsigned a_off = (unsigned(min(m0 + row, M - 1)) * unsigned(K) + 4u * unsigned(k4)) * 4u;
            piece[i] = *reinterpret_cast<const v4f_ *>(reinterpret_cast<const char *>(a_base) + a_off);
        });
        static_for<0, PIECES>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int item = wave + KS_WAVES * i;
            const int row = 8 * (item % 4) + rr, k4 = 8 * (item / 4) + kk;
            if (item < 4 * groups && k4 < k4s) {
                float *dst = lds_f + 4 * k4 * SMALL_PITCH + row;
                dst[0] = piece[i][0];
                dst[SMALL_PITCH] = piece[i][1];
                dst[2 * SMALL_PITCH] = piece[i][2];
                dst[3 * SMALL_PITCH] = piece[i][3];
            }
        });
    }
    __syncthreads();

    v16f acc;
    static_for<0, 16>([&](auto rc) { acc[decltype(rc)::value] = 0.f; });
    const float *arow = lds_f + lane % 32;
    static_for<0, T>([&](auto tc) {
        constexpr int t = decltype(tc)::value;
        const int ci = 2 * (wave + KS_WAVES * t) + hf;
        const bool c_ok = 2 * (wave + KS_WAVES * t) < C;
        const float *ak = arow + (c_ok ? ci : 0) * (TAPS * SMALL_PITCH);
        static_for<0, TAPS>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const float av = c_ok ? ak[j * SMALL_PITCH] : 0.f;
            // a tap in the padding reads padding_value; a column beyond n or a channel beyond c contributes nothing
            const float bv = !(c_ok && col_ok) ? 0.f : ((inside >> j) & 1u) ? b_reg[t][j] : padding_value;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
        });
    });

    float bias[16];
    if (wave == 0) tile_bias_load(g, m0, lane, bias);
    __syncthreads();                                    // every wavefront is done with A: its space takes the partial tiles
    float (*red)[16][64] = reinterpret_cast<float (*)[16][64]>(lds_f);
    if (wave > 0) {
        static_for<0, 16>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            red[wave - 1][r][lane] = acc[r];
        });
    }
    __syncthreads();
    if (wave > 0) return;
    static_for<0, KS_WAVES - 1>([&](auto wc) {
        constexpr int w = decltype(wc)::value;
        static_for<0, 16>([&](auto rc) {
            constexpr int r = decltype(rc)::value;
            acc[r] += red[w][r][lane];
        });
    });
    if (!col_ok) return;
    tile_store(g, g.c, acc, bias, m0, lane, int64_t(img_n) * M * howo + rpos, howo);
}

// Whether the small-layer kernel takes a convolution, and its launch.  Dynamic LDS beyond 64 KiB has to be granted per
// kernel and device.
template <int T>
int launch_conv3x3_small(const GemmArgs &g, const ConvLoader &ld, hipStream_t stream) {
    const size_t lds_bytes = std::max(size_t(g.k) * SMALL_PITCH * 4, size_t(KS_WAVES - 1) * 16 * 64 * 4);
    static std::atomic<bool> granted[64];
    int dev = 0;
    TSX_HIP(hipGetDevice(&dev));
    auto kernel = conv3x3_f32_small_kernel<T>;
    if (lds_bytes > 65536 && dev < 64 && !granted[dev].load()) {
        TSX_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        granted[dev].store(true);
    }
    const dim3 grid(unsigned(ceil_div(g.n, 32)), unsigned(ceil_div(g.m, 32)));
    hipLaunchKernelGGL(kernel, grid, dim3(64 * KS_WAVES), lds_bytes, stream, g, ld);
    TSX_LAUNCH_CHECK("conv3x3_f32_small_kernel");
    return 0;
}

inline bool conv3x3_small_takes(const GemmArgs &g, const ConvLoader &ld) {
    const char *e = std::getenv("TSX_CONV_F32_SMALL");      // "0": never; "force": wherever the layer allows (tests)
    if (e && e[0] == '0') return false;
    if (ld.kh != 3 || ld.kw != 3 || ld.c > 64 || ld.c % 2 != 0 || g.k % 4 != 0 || reinterpret_cast<uintptr_t>(g.a) % 16 != 0)
        return false;
    // 32-bit byte offsets into the input and the weights
    const int64_t images = ceil_div(int64_t(g.n), int64_t(ld.howo));
    if (images * ld.c * ld.h * ld.w * 4 >= (int64_t(1) << 32) || int64_t(g.m) * g.k * 4 >= (int64_t(1) << 32)) return false;
    const int64_t tiles32 = ceil_div(g.m, 32) * ceil_div(g.n, 32);
    return (e && e[0] == 'f') || tiles32 <= 512;
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

enum GemmKernel { GEMM_REGISTER_FED, GEMM_STAGED_64, GEMM_STAGED_32_KSPLIT };

inline GemmKernel choose_gemm(const GemmArgs &g, int batches) {
    // Big problems: 64x64 tiles, no K split.  Small ones (fewer tiles than SIMDs): 32x32 tiles
    // with the four wavefronts splitting K, so a single small layer still spreads over the chip.
    const int64_t tiles64 = ceil_div(g.m, 64) * ceil_div(g.n, 64) * batches;
    // TSX_GEMM_F32_REGFED: "0" never, "force" wherever the operands allow (tests); otherwise small problems
    const char *e = std::getenv("TSX_GEMM_F32_REGFED");
    const bool regfed_ok = g.k % 4 == 0 && g.k >= KC && reinterpret_cast<uintptr_t>(g.a) % 16 == 0 && g.a_batch % 4 == 0;
    const int64_t tiles32 = ceil_div(g.m, 32) * ceil_div(g.n, 32) * batches;
    if (regfed_ok && !(e && e[0] == '0') && ((e && e[0] == 'f') || tiles32 <= 512)) return GEMM_REGISTER_FED;
    return tiles64 >= 512 || g.k < 4 * KC ? GEMM_STAGED_64 : GEMM_STAGED_32_KSPLIT;
}

template <class Loader>
int launch(const GemmArgs &g, const Loader &ld, int batches, hipStream_t stream) {
    const GemmKernel kernel = choose_gemm(g, batches);
    if (kernel == GEMM_REGISTER_FED) {
        dim3 grid(unsigned(ceil_div(g.n, 32)), unsigned(ceil_div(g.m, 32)), unsigned(batches));
        hipLaunchKernelGGL((gemm_f32_regfed_kernel<Loader>), grid, dim3(64 * KS_WAVES), 0, stream, g, ld);
        TSX_LAUNCH_CHECK("gemm_f32_regfed_kernel");
        return 0;
    }
    if (kernel == GEMM_STAGED_64) {
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

// The GEMM view of a convolution: weights [cout][c kh kw] x implicit im2col [c kh kw][n ho wo].
static int conv_f32_problem(const tsx_conv2d_geom *geo, const float *x_dev, const float *w_oihw_dev, float padding_value,
                            const float *bias_dev, int32_t act, float slope, float *out_dev, tsx::GemmArgs &g,
                            tsx::ConvLoader &ld) {
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
    g = tsx::GemmArgs{};
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
    ld = tsx::ConvLoader{};
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
    return 0;
}

int tsx_conv2d_f32_nchw(const tsx_conv2d_geom *geo, const float *x_dev, const float *w_oihw_dev, float padding_value,
                        const float *bias_dev, int32_t act, float slope, float *out_dev, void *stream) {
    TSX_REQUIRE(geo && x_dev && w_oihw_dev && out_dev, "conv2d_f32: null argument");
    tsx::GemmArgs g;
    tsx::ConvLoader ld;
    const int rc = conv_f32_problem(geo, x_dev, w_oihw_dev, padding_value, bias_dev, act, slope, out_dev, g, ld);
    if (rc) return rc;
    if (tsx::conv3x3_small_takes(g, ld))
        return geo->c <= 32 ? tsx::launch_conv3x3_small<2>(g, ld, tsx::as_stream(stream))
                            : tsx::launch_conv3x3_small<4>(g, ld, tsx::as_stream(stream));
    return tsx::launch(g, ld, 1, tsx::as_stream(stream));
}

int tsx_conv2d_f32_plan_info(const tsx_conv2d_geom *geo, const float *w_oihw_dev, char *text, size_t text_bytes) {
    TSX_REQUIRE(geo && w_oihw_dev && text && text_bytes > 0, "conv2d_f32_plan_info: null argument");
    tsx::GemmArgs g;
    tsx::ConvLoader ld;
    const int rc = conv_f32_problem(geo, nullptr, w_oihw_dev, 0.f, nullptr, TSX_ACT_NONE, 0.f, nullptr, g, ld);
    if (rc) return rc;
    const char *name = "small_3x3";
    int tile = 32;
    if (!tsx::conv3x3_small_takes(g, ld)) {
        const tsx::GemmKernel k = tsx::choose_gemm(g, 1);
        name = k == tsx::GEMM_REGISTER_FED ? "register_fed" : k == tsx::GEMM_STAGED_64 ? "staged_64x64" : "staged_32x32_ksplit";
        if (k == tsx::GEMM_STAGED_64) tile = 64;
    }
    std::snprintf(text, text_bytes, "kernel=%s tiles=%lld", name,
                  (long long)(tsx::ceil_div(g.m, tile) * tsx::ceil_div(g.n, tile)));
    return 0;
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
