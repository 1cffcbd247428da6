// int8 conv2d / GEMM on the gfx950 i8 MFMA units: implicit-im2col GEMM with int32
// accumulation and a fused dequant + bias + activation (+ requantize) epilogue.
//
// Stands in for cpu::Conv2DQuantizedCore::conv2d
// (src/kernels/cpu/quantized/conv2d_quantized_core.cpp:18-147): per-image im2col<int8>
// (src/kernels/cpu/im2col.cpp:37-111) + math<int8,int32>::gemm (math_cpu.cpp:143-244) +
// float(acc)*dq[c].  Integer accumulation is exact, so the contraction order is free:
//
//   * activations are first *staged* into a channel-blocked, spatially padded copy
//     xs[n][hs][ws][cp] (cp = channels rounded up to 64, halo = int8(padding_value)); a
//     (tap, 64-channel block) K-step of any output position is then 64 contiguous bytes;
//   * weights are packed once into MFMA operand order, K ordered (kh, kw, c-block) to match;
//   * one workgroup computes a BM(cout) x BN(positions) tile, positions flattened over
//     (n, ho, wo); operands go HBM/L2 -> registers -> LDS (double buffered) -> MFMA
//     v_mfma_i32_32x32x32_i8.  Which operand is "rows" is a template switch so the
//     accumulator lanes run along the contiguous output dimension (positions for NCHW
//     conv output, features for row-major GEMM output).
//
// MFMA operand layout used (v_mfma_i32_32x32x32_i8, 64 lanes): lane l supplies row/column
// (l % 32) and 16 consecutive K bytes of K-group (l / 32); A and B use the same K mapping,
// so any consistent K permutation gives the same exact integer result.  Accumulator register
// r of lane l holds row 8*(r/4) + 4*(l/32) + (r%4), column l % 32.
#include "igemm_i8.hpp"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdlib>
#include <mutex>

namespace {

using tsx::v4i;
using tsx::v16i;

constexpr int KSTEP = 64;  // bytes of K per pipeline step (two MFMAs of K=32)

// ------------------------------------------------------------------ staging kernels

struct StageGeom {
    int n, c, h, w;        // source NCHW
    int hs, ws, cp;        // staged extent
    int pad_top, pad_left;
    int pad_value;         // int8 halo value
};

// One lane produces one 16-byte channel chunk of one staged pixel.  Adjacent lanes take
// adjacent ws, so each of the 16 byte loads is coalesced along W of the NCHW source.
// QUANT: the source is fp32 and is quantized on the fly with the semantics of
// cpu::Quantize (quantize.cpp:70-125) evaluated at the element's NCHW linear index.
template <bool QUANT>
__global__ __launch_bounds__(256) void stage_nchw_kernel(const void *__restrict__ src, StageGeom g,
                                                        const float *__restrict__ scales, int n_scales,
                                                        int64_t group_len, int64_t bulk8,
                                                        int8_t *__restrict__ xs) {
    const int chunks = g.cp / 16;
    const int64_t total = int64_t(g.n) * g.hs * chunks * g.ws;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    int wsi, chunk, hsi, ni;
    if (total <= 0xffffffffll) {   // the usual case: three 32-bit divisions instead of three 64-bit ones per lane
        const uint32_t id32 = uint32_t(id);
        uint32_t rest = id32 / uint32_t(g.ws);
        wsi = int(id32 - rest * uint32_t(g.ws));
        const uint32_t r2 = rest / uint32_t(chunks);
        chunk = int(rest - r2 * uint32_t(chunks));
        ni = int(r2 / uint32_t(g.hs));
        hsi = int(r2 - uint32_t(ni) * uint32_t(g.hs));
    } else {
        wsi = int(id % g.ws);
        int64_t rest = id / g.ws;
        chunk = int(rest % chunks);
        rest /= chunks;
        hsi = int(rest % g.hs);
        ni = int(rest / g.hs);
    }
    const int hi = hsi - g.pad_top, wi = wsi - g.pad_left;
    const bool inside = hi >= 0 && hi < g.h && wi >= 0 && wi < g.w;
    // one scale group per image (the usual case when there are several): no division per element
    const bool per_image = group_len == int64_t(g.c) * g.h * g.w;
    uint32_t words[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int ci = chunk * 16 + v * 4 + j;
            int q = 0;  // channel padding: weights there are zero as well
            if (ci < g.c) {
                q = g.pad_value;
                if (inside) {
                    const int64_t idx = ((int64_t(ni) * g.c + ci) * g.h + hi) * g.w + wi;
                    if (QUANT) {
                        const float s = n_scales == 1 ? scales[0] : per_image ? scales[ni] : scales[idx / group_len];
                        q = tsx::quantize_value(__fmul_rn(static_cast<const float *>(src)[idx], s),
                                                n_scales == 1 && idx < bulk8);
                    } else {
                        q = static_cast<const int8_t *>(src)[idx];
                    }
                }
            }
            word |= uint32_t(q & 0xff) << (8 * j);
        }
        words[v] = word;
    }
    const int64_t o = ((int64_t(ni) * g.hs + hsi) * g.ws + wsi) * g.cp + chunk * 16;
    *reinterpret_cast<uint4 *>(xs + o) = make_uint4(words[0], words[1], words[2], words[3]);
}

// Row-at-a-time staging through LDS: one workgroup builds one staged row xs[n][hs][0..ws)[c0..c0+CG)
// for a group of CG <= 256 channels.  Phase 1 reads the NCHW source coalesced along W (runs of
// W elements per channel), quantizes (QUANT) and scatters bytes into an LDS tile [ws][CG+16]
// pre-filled with the halo value; phase 2 writes the tile out as whole 16-byte chunks, a pixel's
// channel group contiguous.  HBM traffic is exactly the algorithmic 4 B (or 1 B) read + 1 B
// written per element; the older one-lane-per-chunk kernel remains for very wide rows.
constexpr int STAGE_CG = 256;                 // channels per pass
constexpr int STAGE_LROW = STAGE_CG + 16;     // LDS bytes per pixel: 16-byte aligned, bank-shifted
constexpr int STAGE_MAX_WS = 232;             // ws * LROW <= 63 KiB

struct StageRow {
    const void *src;
    const float *scales;
    int n_scales;
    int64_t group_len, bulk8;
    bool uniform_scale;
    float row_scale;
    int ni, hi, c0, creal;
};

// Phase 1 of stage_rows_kernel for one source row and one channel group.  Lane = (run of VW pixels
// along W, channel quad): a lane loads the same VW pixels of 4 consecutive channels (one VW-wide load
// per channel, coalesced along W across lanes), packs the 4 quantized bytes of each pixel into one
// dword and writes VW dwords to the tile -- no byte-granular LDS traffic.  WL = power of two >= W/VW
// keeps the mapping division-free; loads are issued in batches of NB quads before any is consumed.
// RMODE says how the row's elements round: 0 = all half away from zero (the reference's scalar loop),
// 1 = all half to even (its AVX body), 2 = per element (the one row that holds the body/tail border).
template <bool QUANT, int VW, int RMODE, bool UNIFORM = false>
__device__ __forceinline__ void stage_quads(const StageGeom &g, const StageRow &r, int8_t *tile, int tid) {
    typedef float vf __attribute__((ext_vector_type(VW == 1 ? 2 : VW)));   // VW == 1 uses scalars
    constexpr int NB = VW == 4 ? 2 : 4;
    const int pw = g.w / VW;
    int wl = 1, wl_shift = 0;
    while (wl < pw) {
        wl <<= 1;
        ++wl_shift;
    }
    const int lane = tid & 63, wave = tid >> 6;
    const int qpw = 64 >> wl_shift;                 // channel quads per wavefront per step
    const int pi = lane & (wl - 1);
    const int wi = pi * VW;
    const int q_lane = wave * qpw + (lane >> wl_shift);
    const int qstep = 4 * qpw;                      // quads per workgroup step
    const bool lane_ok = pi < pw;
    const int64_t plane = int64_t(g.h) * g.w;
    const int64_t row_base = (int64_t(r.ni) * g.c + r.c0) * plane + int64_t(r.hi) * g.w + wi;
    const int quads = (r.creal + 3) / 4;
    for (int qb = 0; qb < quads; qb += NB * qstep) {
        float fv[NB][4][VW];
        int bv[NB][4][VW];
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int c = (qb + u * qstep + q_lane) * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool ok = lane_ok && c + j < r.creal;
                const int64_t e = row_base + int64_t(c + j) * plane;
                if (QUANT) {
                    const float *p = static_cast<const float *>(r.src) + e;
                    if (VW == 1) {
                        fv[u][j][0] = ok ? *p : 0.f;
                    } else {
                        vf t;
#pragma unroll
                        for (int v = 0; v < VW; ++v) t[v] = 0.f;
                        if (ok) t = *reinterpret_cast<const vf *>(p);
#pragma unroll
                        for (int v = 0; v < VW; ++v) fv[u][j][v] = t[v];
                    }
                } else {
                    const int8_t *p = static_cast<const int8_t *>(r.src) + e;
                    uint32_t t = 0;
                    if (ok) {
                        if (VW == 4) t = *reinterpret_cast<const uint32_t *>(p);
                        else if (VW == 2) t = *reinterpret_cast<const uint16_t *>(p);
                        else t = uint8_t(*p);
                    }
#pragma unroll
                    for (int v = 0; v < VW; ++v) bv[u][j][v] = int8_t(t >> (8 * v));
                }
            }
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int c = (qb + u * qstep + q_lane) * 4;
            if (!(lane_ok && c < r.creal)) continue;
            // bytes of the quad that are real channels (the last quad of a ragged channel count keeps zeros above)
            const uint32_t keep = c + 3 < r.creal ? 0xffffffffu : 0xffffffffu >> (8 * (c + 4 - r.creal));
#pragma unroll
            for (int v = 0; v < VW; ++v) {
                int q[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (QUANT) {
                        float sc = r.row_scale;
                        bool half_even = RMODE == 1;
                        if (RMODE == 2 || (!UNIFORM && !r.uniform_scale)) {   // the element's linear index is only needed here
                            const int64_t e = row_base + int64_t(c + j) * plane + v;
                            if (!UNIFORM && !r.uniform_scale) sc = c + j < r.creal ? r.scales[e / r.group_len] : 0.f;
                            if (RMODE == 2) half_even = e < r.bulk8;
                        }
                        q[j] = tsx::quantize_value(__fmul_rn(fv[u][j][v], sc), half_even);
                    } else {
                        q[j] = bv[u][j][v];
                    }
                }
                // low bytes of q[0..3] into one dword: three byte permutes (selector 0-3 = bytes of the second
                // operand, 4-7 = bytes of the first, 0x0c = zero)
                const uint32_t lo = __builtin_amdgcn_perm(uint32_t(q[1]), uint32_t(q[0]), 0x0c0c0400u);
                const uint32_t hi = __builtin_amdgcn_perm(uint32_t(q[3]), uint32_t(q[2]), 0x0c0c0400u);
                const uint32_t word = __builtin_amdgcn_perm(hi, lo, 0x05040100u) & keep;
                *reinterpret_cast<uint32_t *>(&tile[(wi + v + g.pad_left) * STAGE_LROW + c]) = word;
            }
        }
    }
}

// FAST: what the launcher has checked for the whole launch -- rows of a multiple of 4 elements from a 16-byte
// aligned tensor (4-byte aligned for int8), at most 256 of them, one scale per image and more than one image (so
// every element rounds half away from zero, base_quantize / quantize.cpp's scalar path).  The general kernel
// carries the per-element 64-bit divisions and the three rounding variants of every load width inline, ~47 000
// instructions of which a row executes a few hundred scattered over 40 KiB of code; this one is the row's own code.
template <bool QUANT, bool FAST = false>
__global__ __launch_bounds__(256) void stage_rows_kernel(const void *__restrict__ src, StageGeom g,
                                                        const float *__restrict__ scales, int n_scales,
                                                        int64_t group_len, int64_t bulk8,
                                                        int8_t *__restrict__ xs) {
    extern __shared__ __attribute__((aligned(16))) int8_t tile[];   // [ws][STAGE_LROW]
    const int tid = threadIdx.x;
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Neighbouring rows of a
    // channel plane share cache lines (a W-float run is rarely line-aligned), so give each XCD a
    // contiguous run of rows: the shared lines are then fetched from HBM once, not once per XCD.
    const unsigned total_rows = unsigned(g.n) * g.hs, per_xcd = (total_rows + 7) / 8;
    const unsigned row_id = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (row_id >= total_rows) return;
    const int hsi = row_id % g.hs, ni = row_id / g.hs;
    const int hi = hsi - g.pad_top;
    const bool row_inside = hi >= 0 && hi < g.h;
    const uint32_t pad4 = uint32_t(g.pad_value & 0xff) * 0x01010101u;
    // The scale group of element e is e / group_len (a 64-bit division).  With one scale, or one
    // group per image (the usual case: the count divides evenly), it is uniform for this row.
    const bool uniform_scale = QUANT && (n_scales == 1 || group_len == int64_t(g.c) * g.h * g.w);
    const float row_scale = uniform_scale ? scales[n_scales == 1 ? 0 : ni] : 0.f;
    for (int c0 = 0; c0 < g.cp; c0 += STAGE_CG) {
        const int cg = min(STAGE_CG, g.cp - c0);        // multiple of 64
        const int creal = max(0, min(cg, g.c - c0));    // channels that exist in the source
        // Lane = (run of VW pixels along W, channel quad): see stage_quads.  The widest run the row
        // length and the source alignment allow keeps the number of load instructions down.
        const uintptr_t addr = reinterpret_cast<uintptr_t>(src);
        const int esz = QUANT ? 4 : 1;
        int vw = 1;
        if (FAST || (g.w % 4 == 0 && addr % (4 * esz) == 0)) vw = 4;
        else if (g.w % 2 == 0 && addr % (2 * esz) == 0) vw = 2;
        int wl = 1;
        while (wl * vw < g.w) wl <<= 1;
        // stage_quads writes every dword of the interior pixels up to the last real channel quad, so
        // on that path the pre-fill only has to cover the halo pixels and the channel padding: the
        // two write disjoint dwords and need no barrier between them.
        const bool quad_path = row_inside && (FAST || wl <= 64);
        const int real_words = (creal + 3) / 4;
        // pre-fill: halo value for real channels, zero for channel padding
        const int wpr = cg / 4;   // dwords per pixel
        auto fill_word = [&](int pix, int cw) {
            uint32_t v = pad4;
            if (cw * 4 + 4 > creal) {
                v = 0;
                for (int j = 0; j < 4; ++j)
                    if (cw * 4 + j < creal) v |= uint32_t(g.pad_value & 0xff) << (8 * j);
            }
            *reinterpret_cast<uint32_t *>(&tile[pix * STAGE_LROW + cw * 4]) = v;
        };
        if (quad_path) {
            // only the halo pixels (left and right of the row) and the channel padding of the interior pixels:
            // a loop over the whole tile costs a division per dword, as much arithmetic as the row itself
            const int halo_px = g.ws - g.w;
            for (int idx = tid; idx < halo_px * wpr; idx += 256) {
                const int hp = idx / wpr, cw = idx - hp * wpr;
                fill_word(hp < g.pad_left ? hp : hp + g.w, cw);
            }
            const int pad_words = wpr - real_words;
            if (pad_words > 0)
                for (int idx = tid; idx < g.w * pad_words; idx += 256) {
                    const int ip = idx / pad_words;
                    fill_word(g.pad_left + ip, real_words + idx - ip * pad_words);
                }
        } else {
            for (int idx = tid; idx < g.ws * wpr; idx += 256) {
                const int pix = idx / wpr;
                fill_word(pix, idx - pix * wpr);
            }
            __syncthreads();
        }
        if (row_inside) {
            if constexpr (FAST) {
                const StageRow r{src, scales, n_scales, group_len, bulk8, true, row_scale, ni, hi, c0, creal};
                stage_quads<QUANT, 4, 0, true>(g, r, tile, tid);
            } else if (quad_path) {
                const StageRow r{src, scales, n_scales, group_len, bulk8, uniform_scale, row_scale, ni, hi, c0, creal};
                // how this row's elements round: linear indices run from lo to hi_e, the AVX body ends at bulk8
                int rmode = 0;
                if (QUANT && n_scales == 1) {
                    const int64_t lo = ((int64_t(ni) * g.c + c0) * g.h + hi) * g.w;
                    const int64_t hi_e = lo + int64_t(creal - 1) * g.h * g.w + g.w - 1;
                    rmode = hi_e < bulk8 ? 1 : lo >= bulk8 ? 0 : 2;
                }
                if (vw == 4) {
                    if (rmode == 0) stage_quads<QUANT, 4, 0>(g, r, tile, tid);
                    else if (rmode == 1) stage_quads<QUANT, 4, 1>(g, r, tile, tid);
                    else stage_quads<QUANT, 4, 2>(g, r, tile, tid);
                } else if (vw == 2) {
                    if (rmode == 0) stage_quads<QUANT, 2, 0>(g, r, tile, tid);
                    else if (rmode == 1) stage_quads<QUANT, 2, 1>(g, r, tile, tid);
                    else stage_quads<QUANT, 2, 2>(g, r, tile, tid);
                } else {
                    if (rmode == 0) stage_quads<QUANT, 1, 0>(g, r, tile, tid);
                    else if (rmode == 1) stage_quads<QUANT, 1, 1>(g, r, tile, tid);
                    else stage_quads<QUANT, 1, 2>(g, r, tile, tid);
                }
            } else {
                for (int idx = tid; idx < creal * g.w; idx += 256) {
                    const int c = idx / g.w, wi = idx - c * g.w;
                    const int64_t e = ((int64_t(ni) * g.c + c0 + c) * g.h + hi) * g.w + wi;
                    int q;
                    if (QUANT) {
                        const float sc = uniform_scale ? row_scale : scales[e / group_len];
                        q = tsx::quantize_value(__fmul_rn(static_cast<const float *>(src)[e], sc), n_scales == 1 && e < bulk8);
                    } else {
                        q = static_cast<const int8_t *>(src)[e];
                    }
                    tile[(wi + g.pad_left) * STAGE_LROW + c] = int8_t(q);
                }
            }
        }
        __syncthreads();
        const int chunks = cg / 16;
        int8_t *dst = xs + ((int64_t(ni) * g.hs + hsi) * g.ws) * g.cp + c0;
        for (int idx = tid; idx < g.ws * chunks; idx += 256) {
            const int pix = idx / chunks, ch = idx - pix * chunks;
            *reinterpret_cast<v4i *>(dst + int64_t(pix) * g.cp + ch * 16) =
                *reinterpret_cast<const v4i *>(&tile[pix * STAGE_LROW + ch * 16]);
        }
        if (c0 + STAGE_CG < g.cp) __syncthreads();     // the next pass refills the tile
    }
}

// Explicit im2col staging for layers with very few input channels and a large kernel (a 7x7 stem on
// 3 channels): padding 3 channels to a 64-byte K block per tap would make 95 % of the MFMA work
// zeros, so the K axis is packed as the reference's im2col does (k = (c*KH + kh)*KW + kw,
// src/kernels/cpu/im2col.cpp:37-111) and the layer runs as a 1x1 convolution over
// [n][ho][wo][round_up(C*KH*KW, 64)].  One lane = one 16-byte K chunk of one output pixel; lanes of a
// pixel are adjacent, so stores are contiguous and the gathered loads stay inside one small patch.
struct Im2colGeom {
    int n, c, h, w, ho, wo, kh, kw, sh, sw, dh, dw, pad_top, pad_left, kk, cp, pad_value;
};

template <bool QUANT>
__global__ __launch_bounds__(256) void stage_im2col_kernel(const void *__restrict__ src, Im2colGeom g,
                                                          const float *__restrict__ scales, int n_scales,
                                                          int64_t group_len, int64_t bulk8, int8_t *__restrict__ xs) {
    const int chunks = g.cp / 16;
    const int64_t total = int64_t(g.n) * g.ho * g.wo * chunks;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int chunk = int(id % chunks);
    int64_t rest = id / chunks;
    const int ow = int(rest % g.wo);
    rest /= g.wo;
    const int oh = int(rest % g.ho);
    const int ni = int(rest / g.ho);
    const int taps = g.kh * g.kw;
    // one quantize group per image (the usual case) or a single scale: no per-element 64-bit division
    const bool uniform_scale = QUANT && (n_scales == 1 || group_len == int64_t(g.c) * g.h * g.w);
    const float img_scale = uniform_scale ? scales[n_scales == 1 ? 0 : ni] : 0.f;
    // (ci, kh, kw) of the chunk's first K index, then stepped without divisions
    int k = chunk * 16;
    int ci = k / taps;
    int kh = (k - ci * taps) / g.kw;
    int kw = k - ci * taps - kh * g.kw;
    const int h0 = oh * g.sh - g.pad_top, w0 = ow * g.sw - g.pad_left;
    uint32_t words[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int q = 0;   // K padding: the packed weights are zero there as well
            if (k < g.kk) {
                const int hi = h0 + kh * g.dh, wi = w0 + kw * g.dw;
                q = g.pad_value;
                if (hi >= 0 && hi < g.h && wi >= 0 && wi < g.w) {
                    const int64_t e = ((int64_t(ni) * g.c + ci) * g.h + hi) * g.w + wi;
                    if (QUANT) {
                        const float sc = uniform_scale ? img_scale : scales[e / group_len];
                        q = tsx::quantize_value(__fmul_rn(static_cast<const float *>(src)[e], sc), n_scales == 1 && e < bulk8);
                    } else {
                        q = static_cast<const int8_t *>(src)[e];
                    }
                }
            }
            word |= uint32_t(q & 0xff) << (8 * j);
            ++k;
            if (++kw == g.kw) {
                kw = 0;
                if (++kh == g.kh) {
                    kh = 0;
                    ++ci;
                }
            }
        }
        words[v] = word;
    }
    *reinterpret_cast<uint4 *>(xs + id * 16) = make_uint4(words[0], words[1], words[2], words[3]);
}

// The same staging with one workgroup per (image, output row).  Phase 1 quantizes the C x KH input rows
// the output row reads once each into an LDS patch [c][kh][patch columns] (coalesced loads along W; the
// lane-per-chunk kernel above quantizes every input element KH*KW/(SH*SW) times and gathers from global
// memory); phase 2 assembles the 16-byte K chunks from patch bytes and stores them contiguously.
template <bool QUANT>
__global__ __launch_bounds__(256) void stage_im2col_rows_kernel(const void *__restrict__ src, Im2colGeom g, int wpatch,
                                                               const float *__restrict__ scales, int n_scales,
                                                               int64_t group_len, int64_t bulk8, int8_t *__restrict__ xs) {
    extern __shared__ __attribute__((aligned(16))) int8_t patch[];   // [c * kh][wpatch]
    const int tid = threadIdx.x;
    const int oh = blockIdx.x % g.ho, ni = blockIdx.x / g.ho;
    const bool uniform_scale = QUANT && (n_scales == 1 || group_len == int64_t(g.c) * g.h * g.w);
    const float img_scale = uniform_scale ? scales[n_scales == 1 ? 0 : ni] : 0.f;
    const int h0 = oh * g.sh - g.pad_top;
    const int rows = g.c * g.kh;
    // phase 1: wavefront per patch row, lanes along W (no per-element index arithmetic)
    for (int row = tid >> 6; row < rows; row += 4) {
        const int ci = row / g.kh, r = row - ci * g.kh;
        const int hi = h0 + r * g.dh;
        const bool row_in = hi >= 0 && hi < g.h;
        const int64_t e0 = ((int64_t(ni) * g.c + ci) * g.h + hi) * g.w;
        // four column steps at a time with their loads issued together: a loop that loads, converts and stores
        // one step at a time pays one memory round trip per step, and this phase was most of the kernel's time
        for (int cb = 0; cb < wpatch; cb += 256) {
            float fv[4];
            int bv[4];
            bool in[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int wi = cb + u * 64 + (tid & 63) - g.pad_left;
                in[u] = row_in && wi >= 0 && wi < g.w && cb + u * 64 + (tid & 63) < wpatch;
                // unconditional loads (element 0 where the patch cell is halo): a load behind a branch is waited
                // for before the next one is issued
                const int64_t a = in[u] ? e0 + wi : 0;
                fv[u] = 0.f;
                bv[u] = 0;
                if (QUANT) fv[u] = static_cast<const float *>(src)[a];
                else bv[u] = static_cast<const int8_t *>(src)[a];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int col = cb + u * 64 + (tid & 63);
                if (col >= wpatch) continue;
                int q = g.pad_value;
                if (in[u]) {
                    if (QUANT) {
                        const int64_t e = e0 + (col - g.pad_left);
                        const float sc = uniform_scale ? img_scale : scales[e / group_len];
                        q = tsx::quantize_value(__fmul_rn(fv[u], sc), n_scales == 1 && e < bulk8);
                    } else {
                        q = bv[u];
                    }
                }
                patch[row * wpatch + col] = int8_t(q);
            }
        }
    }
    __syncthreads();
    // phase 2: a lane keeps one K chunk for the whole row, so the patch offsets of its 16 bytes are
    // computed once; per output pixel it reads 16 bytes at (pixel origin + offset) and stores 16 bytes.
    const int chunks = g.cp / 16;          // <= 256 (K <= 4096)
    const int ppi = 256 / chunks;          // pixels per pass over the workgroup
    const int chunk = tid % chunks, p0 = tid / chunks;
    if (p0 >= ppi) return;
    const int taps = g.kh * g.kw;
    int off[16];
    {
        int k = chunk * 16;
        int ci = k / taps;
        int kh = (k - ci * taps) / g.kw;
        int kw = k - ci * taps - kh * g.kw;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            off[j] = k < g.kk ? (ci * g.kh + kh) * wpatch + kw * g.dw : -1;   // K padding reads as zero
            ++k;
            if (++kw == g.kw) {
                kw = 0;
                if (++kh == g.kh) {
                    kh = 0;
                    ++ci;
                }
            }
        }
    }
    int8_t *dst = xs + (int64_t(ni) * g.ho + oh) * g.wo * g.cp + chunk * 16;
    for (int ow = p0; ow < g.wo; ow += ppi) {
        const int8_t *base = patch + ow * g.sw;
        uint32_t words[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            uint32_t word = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int o = off[v * 4 + j];
                const int b = base[o >= 0 ? o : 0];
                const int q = o >= 0 ? b : 0;
                word |= uint32_t(q & 0xff) << (8 * j);
            }
            words[v] = word;
        }
        *reinterpret_cast<uint4 *>(dst + int64_t(ow) * g.cp) = make_uint4(words[0], words[1], words[2], words[3]);
    }
}

// Whole staged buffer = halo: T(padding_value) in the real channels, 0 in the channel padding.
__global__ __launch_bounds__(256) void stage_fill_kernel(int8_t *__restrict__ xs, int64_t chunks, int cp, int c, int pad_value) {
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= chunks) return;
    const int c0 = int((id * 16) % cp);
    uint32_t words[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (c0 + v * 4 + j < c) word |= uint32_t(pad_value & 0xff) << (8 * j);
        words[v] = word;
    }
    *reinterpret_cast<uint4 *>(xs + id * 16) = make_uint4(words[0], words[1], words[2], words[3]);
}

// The same for a buffer whose interior a producer is about to write: only the halo pixels and the channel padding
// (every 16-byte chunk that is not wholly real channels of an interior pixel; the producer's epilogue writes
// those, 16 channels at a time).
__global__ __launch_bounds__(256) void stage_fill_halo_kernel(int8_t *__restrict__ xs, int64_t chunks, int hs, int ws, int cp, int c,
                                                             int pad_top, int pad_left, int h, int w, int pad_value) {
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= chunks) return;
    const int cpc = cp / 16;
    const int64_t pixel = id / cpc;
    const int c0 = int(id - pixel * cpc) * 16;
    const int col = int(pixel % ws), row = int((pixel / ws) % hs);
    const bool inside = row >= pad_top && row < pad_top + h && col >= pad_left && col < pad_left + w;
    if (inside && c0 + 16 <= c) return;
    uint32_t words[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        uint32_t word = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (c0 + v * 4 + j < c) word |= uint32_t(pad_value & 0xff) << (8 * j);
        words[v] = word;
    }
    *reinterpret_cast<uint4 *>(xs + id * 16) = make_uint4(words[0], words[1], words[2], words[3]);
}

// ... and when the layer has no channel padding at all, one lane per 16-byte chunk of a HALO pixel only: the lanes
// of the scan above that land on interior pixels are most of a large map.
__global__ __launch_bounds__(256) void stage_fill_halo_only_kernel(int8_t *__restrict__ xs, int64_t chunks, int hs, int ws, int cp,
                                                                  int pad_top, int pad_left, int h, int w, int pad_value) {
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= chunks) return;
    const int cpc = cp / 16;
    const int halo_px = hs * ws - h * w;                  // per image
    const int64_t hp_all = id / cpc;
    const int chunk = int(id - hp_all * cpc);
    const int img = int(hp_all / halo_px);
    int hp = int(hp_all - int64_t(img) * halo_px);
    int row, col;
    const int above = pad_top * ws, below = (hs - pad_top - h) * ws;
    if (hp < above) {
        row = hp / ws;
        col = hp - row * ws;
    } else if (hp < above + below) {
        hp -= above;
        row = hp / ws;
        col = hp - row * ws;
        row += pad_top + h;
    } else {
        hp -= above + below;
        const int side = ws - w;                          // halo pixels beside one interior row
        row = hp / side;
        const int k = hp - row * side;
        row += pad_top;
        col = k < pad_left ? k : w + k;
    }
    const uint32_t word = uint32_t(pad_value & 0xff) * 0x01010101u;
    *reinterpret_cast<uint4 *>(xs + ((int64_t(img) * hs + row) * ws + col) * cp + chunk * 16) = make_uint4(word, word, word, word);
}

// ------------------------------------------------------------------ weight packing

// packed[ks][frag][half][lane][16]: ks = tap * cblocks + cb (tap = kh*KW + kw),
// frag = cout / 32, and lane l of (frag, half) holds, for cout = frag*32 + l%32, the 16
// channels cb*64 + half*32 + (l/32)*16 + 0..15 of that tap.  Rows >= cout and channels >= c
// are zero.  w is OIHW ([cout][c][kh][kw]); for GEMM weights kh = kw = 1 and the element
// (k, n) sits at w[k * ldk + n * ldn].
__global__ __launch_bounds__(256) void pack_weights_kernel(const int8_t *__restrict__ w, int cout, int c, int taps,
                                                          int64_t ld_cout, int64_t ld_c, int64_t ld_tap,
                                                          int coutp, int cblocks, int8_t *__restrict__ packed) {
    const int frags = coutp / 32;
    const int64_t total = int64_t(taps) * cblocks * frags * 2 * 64;
    const int64_t id = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (id >= total) return;
    const int lane = int(id % 64);
    int64_t rest = id / 64;
    const int half = int(rest % 2);
    rest /= 2;
    const int frag = int(rest % frags);
    const int ks = int(rest / frags);
    const int tap = ks / cblocks, cb = ks % cblocks;
    const int co = frag * 32 + lane % 32;
    const int c0 = cb * 64 + half * 32 + (lane / 32) * 16;
    uint32_t words[4] = {0, 0, 0, 0};
    if (co < cout) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int ci = c0 + j;
            const int v = ci < c ? w[co * ld_cout + ci * ld_c + tap * ld_tap] : 0;
            words[j / 4] |= uint32_t(v & 0xff) << (8 * (j % 4));
        }
    }
    *reinterpret_cast<uint4 *>(packed + id * 16) = make_uint4(words[0], words[1], words[2], words[3]);
}

// ------------------------------------------------------------------ implicit GEMM

struct GemmParams : tsx::EpiParams {
    const int8_t *xs;      // staged activations
    const int8_t *wp;      // packed weights
    int positions;         // N*Ho*Wo (GEMM: rows)
    int howo, wo;          // Ho*Wo, Wo
    int hs, ws, cp;        // staged extent
    int stride_h, stride_w, dil_h, dil_w, kw;
    int taps, cblocks;
    int cout, coutp;
};

using tsx::emit;

// BM x BN tile, WGM x WGN wavefronts.  SWAP=false: MFMA rows = cout, columns = positions
// (lanes along positions: NCHW conv output).  SWAP=true: rows = positions, columns = cout
// (lanes along cout: row-major GEMM output, howo == 1).
template <int BM, int BN, int WGM, int WGN, bool SWAP>
__global__ __launch_bounds__(WGM *WGN * 64) void igemm_i8_kernel(GemmParams p) {
    constexpr int THREADS = WGM * WGN * 64;
    constexpr int FM = BM / WGM / 32, FN = BN / WGN / 32;
    constexpr int A_BYTES = BM * KSTEP, B_BYTES = BN * KSTEP;
    constexpr int A_LOADS = A_BYTES / 16 / THREADS, B_LOADS = B_BYTES / 16 / THREADS;
    static_assert(A_LOADS >= 1 && B_LOADS >= 1, "tile too small for the workgroup");
    static_assert(A_BYTES % (16 * THREADS) == 0 && B_BYTES % (16 * THREADS) == 0, "tile/threads mismatch");

    __shared__ __attribute__((aligned(16))) int8_t lds[2][A_BYTES + B_BYTES];

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wm = wave / WGN, wn = wave % WGN;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    // Source pointers of the 16-byte chunks this thread copies per K-step.
    const int8_t *b_src[B_LOADS];
    int b_dst[B_LOADS];
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
        const int q = tid + i * THREADS;
        const int row = q / 4, chunk = q % 4;
        int pos = n0 + row;
        if (pos >= p.positions) pos = 0;  // clamp: computed but never stored
        const int n = pos / p.howo;
        const int r = pos - n * p.howo;
        const int ho = r / p.wo, wo = r - ho * p.wo;
        b_src[i] = p.xs + ((int64_t(n) * p.hs + ho * p.stride_h) * p.ws + wo * p.stride_w) * p.cp + chunk * 16;
        b_dst[i] = A_BYTES + row * 64 + ((chunk ^ ((row >> 1) & 3)) * 16);
    }
    const int8_t *a_src = p.wp + (int64_t(m0 / 32) * 2 * 64 + tid) * 16;
    const int64_t a_kstride = int64_t(p.coutp / 32) * 2 * 64 * 16;

    // LDS read offsets of this lane's MFMA operands (per half: + 1024 for A, chunk swizzle for B)
    int a_off[FM], b_off[FN][2];
#pragma unroll
    for (int i = 0; i < FM; ++i) a_off[i] = ((wm * FM + i) * 2 * 64 + lane) * 16;
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int row = (wn * FN + j) * 32 + lane % 32;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int chunk = half * 2 + lane / 32;
            b_off[j][half] = A_BYTES + row * 64 + ((chunk ^ ((row >> 1) & 3)) * 16);
        }
    }

    v16i acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int ksteps = p.taps * p.cblocks;
    v4i a_reg[A_LOADS], b_reg[B_LOADS];   // native vectors: arrays of HIP's uint4 struct can end up in scratch

    // K-step ks = tap * cblocks + cb; (tap, cb) advance incrementally.
    int tap = 0, cb = 0;
    int64_t tap_off = 0;
#define TSX_LOAD_GLOBAL()                                                                                       \
    {                                                                                                           \
        _Pragma("unroll") for (int i = 0; i < A_LOADS; ++i) a_reg[i] =  \
            *reinterpret_cast<const v4i *>(a_src + int64_t(i) * THREADS * 16);                               \
        _Pragma("unroll") for (int i = 0; i < B_LOADS; ++i) b_reg[i] =  \
            *reinterpret_cast<const v4i *>(b_src[i] + tap_off);                                                \
    }
#define TSX_ADVANCE()                                                                                           \
    {                                                                                                           \
        a_src += a_kstride;                                                                                     \
        if (++cb == p.cblocks) {                                                                                \
            cb = 0;                                                                                             \
            ++tap;                                                                                              \
            const int kr = tap / p.kw, kc = tap - kr * p.kw;                                                    \
            tap_off = (int64_t(kr) * p.dil_h * p.ws + kc * p.dil_w) * p.cp;                                     \
        } else {                                                                                                \
            tap_off += 64;                                                                                      \
        }                                                                                                       \
    }
#define TSX_STORE_LDS(buf)                                                                                      \
    {                                                                                                           \
        _Pragma("unroll") for (int i = 0; i < A_LOADS; ++i)                                                     \
            *reinterpret_cast<v4i *>(&lds[buf][(tid + i * THREADS) * 16]) = a_reg[i];                           \
        _Pragma("unroll") for (int i = 0; i < B_LOADS; ++i)                                                     \
            *reinterpret_cast<v4i *>(&lds[buf][b_dst[i]]) = b_reg[i];                                           \
    }
#define TSX_COMPUTE(buf)                                                                                        \
    {                                                                                                           \
        _Pragma("unroll") for (int half = 0; half < 2; ++half) {                                               \
            v4i a[FM], b[FN];                                                                                   \
            _Pragma("unroll") for (int i = 0; i < FM; ++i) a[i] =                                             \
                *reinterpret_cast<const v4i *>(&lds[buf][a_off[i] + half * 1024]);                              \
            _Pragma("unroll") for (int j = 0; j < FN; ++j) b[j] =                                             \
                *reinterpret_cast<const v4i *>(&lds[buf][b_off[j][half]]);                                      \
            _Pragma("unroll") for (int i = 0; i < FM; ++i) _Pragma("unroll") for (int j = 0; j < FN; ++j)     \
                acc[i][j] = SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(b[j], a[i], acc[i][j], 0, 0, 0)        \
                                 : __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);       \
        }                                                                                                       \
    }

    TSX_LOAD_GLOBAL();
    TSX_STORE_LDS(0);
    __syncthreads();
    int buf = 0;
    for (int ks = 0; ks + 1 < ksteps; ++ks) {
        TSX_ADVANCE();
        TSX_LOAD_GLOBAL();      // K-step ks+1 -> registers, in flight during the MFMAs below
        TSX_COMPUTE(buf);
        TSX_STORE_LDS(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
    TSX_COMPUTE(buf);
#undef TSX_LOAD_GLOBAL
#undef TSX_ADVANCE
#undef TSX_STORE_LDS
#undef TSX_COMPUTE

    // Accumulator register r of lane l: row 8*(r/4) + 4*(l/32) + r%4, column l%32.
    if (!SWAP) {
        // columns = positions (one per lane and j), rows = cout
        int64_t base[FN];
        bool ok[FN];
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int pos = n0 + (wn * FN + j) * 32 + lane % 32;
            ok[j] = pos < p.positions;
            const int n = pos / p.howo;
            base[j] = int64_t(n) * p.cout * p.howo + (pos - n * p.howo);
        }
        // Fast path per 32-channel fragment: taken when no raw accumulators are wanted, every element is in
        // the activation's SIMD-body range and the consumer's quantize scale is uniform per image (one
        // group per image, or a single scale whose half-even bulk covers everything).
        const int64_t count = int64_t(p.positions) * p.cout;
        const bool want_q = p.out_i8 || p.st_out;
        const bool q_uniform = !want_q || (p.n_qscales == 1 ? p.q_bulk8 == count : p.q_group_len == int64_t(p.cout) * p.howo);
        const bool fast = (p.out_f32 || want_q) && !p.out_acc && p.act_body == count && q_uniform;
        tsx::static_for<0, FM>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const int cf = m0 + (wm * FM + i) * 32;            // first channel of the fragment (uniform)
            if (fast && cf + 32 <= p.cout) {
                const int co0 = cf + 4 * (lane / 32);
                float dq[16], bias[16];
                tsx::static_for<0, 16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    const int co = co0 + 8 * (r / 4) + (r % 4);
                    dq[r] = p.dq[co];
                    bias[r] = p.bias ? p.bias[co] : 0.f;
                });
                tsx::static_for<0, FN>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    if (ok[j]) {
                        const int pos = n0 + (wn * FN + j) * 32 + lane % 32;
                        const int n = pos / p.howo;
                        int8_t *st_dst = nullptr;
                        if (p.st_out) {
                            const int rem = pos - n * p.howo;
                            const int oh = rem / p.wo, ow = rem - oh * p.wo;
                            const int up = p.st_up == 2 ? 2 : 1;
                            st_dst = p.st_out + ((int64_t(n) * p.st_hs + up * oh + p.st_pt) * p.st_ws + up * ow + p.st_pl) * p.st_cp + co0;
                        }
                        const float qs = want_q ? p.q_scales[p.n_qscales == 1 ? 0 : n] : 0.f;
                        tsx::epilogue_rows16(p, acc[i][j], dq, bias, base[j] + int64_t(co0) * p.howo, p.howo, qs,
                                             p.n_qscales == 1, st_dst);
                    }
                });
            } else {
                tsx::static_for<0, 16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    const int co = cf + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
                    if (co < p.cout) {
                        const float dq = p.dq ? p.dq[co] : 0.f;
                        const float bias = p.bias ? p.bias[co] : 0.f;
                        tsx::static_for<0, FN>([&](auto jc) {
                            constexpr int j = decltype(jc)::value;
                            if (ok[j]) emit(p, acc[i][j][r], base[j] + int64_t(co) * p.howo, dq, bias, 0.f);
                        });
                    }
                });
            }
        });
    } else {
        // columns = cout (one per lane and i), rows = positions; output is [positions][cout]
        float dq[FM], bias[FM];
        int co[FM];
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            co[i] = m0 + (wm * FM + i) * 32 + lane % 32;
            const bool in = co[i] < p.cout;
            dq[i] = (in && p.dq) ? p.dq[co[i]] : 0.f;
            bias[i] = (in && p.bias) ? p.bias[co[i]] : 0.f;
        }
        tsx::static_for<0, FN>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            tsx::static_for<0, 16>([&](auto rc) {
                constexpr int r = decltype(rc)::value;
                const int pos = n0 + (wn * FN + j) * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
                if (pos < p.positions) {
                    const float rs = p.row_scale ? p.row_scale[pos] : 0.f;
                    tsx::static_for<0, FM>([&](auto ic) {
                        constexpr int i = decltype(ic)::value;
                        if (co[i] < p.cout) emit(p, acc[i][j][r], int64_t(pos) * p.cout + co[i], dq[i], bias[i], rs);
                    });
                }
            });
        });
    }
}

// ------------------------------------------------------------------ skinny int8 GEMM (m <= 32 rows)
// With at most 32 activation rows the whole left operand is ONE MFMA B fragment and the GEMM is a
// stream over the packed weights: HBM-bound (K*N bytes), not MFMA-bound.  The 128x128-tile kernel
// would launch N/128 workgroups and walk K serially; here one workgroup owns 32 output columns and
// its 8 wavefronts split K (interleaved K-steps, 4 in flight each), then add their int32 partial
// sums through LDS -- exact, so results equal the tiled kernel's and the oracle's.
// acc register r of lane l: column (weight row) 8*(r/4) + 4*(l/32) + r%4 of the fragment, activation row l%32.
constexpr int SK_WAVES = 8;
constexpr int SK_BATCH = 4;

__global__ __launch_bounds__(SK_WAVES * 64) void gemm_i8_skinny_kernel(GemmParams p) {
    __shared__ int red[SK_WAVES][16][64];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int frag = blockIdx.x;
    const int frags = p.coutp / 32;
    const int ksteps = p.cblocks;
    const int row = lane % 32;
    const bool row_ok = row < p.positions;
    // B operand: activation row `row`, the 16 K bytes of group lane/32 of each half K-step
    const int8_t *b_ptr = p.xs + int64_t(row_ok ? row : 0) * p.cp + (lane / 32) * 16;
    // A operand: packed[ks][frag][half][lane][16]
    const int8_t *a_ptr = p.wp + (int64_t(frag) * 128 + lane) * 16;
    const int64_t a_kstride = int64_t(frags) * 2048;
    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0;
    const v4i zero = {0, 0, 0, 0};
    for (int ks0 = wave; ks0 < ksteps; ks0 += SK_WAVES * SK_BATCH) {
        v4i a[SK_BATCH][2], b[SK_BATCH][2];
        tsx::static_for<0, SK_BATCH>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            const int ks = ks0 + u * SK_WAVES;
            const bool on = ks < ksteps;
            const int kk = on ? ks : 0;
            tsx::static_for<0, 2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                a[u][h] = on ? *reinterpret_cast<const v4i *>(a_ptr + kk * a_kstride + h * 1024) : zero;
                b[u][h] = (on && row_ok) ? *reinterpret_cast<const v4i *>(b_ptr + kk * 64 + h * 32) : zero;
            });
        });
        tsx::static_for<0, SK_BATCH>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u][0], b[u][0], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u][1], b[u][1], acc, 0, 0, 0);
        });
    }
    tsx::static_for<0, 16>([&](auto rc) { red[wave][decltype(rc)::value][lane] = acc[decltype(rc)::value]; });
    __syncthreads();
    // wavefront w finishes accumulator registers 2w and 2w+1
    tsx::static_for<0, 2>([&](auto tc) {
        const int r = wave * 2 + decltype(tc)::value;
        int sum = 0;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w) sum += red[w][r][lane];
        const int co = frag * 32 + 8 * (r / 4) + 4 * (lane / 32) + (r % 4);
        if (row_ok && co < p.cout) {
            const float rs = p.row_scale ? p.row_scale[row] : 0.f;
            emit(p, sum, int64_t(row) * p.cout + co, p.dq ? p.dq[co] : 0.f, p.bias ? p.bias[co] : 0.f, rs);
        }
    });
}

// ------------------------------------------------------------------ K-split int8 GEMM (a few hundred rows)
// A GEMM with a few hundred activation rows and a large weight matrix has too few output tiles to give every CU a
// tile of a shape that reuses its operands: the tiled kernels would walk K serially on a fraction of the chip, or
// read the weights once per 32 rows.  Here a workgroup owns FR x FC fragments (32 FR rows x
// 32 FC output columns) and its 8 wavefronts SPLIT K (interleaved K-steps): each wavefront loads the operands of
// BATCH K-steps straight from global memory into MFMA operand registers (no LDS on the way in: no two wavefronts
// read the same bytes), multiplies them into its own FR x FC accumulators, and the eight partial tiles are added
// through LDS -- int32, exact, so the order is free and results equal the tiled kernels' and the oracle's.  The
// epilogue then runs on all eight wavefronts with lanes along 4 consecutive output columns (one 16-byte store per
// lane for plain fp32 output).
// acc register r of lane l: column (weight row) 8*(r/4) + 4*(l/32) + r%4 of the fragment, activation row l%32.
constexpr int KS_WAVES = 8;

// The end of a K-split tile: the eight wavefronts' partial accumulators go to LDS (SLOTS = 8: all eight and one
// barrier; SLOTS = 4, for a kernel with 64 KiB of LDS: wavefronts 4..7 hand theirs to 0..3 first), where every
// wavefront picks up its share of the sums and runs the epilogue on it: (fragment f, register group g) -- registers
// 4g .. 4g+3 of a lane are 4 consecutive output columns of one row.  The scales and biases of a wavefront's share are
// requested before the reduction and arrive under it.  red: SLOTS x FR FC x 16 x 64 ints.
template <int FR, int FC, int SLOTS>
__device__ __forceinline__ void ksplit_finish(const GemmParams &p, v16i (&acc)[FR][FC], int (*red)[FR * FC][16][64], int frag0,
                                              int row0, int lane, int wave) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    constexpr int FRAGS = FR * FC;
    constexpr int ITEMS = (FRAGS * 4 + KS_WAVES - 1) / KS_WAVES;
    const bool plain = p.out_f32 && !p.out_i8 && !p.st_out && !p.out_acc && !p.residual && p.act <= TSX_ACT_LEAKY_RELU &&
                       p.cout % 4 == 0 && reinterpret_cast<uintptr_t>(p.out_f32) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(p.dq) % 16 == 0 && reinterpret_cast<uintptr_t>(p.bias) % 16 == 0;
    int row[ITEMS], co[ITEMS];
    bool ok[ITEMS];
    float rs[ITEMS];
    v4f dq[ITEMS], bias[ITEMS];
    tsx::static_for<0, ITEMS>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        const int item = wave + KS_WAVES * i;
        const int f = item / 4, g4 = item % 4;
        row[i] = row0 + (f / FC) * 32 + lane % 32;
        co[i] = (frag0 + f % FC) * 32 + 8 * g4 + 4 * (lane / 32);
        ok[i] = item < FRAGS * 4 && row[i] < p.positions && co[i] < p.cout;
        rs[i] = (ok[i] && p.row_scale) ? p.row_scale[row[i]] : 0.f;
        const v4f z = {0.f, 0.f, 0.f, 0.f};
        dq[i] = (plain && ok[i]) ? *reinterpret_cast<const v4f *>(p.dq + co[i]) : z;      // co % 4 == 0
        bias[i] = (plain && ok[i] && p.bias) ? *reinterpret_cast<const v4f *>(p.bias + co[i]) : z;
    });
    if (SLOTS == 8) {
        tsx::static_for<0, FRAGS>([&](auto fc_) {
            constexpr int f = decltype(fc_)::value;
            tsx::static_for<0, 16>([&](auto rc) { red[wave][f][decltype(rc)::value][lane] = acc[f / FC][f % FC][decltype(rc)::value]; });
        });
        __syncthreads();
    } else {
        if (wave >= 4) {
            tsx::static_for<0, FRAGS>([&](auto fc_) {
                constexpr int f = decltype(fc_)::value;
                tsx::static_for<0, 16>([&](auto rc) { red[wave - 4][f][decltype(rc)::value][lane] = acc[f / FC][f % FC][decltype(rc)::value]; });
            });
        }
        __syncthreads();
        if (wave < 4) {
            tsx::static_for<0, FRAGS>([&](auto fc_) {
                constexpr int f = decltype(fc_)::value;
                tsx::static_for<0, 16>([&](auto rc) { acc[f / FC][f % FC][decltype(rc)::value] += red[wave][f][decltype(rc)::value][lane]; });
            });
        }
        __syncthreads();
        if (wave < 4) {
            tsx::static_for<0, FRAGS>([&](auto fc_) {
                constexpr int f = decltype(fc_)::value;
                tsx::static_for<0, 16>([&](auto rc) { red[wave][f][decltype(rc)::value][lane] = acc[f / FC][f % FC][decltype(rc)::value]; });
            });
        }
        __syncthreads();
    }
    tsx::static_for<0, ITEMS>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        const int item = wave + KS_WAVES * i;
        if (item < FRAGS * 4) {         // uniform
            const int f = item / 4, g4 = item % 4;
            int sum[4] = {0, 0, 0, 0};
            tsx::static_for<0, SLOTS>([&](auto sc) {
                constexpr int sl = decltype(sc)::value;
#pragma unroll
                for (int j = 0; j < 4; ++j) sum[j] += red[sl][f][4 * g4 + j][lane];
            });
            if (ok[i]) {
                const int64_t idx = int64_t(row[i]) * p.cout + co[i];
                if (plain) {
                    v4f v;
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = tsx::epi_value<false>(p, sum[j], idx + j, dq[i][j], bias[i][j], rs[i]);
                    *reinterpret_cast<v4f *>(p.out_f32 + idx) = v;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (co[i] + j < p.cout)
                            emit(p, sum[j], idx + j, p.dq ? p.dq[co[i] + j] : 0.f, p.bias ? p.bias[co[i] + j] : 0.f, rs[i]);
                }
            }
        }
    });
}

template <int FR, int FC, int BATCH>
__global__ __launch_bounds__(KS_WAVES * 64) void gemm_i8_ksplit_kernel(GemmParams p) {
    constexpr int FRAGS = FR * FC;
    __shared__ int red[4][FRAGS][16][64];
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int frag0 = blockIdx.x * FC, row0 = blockIdx.y * FR * 32;
    const int frags = p.coutp / 32;
    const int ksteps = p.cblocks;
    // B operands: activation rows row0 + 32 fr + lane % 32 (beyond m: the last row, never stored), the 16 K bytes
    // of group lane / 32 of each half K-step.  Lanes of rows beyond m load nothing (a masked lane costs the
    // memory pipeline nothing; with a single row the B loads all but vanish).
    const int8_t *b_ptr[FR];
    bool row_ok[FR];
    tsx::static_for<0, FR>([&](auto fc_) {
        constexpr int fr = decltype(fc_)::value;
        b_ptr[fr] = p.xs + int64_t(min(row0 + fr * 32 + lane % 32, p.positions - 1)) * p.cp + (lane / 32) * 16;
        row_ok[fr] = row0 + fr * 32 + lane % 32 < p.positions;
    });
    // A operands: packed[ks][frag][half][lane][16]; fragments beyond the packed columns: the last one, never stored
    const int8_t *a_ptr[FC];
    tsx::static_for<0, FC>([&](auto fc_) {
        constexpr int fc = decltype(fc_)::value;
        a_ptr[fc] = p.wp + (int64_t(min(frag0 + fc, frags - 1)) * 128 + lane) * 16;
    });
    const int64_t a_kstride = int64_t(frags) * 2048;
    v16i acc[FR][FC];
    tsx::static_for<0, FRAGS>([&](auto fc_) {
        constexpr int f = decltype(fc_)::value;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[f / FC][f % FC][r] = 0;
    });
    const v4i zero = {0, 0, 0, 0};
    for (int ks0 = wave; ks0 < ksteps; ks0 += KS_WAVES * BATCH) {
        v4i a[BATCH][FC][2], b[BATCH][FR][2];
        tsx::static_for<0, BATCH>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            const int ks = ks0 + u * KS_WAVES;
            const bool on = ks < ksteps;        // uniform
            const int kk = on ? ks : 0;
            tsx::static_for<0, 2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                tsx::static_for<0, FC>([&](auto fc_) {
                    constexpr int fc = decltype(fc_)::value;
                    a[u][fc][h] = on ? *reinterpret_cast<const v4i *>(a_ptr[fc] + kk * a_kstride + h * 1024) : zero;
                });
                tsx::static_for<0, FR>([&](auto fr_) {
                    constexpr int fr = decltype(fr_)::value;
                    b[u][fr][h] = (on && row_ok[fr]) ? *reinterpret_cast<const v4i *>(b_ptr[fr] + kk * 64 + h * 32) : zero;
                });
            });
        });
        tsx::static_for<0, BATCH>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            tsx::static_for<0, 2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                tsx::static_for<0, FRAGS>([&](auto fc_) {
                    constexpr int fr = decltype(fc_)::value / FC, fc = decltype(fc_)::value % FC;
                    acc[fr][fc] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u][fc][h], b[u][fr][h], acc[fr][fc], 0, 0, 0);
                });
            });
        });
    }
    ksplit_finish<FR, FC, 4>(p, acc, red, frag0, row0, lane, wave);
}

// The same tile with the activations through LDS.  Read straight into MFMA operand registers, the activation
// operand of a K-step is 32 rows x 32 bytes per load instruction, which the CU's vector memory path serves at half
// the rate of whole cache lines.  Here the workgroup copies its 64 rows in chunks of 16 K-steps (1 KiB per row, one
// row per load instruction, double-buffered: chunk c + 1 is on its way while chunk c is multiplied, one barrier per
// chunk) and every wavefront reads the operands of its own two K-steps of the chunk from LDS; the weights still go
// from global memory straight into registers (1 KiB contiguous per operand).  For K of 2048 and more.
constexpr int KL_CHUNK = 16;                      // K-steps per chunk
constexpr int KL_PITCH = KL_CHUNK * KSTEP + 16;   // bytes per row and chunk in LDS (the 16: rows 8 apart share banks, not all)
constexpr int KL_LDS = 2 * 64 * KL_PITCH;         // two chunk buffers; the partial tiles reuse them (131 072 bytes)

__global__ __launch_bounds__(KS_WAVES * 64) void gemm_i8_ksplit_lds_kernel(GemmParams p) {
    extern __shared__ __attribute__((aligned(16))) int8_t kl_lds[];
    static_assert(KL_LDS >= 8 * 4 * 16 * 64 * 4, "the chunk buffers hold the eight partial tiles");
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int frag0 = blockIdx.x * 2, row0 = blockIdx.y * 64;
    const int frags = p.coutp / 32;
    const int ksteps = p.cblocks;
    const int chunks = (ksteps + KL_CHUNK - 1) / KL_CHUNK;
    const v4i zero = {0, 0, 0, 0};
    // chunk copy: wavefront w moves rows w, w + 8, ... (beyond m: the last row, never stored), lane l bytes 16 l ..
    const int8_t *src[8];
    tsx::static_for<0, 8>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        src[i] = p.xs + int64_t(min(row0 + wave + 8 * i, p.positions - 1)) * p.cp + lane * 16;
    });
    v4i stage[8];
    auto load_chunk = [&](int c) __attribute__((always_inline)) {
        const int koff = c * (KL_CHUNK * KSTEP);
        const bool inside = koff + lane * 16 < p.cp;             // K-steps beyond K: zeros
        tsx::static_for<0, 8>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            stage[i] = inside ? *reinterpret_cast<const v4i *>(src[i] + koff) : zero;
        });
    };
    auto store_chunk = [&](int buf) __attribute__((always_inline)) {
        tsx::static_for<0, 8>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            *reinterpret_cast<v4i *>(kl_lds + (buf * 64 + wave + 8 * i) * KL_PITCH + lane * 16) = stage[i];
        });
    };
    const int8_t *a_ptr[2];
    tsx::static_for<0, 2>([&](auto fc_) {
        constexpr int fc = decltype(fc_)::value;
        a_ptr[fc] = p.wp + (int64_t(min(frag0 + fc, frags - 1)) * 128 + lane) * 16;
    });
    const int64_t a_kstride = int64_t(frags) * 2048;
    v16i acc[2][2];
    tsx::static_for<0, 4>([&](auto fc_) {
        constexpr int f = decltype(fc_)::value;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[f / 2][f % 2][r] = 0;
    });
    // this wavefront's K-steps of a chunk: wave and wave + 8; their weights are requested a chunk ahead
    v4i a_next[2][2][2];
    auto load_weights = [&](int c) __attribute__((always_inline)) {
        tsx::static_for<0, 2>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            const int ks = c * KL_CHUNK + wave + 8 * u;
            const bool on = ks < ksteps;        // uniform
            const int kk = on ? ks : 0;
            tsx::static_for<0, 2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                tsx::static_for<0, 2>([&](auto fc_) {
                    constexpr int fc = decltype(fc_)::value;
                    a_next[u][fc][h] = on ? *reinterpret_cast<const v4i *>(a_ptr[fc] + kk * a_kstride + h * 1024) : zero;
                });
            });
        });
    };
    load_chunk(0);
    load_weights(0);
    store_chunk(0);
    __syncthreads();
    for (int c = 0; c < chunks; ++c) {
        v4i a[2][2][2], b[2][2][2];
        tsx::static_for<0, 8>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            a[i / 4][(i / 2) % 2][i % 2] = a_next[i / 4][(i / 2) % 2][i % 2];
        });
        if (c + 1 < chunks) {
            load_chunk(c + 1);
            load_weights(c + 1);
        }
        tsx::static_for<0, 2>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            tsx::static_for<0, 2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                tsx::static_for<0, 2>([&](auto fr_) {
                    constexpr int fr = decltype(fr_)::value;
                    b[u][fr][h] = *reinterpret_cast<const v4i *>(kl_lds + ((c & 1) * 64 + fr * 32 + lane % 32) * KL_PITCH +
                                                                 (wave + 8 * u) * KSTEP + h * 32 + (lane / 32) * 16);
                });
            });
        });
        tsx::static_for<0, 2>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            tsx::static_for<0, 2>([&](auto hc) {
                constexpr int h = decltype(hc)::value;
                tsx::static_for<0, 4>([&](auto fc_) {
                    constexpr int fr = decltype(fc_)::value / 2, fc = decltype(fc_)::value % 2;
                    acc[fr][fc] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u][fc][h], b[u][fr][h], acc[fr][fc], 0, 0, 0);
                });
            });
        });
        if (c + 1 < chunks) store_chunk((c + 1) & 1);
        __syncthreads();
    }
    ksplit_finish<2, 2, 8>(p, acc, reinterpret_cast<int (*)[4][16][64]>(kl_lds), frag0, row0, lane, wave);
}

// ------------------------------------------------------------------ host side

constexpr int BM = 128, BN = 128;

struct Plan {
    int ho, wo, hs, ws, cp, cblocks, taps, coutp;
    int64_t positions;
    size_t staged_bytes, packed_bytes;
    // few input channels x large kernel: K packed by explicit im2col, the layer runs as a 1x1 convolution
    bool im2col;
    int kk;   // C*KH*KW
    // layers whose tap window fits LDS take the window-stationary kernel
    bool use_ws;
    tsx::WsGeom wsg;
    tsx::WsPlan wsp;
};

int make_plan(const tsx_conv2d_geom *g, Plan *pl) {
    TSX_REQUIRE(g, "null geometry");
    TSX_REQUIRE(g->n > 0 && g->c > 0 && g->h > 0 && g->w > 0 && g->cout > 0 && g->kh > 0 && g->kw > 0,
                "conv2d_i8: non-positive extent");
    TSX_REQUIRE(g->stride_h > 0 && g->stride_w > 0 && g->dilation_h > 0 && g->dilation_w > 0,
                "conv2d_i8: stride and dilation must be positive");
    TSX_REQUIRE(g->pad_top >= 0 && g->pad_bottom >= 0 && g->pad_left >= 0 && g->pad_right >= 0,
                "conv2d_i8: negative padding is not supported");
    pl->ho = tsx::conv_out(g->h, g->pad_top, g->pad_bottom, g->kh, g->stride_h, g->dilation_h);
    pl->wo = tsx::conv_out(g->w, g->pad_left, g->pad_right, g->kw, g->stride_w, g->dilation_w);
    TSX_REQUIRE(pl->ho > 0 && pl->wo > 0, "conv2d_i8: empty output %dx%d", pl->ho, pl->wo);
    // Rows/columns the kernel actually reads: up to (ho-1)*stride + (k-1)*dilation.
    pl->hs = (pl->ho - 1) * g->stride_h + (g->kh - 1) * g->dilation_h + 1;
    pl->ws = (pl->wo - 1) * g->stride_w + (g->kw - 1) * g->dilation_w + 1;
    pl->cp = int(tsx::round_up(g->c, KSTEP));
    pl->cblocks = pl->cp / KSTEP;
    pl->taps = g->kh * g->kw;
    pl->kk = g->c * pl->taps;
    // padding C to 64 per tap wastes (64-C)/64 of the MFMA work; packing K costs a larger staged copy
    pl->im2col = pl->taps > 1 && g->c <= 8 && pl->kk <= 512;
    if (pl->im2col) {
        pl->hs = pl->ho;
        pl->ws = pl->wo;
        pl->cp = int(tsx::round_up(pl->kk, KSTEP));
        pl->cblocks = pl->cp / KSTEP;
        pl->taps = 1;
    }
    pl->coutp = int(tsx::round_up(g->cout, BM));
    pl->positions = int64_t(g->n) * pl->ho * pl->wo;
    TSX_REQUIRE(pl->positions < (int64_t(1) << 31), "conv2d_i8: too many output positions");
    pl->staged_bytes = size_t(g->n) * pl->hs * pl->ws * pl->cp;
    pl->packed_bytes = size_t(pl->taps) * pl->cblocks * pl->coutp * KSTEP;
    pl->use_ws = false;
    {
        pl->wsg = tsx::WsGeom{g->n, g->cout, pl->ho, pl->wo, pl->hs, pl->ws, pl->cp, pl->cblocks,
                              pl->im2col ? 1 : g->kh, pl->im2col ? 1 : g->kw,
                              pl->im2col ? 1 : g->dilation_h, pl->im2col ? 1 : g->dilation_w,
                              pl->im2col ? 1 : g->stride_h, pl->im2col ? 1 : g->stride_w, 0};
        pl->wsp = tsx::ws_plan(pl->wsg);
        // a strided 1x1 layer would fill its window with pixels it skips (3 of 4 at stride 2): the generic
        // kernel, which gathers only the pixels it multiplies, is the faster one there
        const bool strided_1x1 = !pl->im2col && pl->taps == 1 && (g->stride_h > 1 || g->stride_w > 1);
        if (pl->wsp.ok && !strided_1x1) {
            pl->use_ws = true;
            pl->packed_bytes = pl->wsp.packed_bytes;
        }
    }
    return 0;
}

int check_epilogue(const tsx_epilogue *ep, const float *out_f32, const int8_t *out_i8, const int32_t *out_acc,
                   int64_t groups, int cout = 0, int ho = 0, int wo = 0) {
    const bool staged_out = ep && ep->staged_out_dev;
    TSX_REQUIRE(out_f32 || out_i8 || out_acc || staged_out, "no output requested");
    if (staged_out) {
        TSX_REQUIRE(cout > 0, "staged output is a convolution-only epilogue term");
        TSX_REQUIRE(ep->dq_dev && ep->q_scales_dev && ep->n_qscales == groups,
                    "staged output needs dequantize scales and one consumer quantize scale per image");
        TSX_REQUIRE(ep->staged_upsample >= 0 && ep->staged_upsample <= 2, "staged output: upsample factor %d (1 or 2)", ep->staged_upsample);
        const int up = ep->staged_upsample == 2 ? 2 : 1;
        TSX_REQUIRE(ep->staged_pad_top >= 0 && ep->staged_pad_left >= 0 && ep->staged_cp >= cout && ep->staged_cp % 32 == 0 &&
                        up * ho + ep->staged_pad_top <= ep->staged_hs && up * wo + ep->staged_pad_left <= ep->staged_ws,
                    "staged output: %dx%dx%d does not fit [%d][%d][%d] at (%d,%d)", ho, wo, cout, ep->staged_hs,
                    ep->staged_ws, ep->staged_cp, ep->staged_pad_top, ep->staged_pad_left);
        TSX_REQUIRE(reinterpret_cast<uintptr_t>(ep->staged_out_dev) % 16 == 0, "staged output must be 16-byte aligned");
    }
    if (out_f32 || out_i8) {
        TSX_REQUIRE(ep && ep->dq_dev, "epilogue with dequantize scales required for fp32/int8 output");
        TSX_REQUIRE(ep->act >= TSX_ACT_NONE && ep->act <= TSX_ACT_MISH_FAST, "unknown activation %d", ep->act);
    }
    if (out_i8) {
        TSX_REQUIRE(ep->q_scales_dev, "int8 output needs q_scales_dev");
        // base_quantize.cpp:26: the consumer's scale count equals its input's first extent
        TSX_REQUIRE(ep->n_qscales == groups, "n_qscales (%d) must equal the output's first extent (%lld)",
                    ep->n_qscales, (long long)groups);
    }
    return 0;
}

void fill_epilogue(tsx::EpiParams &p, const tsx_epilogue *ep, int64_t count, float *out_f32, int8_t *out_i8,
                   int32_t *out_acc) {
    p.dq = ep ? ep->dq_dev : nullptr;
    p.row_scale = ep ? ep->row_scale_dev : nullptr;
    p.bias = ep ? ep->bias_dev : nullptr;
    p.q_scales = ep ? ep->q_scales_dev : nullptr;
    p.residual = ep ? ep->residual_dev : nullptr;
    p.res_after = (ep && ep->residual_dev && ep->residual_after_act) ? 1 : 0;
    p.act = ep ? ep->act : 0;
    p.slope = ep ? ep->slope : 0.f;
    p.n_qscales = ep ? ep->n_qscales : 0;
    p.q_group_len = p.n_qscales > 0 ? int64_t(std::ceil(static_cast<float>(count) / static_cast<float>(p.n_qscales))) : 1;
    p.q_bulk8 = (count >> 3) << 3;
    p.act_body = count / 4 * 4;
    p.out_f32 = out_f32;
    p.out_i8 = out_i8;
    p.out_acc = out_acc;
    p.st_out = ep ? ep->staged_out_dev : nullptr;
    if (p.st_out) {
        p.st_hs = ep->staged_hs;
        p.st_ws = ep->staged_ws;
        p.st_cp = ep->staged_cp;
        p.st_pt = ep->staged_pad_top;
        p.st_pl = ep->staged_pad_left;
        p.st_up = ep->staged_upsample == 2 ? 2 : 1;
    }
}

template <bool SWAP>
int launch_igemm(const GemmParams &p, hipStream_t stream) {
    dim3 grid(unsigned(tsx::ceil_div(p.positions, BN)), unsigned(p.coutp / BM));
    hipLaunchKernelGGL((igemm_i8_kernel<BM, BN, 2, 2, SWAP>), grid, dim3(256), 0, stream, p);
    TSX_LAUNCH_CHECK("igemm_i8_kernel");
    return 0;
}

int run_stage(const tsx_conv2d_geom *g, const Plan &pl, const void *x, bool x_is_f32, const float *x_scales,
              int n_x_scales, float padding_value, void *staged, size_t staged_bytes, hipStream_t stream) {
    TSX_REQUIRE(x, "conv2d_i8: null input");
    if (!staged || staged_bytes < pl.staged_bytes)
        return tsx::fail(TSX_E_WORKSPACE, "conv2d_i8: workspace %zu < %zu bytes", staged_bytes, pl.staged_bytes);
    TSX_REQUIRE(reinterpret_cast<uintptr_t>(staged) % 16 == 0, "conv2d_i8: workspace must be 16-byte aligned");
    if (pl.im2col) {
        const Im2colGeom ig{g->n, g->c, g->h, g->w, pl.ho, pl.wo, g->kh, g->kw, g->stride_h, g->stride_w, g->dilation_h,
                            g->dilation_w, g->pad_top, g->pad_left, pl.kk, pl.cp, int(int8_t(padding_value))};
        const int64_t threads = int64_t(pl.staged_bytes / 16);
        const dim3 grid(unsigned(tsx::ceil_div(threads, 256)));
        // patch columns an output row touches; the row kernel needs the C x KH patch rows in LDS
        const int wpatch = (pl.wo - 1) * g->stride_w + (g->kw - 1) * g->dilation_w + 1;
        const size_t patch_bytes = size_t(g->c) * g->kh * wpatch;
        const bool by_rows = patch_bytes <= 48 * 1024 && int64_t(g->n) * pl.ho < (int64_t(1) << 31);
        const dim3 row_grid(unsigned(int64_t(g->n) * pl.ho));
        if (x_is_f32) {
            TSX_REQUIRE(x_scales && n_x_scales >= 1, "quantize_conv2d_i8: missing quantize scales");
            TSX_REQUIRE(n_x_scales == g->n, "quantize_conv2d_i8: n_x_scales (%d) must equal the batch (%d)", n_x_scales, g->n);
            const int64_t count = int64_t(g->n) * g->c * g->h * g->w;
            const int64_t group_len = int64_t(std::ceil(static_cast<float>(count) / static_cast<float>(n_x_scales)));
            if (by_rows)
                hipLaunchKernelGGL(stage_im2col_rows_kernel<true>, row_grid, dim3(256), patch_bytes, stream, x, ig, wpatch, x_scales,
                                   n_x_scales, group_len, (count >> 3) << 3, static_cast<int8_t *>(staged));
            else
                hipLaunchKernelGGL(stage_im2col_kernel<true>, grid, dim3(256), 0, stream, x, ig, x_scales, n_x_scales, group_len,
                                   (count >> 3) << 3, static_cast<int8_t *>(staged));
        } else if (by_rows) {
            hipLaunchKernelGGL(stage_im2col_rows_kernel<false>, row_grid, dim3(256), patch_bytes, stream, x, ig, wpatch,
                               static_cast<const float *>(nullptr), 1, int64_t(1), int64_t(0), static_cast<int8_t *>(staged));
        } else {
            hipLaunchKernelGGL(stage_im2col_kernel<false>, grid, dim3(256), 0, stream, x, ig,
                               static_cast<const float *>(nullptr), 1, int64_t(1), int64_t(0), static_cast<int8_t *>(staged));
        }
        TSX_LAUNCH_CHECK("stage_im2col_kernel");
        return 0;
    }
    StageGeom sg{g->n, g->c, g->h, g->w, pl.hs, pl.ws, pl.cp, g->pad_top, g->pad_left,
                 int(int8_t(padding_value))};  // T(padding_value), conv2d_quantized_core.cpp:72
    const int64_t stage_threads = int64_t(g->n) * pl.hs * pl.ws * (pl.cp / 16);
    const unsigned stage_blocks = unsigned(tsx::ceil_div(stage_threads, 256));
    const bool by_rows = pl.ws <= STAGE_MAX_WS;
    const unsigned row_blocks = (unsigned(g->n) * unsigned(pl.hs) + 7) / 8 * 8;   // whole runs per XCD
    const size_t row_lds = size_t(pl.ws) * STAGE_LROW;
    if (x_is_f32) {
        TSX_REQUIRE(x_scales && n_x_scales >= 1, "quantize_conv2d_i8: missing quantize scales");
        // base_quantize.cpp:26
        TSX_REQUIRE(n_x_scales == g->n, "quantize_conv2d_i8: n_x_scales (%d) must equal the batch (%d)", n_x_scales, g->n);
        const int64_t count = int64_t(g->n) * g->c * g->h * g->w;
        const int64_t group_len = int64_t(std::ceil(static_cast<float>(count) / static_cast<float>(n_x_scales)));
        const bool fast = by_rows && n_x_scales > 1 && g->w % 4 == 0 && g->w <= 256 && reinterpret_cast<uintptr_t>(x) % 16 == 0;
        if (fast)
            hipLaunchKernelGGL((stage_rows_kernel<true, true>), dim3(row_blocks), dim3(256), row_lds, stream, x, sg, x_scales,
                               n_x_scales, group_len, (count >> 3) << 3, static_cast<int8_t *>(staged));
        else if (by_rows)
            hipLaunchKernelGGL((stage_rows_kernel<true, false>), dim3(row_blocks), dim3(256), row_lds, stream, x, sg, x_scales,
                               n_x_scales, group_len, (count >> 3) << 3, static_cast<int8_t *>(staged));
        else
            hipLaunchKernelGGL(stage_nchw_kernel<true>, dim3(stage_blocks), dim3(256), 0, stream, x, sg, x_scales,
                               n_x_scales, group_len, (count >> 3) << 3, static_cast<int8_t *>(staged));
    } else {
        const bool fast = by_rows && g->w % 4 == 0 && g->w <= 256 && reinterpret_cast<uintptr_t>(x) % 4 == 0;
        if (fast)
            hipLaunchKernelGGL((stage_rows_kernel<false, true>), dim3(row_blocks), dim3(256), row_lds, stream, x, sg,
                               static_cast<const float *>(nullptr), 1, int64_t(1), int64_t(0),
                               static_cast<int8_t *>(staged));
        else if (by_rows)
            hipLaunchKernelGGL((stage_rows_kernel<false, false>), dim3(row_blocks), dim3(256), row_lds, stream, x, sg,
                               static_cast<const float *>(nullptr), 1, int64_t(1), int64_t(0),
                               static_cast<int8_t *>(staged));
        else
            hipLaunchKernelGGL(stage_nchw_kernel<false>, dim3(stage_blocks), dim3(256), 0, stream, x, sg,
                               static_cast<const float *>(nullptr), 1, int64_t(1), int64_t(0),
                               static_cast<int8_t *>(staged));
    }
    TSX_LAUNCH_CHECK("stage_nchw_kernel");
    return 0;
}

int run_staged(const tsx_conv2d_geom *g, const Plan &pl, const void *staged, const void *packed_w,
               const tsx_epilogue *ep, float *out_f32, int8_t *out_i8, int32_t *out_acc, hipStream_t stream) {
    int rc = check_epilogue(ep, out_f32, out_i8, out_acc, g->n, g->cout, pl.ho, pl.wo);
    if (rc) return rc;
    TSX_REQUIRE(staged && packed_w, "conv2d_i8: null input");
    TSX_REQUIRE(!(ep && ep->row_scale_dev), "conv2d_i8: row_scale is a GEMM-only epilogue term");
    TSX_REQUIRE(reinterpret_cast<uintptr_t>(staged) % 16 == 0 && reinterpret_cast<uintptr_t>(packed_w) % 16 == 0,
                "conv2d_i8: staged activations and packed weights must be 16-byte aligned");
    GemmParams p{};
    p.xs = static_cast<const int8_t *>(staged);
    p.wp = static_cast<const int8_t *>(packed_w);
    p.positions = int(pl.positions);
    p.howo = pl.ho * pl.wo;
    p.wo = pl.wo;
    p.hs = pl.hs;
    p.ws = pl.ws;
    p.cp = pl.cp;
    p.stride_h = pl.im2col ? 1 : g->stride_h;
    p.stride_w = pl.im2col ? 1 : g->stride_w;
    p.dil_h = pl.im2col ? 1 : g->dilation_h;
    p.dil_w = pl.im2col ? 1 : g->dilation_w;
    p.kw = pl.im2col ? 1 : g->kw;
    p.taps = pl.taps;
    p.cblocks = pl.cblocks;
    p.cout = g->cout;
    p.coutp = pl.coutp;
    fill_epilogue(p, ep, int64_t(g->n) * g->cout * pl.ho * pl.wo, out_f32, out_i8, out_acc);
    p.o_c = g->cout;
    p.o_h = pl.ho;
    p.o_w = pl.wo;
    if (pl.use_ws)
        return tsx::ws_launch(pl.wsg, pl.wsp, p.xs, p.wp, static_cast<const tsx::EpiParams &>(p), stream);
    return launch_igemm<false>(p, stream);
}

int run_conv(const tsx_conv2d_geom *g, const void *x, bool x_is_f32, const float *x_scales, int n_x_scales,
             const void *packed_w, float padding_value, const tsx_epilogue *ep, float *out_f32, int8_t *out_i8,
             int32_t *out_acc, void *workspace, size_t workspace_bytes, void *stream_) {
    Plan pl;
    int rc = make_plan(g, &pl);
    if (rc) return rc;
    // validate the second half before launching the first
    rc = check_epilogue(ep, out_f32, out_i8, out_acc, g->n, g->cout, pl.ho, pl.wo);
    if (rc) return rc;
    TSX_REQUIRE(packed_w, "conv2d_i8: null packed weights");
    hipStream_t stream = tsx::as_stream(stream_);
    rc = run_stage(g, pl, x, x_is_f32, x_scales, n_x_scales, padding_value, workspace, workspace_bytes, stream);
    if (rc) return rc;
    return run_staged(g, pl, workspace, packed_w, ep, out_f32, out_i8, out_acc, stream);
}

}  // namespace

extern "C" {

size_t tsx_conv2d_i8_packed_weight_bytes(const tsx_conv2d_geom *g) {
    Plan pl;
    return make_plan(g, &pl) ? 0 : pl.packed_bytes;
}

size_t tsx_conv2d_i8_workspace_bytes(const tsx_conv2d_geom *g) {
    Plan pl;
    return make_plan(g, &pl) ? 0 : pl.staged_bytes;
}

int tsx_conv2d_i8_plan_info(const tsx_conv2d_geom *g, char *text, size_t text_bytes) {
    Plan pl;
    int rc = make_plan(g, &pl);
    if (rc) return rc;
    TSX_REQUIRE(text && text_bytes > 0, "plan_info: no text buffer");
    const char *base = !pl.use_ws ? "igemm" : pl.wsp.flat ? "flat_tile" : "window_stationary";
    const bool rs = pl.use_ws && pl.wsp.rs;
    if (rs)
        std::snprintf(text, text_bytes, "kernel=%s fp32_kernel=weight_stationary fragments_per_tile=%d tiles=%d ring_rows=%d lds_bytes=%d",
                      base, pl.wsp.rs_frags, pl.wsp.rs_ptiles * ((g->cout + 63) / 64), pl.wsp.rs_nr, pl.wsp.rs_lds);
    else if (pl.use_ws && pl.wsp.flat)
        std::snprintf(text, text_bytes, "kernel=%s fp32_kernel=%s fragments_per_tile=%d tiles=%lld resident=%d", base, base,
                      pl.wsp.fl_nta + pl.wsp.fl_ntb, (long long)(pl.wsp.fl_tiles * (pl.wsp.coutp / 128)), int(pl.wsp.fl_resident));
    else if (pl.use_ws)
        std::snprintf(text, text_bytes, "kernel=%s fp32_kernel=%s fragments_per_wavefront=%d wavefronts_along_cout=%d tiles=%lld blocks_per_window=%d",
                      base, base, pl.wsp.nt, pl.wsp.wm, (long long)(pl.wsp.tiles * ((g->cout + 32 * pl.wsp.wm - 1) / (32 * pl.wsp.wm))), pl.wsp.cbs);
    else
        std::snprintf(text, text_bytes, "kernel=%s fp32_kernel=%s", base, base);
    return 0;
}

int tsx_conv2d_i8_pack_weights(const tsx_conv2d_geom *g, const int8_t *w_oihw_dev, void *packed_dev, void *stream) {
    Plan pl;
    int rc = make_plan(g, &pl);
    if (rc) return rc;
    TSX_REQUIRE(w_oihw_dev && packed_dev, "pack_weights: null pointer");
    TSX_REQUIRE(reinterpret_cast<uintptr_t>(packed_dev) % 16 == 0, "pack_weights: packed buffer must be 16-byte aligned");
    // im2col plans see OIHW weights as [cout][C*KH*KW][1][1]: the same bytes, K in the reference's im2col order
    const int c_eff = pl.im2col ? pl.kk : g->c;
    if (pl.use_ws)
        return tsx::ws_pack_weights(pl.wsg, pl.wsp, w_oihw_dev, c_eff, static_cast<int8_t *>(packed_dev),
                                    tsx::as_stream(stream));
    const int64_t threads = int64_t(pl.packed_bytes / 16);
    hipLaunchKernelGGL(pack_weights_kernel, dim3(unsigned(tsx::ceil_div(threads, 256))), dim3(256), 0,
                       tsx::as_stream(stream), w_oihw_dev, g->cout, c_eff, pl.taps, int64_t(c_eff) * pl.taps,
                       int64_t(pl.taps), int64_t(1), pl.coutp, pl.cblocks, static_cast<int8_t *>(packed_dev));
    TSX_LAUNCH_CHECK("pack_weights_kernel");
    return 0;
}

int tsx_conv2d_i8_nchw(const tsx_conv2d_geom *g, const int8_t *x_dev, const void *packed_w_dev, float padding_value,
                       const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev, int32_t *out_acc_dev,
                       void *workspace_dev, size_t workspace_bytes, void *stream) {
    return run_conv(g, x_dev, false, nullptr, 0, packed_w_dev, padding_value, ep, out_f32_dev, out_i8_dev, out_acc_dev,
                    workspace_dev, workspace_bytes, stream);
}

int tsx_quantize_conv2d_i8_nchw(const tsx_conv2d_geom *g, const float *x_f32_dev, const float *x_scales_dev,
                                int32_t n_x_scales, const void *packed_w_dev, float padding_value,
                                const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev, int32_t *out_acc_dev,
                                void *workspace_dev, size_t workspace_bytes, void *stream) {
    return run_conv(g, x_f32_dev, true, x_scales_dev, n_x_scales, packed_w_dev, padding_value, ep, out_f32_dev,
                    out_i8_dev, out_acc_dev, workspace_dev, workspace_bytes, stream);
}

// ---- the allocation-free variant: the staging workspace is a file-scope device array
//
// Every device the library runs on holds its own copy of `scratch` at its own address until the process
// ends.  In host code the array's name is only a handle for hipGetSymbolAddress: the address kernels and
// copies may use is looked up once per device, with that device current, and kept in scratch_ptr[].
static __device__ __align__(256) unsigned char scratch[TSX_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
void *scratch_ptr[MAX_DEVICES] = {nullptr};

// Device address of `scratch` on the current device (looked up on the first call per device).
int scratch_on_current_device(void **out) {
    int dev = -1;
    TSX_HIP(hipGetDevice(&dev));
    TSX_REQUIRE(dev >= 0 && dev < MAX_DEVICES, "noalloc: device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void *ptr = nullptr;
        TSX_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        TSX_REQUIRE(ptr && reinterpret_cast<uintptr_t>(ptr) % 256 == 0, "noalloc: bad scratch address");
        scratch_ptr[dev] = ptr;
    }
    *out = scratch_ptr[dev];
    return 0;
}
}  // namespace

size_t tsx_noalloc_scratch_bytes(void) { return TSX_NOALLOC_SCRATCH_BYTES; }

int tsx_quantize_conv2d_i8_nchw_noalloc(const tsx_conv2d_geom *g, const float *x_f32_dev, const float *x_scales_dev,
                                        int32_t n_x_scales, const void *packed_w_dev, float padding_value,
                                        const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev,
                                        int32_t *out_acc_dev, void *stream) {
    Plan pl;
    int rc = make_plan(g, &pl);
    if (rc) return rc;
    if (pl.staged_bytes > size_t(TSX_NOALLOC_SCRATCH_BYTES))
        return tsx::fail(TSX_E_WORKSPACE,
                         "quantize_conv2d_i8_noalloc: this layer stages %zu bytes, the built-in scratch holds %zu; "
                         "use tsx_quantize_conv2d_i8_nchw with a caller workspace",
                         pl.staged_bytes, size_t(TSX_NOALLOC_SCRATCH_BYTES));
    void *ws = nullptr;
    rc = scratch_on_current_device(&ws);
    if (rc) return rc;
    // The staging kernel writes every byte of the staged extent the MFMA kernel reads (halo and channel
    // padding included), so nothing of the previous call's contents has to be cleared.
    return run_conv(g, x_f32_dev, true, x_scales_dev, n_x_scales, packed_w_dev, padding_value, ep, out_f32_dev,
                    out_i8_dev, out_acc_dev, ws, size_t(TSX_NOALLOC_SCRATCH_BYTES), stream);
}

int tsx_conv2d_i8_stage(const tsx_conv2d_geom *g, const void *x_dev, int32_t x_is_f32, const float *x_scales_dev,
                        int32_t n_x_scales, float padding_value, void *staged_dev, size_t staged_bytes, void *stream) {
    Plan pl;
    int rc = make_plan(g, &pl);
    if (rc) return rc;
    return run_stage(g, pl, x_dev, x_is_f32 != 0, x_scales_dev, n_x_scales, padding_value, staged_dev, staged_bytes,
                     tsx::as_stream(stream));
}

int tsx_conv2d_i8_staged(const tsx_conv2d_geom *g, const void *staged_dev, const void *packed_w_dev,
                         const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev, int32_t *out_acc_dev,
                         void *stream) {
    Plan pl;
    int rc = make_plan(g, &pl);
    if (rc) return rc;
    return run_staged(g, pl, staged_dev, packed_w_dev, ep, out_f32_dev, out_i8_dev, out_acc_dev, tsx::as_stream(stream));
}

int tsx_conv2d_i8_staged_dims(const tsx_conv2d_geom *g, int32_t *hs, int32_t *ws, int32_t *cp) {
    Plan pl;
    int rc = make_plan(g, &pl);
    if (rc) return rc;
    TSX_REQUIRE(hs && ws && cp, "staged_dims: null output");
    TSX_REQUIRE(!pl.im2col, "staged_dims: this layer stages by im2col; a producer cannot write its input");
    *hs = pl.hs;
    *ws = pl.ws;
    *cp = pl.cp;
    return 0;
}

int tsx_conv2d_i8_stage_fill(const tsx_conv2d_geom *g, float padding_value, void *staged_dev, size_t staged_bytes,
                             void *stream) {
    Plan pl;
    int rc = make_plan(g, &pl);
    if (rc) return rc;
    TSX_REQUIRE(!pl.im2col, "stage_fill: this layer stages by im2col; a producer cannot write its input");
    TSX_REQUIRE(staged_dev && reinterpret_cast<uintptr_t>(staged_dev) % 16 == 0, "stage_fill: buffer must be 16-byte aligned");
    TSX_REQUIRE(staged_bytes >= 16 && staged_bytes % size_t(pl.cp) == 0, "stage_fill: size is not a whole number of pixels");
    const int64_t chunks = int64_t(staged_bytes / 16);
    hipLaunchKernelGGL(stage_fill_kernel, dim3(unsigned(tsx::ceil_div(chunks, 256))), dim3(256), 0, tsx::as_stream(stream),
                       static_cast<int8_t *>(staged_dev), chunks, pl.cp, g->c, int(int8_t(padding_value)));
    TSX_LAUNCH_CHECK("stage_fill_kernel");
    return 0;
}

int tsx_conv2d_i8_stage_fill_halo(const tsx_conv2d_geom *g, float padding_value, void *staged_dev, size_t staged_bytes,
                                  void *stream) {
    Plan pl;
    int rc = make_plan(g, &pl);
    if (rc) return rc;
    TSX_REQUIRE(!pl.im2col, "stage_fill_halo: this layer stages by im2col; a producer cannot write its input");
    TSX_REQUIRE(staged_dev && reinterpret_cast<uintptr_t>(staged_dev) % 16 == 0, "stage_fill_halo: buffer must be 16-byte aligned");
    TSX_REQUIRE(staged_bytes == pl.staged_bytes, "stage_fill_halo: the buffer must be this layer's own staged input (%zu bytes, got %zu)",
                pl.staged_bytes, staged_bytes);
    // rows and columns of the map the convolution reads (its last rows / columns may lie behind the last window)
    const int h = std::min(g->h, pl.hs - g->pad_top), w = std::min(g->w, pl.ws - g->pad_left);
    if (pl.hs == h && pl.ws == w && g->c % 16 == 0 && pl.cp == g->c) return 0;   // no halo, no channel padding: nothing to write
    if (pl.cp == g->c) {
        const int64_t halo_chunks = int64_t(g->n) * (pl.hs * pl.ws - h * w) * (pl.cp / 16);
        hipLaunchKernelGGL(stage_fill_halo_only_kernel, dim3(unsigned(tsx::ceil_div(halo_chunks, 256))), dim3(256), 0,
                           tsx::as_stream(stream), static_cast<int8_t *>(staged_dev), halo_chunks, pl.hs, pl.ws, pl.cp, g->pad_top,
                           g->pad_left, h, w, int(int8_t(padding_value)));
        TSX_LAUNCH_CHECK("stage_fill_halo_only_kernel");
        return 0;
    }
    // channels [c rounded down to 16, cp) of interior pixels are written here; the producer's 16-channel stores cover the rest
    const int64_t chunks = int64_t(staged_bytes / 16);
    hipLaunchKernelGGL(stage_fill_halo_kernel, dim3(unsigned(tsx::ceil_div(chunks, 256))), dim3(256), 0, tsx::as_stream(stream),
                       static_cast<int8_t *>(staged_dev), chunks, pl.hs, pl.ws, pl.cp, g->c, g->pad_top, g->pad_left, h, w,
                       int(int8_t(padding_value)));
    TSX_LAUNCH_CHECK("stage_fill_halo_kernel");
    return 0;
}

int tsx_conv2d_i8_staged_at(const tsx_conv2d_geom *g, const void *staged_dev, int32_t staged_hs, int32_t staged_ws,
                            const void *packed_w_dev, const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev,
                            int32_t *out_acc_dev, void *stream) {
    Plan pl;
    int rc = make_plan(g, &pl);
    if (rc) return rc;
    TSX_REQUIRE(!pl.im2col || (staged_hs == pl.hs && staged_ws == pl.ws), "staged_at: im2col layers read their own buffer only");
    TSX_REQUIRE(staged_hs >= pl.hs && staged_ws >= pl.ws, "staged_at: buffer rows/columns %dx%d smaller than the %dx%d read",
                staged_hs, staged_ws, pl.hs, pl.ws);
    // same kernels, with the buffer's own pitches; the window-stationary plan is re-derived for them
    pl.hs = staged_hs;
    pl.ws = staged_ws;
    if (pl.use_ws) {
        pl.wsg.hs = staged_hs;
        pl.wsg.ws = staged_ws;
        const tsx::WsPlan wide = tsx::ws_plan(pl.wsg);
        if (wide.ok && wide.packed_bytes == pl.wsp.packed_bytes) {
            pl.wsp = wide;
        } else {
            // weights were packed for the window-stationary kernel: only that kernel can read them
            return tsx::fail(TSX_E_INVALID, "staged_at: a %dx%d staged buffer does not fit this layer's kernel", staged_hs,
                             staged_ws);
        }
    }
    return run_staged(g, pl, staged_dev, packed_w_dev, ep, out_f32_dev, out_i8_dev, out_acc_dev, tsx::as_stream(stream));
}

// ---- GEMM: a [m][k] is a batch of m "images" with k channels and 1x1 extent.

// K-steps of the packed GEMM weights: padded with zero steps to the window-stationary kernel's ring of 4
// (the tiled and the skinny kernel walk only the first round_up(k, 64) / 64 of them).
static int gemm_packed_ksteps(int32_t k) { return int(tsx::round_up(tsx::round_up(k, KSTEP) / KSTEP, 4)); }

size_t tsx_gemm_i8_packed_weight_bytes(int32_t k, int32_t n) {
    if (k <= 0 || n <= 0) return 0;
    return size_t(gemm_packed_ksteps(k)) * KSTEP * size_t(tsx::round_up(n, BM));
}

int tsx_gemm_i8_pack_weights(int32_t k, int32_t n, int32_t transposed, const int8_t *w_dev, void *packed_dev,
                             void *stream) {
    TSX_REQUIRE(k > 0 && n > 0 && w_dev && packed_dev, "gemm_i8_pack_weights: bad argument");
    TSX_REQUIRE(reinterpret_cast<uintptr_t>(packed_dev) % 16 == 0, "gemm_i8_pack_weights: packed buffer must be 16-byte aligned");
    const int cblocks = gemm_packed_ksteps(k), coutp = int(tsx::round_up(n, BM));
    const int64_t threads = int64_t(cblocks) * coutp * KSTEP / 16;
    // element (k, n): [k][n] row-major -> k*n_ + n ; transposed [n][k] -> n*k_ + k
    const int64_t ld_cout = transposed ? k : 1, ld_c = transposed ? 1 : n;
    hipLaunchKernelGGL(pack_weights_kernel, dim3(unsigned(tsx::ceil_div(threads, 256))), dim3(256), 0,
                       tsx::as_stream(stream), w_dev, n, k, 1, ld_cout, ld_c, int64_t(0), coutp, cblocks,
                       static_cast<int8_t *>(packed_dev));
    TSX_LAUNCH_CHECK("pack_weights_kernel");
    return 0;
}

size_t tsx_gemm_i8_workspace_bytes(int32_t m, int32_t k) {
    if (m <= 0 || k <= 0) return 0;
    return k % KSTEP == 0 ? 0 : size_t(m) * size_t(tsx::round_up(k, KSTEP));
}

int tsx_gemm_i8(int32_t m, int32_t n, int32_t k, const int8_t *a_dev, const void *packed_w_dev,
                const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev, int32_t *out_acc_dev,
                void *workspace_dev, size_t workspace_bytes, void *stream_) {
    TSX_REQUIRE(m > 0 && n > 0 && k > 0, "gemm_i8: non-positive extent");
    TSX_REQUIRE(a_dev && packed_w_dev, "gemm_i8: null input");
    int rc = check_epilogue(ep, out_f32_dev, out_i8_dev, out_acc_dev, m);
    if (rc) return rc;
    hipStream_t stream = tsx::as_stream(stream_);
    const int kp = int(tsx::round_up(k, KSTEP));
    const int8_t *xs = a_dev;
    if (kp != k || reinterpret_cast<uintptr_t>(a_dev) % 16 != 0) {
        const size_t need = size_t(m) * kp;
        if (!workspace_dev || workspace_bytes < need)
            return tsx::fail(TSX_E_WORKSPACE, "gemm_i8: workspace %zu < %zu bytes", workspace_bytes, need);
        TSX_REQUIRE(reinterpret_cast<uintptr_t>(workspace_dev) % 16 == 0, "gemm_i8: workspace must be 16-byte aligned");
        StageGeom sg{m, k, 1, 1, 1, 1, kp, 0, 0, 0};
        const int64_t threads = int64_t(m) * (kp / 16);
        hipLaunchKernelGGL(stage_nchw_kernel<false>, dim3(unsigned(tsx::ceil_div(threads, 256))), dim3(256), 0, stream,
                           static_cast<const void *>(a_dev), sg, static_cast<const float *>(nullptr), 1, int64_t(1),
                           int64_t(0), static_cast<int8_t *>(workspace_dev));
        TSX_LAUNCH_CHECK("stage_nchw_kernel");
        xs = static_cast<const int8_t *>(workspace_dev);
    }
    GemmParams p{};
    p.xs = xs;
    p.wp = static_cast<const int8_t *>(packed_w_dev);
    p.positions = m;
    p.howo = 1;
    p.wo = 1;
    p.hs = 1;
    p.ws = 1;
    p.cp = kp;
    p.stride_h = p.stride_w = p.dil_h = p.dil_w = p.kw = 1;
    p.taps = 1;
    p.cblocks = kp / KSTEP;
    p.cout = n;
    p.coutp = int(tsx::round_up(n, BM));
    fill_epilogue(p, ep, int64_t(m) * n, out_f32_dev, out_i8_dev, out_acc_dev);
    if (m <= 32) {
        hipLaunchKernelGGL(gemm_i8_skinny_kernel, dim3(unsigned(tsx::ceil_div(n, 32))), dim3(SK_WAVES * 64), 0, stream, p);
        TSX_LAUNCH_CHECK("gemm_i8_skinny_kernel");
        return 0;
    }
    // TSX_GEMM_I8_KSPLIT: "0" never, "force" every GEMM of more than 32 rows (tests); otherwise GEMMs with a K long
    // enough to split (2048 and more: the LDS form) whose 64 x 64 tiles run in one round (at most 256: that form holds
    // one workgroup per CU).  Measured against the window-stationary kernel: K = N = 4096 with 48 / 256 rows 10.9 /
    // 12.4 us against 14.1 / 23.0; K = N = 2048 with 64 / 256 / 512 rows 7.5 / 7.9 / 8.6 us against 8.0 / 9.5 / 10.3;
    // K = 4096, N = 1024 with 256 / 1024 rows 10.9 / 14.2 us against 14.2 / 15.4; K = 8192, N = 2048 with 512 rows
    // 20.7 us against 26.8.  Beyond one round it wins or loses by the shape (N = 4096, K = 4096, 512 rows: 23.6 us
    // against 24.0; N = 2048, K = 8192, 768 rows: 37.4 against 29.8), and with K = 1024 (the register form) it loses:
    // 7.9 us against 6.2 at 256 rows.  (Chunks of 8 K-steps kept four deep in flight through rotating register sets
    // measured slower by 0.9 us.)
    {
        const char *e = std::getenv("TSX_GEMM_I8_KSPLIT");
        const int64_t tiles = tsx::ceil_div(m, 64) * tsx::ceil_div(n, 64);
        const bool pays = tiles <= 256 && kp >= 2048;
        if (!(e && e[0] == '0') && ((e && e[0] == 'f') || pays)) {
            const dim3 grid(unsigned(tsx::ceil_div(n, 64)), unsigned(tsx::ceil_div(m, 64)));
            // activations through LDS where K gives the double buffer something to overlap ("forcereg": never)
            if (kp >= 2048 && !(e && e[0] == 'f' && e[5] == 'r')) {
                static std::atomic<bool> granted[64];
                int dev = 0;
                TSX_HIP(hipGetDevice(&dev));
                if (dev < 64 && !granted[dev].load()) {     // dynamic LDS beyond 64 KiB: granted per kernel and device
                    TSX_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_i8_ksplit_lds_kernel),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
                    granted[dev].store(true);
                }
                hipLaunchKernelGGL(gemm_i8_ksplit_lds_kernel, grid, dim3(KS_WAVES * 64), KL_LDS, stream, p);
                TSX_LAUNCH_CHECK("gemm_i8_ksplit_lds_kernel");
                return 0;
            }
            hipLaunchKernelGGL((gemm_i8_ksplit_kernel<2, 2, 4>), grid, dim3(KS_WAVES * 64), 0, stream, p);
            TSX_LAUNCH_CHECK("gemm_i8_ksplit_kernel");
            return 0;
        }
    }
    // Enough rows to fill MFMA fragments: the window-stationary kernel in its GEMM form (a 1x1 layer over m
    // one-pixel rows, row-major output).  Residual terms stay on the tiled kernel.
    if (!p.residual && !p.st_out && p.act != TSX_ACT_MISH) {   // (... and so does the exact Mish)
        const tsx::WsGeom wg{1, n, m, 1, m, 1, kp, kp / KSTEP, 1, 1, 1, 1, 1, 1, 1};
        const tsx::WsPlan wpl = tsx::ws_plan(wg);
        if (wpl.ok && wpl.ksteps_p == gemm_packed_ksteps(k) && wpl.coutp == p.coutp)
            return tsx::ws_launch(wg, wpl, p.xs, p.wp, static_cast<const tsx::EpiParams &>(p), stream);
    }
    return launch_igemm<true>(p, stream);
}

}  // extern "C"
