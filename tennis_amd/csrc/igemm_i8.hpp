// Shared device-side pieces of the int8 MFMA kernels: epilogue parameters and the
// per-accumulator epilogue (dequant -> row scale -> bias -> residual -> activation -> requantize).
#pragma once
#include "tsx_common.hpp"

namespace tsx {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct EpiParams {
    const float *dq, *row_scale, *bias, *q_scales;
    const float *residual;
    int act;
    float slope;
    int n_qscales;
    int64_t q_group_len, q_bulk8, act_body;
    float *out_f32;
    int8_t *out_i8;
    int32_t *out_acc;
    // int8 output in the consumer's staged layout [n][st_hs][st_ws][st_cp] (convolutions only)
    int8_t *st_out;
    int st_hs, st_ws, st_cp, st_pt, st_pl;
    int st_up;           // 2: every output pixel is written to the 2 x 2 staged pixels of a nearest-neighbour resize by 2
    int o_c, o_h, o_w;   // NCHW extents of the output, to decode a linear index
    int res_after;       // residual joins behind the activation instead of in front of it
};

// Division of a non-negative n by a uniform divisor d as one multiply-high: magic = ceil(2^32 / d) gives
// floor(n / d) = mulhi(n, magic) whenever n * d <= 2^32.  0 = no magic number (d = 1, or n_max too large): the
// kernel then divides.
inline unsigned div_magic(int d, int64_t n_max) {
    if (d <= 1 || n_max * d > (int64_t(1) << 32)) return 0u;
    return unsigned(((uint64_t(1) << 32) + unsigned(d) - 1) / unsigned(d));
}
#ifdef __HIPCC__
__device__ __forceinline__ int udiv(int n, int d, unsigned magic) { return magic ? int(__umulhi(unsigned(n), magic)) : n / d; }
#endif

// fp32 value of one accumulator after dequant -> row scale -> bias -> residual -> activation;
// idx is the linear index in the output tensor.
// MISHX: whether the exact Mish is compiled in.  Its double-precision chain costs a kernel some thirty registers at
// the point of the epilogue; the convolution kernels carry it in instantiations of their own, which layers with
// TSX_ACT_MISH are routed to, and every other layer runs code that never saw it.
template <bool MISHX = true>
__device__ __forceinline__ float epi_value(const EpiParams &p, int acc, int64_t idx, float dq, float bias, float row_scale) {
    float v = __fmul_rn(float(acc), dq);
    if (p.row_scale) v = __fmul_rn(v, row_scale);
    if (p.bias) v = __fadd_rn(v, bias);
    if (p.residual && !p.res_after) v = __fadd_rn(v, p.residual[idx]);
    v = MISHX ? apply_act_conv_i8(v, p.act, p.slope, idx < p.act_body) : apply_act_without_exact_mish(v, p.act, p.slope, idx < p.act_body);
    if (p.residual && p.res_after) v = __fadd_rn(v, p.residual[idx]);
    return v;
}

// Epilogue of one accumulator: every requested output of element idx.
template <bool MISHX = true>
__device__ __forceinline__ void emit(const EpiParams &p, int acc, int64_t idx, float dq, float bias, float row_scale) {
    if (p.out_acc) p.out_acc[idx] = acc;
    if (!p.out_f32 && !p.out_i8 && !p.st_out) return;
    const float v = epi_value<MISHX>(p, acc, idx, dq, bias, row_scale);
    if (p.out_f32) p.out_f32[idx] = v;
    if (p.out_i8 || p.st_out) {
        const float s = p.n_qscales == 1 ? p.q_scales[0] : p.q_scales[idx / p.q_group_len];
        const int8_t q = int8_t(quantize_value(__fmul_rn(v, s), p.n_qscales == 1 && idx < p.q_bulk8));
        if (p.out_i8) p.out_i8[idx] = q;
        if (p.st_out) {
            const int ow = int(idx % p.o_w);
            const int64_t t1 = idx / p.o_w;
            const int oh = int(t1 % p.o_h);
            const int64_t t2 = t1 / p.o_h;
            const int co = int(t2 % p.o_c);
            const int64_t n = t2 / p.o_c;
            if (p.st_up == 2) {
                int8_t *d = p.st_out + ((n * p.st_hs + 2 * oh + p.st_pt) * p.st_ws + 2 * ow + p.st_pl) * p.st_cp + co;
                d[0] = q;
                d[p.st_cp] = q;
                d[int64_t(p.st_ws) * p.st_cp] = q;
                d[int64_t(p.st_ws + 1) * p.st_cp] = q;
            } else {
                p.st_out[((n * p.st_hs + oh + p.st_pt) * p.st_ws + ow + p.st_pl) * p.st_cp + co] = q;
            }
        }
    }
}

// Epilogue of one 32x32 accumulator fragment for one lane, rows = output channels: accumulator r is
// channel row 8*(r/4) + (r%4) relative to the lane's first row, at linear index idx0 + row * row_stride.
// One pass per epilogue term behind a single uniform branch each (testing the uniform options per
// element costs more instructions than the arithmetic).  Caller guarantees: no raw-accumulator
// output, every element in the activation's SIMD-body range, one quantize scale for this lane's
// image (q_scale, rounding half to even iff q_even).  st_dst = the lane's pixel in the consumer's
// staged layout at its first channel row, or null.
template <bool MISHX = true>
__device__ __forceinline__ void epilogue_rows16(const EpiParams &p, const v16i &acc, const float (&dq)[16],
                                                const float (&bias)[16], int64_t idx0, int64_t row_stride, float q_scale,
                                                bool q_even, int8_t *st_dst) {
    float v[16];
    static_for<0, 16>([&](auto rc) { constexpr int r = decltype(rc)::value; v[r] = __fmul_rn(float(acc[r]), dq[r]); });
    if (p.bias) {
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = __fadd_rn(v[r], bias[r]);
    }
    float res[16];
    if (p.residual) {
#pragma unroll
        for (int r = 0; r < 16; ++r) res[r] = p.residual[idx0 + int64_t(8 * (r / 4) + (r % 4)) * row_stride];
    }
    if (p.residual && !p.res_after) {
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = __fadd_rn(v[r], res[r]);
    }
    if (p.act == TSX_ACT_RELU) {
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = v[r] > 0.f ? v[r] : 0.f;
    } else if (p.act == TSX_ACT_LEAKY_RELU) {
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = apply_act_conv_i8(v[r], TSX_ACT_LEAKY_RELU, p.slope, true);
    } else if (MISHX && p.act == TSX_ACT_MISH) {
        // nothing but the requantized values leaves: the exact form only where it decides a rounding
        if (!p.out_f32 && (p.out_i8 || st_dst)) mish_fragment_for_rounding(v, res, p.residual && p.res_after, q_scale);
        else mish_fragment(v);
    } else if (p.act == TSX_ACT_MISH_FAST) {
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = apply_act_conv_i8(v[r], TSX_ACT_MISH_FAST, 0.f, true);
    }
    if (p.residual && p.res_after) {
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = __fadd_rn(v[r], res[r]);
    }
    if (p.out_f32) {
#pragma unroll
        for (int r = 0; r < 16; ++r) p.out_f32[idx0 + int64_t(8 * (r / 4) + (r % 4)) * row_stride] = v[r];
    }
    if (p.out_i8 || st_dst) {
        int qv[16];
        if (q_even) {
#pragma unroll
            for (int r = 0; r < 16; ++r) qv[r] = quantize_value(__fmul_rn(v[r], q_scale), true);
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) qv[r] = quantize_value(__fmul_rn(v[r], q_scale), false);
        }
        if (p.out_i8) {
#pragma unroll
            for (int r = 0; r < 16; ++r) p.out_i8[idx0 + int64_t(8 * (r / 4) + (r % 4)) * row_stride] = int8_t(qv[r]);
        }
        if (st_dst) {
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const uint32_t w = uint32_t(qv[4 * g4] & 0xff) | (uint32_t(qv[4 * g4 + 1] & 0xff) << 8) |
                                   (uint32_t(qv[4 * g4 + 2] & 0xff) << 16) | (uint32_t(qv[4 * g4 + 3] & 0xff) << 24);
                *reinterpret_cast<uint32_t *>(st_dst + 8 * g4) = w;
                if (p.st_up == 2) {   // st_dst is staged pixel (2 oh, 2 ow): the other three of the 2 x 2 block
                    *reinterpret_cast<uint32_t *>(st_dst + p.st_cp + 8 * g4) = w;
                    *reinterpret_cast<uint32_t *>(st_dst + int64_t(p.st_ws) * p.st_cp + 8 * g4) = w;
                    *reinterpret_cast<uint32_t *>(st_dst + int64_t(p.st_ws + 1) * p.st_cp + 8 * g4) = w;
                }
            }
        }
    }
}

// ---- window-stationary convolution kernel (conv2d_i8_ws.hip) ----

struct WsPlan {
    bool ok;            // geometry supported
    int th, nt;         // output rows per tile, 32-position fragments per wavefront
    int tw, ctiles;     // output columns per tile, column tiles per row
    int cbs;            // channel blocks per window (1x1 layers: up to 4)
    int wm;             // wavefronts along cout: 4, 2 or 1, with the tile's positions split over the other factor of 4
    int ho, wo, hs, ws; // the map as the kernel walks it: the real one, or rows of one pixel for 1x1 layers without halo
    int64_t tiles;      // tiles over the batch-wide row sequence
    int wr, wc, wp;     // window rows, cols, pixels
    int ksteps_p;       // K-steps padded to the A-ring size
    int coutp;          // cout padded to the workgroup's channels (32 x wm)
    size_t packed_bytes;
    // flat-tile kernel (conv2d_i8_fl.hip) instead: a tile is fl_nta + fl_ntb consecutive fragments of the
    // batch-wide flat position list; same packed weights
    bool flat, fl_resident;
    int fl_nta, fl_ntb, fl_wr, fl_wc, fl_wp, fl_rowp;
    int64_t fl_tiles;
    // weight-stationary kernel (conv2d_i8_rs.hip) for the epilogues it writes: a tile is rs_frags consecutive
    // fragments x 64 output channels; same packed weights
    bool rs;
    int rs_frags, rs_ptiles, rs_nr, rs_rowp, rs_wc, rs_lds;
};

struct WsGeom {
    int n, cout, ho, wo, hs, ws, cp, cblocks, kh, kw, dil_h, dil_w, sh, sw;
    // GEMM form: n = 1 image of ho = m one-pixel rows with k channels; the output is [m][cout] row-major, the
    // epilogue's row_scale applies, and the weights are packed with rows padded to 128 and K-steps to 4
    int gemm;
};

WsPlan ws_plan(const WsGeom &g);
int ws_pack_weights(const WsGeom &g, const WsPlan &pl, const int8_t *w_oihw, int c, int8_t *packed, hipStream_t stream);
int ws_launch(const WsGeom &g, const WsPlan &pl, const int8_t *xs, const int8_t *packed, const EpiParams &ep,
              hipStream_t stream);
// flat-tile kernel: fills the fl_* fields of a valid plan when the layer suits it; launch
void fl_plan(const WsGeom &g, WsPlan *pl);
int fl_launch(const WsGeom &g, const WsPlan &pl, const int8_t *xs, const int8_t *packed, const EpiParams &ep,
              hipStream_t stream);
// weight-stationary kernel: fills the rs_* fields of a valid plan when the layer suits it; whether it writes a
// given epilogue; launch
void rs_plan(const WsGeom &g, WsPlan *pl);
bool rs_takes(const WsPlan &pl, const EpiParams &ep, int64_t count);
int rs_launch(const WsGeom &g, const WsPlan &pl, const int8_t *xs, const int8_t *packed, const EpiParams &ep,
              hipStream_t stream);

}  // namespace tsx
