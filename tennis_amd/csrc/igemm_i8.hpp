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
};

// Epilogue of one accumulator; idx is the linear index in the output tensor.
__device__ __forceinline__ void emit(const EpiParams &p, int acc, int64_t idx, float dq, float bias, float row_scale) {
    if (p.out_acc) p.out_acc[idx] = acc;
    if (!p.out_f32 && !p.out_i8) return;
    float v = __fmul_rn(float(acc), dq);
    if (p.row_scale) v = __fmul_rn(v, row_scale);
    if (p.bias) v = __fadd_rn(v, bias);
    if (p.residual) v = __fadd_rn(v, p.residual[idx]);
    v = apply_act(v, p.act, p.slope, idx < p.act_body);
    if (p.out_f32) p.out_f32[idx] = v;
    if (p.out_i8) {
        const float s = p.n_qscales == 1 ? p.q_scales[0] : p.q_scales[idx / p.q_group_len];
        p.out_i8[idx] = int8_t(quantize_value(__fmul_rn(v, s), p.n_qscales == 1 && idx < p.q_bulk8));
    }
}

// ---- window-stationary stride-1 convolution kernel (conv2d_i8_ws.hip) ----

struct WsPlan {
    bool ok;            // geometry supported
    int th, nt;         // output rows per tile, 32-position fragments per tile
    int tiles_per_image;
    int wr, wc, wp;     // window rows, cols, pixels
    int ksteps_p;       // K-steps padded to the A-ring size
    int coutp;          // cout padded to the workgroup's 256
    size_t packed_bytes;
};

struct WsGeom {
    int n, cout, ho, wo, hs, ws, cp, cblocks, kh, kw, dil_h, dil_w;
};

WsPlan ws_plan(const WsGeom &g);
int ws_pack_weights(const WsGeom &g, const WsPlan &pl, const int8_t *w_oihw, int c, int8_t *packed, hipStream_t stream);
int ws_launch(const WsGeom &g, const WsPlan &pl, const int8_t *xs, const int8_t *packed, const EpiParams &ep,
              hipStream_t stream);

}  // namespace tsx
