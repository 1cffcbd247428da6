/*
 * tsx_hip.h -- the C ABI of the MI355X (gfx950) convolution hot path for TenniS.
 *
 * This is the drop-in boundary: plain pointers and sizes, no C++ or torch types.
 * The "hip" device operator classes (tennis_amd/backend) call these launchers from
 * the core methods TenniS declares per device; each entry point cites the reference
 * interface it stands in for (paths relative to the TenniS tree).
 *
 * Conventions
 *   - every pointer named *_dev is device memory on the current HIP device; the
 *     library never owns, allocates or frees caller memory;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); all
 *     launches are asynchronous on it, nothing synchronises;
 *   - return value 0 = success; > 0 = a hipError_t from the runtime; < 0 = a
 *     TSX_E_* argument/shape error.  tsx_last_error() gives the message (thread-local);
 *   - tensors are NCHW, dense, row-major, exactly as the reference's operators see them.
 */
#ifndef TSX_HIP_H
#define TSX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TSX_E_INVALID   (-1)  /* bad argument / unsupported shape */
#define TSX_E_WORKSPACE (-2)  /* workspace too small */
#define TSX_E_NODEVICE  (-3)  /* no usable gfx950 device */

const char *tsx_last_error(void);
/* Library/ABI version (major*100 + minor). */
int tsx_version(void);
/* Number of compute units of the current device (for launch heuristics and roofline peaks). */
int tsx_device_cu_count(void);

/* Geometry of one 2-D convolution, as base::Conv2D / base::Conv2DQuantized hand it to
 * their core: x [n,c,h,w], w [cout,c,kh,kw], Padding2D{top,bottom,left,right},
 * Stride2D, Dilation2D (include/backend/common_structure.h:10-62).  Output size follows
 * conv2d_forward (include/backend/common_function.h:30-40). */
typedef struct tsx_conv2d_geom {
    int32_t n, c, h, w;
    int32_t cout, kh, kw;
    int32_t pad_top, pad_bottom, pad_left, pad_right;
    int32_t stride_h, stride_w;
    int32_t dilation_h, dilation_w;
} tsx_conv2d_geom;

int tsx_conv2d_out_size(const tsx_conv2d_geom *g, int32_t *out_h, int32_t *out_w);

/* Activation kinds of the fused epilogue. */
#define TSX_ACT_NONE       0
#define TSX_ACT_RELU       1  /* cpu::ReLU      src/kernels/cpu/relu.cpp:30-52 */
#define TSX_ACT_LEAKY_RELU 2  /* cpu::LeakyReLU src/kernels/cpu/leaky_relu.cpp:41-66 */
#define TSX_ACT_MISH       3  /* x * tanh(softplus(x)) as the operators softplus, tanh, mul compose it
                                 (src/kernels/cpu/softplus.cpp:30-39, tanh.cpp:14-23, mul.cpp): the host's chain of
                                 rounded intermediates, its expf restated operation for operation -- bit for bit
                                 the host's values */
#define TSX_ACT_MISH_FAST  4  /* the same function from one hardware exponential and one reciprocal: 1e-7 relative,
                                 a sixth of the arithmetic; for layers bound by the activation.  Opt-in: a
                                 requantized int8 value differs from TSX_ACT_MISH's in about one of a million */

/* Fused epilogue applied to the int32 accumulators.  It reproduces, rounding for
 * rounding, the reference's chain of separate operators on the fp32 tensor:
 *   y = float(acc) * dq[channel]            conv2d_quantized_core.cpp:81-106
 *   y = y * row_scale[row]    if row_scale  (GEMM only: per-row activation dequant)
 *   y = y + bias[channel]     if bias       add_bias.cpp:47-85
 *   y = y + residual[i]       if residual   add.cpp on equal shapes (a residual join: the
 *                                           other branch of the block, same shape as the output)
 *   y = act(y)                              relu.cpp / leaky_relu.cpp (incl. their SIMD-body /
 *                                           scalar-tail difference in signed zero and NaN)
 *   (residual_after_act != 0 swaps the last two: y = act(y) + residual[i], a shortcut that joins
 *   behind the activation, as in darknet-style residual units)
 *   q = quantize(y)           if out_i8     quantize.cpp:70-125 with q_scales[n_qscales]
 * All pointers are device pointers; unused ones are NULL. */
typedef struct tsx_epilogue {
    const float *dq_dev;        /* [channels] dequantize_scales */
    const float *row_scale_dev; /* [rows] or NULL */
    const float *bias_dev;      /* [channels] or NULL */
    int32_t act;                /* TSX_ACT_* */
    float slope;                /* leaky_relu scale */
    const float *q_scales_dev;  /* [n_qscales] quantize_scale of the consumer, or NULL */
    int32_t n_qscales;          /* must equal n (or rows) when q_scales_dev != NULL, as
                                   base_quantize.cpp:26 requires of the consumer */
    const float *residual_dev;  /* fp32 tensor of the output's shape added before the activation, or NULL */
    /* Convolutions only: write the requantized int8 output straight into the staged (channel-blocked,
     * padded) input of the convolution that consumes it, [n][staged_hs][staged_ws][staged_cp] with output
     * pixel (oh, ow) at (oh + staged_pad_top, ow + staged_pad_left), instead of NCHW -- the consumer then
     * runs tsx_conv2d_i8_staged_at without a staging pass.  Needs q_scales_dev; the buffer's halo and
     * channel padding are written once by tsx_conv2d_i8_stage_fill.  staged_cp is a multiple of 32 (a
     * consumer's own channel pitch is a multiple of 64; 32 describes a consumer that reads pairs of columns of
     * a 32-channel tensor as one 64-channel pixel: staged_ws and staged_pad_left then count columns, not
     * pairs).  NULL = not used. */
    int8_t *staged_out_dev;
    int32_t staged_hs, staged_ws, staged_cp, staged_pad_top, staged_pad_left;
    int32_t residual_after_act; /* 0: act(y + residual); 1: act(y) + residual */
    /* 0 or 1: output pixel (oh, ow) goes to staged pixel (oh, ow) as described above.  2: a nearest-neighbour
     * resize by 2 (cpu::Resize2D NEAREST at an integer factor, src/kernels/cpu/resize2d.cpp:186-215) is folded in:
     * the pixel is written to the four staged pixels (2 oh + dy, 2 ow + dx), so that a convolution -> upsample ->
     * (concatenation ->) convolution chain needs no fp32 tensor in between. */
    int32_t staged_upsample;
} tsx_epilogue;

/* ---------------------------------------------------------------- quantize
 * cpu::Quantize::quantize (src/kernels/cpu/quantize.cpp:70-125; declared
 * include/backend/base/base_quantize.h:24):  q = clamp(round(x * scale_g), -128, 127).
 * n_scales == 1: first 8*floor(count/8) elements round half to even, the rest half away
 * from zero; n_scales > 1: scale g covers the next ceil(count/n_scales) elements, all half
 * away.  NaN / out-of-int32-range products give -128 (x86 conversion semantics). */
int tsx_quantize_f32_i8(const float *x_dev, int64_t count, const float *scales_dev, int32_t n_scales,
                        int8_t *out_dev, void *stream);

/* ---------------------------------------------------------------- int8 conv2d
 * cpu::Conv2DQuantizedCore::conv2d (src/kernels/cpu/quantized/conv2d_quantized_core.cpp:128-147,
 * interface include/backend/base/base_conv2d_quantized_core.h:14-16): im2col<int8> + int8 GEMM
 * with int32 accumulation + dequant, done here as one implicit-GEMM on the i8 MFMA units.
 *
 * Weights are repacked once (operator init) from OIHW int8 into MFMA operand tiles. */
size_t tsx_conv2d_i8_packed_weight_bytes(const tsx_conv2d_geom *g);
int tsx_conv2d_i8_pack_weights(const tsx_conv2d_geom *g, const int8_t *w_oihw_dev, void *packed_dev, void *stream);
/* Scratch the conv needs (channel-blocked padded copy of the activations). */
size_t tsx_conv2d_i8_workspace_bytes(const tsx_conv2d_geom *g);
/* Which kernel the plan of this layer launches, as text ("kernel=flat_tile fp32_kernel=weight_stationary ..."):
 * kernel = igemm | window_stationary | flat_tile, and fp32_kernel = the kernel that takes the layer when the
 * epilogue is fp32 output with dequantize scales, bias and activation only.  No counterpart in the reference; for
 * tests that must know a given kernel ran, and for logs.  The environment variables TSX_CONV_I8_FLAT and
 * TSX_CONV_I8_RS ("0" = never, "force" = wherever the geometry allows) are read at every call that plans. */
int tsx_conv2d_i8_plan_info(const tsx_conv2d_geom *g, char *text, size_t text_bytes);
/* padding_value is the reference's float parameter; it is cast to int8 as the reference
 * does (conv2d_quantized_core.cpp:72).  Any of out_f32_dev / out_i8_dev / out_acc_dev may be
 * NULL; out_acc_dev receives the raw int32 accumulators (the reference's INT32 scratch). */
int tsx_conv2d_i8_nchw(const tsx_conv2d_geom *g, const int8_t *x_dev, const void *packed_w_dev,
                       float padding_value, const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev,
                       int32_t *out_acc_dev, void *workspace_dev, size_t workspace_bytes, void *stream);
/* Same, but takes the fp32 activations and the consumer-side quantize parameters, fusing
 * base::Quantize (a1) into the layout pass that precedes the MFMA kernel. */
int tsx_quantize_conv2d_i8_nchw(const tsx_conv2d_geom *g, const float *x_f32_dev, const float *x_scales_dev,
                                int32_t n_x_scales, const void *packed_w_dev, float padding_value,
                                const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev,
                                int32_t *out_acc_dev, void *workspace_dev, size_t workspace_bytes, void *stream);

/* tsx_quantize_conv2d_i8_nchw for callers that cannot allocate device memory or pass a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments, kernels and results as tsx_quantize_conv2d_i8_nchw, minus the workspace: the staged copy of
 * the activations lives in a device array built into the library, TSX_NOALLOC_SCRATCH_BYTES per GPU (held until
 * the process ends).  A layer whose tsx_conv2d_i8_workspace_bytes() exceeds that is rejected with
 * TSX_E_WORKSPACE.  The call allocates and frees nothing; its first call on a device looks the array's address
 * up once.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two
 * threads) race -- serialise them. */
#define TSX_NOALLOC_SCRATCH_BYTES (8u << 20)
size_t tsx_noalloc_scratch_bytes(void);
int tsx_quantize_conv2d_i8_nchw_noalloc(const tsx_conv2d_geom *g, const float *x_f32_dev, const float *x_scales_dev,
                                        int32_t n_x_scales, const void *packed_w_dev, float padding_value,
                                        const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev,
                                        int32_t *out_acc_dev, void *stream);

/* The two halves of the calls above, for callers that keep the staged activations around
 * (several convolutions reading one tensor, or timing the MFMA kernel by itself):
 *   stage  : NCHW int8 (x_is_f32 == 0) or NCHW fp32 + quantize (x_is_f32 != 0) -> channel-blocked
 *            padded copy [n][hs][ws][round_up(c,64)], tsx_conv2d_i8_workspace_bytes() bytes;
 *   staged : the implicit GEMM + epilogue on that copy. */
int tsx_conv2d_i8_stage(const tsx_conv2d_geom *g, const void *x_dev, int32_t x_is_f32, const float *x_scales_dev,
                        int32_t n_x_scales, float padding_value, void *staged_dev, size_t staged_bytes, void *stream);
int tsx_conv2d_i8_staged(const tsx_conv2d_geom *g, const void *staged_dev, const void *packed_w_dev,
                         const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev, int32_t *out_acc_dev,
                         void *stream);

/* Chaining quantized convolutions without staging passes (no counterpart in the reference, whose operators
 * exchange NCHW tensors; values are those of quantize(relu(add_bias(conv))) either way):
 *   staged_dims : extents [hs][ws][cp] of the staged input the convolution `g` reads (bytes = n*hs*ws*cp);
 *   stage_fill  : writes the halo value T(padding_value) to every real channel and 0 to the channel padding
 *                 of a whole staged buffer -- once per buffer; producers only overwrite the interior;
 *   staged_at   : tsx_conv2d_i8_staged on a staged buffer whose row/column extents are larger than the
 *                 convolution needs (a buffer shared with another consumer of the same tensor, e.g. a
 *                 stride-2 1x1 projection reading the staged input of a stride-1 1x1 convolution). */
int tsx_conv2d_i8_staged_dims(const tsx_conv2d_geom *g, int32_t *hs, int32_t *ws, int32_t *cp);
int tsx_conv2d_i8_stage_fill(const tsx_conv2d_geom *g, float padding_value, void *staged_dev, size_t staged_bytes,
                             void *stream);
/*   stage_fill_halo : the same for a buffer of exactly tsx_conv2d_i8_workspace_bytes(g) bytes whose interior a
 *                 producer's epilogue is about to write: only the halo pixels and the channel padding are
 *                 written (nothing at all for a layer without either) -- for callers whose staged buffer is fresh
 *                 memory on every run, such as an operator output. */
int tsx_conv2d_i8_stage_fill_halo(const tsx_conv2d_geom *g, float padding_value, void *staged_dev, size_t staged_bytes,
                                  void *stream);
int tsx_conv2d_i8_staged_at(const tsx_conv2d_geom *g, const void *staged_dev, int32_t staged_hs, int32_t staged_ws,
                            const void *packed_w_dev, const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev,
                            int32_t *out_acc_dev, void *stream);

/* ---------------------------------------------------------------- int8 GEMM (quantized inner_prod)
 * cpu::math<int8_t,int32_t>::gemm (src/kernels/cpu/math_cpu.cpp:238-244) followed by the
 * epilogue above: out[m][n] = ((float(acc)*dq[n]) * row_scale[m]) + bias[n].
 * a: [m][k] int8 row-major (activations); weights packed from [k][n] row-major (the rhs of
 * base::InnerProd, include/backend/base/base_inner_prod.h:32-48) or [n][k] when transposed. */
size_t tsx_gemm_i8_packed_weight_bytes(int32_t k, int32_t n);
int tsx_gemm_i8_pack_weights(int32_t k, int32_t n, int32_t transposed, const int8_t *w_dev, void *packed_dev,
                             void *stream);
size_t tsx_gemm_i8_workspace_bytes(int32_t m, int32_t k);
int tsx_gemm_i8(int32_t m, int32_t n, int32_t k, const int8_t *a_dev, const void *packed_w_dev,
                const tsx_epilogue *ep, float *out_f32_dev, int8_t *out_i8_dev, int32_t *out_acc_dev,
                void *workspace_dev, size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- fp32 conv2d / inner_prod
 * cpu::Conv2DCore::conv2d (src/kernels/cpu/conv2d_core.cpp:101-119, interface
 * include/backend/base/base_conv2d_core.h:14-32): im2col + GEMM, here one implicit-GEMM kernel on
 * the fp32 MFMA reading NCHW directly (weights are used as they are: no packing, no workspace).
 * bias_dev (optional, [cout]) and act fuse the add_bias / relu operators that follow the conv in
 * BASELINE config 1; pass NULL / TSX_ACT_NONE for the bare operator.  Parity bar for this
 * floating-point path: 1e-4 relative / 1e-5 absolute against the reference CPU kernels. */
int tsx_conv2d_f32_nchw(const tsx_conv2d_geom *g, const float *x_dev, const float *w_oihw_dev, float padding_value,
                        const float *bias_dev, int32_t act, float slope, float *out_dev, void *stream);
/* Which kernel tsx_conv2d_f32_nchw launches for this layer and these weights (their alignment counts), as text:
 * "kernel=small_3x3 | register_fed | staged_64x64 | staged_32x32_ksplit tiles=<output tiles>".  No counterpart in
 * the reference; for tests that must know a given kernel ran, and for logs.  The environment variables
 * TSX_CONV_F32_SMALL and TSX_GEMM_F32_REGFED ("0" = never, "force" = wherever the operands allow) are read at every
 * call. */
int tsx_conv2d_f32_plan_info(const tsx_conv2d_geom *g, const float *w_oihw_dev, char *text, size_t text_bytes);

/* cpu::InnerProd::inner_prod (src/kernels/cpu/inner_prod.cpp:54-69, interface
 * include/backend/base/base_inner_prod.h:32-48): out[m][n] = lhs[m][k] * rhs, rhs being [k][n], or
 * [n][k] when transpose != 0. */
int tsx_inner_prod_f32(int32_t m, int32_t n, int32_t k, const float *lhs_dev, const float *rhs_dev, int32_t transpose,
                       float *out_dev, void *stream);

/* ---------------------------------------------------------------- stand-alone epilogue operators
 * For graphs that keep them as separate nodes (HBM-bound: 4 B in + 4 B out per element).
 *   tsx_add_bias_f32   cpu::AddBias   (src/kernels/cpu/add_bias.cpp:47-85): x is [pre][channels][inner]
 *   tsx_relu_f32       cpu::ReLU      (src/kernels/cpu/relu.cpp:30-52)
 *   tsx_leaky_relu_f32 cpu::LeakyReLU (src/kernels/cpu/leaky_relu.cpp:41-66)
 * The activations reproduce the reference's SIMD-body / scalar-tail split (signed zero, NaN). */
int tsx_add_bias_f32(const float *x_dev, int64_t pre, int32_t channels, int64_t inner, const float *bias_dev,
                     float *out_dev, void *stream);
int tsx_relu_f32(const float *x_dev, int64_t count, float *out_dev, void *stream);
int tsx_leaky_relu_f32(const float *x_dev, int64_t count, float scale, float *out_dev, void *stream);

/* Batch normalisation nodes of graphs whose BN was not folded into the convolution, x = [pre][channels][inner]:
 *   tsx_batch_norm_f32        cpu::BatchNorm      (src/kernels/cpu/batch_norm.cpp:61-105; interface
 *                             include/backend/base/base_batch_norm.h): (x - mean[c]) * (1 / sqrt(variance[c] + epsilon))
 *   tsx_batch_scale_f32       cpu::BatchScale     (src/kernels/cpu/batch_scale.cpp:57-97): x * scale[c] + bias[c]
 *   tsx_fused_batch_norm_f32  cpu::FusedBatchNorm (src/kernels/cpu/fused_batch_norm.cpp:70-125): the two in one pass
 * Same roundings as the reference's AVX2/FMA build (reciprocal root evaluated in double and rounded once, the
 * scale-and-shift a single fused multiply-add): results match it bit for bit. */
int tsx_batch_norm_f32(const float *x_dev, int64_t pre, int32_t channels, int64_t inner, const float *mean_dev,
                       const float *variance_dev, float epsilon, float *out_dev, void *stream);
int tsx_batch_scale_f32(const float *x_dev, int64_t pre, int32_t channels, int64_t inner, const float *scale_dev,
                        const float *bias_dev, float *out_dev, void *stream);
int tsx_fused_batch_norm_f32(const float *x_dev, int64_t pre, int32_t channels, int64_t inner, const float *mean_dev,
                             const float *variance_dev, const float *scale_dev, const float *bias_dev, float epsilon,
                             float *out_dev, void *stream);

/* ---------------------------------------------------------------- glue between convolutions
 * The HBM-bound operators that sit between the convolutions of whole networks, so that a graph stays
 * on the device:
 *   tsx_add_f32        cpu::Add on equal shapes (src/kernels/cpu/add.cpp; a residual join), optionally
 *                      followed by relu / leaky_relu in the same pass (same semantics as the separate
 *                      activation operator on the sum)
 *   tsx_pooling2d_f32  cpu::Pooling2DCore::pooling2d (src/kernels/cpu/pooling2d_core.cpp:48-186) behind
 *                      base::Pooling2D and base::GlobalPooling2D (base_global_pooling2d.cpp:58-79: window =
 *                      whole map, stride 1, no padding).  type 0 = MAX, 1 = AVG (Pooling2DType,
 *                      include/backend/common_structure.h:84-87); white_padding selects Padding2DType WHITE
 *                      (AVG divides by kh*kw) instead of BLACK (by the valid count).  planes = N*C.
 *   tsx_pooling2d_out_size  pooling2d_forward (include/backend/common_function.h:14-20): ceil mode. */
int tsx_add_f32(const float *a_dev, const float *b_dev, int64_t count, int32_t act, float slope, float *out_dev,
                void *stream);
/*   tsx_add_broadcast_f32   cpu::Add::reduce_with_broadcast (src/kernels/cpu/add.cpp) for operands whose shapes,
 *                      already aligned to `dims` axes (at most 8) as ElementWiseReduce::reduce leaves them
 *                      (src/backend/base/element_wise_reduce.cpp:150-206), differ: an extent of 1 repeats.  The
 *                      shape arrays are host memory. */
int tsx_add_broadcast_f32(const float *lhs_dev, const int32_t *lhs_shape, const float *rhs_dev, const int32_t *rhs_shape,
                          int32_t dims, float *out_dev, void *stream);
/*   tsx_mish_f32       mul(x, tanh(softplus(x))) in one pass (TSX_ACT_MISH above)
 *   tsx_concat_channels_f32  cpu::Concat (src/kernels/cpu/concat.cpp) on dim 1 of NCHW, one call per input:
 *                      copies src [n][c_src][inner] into channels [c_offset, c_offset + c_src) of dst [n][c_dst][inner]
 *   tsx_resize_nearest_f32   cpu::Resize2D, Resize2DType::NEAREST, on [planes][h][w] (src/kernels/cpu/resize2d.cpp:186-215:
 *                      source index round(scale * d + scale/2 - 0.5) in double, clamped)
 *   tsx_depthwise_conv2d_f32 cpu::DepthwiseConv2D (src/kernels/cpu/depthwise_conv2d_algorithm.cpp:44-85), weights
 *                      [1][C][KH][KW] (base_depthwise_conv2d.cpp:11-24), geometry as tsx_conv2d_geom with cout == c;
 *                      optional add_bias + activation fused behind it; same fused-multiply-add order as the reference */
int tsx_mish_f32(const float *x_dev, int64_t count, float *out_dev, void *stream);
/* The nodes TenniS graphs compose Mish from, one by one:
 *   tsx_softplus_f32   cpu::Softplus (src/kernels/cpu/softplus.cpp:30-39): float(log(double(expf(x)) + 1.0))
 *   tsx_tanh_f32       cpu::Tanh (src/kernels/cpu/tanh.cpp:14-23): 2 * (1 / (1 + expf(-2x))) - 1 in float
 *   tsx_mul_f32 / tsx_mul_broadcast_f32   cpu::Mul (src/kernels/cpu/mul.cpp) on equal shapes / with the shape
 *                      alignment of tsx_add_broadcast_f32 above; one IEEE multiplication per element (bit-exact)
 * expf / log are the device's library routines: softplus and tanh agree with the host's to a few ulp. */
int tsx_softplus_f32(const float *x_dev, int64_t count, float *out_dev, void *stream);
int tsx_tanh_f32(const float *x_dev, int64_t count, float *out_dev, void *stream);
int tsx_mul_f32(const float *a_dev, const float *b_dev, int64_t count, float *out_dev, void *stream);
int tsx_mul_broadcast_f32(const float *lhs_dev, const int32_t *lhs_shape, const float *rhs_dev, const int32_t *rhs_shape,
                          int32_t dims, float *out_dev, void *stream);
int tsx_concat_channels_f32(const float *src_dev, int64_t n, int32_t c_src, int64_t inner, float *dst_dev, int32_t c_dst,
                            int32_t c_offset, void *stream);
int tsx_resize_nearest_f32(const float *x_dev, int64_t planes, int32_t h, int32_t w, float *out_dev, int32_t out_h,
                           int32_t out_w, void *stream);
int tsx_depthwise_conv2d_f32(const tsx_conv2d_geom *g, const float *x_dev, const float *w_dev, float padding_value,
                             const float *bias_dev, int32_t act, float slope, float *out_dev, void *stream);
int tsx_pooling2d_out_size(int32_t h, int32_t w, int32_t kh, int32_t kw, int32_t pad_top, int32_t pad_bottom,
                           int32_t pad_left, int32_t pad_right, int32_t stride_h, int32_t stride_w, int32_t *out_h,
                           int32_t *out_w);
int tsx_pooling2d_f32(const float *x_dev, int64_t planes, int32_t h, int32_t w, int32_t type, int32_t pad_top,
                      int32_t pad_left, int32_t kh, int32_t kw, int32_t stride_h, int32_t stride_w, int32_t white_padding,
                      float *out_dev, int32_t out_h, int32_t out_w, void *stream);

/* An h x w x c int8 map inside a pixel-major staged buffer [n][hs][ws][cp] (the layout
 * tsx_conv2d_i8_staged_dims describes and tsx_epilogue.staged_out_dev is written in): the map's element
 * (y, x, ch) of image i sits at ((i*hs + y + pad_top)*ws + x + pad_left)*cp + ch. */
typedef struct tsx_staged_map {
    void *data;
    int32_t n, hs, ws, cp;
    int32_t pad_top, pad_left;
    int32_t h, w, c;
} tsx_staged_map;

/* cpu::Pooling2DCore MAX (src/kernels/cpu/pooling2d_core.cpp:48-93) applied between a quantized producer and a
 * quantized consumer, on the producer's requantized int8 output: quantize (src/kernels/cpu/quantize.cpp:70-125) is
 * monotone non-decreasing for a positive scale, so max-pooling the int8 values gives byte for byte what
 * pooling2d(fp32) -> quantize gives.  Window clipped to the map as in the reference; dst->h, dst->w are the
 * output size (tsx_pooling2d_out_size); dst's halo is left as it is, its channels from c up to the next multiple of 64
 * are zeroed (the channel padding of the map's last 64-channel block) and none beyond: `data` may point at a run of
 * channels (a multiple of 64 of them, at a multiple of 16) inside a wider staged buffer whose pitch is cp -- an SPP
 * block pools one run of a concatenation's channels into the next. */
int tsx_max_pooling2d_i8_staged(const tsx_staged_map *src, const tsx_staged_map *dst, int32_t kh, int32_t kw, int32_t pad_top,
                                int32_t pad_left, int32_t stride_h, int32_t stride_w, void *stream);

/* ---------------------------------------------------------------- Winograd F(6x6, 3x3) fp32 conv2d
 * Conv2dWinogradAlgorithm<float>::winograd_f63 (src/kernels/cpu/winograd_algorithm.cpp:846-947),
 * reached in the reference through base::Conv2DWinograd's two core calls
 * (include/backend/base/base_conv2d_winograd.h:24-27):
 *   conv2d_tranform_kernel(mode, kernel, kernel_transformed)  -> tsx_winograd_f63_transform_kernel
 *   conv2d_winograd(x, mode, padding, padding_value, w, ...)   -> tsx_conv2d_winograd_f63_nchw
 * 3x3 kernels, stride 1, dilation 1 only.  The transformed kernel u_dev ([64][cout][cin] floats,
 * tsx_winograd_f63_kernel_bytes) is this backend's own layout, produced and consumed only here.
 * Transforms and accumulation order restate the reference's arithmetic exactly (including the
 * fused multiply-adds of its AVX2/FMA build), so results match its F(6,3) to the bit; optional
 * bias/activation are the add_bias / relu operators fused behind the output transform. */
size_t tsx_winograd_f63_kernel_bytes(int32_t cout, int32_t cin);
int tsx_winograd_f63_transform_kernel(int32_t cout, int32_t cin, const float *w_oihw_dev, float *u_dev, void *stream);
size_t tsx_winograd_f63_workspace_bytes(const tsx_conv2d_geom *g);
int tsx_conv2d_winograd_f63_nchw(const tsx_conv2d_geom *g, const float *x_dev, const float *u_dev, float padding_value,
                                 const float *bias_dev, int32_t act, float slope, float *out_dev, void *workspace_dev,
                                 size_t workspace_bytes, void *stream);
/* The same operator (same u_dev, same arguments) with the 64 frequency GEMMs on the fp32 MFMA and the output
 * transform fused behind them: two launches instead of three, the products M never reach memory, workspace = the
 * transformed input only (tsx_winograd_f63_fast_workspace_bytes).  The MFMA sums the channel products in another
 * order than the reference's FMA chains, so this entry is held to a floating-point bar -- the one TenniS's own
 * backend test applies between devices, max 1e-4 / mean 1e-5 (tools/run_test/test_case.hpp:491-503) -- against
 * winograd_f63 (src/kernels/cpu/winograd_algorithm.cpp:846-947), not to its bits; tsx_conv2d_winograd_f63_nchw is
 * the bit-exact one. */
size_t tsx_winograd_f63_fast_workspace_bytes(const tsx_conv2d_geom *g);
int tsx_conv2d_winograd_f63_fast_nchw(const tsx_conv2d_geom *g, const float *x_dev, const float *u_dev, float padding_value,
                                      const float *bias_dev, int32_t act, float slope, float *out_dev, void *workspace_dev,
                                      size_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- Winograd F(2x2, 3x3) fp32 conv2d
 * Conv2dWinogradAlgorithm<float>::winograd_f23 (src/kernels/cpu/winograd_algorithm.cpp:347-459), the
 * mode base::Conv2DWinograd picks unless Cin*Cout >= 256*256 on maps larger than 16x16
 * (KernelCommonFunc::winograd_mode_select_on_arm, src/kernels/common/function.cpp:154-173).  Same
 * contract as the F(6,3) calls above with 16 instead of 64 tile positions (u_dev is [16][cout][cin]);
 * results match the reference's F(2,3) to the bit. */
size_t tsx_winograd_f23_kernel_bytes(int32_t cout, int32_t cin);
int tsx_winograd_f23_transform_kernel(int32_t cout, int32_t cin, const float *w_oihw_dev, float *u_dev, void *stream);
size_t tsx_winograd_f23_workspace_bytes(const tsx_conv2d_geom *g);
int tsx_conv2d_winograd_f23_nchw(const tsx_conv2d_geom *g, const float *x_dev, const float *u_dev, float padding_value,
                                 const float *bias_dev, int32_t act, float slope, float *out_dev, void *workspace_dev,
                                 size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TSX_HIP_H */
