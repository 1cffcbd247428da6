// conv2d_quantized_fused: the operator chain of the int8 hot path as ONE node of device "hip",
//     quantize -> conv2d_quantized -> add_bias -> relu / leaky_relu
// (src/kernels/cpu/quantize.cpp, quantized/conv2d_quantized_core.cpp, add_bias.cpp, relu.cpp, leaky_relu.cpp),
// run as the two kernels of tsx_quantize_conv2d_i8_nchw (staging with the quantize fused in, MFMA kernel with the
// dequantize + bias + activation epilogue) instead of four operators exchanging fp32 tensors.  TenniS has no such
// node: it is what a graph rewrite for this device puts in the chain's place (TenniS's own rewrites of this kind
// are its zipper options, src/compiler/option/winograd_zipper_option.cpp:16-96); tennis_amd/module_file.py holds
// that rewrite for module graphs.  Values are those of the chain, bit for bit.
//
// Inputs: x fp32 NCHW, w int8 OIHW[, bias fp32 [cout]][, residual fp32].  Parameters: those of conv2d_quantized
// (format, padding [4,2], padding_value, stride [4], dilation [4], dequantize_scales [cout]) plus quantize_scale
// [n] (the quantize node's) and, optionally, activation ("relu" or "leaky_relu") with scale (leaky_relu's slope)
// and residual: 1 = the last input is the other operand of an `add` node (src/kernels/cpu/add.cpp) that joined
// the chain in front of the activation, act(y + residual) -- a ResNet block's join --, 2 = behind it,
// act(y) + residual -- a darknet shortcut.  A residual of the output's shape is added in the MFMA kernel's
// epilogue; one that broadcasts into it (the general `add`) takes a broadcast pass behind the convolution.
//
// Two such nodes in a row -- the first's output read by the second's quantize and by nothing else -- exchange the
// activation as int8 in the second's staged layout (pixel-major, channel-blocked, halo included;
// tsx_conv2d_i8_staged_dims) instead of fp32 NCHW: the producer carries the consumer's quantize_scale and
// convolution geometry as next_quantize_scale, next_ksize [2], next_padding [top, bottom, left, right],
// next_stride [2], next_dilation [2], next_padding_value, requantizes in its epilogue
// (quantize(act(...)) of the consumer's quantize node, value for value) and returns an INT8 tensor
// [n, hs, ws, cp]; the consumer is marked staged_input = 1 and runs the MFMA kernel on that tensor directly.
// No staging pass, a quarter of the bytes.  The reference leaves this to a TODO
// (src/backend/base/base_conv2d_quantized.cpp:163).  With dual_output = 1 as well the node returns BOTH forms as
// one packed tensor -- field 0 the fp32 NCHW result, field 1 the staged int8 one -- for a tensor that quantized
// convolutions and other nodes (a later residual join) both read; `_field` nodes pick the form
// (src/runtime/instruction/tensor_instruction.cpp:38-61).
#define TSX_TS_QUANTIZED_OPS   // Padding2D / Stride2D / Dilation2D come with the quantized skeleton
#include "hip_ops_common.h"

#include <string>
#include <vector>

namespace ts {
namespace hip {

class Conv2DQuantizedFused : public Operator {
public:
    using self = Conv2DQuantizedFused;
    using supper = Operator;

    Conv2DQuantizedFused() {
        field(name::format, REQUIRED);
        field(name::padding, REQUIRED);
        field(name::padding_value, OPTIONAL, tensor::from(0.0f));
        field(name::stride, REQUIRED);
        field(name::dilation, OPTIONAL);
        field(name::typo::dialations, OPTIONAL);
        field(name::dequantize_scales, REQUIRED);
        field(name::quantize_scale, REQUIRED);
        field("activation", OPTIONAL, tensor::from("none"));
        field(name::scale, OPTIONAL, tensor::from(0.0f));
        field("residual", OPTIONAL, tensor::from(int(0)));
        field("staged_input", OPTIONAL, tensor::from(int(0)));
        field("next_quantize_scale", OPTIONAL);
        field("next_ksize", OPTIONAL);
        field("next_padding", OPTIONAL);
        field("next_stride", OPTIONAL);
        field("next_dilation", OPTIONAL);
        field("next_padding_value", OPTIONAL, tensor::from(0.0f));
        field("dual_output", OPTIONAL, tensor::from(int(0)));
    }

    void init() override {
        supper::init();
        if (tensor::to_string(get(name::format)) != "NCHW") TS_LOG_ERROR << "conv2d_quantized_fused only support NCHW" << eject;
        const std::vector<int32_t> pad = ints(name::padding, 8), stride = ints(name::stride, 4);
        if (!has(name::dilation) && !has(name::typo::dialations))
            TS_LOG_ERROR << "conv2d_quantized_fused: dilation must be set" << eject;
        const std::vector<int32_t> dil = ints(has(name::dilation) ? std::string(name::dilation) : std::string(name::typo::dialations), 4);
        if (pad[0] || pad[1] || pad[2] || pad[3] || stride[0] != 1 || stride[1] != 1 || dil[0] != 1 || dil[1] != 1)
            TS_LOG_ERROR << "conv2d_quantized_fused: padding / stride / dilation of the batch and channel axes must be 0 / 1 / 1" << eject;
        m_pad = {pad[4], pad[5], pad[6], pad[7]};
        m_stride = {stride[2], stride[3]};
        m_dil = {dil[2], dil[3]};
        m_padding_value = tensor::to_float(get(name::padding_value));
        m_dq = tensor::array::to_float(get(name::dequantize_scales));
        m_q = tensor::array::to_float(get(name::quantize_scale));
        const std::string act = tensor::to_string(get("activation"));
        if (act == "none") m_act = TSX_ACT_NONE;
        else if (act == "relu") m_act = TSX_ACT_RELU;
        else if (act == "leaky_relu") m_act = TSX_ACT_LEAKY_RELU;
        else TS_LOG_ERROR << "conv2d_quantized_fused: activation must be none, relu or leaky_relu, got " << act << eject;
        m_slope = tensor::to_float(get(name::scale));
        m_residual = tensor::to_int(get("residual"));
        if (m_residual < 0 || m_residual > 2) TS_LOG_ERROR << "conv2d_quantized_fused: residual must be 0, 1 or 2" << eject;
        m_staged_input = tensor::to_int(get("staged_input")) != 0;
        m_next = has("next_quantize_scale");
        if (m_next) {
            m_next_q = tensor::array::to_float(get("next_quantize_scale"));
            m_next_ksize = ints("next_ksize", 2);
            m_next_pad = ints("next_padding", 4);
            m_next_stride = ints("next_stride", 2);
            m_next_dil = ints("next_dilation", 2);
            m_next_padding_value = tensor::to_float(get("next_padding_value"));
        }
        m_dual = tensor::to_int(get("dual_output")) != 0;
        if (m_dual && !m_next) TS_LOG_ERROR << "conv2d_quantized_fused: dual_output needs the next_* parameters" << eject;
    }

    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override {
        tsx_conv2d_geom g, gn;
        const Tensor::Prototype proto = out_proto(stack, g, gn);
        output.clear();
        if (m_dual) output.push_back(Tensor::Prototype(FLOAT32, m_out_shape));
        output.push_back(proto);
        return int(output.size());
    }

    int run(Stack &stack) override {
        tsx_conv2d_geom g, gn;
        const Tensor::Prototype proto = out_proto(stack, g, gn);
        auto &context = ctx::ref<DeviceContext>();
        const MemoryDevice device = context.memory_device;
        Tensor x = stack[0].view(device), w = stack[1].view(device);
        Tensor bias, residual;
        const int extra = int(stack.size()) - 2 - (m_residual ? 1 : 0);
        const bool with_bias = extra == 1;
        if (with_bias) bias = stack[2].view(device);
        if (m_residual) residual = stack[int(stack.size()) - 1].view(device);
        const Shape conv_shape({g.n, g.cout, m_ho, m_wo});
        const bool same_shape = m_residual && residual.sizes() == conv_shape;
        // A residual of another shape (it broadcasts into the convolution's output, or the output into it) joins in a
        // pass of its own, as the separate `add` did: the epilogue writes fp32, the activation in front of the join
        // (mode 2) stays in the epilogue, the one behind it (mode 1) follows the pass, and a staged int8 output is
        // then quantized and staged from the sum by the staging kernel.
        const bool split = m_residual && !same_shape;
        // The staged int8 output lives in a tensor this operator keeps from run to run: its halo and channel padding
        // are written once, when it is allocated, and every run's epilogue overwrites exactly the interior -- a
        // tensor from the stack is fresh memory each time and would need the halo filled again (one more launch per
        // node and run).  Readers run behind this node on the same stream and the next run's epilogue behind them.
        // Dual output: that tensor plus the fp32 one, pushed as one packed tensor at the end.
        Tensor out;
        bool fill_halo = false;
        if (m_next) {
            if (m_staged_out.empty() || m_staged_out.device() != device || m_staged_out.dtype() != proto.dtype() ||
                !(m_staged_out.sizes() == proto.sizes())) {
                m_staged_out = Tensor(device, proto.dtype(), proto.sizes());
                fill_halo = true;
            }
            out = m_staged_out;
            if (!m_dual) stack.push(out);
        } else {
            out = *stack.push(proto, device);
        }
        Tensor out_plain;
        if (m_dual || (split && m_next)) out_plain = stack.make(Tensor::Prototype(FLOAT32, m_out_shape), device);
        // the convolution's own result where it is not the node's fp32 output already
        Tensor conv_out;
        if (split && (m_next || !(m_out_shape == conv_shape))) conv_out = stack.make(Tensor::Prototype(FLOAT32, conv_shape), device);
        void *stream = current_stream();
        const bool pairs = pairs_apply(g, gn, out);
        const void *packed = pairs ? nullptr : m_state.packed(g, w, device, stream, "conv2d_quantized_fused");
        tsx_epilogue ep{};
        ep.dq_dev = m_dq_dev.get(m_dq, device);
        ep.bias_dev = with_bias ? bias.data<float>() : nullptr;
        ep.act = (split && m_residual == 1) ? TSX_ACT_NONE : m_act;
        ep.slope = m_slope;
        if (same_shape) {
            ep.residual_dev = residual.data<float>();
            ep.residual_after_act = m_residual == 2 ? 1 : 0;
        }
        float *out_f32 = !conv_out.empty() ? conv_out.data<float>() : out.data<float>();
        if (m_next && !split) {
            // the consumer's staged input: halo and channel padding (once), then the interior from the epilogue
            if (fill_halo)
                check(tsx_conv2d_i8_stage_fill_halo(&gn, m_next_padding_value, out.data(), size_t(out.count()), stream),
                      "tsx_conv2d_i8_stage_fill_halo");
            ep.q_scales_dev = m_next_q_dev.get(m_next_q, device);
            ep.n_qscales = int32_t(m_next_q.size());
            ep.staged_out_dev = static_cast<int8_t *>(out.data());
            ep.staged_hs = out.size(1);
            ep.staged_ws = out.size(2);
            ep.staged_cp = out.size(3);
            ep.staged_pad_top = gn.pad_top;
            ep.staged_pad_left = gn.pad_left;
            out_f32 = m_dual ? out_plain.data<float>() : nullptr;
        }
        if (m_staged_input) {
            check(tsx_conv2d_i8_staged_at(&g, x.data(), x.size(1), x.size(2), packed, &ep, out_f32, nullptr, nullptr, stream),
                  "tsx_conv2d_i8_staged_at");
        } else if (pairs) {
            // A few-channel stem whose only output is the staged int8 one: computed as PAIRS of output columns -- a
            // kh x (kw + stride) window at twice the column stride with 2 x cout output channels (the even column's
            // weights in window columns 0..kw-1, the odd one's in stride..stride+kw-1, zeros elsewhere, which add
            // nothing to an integer sum).  A pair's 2 x cout channels are the two pixels' bytes in the staged layout,
            // so the output is the same; the explicit im2col matrix has half the rows of the same padded length.
            tsx_conv2d_geom g2 = g;
            g2.kw = g.kw + g.stride_w;
            g2.stride_w = 2 * g.stride_w;
            g2.cout = 2 * g.cout;
            if (m_pair_w.empty() || m_pair_source.data() != w.data() || m_pair_w.device() != device) {
                const Tensor hw = w.view(MemoryDevice(CPU));
                std::vector<int8_t> w2(size_t(g2.cout) * g.c * g.kh * g2.kw, 0);
                const int8_t *src = hw.data<int8_t>();
                for (int co = 0; co < g.cout; ++co)
                    for (int r = 0; r < g.c * g.kh; ++r)
                        for (int kx = 0; kx < g.kw; ++kx) {
                            const int8_t v = src[(size_t(co) * g.c * g.kh + r) * g.kw + kx];
                            w2[(size_t(co) * g.c * g.kh + r) * g2.kw + kx] = v;
                            w2[(size_t(g.cout + co) * g.c * g.kh + r) * g2.kw + g.stride_w + kx] = v;
                        }
                m_pair_w = tensor::build(INT8, Shape({g2.cout, g.c, g.kh, g2.kw}), w2.data()).view(device);
                m_pair_source = w;
                m_pair_dq = m_dq;
                m_pair_dq.insert(m_pair_dq.end(), m_dq.begin(), m_dq.end());
            }
            if (with_bias && (m_pair_bias.empty() || m_pair_bias_source.data() != bias.data() || m_pair_bias.device() != device)) {
                const Tensor hb = bias.view(MemoryDevice(CPU));
                std::vector<float> b2(hb.data<float>(), hb.data<float>() + g.cout);
                b2.insert(b2.end(), hb.data<float>(), hb.data<float>() + g.cout);
                m_pair_bias = tensor::build(FLOAT32, Shape({g2.cout}), b2.data()).view(device);
                m_pair_bias_source = bias;
            }
            const void *packed2 = m_pair_state.packed(g2, m_pair_w, device, stream, "conv2d_quantized_fused");
            ep.dq_dev = m_pair_dq_dev.get(m_pair_dq, device);
            ep.bias_dev = with_bias ? m_pair_bias.data<float>() : nullptr;
            ep.staged_ws = out.size(2) / 2;
            ep.staged_cp = 2 * out.size(3);
            ep.staged_pad_left = gn.pad_left / 2;
            const size_t ws_bytes = tsx_conv2d_i8_workspace_bytes(&g2);
            void *workspace = m_pair_state.workspace(ws_bytes, device);
            check(tsx_quantize_conv2d_i8_nchw(&g2, x.data<float>(), m_q_dev.get(m_q, device), int32_t(m_q.size()), packed2,
                                              m_padding_value, &ep, nullptr, nullptr, nullptr, workspace, ws_bytes, stream),
                  "tsx_quantize_conv2d_i8_nchw");
        } else {
            const size_t ws_bytes = tsx_conv2d_i8_workspace_bytes(&g);
            void *workspace = m_state.workspace(ws_bytes, device);
            check(tsx_quantize_conv2d_i8_nchw(&g, x.data<float>(), m_q_dev.get(m_q, device), int32_t(m_q.size()), packed,
                                              m_padding_value, &ep, out_f32, nullptr, nullptr, workspace, ws_bytes, stream),
                  "tsx_quantize_conv2d_i8_nchw");
        }
        if (split) {
            Tensor &sum = m_next ? out_plain : out;
            std::vector<int32_t> lhs(conv_shape.begin(), conv_shape.end()), rhs(lhs.size(), 1);
            const Shape &rs = residual.sizes();
            for (size_t i = 0; i < rs.size(); ++i) rhs[lhs.size() - rs.size() + i] = rs[i];
            check(tsx_add_broadcast_f32(out_f32, lhs.data(), residual.data<float>(), rhs.data(), int32_t(lhs.size()),
                                        sum.data<float>(), stream),
                  "tsx_add_broadcast_f32");
            if (m_residual == 1 && m_act == TSX_ACT_RELU)
                check(tsx_relu_f32(sum.data<float>(), sum.count(), sum.data<float>(), stream), "tsx_relu_f32");
            else if (m_residual == 1 && m_act == TSX_ACT_LEAKY_RELU)
                check(tsx_leaky_relu_f32(sum.data<float>(), sum.count(), m_slope, sum.data<float>(), stream), "tsx_leaky_relu_f32");
            if (m_next)   // the whole staged tensor, halo included
                check(tsx_conv2d_i8_stage(&gn, sum.data<float>(), 1, m_next_q_dev.get(m_next_q, device), int32_t(m_next_q.size()),
                                          m_next_padding_value, out.data(), size_t(out.count()), stream),
                      "tsx_conv2d_i8_stage");
        }
        if (m_dual) stack.push(Tensor::Pack({out_plain, out}));
        return 1;
    }

private:
    std::vector<int32_t> ints(const std::string &param, size_t count) {
        const std::vector<int32_t> v = tensor::array::to_int(get(param));
        if (v.size() != count) TS_LOG_ERROR << "conv2d_quantized_fused: " << param << " must hold " << count << " integers" << eject;
        return v;
    }

    // the stem-as-pairs form applies: fp32 input of few channels, a kernel wider than one tap, only the staged int8
    // output, an even number of output columns that pair up with whole staged pixels, and a window whose K pads to the
    // same number of 64-byte steps
    bool pairs_apply(const tsx_conv2d_geom &g, const tsx_conv2d_geom &gn, const Tensor &out) const {
        if (!m_next || m_dual || m_residual || m_staged_input) return false;
        if (g.c > 8 || g.kh * g.kw <= 1 || g.dilation_h != 1 || g.dilation_w != 1) return false;
        if (m_wo % 2 || gn.pad_left % 2 || out.size(2) % 2 || out.size(3) != g.cout || g.cout % 32) return false;
        const int k1 = g.c * g.kh * g.kw, k2 = g.c * g.kh * (g.kw + g.stride_w);
        if ((k1 + 63) / 64 != (k2 + 63) / 64 || k2 > 512) return false;
        const int wo2 = (g.w + g.pad_left + g.pad_right - (g.kw + g.stride_w)) / (2 * g.stride_w) + 1;
        return wo2 == m_wo / 2;
    }

    // checks the inputs against the parameters; fills the geometry (and, with next_*, the consumer's); returns the
    // output prototype
    Tensor::Prototype out_proto(Stack &stack, tsx_conv2d_geom &g, tsx_conv2d_geom &gn) {
        const size_t fixed = m_residual ? 3 : 2;
        if (stack.size() != fixed && stack.size() != fixed + 1)
            TS_LOG_ERROR << "conv2d_quantized_fused expects " << fixed << " or " << fixed + 1 << " inputs (x, w[, bias]"
                         << (m_residual ? ", residual" : "") << "), got " << stack.size() << eject;
        const Tensor &x = stack[0], &w = stack[1];
        if (w.dims() != 4 || w.dtype() != INT8) TS_LOG_ERROR << "conv2d_quantized_fused: w must be int8 OIHW" << eject;
        const Padding2D padding(m_pad[0], m_pad[1], m_pad[2], m_pad[3]);
        if (m_staged_input) {
            // x is this convolution's staged input [n, hs, ws, cp], written by the producing node
            if (x.dims() != 4 || x.dtype() != INT8)
                TS_LOG_ERROR << "conv2d_quantized_fused: staged_input expects an int8 tensor [n, hs, ws, cp]" << eject;
            // a map of hs - pads by ws - pads reads exactly the staged rows and columns (the producer's true extent may
            // be up to stride - 1 larger: those rows and columns lie behind the last window)
            g = tsx_conv2d_geom{x.size(0), w.size(1), x.size(1) - m_pad[0] - m_pad[1], x.size(2) - m_pad[2] - m_pad[3],
                                w.size(0), w.size(2), w.size(3), m_pad[0], m_pad[1], m_pad[2], m_pad[3],
                                m_stride[0], m_stride[1], m_dil[0], m_dil[1]};
            if (g.h < 1 || g.w < 1) TS_LOG_ERROR << "conv2d_quantized_fused: staged input smaller than the padding" << eject;
            int32_t hs = 0, ws = 0, cp = 0;
            if (tsx_conv2d_i8_staged_dims(&g, &hs, &ws, &cp) != 0)
                TS_LOG_ERROR << "[hip] conv2d_quantized_fused: " << tsx_last_error() << eject;
            if (hs > x.size(1) || ws > x.size(2) || cp != x.size(3))
                TS_LOG_ERROR << "conv2d_quantized_fused: staged input " << to_string(x.sizes()) << " does not hold the [" << hs << ", "
                             << ws << ", " << cp << "] this convolution reads" << eject;
        } else {
            if (x.dims() != 4 || x.dtype() != FLOAT32)
                TS_LOG_ERROR << "conv2d_quantized_fused: x must be float32 NCHW and w int8 OIHW" << eject;
            if (x.size(1) != w.size(1))
                TS_LOG_ERROR << "conv2d_quantized_fused: x has " << x.size(1) << " channels, w " << w.size(1) << eject;
            g = make_geom(x, w, padding, Stride2D(m_stride[0], m_stride[1]), Dilation2D(m_dil[0], m_dil[1]));
        }
        if (int32_t(m_dq.size()) != w.size(0))
            TS_LOG_ERROR << "conv2d_quantized_fused: " << m_dq.size() << " dequantize scales for " << w.size(0) << " output channels" << eject;
        if (int32_t(m_q.size()) != x.size(0))      // base_quantize.cpp:26
            TS_LOG_ERROR << "conv2d_quantized_fused: " << m_q.size() << " quantize scales for a batch of " << x.size(0) << eject;
        if (stack.size() == fixed + 1 && !(stack[2].dtype() == FLOAT32 && stack[2].count() == w.size(0)))
            TS_LOG_ERROR << "conv2d_quantized_fused: bias must hold one float32 per output channel" << eject;
        // include/backend/common_function.h:30-40
        const int ho = (g.h + g.pad_top + g.pad_bottom - (g.dilation_h * (g.kh - 1) + 1)) / g.stride_h + 1;
        const int wo = (g.w + g.pad_left + g.pad_right - (g.dilation_w * (g.kw - 1) + 1)) / g.stride_w + 1;
        if (ho <= 0 || wo <= 0) TS_LOG_ERROR << "conv2d_quantized_fused: empty output " << ho << "x" << wo << eject;
        m_ho = ho;
        m_wo = wo;
        Shape out({g.n, w.size(0), ho, wo});
        if (m_residual) {
            // the other operand of the `add` this node absorbed: the two broadcast against each other as the operator's
            // operands did (src/backend/base/element_wise_reduce.cpp:150-206), either one may be the one that repeats
            const Tensor &r = stack[int(stack.size()) - 1];
            bool fits = r.dtype() == FLOAT32 && r.dims() <= out.size();
            for (size_t i = 0; fits && i < r.dims(); ++i) {
                int32_t &target = out[out.size() - r.dims() + i];
                const int32_t extent = r.size(i);
                fits = extent == target || extent == 1 || target == 1;
                if (target == 1) target = extent;
            }
            if (!fits)
                TS_LOG_ERROR << "conv2d_quantized_fused: residual " << to_string(r.sizes()) << " and the convolution's output "
                             << to_string(Shape({g.n, w.size(0), ho, wo})) << " do not broadcast" << eject;
        }
        m_out_shape = out;
        if (!m_next) return Tensor::Prototype(FLOAT32, out);
        // the consumer's staged input
        if (int32_t(m_next_q.size()) != out[0])
            TS_LOG_ERROR << "conv2d_quantized_fused: " << m_next_q.size() << " next_quantize_scale values for a batch of " << out[0] << eject;
        gn = tsx_conv2d_geom{out[0], out[1], out[2], out[3], 1, m_next_ksize[0], m_next_ksize[1], m_next_pad[0], m_next_pad[1],
                             m_next_pad[2], m_next_pad[3], m_next_stride[0], m_next_stride[1], m_next_dil[0], m_next_dil[1]};
        int32_t hs = 0, ws = 0, cp = 0;
        if (tsx_conv2d_i8_staged_dims(&gn, &hs, &ws, &cp) != 0) TS_LOG_ERROR << "[hip] conv2d_quantized_fused: " << tsx_last_error() << eject;
        return Tensor::Prototype(INT8, Shape({g.n, hs, ws, cp}));
    }

    std::vector<int32_t> m_pad, m_stride, m_dil;
    float m_padding_value = 0.f, m_slope = 0.f;
    int m_act = TSX_ACT_NONE;
    int m_residual = 0;   // 0: none; 1: act(y + residual); 2: act(y) + residual
    bool m_staged_input = false, m_next = false, m_dual = false;
    std::vector<float> m_next_q;
    std::vector<int32_t> m_next_ksize, m_next_pad, m_next_stride, m_next_dil;
    float m_next_padding_value = 0.f;
    int m_ho = 0, m_wo = 0;
    Shape m_out_shape;   // the node's output as NCHW: the convolution's, or its broadcast against the residual
    DeviceFloats m_next_q_dev;
    Tensor m_staged_out;
    std::vector<float> m_dq, m_q;
    DeviceFloats m_dq_dev, m_q_dev;
    PackedConv m_state;
    // the stem computed as pairs of output columns: rearranged weights, scales and bias, and their pack
    PackedConv m_pair_state;
    Tensor m_pair_w, m_pair_source, m_pair_bias, m_pair_bias_source;
    std::vector<float> m_pair_dq;
    DeviceFloats m_pair_dq_dev;
};

// max_pooling2d_staged: a MAX pooling2d node (src/kernels/cpu/pooling2d_core.cpp:48-93) between a fused producer and
// quantized convolutions, on the producer's requantized int8 output instead of its fp32 one: quantize is monotone,
// so pooling the int8 values gives what pooling2d -> quantize gives, byte for byte (tsx_max_pooling2d_i8_staged).
// Input: INT8 [n, h, w, cp], the producer's staged output without halo (next_ksize 1x1, no padding).  Parameters:
// ksize [2], stride [2], padding [top, bottom, left, right] of the pooling, and the reading convolutions' geometry
// as next_ksize / next_padding / next_stride / next_dilation / next_padding_value.  Output: their staged input,
// INT8 [n, hs, ws, cp], in a tensor the operator keeps (halo written once, see conv2d_quantized_fused).
class MaxPooling2DStaged : public Operator {
public:
    using self = MaxPooling2DStaged;
    using supper = Operator;

    MaxPooling2DStaged() {
        field(name::ksize, REQUIRED);
        field(name::stride, REQUIRED);
        field(name::padding, REQUIRED);
        field("next_ksize", REQUIRED);
        field("next_padding", REQUIRED);
        field("next_stride", REQUIRED);
        field("next_dilation", REQUIRED);
        field("next_padding_value", OPTIONAL, tensor::from(0.0f));
    }

    void init() override {
        supper::init();
        m_ksize = ints(name::ksize, 2);
        m_stride = ints(name::stride, 2);
        m_pad = ints(name::padding, 4);
        m_next_ksize = ints("next_ksize", 2);
        m_next_pad = ints("next_padding", 4);
        m_next_stride = ints("next_stride", 2);
        m_next_dil = ints("next_dilation", 2);
        m_next_padding_value = tensor::to_float(get("next_padding_value"));
    }

    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override {
        tsx_conv2d_geom gn;
        int32_t oh, ow;
        output.assign(1, out_proto(stack, gn, oh, ow));
        return 1;
    }

    int run(Stack &stack) override {
        tsx_conv2d_geom gn;
        int32_t oh = 0, ow = 0;
        const Tensor::Prototype proto = out_proto(stack, gn, oh, ow);
        const MemoryDevice device = ctx::ref<DeviceContext>().memory_device;
        Tensor x = stack[0].view(device);
        void *stream = current_stream();
        if (m_out.empty() || m_out.device() != device || !(m_out.sizes() == proto.sizes())) {
            m_out = Tensor(device, proto.dtype(), proto.sizes());
            check(tsx_conv2d_i8_stage_fill(&gn, m_next_padding_value, m_out.data(), size_t(m_out.count()), stream),
                  "tsx_conv2d_i8_stage_fill");
        }
        const tsx_staged_map src{x.data(), x.size(0), x.size(1), x.size(2), x.size(3), 0, 0, x.size(1), x.size(2), x.size(3)};
        const tsx_staged_map dst{m_out.data(), m_out.size(0), m_out.size(1), m_out.size(2), m_out.size(3),
                                 gn.pad_top, gn.pad_left, oh, ow, x.size(3)};
        check(tsx_max_pooling2d_i8_staged(&src, &dst, m_ksize[0], m_ksize[1], m_pad[0], m_pad[2], m_stride[0], m_stride[1], stream),
              "tsx_max_pooling2d_i8_staged");
        stack.push(m_out);
        return 1;
    }

private:
    std::vector<int32_t> ints(const std::string &param, size_t count) {
        const std::vector<int32_t> v = tensor::array::to_int(get(param));
        if (v.size() != count) TS_LOG_ERROR << "max_pooling2d_staged: " << param << " must hold " << count << " integers" << eject;
        return v;
    }

    Tensor::Prototype out_proto(Stack &stack, tsx_conv2d_geom &gn, int32_t &oh, int32_t &ow) {
        if (stack.size() != 1) TS_LOG_ERROR << "max_pooling2d_staged expects 1 input, got " << stack.size() << eject;
        const Tensor &x = stack[0];
        if (x.dims() != 4 || x.dtype() != INT8 || x.size(3) % 64 != 0)
            TS_LOG_ERROR << "max_pooling2d_staged expects an int8 tensor [n, h, w, cp]" << eject;
        if (tsx_pooling2d_out_size(x.size(1), x.size(2), m_ksize[0], m_ksize[1], m_pad[0], m_pad[1], m_pad[2], m_pad[3], m_stride[0],
                                   m_stride[1], &oh, &ow) != 0)
            TS_LOG_ERROR << "[hip] max_pooling2d_staged: " << tsx_last_error() << eject;
        gn = tsx_conv2d_geom{x.size(0), x.size(3), oh, ow, 1, m_next_ksize[0], m_next_ksize[1], m_next_pad[0], m_next_pad[1],
                             m_next_pad[2], m_next_pad[3], m_next_stride[0], m_next_stride[1], m_next_dil[0], m_next_dil[1]};
        int32_t hs = 0, ws = 0, cp = 0;
        if (tsx_conv2d_i8_staged_dims(&gn, &hs, &ws, &cp) != 0) TS_LOG_ERROR << "[hip] max_pooling2d_staged: " << tsx_last_error() << eject;
        return Tensor::Prototype(INT8, Shape({x.size(0), hs, ws, cp}));
    }

    std::vector<int32_t> m_ksize, m_stride, m_pad, m_next_ksize, m_next_pad, m_next_stride, m_next_dil;
    float m_next_padding_value = 0.f;
    Tensor m_out;
};

}  // namespace hip
}  // namespace ts

using namespace ts;
using namespace ts::hip;
TS_REGISTER_OPERATOR(Conv2DQuantizedFused, ts::hip::DEVICE, "conv2d_quantized_fused")
TS_REGISTER_OPERATOR(MaxPooling2DStaged, ts::hip::DEVICE, "max_pooling2d_staged")
