// The quantized "hip" device operators of the convolution hot path.  Each class inherits the
// device-agnostic skeleton (parameter parsing, infer, run) and implements only the core method,
// which hands raw device pointers to the C ABI in include/tsx_hip.h -- the structure of TenniS's
// own device backends (src/kernels/cpu/quantize.cpp:147,
// src/kernels/cpu/quantized/conv2d_quantized.cpp:7).
//
// Registered (device "hip"): quantize, conv2d_quantized.  They live in their own translation
// unit because TenniS's base_conv2d_core.h and base_conv2d_quantized_core.h both define a
// template named Conv2DWithCore and cannot be included together.
#define TSX_TS_QUANTIZED_OPS
#include "hip_ops_common.h"

namespace ts {
namespace hip {

// ---------------------------------------------------------------- quantize
class Quantize : public OperatorOnHip<base::Quantize> {
public:
    void quantize(const Tensor &x, std::vector<float> quantize_scales, Tensor &out) override {
        if (x.dtype() != FLOAT32)
            TS_LOG_ERROR << this->op() << " not support this data type: " << type_str(x.dtype()) << eject;
        const float *scales = m_scales.get(quantize_scales, out.device());
        check(tsx_quantize_f32_i8(x.data<float>(), x.count(), scales, int32_t(quantize_scales.size()), out.data<int8_t>(),
                                  current_stream()),
              "tsx_quantize_f32_i8");
    }

protected:
    // cpu::Quantize also takes fp64 input (src/kernels/cpu/quantize.cpp:109-125): that runs the host operator
    bool covers(Stack &stack) override { return inputs_are(stack, 1, FLOAT32); }

private:
    DeviceFloats m_scales;
};

// ---------------------------------------------------------------- conv2d_quantized
class Conv2DQuantized : public OperatorOnHip<base::Conv2DQuantized> {
public:
    void conv2d(const Tensor &x, const Padding2D &padding, float padding_value, const Tensor &w, const Stride2D &stride,
                const Dilation2D &dilation, Conv2DFormat format, std::vector<float> dequantize_scale, Tensor &out,
                Stack &stack) override {
        if (format != FORMAT_NCHW) TS_LOG_ERROR << "Conv2D_quantized only support NCHW" << eject;
        if (x.dtype() != INT8) TS_LOG_ERROR << "Conv2D_quantized not support this data type: " << type_str(x.dtype()) << eject;
        const tsx_conv2d_geom g = make_geom(x, w, padding, stride, dilation);
        void *stream = current_stream();
        // Weights are constant graph data: packed into MFMA operand tiles once per weight tensor and geometry,
        // on first use (the pack translator leaves them unpacked for a device that registers its own operator).
        const void *packed = m_state.packed(g, w, out.device(), stream, "conv2d_quantized");
        const size_t ws_bytes = tsx_conv2d_i8_workspace_bytes(&g);
        void *workspace = m_state.workspace(ws_bytes, out.device());
        (void) stack;
        tsx_epilogue ep{};
        ep.dq_dev = m_dq.get(dequantize_scale, out.device());
        ep.act = TSX_ACT_NONE;
        check(tsx_conv2d_i8_nchw(&g, x.data<int8_t>(), packed, padding_value, &ep, out.data<float>(), nullptr, nullptr,
                                 workspace, ws_bytes, stream),
              "tsx_conv2d_i8_nchw");
    }

private:
    PackedConv m_state;
    DeviceFloats m_dq;
};

}  // namespace hip
}  // namespace ts

using namespace ts;
using namespace ts::hip;
TS_REGISTER_OPERATOR(Quantize, ts::hip::DEVICE, name::layer::quantize())
TS_REGISTER_OPERATOR(Conv2DQuantized, ts::hip::DEVICE, name::layer::conv2d_quantized())
