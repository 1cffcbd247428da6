// The "hip" device operators of the convolution hot path: each class inherits the
// device-agnostic skeleton (parameter parsing, infer, run) and implements only the core
// method, which hands raw device pointers to the C ABI in include/tsx_hip.h -- the structure
// of TenniS's own device backends (src/kernels/gpu/conv2d.cu:8, inner_prod.cu:71-131,
// src/kernels/cpu/quantize.cpp:147, src/kernels/cpu/quantized/conv2d_quantized.cpp:7).
//
// Registered (device "hip"): quantize, conv2d_quantized, conv2d, conv2d_winograd, inner_prod,
// add_bias, relu, leaky_relu.  Everything else in a graph falls back to the host operators
// through OperatorCreator::Query's device -> memory device -> cpu order.
#include <mutex>

#include "hip_device.h"
#include "tsx_hip.h"

namespace ts {
namespace hip {

namespace {

tsx_conv2d_geom make_geom(const Tensor &x, const Tensor &w, const Padding2D &padding, const Stride2D &stride,
                          const Dilation2D &dilation) {
    tsx_conv2d_geom g;
    g.n = x.size(0);
    g.c = x.size(1);
    g.h = x.size(2);
    g.w = x.size(3);
    g.cout = w.size(0);
    g.kh = w.size(2);
    g.kw = w.size(3);
    g.pad_top = padding.top;
    g.pad_bottom = padding.bottom;
    g.pad_left = padding.left;
    g.pad_right = padding.right;
    g.stride_h = stride.height;
    g.stride_w = stride.width;
    g.dilation_h = dilation.height;
    g.dilation_w = dilation.width;
    return g;
}

// Host vector -> device tensor, cached while the host values stay the same (parameters such as
// quantize_scale / dequantize_scales are fixed at init(); the reference hands them to the core by
// value on every run).
class DeviceFloats {
public:
    const float *get(const std::vector<float> &host, const MemoryDevice &device) {
        if (m_tensor.empty() || host != m_host || m_tensor.device() != device) {
            Tensor staged = tensor::build(FLOAT32, Shape({int32_t(host.size())}), host.data());
            m_tensor = staged.view(device);
            m_host = host;
        }
        return m_tensor.data<float>();
    }

private:
    std::vector<float> m_host;
    Tensor m_tensor;
};

}  // namespace

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
        // Weights are constant graph data: pack them into MFMA operand tiles once per weight
        // tensor and geometry, on first use (the pack translator leaves them unpacked for a
        // device that registers its own operator).
        const size_t packed_bytes = tsx_conv2d_i8_packed_weight_bytes(&g);
        if (packed_bytes == 0) TS_LOG_ERROR << "[hip] conv2d_quantized: " << tsx_last_error() << eject;
        if (m_packed.empty() || m_packed_from != w.data() || size_t(m_packed.count()) != packed_bytes || m_packed_cin != g.c) {
            m_packed = Tensor(out.device(), INT8, Shape({int32_t(packed_bytes)}));
            check(tsx_conv2d_i8_pack_weights(&g, w.data<int8_t>(), m_packed.data(), stream), "tsx_conv2d_i8_pack_weights");
            m_packed_from = w.data();
            m_packed_cin = g.c;
        }
        // staging scratch for the activations: kept across runs instead of taken from the stack's
        // scratch frame, so the steady state allocates nothing
        const size_t ws_bytes = tsx_conv2d_i8_workspace_bytes(&g);
        if (m_workspace.empty() || size_t(m_workspace.count()) < ws_bytes || m_workspace.device() != out.device())
            m_workspace = Tensor(out.device(), INT8, Shape({int32_t(ws_bytes ? ws_bytes : 16)}));
        Tensor &workspace = m_workspace;
        (void) stack;
        tsx_epilogue ep{};
        ep.dq_dev = m_dq.get(dequantize_scale, out.device());
        ep.act = TSX_ACT_NONE;
        check(tsx_conv2d_i8_nchw(&g, x.data<int8_t>(), m_packed.data(), padding_value, &ep, out.data<float>(), nullptr,
                                 nullptr, workspace.data(), ws_bytes, stream),
              "tsx_conv2d_i8_nchw");
    }

private:
    Tensor m_packed;
    Tensor m_workspace;
    const void *m_packed_from = nullptr;
    int m_packed_cin = 0;
    DeviceFloats m_dq;
};

// ---------------------------------------------------------------- conv2d (fp32)
class Conv2D : public OperatorOnHip<base::Conv2D> {
public:
    void conv2d(const Tensor &x, const Padding2D &padding, float padding_value, const Tensor &w, const Stride2D &stride,
                const Dilation2D &dilation, Conv2DFormat format, Tensor &out, Stack &, bool kernel_packed) override {
        if (format != FORMAT_NCHW) TS_LOG_ERROR << "Conv2D only support NCHW" << eject;
        if (out.dtype() != FLOAT32)
            TS_LOG_ERROR << "Conv2D not support data type(" << out.dtype() << "): " << type_str(out.dtype()) << eject;
        // kernel_packed marks weights pre-packed for the host GEMM; a device with its own conv2d
        // receives them unpacked (src/compiler/option/pack_translator_option.cpp:14-27)
        if (kernel_packed) TS_LOG_ERROR << "[hip] conv2d expects OIHW weights (kernel_packed=false)" << eject;
        const tsx_conv2d_geom g = make_geom(x, w, padding, stride, dilation);
        check(tsx_conv2d_f32_nchw(&g, x.data<float>(), w.data<float>(), padding_value, nullptr, TSX_ACT_NONE, 0.f,
                                  out.data<float>(), current_stream()),
              "tsx_conv2d_f32_nchw");
    }
};

// ---------------------------------------------------------------- conv2d_winograd (fp32, F(6,3))
class Conv2DWinograd : public OperatorOnHip<base::Conv2DWinograd> {
public:
    void conv2d_tranform_kernel(WinogradConv2DMode, const Tensor &kernel, Tensor &kernel_transformed) override {
        if (kernel.dtype() != FLOAT32) TS_LOG_ERROR << "Conv2DWinograd not support data type: " << type_str(kernel.dtype()) << eject;
        if (kernel.size(2) != 3 || kernel.size(3) != 3) TS_LOG_ERROR << "Conv2DWinograd needs a 3x3 kernel" << eject;
        // [cout, cin, 8, 8] floats = the 64 x cout x cin transformed kernel
        check(tsx_winograd_f63_transform_kernel(kernel.size(0), kernel.size(1), kernel.data<float>(),
                                                kernel_transformed.data<float>(), current_stream()),
              "tsx_winograd_f63_transform_kernel");
    }

    void conv2d_winograd(const Tensor &x, WinogradConv2DMode, const Padding2D &padding, float padding_value, const Tensor &w,
                         Conv2DFormat format, Tensor &out, bool) override {
        if (format != FORMAT_NCHW) TS_LOG_ERROR << "Conv2DWinograd only support NCHW" << eject;
        if (x.dtype() != FLOAT32) TS_LOG_ERROR << "Conv2DWinograd not support data type: " << type_str(x.dtype()) << eject;
        tsx_conv2d_geom g{};
        g.n = x.size(0);
        g.c = x.size(1);
        g.h = x.size(2);
        g.w = x.size(3);
        g.cout = w.size(0);
        g.kh = g.kw = 3;
        g.pad_top = padding.top;
        g.pad_bottom = padding.bottom;
        g.pad_left = padding.left;
        g.pad_right = padding.right;
        g.stride_h = g.stride_w = g.dilation_h = g.dilation_w = 1;
        const size_t ws_bytes = tsx_winograd_f63_workspace_bytes(&g);
        if (ws_bytes == 0) TS_LOG_ERROR << "[hip] conv2d_winograd: " << tsx_last_error() << eject;
        if (m_workspace.empty() || size_t(m_workspace.count()) < ws_bytes)
            m_workspace = Tensor(out.device(), INT8, Shape({int32_t(ws_bytes)}));
        check(tsx_conv2d_winograd_f63_nchw(&g, x.data<float>(), w.data<float>(), padding_value, nullptr, TSX_ACT_NONE, 0.f,
                                           out.data<float>(), m_workspace.data(), ws_bytes, current_stream()),
              "tsx_conv2d_winograd_f63_nchw");
    }

private:
    Tensor m_workspace;
};

// ---------------------------------------------------------------- inner_prod (fp32)
class InnerProd : public OperatorOnHip<base::InnerProd> {
public:
    void inner_prod(const Tensor &lhs, const Tensor &rhs, bool transpose, Tensor &out, Stack &, bool kernel_packed) override {
        if (out.dtype() != FLOAT32) TS_LOG_ERROR << this->op() << " not support data type: " << type_str(out.dtype()) << eject;
        if (kernel_packed) TS_LOG_ERROR << "[hip] inner_prod expects unpacked weights (kernel_packed=false)" << eject;
        check(tsx_inner_prod_f32(out.size(0), out.size(1), lhs.size(1), lhs.data<float>(), rhs.data<float>(), transpose ? 1 : 0,
                                 out.data<float>(), current_stream()),
              "tsx_inner_prod_f32");
    }
};

// ---------------------------------------------------------------- add_bias / relu / leaky_relu
class AddBias : public OperatorOnHip<base::AddBias> {
public:
    void add(const Tensor &x, const Tensor &b, int dim, Tensor &out) override {
        if (x.dtype() != FLOAT32) TS_LOG_ERROR << this->op() << " not support data type: " << type_str(x.dtype()) << eject;
        int64_t pre = 1, inner = 1;
        for (int i = 0; i < dim; ++i) pre *= x.size(size_t(i));
        for (size_t i = size_t(dim) + 1; i < x.dims(); ++i) inner *= x.size(i);
        check(tsx_add_bias_f32(x.data<float>(), pre, x.size(size_t(dim)), inner, b.data<float>(), out.data<float>(),
                               current_stream()),
              "tsx_add_bias_f32");
    }
};

class ReLU : public OperatorOnHip<base::Activation> {
public:
    void active(const Tensor &x, Tensor &out) override {
        if (x.dtype() != FLOAT32) TS_LOG_ERROR << this->op() << " not support data type: " << type_str(x.dtype()) << eject;
        check(tsx_relu_f32(x.data<float>(), x.count(), out.data<float>(), current_stream()), "tsx_relu_f32");
    }
};

class LeakyReLU : public OperatorOnHip<base::LeakyReLU> {
public:
    void leaky_relu(const Tensor &x, float scale, Tensor &out) override {
        if (x.dtype() != FLOAT32) TS_LOG_ERROR << this->op() << " not support data type: " << type_str(x.dtype()) << eject;
        check(tsx_leaky_relu_f32(x.data<float>(), x.count(), scale, out.data<float>(), current_stream()), "tsx_leaky_relu_f32");
    }
};

}  // namespace hip
}  // namespace ts

using namespace ts;
using namespace ts::hip;
TS_REGISTER_OPERATOR(ts::hip::Quantize, ts::hip::DEVICE, name::layer::quantize())
TS_REGISTER_OPERATOR(ts::hip::Conv2DQuantized, ts::hip::DEVICE, name::layer::conv2d_quantized())
TS_REGISTER_OPERATOR(ts::hip::Conv2D, ts::hip::DEVICE, name::layer::conv2d())
TS_REGISTER_OPERATOR(ts::hip::Conv2DWinograd, ts::hip::DEVICE, name::layer::conv2d_winograd())
TS_REGISTER_OPERATOR(ts::hip::InnerProd, ts::hip::DEVICE, name::layer::inner_prod())
TS_REGISTER_OPERATOR(ts::hip::AddBias, ts::hip::DEVICE, name::layer::add_bias())
TS_REGISTER_OPERATOR(ts::hip::ReLU, ts::hip::DEVICE, name::layer::relu())
TS_REGISTER_OPERATOR(ts::hip::LeakyReLU, ts::hip::DEVICE, name::layer::leaky_relu())
