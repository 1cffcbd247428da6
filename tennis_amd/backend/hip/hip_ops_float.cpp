// The fp32 "hip" device operators of the convolution hot path: each class inherits the
// device-agnostic skeleton (parameter parsing, infer, run) and implements only the core
// method, which hands raw device pointers to the C ABI in include/tsx_hip.h -- the structure
// of TenniS's own device backends (src/kernels/gpu/conv2d.cu:8, inner_prod.cu:71-131).
//
// Registered (device "hip"): conv2d, conv2d_winograd, inner_prod, add_bias, relu, leaky_relu.
// Everything else in a graph falls back to the host operators through OperatorCreator::Query's
// device -> memory device -> cpu order.
#define TSX_TS_FLOAT_OPS
#include "hip_ops_common.h"

namespace ts {
namespace hip {

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

protected:
    // fp32 NCHW on the MFMA kernel; fp64 and NHWC graphs (the reference's device classes take both,
    // src/kernels/gpu/conv2d_core.cu) run the host operator
    bool covers(Stack &stack) override { return format_is_nchw(*this) && inputs_are(stack, 2, FLOAT32); }
};

// ---------------------------------------------------------------- conv2d_winograd (fp32, F(6,3) and F(2,3))
// base::Conv2DWinograd::run (src/backend/base/base_conv2d_winograd.cpp:124-167) picks the mode from
// the shapes, allocates the transformed-kernel tensor on the HOST whatever the device, and hands it
// back on every run.  This backend keeps its own transformed kernel in device memory, in its own
// layout, and leaves that host tensor untouched.
class Conv2DWinograd : public OperatorOnHip<base::Conv2DWinograd> {
public:
    void conv2d_tranform_kernel(WinogradConv2DMode mode, const Tensor &kernel, Tensor &) override {
        if (kernel.dtype() != FLOAT32) TS_LOG_ERROR << "Conv2DWinograd not support data type: " << type_str(kernel.dtype()) << eject;
        // weights already transformed for the host algorithm ([cout, cin, 8, 8] in its packed layout,
        // the output of the winograd_transform_kernel operator) cannot be used here
        if (kernel.dims() != 4 || kernel.size(2) != 3 || kernel.size(3) != 3)
            TS_LOG_ERROR << "[hip] conv2d_winograd needs the raw OIHW 3x3 kernel, got " << to_string(kernel.sizes()) << eject;
        const int cout = kernel.size(0), cin = kernel.size(1);
        const bool f23 = mode == F2X2_3X3;
        const size_t bytes = f23 ? tsx_winograd_f23_kernel_bytes(cout, cin) : tsx_winograd_f63_kernel_bytes(cout, cin);
        m_u = byte_tensor(kernel.device(), bytes);
        if (f23)
            check(tsx_winograd_f23_transform_kernel(cout, cin, kernel.data<float>(), static_cast<float *>(m_u.data()), current_stream()),
                  "tsx_winograd_f23_transform_kernel");
        else
            check(tsx_winograd_f63_transform_kernel(cout, cin, kernel.data<float>(), static_cast<float *>(m_u.data()), current_stream()),
                  "tsx_winograd_f63_transform_kernel");
        m_mode = mode;
        m_cout = cout;
        m_cin = cin;
    }

    void conv2d_winograd(const Tensor &x, WinogradConv2DMode mode, const Padding2D &padding, float padding_value, const Tensor &,
                         Conv2DFormat format, Tensor &out, bool) override {
        if (format != FORMAT_NCHW) TS_LOG_ERROR << "Conv2DWinograd only support NCHW" << eject;
        if (x.dtype() != FLOAT32) TS_LOG_ERROR << "Conv2DWinograd not support data type: " << type_str(x.dtype()) << eject;
        if (m_u.empty() || mode != m_mode || x.size(1) != m_cin)
            TS_LOG_ERROR << "[hip] conv2d_winograd: kernel was not transformed for this mode and shape" << eject;
        tsx_conv2d_geom g{};
        g.n = x.size(0);
        g.c = x.size(1);
        g.h = x.size(2);
        g.w = x.size(3);
        g.cout = m_cout;
        g.kh = g.kw = 3;
        g.pad_top = padding.top;
        g.pad_bottom = padding.bottom;
        g.pad_left = padding.left;
        g.pad_right = padding.right;
        g.stride_h = g.stride_w = g.dilation_h = g.dilation_w = 1;
        const bool f23 = mode == F2X2_3X3;
        const size_t ws_bytes = f23 ? tsx_winograd_f23_workspace_bytes(&g) : tsx_winograd_f63_workspace_bytes(&g);
        if (ws_bytes == 0) TS_LOG_ERROR << "[hip] conv2d_winograd: " << tsx_last_error() << eject;
        if (m_workspace.empty() || size_t(m_workspace.count()) < ws_bytes)
            m_workspace = byte_tensor(out.device(), ws_bytes);
        if (f23)
            check(tsx_conv2d_winograd_f23_nchw(&g, x.data<float>(), static_cast<float *>(m_u.data()), padding_value, nullptr, TSX_ACT_NONE,
                                               0.f, out.data<float>(), m_workspace.data(), ws_bytes, current_stream()),
                  "tsx_conv2d_winograd_f23_nchw");
        else
            check(tsx_conv2d_winograd_f63_nchw(&g, x.data<float>(), static_cast<float *>(m_u.data()), padding_value, nullptr, TSX_ACT_NONE,
                                               0.f, out.data<float>(), m_workspace.data(), ws_bytes, current_stream()),
                  "tsx_conv2d_winograd_f63_nchw");
    }

protected:
    bool covers(Stack &stack) override { return format_is_nchw(*this) && inputs_are(stack, 2, FLOAT32); }

private:
    Tensor m_u;          // transformed kernel, [64 or 16][cout][cin], device memory
    Tensor m_workspace;
    WinogradConv2DMode m_mode = F6X6_3X3;
    int m_cout = 0, m_cin = 0;
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

protected:
    bool covers(Stack &stack) override { return inputs_are(stack, 2, FLOAT32); }
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

protected:
    bool covers(Stack &stack) override { return inputs_are(stack, 2, FLOAT32); }
};

class ReLU : public OperatorOnHip<base::Activation> {
public:
    void active(const Tensor &x, Tensor &out) override {
        if (x.dtype() != FLOAT32) TS_LOG_ERROR << this->op() << " not support data type: " << type_str(x.dtype()) << eject;
        check(tsx_relu_f32(x.data<float>(), x.count(), out.data<float>(), current_stream()), "tsx_relu_f32");
    }

protected:
    bool covers(Stack &stack) override { return inputs_are(stack, 1, FLOAT32); }
};

class LeakyReLU : public OperatorOnHip<base::LeakyReLU> {
public:
    void leaky_relu(const Tensor &x, float scale, Tensor &out) override {
        if (x.dtype() != FLOAT32) TS_LOG_ERROR << this->op() << " not support data type: " << type_str(x.dtype()) << eject;
        check(tsx_leaky_relu_f32(x.data<float>(), x.count(), scale, out.data<float>(), current_stream()), "tsx_leaky_relu_f32");
    }

protected:
    bool covers(Stack &stack) override { return inputs_are(stack, 1, FLOAT32); }
};

// ---------------------------------------------------------------- batch_norm / batch_scale / fused_batch_norm
// Graphs whose batch normalisation was not folded into the convolution carry these nodes behind it
// (src/kernels/cpu/batch_norm.cpp, batch_scale.cpp, fused_batch_norm.cpp; device classes
// src/kernels/gpu/batch_norm.cu, batch_scale.cu, fused_batch_norm.cu).  One HBM-bound pass each, the
// reference's roundings; other element types than fp32 run the host operator.
namespace {
void channel_layout(const Tensor &x, int dim, int64_t &pre, int64_t &inner) {
    pre = inner = 1;
    for (int i = 0; i < dim; ++i) pre *= x.size(size_t(i));
    for (size_t i = size_t(dim) + 1; i < x.dims(); ++i) inner *= x.size(i);
}
}  // namespace

class BatchNorm : public OperatorOnHip<base::BatchNorm> {
public:
    void batch_norm(const Tensor &x, const Tensor &mean, const Tensor &variance, int dim, float epsilon, Tensor &out) override {
        int64_t pre, inner;
        channel_layout(x, dim, pre, inner);
        check(tsx_batch_norm_f32(x.data<float>(), pre, x.size(size_t(dim)), inner, mean.data<float>(), variance.data<float>(),
                                 epsilon, out.data<float>(), current_stream()),
              "tsx_batch_norm_f32");
    }

protected:
    bool covers(Stack &stack) override { return inputs_are(stack, 3, FLOAT32); }
};

class BatchScale : public OperatorOnHip<base::BatchScale> {
public:
    void batch_scale(const Tensor &x, const Tensor &scale, const Tensor &bias, int dim, Tensor &out) override {
        int64_t pre, inner;
        channel_layout(x, dim, pre, inner);
        check(tsx_batch_scale_f32(x.data<float>(), pre, x.size(size_t(dim)), inner, scale.data<float>(), bias.data<float>(),
                                  out.data<float>(), current_stream()),
              "tsx_batch_scale_f32");
    }

protected:
    bool covers(Stack &stack) override { return inputs_are(stack, 3, FLOAT32); }
};

class FusedBatchNorm : public OperatorOnHip<base::FusedBatchNorm> {
public:
    void batch_norm(const Tensor &x, const Tensor &mean, const Tensor &variance, const Tensor &scale, const Tensor &bias, int dim,
                    float epsilon, Tensor &out) override {
        int64_t pre, inner;
        channel_layout(x, dim, pre, inner);
        check(tsx_fused_batch_norm_f32(x.data<float>(), pre, x.size(size_t(dim)), inner, mean.data<float>(),
                                       variance.data<float>(), scale.data<float>(), bias.data<float>(), epsilon,
                                       out.data<float>(), current_stream()),
              "tsx_fused_batch_norm_f32");
    }

protected:
    bool covers(Stack &stack) override { return inputs_are(stack, 5, FLOAT32); }
};

}  // namespace hip
}  // namespace ts

using namespace ts;
using namespace ts::hip;
TS_REGISTER_OPERATOR(Conv2D, ts::hip::DEVICE, name::layer::conv2d())
TS_REGISTER_OPERATOR(Conv2DWinograd, ts::hip::DEVICE, name::layer::conv2d_winograd())
TS_REGISTER_OPERATOR(InnerProd, ts::hip::DEVICE, name::layer::inner_prod())
TS_REGISTER_OPERATOR(AddBias, ts::hip::DEVICE, name::layer::add_bias())
TS_REGISTER_OPERATOR(ReLU, ts::hip::DEVICE, name::layer::relu())
TS_REGISTER_OPERATOR(LeakyReLU, ts::hip::DEVICE, "leaky_relu")
TS_REGISTER_OPERATOR(BatchNorm, ts::hip::DEVICE, "batch_norm")
TS_REGISTER_OPERATOR(BatchScale, ts::hip::DEVICE, "batch_scale")
TS_REGISTER_OPERATOR(FusedBatchNorm, ts::hip::DEVICE, "fused_batch_norm")
