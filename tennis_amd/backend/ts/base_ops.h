// Device-agnostic operator skeletons of the hot path, restating the reference's
// src/backend/base classes: parameter declaration and parsing in the constructor / init(),
// shape inference in infer(), and run() = infer + view inputs on the running memory device +
// push the output + call the pure-virtual device core.  A device backend overrides only the
// core method and running_memory_device(), exactly as with TenniS's own skeletons:
//   OperatorOnDevice      include/backend/base/operator_on_device.h:10-25
//   base::Quantize        src/backend/base/base_quantize.cpp:12-50
//   base::Conv2DQuantized src/backend/base/base_conv2d_quantized.cpp:13-219
//   base::Conv2D          src/backend/base/base_conv2d.cpp:17-207
//   base::Conv2DWinograd  src/backend/base/base_conv2d_winograd.cpp:15-169
//   base::InnerProd       src/backend/base/base_inner_prod.cpp:14-93
//   base::AddBias         src/backend/base/base_add_bias.cpp:15-90
//   base::Activation      src/backend/base/base_activation.cpp (relu), base_leaky_relu.cpp
#pragma once
#include "ts_api.h"

namespace ts {

class OperatorOnDevice : public Operator {
public:
    // the memory device the core method's tensors live on
    virtual MemoryDevice running_memory_device() = 0;
};

namespace base {

class Quantize : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    Quantize();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void quantize(const Tensor &x, std::vector<float> quantize_scales, Tensor &out) = 0;

protected:
    std::vector<float> m_quantize_scales;
};

// Shared parsing of format / padding / stride / dilation of the conv operators.
class Conv2DParams {
protected:
    void declare_conv_fields(Operator &op, bool with_stride);
    void parse_conv_fields(Operator &op, bool with_stride);
    Padding2D padding() const;
    Stride2D stride() const;
    Dilation2D dilation() const;
    Conv2DFormat m_format = FORMAT_NCHW;
    std::vector<int32_t> m_padding4x2, m_stride4, m_dilation4;
    float m_padding_value = 0;
};

class Conv2DQuantized : public OperatorOnDevice, protected Conv2DParams {
public:
    using supper = OperatorOnDevice;
    Conv2DQuantized();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void conv2d(const Tensor &x, const Padding2D &padding, float padding_value, const Tensor &w,
                        const Stride2D &stride, const Dilation2D &dilation, Conv2DFormat format,
                        std::vector<float> dequantize_scale, Tensor &out, Stack &stack) = 0;

protected:
    std::vector<float> m_dequantize_scales;
};

class Conv2D : public OperatorOnDevice, protected Conv2DParams {
public:
    using supper = OperatorOnDevice;
    Conv2D();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void conv2d(const Tensor &x, const Padding2D &padding, float padding_value, const Tensor &w,
                        const Stride2D &stride, const Dilation2D &dilation, Conv2DFormat format, Tensor &out,
                        Stack &stack, bool kernel_packed) = 0;

protected:
    bool m_kernel_packed = false;
};

class Conv2DWinograd : public OperatorOnDevice, protected Conv2DParams {
public:
    using supper = OperatorOnDevice;
    Conv2DWinograd();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void conv2d_tranform_kernel(WinogradConv2DMode mode, const Tensor &kernel, Tensor &kernel_transformed) = 0;
    virtual void conv2d_winograd(const Tensor &x, WinogradConv2DMode mode, const Padding2D &padding, float padding_value,
                                 const Tensor &w, Conv2DFormat format, Tensor &out, bool kernel_transformed) = 0;

protected:
    bool m_kernel_transformed = false;
    WinogradConv2DMode m_winograd_mode = F6X6_3X3;
    Tensor m_k_transformed;
};

// base::DepthwiseConv2D (include/backend/base/base_depthwise_conv2d.h:12): base::Conv2D with weights
// [1, C, KH, KW] and C * 1 output channels.
class DepthwiseConv2D : public Conv2D {
public:
    using supper = Conv2D;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
};

// base::Pooling2DCore / Pooling2D / GlobalPooling2D (include/backend/base/base_pooling2d_core.h:12-21,
// base_pooling2d.h:16-41, base_global_pooling2d.h:16)
class Pooling2DCore {
public:
    virtual ~Pooling2DCore() = default;
    virtual void pooling2d(const Tensor &x, Pooling2DType type, const Padding2D &padding, Padding2DType padding_type,
                           const Size2D &ksize, const Stride2D &stride, Conv2DFormat format, Tensor &out) = 0;
};

class Pooling2D : public OperatorOnDevice, public Pooling2DCore {
public:
    using supper = OperatorOnDevice;
    Pooling2D();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;

private:
    Conv2DFormat m_format = FORMAT_NCHW;
    Pooling2DType m_type = Pooling2DType::MAX;
    Padding2DType m_padding_type = Padding2DType::BLACK;
    std::vector<int32_t> m_padding4x2, m_ksize4, m_stride4;
};

class GlobalPooling2D : public OperatorOnDevice, public Pooling2DCore {
public:
    using supper = OperatorOnDevice;
    GlobalPooling2D();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;

private:
    Conv2DFormat m_format = FORMAT_NCHW;
    Pooling2DType m_type = Pooling2DType::MAX;
};

class InnerProd : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    InnerProd();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void inner_prod(const Tensor &lhs, const Tensor &rhs, bool transpose, Tensor &out, Stack &stack,
                            bool kernel_packed) = 0;

private:
    bool m_transpose = false;
    bool m_kernel_packed = false;
};

class AddBias : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    AddBias();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void add(const Tensor &x, const Tensor &b, int dim, Tensor &out) = 0;

private:
    bool check_inputs(Stack &stack) const;
    int m_dim = -1;
    std::string m_format;
};

// base::BatchNorm / BatchScale / FusedBatchNorm (src/backend/base/base_batch_norm.cpp, base_batch_scale.cpp,
// base_fused_batch_norm.cpp): one parameter vector per extent of axis `dim`, same dtype as x.
class BatchNorm : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    BatchNorm();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void batch_norm(const Tensor &x, const Tensor &mean, const Tensor &variance, int dim, float epsilon, Tensor &out) = 0;

private:
    float m_epsilon = 1e-5f;
    int m_dim = -1;
};

class BatchScale : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    BatchScale();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void batch_scale(const Tensor &x, const Tensor &scale, const Tensor &bias, int dim, Tensor &out) = 0;

private:
    int m_dim = -1;
};

class FusedBatchNorm : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    FusedBatchNorm();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void batch_norm(const Tensor &x, const Tensor &mean, const Tensor &variance, const Tensor &scale, const Tensor &bias,
                            int dim, float epsilon, Tensor &out) = 0;

private:
    float m_epsilon = 1e-5f;
    int m_dim = -1;
};

class Activation : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void active(const Tensor &x, Tensor &out) = 0;
};

class LeakyReLU : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    LeakyReLU();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void leaky_relu(const Tensor &x, float scale, Tensor &out) = 0;

private:
    float m_scale = 0;
};

// concat (src/backend/base/base_concat.cpp:13-130): inputs of one dtype and equal shape except along `dim`
// (negative counts from the end) joined along it.
class Concat : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    Concat();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void concat(const std::vector<Tensor> &x, int dim, Tensor &out) = 0;

private:
    int m_dim = 0;
};

// _resize2d (src/backend/base/base_resize2d.cpp:12-121): inputs x and an INT32 size vector with one entry per
// axis of x; the two neighbouring positive entries that differ from x's extents (or, all equal, the first
// positive pair) are the new height and width, -1 keeps an axis.
class Resize2D : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    Resize2D();
    void init() override;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    // axes dim and dim + 1 of x are resized to those of out
    virtual void resize2d(const Tensor &x, int dim, Resize2DType type, Tensor &out) = 0;

private:
    Resize2DType m_type = Resize2DType::LINEAR;
};

}  // namespace base

// ts::ElementWiseReduce (include/backend/base/element_wise_reduce.h:12-118; src/backend/base/
// element_wise_reduce.cpp): the skeleton of add / sub / mul / div.  Shapes are aligned, broadcast and
// collapsed as in the reference and the matching core method is called; this slice has no `_cast`
// operator, so operands of different dtype are rejected instead of up-cast.
class ElementWiseReduce : public OperatorOnDevice {
public:
    using supper = OperatorOnDevice;
    int run(Stack &stack) override;
    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override;
    virtual void reduce_with_broadcast(const Tensor &lhs, const Tensor &rhs, Tensor &out) = 0;
    virtual void reduce_with_same_shape(const Tensor &lhs, const Tensor &rhs, Tensor &out) { reduce_with_broadcast(lhs, rhs, out); }
    virtual void reduce_with_bias(const Tensor &lhs, const Tensor &rhs, Tensor &out, int) { reduce_with_broadcast(lhs, rhs, out); }
    virtual void reduce_with_scalar(const Tensor &lhs, const Tensor &rhs, Tensor &out) { reduce_with_broadcast(lhs, rhs, out); }
    virtual void reduce_with_bias_cross(const Tensor &lhs, const Tensor &rhs, Tensor &out, int) { reduce_with_broadcast(lhs, rhs, out); }
    virtual void reduce_with_scalar_cross(const Tensor &lhs, const Tensor &rhs, Tensor &out) { reduce_with_broadcast(lhs, rhs, out); }
    static bool reduce(Operator *op, Shape &lhs_shape, Shape &rhs_shape, Shape &out_shape, bool broadcast = true);
    static bool reduce_shape(Shape &lhs, Shape &rhs, Shape &out);
    static bool is_scalar(const Shape &shape);
    static bool is_bias(Shape &lhs_shape, Shape &rhs_shape, int &dim);
};

namespace base {
using Add = ElementWiseReduce;   // include/backend/base/base_add.h:12
using Mul = ElementWiseReduce;   // include/backend/base/base_mul.h
}
}  // namespace ts
