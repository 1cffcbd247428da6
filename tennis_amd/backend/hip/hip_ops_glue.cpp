// The "hip" device operators that sit between the convolutions of whole networks, so that a graph
// running on the device does not bounce through host memory between two convolutions: pooling2d,
// global_pooling2d, add (a residual join, with the general broadcast behind it) and depthwise_conv2d.
// Each class inherits TenniS's device-agnostic skeleton and implements the core method over the
// C ABI in include/tsx_hip.h, as TenniS's own device backends do (src/kernels/gpu/pooling2d.cu,
// add.cu, depthwise_conv2d.cu).
#define TSX_TS_GLUE_OPS
#include "hip_ops_common.h"

namespace ts {
namespace hip {

namespace {
// The pooling kernel works on [planes][h][w]: only NCHW maps fold into that.
void pool_nchw(const char *who, const Tensor &x, Pooling2DType type, const Padding2D &padding, Padding2DType padding_type,
               const Size2D &ksize, const Stride2D &stride, Conv2DFormat format, Tensor &out) {
    if (format != FORMAT_NCHW) TS_LOG_ERROR << who << " only support NCHW" << eject;
    if (x.dtype() != FLOAT32) TS_LOG_ERROR << who << " not support data type(" << x.dtype() << "): " << type_str(x.dtype()) << eject;
    if (type != Pooling2DType::MAX && type != Pooling2DType::AVG)
        TS_LOG_ERROR << who << " not support pooling type: " << int(type) << eject;
    // cpu::Pooling2DCore (src/kernels/cpu/pooling2d_core.cpp:48-186) knows BLACK and WHITE only
    if (padding_type != Padding2DType::BLACK && padding_type != Padding2DType::WHITE)
        TS_LOG_ERROR << who << " not support padding type: " << int(padding_type) << eject;
    check(tsx_pooling2d_f32(x.data<float>(), int64_t(x.size(0)) * x.size(1), x.size(2), x.size(3), int(type), padding.top,
                            padding.left, ksize.height, ksize.width, stride.height, stride.width,
                            padding_type == Padding2DType::WHITE ? 1 : 0, out.data<float>(), out.size(2), out.size(3),
                            current_stream()),
          "tsx_pooling2d_f32");
}
}  // namespace

class Pooling2D : public OperatorOnHip<base::Pooling2D> {
public:
    void pooling2d(const Tensor &x, Pooling2DType type, const Padding2D &padding, Padding2DType padding_type,
                   const Size2D &ksize, const Stride2D &stride, Conv2DFormat format, Tensor &out) override {
        pool_nchw("Pooling2D", x, type, padding, padding_type, ksize, stride, format, out);
    }

protected:
    // the kernel pools fp32 [planes][h][w] maps: NHWC graphs and other element types run the host operator
    bool covers(Stack &stack) override { return format_is_nchw(*this) && inputs_are(stack, 1, FLOAT32); }
};

class GlobalPooling2D : public OperatorOnHip<base::GlobalPooling2D> {
public:
    void pooling2d(const Tensor &x, Pooling2DType type, const Padding2D &padding, Padding2DType padding_type,
                   const Size2D &ksize, const Stride2D &stride, Conv2DFormat format, Tensor &out) override {
        pool_nchw("GlobalPooling2D", x, type, padding, padding_type, ksize, stride, format, out);
    }

protected:
    bool covers(Stack &stack) override { return format_is_nchw(*this) && inputs_are(stack, 1, FLOAT32); }
};

// add: equal shapes take the vectorised pass; every other case of ElementWiseReduce::run (scalar,
// bias along one axis, general broadcast, either operand) is one broadcast kernel, so the
// specialised hooks keep the skeleton's default (which forwards to reduce_with_broadcast).
class Add : public OperatorOnHip<base::Add> {
public:
    void reduce_with_same_shape(const Tensor &lhs, const Tensor &rhs, Tensor &out) override {
        check_type(out);
        check(tsx_add_f32(lhs.data<float>(), rhs.data<float>(), out.count(), TSX_ACT_NONE, 0.f, out.data<float>(), current_stream()),
              "tsx_add_f32");
    }

    void reduce_with_broadcast(const Tensor &lhs, const Tensor &rhs, Tensor &out) override {
        check_type(out);
        const Shape &ls = lhs.sizes(), &rs = rhs.sizes();
        if (ls.size() != rs.size() || ls.size() > 8)
            TS_LOG_ERROR << "[hip] add: can not broadcast " << to_string(ls) << " with " << to_string(rs) << eject;
        const std::vector<int32_t> l(ls.begin(), ls.end()), r(rs.begin(), rs.end());
        check(tsx_add_broadcast_f32(lhs.data<float>(), l.data(), rhs.data<float>(), r.data(), int32_t(l.size()), out.data<float>(),
                                    current_stream()),
              "tsx_add_broadcast_f32");
    }

protected:
    // the reference's device classes take every numeric type (src/kernels/gpu/add.cu:211-214); the kernels
    // here are fp32, anything else (an int32 index sum, fp64) runs the host operator
    bool covers(Stack &stack) override { return inputs_are(stack, 2, FLOAT32); }

private:
    static void check_type(const Tensor &out) {
        if (out.dtype() != FLOAT32) TS_LOG_ERROR << "[hip] add not support data type(" << out.dtype() << "): " << type_str(out.dtype()) << eject;
    }
};

// mul: as add, one IEEE multiplication per element.
class Mul : public OperatorOnHip<base::Mul> {
public:
    void reduce_with_same_shape(const Tensor &lhs, const Tensor &rhs, Tensor &out) override {
        check_type(out);
        check(tsx_mul_f32(lhs.data<float>(), rhs.data<float>(), out.count(), out.data<float>(), current_stream()), "tsx_mul_f32");
    }

    void reduce_with_broadcast(const Tensor &lhs, const Tensor &rhs, Tensor &out) override {
        check_type(out);
        const Shape &ls = lhs.sizes(), &rs = rhs.sizes();
        if (ls.size() != rs.size() || ls.size() > 8)
            TS_LOG_ERROR << "[hip] mul: can not broadcast " << to_string(ls) << " with " << to_string(rs) << eject;
        const std::vector<int32_t> l(ls.begin(), ls.end()), r(rs.begin(), rs.end());
        check(tsx_mul_broadcast_f32(lhs.data<float>(), l.data(), rhs.data<float>(), r.data(), int32_t(l.size()), out.data<float>(),
                                    current_stream()),
              "tsx_mul_broadcast_f32");
    }

protected:
    bool covers(Stack &stack) override { return inputs_are(stack, 2, FLOAT32); }

private:
    static void check_type(const Tensor &out) {
        if (out.dtype() != FLOAT32) TS_LOG_ERROR << "[hip] mul not support data type(" << out.dtype() << "): " << type_str(out.dtype()) << eject;
    }
};

// softplus and tanh: the two activations (with mul) that TenniS graphs compose Mish from
// (src/kernels/cpu/softplus.cpp:30-39, tanh.cpp:14-23).
class Softplus : public OperatorOnHip<base::Activation> {
public:
    void active(const Tensor &x, Tensor &out) override {
        if (x.dtype() != FLOAT32) TS_LOG_ERROR << "[hip] softplus not support data type: " << type_str(x.dtype()) << eject;
        check(tsx_softplus_f32(x.data<float>(), x.count(), out.data<float>(), current_stream()), "tsx_softplus_f32");
    }

protected:
    bool covers(Stack &stack) override { return inputs_are(stack, 1, FLOAT32); }
};

class Tanh : public OperatorOnHip<base::Activation> {
public:
    void active(const Tensor &x, Tensor &out) override {
        if (x.dtype() != FLOAT32) TS_LOG_ERROR << "[hip] tanh not support data type: " << type_str(x.dtype()) << eject;
        check(tsx_tanh_f32(x.data<float>(), x.count(), out.data<float>(), current_stream()), "tsx_tanh_f32");
    }

protected:
    bool covers(Stack &stack) override { return inputs_are(stack, 1, FLOAT32); }
};

// depthwise_conv2d: weights [1, C, KH, KW]; the core signature is base::Conv2D's.
class DepthwiseConv2D : public OperatorOnHip<base::DepthwiseConv2D> {
public:
    void conv2d(const Tensor &x, const Padding2D &padding, float padding_value, const Tensor &w, const Stride2D &stride,
                const Dilation2D &dilation, Conv2DFormat format, Tensor &out, Stack &, bool kernel_packed) override {
        if (format != FORMAT_NCHW) TS_LOG_ERROR << "DepthwiseConv2D only support NCHW" << eject;
        if (out.dtype() != FLOAT32)
            TS_LOG_ERROR << "DepthwiseConv2D not support data type(" << out.dtype() << "): " << type_str(out.dtype()) << eject;
        if (kernel_packed) TS_LOG_ERROR << "[hip] depthwise_conv2d expects [1, C, KH, KW] weights (kernel_packed=false)" << eject;
        tsx_conv2d_geom g = make_geom(x, w, padding, stride, dilation);
        g.cout = x.size(1);
        check(tsx_depthwise_conv2d_f32(&g, x.data<float>(), w.data<float>(), padding_value, nullptr, TSX_ACT_NONE, 0.f,
                                       out.data<float>(), current_stream()),
              "tsx_depthwise_conv2d_f32");
    }

protected:
    bool covers(Stack &stack) override { return format_is_nchw(*this) && inputs_are(stack, 2, FLOAT32); }
};

// concat along any axis: every input is one strided copy [outer][extent_i * inner] into its slot of the
// output rows (src/kernels/cpu/concat.cpp copies the same blocks with memcpy).  Elements of 4 bytes.
class Concat : public OperatorOnHip<base::Concat> {
public:
    void concat(const std::vector<Tensor> &x, int dim, Tensor &out) override {
        if (type_bytes(out.dtype()) != 4)
            TS_LOG_ERROR << "[hip] concat not support data type(" << out.dtype() << "): " << type_str(out.dtype()) << eject;
        int64_t outer = 1, inner = 1;
        for (int i = 0; i < dim; ++i) outer *= out.size(size_t(i));
        for (size_t i = size_t(dim) + 1; i < out.dims(); ++i) inner *= out.size(i);
        int32_t offset = 0;
        for (auto &t : x) {
            const int32_t extent = t.size(size_t(dim));
            if (extent > 0 && outer > 0 && inner > 0)
                check(tsx_concat_channels_f32(t.data<float>(), outer, extent, inner, out.data<float>(), out.size(size_t(dim)), offset,
                                              current_stream()),
                      "tsx_concat_channels_f32");
            offset += extent;
        }
    }

protected:
    // blocks of 4-byte elements; other element sizes (int8 maps, fp64) are concatenated by the host operator
    bool covers(Stack &stack) override {
        for (size_t i = 1; i < stack.size(); ++i)
            if (stack[int(i)].dtype() != stack[0].dtype()) return true;   // the skeleton rejects mixed types
        return stack.size() == 0 || type_bytes(stack[0].dtype()) == 4;
    }
};

// _resize2d: the nearest-neighbour mode on the two innermost axes (NCHW maps, the upsampling of detection necks).
class Resize2D : public OperatorOnHip<base::Resize2D> {
public:
    void resize2d(const Tensor &x, int dim, Resize2DType type, Tensor &out) override {
        if (type != Resize2DType::NEAREST)
            TS_LOG_ERROR << "[hip] _resize2d supports type NEAREST (2) only, got " << int(type) << eject;
        if (x.dtype() != FLOAT32) TS_LOG_ERROR << "[hip] _resize2d not support data type(" << x.dtype() << "): " << type_str(x.dtype()) << eject;
        if (size_t(dim) + 2 != x.dims()) TS_LOG_ERROR << "[hip] _resize2d resizes the two innermost axes only (NCHW)" << eject;
        int64_t planes = 1;
        for (int i = 0; i < dim; ++i) planes *= x.size(size_t(i));
        check(tsx_resize_nearest_f32(x.data<float>(), planes, x.size(size_t(dim)), x.size(size_t(dim) + 1), out.data<float>(),
                                     out.size(size_t(dim)), out.size(size_t(dim) + 1), current_stream()),
              "tsx_resize_nearest_f32");
    }

protected:
    // nearest-neighbour resizing of the two innermost axes of an fp32 tensor; the interpolating modes
    // (LINEAR, CUBIC, HARD) and other layouts run the host operator (src/kernels/cpu/resize2d.cpp)
    bool covers(Stack &stack) override {
        if (Resize2DType(tensor::to_int(get(name::type))) != Resize2DType::NEAREST) return false;
        if (stack.size() != 2 || stack[0].dtype() != FLOAT32) return false;
        std::vector<Tensor::Prototype> out;
        infer(stack, out);
        const Shape &from = stack[0].sizes(), &to = out[0].sizes();
        if (from.size() < 2 || from.size() != to.size()) return false;
        for (size_t i = 0; i + 2 < from.size(); ++i)
            if (from[i] != to[i]) return false;
        return true;
    }
};

}  // namespace hip
}  // namespace ts

using namespace ts;
using namespace ts::hip;
TS_REGISTER_OPERATOR(Pooling2D, ts::hip::DEVICE, name::layer::pooling2d())
TS_REGISTER_OPERATOR(GlobalPooling2D, ts::hip::DEVICE, name::layer::global_pooling2d())
TS_REGISTER_OPERATOR(Add, ts::hip::DEVICE, name::layer::add())
TS_REGISTER_OPERATOR(Mul, ts::hip::DEVICE, name::layer::mul())
TS_REGISTER_OPERATOR(Softplus, ts::hip::DEVICE, "softplus")
TS_REGISTER_OPERATOR(Tanh, ts::hip::DEVICE, "tanh")
TS_REGISTER_OPERATOR(DepthwiseConv2D, ts::hip::DEVICE, name::layer::depthwise_conv2d())
TS_REGISTER_OPERATOR(Concat, ts::hip::DEVICE, name::layer::concat())
TS_REGISTER_OPERATOR(Resize2D, ts::hip::DEVICE, name::layer::resize2d())
