// See base_ops.h.  Error conditions and messages follow the reference's skeletons so that a
// graph which TenniS rejects at init()/infer() is rejected here for the same reason.
#include "base_ops.h"

#include <sstream>

namespace ts {
namespace base {

namespace {
std::string list(const std::vector<int32_t> &a) {
    std::ostringstream out;
    out << "[";
    for (size_t i = 0; i < a.size(); ++i) out << (i ? ", " : "") << a[i];
    out << "]";
    return out.str();
}

// RAII scratch frame: the core sees an empty stack and whatever it makes is dropped afterwards
// (base_conv2d.cpp:195-204).
struct ScratchFrame {
    explicit ScratchFrame(Stack &s, int base) : stack(s) {
        stack.push_base(base);
        TS_AUTO_CHECK(stack.size() == 0);
    }
    ~ScratchFrame() {
        stack.clear();
        stack.pop_base();
    }
    Stack &stack;
};
}  // namespace

// ---------------------------------------------------------------- quantize
Quantize::Quantize() { field(name::quantize_scale, REQUIRED); }

void Quantize::init() {
    supper::init();
    m_quantize_scales = tensor::array::to_float(get(name::quantize_scale));
}

int Quantize::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    TS_AUTO_CHECK(stack.size() == 1);
    auto &x = stack[0];
    TS_AUTO_CHECK(x.dims() >= 1);
    // one scale per first-dimension slice
    TS_AUTO_CHECK(int(m_quantize_scales.size()) == x.sizes()[0]);
    output.resize(1);
    output[0] = Tensor::Prototype(INT8, x.sizes());
    return 1;
}

int Quantize::run(Stack &stack) {
    std::vector<Tensor::Prototype> protos;
    infer(stack, protos);
    auto memory_device = running_memory_device();
    auto x = stack[0].view(memory_device);
    auto out = *stack.push(protos[0], memory_device);
    quantize(x, m_quantize_scales, out);
    return 1;
}

// ---------------------------------------------------------------- conv parameter block
void Conv2DParams::declare_conv_fields(Operator &op, bool with_stride) {
    op.field(name::format, Operator::REQUIRED);
    op.field(name::padding, Operator::REQUIRED);
    op.field(name::padding_value, Operator::OPTIONAL, tensor::from(0.0f));
    if (with_stride) {
        op.field(name::stride, Operator::REQUIRED);
        op.field(name::dilation, Operator::OPTIONAL);
        op.field(name::typo::dialations, Operator::OPTIONAL);
    }
}

void Conv2DParams::parse_conv_fields(Operator &op, bool with_stride) {
    auto format = tensor::to_string(op.get(name::format));
    auto padding_tensor = tensor::cast(INT32, op.get(name::padding));
    m_padding_value = tensor::to_float(op.get(name::padding_value));
    TS_AUTO_CHECK(padding_tensor.has_shape({4, 2}));
    if (format == name::NCHW) m_format = FORMAT_NCHW;
    else if (format == name::NHWC) m_format = FORMAT_NHWC;
    else TS_LOG_ERROR << op.op() << " do not support format: " << format << eject;
    m_padding4x2 = tensor::array::to_int(padding_tensor);
    m_stride4 = {1, 1, 1, 1};
    m_dilation4 = {1, 1, 1, 1};
    if (with_stride) {
        auto stride_tensor = tensor::cast(INT32, op.get(name::stride));
        Tensor dilation_tensor;
        if (op.has(name::dilation)) dilation_tensor = tensor::cast(INT32, op.get(name::dilation));
        else if (op.has(name::typo::dialations)) dilation_tensor = tensor::cast(INT32, op.get(name::typo::dialations));
        if (dilation_tensor.empty())
            TS_LOG_ERROR << op.op() << " must set " << name::dilation << " or " << name::typo::dialations << eject;
        TS_AUTO_CHECK(stride_tensor.has_shape({4}));
        TS_AUTO_CHECK(dilation_tensor.has_shape({4}));
        m_stride4 = tensor::array::to_int(stride_tensor);
        m_dilation4 = tensor::array::to_int(dilation_tensor);
    }
    // only the two spatial dimensions may be padded / strided / dilated
    const int n = 0, c = m_format == FORMAT_NCHW ? 1 : 3;
    if (m_padding4x2[2 * n] || m_padding4x2[2 * n + 1] || m_padding4x2[2 * c] || m_padding4x2[2 * c + 1])
        TS_LOG_ERROR << op.op() << " do not support padding: " << list(m_padding4x2) << eject;
    if (m_stride4[n] != 1 || m_stride4[c] != 1) TS_LOG_ERROR << op.op() << " do not support stride: " << list(m_stride4) << eject;
    if (m_dilation4[n] != 1 || m_dilation4[c] != 1)
        TS_LOG_ERROR << op.op() << " do not support dialations: " << list(m_dilation4) << eject;
}

Padding2D Conv2DParams::padding() const {
    const int h = m_format == FORMAT_NCHW ? 2 : 1;
    return Padding2D(m_padding4x2[2 * h], m_padding4x2[2 * h + 1], m_padding4x2[2 * h + 2], m_padding4x2[2 * h + 3]);
}
Stride2D Conv2DParams::stride() const {
    const int h = m_format == FORMAT_NCHW ? 2 : 1;
    return Stride2D(m_stride4[h], m_stride4[h + 1]);
}
Dilation2D Conv2DParams::dilation() const {
    const int h = m_format == FORMAT_NCHW ? 2 : 1;
    return Dilation2D(m_dilation4[h], m_dilation4[h + 1]);
}

namespace {
Tensor::Prototype conv_out_proto(DTYPE dtype, Conv2DFormat format, const Tensor &x, const Tensor &w, const Padding2D &padding,
                                 const Stride2D &stride, const Dilation2D &dilation) {
    const bool nchw = format == FORMAT_NCHW;
    Size2D xs(x.size(nchw ? 2 : 1), x.size(nchw ? 3 : 2));
    KSize2D ks(w.size(nchw ? 2 : 1), w.size(nchw ? 3 : 2));
    Size2D y = conv2d_forward(xs, padding, ks, stride, dilation);
    if (nchw) return Tensor::Prototype(dtype, {x.size(0), w.size(0), y.height, y.width});
    return Tensor::Prototype(dtype, {x.size(0), y.height, y.width, w.size(0)});
}
}  // namespace

// ---------------------------------------------------------------- conv2d_quantized
Conv2DQuantized::Conv2DQuantized() {
    declare_conv_fields(*this, true);
    field(name::dequantize_scales, REQUIRED);
}

void Conv2DQuantized::init() {
    supper::init();
    parse_conv_fields(*this, true);
    m_dequantize_scales = tensor::array::to_float(get(name::dequantize_scales));
}

int Conv2DQuantized::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    TS_AUTO_CHECK(stack.size() == 2);
    auto &x = stack[0];
    auto &w = stack[1];
    TS_AUTO_CHECK(x.dims() == 4);
    TS_AUTO_CHECK(w.dims() == 4);
    TS_AUTO_CHECK(x.dtype() == w.dtype());
    TS_AUTO_CHECK(w.size(1) == x.size(1));
    TS_AUTO_CHECK(x.dtype() == INT8);                                  // quantized input
    TS_AUTO_CHECK(int(m_dequantize_scales.size()) == w.size(0));       // one scale per output channel
    output.resize(1);
    output[0] = conv_out_proto(FLOAT32, m_format, x, w, padding(), stride(), dilation());   // no requantize: fp32 out
    return 1;
}

int Conv2DQuantized::run(Stack &stack) {
    std::vector<Tensor::Prototype> protos;
    infer(stack, protos);
    auto memory_device = running_memory_device();
    Tensor x = stack[0].view(memory_device);
    Tensor w = stack[1].view(memory_device);
    Tensor out = *stack.push(protos[0], memory_device);
    {
        ScratchFrame frame(stack, 3);
        conv2d(x, padding(), m_padding_value, w, stride(), dilation(), m_format, m_dequantize_scales, out, stack);
    }
    return 1;
}

// ---------------------------------------------------------------- conv2d
Conv2D::Conv2D() {
    declare_conv_fields(*this, true);
    field(name::kernel_packed, OPTIONAL, tensor::from<bool>(false));
}

void Conv2D::init() {
    supper::init();
    parse_conv_fields(*this, true);
    if (has(name::kernel_packed)) m_kernel_packed = tensor::to_bool(get(name::kernel_packed));
}

int Conv2D::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    TS_AUTO_CHECK(stack.size() == 2);
    auto &x = stack[0];
    auto &w = stack[1];
    TS_AUTO_CHECK(x.dims() == 4);
    TS_AUTO_CHECK(w.dims() == 4);
    TS_AUTO_CHECK(x.dtype() == w.dtype());
    if (w.size(1) != x.size(1))
        TS_LOG_ERROR << "Conv2D assert failed when x=" << to_string(x.sizes()) << ", w=" << to_string(w.sizes()) << eject;
    output.resize(1);
    output[0] = conv_out_proto(x.dtype(), m_format, x, w, padding(), stride(), dilation());
    return 1;
}

int Conv2D::run(Stack &stack) {
    std::vector<Tensor::Prototype> protos;
    infer(stack, protos);
    auto memory_device = running_memory_device();
    Tensor x = stack[0].view(memory_device);
    Tensor w = stack[1].view(memory_device);
    Tensor out = *stack.push(protos[0], memory_device);
    {
        ScratchFrame frame(stack, 3);
        conv2d(x, padding(), m_padding_value, w, stride(), dilation(), m_format, out, stack, m_kernel_packed);
    }
    return 1;
}

// ---------------------------------------------------------------- conv2d_winograd
Conv2DWinograd::Conv2DWinograd() {
    declare_conv_fields(*this, false);
    field(name::kernel_winograd_transformed, OPTIONAL, tensor::from<bool>(false));
}

void Conv2DWinograd::init() {
    supper::init();
    parse_conv_fields(*this, false);
    if (has(name::kernel_winograd_transformed)) m_kernel_transformed = tensor::to_bool(get(name::kernel_winograd_transformed));
}

int Conv2DWinograd::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    TS_AUTO_CHECK(stack.size() == 2);
    auto &x = stack[0];
    auto &k = stack[1];
    TS_AUTO_CHECK(x.dims() == 4);
    TS_AUTO_CHECK(k.dims() == 4);
    const bool nchw = m_format == FORMAT_NCHW;
    // 3x3, stride 1, dilation 1 whatever the kernel tensor's spatial extent says (it may hold
    // a transformed kernel)
    Size2D y = conv2d_forward(Size2D(x.size(nchw ? 2 : 1), x.size(nchw ? 3 : 2)), padding(), KSize2D(3, 3), Stride2D(1, 1),
                              Dilation2D(1, 1));
    output.resize(1);
    if (nchw) output[0] = Tensor::Prototype(x.dtype(), {x.size(0), k.size(0), y.height, y.width});
    else output[0] = Tensor::Prototype(x.dtype(), {x.size(0), y.height, y.width, k.size(0)});
    return 1;
}

// KernelCommonFunc<float>::winograd_mode_select_on_arm (src/kernels/common/function.cpp:154-173):
// F(6,3) only for Cin*Cout >= 256*256 on maps larger than 16x16, F(2,3) otherwise.
static WinogradConv2DMode select_winograd_mode(const Shape &input_shape, int out_channels) {
    const int input_channels = input_shape[1], input_height = input_shape[2], input_width = input_shape[3];
    if (input_channels * out_channels >= 256 * 256 && input_height > 16 && input_width > 16) return F6X6_3X3;
    return F2X2_3X3;
}

int Conv2DWinograd::run(Stack &stack) {
    std::vector<Tensor::Prototype> protos;
    infer(stack, protos);
    auto memory_device = running_memory_device();
    Tensor x = stack[0].view(memory_device);
    Tensor kernel = stack[1].view(memory_device);
    Tensor out = *stack.push(protos[0], memory_device);
    // first run: pick the mode and transform the incoming weights; the cache is empty on the first
    // run even when kernel_winograd_transformed was set, and the transformed-kernel tensor is a HOST
    // tensor whatever the device (base_conv2d_winograd.cpp:144-164) -- a device backend keeps its
    // own transformed copy and treats this tensor as opaque
    if (!m_kernel_transformed || m_k_transformed.empty()) {
        m_winograd_mode = select_winograd_mode(x.sizes(), kernel.size(0));
        const int tile = m_winograd_mode == F2X2_3X3 ? 4 : 8;
        m_k_transformed = Tensor(MemoryDevice(CPU), kernel.dtype(), Shape({kernel.size(0), kernel.size(1), tile, tile}));
        conv2d_tranform_kernel(m_winograd_mode, kernel, m_k_transformed);
        m_kernel_transformed = true;
    }
    conv2d_winograd(x, m_winograd_mode, padding(), m_padding_value, m_k_transformed, m_format, out, m_kernel_transformed);
    return 1;
}

// ---------------------------------------------------------------- depthwise_conv2d
int DepthwiseConv2D::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    supper::infer(stack, output);
    auto &x = stack[0];
    auto &w = stack[1];
    TS_AUTO_CHECK(w.size(0) == 1);
    Shape output_shape = output[0].sizes();
    output_shape[1] = x.size(1) * w.size(0);
    output[0] = Tensor::Prototype(output[0].dtype(), output_shape);
    return 1;
}

// ---------------------------------------------------------------- pooling2d / global_pooling2d
static std::string ints_str(const std::vector<int32_t> &v) {
    std::string s = "[";
    for (size_t i = 0; i < v.size(); ++i) s += (i ? ", " : "") + std::to_string(v[i]);
    return s + "]";
}

Pooling2D::Pooling2D() {
    field(name::format, REQUIRED);
    field(name::type, REQUIRED);
    field(name::padding, REQUIRED);
    field(name::padding_type, OPTIONAL, tensor::from(int(Padding2DType::BLACK)));
    field(name::ksize, REQUIRED);
    field(name::stride, REQUIRED);
}

void Pooling2D::init() {
    supper::init();
    const std::string format = tensor::to_string(get(name::format));
    m_type = static_cast<Pooling2DType>(tensor::to_int(get(name::type)));
    Tensor padding_tensor = tensor::cast(INT32, get(name::padding));
    m_padding_type = static_cast<Padding2DType>(tensor::to_int(get(name::padding_type)));
    Tensor ksize_tensor = tensor::cast(INT32, get(name::ksize));
    Tensor stride_tensor = tensor::cast(INT32, get(name::stride));
    TS_AUTO_CHECK(padding_tensor.has_shape({4, 2}));
    TS_AUTO_CHECK(ksize_tensor.has_shape({4}));
    TS_AUTO_CHECK(stride_tensor.has_shape({4}));
    if (format == name::NCHW) m_format = FORMAT_NCHW;
    else if (format == name::NHWC) m_format = FORMAT_NHWC;
    else TS_LOG_ERROR << this->op() << " do not support format: " << format << eject;
    m_padding4x2.assign(padding_tensor.data<int32_t>(), padding_tensor.data<int32_t>() + 8);
    m_ksize4.assign(ksize_tensor.data<int32_t>(), ksize_tensor.data<int32_t>() + 4);
    m_stride4.assign(stride_tensor.data<int32_t>(), stride_tensor.data<int32_t>() + 4);
    // only the two image axes may be pooled (base_pooling2d.cpp:66-98)
    const int a = m_format == FORMAT_NCHW ? 1 : 3;   // the channel axis
    if (m_padding4x2[0] || m_padding4x2[1] || m_padding4x2[2 * a] || m_padding4x2[2 * a + 1])
        TS_LOG_ERROR << this->op() << " do not support padding: " << ints_str(m_padding4x2) << eject;
    if (m_ksize4[0] != 1 || m_ksize4[a] != 1) TS_LOG_ERROR << this->op() << " do not support ksize: " << ints_str(m_ksize4) << eject;
    if (m_stride4[0] != 1 || m_stride4[a] != 1) TS_LOG_ERROR << this->op() << " do not support stride: " << ints_str(m_stride4) << eject;
}

int Pooling2D::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    TS_AUTO_CHECK(stack.size() == 1);
    auto &x_tensor = stack[0];
    TS_AUTO_CHECK(x_tensor.dims() == 4);
    const int hd = m_format == FORMAT_NCHW ? 2 : 1;
    const Size2D x(x_tensor.size(hd), x_tensor.size(hd + 1));
    const Size2D ksize(m_ksize4[hd], m_ksize4[hd + 1]);
    const Padding2D padding(m_padding4x2[2 * hd], m_padding4x2[2 * hd + 1], m_padding4x2[2 * hd + 2], m_padding4x2[2 * hd + 3]);
    const Stride2D stride(m_stride4[hd], m_stride4[hd + 1]);
    const Size2D y = pooling2d_forward(x, padding, ksize, stride);
    output.resize(1);
    if (m_format == FORMAT_NCHW) output[0] = Tensor::Prototype(x_tensor.dtype(), {x_tensor.size(0), x_tensor.size(1), y.height, y.width});
    else output[0] = Tensor::Prototype(x_tensor.dtype(), {x_tensor.size(0), y.height, y.width, x_tensor.size(3)});
    return 1;
}

int Pooling2D::run(Stack &stack) {
    std::vector<Tensor::Prototype> protos;
    infer(stack, protos);
    auto memory_device = running_memory_device();
    Tensor x = stack[0].view(memory_device);
    Tensor out = *stack.push(protos[0], memory_device);
    const int hd = m_format == FORMAT_NCHW ? 2 : 1;
    const Size2D ksize(m_ksize4[hd], m_ksize4[hd + 1]);
    const Padding2D padding(m_padding4x2[2 * hd], m_padding4x2[2 * hd + 1], m_padding4x2[2 * hd + 2], m_padding4x2[2 * hd + 3]);
    const Stride2D stride(m_stride4[hd], m_stride4[hd + 1]);
    pooling2d(x, m_type, padding, m_padding_type, ksize, stride, m_format, out);
    return 1;
}

GlobalPooling2D::GlobalPooling2D() {
    field(name::format, REQUIRED);
    field(name::type, REQUIRED);
}

void GlobalPooling2D::init() {
    supper::init();
    const std::string format = tensor::to_string(get(name::format));
    m_type = static_cast<Pooling2DType>(tensor::to_int(get(name::type)));
    if (format == name::NCHW) m_format = FORMAT_NCHW;
    else if (format == name::NHWC) m_format = FORMAT_NHWC;
    else TS_LOG_ERROR << this->op() << " do not support format: " << format << eject;
}

int GlobalPooling2D::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    TS_AUTO_CHECK(stack.size() == 1);
    auto &x = stack[0];
    TS_AUTO_CHECK(x.dims() == 4);
    output.resize(1);
    if (m_format == FORMAT_NCHW) output[0] = Tensor::Prototype(x.dtype(), {x.size(0), x.size(1), 1, 1});
    else output[0] = Tensor::Prototype(x.dtype(), {x.size(0), 1, 1, x.size(3)});
    return 1;
}

int GlobalPooling2D::run(Stack &stack) {
    std::vector<Tensor::Prototype> protos;
    infer(stack, protos);
    auto memory_device = running_memory_device();
    Tensor x = stack[0].view(memory_device);
    Tensor out = *stack.push(protos[0], memory_device);
    const int hd = m_format == FORMAT_NCHW ? 2 : 1;
    pooling2d(x, m_type, Padding2D(0, 0, 0, 0), Padding2DType::BLACK, Size2D(x.size(hd), x.size(hd + 1)), Stride2D(1, 1), m_format, out);
    return 1;
}

// ---------------------------------------------------------------- inner_prod
InnerProd::InnerProd() {
    field("transpose", OPTIONAL, tensor::from<bool>(false));
    field(name::kernel_packed, OPTIONAL, tensor::from<bool>(false));
}

void InnerProd::init() {
    supper::init();
    m_transpose = tensor::to_bool(get("transpose"));
    if (has(name::kernel_packed)) m_kernel_packed = tensor::to_bool(get(name::kernel_packed));
}

namespace {
void inner_prod_size(bool transpose, Tensor &lhs, const Tensor &rhs, std::vector<Tensor::Prototype> &output) {
    if (lhs.dims() == 0) TS_LOG_ERROR << "InnerProd failed with LHS is scalar." << eject;
    if (lhs.dims() != 2) lhs = lhs.reshape({lhs.size(0), -1});
    const bool ok = rhs.dims() == 2 && lhs.size(1) == (transpose ? rhs.size(1) : rhs.size(0));
    if (!ok)
        TS_LOG_ERROR << "Can not inner-product between " << to_string(lhs.sizes()) << " and " << to_string(rhs.sizes())
                     << (transpose ? "^T" : "") << eject;
    TS_AUTO_CHECK(lhs.dtype() == rhs.dtype());
    output.resize(1);
    output[0] = Tensor::Prototype(lhs.dtype(), {lhs.size(0), transpose ? rhs.size(0) : rhs.size(1)});
}
}  // namespace

int InnerProd::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    TS_AUTO_CHECK(stack.size() == 2);
    auto lhs = stack[0];
    inner_prod_size(m_transpose, lhs, stack[1], output);
    return 1;
}

int InnerProd::run(Stack &stack) {
    TS_AUTO_CHECK(stack.size() == 2);
    std::vector<Tensor::Prototype> output;
    auto lhs = stack[0];
    auto rhs = stack[1];
    inner_prod_size(m_transpose, lhs, rhs, output);
    auto memory_device = running_memory_device();
    lhs = lhs.view(memory_device);
    rhs = rhs.view(memory_device);
    auto &out = *stack.push(output[0], memory_device);
    inner_prod(lhs, rhs, m_transpose, out, stack, m_kernel_packed);
    return 1;
}

// ---------------------------------------------------------------- add_bias
AddBias::AddBias() {
    field(name::format, OPTIONAL);
    field(name::dim, OPTIONAL);
}

void AddBias::init() {
    supper::init();
    const bool has_format = has(name::format), has_dim = has(name::dim);
    TS_AUTO_CHECK(has_format || has_dim);
    if (has_format) {
        m_format = tensor::to_string(get(name::format));
        TS_AUTO_CHECK(m_format == name::NCHW || m_format == name::NHWC);
        m_dim = int(m_format.find('C'));
    }
    if (has_dim) m_dim = tensor::to_int(get(name::dim));
    TS_AUTO_CHECK(m_dim >= 0);
}

bool AddBias::check_inputs(Stack &stack) const {
    TS_AUTO_CHECK(stack.size() == 2);
    auto &x = stack[0];
    auto &b = stack[1];
    TS_AUTO_CHECK(m_dim < int(x.dims()));
    if (!b.has_shape(x.size(size_t(m_dim))))
        TS_LOG_ERROR << "Miss matched: x:" << to_string(x.sizes()) << ", dim=" << m_dim << ", b:" << to_string(b.sizes()) << eject;
    TS_AUTO_CHECK(x.dtype() == b.dtype());
    return true;
}

int AddBias::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    check_inputs(stack);
    output.resize(1);
    output[0] = stack[0].proto();
    return 1;
}

int AddBias::run(Stack &stack) {
    check_inputs(stack);
    auto memory_device = running_memory_device();
    auto x = stack[0].view(memory_device);
    auto b = stack[1].view(memory_device);
    auto &out = *stack.push(x.proto(), memory_device);
    add(x, b, m_dim, out);
    return 1;
}

// ---------------------------------------------------------------- batch_norm / batch_scale / fused_batch_norm
namespace {
// the checks of BatchNorm::check_inputs and its two siblings: `count` vectors of x.size(dim) values behind x
void check_channel_vectors(Stack &stack, size_t count, int dim, const char *const *names) {
    TS_AUTO_CHECK(stack.size() == count + 1);
    auto &x = stack[0];
    TS_AUTO_CHECK(dim < int(x.dims()));
    for (size_t i = 1; i <= count; ++i) {
        auto &v = stack[int(i)];
        if (!v.has_shape(x.size(size_t(dim))))
            TS_LOG_ERROR << "Miss matched: x:" << to_string(x.sizes()) << ", dim=" << dim << ", " << names[i - 1] << ":"
                         << to_string(v.sizes()) << eject;
    }
    for (size_t i = 1; i <= count; ++i) TS_AUTO_CHECK(x.dtype() == stack[int(i)].dtype());
}
const char *const kNormNames[] = {"mean", "variance", "scale", "bias"};
const char *const kScaleNames[] = {"scale", "bias"};
}  // namespace

BatchNorm::BatchNorm() {
    field(name::epsilon, OPTIONAL);
    field(name::dim, REQUIRED);
}

void BatchNorm::init() {
    supper::init();
    if (has(name::epsilon)) m_epsilon = tensor::to_float(get(name::epsilon));
    m_dim = tensor::to_int(get(name::dim));
    TS_AUTO_CHECK(m_dim >= 0);
}

int BatchNorm::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    check_channel_vectors(stack, 2, m_dim, kNormNames);
    output.assign(1, stack[0].proto());
    return 1;
}

int BatchNorm::run(Stack &stack) {
    check_channel_vectors(stack, 2, m_dim, kNormNames);
    auto memory_device = running_memory_device();
    auto x = stack[0].view(memory_device);
    auto mean = stack[1].view(memory_device);
    auto variance = stack[2].view(memory_device);
    auto out = *stack.push(x.proto(), memory_device);
    batch_norm(x, mean, variance, m_dim, m_epsilon, out);
    return 1;
}

BatchScale::BatchScale() { field(name::dim, REQUIRED); }

void BatchScale::init() {
    supper::init();
    m_dim = tensor::to_int(get(name::dim));
    TS_AUTO_CHECK(m_dim >= 0);
}

int BatchScale::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    check_channel_vectors(stack, 2, m_dim, kScaleNames);
    output.assign(1, stack[0].proto());
    return 1;
}

int BatchScale::run(Stack &stack) {
    check_channel_vectors(stack, 2, m_dim, kScaleNames);
    auto memory_device = running_memory_device();
    auto x = stack[0].view(memory_device);
    auto scale = stack[1].view(memory_device);
    auto bias = stack[2].view(memory_device);
    auto out = *stack.push(x.proto(), memory_device);
    batch_scale(x, scale, bias, m_dim, out);
    return 1;
}

FusedBatchNorm::FusedBatchNorm() {
    field(name::epsilon, OPTIONAL);
    field(name::dim, REQUIRED);
}

void FusedBatchNorm::init() {
    supper::init();
    if (has(name::epsilon)) m_epsilon = tensor::to_float(get(name::epsilon));
    m_dim = tensor::to_int(get(name::dim));
    TS_AUTO_CHECK(m_dim >= 0);
}

int FusedBatchNorm::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    check_channel_vectors(stack, 4, m_dim, kNormNames);
    output.assign(1, stack[0].proto());
    return 1;
}

int FusedBatchNorm::run(Stack &stack) {
    check_channel_vectors(stack, 4, m_dim, kNormNames);
    auto memory_device = running_memory_device();
    auto x = stack[0].view(memory_device);
    auto mean = stack[1].view(memory_device);
    auto variance = stack[2].view(memory_device);
    auto scale = stack[3].view(memory_device);
    auto bias = stack[4].view(memory_device);
    auto out = *stack.push(x.proto(), memory_device);
    batch_norm(x, mean, variance, scale, bias, m_dim, m_epsilon, out);
    return 1;
}

// ---------------------------------------------------------------- activations
int Activation::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    TS_AUTO_CHECK(stack.size() == 1);
    output.resize(1);
    output[0] = stack[0].proto();
    return 1;
}

int Activation::run(Stack &stack) {
    TS_AUTO_CHECK(stack.size() == 1);
    auto memory_device = running_memory_device();
    auto x = stack[0].view(memory_device);
    auto &out = *stack.push(x.proto(), memory_device);
    active(x, out);
    return 1;
}

LeakyReLU::LeakyReLU() { field(name::scale, REQUIRED); }

void LeakyReLU::init() {
    supper::init();
    m_scale = tensor::to_float(get(name::scale));
}

int LeakyReLU::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    TS_AUTO_CHECK(stack.size() == 1);
    output.resize(1);
    output[0] = stack[0].proto();
    return 1;
}

int LeakyReLU::run(Stack &stack) {
    TS_AUTO_CHECK(stack.size() == 1);
    auto memory_device = running_memory_device();
    auto x = stack[0].view(memory_device);
    auto &out = *stack.push(x.proto(), memory_device);
    leaky_relu(x, m_scale, out);
    return 1;
}

// ---------------------------------------------------------------- concat
Concat::Concat() { field(name::dim, REQUIRED); }

void Concat::init() {
    supper::init();
    m_dim = tensor::to_int(get(name::dim));
}

namespace {
[[noreturn]] void concat_mismatch(Stack &stack, int dim) {
    std::ostringstream oss;
    for (size_t j = 0; j < stack.size(); ++j)
        oss << (j ? ", " : "") << type_str(stack[j].dtype()) << ":" << to_string(stack[j].sizes());
    TS_LOG_ERROR << "Can not concat {" << oss.str() << "} at dim=" << dim << eject;
    throw Exception("unreachable");
}
}  // namespace

int Concat::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    const size_t inputs = stack.size();
    if (inputs == 0) TS_LOG_ERROR << "concat needs at least one input" << eject;
    output.resize(1);
    if (inputs == 1) {
        output[0] = stack[0].proto();
        return 1;
    }
    const DTYPE dtype = stack[0].dtype();
    Shape shape = stack[0].sizes();
    const int dims = int(shape.size());
    const int dim = m_dim >= 0 ? m_dim : dims + m_dim;
    if (dim < 0 || dim >= dims) TS_LOG_ERROR << "Concat dim must in [-" << dims << ", " << dims << ")" << eject;
    for (size_t i = 1; i < inputs; ++i) {
        const Tensor &t = stack[i];
        if (t.dtype() != dtype || int(t.dims()) != dims) concat_mismatch(stack, m_dim);
        for (int j = 0; j < dims; ++j)
            if (j != dim && t.size(size_t(j)) != shape[size_t(j)]) concat_mismatch(stack, m_dim);
        shape[size_t(dim)] += t.size(size_t(dim));
    }
    output[0] = Tensor::Prototype(dtype, shape);
    return 1;
}

int Concat::run(Stack &stack) {
    std::vector<Tensor::Prototype> protos;
    infer(stack, protos);
    const size_t inputs = stack.size();
    auto memory_device = running_memory_device();
    std::vector<Tensor> x;
    for (size_t i = 0; i < inputs; ++i) x.push_back(stack[i].view(memory_device));
    Tensor out = *stack.push(protos[0], memory_device);
    const int dims = int(x[0].dims());
    concat(x, m_dim >= 0 ? m_dim : dims + m_dim, out);
    return 1;
}

// ---------------------------------------------------------------- _resize2d
Resize2D::Resize2D() { field(name::type, OPTIONAL, tensor::from(int(Resize2DType::LINEAR))); }

void Resize2D::init() { m_type = Resize2DType(tensor::to_int(get(name::type))); }

namespace {
// The axis that becomes the new height (base_resize2d.cpp:27-63): the first positive entry of `size` that is
// not merely a copy of the extent with an unchanged tail behind the pair; -1 when the request is not a 2-D resize.
int resized_height_dim(const Shape &shape, const int32_t *size, int n) {
    int found = -1;
    for (int i = 0; i < n; ++i) {
        if (size[i] == 0) return -1;
        if (size[i] < 0) continue;
        if (shape[size_t(i)] == size[i]) {
            bool tail_kept = true;
            for (int j = i + 2; j < n && tail_kept; ++j) tail_kept = shape[size_t(j)] == size[j] || size[j] < 0;
            if (!tail_kept) continue;
        }
        found = i;
        break;
    }
    if (found < 0 || found >= n - 1 || size[found + 1] <= 0) return -1;
    for (int i = found + 2; i < n; ++i)
        if (size[i] == 0 || !(shape[size_t(i)] == size[i] || size[i] < 0)) return -1;
    return found;
}

Tensor::Prototype resized_proto(Stack &stack, int &dim, bool &same) {
    if (stack.size() != 2) TS_LOG_ERROR << "_resize2d expects 2 inputs (x, size), got " << stack.size() << eject;
    const Tensor &x = stack[0];
    Tensor size = tensor::cast(INT32, stack[1].view(MemoryDevice(CPU)));
    if (!(size.dims() == 1 && int(x.dims()) == size.size(0) && size.size(0) >= 2))
        TS_LOG_ERROR << "_resize2d: size must hold one entry per axis of x (at least 2)" << eject;
    const int n = size.size(0);
    const int32_t *data = size.data<int32_t>();
    dim = resized_height_dim(x.sizes(), data, n);
    if (dim < 0) TS_LOG_ERROR << "Can not resize " << to_string(x.sizes()) << " to " << to_string(Shape(std::vector<int32_t>(data, data + n))) << eject;
    Shape out = x.sizes();
    same = out[size_t(dim)] == data[dim] && out[size_t(dim) + 1] == data[dim + 1];
    out[size_t(dim)] = data[dim];
    out[size_t(dim) + 1] = data[dim + 1];
    return Tensor::Prototype(x.dtype(), out);
}
}  // namespace

int Resize2D::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    int dim;
    bool same;
    output.assign(1, resized_proto(stack, dim, same));
    return 1;
}

int Resize2D::run(Stack &stack) {
    int dim;
    bool same;
    const Tensor::Prototype proto = resized_proto(stack, dim, same);
    if (same) {   // nothing to resize: the input is the output
        const Tensor x = stack[0];
        stack.push(x);
        return 1;
    }
    auto memory_device = running_memory_device();
    Tensor x = stack[0].view(memory_device);
    Tensor out = *stack.push(proto, memory_device);
    resize2d(x, dim, m_type, out);
    return 1;
}

}  // namespace base

// ---------------------------------------------------------------- element-wise reduce (add ...)
bool ElementWiseReduce::reduce(Operator *op, Shape &_lhs_shape, Shape &_rhs_shape, Shape &_out_shape, bool broadcast) {
    if (_lhs_shape == _rhs_shape) {
        _out_shape = _lhs_shape;
        return false;
    }
    if (!broadcast)
        TS_LOG_ERROR << "[" << op->op() << ":" << op->name() << "] Can not reduce shape: " << to_string(_lhs_shape) << " vs. " << to_string(_rhs_shape) << eject;
    Shape lhs_shape = _lhs_shape, rhs_shape = _rhs_shape;
    while (lhs_shape.size() < rhs_shape.size()) lhs_shape.insert(lhs_shape.begin(), 1);
    while (rhs_shape.size() < lhs_shape.size()) rhs_shape.insert(rhs_shape.begin(), 1);
    const size_t dims = lhs_shape.size();
    Shape out_shape;
    out_shape.resize(dims);
    bool do_broadcast = false;
    for (size_t i = 0; i < dims; ++i) {
        int size = lhs_shape[i];
        if (lhs_shape[i] != rhs_shape[i]) {
            if (lhs_shape[i] != 1 && rhs_shape[i] != 1)
                TS_LOG_ERROR << "[" << op->op() << ":" << op->name() << "] Can not reduce shape: " << to_string(_lhs_shape) << " vs. " << to_string(_rhs_shape) << eject;
            do_broadcast = true;
            size = lhs_shape[i] * rhs_shape[i];
        }
        out_shape[i] = size;
    }
    _lhs_shape = lhs_shape;
    _rhs_shape = rhs_shape;
    _out_shape = out_shape;
    return do_broadcast;
}

static int shape_count(const Shape &s, size_t b, size_t e) {
    int c = 1;
    for (size_t i = b; i < e; ++i) c *= s[i];
    return c;
}

bool ElementWiseReduce::is_scalar(const Shape &shape) { return shape_count(shape, 0, shape.size()) == 1; }

bool ElementWiseReduce::is_bias(Shape &lhs_shape, Shape &rhs_shape, int &dim) {
    const int count = shape_count(rhs_shape, 0, rhs_shape.size());
    for (size_t i = 0; i < rhs_shape.size(); ++i)
        if (rhs_shape[i] == count && lhs_shape[i] == count) {
            dim = int(i);
            return true;
        }
    return false;
}

// collapses runs of axes on which both operands behave alike (element_wise_reduce.cpp:226-273)
bool ElementWiseReduce::reduce_shape(Shape &lhs, Shape &rhs, Shape &out) {
    bool reduced = false;
    for (size_t i = 0; i < out.size();) {
        bool lhs_ones = lhs[i] == 1, rhs_ones = rhs[i] == 1, same = lhs[i] == rhs[i];
        if (!(lhs_ones || rhs_ones || same)) {
            ++i;
            continue;
        }
        size_t j = i + 1;
        for (; j < out.size(); ++j) {
            if (lhs_ones) lhs_ones = lhs[j] == 1;
            if (rhs_ones) rhs_ones = rhs[j] == 1;
            if (same) same = lhs[j] == rhs[j];
            if (!(lhs_ones || rhs_ones || same)) break;
        }
        if (j - i > 1) {
            const int a = shape_count(lhs, i, j), b = shape_count(rhs, i, j), c = shape_count(out, i, j);
            lhs.erase(lhs.begin() + i, lhs.begin() + j);
            rhs.erase(rhs.begin() + i, rhs.begin() + j);
            out.erase(out.begin() + i, out.begin() + j);
            lhs.insert(lhs.begin() + i, a);
            rhs.insert(rhs.begin() + i, b);
            out.insert(out.begin() + i, c);
            reduced = true;
            ++i;
        } else {
            i = j + 1;
        }
    }
    return reduced;
}

int ElementWiseReduce::infer(Stack &stack, std::vector<Tensor::Prototype> &output) {
    TS_AUTO_CHECK(stack.size() == 2);
    auto &lhs = stack[0];
    auto &rhs = stack[1];
    if (lhs.dtype() != rhs.dtype())
        TS_LOG_ERROR << "[" << this->op() << ":" << this->name() << "] Can not reduce mismatch type: " << type_str(lhs.dtype())
                     << " vs. " << type_str(rhs.dtype()) << eject;
    Shape lhs_shape = lhs.sizes(), rhs_shape = rhs.sizes(), out_shape;
    reduce(this, lhs_shape, rhs_shape, out_shape, true);
    output.resize(1);
    output[0] = Tensor::Prototype(lhs.dtype(), out_shape);
    return 1;
}

int ElementWiseReduce::run(Stack &stack) {
    std::vector<Tensor::Prototype> output;
    infer(stack, output);
    Shape lhs_shape = stack[0].sizes(), rhs_shape = stack[1].sizes(), out_shape;
    const bool do_broadcast = reduce(this, lhs_shape, rhs_shape, out_shape, true);
    auto memory_device = running_memory_device();
    Tensor lhs = stack[0].view(memory_device).reshape(lhs_shape);
    Tensor rhs = stack[1].view(memory_device).reshape(rhs_shape);
    Tensor out = *stack.push(output[0], memory_device);
    if (reduce_shape(lhs_shape, rhs_shape, out_shape)) {
        lhs = lhs.reshape(lhs_shape);
        rhs = rhs.reshape(rhs_shape);
        out = out.reshape(out_shape);
    }
    int dim;
    if (!do_broadcast) reduce_with_same_shape(lhs, rhs, out);
    else if (is_scalar(rhs_shape)) reduce_with_scalar(lhs, rhs, out);
    else if (is_scalar(lhs_shape)) reduce_with_scalar_cross(lhs, rhs, out);
    else if (is_bias(lhs_shape, rhs_shape, dim)) reduce_with_bias(lhs, rhs, out, dim);
    else if (is_bias(rhs_shape, lhs_shape, dim)) reduce_with_bias_cross(lhs, rhs, out, dim);
    else reduce_with_broadcast(lhs, rhs, out);
    return 1;
}

}  // namespace ts
