// The "_v2" operators for device "hip": conv2d_v2, conv2d_winograd_v2, depthwise_conv2d_v2 and pooling2d_v2.
// A "_v2" operator receives what its plain twin takes as parameters (padding; for pooling also ksize and
// stride) as input tensors, because a graph computes them at run time (TensorFlow's SAME padding depends on
// the input size).  TenniS implements each as a wrapper that owns the plain operator of the current
// computing device and re-runs its init() whenever the dynamic values change
// (src/kernels/cpu/conv2d_v2.cpp:14-92, conv2d_winograd_v2.cpp:16-83, depthwise_conv2d_v2.cpp:14-92,
// pooling2d_v2.cpp:15-120), and registers those wrappers for its GPU device as they are
// (src/kernels/gpu/inherit_cpu.cpp:35-37).  Same here, as one class: the wrapped operators are this backend's.
#define TSX_TS_GLUE_OPS   // Pooling2DType / Padding2DType come with the pooling skeleton
#include "tsx_ts.h"
#include "hip_device.h"

#include <string>
#include <utility>
#include <vector>

namespace ts {
namespace hip {

class DynamicParamOperator : public Operator {
public:
    using self = DynamicParamOperator;
    using supper = Operator;

    // inner: the wrapped operator; dynamic: (input index, parameter name) pairs; the remaining inputs are the
    // wrapped operator's inputs, in order
    DynamicParamOperator(const char *v2_name, const char *inner, std::vector<std::pair<int, std::string>> dynamic, int inputs)
        : m_v2_name(v2_name), m_inner_name(inner), m_dynamic(std::move(dynamic)), m_inputs(inputs) {}

    void init() override {
        supper::init();
        auto &context = ctx::ref<DeviceContext>();
        m_inner = OperatorCreator::Create(context.computing_device.type(), m_inner_name, false);
        if (m_inner == nullptr) TS_LOG_ERROR << "Can not find operator: " << m_inner_name << eject;
        m_inner->set("#op", tensor::from(std::string(m_v2_name)));
        m_inner->set("#name", tensor::from("_core" + (has("#name") ? tensor::to_string(get("#name")) : std::string(m_v2_name))));
        for (auto &param : m_static)
            if (has(param)) m_inner->set(param, get(param));
        // the wrapped operator is new: it has none of the dynamic values yet
        m_values.assign(m_dynamic.size(), std::vector<int32_t>());
        m_known = false;
    }

    int infer(Stack &stack, std::vector<Tensor::Prototype> &output) override {
        update(stack);
        Frame frame(stack, forward_inputs(stack));
        const int returned = m_inner->infer(stack, output);
        stack.clear();
        return returned;
    }

    int run(Stack &stack) override {
        update(stack);
        Frame frame(stack, forward_inputs(stack));
        const int returned = m_inner->run(stack);
        if (int(stack.size()) < returned) TS_LOG_ERROR << m_inner_name << " returned fewer tensors than it reports" << eject;
        stack.erase(0, -returned);   // the arguments go, the results stay on top of the caller's frame
        return returned;
    }

protected:
    // a parameter handed on to the wrapped operator unchanged
    void forward(const std::string &param) { m_static.push_back(param); }

private:
    // RunOperator / InferOperator of the reference (src/runtime/operator.cpp:262-292): the last n entries
    // become the visible stack for the call
    struct Frame {
        Frame(Stack &s, int n) : stack(s) { stack.push_base(-n); }
        ~Frame() { stack.pop_base(); }
        Stack &stack;
    };

    bool is_dynamic(int input) const {
        for (auto &d : m_dynamic)
            if (d.first == input) return true;
        return false;
    }

    void update(Stack &stack) {
        if (int(stack.size()) != m_inputs) TS_LOG_ERROR << m_v2_name << " expects " << m_inputs << " inputs, got " << stack.size() << eject;
        bool changed = !m_known;
        std::vector<Tensor> now(m_dynamic.size());
        for (size_t i = 0; i < m_dynamic.size(); ++i) {
            now[i] = tensor::cast(INT32, stack[m_dynamic[i].first].view(MemoryDevice(CPU)));
            const int32_t *data = now[i].data<int32_t>();
            const std::vector<int32_t> values(data, data + now[i].count());
            if (values != m_values[i]) {
                m_values[i] = values;
                changed = true;
            }
        }
        if (!changed) return;
        for (size_t i = 0; i < m_dynamic.size(); ++i) m_inner->set(m_dynamic[i].second, now[i].clone());
        m_inner->init();
        m_known = true;
    }

    // pushes copies of the wrapped operator's inputs; returns how many
    int forward_inputs(Stack &stack) {
        int n = 0;
        for (int i = 0; i < m_inputs; ++i) {
            if (is_dynamic(i)) continue;
            const Tensor input = stack[i];
            stack.push(input);
            ++n;
        }
        return n;
    }

    const char *m_v2_name;
    const char *m_inner_name;
    std::vector<std::pair<int, std::string>> m_dynamic;
    int m_inputs;
    std::vector<std::string> m_static;
    Operator::shared m_inner;
    std::vector<std::vector<int32_t>> m_values;
    bool m_known = false;
};

// inputs: x, padding [4,2], w
class Conv2DV2 : public DynamicParamOperator {
public:
    explicit Conv2DV2(const char *v2_name = "conv2d_v2", const char *inner = "conv2d")
        : DynamicParamOperator(v2_name, inner, {{1, name::padding}}, 3) {
        field(name::format, REQUIRED);
        field(name::padding_value, OPTIONAL, tensor::from(0.0f));
        field(name::stride, REQUIRED);
        field(name::dilation, OPTIONAL);
        field(name::typo::dialations, OPTIONAL);
        field(name::kernel_packed, OPTIONAL, tensor::from<bool>(false));
        for (const std::string &p : std::vector<std::string>{name::format, name::padding_value, name::stride, name::dilation,
                                                              name::typo::dialations, name::kernel_packed})
            forward(p);
    }
};

class DepthwiseConv2DV2 : public Conv2DV2 {
public:
    DepthwiseConv2DV2() : Conv2DV2("depthwise_conv2d_v2", "depthwise_conv2d") {}
};

// inputs: x, padding [4,2], w
class Conv2DWinogradV2 : public DynamicParamOperator {
public:
    Conv2DWinogradV2() : DynamicParamOperator("conv2d_winograd_v2", "conv2d_winograd", {{1, name::padding}}, 3) {
        field(name::format, REQUIRED);
        field(name::padding_value, OPTIONAL, tensor::from(0.0f));
        field(name::kernel_winograd_transformed, OPTIONAL, tensor::from<bool>(false));
        for (const std::string &p : std::vector<std::string>{name::format, name::padding_value, name::kernel_winograd_transformed})
            forward(p);
    }
};

// inputs: x, padding [4,2], ksize [4], stride [4]
class Pooling2DV2 : public DynamicParamOperator {
public:
    Pooling2DV2()
        : DynamicParamOperator("pooling2d_v2", "pooling2d", {{1, name::padding}, {2, name::ksize}, {3, name::stride}}, 4) {
        field(name::format, REQUIRED);
        field(name::type, OPTIONAL, tensor::from(int(Pooling2DType::MAX)));
        field(name::padding_type, OPTIONAL, tensor::from(int(Padding2DType::BLACK)));
        for (const std::string &p : std::vector<std::string>{name::format, name::type, name::padding_type}) forward(p);
    }
};

}  // namespace hip
}  // namespace ts

using namespace ts;
using namespace ts::hip;
TS_REGISTER_OPERATOR(Conv2DV2, ts::hip::DEVICE, "conv2d_v2")
TS_REGISTER_OPERATOR(DepthwiseConv2DV2, ts::hip::DEVICE, "depthwise_conv2d_v2")
TS_REGISTER_OPERATOR(Conv2DWinogradV2, ts::hip::DEVICE, "conv2d_winograd_v2")
TS_REGISTER_OPERATOR(Pooling2DV2, ts::hip::DEVICE, "pooling2d_v2")
