// Shared by the "hip" operator translation units: geometry marshalling and a small cache for
// parameter vectors that the kernels read from device memory.
#pragma once
#include <vector>

#include "hip_device.h"
#include "tsx_hip.h"

namespace ts {
namespace hip {

inline tsx_conv2d_geom make_geom(const Tensor &x, const Tensor &w, const Padding2D &padding, const Stride2D &stride,
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

// Predicates for OperatorOnHip::covers: what the kernels behind a "hip" class take.
inline bool inputs_are(Stack &stack, size_t count, DTYPE dtype) {
    if (stack.size() < count) return true;   // let the skeleton report the wrong input count
    for (size_t i = 0; i < count; ++i)
        if (stack[int(i)].dtype() != dtype) return false;
    return true;
}

inline bool format_is_nchw(const Operator &op) {
    return !op.has(name::format) || tensor::to_string(op.get(name::format)) == name::NCHW;
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

}  // namespace hip
}  // namespace ts
