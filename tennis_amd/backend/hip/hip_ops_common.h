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

// Packed weights and staging workspace of one quantized-convolution operator instance.
class PackedConv {
public:
    // The weights in MFMA operand order for geometry g: packed on first use, and again when another weight
    // tensor, weight shape or device shows up.  The operator keeps a reference to the tensor the pack was made
    // from: while it lives its address cannot be handed to a different tensor, so "same address and shape"
    // does mean "same weights" (weights are constant graph data, src/runtime/instruction.cpp:143-150).
    const void *packed(const tsx_conv2d_geom &g, const Tensor &w, const MemoryDevice &device, void *stream, const char *who) {
        const size_t bytes = tsx_conv2d_i8_packed_weight_bytes(&g);
        if (bytes == 0) TS_LOG_ERROR << "[hip] " << who << ": " << tsx_last_error() << eject;
        const bool same = !m_packed.empty() && m_bytes == bytes && m_packed.device() == device && !m_source.empty() &&
                          m_source.data() == w.data() && m_source.device() == w.device() && m_source.sizes() == w.sizes();
        if (!same) {
            m_packed = byte_tensor(device, bytes);
            check(tsx_conv2d_i8_pack_weights(&g, w.data<int8_t>(), m_packed.data(), stream), "tsx_conv2d_i8_pack_weights");
            m_source = w;
            m_bytes = bytes;
        }
        return m_packed.data();
    }

    // staging scratch for the activations: the context's shared buffer (nothing allocated in the steady state,
    // one buffer of the largest layer's size per context instead of one per operator)
    void *workspace(size_t bytes, const MemoryDevice &device) { return context_scratch(bytes ? bytes : 16, device, m_workspace); }

private:
    Tensor m_packed, m_source, m_workspace;
    size_t m_bytes = 0;
};

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
