// A zipper option of TenniS's graph compiler for device "hip" (in-tree build only: it derives from
// ts::ZipperOption, include/compiler/option/zipper_option.h:13-38, and is walked by Zipper::zip,
// src/compiler/zipper.cpp:15-75, from the graph's outputs towards its inputs).  It replaces the END of a chain
//     quantize -> conv2d_quantized [-> add_bias (channel axis, constant bias)] [-> relu | leaky_relu]
// whose intermediate tensors have no other consumer by one conv2d_quantized_fused node (hip_ops_fused.cpp);
// the zipper then continues with that node's inputs (x, w, bias), so the chain's inner nodes drop out of the
// program.  The pattern is TenniS's own winograd option (src/compiler/option/winograd_zipper_option.cpp:16-96).
// tennis_amd/module_file.py holds the same rewrite for module graphs outside TenniS.
#ifdef TSX_WITH_TENNIS
#include <compiler/option/zipper_option.h>
#include <backend/name.h>
#include <core/tensor_builder.h>
#include <module/menu.h>

#include <atomic>
#include <string>
#include <vector>

#include "hip_device.h"

static std::atomic<long> g_fused_chains{0};

// how many chains the option has replaced in this process (tests read it to see that the option fired)
extern "C" __attribute__((visibility("default"))) long tsx_hip_fused_chain_count() { return g_fused_chains.load(); }

namespace ts {
namespace hip {

class FusedQuantizedConvOption : public ZipperOption {
public:
    bool zip(const ComputingDevice &device, Node node, Node &zipped_node) const final {
        if (device.type() != DeviceType(DEVICE)) return false;
        Node cur = node;
        std::string activation = "none";
        Tensor slope;
        const std::string tail = cur.bubble().op();
        if (tail == name::layer::relu() || tail == "leaky_relu") {
            if (cur.inputs().size() != 1) return false;
            if (tail == "leaky_relu") {
                if (!cur.bubble().has(name::scale)) return false;
                slope = cur.bubble().get(name::scale);
            }
            activation = tail;
            cur = cur.input(0);
            if (cur.outputs().size() != 1) return false;       // someone else reads the tensor in front of the activation
        }
        std::vector<Node> bias;      // empty or the add_bias node's constant
        if (cur.bubble().op() == name::layer::add_bias()) {
            if (cur.inputs().size() != 2 || cur.input(1).bubble().op() != Bubble::Const) return false;
            // the axis as AddBias::init resolves it (src/backend/base/base_add_bias.cpp:27-40): from the format's
            // 'C', overridden by dim when that is set too; the fused epilogue adds along the channel axis 1 only
            const Bubble &b = cur.bubble();
            int axis = -1;
            if (b.has(name::format)) {
                const std::string format = tensor::to_string(b.get(name::format));
                if (format != name::NCHW && format != name::NHWC) return false;
                axis = int(format.find('C'));
            }
            if (b.has(name::dim)) axis = tensor::to_int(b.get(name::dim));
            if (axis != 1) return false;
            bias.push_back(cur.input(1));
            cur = cur.input(0);
            if (cur.outputs().size() != 1) return false;
        }
        if (cur.bubble().op() != name::layer::conv2d_quantized() || cur.inputs().size() != 2) return false;
        Node q = cur.input(0), w = cur.input(1);
        if (q.bubble().op() != name::layer::quantize() || q.inputs().size() != 1 || w.bubble().op() != Bubble::Const) return false;
        const Bubble &conv = cur.bubble();
        if (!conv.has(name::format) || tensor::to_string(conv.get(name::format)) != name::NCHW) return false;
        // what the fused operator checks at run time, checked here where the graph shows it, so that a chain which
        // ran unfused is not turned into one that ejects: int8 OIHW weights, one float32 bias value per output
        // channel, and -- where the graph carries the inferred type -- a float32 tensor in front of the quantize
        if (!w.bubble().has(name::value)) return false;
        const Tensor weights = w.bubble().get(name::value);
        if (weights.dtype() != INT8 || weights.dims() != 4) return false;
        if (!bias.empty()) {
            if (!bias[0].bubble().has(name::value)) return false;
            const Tensor b = bias[0].bubble().get(name::value);
            if (b.dtype() != FLOAT32 || b.count() != weights.size(0)) return false;
        }
        const Bubble &source = q.input(0).bubble();
        if (source.has("#dtype") && DTYPE(tensor::to_int(source.get("#dtype"))) != FLOAT32) return false;

        std::vector<Node> inputs = {q.input(0), w};
        inputs.insert(inputs.end(), bias.begin(), bias.end());
        zipped_node = bubble::op(node.bubble().name(), "conv2d_quantized_fused", inputs);
        Bubble &fused = zipped_node.bubble();
        for (const std::string &param : {name::format, name::padding, name::padding_value, name::stride, name::dilation,
                                         name::typo::dialations, name::dequantize_scales})
            if (conv.has(param)) fused.set(param, conv.get(param));
        fused.set(name::quantize_scale, q.bubble().get(name::quantize_scale));
        fused.set("activation", tensor::from(activation));
        if (activation == "leaky_relu") fused.set(name::scale, slope);
        ++g_fused_chains;
        return true;
    }
};

}  // namespace hip
}  // namespace ts

TS_REGISTER_ZIPPER_OPTION(ts::hip::FusedQuantizedConvOption)
#endif  // TSX_WITH_TENNIS
