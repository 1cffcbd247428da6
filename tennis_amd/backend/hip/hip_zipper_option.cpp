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
            const Bubble &b = cur.bubble();
            const bool on_channels = (b.has(name::format) && tensor::to_string(b.get(name::format)) == name::NCHW) ||
                                     (b.has(name::dim) && tensor::to_int(b.get(name::dim)) == 1);
            if (!on_channels) return false;
            bias.push_back(cur.input(1));
            cur = cur.input(0);
            if (cur.outputs().size() != 1) return false;
        }
        if (cur.bubble().op() != name::layer::conv2d_quantized() || cur.inputs().size() != 2) return false;
        Node q = cur.input(0), w = cur.input(1);
        if (q.bubble().op() != name::layer::quantize() || q.inputs().size() != 1 || w.bubble().op() != Bubble::Const) return false;
        const Bubble &conv = cur.bubble();
        if (!conv.has(name::format) || tensor::to_string(conv.get(name::format)) != name::NCHW) return false;

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
