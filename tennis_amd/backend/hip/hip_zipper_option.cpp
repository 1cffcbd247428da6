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

namespace {

bool is_activation(const std::string &op) { return op == name::layer::relu() || op == "leaky_relu"; }

// A chain  quantize -> conv2d_quantized [-> add_bias (channel axis, constant bias)] [-> relu | leaky_relu]
// matched backwards from its last node; the tensors inside it have no reader outside it.
struct Chain {
    std::vector<Node> nodes;         // quantize, conv2d_quantized, weights constant (Node has no empty state)
    const Node &quantize() const { return nodes[0]; }
    const Node &conv() const { return nodes[1]; }
    const Node &weights() const { return nodes[2]; }
    std::vector<Node> bias;          // empty or the add_bias node's constant
    std::string activation = "none";
    Tensor slope;

    // `tail` is the chain's last node; with allow_activation = false a trailing activation does not match
    bool match(Node tail, bool allow_activation) {
        Node cur = tail;
        const std::string op = cur.bubble().op();
        if (is_activation(op)) {
            if (!allow_activation || cur.inputs().size() != 1) return false;
            if (op == "leaky_relu") {
                if (!cur.bubble().has(name::scale)) return false;
                slope = cur.bubble().get(name::scale);
            }
            activation = op;
            cur = cur.input(0);
            if (cur.outputs().size() != 1) return false;       // someone else reads the tensor in front of the activation
        }
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
        nodes = {cur.input(0), cur, cur.input(1)};
        if (quantize().bubble().op() != name::layer::quantize() || quantize().inputs().size() != 1 ||
            weights().bubble().op() != Bubble::Const)
            return false;
        const Bubble &c = conv().bubble();
        if (!c.has(name::format) || tensor::to_string(c.get(name::format)) != name::NCHW) return false;
        // what the fused operator checks at run time, checked here where the graph shows it, so that a chain which
        // ran unfused is not turned into one that ejects: int8 OIHW weights, one float32 bias value per output
        // channel, and -- where the graph carries the inferred type -- a float32 tensor in front of the quantize
        if (!weights().bubble().has(name::value)) return false;
        const Tensor w = weights().bubble().get(name::value);
        if (w.dtype() != INT8 || w.dims() != 4) return false;
        if (!bias.empty()) {
            if (!bias[0].bubble().has(name::value)) return false;
            const Tensor b = bias[0].bubble().get(name::value);
            if (b.dtype() != FLOAT32 || b.count() != w.size(0)) return false;
        }
        const Bubble &source = quantize().input(0).bubble();
        if (source.has("#dtype") && DTYPE(tensor::to_int(source.get("#dtype"))) != FLOAT32) return false;
        return true;
    }
};

}  // namespace

class FusedQuantizedConvOption : public ZipperOption {
public:
    bool zip(const ComputingDevice &device, Node node, Node &zipped_node) const final {
        if (device.type() != DeviceType(DEVICE)) return false;
        // Three shapes of the same rewrite, all ending in `node`:
        //   chain                               -> fused(x, w[, bias])
        //   [relu | leaky_relu <-] add(chain without activation, other)   -> fused(..., other), residual = 1:
        //                                          the join of a residual block, act(y + other), in the epilogue
        //   add(chain with activation, other)   -> fused(..., other), residual = 2: act(y) + other (darknet shortcut)
        // `add` broadcasts; the fused operator adds an operand of the output's shape in the MFMA kernel's epilogue
        // and any other in a broadcast pass of its own, so every add that ran still runs.
        Chain chain;
        std::vector<Node> residual;
        int residual_mode = 0;
        std::string activation = "none";
        Tensor slope;
        Node cur = node;
        if (is_activation(cur.bubble().op()) && cur.inputs().size() == 1 && cur.input(0).bubble().op() == name::layer::add() &&
            cur.input(0).outputs().size() == 1) {
            activation = cur.bubble().op();
            if (activation == "leaky_relu") {
                if (!cur.bubble().has(name::scale)) return false;
                slope = cur.bubble().get(name::scale);
            }
            cur = cur.input(0);
        }
        if (cur.bubble().op() == name::layer::add() && cur.inputs().size() == 2) {
            for (int k = 0; k < 2 && !residual_mode; ++k) {
                Node candidate = cur.input(k), other = cur.input(1 - k);
                if (candidate.outputs().size() != 1 || candidate == other) continue;
                Chain c;
                if (!c.match(candidate, activation == "none")) continue;   // never two activations in one epilogue
                chain = c;
                residual.push_back(other);
                residual_mode = c.activation != "none" ? 2 : 1;
                if (residual_mode == 2) {
                    activation = c.activation;
                    slope = c.slope;
                }
            }
            if (!residual_mode) return false;
        } else {
            if (cur != node) return false;          // an activation behind an add that did not fold: not a chain's end
            if (!chain.match(node, true)) return false;
            activation = chain.activation;
            slope = chain.slope;
        }

        std::vector<Node> inputs = {chain.quantize().input(0), chain.weights()};
        inputs.insert(inputs.end(), chain.bias.begin(), chain.bias.end());
        inputs.insert(inputs.end(), residual.begin(), residual.end());
        zipped_node = bubble::op(node.bubble().name(), "conv2d_quantized_fused", inputs);
        Bubble &fused = zipped_node.bubble();
        const Bubble &conv = chain.conv().bubble();
        for (const std::string &param : {name::format, name::padding, name::padding_value, name::stride, name::dilation,
                                         name::typo::dialations, name::dequantize_scales})
            if (conv.has(param)) fused.set(param, conv.get(param));
        fused.set(name::quantize_scale, chain.quantize().bubble().get(name::quantize_scale));
        fused.set("activation", tensor::from(activation));
        if (activation == "leaky_relu") fused.set(name::scale, slope);
        if (residual_mode) fused.set("residual", tensor::from(int(residual_mode)));
        ++g_fused_chains;
        return true;
    }
};

}  // namespace hip
}  // namespace ts

TS_REGISTER_ZIPPER_OPTION(ts::hip::FusedQuantizedConvOption)
#endif  // TSX_WITH_TENNIS
