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

        zipped_node = build(chain, activation, slope, residual, residual_mode, nullptr, node.bubble().name());
        return true;
    }

private:
    // What a producer has to know about the chain that reads its output to write that chain's staged int8 input.
    struct Next {
        Tensor quantize_scale, ksize, padding, stride, dilation, padding_value;
    };

    static Tensor int_vector(std::initializer_list<int32_t> values) {
        const std::vector<int32_t> v(values);
        return tensor::build(INT32, Shape({int32_t(v.size())}), v.data());
    }

    // The consumer side of an int8 hand-over, from the chain's conv2d_quantized node; false when the layer cannot
    // read a staged buffer a producer wrote (few input channels under a large kernel are staged by im2col).
    static bool describe(const Chain &chain, Next &next) {
        const Bubble &conv = chain.conv().bubble();
        const Tensor w = chain.weights().bubble().get(name::value);
        const int c = w.size(1), kh = w.size(2), kw = w.size(3);
        if (kh * kw > 1 && c <= 8 && c * kh * kw <= 512) return false;
        if (!conv.has(name::padding) || !conv.has(name::stride)) return false;
        const std::vector<int32_t> pad = tensor::array::to_int(conv.get(name::padding));
        const std::vector<int32_t> stride = tensor::array::to_int(conv.get(name::stride));
        const std::string dil_name = conv.has(name::dilation) ? name::dilation : name::typo::dialations;
        if (!conv.has(dil_name)) return false;
        const std::vector<int32_t> dil = tensor::array::to_int(conv.get(dil_name));
        if (pad.size() != 8 || stride.size() != 4 || dil.size() != 4) return false;
        next.quantize_scale = chain.quantize().bubble().get(name::quantize_scale);
        next.ksize = int_vector({kh, kw});
        next.padding = int_vector({pad[4], pad[5], pad[6], pad[7]});
        next.stride = int_vector({stride[2], stride[3]});
        next.dilation = int_vector({dil[2], dil[3]});
        next.padding_value = conv.has(name::padding_value) ? conv.get(name::padding_value) : tensor::from(0.0f);
        return true;
    }

    // The conv2d_quantized_fused node for `chain`.  When the tensor in front of the chain's quantize is itself the
    // end of a chain and nothing else reads it, that chain is built here too, as a producer that writes this one's
    // staged int8 input (and so on up the line): consecutive quantized convolutions exchange int8 in the consumer's
    // layout, with no staging pass and no fp32 tensor in between.
    static Node build(const Chain &chain, const std::string &activation, const Tensor &slope, const std::vector<Node> &residual,
                      int residual_mode, const Next *next, const std::string &node_name) {
        Node source = chain.quantize().input(0);
        bool staged_input = false;
        Next mine;
        Chain producer;
        if (chain.quantize().outputs().size() == 1 && source.outputs().size() == 1 && describe(chain, mine) &&
            producer.match(source, true)) {
            source = build(producer, producer.activation, producer.slope, {}, 0, &mine, source.bubble().name());
            staged_input = true;
        }
        std::vector<Node> inputs = {source, chain.weights()};
        inputs.insert(inputs.end(), chain.bias.begin(), chain.bias.end());
        inputs.insert(inputs.end(), residual.begin(), residual.end());
        Node made = bubble::op(node_name, "conv2d_quantized_fused", inputs);
        Bubble &fused = made.bubble();
        const Bubble &conv = chain.conv().bubble();
        for (const std::string &param : {name::format, name::padding, name::padding_value, name::stride, name::dilation,
                                         name::typo::dialations, name::dequantize_scales})
            if (conv.has(param)) fused.set(param, conv.get(param));
        fused.set(name::quantize_scale, chain.quantize().bubble().get(name::quantize_scale));
        fused.set("activation", tensor::from(activation));
        if (activation == "leaky_relu") fused.set(name::scale, slope);
        if (residual_mode) fused.set("residual", tensor::from(int(residual_mode)));
        if (staged_input) fused.set("staged_input", tensor::from(int(1)));
        if (next) {
            fused.set("next_quantize_scale", next->quantize_scale);
            fused.set("next_ksize", next->ksize);
            fused.set("next_padding", next->padding);
            fused.set("next_stride", next->stride);
            fused.set("next_dilation", next->dilation);
            fused.set("next_padding_value", next->padding_value);
        }
        ++g_fused_chains;
        return made;
    }
};

}  // namespace hip
}  // namespace ts

TS_REGISTER_ZIPPER_OPTION(ts::hip::FusedQuantizedConvOption)
#endif  // TSX_WITH_TENNIS
