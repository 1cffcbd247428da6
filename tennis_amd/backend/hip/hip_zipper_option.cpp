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
#include <cstring>
#include <iterator>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "hip_device.h"

static std::atomic<long> g_fused_chains{0}, g_handovers{0}, g_dual_outputs{0};

// how many chains the option has replaced in this process (tests read it to see that the option fired)
extern "C" __attribute__((visibility("default"))) long tsx_hip_fused_chain_count() { return g_fused_chains.load(); }
// ... how many of them write a staged int8 output for the quantized convolutions behind them, and how many of
// those return the fp32 form as well (dual output)
extern "C" __attribute__((visibility("default"))) long tsx_hip_handover_count() { return g_handovers.load(); }
extern "C" __attribute__((visibility("default"))) long tsx_hip_dual_output_count() { return g_dual_outputs.load(); }

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
        return core(cur);
    }

    // the part of the match that does not depend on what follows the convolution: every conv2d_quantized node
    // that passes it ends up inside a fused node, whichever way the walker reaches it
    bool core(Node cur) {
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

// What ends at a node: a chain, or a chain joined with another tensor by an `add` (activation in front of or
// behind the add).  Three shapes of the same rewrite:
//   chain                               -> fused(x, w[, bias])
//   [relu | leaky_relu <-] add(chain without activation, other)   -> fused(..., other), residual = 1:
//                                          the join of a residual block, act(y + other), in the epilogue
//   add(chain with activation, other)   -> fused(..., other), residual = 2: act(y) + other (darknet shortcut)
// `add` broadcasts; the fused operator adds an operand of the output's shape in the MFMA kernel's epilogue
// and any other in a broadcast pass of its own, so every add that ran still runs.
struct Pattern {
    Chain chain;
    std::vector<Node> residual;
    int residual_mode = 0;
    std::string activation = "none";
    Tensor slope;

    bool match(Node node) {
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
            return residual_mode != 0;
        }
        if (cur != node) return false;          // an activation behind an add that did not fold: not a chain's end
        if (!chain.match(node, true)) return false;
        activation = chain.activation;
        slope = chain.slope;
        return true;
    }
};

// What a producer has to know about the chains that read its output to write their staged int8 input.
struct Next {
    Tensor quantize_scale, ksize, padding, stride, dilation, padding_value;
};

Tensor int_vector(std::initializer_list<int32_t> values) {
    const std::vector<int32_t> v(values);
    return tensor::build(INT32, Shape({int32_t(v.size())}), v.data());
}

bool same_values(const Tensor &a, const Tensor &b) {
    if (a.dtype() != b.dtype() || a.count() != b.count()) return false;
    const Tensor ha = a.view(MemoryDevice(CPU)), hb = b.view(MemoryDevice(CPU));
    return std::memcmp(ha.data(), hb.data(), size_t(a.count()) * type_bytes(a.dtype())) == 0;
}

// The consumer side of an int8 hand-over, from the chain's conv2d_quantized node; false when the layer cannot
// read a staged buffer a producer wrote (few input channels under a large kernel are staged by im2col).
bool describe(const Chain &chain, Next &next) {
    const Bubble &conv = chain.conv().bubble();
    const Tensor w = chain.weights().bubble().get(name::value);
    const int c = w.size(1), kh = w.size(2), kw = w.size(3);
    if (kh * kw > 1 && c <= 8 && c * kh * kw <= 512) return false;
    if (!conv.has(name::padding) || !conv.has(name::stride)) return false;
    if (!chain.quantize().bubble().has(name::quantize_scale)) return false;
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

// How the value of one original node is computed in the rewritten graph: by a conv2d_quantized_fused node
// whose output is the fp32 tensor (`plain`), the staged int8 input of the quantized convolutions that read it
// (`staged`), or both (a dual-output node behind two `_field` nodes).
struct Product {
    std::vector<Node> plain, staged;    // empty or one node
    std::vector<Node> staged_readers;   // the conv2d_quantized nodes that take the staged form
    bool alive() const {
        for (const Node &n : plain) if (n.ptr() == nullptr) return false;
        for (const Node &n : staged) if (n.ptr() == nullptr) return false;
        return !(plain.empty() && staged.empty());
    }
};

std::mutex g_memo_mutex;
// per graph under compilation (ctx Graph) and original node; entries of finished compilations hold expired nodes
std::unordered_map<const void *, std::unordered_map<Node, Product>> g_memo;

}  // namespace

class FusedQuantizedConvOption : public ZipperOption {
public:
    bool zip(const ComputingDevice &device, Node node, Node &zipped_node) const final {
        if (device.type() != DeviceType(DEVICE)) return false;
        std::lock_guard<std::mutex> lock(g_memo_mutex);
        Product product;
        if (!produce(node, product)) return false;
        if (!product.plain.empty()) {
            zipped_node = product.plain[0];
            return true;
        }
        // every reader seen in the graph takes the staged form, yet the walker asks for the tensor itself (a graph
        // output): a node of its own for the fp32 form
        Pattern p;
        if (!p.match(node)) return false;
        zipped_node = build(p, nullptr, false, node.bubble().name());
        return true;
    }

private:
    // The quantized convolutions that read `node` through a quantize node of their own (or a shared one), when
    // they can all read ONE staged buffer: the same quantize scale, kernel extent, padding, dilation and padding
    // value (strides may differ: a strided reader skips pixels of the same buffer), `next` from the reader with
    // the smallest stride, which must be 1 when strides differ.  `others` = whether anything else reads the node.
    static bool staged_readers(const Node &node, std::vector<Node> &convs, Next &next, bool &others) {
        convs.clear();
        others = false;
        std::vector<Next> all;
        for (const Node &reader : node.outputs()) {
            bool chains = reader.bubble().op() == name::layer::quantize() && reader.inputs().size() == 1 &&
                          !reader.outputs().empty();
            std::vector<Node> mine;
            std::vector<Next> mine_next;
            if (chains)
                for (const Node &conv : reader.outputs()) {
                    Chain c;
                    Next n;
                    if (!c.core(conv) || !describe(c, n)) {
                        chains = false;
                        break;
                    }
                    mine.push_back(conv);
                    mine_next.push_back(n);
                }
            if (!chains) {
                others = true;
                continue;
            }
            convs.insert(convs.end(), mine.begin(), mine.end());
            all.insert(all.end(), mine_next.begin(), mine_next.end());
        }
        if (convs.empty()) return false;
        size_t primary = 0;
        auto area = [](const Next &n) {
            const std::vector<int32_t> s = tensor::array::to_int(n.stride);
            return s[0] * s[1];
        };
        bool strides_differ = false;
        for (size_t i = 1; i < all.size(); ++i) {
            if (!same_values(all[i].quantize_scale, all[0].quantize_scale) || !same_values(all[i].ksize, all[0].ksize) ||
                !same_values(all[i].padding, all[0].padding) || !same_values(all[i].dilation, all[0].dilation) ||
                !same_values(all[i].padding_value, all[0].padding_value))
                return false;
            if (!same_values(all[i].stride, all[0].stride)) strides_differ = true;
            if (area(all[i]) < area(all[primary])) primary = i;
        }
        if (strides_differ && area(all[primary]) != 1) return false;
        next = all[primary];
        return true;
    }

    // Fills `product` for original node `node`; false when no fused node computes it.
    static bool produce(const Node &node, Product &product) {
        auto &memo = g_memo[ctx::get<Graph>()];
        for (auto it = memo.begin(); it != memo.end();)     // entries of an earlier compilation at this address
            it = (it->first.ptr() == nullptr || !it->second.alive()) ? memo.erase(it) : std::next(it);
        auto hit = memo.find(node);
        if (hit != memo.end()) {
            product = hit->second;
            return true;
        }
        if (node.bubble().op() == name::layer::pooling2d()) {
            Product pooled;
            if (!through_max_pooling(node, pooled)) return false;
            memo.insert(std::make_pair(node, pooled));
            product = pooled;
            return true;
        }
        Pattern p;
        if (!p.match(node)) return false;
        Next next;
        bool others = false;
        Product made;
        const std::string name = node.bubble().name();
        if (!staged_readers(node, made.staged_readers, next, others)) {
            made.plain.push_back(build(p, nullptr, false, name));
        } else if (!others) {
            made.staged.push_back(build(p, &next, false, name));
            ++g_handovers;
        } else {
            Node dual = build(p, &next, true, name);
            Node f32 = bubble::op(name, name::layer::field(), {dual});
            f32.bubble().set(name::offset, tensor::from(int(0)));
            Node i8 = bubble::op(name + "#staged", name::layer::field(), {dual});
            i8.bubble().set(name::offset, tensor::from(int(1)));
            made.plain.push_back(f32);
            made.staged.push_back(i8);
            ++g_handovers;
            ++g_dual_outputs;
        }
        memo.insert(std::make_pair(node, made));
        product = made;
        return true;
    }

    // pattern -> MAX pooling2d -> quantized convolutions only (a ResNet stem): quantize is monotone, so it commutes
    // with max -- the producer requantizes in its epilogue into a staged tensor without halo, max_pooling2d_staged
    // pools the int8 values straight into the convolutions' staged input.  Nothing else may read either tensor.
    static bool through_max_pooling(const Node &node, Product &made) {
        const Bubble &b = node.bubble();
        if (node.inputs().size() != 1) return false;
        for (const std::string &param : {name::format, name::type, name::padding, name::ksize, name::stride})
            if (!b.has(param)) return false;
        if (tensor::to_string(b.get(name::format)) != name::NCHW || tensor::to_int(b.get(name::type)) != 0) return false;
        const std::vector<int32_t> pad = tensor::array::to_int(b.get(name::padding));
        const std::vector<int32_t> ksize = tensor::array::to_int(b.get(name::ksize));
        const std::vector<int32_t> stride = tensor::array::to_int(b.get(name::stride));
        if (pad.size() != 8 || ksize.size() != 4 || stride.size() != 4) return false;
        if (pad[0] || pad[1] || pad[2] || pad[3] || ksize[0] != 1 || ksize[1] != 1 || stride[0] != 1 || stride[1] != 1) return false;
        if (pad[4] < 0 || pad[6] < 0 || pad[4] >= ksize[2] || pad[6] >= ksize[3] || stride[2] < 1 || stride[3] < 1) return false;
        Node source = node.input(0);
        if (source.outputs().size() != 1) return false;
        Pattern p;
        if (!p.match(source)) return false;
        Next next;
        bool others = false;
        if (!staged_readers(node, made.staged_readers, next, others) || others) return false;
        Next flat = next;                       // the producer's side: the same scale into [n][h][w][cp], no halo
        flat.ksize = int_vector({1, 1});
        flat.padding = int_vector({0, 0, 0, 0});
        flat.stride = int_vector({1, 1});
        flat.dilation = int_vector({1, 1});
        flat.padding_value = tensor::from(0.0f);
        Node producer = build(p, &flat, false, source.bubble().name());
        Node pool = bubble::op(node.bubble().name(), "max_pooling2d_staged", {producer});
        Bubble &staged = pool.bubble();
        staged.set(name::ksize, int_vector({ksize[2], ksize[3]}));
        staged.set(name::stride, int_vector({stride[2], stride[3]}));
        staged.set(name::padding, int_vector({pad[4], pad[5], pad[6], pad[7]}));
        staged.set("next_ksize", next.ksize);
        staged.set("next_padding", next.padding);
        staged.set("next_stride", next.stride);
        staged.set("next_dilation", next.dilation);
        staged.set("next_padding_value", next.padding_value);
        made.staged.push_back(pool);
        g_handovers += 2;
        return true;
    }

    // The conv2d_quantized_fused node for pattern `p`.  When the tensor in front of the chain's quantize is itself
    // computed by a fused node that hands this convolution its staged int8 input, that node is built here too (and
    // so on up the line): consecutive quantized convolutions exchange int8 in the consumer's layout, with no staging
    // pass and no fp32 tensor in between.
    static Node build(const Pattern &p, const Next *next, bool dual, const std::string &node_name) {
        const Chain &chain = p.chain;
        Node source = chain.quantize().input(0);
        bool staged_input = false;
        Product from;
        if (produce(source, from) && !from.staged.empty())
            for (const Node &reader : from.staged_readers)
                if (reader == chain.conv()) {
                    source = from.staged[0];
                    staged_input = true;
                }
        std::vector<Node> inputs = {source, chain.weights()};
        inputs.insert(inputs.end(), chain.bias.begin(), chain.bias.end());
        inputs.insert(inputs.end(), p.residual.begin(), p.residual.end());
        Node made = bubble::op(node_name, "conv2d_quantized_fused", inputs);
        Bubble &fused = made.bubble();
        const Bubble &conv = chain.conv().bubble();
        for (const std::string &param : {name::format, name::padding, name::padding_value, name::stride, name::dilation,
                                         name::typo::dialations, name::dequantize_scales})
            if (conv.has(param)) fused.set(param, conv.get(param));
        fused.set(name::quantize_scale, chain.quantize().bubble().get(name::quantize_scale));
        fused.set("activation", tensor::from(p.activation));
        if (p.activation == "leaky_relu") fused.set(name::scale, p.slope);
        if (p.residual_mode) fused.set("residual", tensor::from(int(p.residual_mode)));
        if (staged_input) fused.set("staged_input", tensor::from(int(1)));
        if (next) {
            fused.set("next_quantize_scale", next->quantize_scale);
            fused.set("next_ksize", next->ksize);
            fused.set("next_padding", next->padding);
            fused.set("next_stride", next->stride);
            fused.set("next_dilation", next->dilation);
            fused.set("next_padding_value", next->padding_value);
        }
        if (dual) fused.set("dual_output", tensor::from(int(1)));
        ++g_fused_chains;
        return made;
    }
};

}  // namespace hip
}  // namespace ts

TS_REGISTER_ZIPPER_OPTION(ts::hip::FusedQuantizedConvOption)
#endif  // TSX_WITH_TENNIS
