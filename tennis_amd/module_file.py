"""TenniS module files (`.tsm`): reader, writer and an operator-by-operator runner on device "hip".

Format (doc/zh_CN/module.md section 4; Module::Save / Module::Load, src/module/module.cpp:236-320; nodes
src/module/menu.cpp:88-122; parameters src/module/bubble.cpp:140-189), all little-endian:

    header   uint32 fake, uint32 code = 0x19910929, 120 reserved bytes
    inputs   uint32 n, uint32 node index * n
    outputs  uint32 n, uint32 node index * n
    graph    uint32 n, then per node:
               bubble   uint32 params, per parameter: uint32 name length, name, a packed tensor (tensor_file)
               inputs   uint32 n, uint32 node index * n

A node's operator and name are the retention parameters "#op" and "#name"; "<param>" nodes are the module's
inputs, "<const>" nodes carry their tensor in parameter "value".

`run_module` evaluates the graph in dependency order, one `operators.run_op` per node, on the device's own
operator classes: it is the counterpart of loading the module into a Workbench of ComputingDevice("hip"), without
TenniS's graph compiler (no operator fusion, no constant folding; every node must be an operator the device
registers -- there is no host fallback).
"""
import struct

import numpy as np

from . import operators, tensor_file

MODULE_CODE_V1 = 0x19910929
PARAMETER, CONST = "<param>", "<const>"


class ModuleFileError(ValueError):
    pass


class Node:
    def __init__(self, op, name, params=None, inputs=()):
        self.op, self.name = op, name
        self.params = dict(params or {})   # without the "#op" / "#name" retention parameters
        self.inputs = list(inputs)         # node indices

    def __repr__(self):
        return "Node(%r, %r, inputs=%r)" % (self.op, self.name, self.inputs)


class Module:
    def __init__(self, nodes, inputs, outputs):
        self.nodes, self.inputs, self.outputs = list(nodes), list(inputs), list(outputs)


def _u32(buf, pos, what):
    if pos + 4 > len(buf):
        raise ModuleFileError("truncated module file: %s at offset %d" % (what, pos))
    return struct.unpack_from("<I", buf, pos)[0], pos + 4


def _index_list(buf, pos, what, limit=None):
    n, pos = _u32(buf, pos, what)
    out = []
    for _ in range(n):
        v, pos = _u32(buf, pos, what)
        if limit is not None and v >= limit:
            raise ModuleFileError("%s: node index %d out of range (%d nodes)" % (what, v, limit))
        out.append(v)
    return out, pos


def _packed_tensor(buf, pos):
    """One serialized (packed) tensor starting at pos; returns (value, end)."""
    fields, p = _u32(buf, pos, "tensor field count")
    for _ in range(fields):
        if p + 5 > len(buf):
            raise ModuleFileError("truncated module file: tensor prototype at offset %d" % p)
        code, ndims = struct.unpack_from("<BI", buf, p)
        p += 5
        if p + 4 * ndims > len(buf):
            raise ModuleFileError("truncated module file: tensor sizes at offset %d" % p)
        shape = struct.unpack_from("<%dI" % ndims, buf, p)
        p += 4 * ndims
        if code not in tensor_file._TS2NP:
            raise ModuleFileError("tensor dtype code %d has no fixed-size element" % code)
        p += int(np.prod(shape, dtype=np.int64)) * np.dtype(tensor_file._TS2NP[code]).itemsize
    if p > len(buf):
        raise ModuleFileError("truncated module file: tensor data runs past the end")
    vals = [tensor_file._value(c, a) for c, a in tensor_file.parse_fields(bytes(buf[pos:p]))]
    return (vals[0] if len(vals) == 1 else vals), p


def parse_module(buf):
    if len(buf) < 128:
        raise ModuleFileError("truncated module file: no header")
    _, code = struct.unpack_from("<II", buf, 0)
    if code != MODULE_CODE_V1:
        raise ModuleFileError("module code 0x%08x is not format V1 (0x%08x)" % (code, MODULE_CODE_V1))
    pos = 128
    inputs, pos = _index_list(buf, pos, "module inputs")
    outputs, pos = _index_list(buf, pos, "module outputs")
    count, pos = _u32(buf, pos, "node count")
    nodes = []
    for i in range(count):
        nparams, pos = _u32(buf, pos, "parameter count of node %d" % i)
        params = {}
        for _ in range(nparams):
            n, pos = _u32(buf, pos, "parameter name length")
            if pos + n > len(buf):
                raise ModuleFileError("truncated module file: parameter name at offset %d" % pos)
            name = bytes(buf[pos:pos + n]).decode()
            pos += n
            params[name], pos = _packed_tensor(buf, pos)
        node_inputs, pos = _index_list(buf, pos, "inputs of node %d" % i, count)
        if "#op" not in params or "#name" not in params:
            raise ModuleFileError("node %d has no #op / #name" % i)
        nodes.append(Node(params.pop("#op"), params.pop("#name"), params, node_inputs))
    for what, idx in (("input", inputs), ("output", outputs)):
        for v in idx:
            if v >= count:
                raise ModuleFileError("module %s index %d out of range (%d nodes)" % (what, v, count))
    if pos != len(buf):
        raise ModuleFileError("%d bytes behind the graph" % (len(buf) - pos))
    return Module(nodes, inputs, outputs)


def read_module(path):
    with open(path, "rb") as fh:
        return parse_module(fh.read())


def serialize_module(module):
    out = [struct.pack("<II", 0, MODULE_CODE_V1), bytes(120)]
    for idx in (module.inputs, module.outputs):
        out.append(struct.pack("<I%dI" % len(idx), len(idx), *idx))
    out.append(struct.pack("<I", len(module.nodes)))
    for node in module.nodes:
        params = dict(node.params)
        params["#op"], params["#name"] = node.op, node.name
        out.append(struct.pack("<I", len(params)))
        for name in sorted(params):          # TenniS keeps parameters in an ordered map
            raw = name.encode()
            out.append(struct.pack("<I", len(raw)) + raw + tensor_file.serialize(params[name]))
        out.append(struct.pack("<I%dI" % len(node.inputs), len(node.inputs), *node.inputs))
    return b"".join(out)


def write_module(path, module):
    with open(path, "wb") as fh:
        fh.write(serialize_module(module))


def run_module(module, feeds, device="hip", device_id=0):
    """Outputs of ``module`` for ``feeds`` (one array per module input, in the module's input order)."""
    if len(feeds) != len(module.inputs):
        raise ModuleFileError("module has %d inputs, %d fed" % (len(module.inputs), len(feeds)))
    values = {i: np.asarray(v) for i, v in zip(module.inputs, feeds)}
    entered = set()              # nodes whose inputs are being evaluated (cycle detection)
    stack = list(reversed(module.outputs))
    while stack:                 # depth-first without recursion: graphs are hundreds of nodes deep
        i = stack[-1]
        if i in values:
            stack.pop()
            continue
        node = module.nodes[i]
        if node.op == PARAMETER:
            raise ModuleFileError("input node %r (%d) is not among the module's inputs" % (node.name, i))
        if node.op == CONST:
            if "value" not in node.params:
                raise ModuleFileError("<const> node %r has no value" % node.name)
            values[i] = np.asarray(node.params["value"])
            stack.pop()
            continue
        missing = [j for j in node.inputs if j not in values]
        if missing:
            if i in entered:
                raise ModuleFileError("the graph has a cycle through node %d" % i)
            entered.add(i)
            stack.extend(reversed(missing))
            continue
        params = {k: v for k, v in node.params.items() if not k.startswith("#")}
        values[i] = operators.run_op(node.op, params, [values[j] for j in node.inputs], device=device, device_id=device_id)
        stack.pop()
    return [values[i] for i in module.outputs]


FUSED = "conv2d_quantized_fused"


def fuse_quantized_chains(module):
    """The graph rewrite for device "hip": every chain

        quantize -> conv2d_quantized [-> add_bias (channel axis, constant bias)] [-> relu | leaky_relu]

    whose intermediate tensors have no other consumer becomes one `conv2d_quantized_fused` node (two kernels
    instead of up to four operators exchanging fp32 / int8 tensors; same values bit for bit), and an `add` that joins
    such a chain to another tensor -- with the activation behind it -- moves into the node's epilogue as well.  A quantize node that
    feeds several convolutions is folded into each of them.  Returns a new Module without the dead nodes; TenniS's
    counterpart of such a pass is a zipper option of its graph compiler
    (src/compiler/option/winograd_zipper_option.cpp:16-96)."""
    nodes = [Node(n.op, n.name, n.params, n.inputs) for n in module.nodes]
    users = {}
    for i, n in enumerate(nodes):
        for j in n.inputs:
            users.setdefault(j, []).append(i)
    for j in module.outputs:
        users.setdefault(j, []).append(-1)

    def only_user(i, op):
        u = users.get(i, [])
        return u[0] if len(u) == 1 and u[0] >= 0 and nodes[u[0]].op == op and nodes[u[0]].inputs[0] == i else None

    for ci, conv in enumerate(list(nodes)):
        if conv.op != "conv2d_quantized" or len(conv.inputs) != 2:
            continue
        q = nodes[conv.inputs[0]]
        if q.op != "quantize" or len(q.inputs) != 1 or nodes[conv.inputs[1]].op != CONST:
            continue
        params = dict(conv.params)
        params["quantize_scale"] = q.params["quantize_scale"]
        inputs = [q.inputs[0], conv.inputs[1]]
        last = ci
        bi = only_user(last, "add_bias")
        if bi is not None:
            b = nodes[bi]
            # the axis as AddBias::init resolves it (src/backend/base/base_add_bias.cpp:27-40): from the format's 'C',
            # overridden by dim when that is set too; the fused epilogue adds along the channel axis 1 only
            axis = -1
            fmt = b.params.get("format")
            if isinstance(fmt, bytes):
                fmt = fmt.decode()
            if fmt in ("NCHW", "NHWC"):
                axis = fmt.index("C")
            if "dim" in b.params:
                axis = int(np.asarray(b.params["dim"]).ravel()[0])
            bias_ok = False
            if len(b.inputs) == 2 and nodes[b.inputs[1]].op == CONST:
                value = np.asarray(nodes[b.inputs[1]].params.get("value"))
                wvalue = np.asarray(nodes[conv.inputs[1]].params.get("value"))
                bias_ok = value.dtype == np.float32 and wvalue.ndim == 4 and value.size == wvalue.shape[0]
            if bias_ok and axis == 1 and (fmt is None or fmt in ("NCHW", "NHWC")):
                inputs.append(b.inputs[1])
                last = bi
        ai = only_user(last, "relu")
        if ai is not None:
            params["activation"] = "relu"
            last = ai
        else:
            ai = only_user(last, "leaky_relu")
            if ai is not None and "scale" in nodes[ai].params:
                params["activation"] = "leaky_relu"
                params["scale"] = nodes[ai].params["scale"]
                last = ai
        # the fused node takes the place of the chain's last node, so its consumers keep their links
        nodes[last] = Node(FUSED, nodes[last].name, params, inputs)
    # second pass: an `add` that joins a fused chain to another tensor (the residual join of a ResNet block, a darknet
    # shortcut) moves into that chain's epilogue, with the activation behind it:
    #   [relu | leaky_relu <-] add(chain without activation, other) -> residual = 1: act(y + other)
    #   add(chain with activation, other)                          -> residual = 2: act(y) + other
    users = {}
    for i, n in enumerate(nodes):
        for j in n.inputs:
            users.setdefault(j, []).append(i)
    for j in module.outputs:
        users.setdefault(j, []).append(-1)
    for ai, add in enumerate(list(nodes)):
        if add.op != "add" or len(add.inputs) != 2:
            continue
        for k in (0, 1):
            ci, other = add.inputs[k], add.inputs[1 - k]
            cand = nodes[ci]
            if cand.op != FUSED or users.get(ci) != [ai] or ci == other or "residual" in cand.params:
                continue
            params = dict(cand.params)
            last = ai
            if params.get("activation", "none") != "none":
                params["residual"] = np.array([2], np.int32)
            else:
                params["residual"] = np.array([1], np.int32)
                act = only_user(ai, "relu")
                if act is not None:
                    params["activation"] = "relu"
                    last = act
                else:
                    act = only_user(ai, "leaky_relu")
                    if act is not None and "scale" in nodes[act].params:
                        params["activation"] = "leaky_relu"
                        params["scale"] = nodes[act].params["scale"]
                        last = act
            nodes[last] = Node(FUSED, nodes[last].name, params, list(cand.inputs) + [other])
            break
    # third pass: a fused node whose output only another fused node reads hands it over as int8 in that node's
    # staged layout (next_* parameters on the producer, staged_input on the consumer): no staging pass, no fp32
    # tensor in between
    live, todo = set(), list(module.outputs)
    while todo:                        # the chains' inner nodes are dead by now and must not count as readers
        i = todo.pop()
        if i not in live:
            live.add(i)
            todo.extend(nodes[i].inputs)
    users = {}
    for i in sorted(live):
        for j in nodes[i].inputs:
            users.setdefault(j, []).append(i)
    for j in module.outputs:
        users.setdefault(j, []).append(-1)
    for ci, cons in enumerate(nodes):
        if ci not in live:
            continue
        if cons.op != FUSED or "staged_input" in cons.params:
            continue
        pi = cons.inputs[0]
        prod = nodes[pi]
        if prod.op != FUSED or users.get(pi) != [ci] or "residual" in prod.params or "next_quantize_scale" in prod.params:
            continue
        wv = np.asarray(nodes[cons.inputs[1]].params.get("value"))
        if wv.ndim != 4:
            continue
        c, kh, kw = wv.shape[1], wv.shape[2], wv.shape[3]
        if kh * kw > 1 and c <= 8 and c * kh * kw <= 512:      # staged by im2col: cannot read a producer's buffer
            continue
        dil = cons.params.get("dilation", cons.params.get("dialations"))
        if dil is None or "padding" not in cons.params or "stride" not in cons.params:
            continue
        pad = np.asarray(cons.params["padding"]).reshape(4, 2)
        stride, dil = np.asarray(cons.params["stride"]).ravel(), np.asarray(dil).ravel()
        pp = dict(prod.params)
        pp["next_quantize_scale"] = cons.params["quantize_scale"]
        pp["next_ksize"] = np.array([kh, kw], np.int32)
        pp["next_padding"] = np.array([pad[2, 0], pad[2, 1], pad[3, 0], pad[3, 1]], np.int32)
        pp["next_stride"] = np.array([stride[2], stride[3]], np.int32)
        pp["next_dilation"] = np.array([dil[2], dil[3]], np.int32)
        pp["next_padding_value"] = np.asarray(cons.params.get("padding_value", np.zeros(1, np.float32)), np.float32).reshape(-1)[:1]
        nodes[pi] = Node(FUSED, prod.name, pp, prod.inputs)
        nodes[ci] = Node(FUSED, cons.name, dict(cons.params, staged_input=np.array([1], np.int32)), cons.inputs)
    # drop what no output reaches any more, renumber
    keep, stack = set(), list(module.outputs) + list(module.inputs)
    while stack:
        i = stack.pop()
        if i not in keep:
            keep.add(i)
            stack.extend(nodes[i].inputs)
    order = sorted(keep)
    new_index = {old: new for new, old in enumerate(order)}
    out_nodes = [Node(nodes[i].op, nodes[i].name, nodes[i].params, [new_index[j] for j in nodes[i].inputs]) for i in order]
    return Module(out_nodes, [new_index[i] for i in module.inputs], [new_index[i] for i in module.outputs])
