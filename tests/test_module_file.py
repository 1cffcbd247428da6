"""TenniS module files (`.tsm`, doc/zh_CN/module.md section 4): reader, writer and the operator-by-operator
runner.  The fixture under tests/golden/modules was written by tennis_amd.module_file and then loaded and run by
the reference itself (tests/golden/make_modules.py), whose output is the expected tensor."""
import os
import struct

import numpy as np
import pytest

from _util import bits
from tennis_amd import module_file as mf, tensor_file

MODULES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "modules")
BLOCK = os.path.join(MODULES, "quantized_block.tsm")


def test_reads_the_module_the_reference_accepted():
    m = mf.read_module(BLOCK)
    assert m.inputs == [0] and m.outputs == [10] and len(m.nodes) == 11
    assert [n.op for n in m.nodes] == ["<param>", "quantize", "<const>", "conv2d_quantized", "<const>", "add_bias", "relu",
                                      "pooling2d", "<const>", "conv2d_quantized", "concat"]
    conv = m.nodes[3]
    assert conv.name == "conv3" and conv.inputs == [1, 2] and conv.params["format"] == "NCHW"
    assert conv.params["dequantize_scales"].dtype == np.float32 and conv.params["dequantize_scales"].shape == (24,)
    assert "#op" not in conv.params and "#name" not in conv.params
    assert m.nodes[2].params["value"].dtype == np.int8 and m.nodes[2].params["value"].shape == (24, 16, 3, 3)
    with open(BLOCK, "rb") as fh:
        raw = fh.read()
    assert mf.serialize_module(m) == raw                                   # writer and reader are inverse
    assert struct.unpack_from("<II", raw, 0) == (0, 0x19910929) and raw[8:128] == bytes(120)


def test_known_bytes_of_a_one_node_module():
    """<param> x -> relu, spelled out byte by byte."""
    def tensor_str(s):
        return struct.pack("<IBII", 1, 13, 1, len(s)) + s.encode()
    def param(name, value):
        return struct.pack("<I", len(name)) + name.encode() + value
    node0 = struct.pack("<I", 2) + param("#name", tensor_str("x")) + param("#op", tensor_str("<param>")) + struct.pack("<I", 0)
    node1 = struct.pack("<I", 2) + param("#name", tensor_str("y")) + param("#op", tensor_str("relu")) + struct.pack("<II", 1, 0)
    raw = (struct.pack("<II", 0, 0x19910929) + bytes(120) + struct.pack("<II", 1, 0) + struct.pack("<II", 1, 1) +
           struct.pack("<I", 2) + node0 + node1)
    m = mf.parse_module(raw)
    assert [(n.op, n.name, n.inputs) for n in m.nodes] == [("<param>", "x", []), ("relu", "y", [0])]
    assert mf.serialize_module(mf.Module([mf.Node("<param>", "x"), mf.Node("relu", "y", {}, [0])], [0], [1])) == raw


def test_broken_files_are_reported():
    with open(BLOCK, "rb") as fh:
        raw = fh.read()
    with pytest.raises(mf.ModuleFileError, match="truncated"):
        mf.parse_module(raw[:-3])
    with pytest.raises(mf.ModuleFileError, match="behind the graph"):
        mf.parse_module(raw + b"\0\0\0\0")
    with pytest.raises(mf.ModuleFileError, match="not format V1"):
        mf.parse_module(raw[:4] + struct.pack("<I", 0x12345678) + raw[8:])
    bad = bytearray(raw)
    struct.pack_into("<I", bad, 128 + 4, 999)           # the module's input index
    with pytest.raises(mf.ModuleFileError, match="out of range"):
        mf.parse_module(bytes(bad))
    with pytest.raises(mf.ModuleFileError, match="no header"):
        mf.parse_module(raw[:100])


def test_runner_rejects_bad_graphs_before_touching_the_device():
    m = mf.read_module(BLOCK)
    with pytest.raises(mf.ModuleFileError, match="1 inputs, 0 fed"):
        mf.run_module(m, [])
    loop = mf.Module([mf.Node("<param>", "x"), mf.Node("relu", "a", {}, [2]), mf.Node("relu", "b", {}, [1])], [0], [2])
    with pytest.raises(mf.ModuleFileError, match="cycle"):
        mf.run_module(loop, [np.zeros(3, np.float32)])
    stray = mf.Module([mf.Node("<param>", "x"), mf.Node("<param>", "z"), mf.Node("relu", "a", {}, [1])], [0], [2])
    with pytest.raises(mf.ModuleFileError, match="not among the module's inputs"):
        mf.run_module(stray, [np.zeros(3, np.float32)])


def test_reference_loads_and_runs_a_freshly_written_module(ref, tmp_path):
    """Where the compiled reference is built: its Module::Load reads the writer's file and its Workbench gives
    the values of the graph (add_bias + relu on a constant bias: exact)."""
    rng = np.random.default_rng(5)
    b = rng.standard_normal(6).astype(np.float32)
    m = mf.Module([mf.Node("<param>", "x"), mf.Node("<const>", "b", {"value": b}),
                   mf.Node("add_bias", "ab", {"format": "NCHW"}, [0, 1]), mf.Node("relu", "y", {}, [2])], [0], [3])
    path = str(tmp_path / "m.tsm")
    mf.write_module(path, m)
    x = rng.standard_normal((2, 6, 5, 4)).astype(np.float32)
    y = ref.run_module(path, [x])
    assert np.array_equal(y, np.maximum(x + b.reshape(1, 6, 1, 1), 0))


@pytest.fixture(scope="module")
def hip_device():
    """torch initialises its HIP runtime before the operator library loads its own, as in the other GPU tests."""
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return "hip"


@pytest.mark.gpu
def test_module_runs_on_hip_like_in_the_reference(hip_device):
    m = mf.read_module(BLOCK)
    x = tensor_file.read_tensor(os.path.join(MODULES, "quantized_block.input_0.t"))
    want = tensor_file.read_tensor(os.path.join(MODULES, "quantized_block.output_0.t"))
    (got,) = mf.run_module(m, [x])
    assert got.dtype == want.dtype and got.shape == want.shape
    assert np.array_equal(bits(got), bits(want))       # int8 chain and exact glue operators: bit for bit


def test_fusing_rewrite_structure():
    """quantize -> conv2d_quantized -> add_bias -> relu becomes one node; the quantize node shared with the shortcut
    convolution is folded into both; dead nodes go and links are renumbered."""
    m = mf.read_module(BLOCK)
    f = mf.fuse_quantized_chains(m)
    ops = [n.op for n in f.nodes]
    assert ops.count(mf.FUSED) == 2 and not {"quantize", "conv2d_quantized", "add_bias", "relu"} & set(ops)
    assert len(f.nodes) == 8 and f.inputs == [0]
    main = next(n for n in f.nodes if n.op == mf.FUSED and len(n.inputs) == 3)
    assert main.params["activation"] == "relu" and [f.nodes[i].op for i in main.inputs] == ["<param>", "<const>", "<const>"]
    assert np.array_equal(main.params["quantize_scale"], m.nodes[1].params["quantize_scale"])
    short = next(n for n in f.nodes if n.op == mf.FUSED and len(n.inputs) == 2)
    assert "activation" not in short.params
    assert f.nodes[f.outputs[0]].op == "concat"
    mf.parse_module(mf.serialize_module(f))                  # still a well-formed module
    # a convolution whose output has a second consumer keeps its add_bias outside the fused node
    N = mf.Node
    w = np.zeros((4, 8, 1, 1), np.int8)
    conv = dict(m.nodes[9].params, dequantize_scales=np.ones(4, np.float32))
    g = mf.Module([N("<param>", "x"), N("quantize", "q", {"quantize_scale": np.ones(1, np.float32)}, [0]), N("<const>", "w", {"value": w}),
                   N("conv2d_quantized", "c", conv, [1, 2]), N("<const>", "b", {"value": np.zeros(4, np.float32)}),
                   N("add_bias", "ab", {"format": "NCHW"}, [3, 4]), N("add", "sum", {}, [3, 5])], [0], [6])
    fg = mf.fuse_quantized_chains(g)
    assert [n.op for n in fg.nodes].count("add_bias") == 1 and [n.op for n in fg.nodes].count(mf.FUSED) == 1

    # the bias axis as AddBias::init resolves it: dim overrides the format's 'C' (base_add_bias.cpp:27-40), and only
    # axis 1 with one float32 value per output channel is a channel bias the fused epilogue can add
    def chain(bias_params, bias_value):
        return mf.Module([N("<param>", "x"), N("quantize", "q", {"quantize_scale": np.ones(1, np.float32)}, [0]),
                          N("<const>", "w", {"value": w}), N("conv2d_quantized", "c", conv, [1, 2]),
                          N("<const>", "b", {"value": bias_value}), N("add_bias", "ab", bias_params, [3, 4])], [0], [5])

    def bias_fused(bias_params, bias_value=np.zeros(4, np.float32)):
        ops = [n.op for n in mf.fuse_quantized_chains(chain(bias_params, bias_value)).nodes]
        assert ops.count(mf.FUSED) == 1
        return "add_bias" not in ops

    one, three = np.array([1], np.int32), np.array([3], np.int32)
    assert bias_fused({"format": "NCHW"}) and bias_fused({"dim": one}) and bias_fused({"format": "NHWC", "dim": one})
    assert not bias_fused({"format": "NCHW", "dim": three})       # dim wins: the bias runs along W
    assert not bias_fused({"format": "NHWC"}) and not bias_fused({"dim": three})
    assert not bias_fused({"format": "NCHW"}, np.zeros(4, np.float64))
    assert not bias_fused({"format": "NCHW"}, np.zeros(1, np.float32))


@pytest.mark.gpu
def test_fused_module_equals_the_unfused_one(hip_device):
    m = mf.read_module(BLOCK)
    x = tensor_file.read_tensor(os.path.join(MODULES, "quantized_block.input_0.t"))
    want = tensor_file.read_tensor(os.path.join(MODULES, "quantized_block.output_0.t"))
    (got,) = mf.run_module(mf.fuse_quantized_chains(m), [x])
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.gpu
def test_fused_operator_against_the_operator_chain(hip_device):
    from tennis_amd import operators as ops
    rng = np.random.default_rng(41)
    x = (rng.standard_normal((3, 20, 9, 11)) * 6).astype(np.float32)
    w = rng.integers(-127, 128, (10, 20, 3, 3)).astype(np.int8)
    bias = rng.standard_normal(10).astype(np.float32)
    qs = np.array([7.0, 9.5, 12.25], np.float32)
    for pads, strides, dil, pv, act in (((1, 1, 1, 1), (1, 1), (1, 1), 0.0, "relu"), ((0, 2, 1, 0), (2, 1), (1, 2), 3.0, "leaky_relu"),
                                        ((1, 0, 0, 1), (1, 2), (1, 1), 0.0, "none")):
        conv = dict(ops.conv_params(pads, strides, dil, pv), dequantize_scales=rng.uniform(1e-4, 1e-3, 10).astype(np.float32))
        y = ops.run_op("conv2d_quantized", conv, [ops.run_op("quantize", {"quantize_scale": qs}, [x]), w])
        y = ops.run_op("add_bias", {"format": "NCHW"}, [y, bias])
        if act == "relu":
            y = ops.run_op("relu", {}, [y])
        elif act == "leaky_relu":
            y = ops.run_op("leaky_relu", {"scale": np.array([0.1], np.float32)}, [y])
        fused = dict(conv, quantize_scale=qs, activation=act, scale=np.array([0.1], np.float32))
        assert ops.run_op(mf.FUSED, fused, [x, w, bias], infer_only=True)[1] == y.shape
        got = ops.run_op(mf.FUSED, fused, [x, w, bias])
        assert np.array_equal(bits(got), bits(y)), (pads, strides, dil, act)
    with pytest.raises(ops.OperatorError, match="quantize scales for a batch"):
        ops.run_op(mf.FUSED, dict(fused, quantize_scale=qs[:2]), [x, w, bias])
    with pytest.raises(ops.OperatorError, match="activation must be"):
        ops.run_op(mf.FUSED, dict(fused, activation="gelu"), [x, w, bias])


def test_fusing_rewrite_folds_residual_joins():
    """add (+ relu) behind a chain moves into the fused node: a ResNet-shaped module keeps no add and no relu node;
    a darknet-style shortcut behind an activated chain becomes residual = 2; an add whose chain operand has a second
    reader stays."""
    from tennis_amd import resnet50
    desc, params = resnet50.make_parameters(seed=3, width=0.25, blocks=(2, 1, 1, 1), classes=10)
    f = mf.fuse_quantized_chains(resnet50.to_module(desc, params, batch=2))
    ops = [n.op for n in f.nodes]
    assert "add" not in ops and "relu" not in ops and "quantize" not in ops
    joins = [n for n in f.nodes if n.op == mf.FUSED and "residual" in n.params]
    assert len(joins) == 5 and all(int(n.params["residual"][0]) == 1 and n.params["activation"] == "relu" for n in joins)
    assert all(len(n.inputs) == 4 for n in joins)             # x, w, bias, the other branch
    mf.parse_module(mf.serialize_module(f))
    N = mf.Node
    w = np.zeros((4, 8, 1, 1), np.int8)
    conv = {"format": "NCHW", "padding": np.zeros((4, 2), np.int32), "padding_value": np.zeros(1, np.float32),
            "stride": np.ones(4, np.int32), "dilation": np.ones(4, np.int32), "dequantize_scales": np.ones(4, np.float32)}
    g = mf.Module([N("<param>", "x"), N("<param>", "s"), N("quantize", "q", {"quantize_scale": np.ones(1, np.float32)}, [0]),
                   N("<const>", "w", {"value": w}), N("conv2d_quantized", "c", conv, [2, 3]),
                   N("leaky_relu", "act", {"scale": np.array([0.1], np.float32)}, [4]), N("add", "shortcut", {}, [1, 5])], [0, 1], [6])
    fg = mf.fuse_quantized_chains(g)
    fused = [n for n in fg.nodes if n.op == mf.FUSED]
    assert len(fused) == 1 and int(fused[0].params["residual"][0]) == 2 and fused[0].params["activation"] == "leaky_relu"
    assert [fg.nodes[i].name for i in fused[0].inputs] == ["x", "w", "s"] and "add" not in [n.op for n in fg.nodes]
    g2 = mf.Module(g.nodes + [N("relu", "second_reader", {}, [5]), N("add", "sum", {}, [6, 7])], [0, 1], [8])
    ops2 = [n.op for n in mf.fuse_quantized_chains(g2).nodes]
    assert ops2.count("add") == 2 and ops2.count(mf.FUSED) == 1


@pytest.mark.gpu
def test_fused_operator_with_residual_against_the_operator_chain(hip_device):
    """conv2d_quantized_fused with a residual input against quantize -> conv2d_quantized -> add_bias -> [act] -> add
    [-> act] run operator by operator: residual of the output's shape (the MFMA kernel's epilogue) and residuals that
    broadcast into it (the broadcast pass), both join orders."""
    from tennis_amd import operators as ops
    rng = np.random.default_rng(43)
    x = (rng.standard_normal((2, 24, 9, 11)) * 6).astype(np.float32)
    w = rng.integers(-127, 128, (130, 24, 3, 3)).astype(np.int8)
    bias = rng.standard_normal(130).astype(np.float32)
    qs = np.array([7.0, 9.5], np.float32)
    conv = dict(ops.conv_params((1, 1, 1, 1)), dequantize_scales=rng.uniform(1e-4, 1e-3, 130).astype(np.float32))
    y0 = ops.run_op("add_bias", {"format": "NCHW"},
                    [ops.run_op("conv2d_quantized", conv, [ops.run_op("quantize", {"quantize_scale": qs}, [x]), w]), bias])
    slope = {"scale": np.array([0.1], np.float32)}
    for shape in ((2, 130, 9, 11), (1, 130, 1, 1), (9, 11), (1,)):
        r = rng.standard_normal(shape).astype(np.float32)
        for act in ("none", "relu", "leaky_relu"):
            apply = lambda t: t if act == "none" else ops.run_op(act, slope if act == "leaky_relu" else {}, [t])
            want1 = apply(ops.run_op("add", {}, [y0, r]))                    # act(y + r)
            want2 = ops.run_op("add", {}, [apply(y0), r])                    # act(y) + r
            base = dict(conv, quantize_scale=qs, activation=act, scale=slope["scale"])
            got1 = ops.run_op(mf.FUSED, dict(base, residual=np.array([1], np.int32)), [x, w, bias, r])
            assert np.array_equal(bits(got1), bits(want1)), (shape, act, 1)
            got2 = ops.run_op(mf.FUSED, dict(base, residual=np.array([2], np.int32)), [x, w, bias, r])
            assert np.array_equal(bits(got2), bits(want2)), (shape, act, 2)
    with pytest.raises(ops.OperatorError, match="do not broadcast"):
        ops.run_op(mf.FUSED, dict(base, residual=np.array([1], np.int32)), [x, w, bias, np.zeros((3, 130, 9, 11), np.float32)])
    with pytest.raises(ops.OperatorError, match="inputs"):
        ops.run_op(mf.FUSED, dict(base, residual=np.array([1], np.int32)), [x, w])


def test_fusing_rewrite_hands_int8_over_between_chains():
    """c1 -> c2 -> c3 of a bottleneck: c1 and c2 become producers (next_* of their consumer), c2 and c3 consumers
    (staged_input); the block's first convolution and its projection read the fp32 block input as before."""
    from tennis_amd import resnet50
    desc, params = resnet50.make_parameters(seed=3, width=0.25, blocks=(1, 1, 1, 1), classes=10)
    f = mf.fuse_quantized_chains(resnet50.to_module(desc, params, batch=2))
    fused = [n for n in f.nodes if n.op == mf.FUSED]
    assert len(fused) == 17
    producers = [n for n in fused if "next_quantize_scale" in n.params]
    consumers = [n for n in fused if "staged_input" in n.params]
    assert len(producers) == 8 and len(consumers) == 8          # two hand-overs per block
    c2 = next(n for n in fused if n.name == "s1b0.c2.relu")
    assert "staged_input" in c2.params and list(c2.params["next_ksize"]) == [1, 1] and list(c2.params["next_padding"]) == [0, 0, 0, 0]
    c1 = f.nodes[c2.inputs[0]]
    assert c1.op == mf.FUSED and list(c1.params["next_ksize"]) == [3, 3] and list(c1.params["next_padding"]) == [1, 1, 1, 1]
    assert np.array_equal(c1.params["next_quantize_scale"], c2.params["quantize_scale"]) and "staged_input" not in c1.params
    stem = next(n for n in fused if n.name.startswith("stem"))
    assert "next_quantize_scale" not in stem.params             # a pooling node reads the stem
    mf.parse_module(mf.serialize_module(f))
