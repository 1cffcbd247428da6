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


@pytest.mark.gpu
def test_module_runs_on_hip_like_in_the_reference():
    m = mf.read_module(BLOCK)
    x = tensor_file.read_tensor(os.path.join(MODULES, "quantized_block.input_0.t"))
    want = tensor_file.read_tensor(os.path.join(MODULES, "quantized_block.output_0.t"))
    (got,) = mf.run_module(m, [x])
    assert got.dtype == want.dtype and got.shape == want.shape
    assert np.array_equal(bits(got), bits(want))       # int8 chain and exact glue operators: bit for bit
