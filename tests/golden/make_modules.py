"""Writes tests/golden/modules/: a small TenniS module file (`.tsm`) with its input and the output the
reference computes for it.  The module is written by tennis_amd.module_file and then LOADED AND RUN BY THE
REFERENCE (Module::Load + Workbench on its CPU device, through the library oracle/ref.mk compiles), so the
fixture pins both the file format (the reference reads what the writer wrote) and the graph's values.

    python tests/golden/make_modules.py        (needs oracle/_ref; run where /root/reference exists)
"""
import os
import shutil
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import ref                                      # noqa: E402
from tennis_amd import module_file as mf, tensor_file       # noqa: E402

OUT = os.path.join(HERE, "modules")


def conv_params(pads, strides=(1, 1)):
    return {"format": "NCHW",
            "padding": np.array([[0, 0], [0, 0], [pads[0], pads[1]], [pads[2], pads[3]]], np.int32),
            "padding_value": np.array([0.0], np.float32),
            "stride": np.array([1, 1, strides[0], strides[1]], np.int32),
            "dilation": np.array([1, 1, 1, 1], np.int32)}


def quantized_block():
    """x -> quantize -> conv2d_quantized -> add_bias -> relu -> pooling2d (max 2x2/2) -> concat with a
    1x1 conv2d_quantized shortcut of the pooled input: the operator chain of the hot path as a graph."""
    rng = np.random.default_rng(31)
    n, c, h, w, cout = 2, 16, 12, 10, 24
    scales = np.array([9.5, 11.25], np.float32)
    w3 = rng.integers(-127, 128, (cout, c, 3, 3)).astype(np.int8)
    w1 = rng.integers(-127, 128, (8, c, 1, 1)).astype(np.int8)
    dq3 = rng.uniform(1e-4, 1e-3, cout).astype(np.float32)
    dq1 = rng.uniform(1e-3, 1e-2, 8).astype(np.float32)
    bias = rng.standard_normal(cout).astype(np.float32)
    pool = {"format": "NCHW", "type": np.array([0], np.int32),
            "padding": np.array([[0, 0], [0, 0], [0, 0], [0, 0]], np.int32), "padding_type": np.array([0], np.int32),
            "ksize": np.array([1, 1, 2, 2], np.int32), "stride": np.array([1, 1, 2, 2], np.int32)}
    N = mf.Node
    nodes = [
        N(mf.PARAMETER, "x"),                                                              # 0
        N("quantize", "q", {"quantize_scale": scales}, [0]),                                # 1
        N(mf.CONST, "w3", {"value": w3}),                                                  # 2
        N("conv2d_quantized", "conv3", dict(conv_params((1, 1, 1, 1)), dequantize_scales=dq3), [1, 2]),   # 3
        N(mf.CONST, "b", {"value": bias}),                                                 # 4
        N("add_bias", "bias", {"format": "NCHW"}, [3, 4]),                                 # 5
        N("relu", "relu", {}, [5]),                                                        # 6
        N("pooling2d", "pool", pool, [6]),                                                 # 7
        N(mf.CONST, "w1", {"value": w1}),                                                  # 8
        N("conv2d_quantized", "conv1", dict(conv_params((0, 0, 0, 0), (2, 2)), dequantize_scales=dq1), [1, 8]),  # 9
        N("concat", "join", {"dim": np.array([1], np.int32)}, [7, 9]),                     # 10
    ]
    x = (rng.standard_normal((n, c, h, w)) * 8).astype(np.float32)
    return mf.Module(nodes, [0], [10]), x


def main():
    if os.path.exists(OUT):
        shutil.rmtree(OUT)
    os.makedirs(OUT)
    module, x = quantized_block()
    path = os.path.join(OUT, "quantized_block.tsm")
    mf.write_module(path, module)
    y = ref.run_module(path, [x])
    tensor_file.write_tensor(os.path.join(OUT, "quantized_block.input_0.t"), x)
    tensor_file.write_tensor(os.path.join(OUT, "quantized_block.output_0.t"), y)
    print("quantized_block", x.shape, "->", y.shape, y.dtype, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
