"""Writes tests/golden/cases/: operator test-case directories in the layout of TenniS's tools/run_test
(test_case.hpp:218-246), every tensor file written by the reference's own serializer and every expected
output computed by the reference's own CPU operator, both through the library that oracle/ref.mk compiles
from /root/reference.  Also a case of an operator this backend does not register (SKIP) and `sample.*.t`
files of every element type the reader knows, for the reader/writer tests.

    python tests/golden/make_cases.py        (needs oracle/_ref; run where /root/reference exists)

The committed cases are data: inputs, parameters and expected outputs.
"""
import os
import shutil
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import ref   # noqa: E402

OUT = os.path.join(HERE, "cases")


def conv_params(pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0):
    return {
        "format": "NCHW",
        "padding": np.array([[0, 0], [0, 0], [pads[0], pads[1]], [pads[2], pads[3]]], np.int32),
        "padding_value": np.array([padding_value], np.float32),
        "stride": np.array([1, 1, strides[0], strides[1]], np.int32),
        "dilation": np.array([1, 1, dilations[0], dilations[1]], np.int32),
    }


def pool_params(kind, ksize, strides, pads, white=False):
    return {"format": "NCHW", "type": np.array([{"max": 0, "avg": 1}[kind]], np.int32),
            "padding": np.array([[0, 0], [0, 0], [pads[0], pads[1]], [pads[2], pads[3]]], np.int32),
            "padding_type": np.array([3 if white else 0], np.int32),
            "ksize": np.array([1, 1, ksize[0], ksize[1]], np.int32),
            "stride": np.array([1, 1, strides[0], strides[1]], np.int32)}


def save_case(name, op, params, inputs, out_bytes=1 << 22):
    root = os.path.join(OUT, name)
    os.makedirs(root)
    output = ref.run_op(op, params, inputs, out_bytes, threads=1)
    with open(os.path.join(root, "0.%s.txt" % op), "w") as fh:
        fh.write("%d\n%d\n1\n" % (len(params), len(inputs)))
    for k, v in params.items():
        ref.save_tensor(os.path.join(root, "1.%s.t" % k), v)
    for i, v in enumerate(inputs):
        ref.save_tensor(os.path.join(root, "2.input_%d.t" % i), v)
    ref.save_tensor(os.path.join(root, "3.output_0.t"), output)
    print(name, op, output.dtype, output.shape)


def main():
    if os.path.exists(OUT):
        shutil.rmtree(OUT)
    os.makedirs(OUT)
    rng = np.random.default_rng(20240)
    f32 = lambda *s: rng.standard_normal(s).astype(np.float32)
    i8 = lambda *s: rng.integers(-128, 128, s).astype(np.int8)

    x = f32(2, 6, 9, 8)
    save_case("conv2d/3x3_pad1", "conv2d", conv_params((1, 1, 1, 1)), [x, f32(5, 6, 3, 3) * 0.2])
    save_case("conv2d/5x3_s2_d2_padvalue", "conv2d", conv_params((2, 1, 0, 3), (2, 1), (1, 2), 0.25), [x, f32(4, 6, 5, 3) * 0.2])
    save_case("conv2d/1x1", "conv2d", conv_params(), [x, f32(7, 6, 1, 1)])
    wino = {"format": "NCHW", "padding": conv_params((1, 1, 1, 1))["padding"], "padding_value": np.array([0], np.float32)}
    # the operator picks its mode itself: F(2,3) at this size (src/kernels/common/function.cpp:154-173)
    save_case("conv2d_winograd/auto_mode", "conv2d_winograd", wino, [f32(1, 6, 14, 13), f32(5, 6, 3, 3) * 0.2])
    xq = i8(2, 16, 7, 7)
    dq = rng.uniform(1e-3, 1e-2, 12).astype(np.float32)
    save_case("conv2d_quantized/3x3_pad1", "conv2d_quantized", dict(conv_params((1, 1, 1, 1)), dequantize_scales=dq),
              [xq, i8(12, 16, 3, 3)])
    save_case("conv2d_quantized/1x1_s2", "conv2d_quantized", dict(conv_params((0, 0, 0, 0), (2, 2)), dequantize_scales=dq),
              [xq, i8(12, 16, 1, 1)])
    save_case("quantize/per_image", "quantize", {"quantize_scale": np.array([20.5, 31.25], np.float32)}, [f32(2, 3, 5, 7)])
    save_case("quantize/single_scale", "quantize", {"quantize_scale": np.array([17.0], np.float32)}, [f32(1, 3, 5, 7)])
    save_case("inner_prod/plain", "inner_prod", {}, [f32(5, 40), f32(40, 24)])
    save_case("inner_prod/transpose", "inner_prod", {"transpose": np.array([True])}, [f32(5, 40), f32(24, 40)])
    save_case("add_bias/nchw", "add_bias", {"format": "NCHW"}, [x, f32(6)])
    save_case("relu/4d", "relu", {}, [x])
    save_case("leaky_relu/0.1", "leaky_relu", {"scale": np.array([0.1], np.float32)}, [x])
    save_case("pooling2d/max_3x3_s2", "pooling2d", pool_params("max", (3, 3), (2, 2), (1, 1, 1, 1)), [x])
    save_case("pooling2d/avg_white", "pooling2d", pool_params("avg", (3, 3), (1, 1), (1, 1, 1, 1), True), [x])
    save_case("global_pooling2d/avg", "global_pooling2d", {"format": "NCHW", "type": np.array([1], np.int32)}, [x])
    save_case("add/broadcast", "add", {}, [x, f32(1, 6, 1, 1)])
    save_case("depthwise_conv2d/3x3", "depthwise_conv2d", conv_params((1, 1, 1, 1)), [x, f32(1, 6, 3, 3)])
    # the "_v2" operators: padding (pooling: also ksize and stride) arrive as inputs
    pad42 = conv_params((1, 2, 0, 1))["padding"]
    v2 = {k: v for k, v in conv_params((0, 0, 0, 0), (2, 1)).items() if k != "padding"}
    save_case("conv2d_v2/3x3_s2x1", "conv2d_v2", v2, [x, pad42, f32(5, 6, 3, 3) * 0.2])
    save_case("depthwise_conv2d_v2/3x3_s2x1", "depthwise_conv2d_v2", v2, [x, pad42, f32(1, 6, 3, 3)])
    save_case("conv2d_winograd_v2/auto_mode", "conv2d_winograd_v2", {"format": "NCHW"},
              [f32(1, 6, 14, 13), conv_params((1, 1, 1, 1))["padding"], f32(5, 6, 3, 3) * 0.2])
    save_case("pooling2d_v2/avg_3x2", "pooling2d_v2", {"format": "NCHW", "type": np.array([1], np.int32)},
              [x, pad42, np.array([1, 1, 3, 2], np.int32), np.array([1, 1, 2, 1], np.int32)])
    # layout operators of detection necks
    save_case("concat/channels", "concat", {"dim": np.array([1], np.int32)}, [x, f32(2, 3, 9, 8), f32(2, 1, 9, 8)])
    save_case("concat/last_axis", "concat", {"dim": np.array([-1], np.int32)}, [f32(3, 5, 2), f32(3, 5, 7)])
    save_case("_resize2d/nearest_up", "_resize2d", {"type": np.array([2], np.int32)}, [x, np.array([-1, -1, 18, 16], np.int32)])
    save_case("_resize2d/nearest_odd", "_resize2d", {"type": np.array([2], np.int32)}, [x, np.array([-1, -1, 13, 5], np.int32)])
    # the nodes graphs compose Mish from
    save_case("softplus/4d", "softplus", {}, [x * 3])
    save_case("tanh/4d", "tanh", {}, [x * 2])
    save_case("mul/broadcast", "mul", {}, [x, f32(1, 6, 1, 1)])
    save_case("mul/same_shape", "mul", {}, [x, f32(2, 6, 9, 8)])
    # an operator the "hip" device does not register: the runner reports SKIP, as TenniS's does
    save_case("softmax/not_on_device", "softmax", {"dim": np.array([1], np.int32)}, [f32(3, 5)])

    # tensor files of every element type, written by the reference's serializer
    samples = {"int8": i8(3, 4), "uint8": rng.integers(0, 256, (5,)).astype(np.uint8),
               "int32": rng.integers(-2 ** 31, 2 ** 31, (2, 1, 3)).astype(np.int32),
               "float32": f32(2, 3, 4), "float64": rng.standard_normal((4, 2)), "bool": np.array([True, False, True]),
               "string": "NCHW"}
    for name, v in samples.items():
        ref.save_tensor(os.path.join(OUT, "sample.%s.t" % name), v)

    # batch normalisation nodes (their own generator, so that the cases above keep their bytes)
    rng = np.random.default_rng(20241)
    xb = (rng.standard_normal((2, 6, 5, 7)) * 2).astype(np.float32)
    mean, var = rng.standard_normal(6).astype(np.float32), rng.uniform(0.05, 3, 6).astype(np.float32)
    scale, bias = rng.standard_normal(6).astype(np.float32), rng.standard_normal(6).astype(np.float32)
    dim1 = {"dim": np.array([1], np.int32)}
    eps = dict(dim1, epsilon=np.array([1e-3], np.float32))
    save_case("batch_norm/nchw", "batch_norm", eps, [xb, mean, var])
    save_case("batch_scale/nchw", "batch_scale", dim1, [xb, scale, bias])
    save_case("fused_batch_norm/nchw", "fused_batch_norm", eps, [xb, mean, var, scale, bias])


if __name__ == "__main__":
    main()
