"""CPU-side checks of the boundary: the C-ABI library exports every symbol include/tsx_hip.h
declares, the C++ operator layer registers the hot-path operators for device "hip", and its
host logic (parameter checking, error behaviour) follows the reference.  No compute calls."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c_abi_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "tsx_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(tsx_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 25
    lib = ctypes.CDLL(os.path.join(ROOT, "tennis_amd", "lib", "libtsx_hip.so"))
    missing = [name for name in sorted(declared) if not hasattr(lib, name)]
    assert not missing, missing
    from tennis_amd import capi
    assert declared == set(capi.SIGNATURES), declared ^ set(capi.SIGNATURES)


def test_argument_errors_need_no_device():
    from tennis_amd import capi
    L = capi.lib()
    assert L.tsx_version() == 100
    g = capi.ConvGeom(1, 8, 2, 2, 4, 3, 3, 0, 0, 0, 0, 1, 1, 1, 1)          # 3x3 on 2x2 without padding
    assert L.tsx_conv2d_i8_workspace_bytes(ctypes.byref(g)) == 0
    assert b"empty output" in L.tsx_last_error()
    g = capi.ConvGeom(1, 8, 5, 5, 4, 3, 3, 1, 1, 1, 1, 0, 1, 1, 1)          # zero stride
    assert L.tsx_conv2d_i8_packed_weight_bytes(ctypes.byref(g)) == 0
    g = capi.ConvGeom(1, 8, 9, 9, 4, 5, 5, 1, 1, 1, 1, 1, 1, 1, 1)          # Winograd needs 3x3
    assert L.tsx_winograd_f63_workspace_bytes(ctypes.byref(g)) == 0
    assert L.tsx_quantize_f32_i8(None, -1, None, 1, None, None) == -1
    # geometry bookkeeping of BASELINE config 2
    g = capi.ConvGeom(32, 256, 28, 28, 256, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1)
    assert L.tsx_conv2d_i8_workspace_bytes(ctypes.byref(g)) == 32 * 30 * 30 * 256
    assert L.tsx_conv2d_i8_packed_weight_bytes(ctypes.byref(g)) == 256 * 256 * 9
    ho, wo = capi.conv_out_size(g)
    assert (ho, wo) == (28, 28)


def test_kernel_choices_need_no_device(monkeypatch):
    """Which kernel a layer takes is decided on the host from the geometry (and the weights' alignment) alone, and the
    plan-info entry points report it: config 2 on the weight-stationary int8 kernel, config 1 on the small-layer fp32
    kernel, and the environment switches that tests use to put small layers on a given kernel."""
    from tennis_amd import capi
    L = capi.lib()
    for name in ("TSX_CONV_I8_FLAT", "TSX_CONV_I8_RS", "TSX_CONV_F32_SMALL", "TSX_GEMM_F32_REGFED"):
        monkeypatch.delenv(name, raising=False)

    def i8(geom):
        buf = ctypes.create_string_buffer(256)
        assert L.tsx_conv2d_i8_plan_info(ctypes.byref(geom), buf, len(buf)) == 0
        return dict(word.split("=", 1) for word in buf.value.decode().split())

    def f32(geom, weights_address=4096):
        buf = ctypes.create_string_buffer(256)
        assert L.tsx_conv2d_f32_plan_info(ctypes.byref(geom), ctypes.c_void_p(weights_address), buf, len(buf)) == 0
        return dict(word.split("=", 1) for word in buf.value.decode().split())

    c2 = capi.ConvGeom(32, 256, 28, 28, 256, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1)
    assert i8(c2)["fp32_kernel"] == "weight_stationary"
    monkeypatch.setenv("TSX_CONV_I8_RS", "0")
    assert i8(c2)["fp32_kernel"] != "weight_stationary"
    c1 = capi.ConvGeom(1, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1)
    assert f32(c1) == {"kernel": "small_3x3", "tiles": "196"}
    assert f32(c1, weights_address=4100)["kernel"] == "staged_32x32_ksplit"       # rows of A not 16-byte aligned
    big = capi.ConvGeom(32, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1)
    assert f32(big)["kernel"] == "staged_64x64"
    monkeypatch.setenv("TSX_CONV_F32_SMALL", "force")
    assert f32(big)["kernel"] == "small_3x3"
    monkeypatch.setenv("TSX_CONV_F32_SMALL", "0")
    assert f32(c1)["kernel"] == "register_fed"
    assert L.tsx_conv2d_f32_plan_info(ctypes.byref(c1), None, None, 0) == -1


def test_hot_path_operators_are_registered_for_hip():
    from tennis_amd import operators as ops
    for name in ops.SYMBOLS:
        assert hasattr(ops.lib(), name)
    for op in ("quantize", "conv2d_quantized", "conv2d", "conv2d_winograd", "inner_prod", "add_bias", "relu", "leaky_relu",
               "pooling2d", "global_pooling2d", "add", "depthwise_conv2d", "conv2d_v2", "conv2d_winograd_v2",
               "depthwise_conv2d_v2", "pooling2d_v2", "concat", "_resize2d", "mul", "softplus", "tanh",
               "conv2d_quantized_fused"):
        assert ops.is_registered("hip", op), op
    assert not ops.is_registered("hip", "softmax")
    assert not ops.is_registered("cpu", "conv2d")            # this library ships no host operators
    with pytest.raises(ops.OperatorNotFound):
        ops.check_params("softmax", {})                       # strict: no silent fallback


def test_parameter_checking_follows_the_reference():
    from tennis_amd import operators as ops
    good = ops.conv_params((1, 1, 1, 1))
    good["dequantize_scales"] = np.ones(4, np.float32)
    ops.check_params("conv2d_quantized", good)
    # required field missing (src/runtime/operator.cpp:174-193)
    missing = dict(good)
    del missing["dequantize_scales"]
    with pytest.raises(ops.OperatorError, match="dequantize_scales"):
        ops.check_params("conv2d_quantized", missing)
    # unknown parameter names are rejected in strict mode (operator.cpp:26-38)
    with pytest.raises(ops.OperatorError, match="Unidentified param"):
        ops.check_params("conv2d_quantized", dict(good, quantize_scale=np.ones(1, np.float32)))
    # the typo'd spelling of dilation is accepted, none at all is not (base_conv2d.cpp:51-60)
    typo = dict(good)
    typo["dialations"] = typo.pop("dilation")
    ops.check_params("conv2d_quantized", typo)
    none = dict(good)
    del none["dilation"]
    with pytest.raises(ops.OperatorError, match="must set dilation or dialations"):
        ops.check_params("conv2d_quantized", none)
    # padding / stride on batch or channel are refused
    bad = dict(good, padding=np.array([[1, 0], [0, 0], [1, 1], [1, 1]], np.int32))
    with pytest.raises(ops.OperatorError, match="do not support padding"):
        ops.check_params("conv2d", {k: v for k, v in bad.items() if k != "dequantize_scales"})
    bad = dict(good, stride=np.array([1, 2, 1, 1], np.int32))
    with pytest.raises(ops.OperatorError, match="do not support stride"):
        ops.check_params("conv2d_quantized", bad)
    with pytest.raises(ops.OperatorError, match="do not support format"):
        ops.check_params("conv2d_quantized", dict(good, format="NCDHW"))
    with pytest.raises(ops.OperatorError):
        ops.check_params("add_bias", {})                      # needs format or dim
    ops.check_params("add_bias", {"dim": np.array([1], np.int32)})
    ops.check_params("quantize", {"quantize_scale": np.ones(3, np.float32)})
    with pytest.raises(ops.OperatorError, match="quantize_scale"):
        ops.check_params("quantize", {})
    with pytest.raises(ops.OperatorError, match="scale"):
        ops.check_params("leaky_relu", {})
    # pooling2d: ksize / stride / padding on the two image axes only (base_pooling2d.cpp:66-98)
    pool = {"format": "NCHW", "type": np.array([0], np.int32), "padding": np.zeros((4, 2), np.int32),
            "ksize": np.array([1, 1, 3, 3], np.int32), "stride": np.array([1, 1, 2, 2], np.int32)}
    ops.check_params("pooling2d", pool)                       # padding_type is optional (BLACK)
    with pytest.raises(ops.OperatorError, match="do not support ksize"):
        ops.check_params("pooling2d", dict(pool, ksize=np.array([1, 2, 3, 3], np.int32)))
    with pytest.raises(ops.OperatorError, match="do not support padding"):
        ops.check_params("pooling2d", dict(pool, padding=np.array([[0, 0], [0, 1], [0, 0], [0, 0]], np.int32)))
    with pytest.raises(ops.OperatorError, match="type"):
        ops.check_params("global_pooling2d", {"format": "NCHW"})
    ops.check_params("add", {})
    ops.check_params("depthwise_conv2d", {k: v for k, v in good.items() if k != "dequantize_scales"})
