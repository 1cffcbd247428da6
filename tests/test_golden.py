"""Golden vectors written by the compiled TenniS reference (tests/golden/make_golden.py): the CPU
oracle and the HIP path are each checked against them, so parity does not hinge on the compiled
reference being present where the tests run.

Bar: bitwise for everything integer, for the fp32 epilogue chain and for Winograd F(6,3); the fp32
MFMA GEMM paths (conv2d, inner_prod) within 1e-4 relative + 1e-5 absolute.
"""
import os

import numpy as np
import pytest

from _util import bits

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hotpath_vectors.npz"))
QCONV = ["c3", "cs", "c1"]


def _geom(tag):
    g = [int(v) for v in G[tag + "_geom"]]
    return tuple(g[0:4]), tuple(g[4:6]), tuple(g[6:8]), float(G[tag + "_pv"][0])


def close(a, b):
    return np.all(np.abs(a.astype(np.float64) - b) <= 1e-4 * np.abs(b) + 1e-5)


# ------------------------------------------------------------------ CPU oracle against the fixtures

@pytest.mark.parametrize("tag", ["q1", "q2", "q3"])
def test_oracle_quantize(port, tag):
    assert np.array_equal(port.quantize(G[tag + "_x"], G[tag + "_s"]), G[tag + "_y"])


@pytest.mark.parametrize("tag", QCONV)
def test_oracle_quantized_conv_chain(port, tag):
    pads, strides, dil, pv = _geom(tag)
    x, w, dq, b = G[tag + "_x"], G[tag + "_w"], G[tag + "_dq"], G[tag + "_b"]
    y = port.conv2d_quantized(x, w, dq, pads, strides, dil, pv)
    assert np.array_equal(bits(y), bits(G[tag + "_y"]))
    yb = port.add_bias(y, b)
    assert np.array_equal(bits(yb), bits(G[tag + "_yb"]))
    assert np.array_equal(bits(port.relu(yb)), bits(G[tag + "_relu"]))
    assert np.array_equal(bits(port.leaky_relu(yb, 0.1)), bits(G[tag + "_leaky"]))
    fused, q = port.conv2d_i8_fused(x, w, dq, b, "relu", 0.0, G[tag + "_qs"], pads, strides, dil, pv)
    assert np.array_equal(bits(fused), bits(G[tag + "_relu"]))
    assert np.array_equal(q, G[tag + "_requant"])


def test_oracle_fp32(port):
    assert np.array_equal(bits(port.conv2d_f32(G["f_x"], G["f_w"], (1, 1, 1, 1))), bits(G["f_y"]))
    assert np.array_equal(bits(port.conv2d_f32(G["f_x"], G["f_w"], (0, 1, 2, 0), (2, 2), (1, 1), 0.5)), bits(G["f_y_s2"]))
    assert np.array_equal(bits(port.inner_prod_f32(G["ip_a"], G["ip_b"], False)), bits(G["ip_y"]))
    assert np.array_equal(bits(port.inner_prod_f32(G["ip_a"], np.ascontiguousarray(G["ip_b"].T), True)), bits(G["ip_yt"]))
    assert np.array_equal(bits(port.winograd_f63(G["wg_x"], G["wg_w"], (1, 1, 1, 1), 0.0)), bits(G["wg_y"]))
    assert np.array_equal(bits(port.winograd_f63(G["wg_x"], G["wg_w"], (1, 1, 1, 1), 0.25)), bits(G["wg_y_pv"]))
    assert np.array_equal(bits(port.winograd_f23(G["wg_x"], G["wg_w"], (1, 1, 1, 1), 0.0)), bits(G["wg23_y"]))
    assert np.array_equal(bits(port.winograd_f23(G["wg_x"], G["wg_w"], (1, 1, 1, 1), 0.25)), bits(G["wg23_y_pv"]))
    assert np.array_equal(port.gemm_i8(G["g8_a"], G["g8_b"]), G["g8_c"])
    assert np.array_equal(port.gemm_i8(G["g8_a"], G["g8_b"], faithful=True), G["g8_c"])


def test_fixture_is_self_consistent():
    """Reference-independent anchors on the fixture itself: exact integer conv by brute force, and
    the fp32 outputs within fp64 accuracy (a fixture from a broken build would fail here)."""
    x, w = G["c1_x"].astype(np.int64), G["c1_w"].astype(np.int64)
    acc = np.einsum("nchw,oc->nohw", x, w[:, :, 0, 0])
    y = (acc.astype(np.int32).astype(np.float32) * G["c1_dq"][None, :, None, None]).astype(np.float32)
    assert np.array_equal(bits(y), bits(G["c1_y"]))
    assert np.array_equal(G["g8_a"].astype(np.int32) @ G["g8_b"].astype(np.int32), G["g8_c"])
    assert close(G["ip_y"], G["ip_a"].astype(np.float64) @ G["ip_b"].astype(np.float64))
    assert np.array_equal(G["q1_y"].ravel()[:8], np.array([0, 2, 2, 0, -2, -2, 126, 127], np.int8))   # half-even bulk
    assert np.array_equal(G["q1_y"].ravel()[8:12], np.array([-128, -128, 127, -128], np.int8))        # half-away tail


# ------------------------------------------------------------------ HIP path against the fixtures

@pytest.fixture(scope="module")
def tsx():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from tennis_amd import capi
    capi.lib()
    return capi


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["q1", "q2", "q3"])
def test_hip_quantize(tsx, tag):
    y = tsx.quantize(_dev(G[tag + "_x"]), _dev(G[tag + "_s"]))
    assert np.array_equal(y.cpu().numpy(), G[tag + "_y"])


@pytest.mark.gpu
@pytest.mark.parametrize("tag", QCONV)
def test_hip_quantized_conv_chain(tsx, tag):
    pads, strides, dil, pv = _geom(tag)
    conv = tsx.Conv2dI8(_dev(G[tag + "_w"]), pads, strides, dil, pv)
    x, dq, b = _dev(G[tag + "_x"]), _dev(G[tag + "_dq"]), _dev(G[tag + "_b"])
    y, _, _ = conv(x, dq=dq)
    assert np.array_equal(bits(y.cpu().numpy()), bits(G[tag + "_y"]))
    yb, _, _ = conv(x, dq=dq, bias=b)
    assert np.array_equal(bits(yb.cpu().numpy()), bits(G[tag + "_yb"]))
    yl, _, _ = conv(x, dq=dq, bias=b, act="leaky_relu", slope=0.1)
    assert np.array_equal(bits(yl.cpu().numpy()), bits(G[tag + "_leaky"]))
    yr, q, _ = conv(x, dq=dq, bias=b, act="relu", q_scales=_dev(G[tag + "_qs"]))
    assert np.array_equal(bits(yr.cpu().numpy()), bits(G[tag + "_relu"]))
    assert np.array_equal(q.cpu().numpy(), G[tag + "_requant"])
    # the standalone elementwise kernels, on the reference's own intermediate tensors
    assert np.array_equal(bits(tsx.add_bias(_dev(G[tag + "_y"]), b).cpu().numpy()), bits(G[tag + "_yb"]))
    assert np.array_equal(bits(tsx.relu(_dev(G[tag + "_yb"])).cpu().numpy()), bits(G[tag + "_relu"]))
    assert np.array_equal(bits(tsx.leaky_relu(_dev(G[tag + "_yb"]), 0.1).cpu().numpy()), bits(G[tag + "_leaky"]))


@pytest.mark.gpu
def test_hip_fp32(tsx):
    y = tsx.conv2d_f32(_dev(G["f_x"]), _dev(G["f_w"]), (1, 1, 1, 1)).cpu().numpy()
    assert close(y, G["f_y"])
    y = tsx.conv2d_f32(_dev(G["f_x"]), _dev(G["f_w"]), (0, 1, 2, 0), (2, 2), (1, 1), 0.5).cpu().numpy()
    assert close(y, G["f_y_s2"])
    assert close(tsx.inner_prod_f32(_dev(G["ip_a"]), _dev(G["ip_b"]), False).cpu().numpy(), G["ip_y"])
    assert close(tsx.inner_prod_f32(_dev(G["ip_a"]), _dev(G["ip_b"].T), True).cpu().numpy(), G["ip_yt"])
    wg = tsx.WinogradF63(_dev(G["wg_w"]), (1, 1, 1, 1))
    assert np.array_equal(bits(wg(_dev(G["wg_x"])).cpu().numpy()), bits(G["wg_y"]))
    wg = tsx.WinogradF63(_dev(G["wg_w"]), (1, 1, 1, 1), 0.25)
    assert np.array_equal(bits(wg(_dev(G["wg_x"])).cpu().numpy()), bits(G["wg_y_pv"]))
    wg = tsx.WinogradF23(_dev(G["wg_w"]), (1, 1, 1, 1))
    assert np.array_equal(bits(wg(_dev(G["wg_x"])).cpu().numpy()), bits(G["wg23_y"]))
    wg = tsx.WinogradF23(_dev(G["wg_w"]), (1, 1, 1, 1), 0.25)
    assert np.array_equal(bits(wg(_dev(G["wg_x"])).cpu().numpy()), bits(G["wg23_y_pv"]))
    g = tsx.GemmI8(_dev(G["g8_b"]))
    _, _, acc = g(_dev(G["g8_a"]), want_acc=True)
    assert np.array_equal(acc.cpu().numpy(), G["g8_c"])
