"""The C++ "hip" operators driven by name, like TenniS's operator test runner drives them
(bench(device) -> create(op, params) -> run(inputs)), checked against the CPU oracle and -- where
the compiled reference is present -- against the reference's own operator on device "cpu" given
the very same parameters and inputs."""
import numpy as np
import pytest

from _util import bits, c2_like

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from tennis_amd import operators
    operators.lib()
    return operators


def _maybe_ref():
    from oracle import ref as r
    return r if r.available() else None


def _close(a, b):
    return np.all(np.abs(a.astype(np.float64) - b) <= 1e-5 + 1e-4 * np.abs(b))


def test_quantize_operator(ops, port):
    rng = np.random.default_rng(500)
    for shape in [(1, 3, 7, 9), (4, 3, 7, 9), (32, 77)]:
        x = (rng.standard_normal(shape) * 40).astype(np.float32)
        x.ravel()[::3] = np.round(x.ravel()[::3]) + 0.5
        s = rng.uniform(0.5, 2, shape[0]).astype(np.float32)
        params = {"quantize_scale": s}
        got = ops.run_op("quantize", params, [x])
        assert got.dtype == np.int8 and got.shape == shape
        assert np.array_equal(got, port.quantize(x, s))
        ref = _maybe_ref()
        if ref:
            assert np.array_equal(got, ref.run_op("quantize", params, [x], x.size))
    with pytest.raises(ops.OperatorError):        # one scale per batch item (base_quantize.cpp:26)
        ops.run_op("quantize", {"quantize_scale": np.ones(3, np.float32)}, [np.zeros((2, 4), np.float32)])


@pytest.mark.parametrize("case", [
    (2, 8, 6, 6, 4, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (1, 5, 10, 9, 6, 3, 2, (2, 1, 0, 1), (1, 2), (2, 1)),
    (2, 16, 5, 5, 8, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),
    (3, 64, 14, 14, 96, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (2, 3, 19, 19, 16, 7, 7, (3, 3, 3, 3), (2, 2), (1, 1)),
])
def test_conv2d_quantized_operator(ops, port, case):
    n, c, h, w, cout, kh, kw, pads, st, dl = case
    rng = np.random.default_rng(501)
    x = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    wt = rng.integers(-128, 128, (cout, c, kh, kw)).astype(np.int8)
    params = ops.conv_params(pads, st, dl)
    params["dequantize_scales"] = rng.uniform(1e-4, 1e-2, cout).astype(np.float32)
    dtype, shape = ops.run_op("conv2d_quantized", params, [x, wt], infer_only=True)
    got = ops.run_op("conv2d_quantized", params, [x, wt])
    assert dtype == ops.FLOAT32 and tuple(shape) == got.shape          # no requantize: fp32 out
    exp = port.conv2d_quantized(x, wt, params["dequantize_scales"], pads, st, dl)
    assert np.array_equal(bits(got), bits(exp))
    ref = _maybe_ref()
    if ref:
        r = ref.run_op("conv2d_quantized", params, [x, wt], got.nbytes, threads=1)
        assert np.array_equal(bits(got), bits(r))


def test_operator_chain_quantize_conv_bias_relu(ops, port):
    """The graph fragment of BASELINE config 2 as four separate operators, small batch."""
    rng = np.random.default_rng(502)
    x, x_scales, wq, dq, bias = c2_like(rng, 3, 64, 14, 14, 64)
    params = ops.conv_params((1, 1, 1, 1))
    params["dequantize_scales"] = dq
    xq = ops.run_op("quantize", {"quantize_scale": x_scales}, [x])
    y = ops.run_op("conv2d_quantized", params, [xq, wq])
    y = ops.run_op("add_bias", {"dim": np.array([1], np.int32)}, [y, bias])
    y = ops.run_op("relu", {}, [y])
    exp, _ = port.conv2d_i8_fused(port.quantize(x, x_scales), wq, dq, bias, "relu", pads=(1, 1, 1, 1))
    assert np.array_equal(bits(y), bits(exp))
    ref = _maybe_ref()
    if ref:
        r = ref.relu(ref.add_bias(ref.conv2d_quantized(ref.quantize(x, x_scales), wq, dq, pads=(1, 1, 1, 1)), bias))
        assert np.array_equal(bits(y), bits(r))


def test_conv2d_inner_prod_winograd_operators(ops, port):
    rng = np.random.default_rng(503)
    x = rng.uniform(-1, 1, (2, 16, 13, 11)).astype(np.float32)
    wt = (rng.standard_normal((24, 16, 3, 3)) * 0.1).astype(np.float32)
    params = ops.conv_params((1, 1, 1, 1))
    got = ops.run_op("conv2d", params, [x, wt])
    assert _close(got, port.conv2d_f32(x, wt, (1, 1, 1, 1)))
    wparams = {k: params[k] for k in ("format", "padding", "padding_value")}
    # the skeleton picks the mode as the reference does: F(2,3) here, F(6,3) for Cin*Cout >= 256*256
    # on maps larger than 16x16 (src/kernels/common/function.cpp:154-173)
    gotw = ops.run_op("conv2d_winograd", wparams, [x, wt])
    assert np.array_equal(bits(gotw), bits(port.winograd_f23(x, wt, (1, 1, 1, 1))))
    xb = rng.uniform(-1, 1, (1, 256, 18, 17)).astype(np.float32)
    wb = (rng.standard_normal((256, 256, 3, 3)) * 0.02).astype(np.float32)
    gotb = ops.run_op("conv2d_winograd", wparams, [xb, wb])
    assert np.array_equal(bits(gotb), bits(port.winograd_f63(xb, wb, (1, 1, 1, 1))))
    lhs = rng.standard_normal((5, 4, 6, 2)).astype(np.float32)          # flattened to [5, 48]
    rhs = rng.standard_normal((48, 10)).astype(np.float32)
    gotp = ops.run_op("inner_prod", {}, [lhs, rhs])
    assert gotp.shape == (5, 10) and _close(gotp, port.inner_prod_f32(lhs.reshape(5, 48), rhs))
    gott = ops.run_op("inner_prod", {"transpose": np.array([True])}, [lhs, np.ascontiguousarray(rhs.T)])
    assert _close(gott, port.inner_prod_f32(lhs.reshape(5, 48), rhs))
    ref = _maybe_ref()
    if ref:
        assert _close(got, ref.run_op("conv2d", params, [x, wt], got.nbytes))
        assert _close(gotp, ref.run_op("inner_prod", {}, [lhs, rhs], gotp.nbytes))


def test_elementwise_operators(ops, port):
    rng = np.random.default_rng(504)
    x = rng.standard_normal((2, 3, 5, 7)).astype(np.float32)
    x.ravel()[:6] = [-1.0, -0.0, 0.0, np.nan, -1e-45, 2.0]
    x.ravel()[-3:] = [-0.0, np.nan, -2.0]                               # 210 elements: last two are the scalar tail
    b = rng.standard_normal(3).astype(np.float32)
    assert np.array_equal(bits(ops.run_op("add_bias", {"format": "NCHW"}, [x, b])), bits(port.add_bias(x, b)))
    assert np.array_equal(bits(ops.run_op("relu", {}, [x])), bits(port.relu(x)))
    got = ops.run_op("leaky_relu", {"scale": np.array([0.1], np.float32)}, [x])
    assert np.array_equal(bits(got), bits(port.leaky_relu(x, 0.1)))
    ref = _maybe_ref()
    if ref:
        assert np.array_equal(bits(got), bits(ref.leaky_relu(x, 0.1)))
    with pytest.raises(ops.OperatorError, match="Miss matched"):
        ops.run_op("add_bias", {"dim": np.array([1], np.int32)}, [x, np.zeros(4, np.float32)])


def _pool_params(kind, ksize, strides, pads, white=False):
    return {"format": "NCHW", "type": np.array([{"max": 0, "avg": 1}[kind]], np.int32),
            "padding": np.array([[0, 0], [0, 0], [pads[0], pads[1]], [pads[2], pads[3]]], np.int32),
            "padding_type": np.array([3 if white else 0], np.int32),
            "ksize": np.array([1, 1, ksize[0], ksize[1]], np.int32),
            "stride": np.array([1, 1, strides[0], strides[1]], np.int32)}


def test_glue_operators(ops, port):
    """pooling2d, global_pooling2d, add (equal shapes, scalar, bias, general broadcast, either side)
    and depthwise_conv2d created by name; bitwise against the oracle."""
    rng = np.random.default_rng(505)
    x = rng.standard_normal((2, 5, 13, 11)).astype(np.float32)
    for kind, k, s, pads, white in (("max", (3, 3), (2, 2), (1, 1, 1, 1), False), ("avg", (2, 3), (2, 1), (1, 0, 1, 1), False),
                                    ("avg", (3, 3), (1, 1), (1, 1, 1, 1), True), ("max", (5, 5), (1, 1), (2, 2, 2, 2), False),
                                    # ceil mode puts the last row of windows behind the map: the average of nothing is 0
                                    ("avg", (3, 2), (2, 1), (1, 2, 0, 1), False), ("avg", (3, 2), (2, 1), (1, 2, 0, 1), True)):
        got = ops.run_op("pooling2d", _pool_params(kind, k, s, pads, white), [x])
        want = port.pooling2d(x, kind, k, s, pads, white)
        assert got.shape == want.shape and np.array_equal(bits(got), bits(want)), (kind, k, s, pads, white)
    for kind in ("max", "avg"):
        got = ops.run_op("global_pooling2d", {"format": "NCHW", "type": np.array([{"max": 0, "avg": 1}[kind]], np.int32)}, [x])
        assert got.shape == (2, 5, 1, 1) and np.array_equal(bits(got), bits(port.global_pooling2d(x, kind)))
    for shape in ((2, 5, 13, 11), (1,), (1, 5, 1, 1), (5, 1, 1), (2, 1, 13, 1), (13, 11), (1, 1, 1, 11)):
        b = rng.standard_normal(shape).astype(np.float32)
        for lhs, rhs in ((x, b), (b, x)):
            got = ops.run_op("add", {}, [lhs, rhs])
            want = lhs + rhs                                   # one IEEE addition per element
            assert got.shape == want.shape and np.array_equal(bits(got), bits(want)), shape
    with pytest.raises(ops.OperatorError, match="windows outside"):      # the reference's MAX reads behind the plane there
        ops.run_op("pooling2d", _pool_params("max", (3, 2), (2, 1), (1, 2, 0, 1)), [x])
    with pytest.raises(ops.OperatorError, match="Can not reduce shape"):
        ops.run_op("add", {}, [x, np.zeros((2, 4, 13, 11), np.float32)])
    w = rng.standard_normal((1, 5, 3, 3)).astype(np.float32)
    for pads, strides, dil, pv in (((1, 1, 1, 1), (1, 1), (1, 1), 0.0), ((0, 2, 1, 0), (2, 1), (1, 2), 0.5)):
        params = ops.conv_params(pads, strides, dil, pv)
        got = ops.run_op("depthwise_conv2d", params, [x, w])
        want = port.depthwise_conv2d(x, w, pads, strides, dil, pv)
        assert got.shape == want.shape and np.array_equal(bits(got), bits(want)), (pads, strides, dil)
    with pytest.raises(ops.OperatorError):                     # multiplier > 1 is depthwise_conv2d_v2's business
        ops.run_op("depthwise_conv2d", ops.conv_params((1, 1, 1, 1)), [x, np.zeros((2, 5, 3, 3), np.float32)])


def test_operator_errors_at_run_time(ops):
    params = ops.conv_params((1, 1, 1, 1))
    params["dequantize_scales"] = np.ones(4, np.float32)
    x = np.zeros((1, 8, 5, 5), np.int8)
    with pytest.raises(ops.OperatorError):        # weight channels differ from input channels
        ops.run_op("conv2d_quantized", params, [x, np.zeros((4, 7, 3, 3), np.int8)])
    with pytest.raises(ops.OperatorError):        # one dequantize scale per output channel
        ops.run_op("conv2d_quantized", params, [x, np.zeros((5, 8, 3, 3), np.int8)])
    with pytest.raises(ops.OperatorError):        # input must be int8
        ops.run_op("conv2d_quantized", params, [x.astype(np.float32), np.zeros((4, 8, 3, 3), np.float32)])
    with pytest.raises(ops.OperatorNotFound):
        ops.run_op("softmax", {}, [np.zeros((2, 2), np.float32)])


def test_v2_operators_equal_their_plain_twins(ops):
    """conv2d_v2 / depthwise_conv2d_v2 / conv2d_winograd_v2 / pooling2d_v2 take padding (ksize, stride) as
    inputs (src/kernels/cpu/conv2d_v2.cpp:60-92) and must give what the plain operator gives for the same values."""
    rng = np.random.default_rng(507)
    x = rng.standard_normal((2, 6, 12, 10)).astype(np.float32)
    w = (rng.standard_normal((7, 6, 3, 3)) * 0.2).astype(np.float32)
    for pads in ((1, 1, 1, 1), (0, 2, 1, 0)):
        full = ops.conv_params(pads, (2, 1), (1, 1), 0.5)
        v2 = {k: v for k, v in full.items() if k != "padding"}
        got = ops.run_op("conv2d_v2", v2, [x, full["padding"], w])
        assert np.array_equal(bits(got), bits(ops.run_op("conv2d", full, [x, w])))
        assert ops.run_op("conv2d_v2", v2, [x, full["padding"], w], infer_only=True)[1] == got.shape
        wd = w[:1].copy()
        got = ops.run_op("depthwise_conv2d_v2", v2, [x, full["padding"].astype(np.int64), wd])   # cast to INT32 inside
        assert np.array_equal(bits(got), bits(ops.run_op("depthwise_conv2d", full, [x, wd])))
        wino = {k: full[k] for k in ("format", "padding_value")}
        got = ops.run_op("conv2d_winograd_v2", wino, [x, full["padding"], w])
        assert np.array_equal(bits(got), bits(ops.run_op("conv2d_winograd", dict(wino, padding=full["padding"]), [x, w])))
        pool = _pool_params("avg", (3, 2), (2, 1), (pads[0], 1, pads[2], pads[3]), True)   # every window touches the map
        got = ops.run_op("pooling2d_v2", {k: pool[k] for k in ("format", "type", "padding_type")},
                         [x, pool["padding"], pool["ksize"], pool["stride"]])
        assert np.array_equal(bits(got), bits(ops.run_op("pooling2d", pool, [x])))
    with pytest.raises(ops.OperatorError, match="expects 3 inputs"):
        ops.run_op("conv2d_v2", v2, [x, w])
    with pytest.raises(ops.OperatorError):      # stride is required (conv2d_v2.cpp:17)
        ops.run_op("conv2d_v2", {"format": "NCHW"}, [x, full["padding"], w])


def test_concat_and_resize2d_operators(ops, port):
    """concat (any axis, 4-byte elements) and _resize2d (nearest) created by name: exact copies."""
    rng = np.random.default_rng(508)
    a, b, c = (rng.standard_normal(s).astype(np.float32) for s in ((2, 5, 7, 6), (2, 3, 7, 6), (2, 1, 7, 6)))
    got = ops.run_op("concat", {"dim": np.array([1], np.int32)}, [a, b, c])
    assert np.array_equal(bits(got), bits(np.concatenate([a, b, c], axis=1)))
    got = ops.run_op("concat", {"dim": np.array([-4], np.int32)}, [a, a])
    assert np.array_equal(bits(got), bits(np.concatenate([a, a], axis=0)))
    i1, i2 = rng.integers(-9, 9, (3, 4, 5)).astype(np.int32), rng.integers(-9, 9, (3, 4, 2)).astype(np.int32)
    got = ops.run_op("concat", {"dim": np.array([2], np.int32)}, [i1, i2])
    assert got.dtype == np.int32 and np.array_equal(got, np.concatenate([i1, i2], axis=2))
    assert np.array_equal(ops.run_op("concat", {"dim": np.array([0], np.int32)}, [a]), a)      # one input: itself
    with pytest.raises(ops.OperatorError, match="Can not concat"):
        ops.run_op("concat", {"dim": np.array([1], np.int32)}, [a, np.zeros((2, 3, 7, 5), np.float32)])
    with pytest.raises(ops.OperatorError, match="Can not concat"):
        ops.run_op("concat", {"dim": np.array([1], np.int32)}, [a, b.astype(np.float64)])
    with pytest.raises(ops.OperatorError, match="Concat dim must in"):
        ops.run_op("concat", {"dim": np.array([4], np.int32)}, [a, b])
    nearest = {"type": np.array([2], np.int32)}
    for ho, wo in ((14, 12), (9, 11), (7, 6), (3, 13)):
        size = np.array([-1, -1, ho, wo], np.int32)
        assert ops.run_op("_resize2d", nearest, [a, size], infer_only=True)[1] == (2, 5, ho, wo)
        got = ops.run_op("_resize2d", nearest, [a, size])
        assert np.array_equal(bits(got), bits(port.resize_nearest(a, ho, wo))), (ho, wo)
    # the default type is LINEAR: the "hip" class hands that to the host operator, which this stand-alone
    # build (API slice, no host operators) does not contain; inside TenniS it runs (tests/test_gpu_intree.py)
    with pytest.raises(ops.OperatorError, match="need the host operator"):
        ops.run_op("_resize2d", {}, [a, np.array([-1, -1, 14, 12], np.int32)])
    with pytest.raises(ops.OperatorError, match="Can not resize"):
        ops.run_op("_resize2d", nearest, [a, np.array([-1, 4, 0, 12], np.int32)])


def test_mish_composition_operators(ops, port):
    """softplus, tanh and mul -- the nodes TenniS graphs compose Mish from -- against the oracle bit for bit (the
    kernels evaluate the host C library's expf operation for operation and log beyond float precision), and the fused
    Mish kernel against their composition bit for bit: a graph gives the same values whether or not the backend
    fuses the three nodes."""
    from tennis_amd import capi
    rng = np.random.default_rng(509)
    x = (rng.standard_normal((2, 5, 13, 11)) * 4).astype(np.float32)
    x.flat[:6] = [0.0, -0.0, 30.0, -30.0, 88.0, -88.0]
    sp = ops.run_op("softplus", {}, [x])
    assert np.array_equal(bits(sp), bits(port.softplus(x)))
    th = ops.run_op("tanh", {}, [x])
    assert np.array_equal(bits(th), bits(port.tanh(x)))
    b = rng.standard_normal((1, 5, 1, 1)).astype(np.float32)
    for lhs, rhs in ((x, x[::-1].copy()), (x, b), (b, x), (x, np.float32([2.5]))):
        got = ops.run_op("mul", {}, [lhs, rhs])
        assert np.array_equal(bits(got), bits(lhs * rhs))
    mish = ops.run_op("mul", {}, [x, ops.run_op("tanh", {}, [sp])])
    import torch
    fused = capi.mish(torch.from_numpy(x).cuda()).cpu().numpy()
    assert np.array_equal(bits(fused), bits(mish)) and np.array_equal(bits(mish), bits(port.mish(x)))
    with pytest.raises(ops.OperatorError):
        ops.run_op("softplus", {}, [x.astype(np.float64)])
