"""Operators of detection-style graphs beside the convolutions: depthwise_conv2d, concat, nearest resize2d and
Mish (softplus -> tanh -> mul).

CPU part: the oracle against the compiled reference operators (bitwise) and closed forms.  GPU part (marked
gpu): HIP kernels through the C ABI against the oracle -- bitwise for depthwise (same fused-multiply-add
order), concat and resize (copies), and bitwise for softplus, tanh and Mish too: the kernels restate the host C
library's expf operation for operation and evaluate log beyond float precision, so every rounded intermediate of
the chain is the host's (tests/test_mish_host.py holds the same arithmetic against the C library on the CPU).
The opt-in fast Mish (one hardware exponential and reciprocal) is held to 1e-4 relative + 1e-5 absolute.
"""
import numpy as np
import pytest

from _util import bits

DW_CASES = [
    # kernel, pads (t, b, l, r), strides, dilations, padding_value
    ((3, 3), (1, 1, 1, 1), (1, 1), (1, 1), 0.0),
    ((3, 3), (1, 1, 1, 1), (2, 2), (1, 1), 0.0),
    ((5, 3), (2, 1, 0, 1), (1, 2), (1, 1), 0.5),
    ((3, 3), (2, 2, 2, 2), (1, 1), (2, 2), 0.0),
    ((1, 1), (0, 0, 0, 0), (1, 1), (1, 1), 0.0),
    # 3x3 / stride 1 / column padding 1 on rows whose length is a multiple of 4: the vector-load path
    ((3, 3), (1, 1, 1, 1), (1, 1), (1, 1), 0.75),
    ((3, 3), (0, 2, 1, 1), (1, 1), (1, 1), -1.5),
]


def _x(seed, shape=(2, 6, 11, 9)):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def mish_fast_close(a, b):
    return np.all(np.abs(a.astype(np.float64) - b) <= 1e-4 * np.abs(b) + 1e-5)


@pytest.mark.parametrize("case", DW_CASES)
def test_oracle_depthwise_vs_reference(port, ref, case):
    k, pads, st, dl, pv = case
    x = _x(11)
    w = np.random.default_rng(12).standard_normal((1, 6, k[0], k[1])).astype(np.float32)
    a, b = port.depthwise_conv2d(x, w, pads, st, dl, pv), ref.depthwise_conv2d(x, w, pads, st, dl, pv)
    assert a.shape == b.shape and np.array_equal(bits(a), bits(b))
    # reference-independent: each channel is an ordinary one-channel convolution (fp64 bound)
    xp = np.full((2, 6, 11 + pads[0] + pads[1], 9 + pads[2] + pads[3]), pv, np.float64)
    xp[:, :, pads[0]:pads[0] + 11, pads[2]:pads[2] + 9] = x
    exp = np.zeros(a.shape)
    for i in range(k[0]):
        for j in range(k[1]):
            exp += w[0, :, i, j][None, :, None, None] * xp[:, :, i * dl[0]:i * dl[0] + st[0] * a.shape[2]:st[0],
                                                         j * dl[1]:j * dl[1] + st[1] * a.shape[3]:st[1]]
    assert np.abs(a - exp).max() < 1e-5


def test_oracle_resize_concat_mish_vs_reference(port, ref):
    x = _x(13)
    for ho, wo in ((22, 18), (11, 9), (7, 20), (33, 5)):
        assert np.array_equal(bits(port.resize_nearest(x, ho, wo)), bits(ref.resize_nearest(x, ho, wo)))
    assert np.array_equal(port.resize_nearest(x, 22, 18), x.repeat(2, axis=2).repeat(2, axis=3))   # 2x: pixel doubling
    parts = [x, x[:, :2], x[:, 1:5]]
    assert np.array_equal(port.concat(parts, 1), ref.concat(parts, 1))
    y = (_x(14, (3, 4, 50)) * 4)
    y.ravel()[:6] = [0.0, -0.0, 30.0, -30.0, 88.0, -100.0]
    assert np.array_equal(bits(port.softplus(y)), bits(ref.unary("softplus", y)))
    assert np.array_equal(bits(port.tanh(y)), bits(ref.unary("tanh", y)))
    composed = ref.mul(y, ref.unary("tanh", ref.unary("softplus", y)))
    assert np.array_equal(bits(port.mish(y)), bits(composed))
    y64 = y.astype(np.float64)
    small = np.abs(y64) < 20
    assert np.allclose(port.mish(y)[small], (y64 * np.tanh(np.log1p(np.exp(y64))))[small], rtol=2e-6, atol=1e-6)


# ------------------------------------------------------------------ HIP kernels

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
@pytest.mark.parametrize("case", DW_CASES)
def test_hip_depthwise(tsx, port, case):
    k, pads, st, dl, pv = case
    for shape in ((2, 6, 11, 9), (3, 70, 28, 28), (1, 3, 40, 64)):
        x = _x(21, shape)
        w = np.random.default_rng(22).standard_normal((1, shape[1], k[0], k[1])).astype(np.float32)
        bias = np.random.default_rng(23).standard_normal(shape[1]).astype(np.float32)
        got = tsx.depthwise_conv2d(_dev(x), _dev(w), pads, st, dl, pv).cpu().numpy()
        exp = port.depthwise_conv2d(x, w, pads, st, dl, pv)
        assert np.array_equal(bits(got), bits(exp))
        got = tsx.depthwise_conv2d(_dev(x), _dev(w), pads, st, dl, pv, bias=_dev(bias), act="relu").cpu().numpy()
        assert np.array_equal(bits(got), bits(port.relu(port.add_bias(exp, bias))))


@pytest.mark.gpu
def test_hip_resize_and_concat(tsx, port):
    x = _x(24, (2, 5, 13, 10))
    for ho, wo in ((26, 20), (13, 10), (7, 23), (40, 3)):
        assert np.array_equal(bits(tsx.resize_nearest(_dev(x), ho, wo).cpu().numpy()), bits(port.resize_nearest(x, ho, wo)))
    parts = [x, x[:, :2].copy(), x[:, 1:5].copy()]
    assert np.array_equal(tsx.concat_channels([_dev(p) for p in parts]).cpu().numpy(), port.concat(parts, 1))
    odd = [_x(25, (1, 3, 3, 3)), _x(26, (1, 2, 3, 3))]      # rows that are not multiples of 4 floats
    assert np.array_equal(tsx.concat_channels([_dev(p) for p in odd]).cpu().numpy(), port.concat(odd, 1))


@pytest.mark.gpu
def test_hip_mish(tsx, port):
    y = (_x(27, (3, 4, 500)) * 4)
    y.ravel()[:6] = [0.0, -0.0, 30.0, -30.0, 88.0, -100.0]
    got = tsx.mish(_dev(y)).cpu().numpy()
    assert np.array_equal(bits(got), bits(port.mish(y)))
    # fused behind an int8 convolution: conv -> add_bias -> mish, the values of the separate operators
    rng = np.random.default_rng(28)
    xq = rng.integers(-128, 128, (2, 64, 9, 9)).astype(np.int8)
    wq = rng.integers(-127, 128, (64, 64, 3, 3)).astype(np.int8)
    dq = rng.uniform(1e-4, 3e-4, 64).astype(np.float32)
    bias = rng.standard_normal(64).astype(np.float32)
    for strides in ((1, 1), (2, 2)):
        conv = tsx.Conv2dI8(_dev(wq), (1, 1, 1, 1), strides)
        exp = port.mish(port.conv2d_i8_fused(xq, wq, dq, bias, None, pads=(1, 1, 1, 1), strides=strides)[0])
        out = conv(_dev(xq), dq=_dev(dq), bias=_dev(bias), act="mish")[0].cpu().numpy()
        assert np.array_equal(bits(out), bits(exp))
        fast = conv(_dev(xq), dq=_dev(dq), bias=_dev(bias), act="mish_fast")[0].cpu().numpy()
        assert mish_fast_close(fast, exp) and not np.array_equal(bits(fast), bits(exp))


@pytest.mark.gpu
def test_hip_mish_dense_sweep(tsx, port):
    """softplus, tanh and Mish kernels on every 61st float in (-200, 200) and the special values, against the host's
    chain (the oracle calls the C library): Mish and tanh bit for bit, softplus bit for bit but for at most one value
    (one float in 2.26e9 has a softplus within 2^-50 of a rounding boundary)."""
    import torch
    u = np.arange(0, 1 << 32, 61, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    x = x[np.abs(x) < 200]
    x = np.concatenate([x, np.float32([np.inf, -np.inf, 1000.0, -1000.0, 88.8, 89.0, -103.9, -104.0, 3.4e38, -3.4e38])])
    xd = _dev(x)
    with np.errstate(all="ignore"):
        exp = {"mish": port.mish(x), "softplus": port.softplus(x), "tanh": port.tanh(x)}
    got = {"mish": tsx.mish(xd), "softplus": tsx.softplus(xd), "tanh": tsx.tanh(xd)}
    for name, budget in (("mish", 0), ("tanh", 0), ("softplus", 1)):
        g = got[name].cpu().numpy()
        bad = np.flatnonzero(bits(g) != bits(exp[name]))
        assert bad.size <= budget, (name, bad.size, x[bad[:5]], g[bad[:5]], exp[name][bad[:5]])
    nan = tsx.mish(_dev(np.float32([np.nan]))).cpu().numpy()
    assert np.isnan(nan).all()
