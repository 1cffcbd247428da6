"""Pins the fp32 half of the CPU oracle: GEMM (pack8 + kernel_8x8 order), conv2d, inner_prod and
Winograd F(6,3).  Independent checks: fp64 brute force (tolerance), closed forms (all-ones kernel =
box sum, 1x1 conv = GEMM), and the compiled reference (bit-exact where the reference's order is
restated exactly)."""
import numpy as np
import pytest


def _conv_fp64(x, w, pads, strides=(1, 1), dilations=(1, 1), pad_value=0.0):
    n, c, h, wd = x.shape
    cout, _, kh, kw = w.shape
    ho = (h + pads[0] + pads[1] - (dilations[0] * (kh - 1) + 1)) // strides[0] + 1
    wo = (wd + pads[2] + pads[3] - (dilations[1] * (kw - 1) + 1)) // strides[1] + 1
    xp = np.full((n, c, h + pads[0] + pads[1], wd + pads[2] + pads[3]), pad_value, np.float64)
    xp[:, :, pads[0]:pads[0] + h, pads[2]:pads[2] + wd] = x
    out = np.zeros((n, cout, ho, wo))
    for r in range(kh):
        for s in range(kw):
            win = xp[:, :, r * dilations[0]: r * dilations[0] + (ho - 1) * strides[0] + 1: strides[0],
                     s * dilations[1]: s * dilations[1] + (wo - 1) * strides[1] + 1: strides[1]]
            out += np.einsum("nchw,oc->nohw", win, w[:, :, r, s].astype(np.float64))
    return out


def _close(a, b, rel=1e-4, ab=1e-5):
    """north-star tolerance: 1e-4 relative / 1e-5 absolute."""
    return np.all(np.abs(a - b) <= ab + rel * np.abs(b))


def test_gemm_f32_vs_fp64(port):
    rng = np.random.default_rng(20)
    for m, n, k in [(8, 8, 4), (16, 24, 64), (9, 13, 37), (64, 100, 64), (3, 5, 7)]:
        a = rng.standard_normal((m, k)).astype(np.float32)
        b = rng.standard_normal((k, n)).astype(np.float32)
        assert _close(port.gemm_f32(a, b), a.astype(np.float64) @ b.astype(np.float64))


def test_gemm_f32_is_sequential_fma_chain(port):
    # k-ascending single FMA chain where M%8==0 and N%8==0: reproduce it in exact rational steps
    rng = np.random.default_rng(21)
    a = rng.standard_normal((8, 19)).astype(np.float32)
    b = rng.standard_normal((19, 8)).astype(np.float32)
    exp = np.zeros((8, 8), np.float32)
    for i in range(8):
        for j in range(8):
            acc = np.float32(0)
            for kk in range(19):
                acc = np.float32(np.float64(a[i, kk]) * np.float64(b[kk, j]) + np.float64(acc))  # exact product, one rounding
            exp[i, j] = acc
    assert np.array_equal(port.gemm_f32(a, b).view(np.int32), exp.view(np.int32))


def test_gemm_f32_vs_reference_bitwise(port, ref):
    rng = np.random.default_rng(22)
    for m, n, k in [(8, 8, 4), (64, 96, 64), (64, 100, 64), (13, 21, 30), (7, 100, 9), (16, 3, 5)]:
        a = rng.standard_normal((m, k)).astype(np.float32)
        b = rng.standard_normal((k, n)).astype(np.float32)
        assert np.array_equal(port.gemm_f32(a, b).view(np.int32), ref.gemm_f32(a, b).view(np.int32)), (m, n, k)


CONV_CASES = [
    (1, 8, 12, 12, 8, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (2, 5, 9, 7, 6, 3, 3, (0, 0, 0, 0), (2, 2), (1, 1)),
    (2, 16, 8, 8, 8, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),
    (1, 3, 10, 11, 4, 3, 2, (2, 1, 0, 1), (1, 2), (2, 1)),
    (1, 64, 56, 56, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # BASELINE config 1
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_f32(port, ref, case):
    n, c, h, w, cout, kh, kw, pads, st, dl = case
    rng = np.random.default_rng(23)
    x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, c, kh, kw)) * np.sqrt(2.0 / (c * kh * kw))).astype(np.float32)
    got = port.conv2d_f32(x, wt, pads, st, dl)
    assert _close(got, _conv_fp64(x, wt, pads, st, dl))
    exp = ref.conv2d(x, wt, pads, st, dl, threads=1)
    assert np.array_equal(got.view(np.int32), exp.view(np.int32))


def test_conv2d_f32_closed_forms(port):
    rng = np.random.default_rng(24)
    x = rng.integers(-8, 9, (1, 4, 6, 6)).astype(np.float32)
    ones = np.ones((2, 4, 3, 3), np.float32)
    got = port.conv2d_f32(x, ones, (1, 1, 1, 1))
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    box = sum(xp[:, :, r:r + 6, s:s + 6] for r in range(3) for s in range(3)).sum(axis=1, keepdims=True)
    assert np.array_equal(got, np.repeat(box, 2, axis=1))       # small integers: exact in fp32
    # padding_value contributes to border outputs
    got = port.conv2d_f32(x, ones, (1, 1, 1, 1), padding_value=2.0)
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)), constant_values=2.0)
    box = sum(xp[:, :, r:r + 6, s:s + 6] for r in range(3) for s in range(3)).sum(axis=1, keepdims=True)
    assert np.array_equal(got, np.repeat(box, 2, axis=1))


def test_inner_prod_f32(port, ref):
    rng = np.random.default_rng(25)
    lhs = rng.standard_normal((12, 96)).astype(np.float32)
    rhs = rng.standard_normal((96, 20)).astype(np.float32)
    a = port.inner_prod_f32(lhs, rhs)
    assert _close(a, lhs.astype(np.float64) @ rhs.astype(np.float64))
    assert np.array_equal(a.view(np.int32), ref.inner_prod(lhs, rhs).view(np.int32))
    t = port.inner_prod_f32(lhs, np.ascontiguousarray(rhs.T), transpose=True)
    assert np.array_equal(t.view(np.int32), ref.inner_prod(lhs, np.ascontiguousarray(rhs.T), transpose=True).view(np.int32))


WINO_CASES = [
    (1, 8, 12, 12, 8, (1, 1, 1, 1)),       # output 12x12: exact multiple of the 6x6 tile
    (2, 16, 9, 11, 8, (1, 1, 1, 1)),       # ragged: padded to 12x12 tiles and cut back
    (1, 8, 10, 10, 16, (0, 0, 0, 0)),      # no padding: output 8x8
    (1, 5, 7, 7, 3, (2, 1, 1, 2)),         # asymmetric padding, channel counts off the 8-blocks
    (1, 64, 56, 56, 64, (1, 1, 1, 1)),     # BASELINE config 1 through F(6,3)
]


@pytest.mark.parametrize("mode", ["f63", "f23"])
@pytest.mark.parametrize("case", WINO_CASES)
def test_winograd(port, ref, case, mode):
    n, c, h, w, cout, pads = case
    rng = np.random.default_rng(26)
    x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, c, 3, 3)) * np.sqrt(2.0 / (c * 9))).astype(np.float32)
    got = getattr(port, "winograd_" + mode)(x, wt, pads)
    # F(6,3) in fp32 is itself ~5e-5 off an exact convolution at these sizes
    assert np.abs(got - _conv_fp64(x, wt, pads)).max() < 2e-4
    exp = ref.winograd(x, wt, pads, f63=mode == "f63", threads=1)
    assert np.array_equal(got.view(np.int32), exp.view(np.int32))


@pytest.mark.parametrize("mode", ["f63", "f23"])
def test_winograd_padding_value(port, ref, mode):
    rng = np.random.default_rng(27)
    x = rng.uniform(-1, 1, (1, 8, 9, 9)).astype(np.float32)
    wt = rng.standard_normal((8, 8, 3, 3)).astype(np.float32) * 0.1
    got = getattr(port, "winograd_" + mode)(x, wt, (1, 1, 1, 1), padding_value=0.5)
    exp = ref.winograd(x, wt, (1, 1, 1, 1), f63=mode == "f63", padding_value=0.5, threads=1)
    assert np.array_equal(got.view(np.int32), exp.view(np.int32))
    assert np.abs(got - _conv_fp64(x, wt, (1, 1, 1, 1), pad_value=0.5)).max() < 2e-4


def test_winograd_all_ones_kernel_is_a_box_sum(port):
    """Reference-independent anchor (the reference's own test/winograd.cpp uses the same input): an
    all-ones 3x3 kernel on small integers makes every transform exact, so both modes must equal the
    3x3 box sum."""
    rng = np.random.default_rng(28)
    x = rng.integers(-4, 5, (1, 2, 9, 10)).astype(np.float32)
    wt = np.ones((3, 2, 3, 3), np.float32)
    box = _conv_fp64(x, wt, (1, 1, 1, 1)).astype(np.float32)
    assert np.array_equal(port.winograd_f23(x, wt, (1, 1, 1, 1)), box)
    assert np.abs(port.winograd_f63(x, wt, (1, 1, 1, 1)) - box).max() < 1e-4
