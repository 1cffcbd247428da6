"""Pins the int8 half of the CPU oracle (oracle/oracle.cpp).

Each oracle function is checked against something it does not share code with:
known-answer vectors, brute force in numpy integers, closed forms, and -- where
oracle/_ref was built -- the compiled TenniS reference itself, bit for bit.
"""
import numpy as np
import pytest


def _brute_conv_i32(x, w, pads, strides, dilations, pad_value=0):
    n, c, h, wd = x.shape
    cout, _, kh, kw = w.shape
    ho = (h + pads[0] + pads[1] - (dilations[0] * (kh - 1) + 1)) // strides[0] + 1
    wo = (wd + pads[2] + pads[3] - (dilations[1] * (kw - 1) + 1)) // strides[1] + 1
    ext_h = max(h + pads[0] + pads[1], (ho - 1) * strides[0] + dilations[0] * (kh - 1) + 1)
    ext_w = max(wd + pads[2] + pads[3], (wo - 1) * strides[1] + dilations[1] * (kw - 1) + 1)
    xp = np.full((n, c, ext_h, ext_w), pad_value, np.int64)
    xp[:, :, pads[0]:pads[0] + h, pads[2]:pads[2] + wd] = x
    out = np.zeros((n, cout, ho, wo), np.int64)
    for r in range(kh):
        for s in range(kw):
            win = xp[:, :, r * dilations[0]: r * dilations[0] + (ho - 1) * strides[0] + 1: strides[0],
                     s * dilations[1]: s * dilations[1] + (wo - 1) * strides[1] + 1: strides[1]]
            out += np.einsum("nchw,oc->nohw", win, w[:, :, r, s].astype(np.int64))
    return out


# ---------------------------------------------------------------- quantize

# Known-answer vectors of both rounding paths of src/kernels/cpu/quantize.cpp:70-125
# (a single scale: first 8 elements round-half-even through the AVX convert, tail of 3
# half-away-from-zero; several scales: every element half-away).
KAT = np.array([.5, 1.5, 2.5, -.5, -1.5, 3.5, 4.5, 5.5, .5, 1.5, 2.5], np.float32)


def test_quantize_known_answers(port):
    assert port.quantize(KAT.reshape(1, 11), [1.0]).ravel().tolist() == [0, 2, 2, 0, -2, 4, 4, 6, 1, 2, 3]
    two = port.quantize(np.stack([KAT, KAT]), [1.0, 1.0])
    assert two.tolist() == [[1, 2, 3, -1, -2, 4, 5, 6, 1, 2, 3]] * 2


def test_quantize_clamp_and_groups(port):
    x = np.array([[300.0, -300.0, 127.4, 127.5, -128.5, -129.0, 0.49, -0.49],
                  [1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0]], np.float32)
    q = port.quantize(x, [1.0, 10.0])
    assert q[0].tolist() == [127, -128, 127, 127, -128, -128, 0, 0]
    assert q[1].tolist() == [10, 20, 30, 40, 50, 60, 70, 80]
    # ragged groups: ceil(7/3)=3 elements for the first two scales, 1 for the last
    r = port.quantize(np.ones(7, np.float32), [1.0, 2.0, 3.0])
    assert r.tolist() == [1, 1, 1, 2, 2, 2, 3]


def test_quantize_matches_numpy_closed_form(port):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((4, 1003)).astype(np.float32) * 40
    s = rng.uniform(0.5, 3.0, 4).astype(np.float32)
    prod = x * s[:, None]                      # fp32 product
    away = np.clip(np.sign(prod) * np.floor(np.abs(prod).astype(np.float64) + 0.5), -128, 127).astype(np.int8)
    assert np.array_equal(port.quantize(x, s), away)
    one = x[:1, :1003]
    p1 = one * s[0]
    rne = np.clip(np.rint(p1), -128, 127).astype(np.int8)
    got = port.quantize(one, s[:1])
    assert np.array_equal(got[0, :1000], rne[0, :1000])
    assert np.array_equal(got[0, 1000:], away[0, 1000:] if False else
                          np.clip(np.sign(p1[0, 1000:]) * np.floor(np.abs(p1[0, 1000:]) + 0.5), -128, 127)
                          .astype(np.int8))


def test_quantize_vs_reference(port, ref):
    rng = np.random.default_rng(2)
    for shape, ns in [((1, 3, 7, 9), 1), ((5, 3, 7, 9), 5), ((32, 77), 32), ((1, 8), 1), ((1, 5), 1)]:
        x = (rng.standard_normal(shape) * 50).astype(np.float32)
        # put exact .5 products in: x = k + 0.5 with scale 1
        x.ravel()[::3] = np.round(x.ravel()[::3]) + 0.5
        s = np.ones(ns, np.float32) if ns == 1 else rng.uniform(0.25, 2, ns).astype(np.float32)
        assert np.array_equal(port.quantize(x, s), ref.quantize(x, s)), shape
    # non-finite and out-of-range inputs follow the x86 conversion ("integer indefinite" -> -128)
    x = np.array([[np.inf, -np.inf, np.nan, 3e9, -3e9, 1e20, 127.5, -128.5, 2147483520.0, 1.0, 2.0]], np.float32)
    assert np.array_equal(port.quantize(x, [1.0]), ref.quantize(x, [1.0]))
    x2 = np.stack([x[0], x[0]])
    assert np.array_equal(port.quantize(x2, [1.0, 1.0]), ref.quantize(x2, [1.0, 1.0]))


# ---------------------------------------------------------------- im2col / gemm

def test_im2col_brute(port):
    rng = np.random.default_rng(3)
    x = rng.integers(-128, 128, (3, 5, 6)).astype(np.int8)
    for kh, kw, pads, st, dl in [(3, 3, (1, 1, 1, 1), (1, 1), (1, 1)), (2, 3, (0, 1, 2, 0), (2, 1), (1, 2)),
                                 (1, 1, (0, 0, 0, 0), (1, 1), (1, 1)), (3, 2, (2, 2, 1, 1), (2, 2), (2, 1))]:
        col = port.im2col(x, kh, kw, pads, st, dl, padding_value=7)
        ho, wo = port.out_hw(5, 6, kh, kw, pads, st, dl)
        exp = np.empty((3 * kh * kw, ho * wo), np.int8)
        for c in range(3):
            for r in range(kh):
                for s in range(kw):
                    for y in range(ho):
                        for xx in range(wo):
                            iy, ix = y * st[0] - pads[0] + r * dl[0], xx * st[1] - pads[2] + s * dl[1]
                            v = x[c, iy, ix] if 0 <= iy < 5 and 0 <= ix < 6 else 7
                            exp[(c * kh + r) * kw + s, y * wo + xx] = v
        assert np.array_equal(col, exp)


def test_gemm_i8_exact(port):
    rng = np.random.default_rng(4)
    for m, n, k in [(1, 1, 1), (7, 5, 13), (64, 33, 257), (3, 130, 2304)]:
        a = rng.integers(-128, 128, (m, k)).astype(np.int8)
        b = rng.integers(-128, 128, (k, n)).astype(np.int8)
        exp = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.int32)
        assert np.array_equal(port.gemm_i8(a, b), exp)
        assert np.array_equal(port.gemm_i8(a, b, faithful=True), exp)
    # extreme operands: -128 * -128 * K stays far inside int32
    a = np.full((2, 2304), -128, np.int8)
    b = np.full((2304, 2), -128, np.int8)
    assert (port.gemm_i8(a, b) == 128 * 128 * 2304).all()


def test_gemm_i8_vs_reference(port, ref):
    rng = np.random.default_rng(5)
    a = rng.integers(-128, 128, (9, 70)).astype(np.int8)
    b = rng.integers(-128, 128, (70, 11)).astype(np.int8)
    assert np.array_equal(port.gemm_i8(a, b), ref.gemm_i8(a, b))


# ---------------------------------------------------------------- conv2d_quantized

CONV_CASES = [
    # n, c, h, w, cout, kh, kw, pads(t,b,l,r), strides, dilations
    (2, 8, 6, 6, 4, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (1, 3, 9, 7, 5, 3, 3, (0, 0, 0, 0), (2, 2), (1, 1)),
    (2, 16, 5, 5, 8, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),      # 1x1 fast path (no im2col)
    (1, 4, 8, 8, 3, 1, 1, (0, 0, 0, 0), (2, 2), (1, 1)),       # 1x1 strided: goes through im2col
    (1, 5, 10, 9, 6, 3, 2, (2, 1, 0, 1), (1, 2), (2, 1)),      # asymmetric pads, dilation
    (3, 2, 7, 7, 7, 7, 7, (3, 3, 3, 3), (2, 2), (1, 1)),       # stem-like 7x7/2
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_quantized_brute(port, case):
    n, c, h, w, cout, kh, kw, pads, st, dl = case
    rng = np.random.default_rng(6)
    x = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    wt = rng.integers(-128, 128, (cout, c, kh, kw)).astype(np.int8)
    dq = rng.uniform(1e-4, 1e-2, cout).astype(np.float32)
    out, acc = port.conv2d_quantized(x, wt, dq, pads, st, dl, return_acc=True)
    exp = _brute_conv_i32(x, wt, pads, st, dl)
    assert np.array_equal(acc, exp.astype(np.int32))
    # closed form: one IEEE single multiply of the RNE-converted accumulator
    assert np.array_equal(out.view(np.int32), (exp.astype(np.float32) * dq[None, :, None, None]).view(np.int32))
    out_f = port.conv2d_quantized(x, wt, dq, pads, st, dl, faithful=True)
    assert np.array_equal(out_f.view(np.int32), out.view(np.int32))


def test_conv2d_quantized_padding_value(port):
    rng = np.random.default_rng(7)
    x = rng.integers(-128, 128, (1, 3, 4, 4)).astype(np.int8)
    wt = rng.integers(-128, 128, (2, 3, 3, 3)).astype(np.int8)
    _, acc = port.conv2d_quantized(x, wt, np.ones(2, np.float32), (1, 1, 1, 1), padding_value=3.7, return_acc=True)
    assert np.array_equal(acc, _brute_conv_i32(x, wt, (1, 1, 1, 1), (1, 1), (1, 1), pad_value=3))


def test_conv2d_quantized_large_acc_rounding(port):
    # |acc| above 2^24 is not exactly representable: the int->float convert must round to nearest even
    x = np.full((1, 2304 // 9, 3, 3), 127, np.int8)
    wt = np.full((1, 2304 // 9, 3, 3), 127, np.int8)
    wt[0, 0, 0, 0] = 126
    out, acc = port.conv2d_quantized(x, wt, np.array([1.0], np.float32), return_acc=True)
    assert acc[0, 0, 0, 0] == 127 * 127 * 2304 - 127
    assert out[0, 0, 0, 0] == np.float32(acc[0, 0, 0, 0])


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_quantized_vs_reference(port, ref, case):
    n, c, h, w, cout, kh, kw, pads, st, dl = case
    rng = np.random.default_rng(8)
    x = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    wt = rng.integers(-128, 128, (cout, c, kh, kw)).astype(np.int8)
    dq = rng.uniform(1e-4, 1e-2, cout).astype(np.float32)
    got = port.conv2d_quantized(x, wt, dq, pads, st, dl)
    exp = ref.conv2d_quantized(x, wt, dq, pads, st, dl, threads=1)
    assert np.array_equal(got.view(np.int32), exp.view(np.int32))


# ---------------------------------------------------------------- bias / activations / epilogue

SPECIAL = np.array([-1.0, -0.0, 0.0, 2.0, -0.0, np.nan, -np.inf, np.inf, 1e-45, -1e-45, -3.5], np.float32)


def test_relu_closed_form(port):
    out = port.relu(SPECIAL)
    # first 8 elements: SIMD max(x, 0) (NaN and -0 give +0); last 3: std::max (keeps -0)
    exp = np.array([0, 0, 0, 2, 0, 0, 0, np.inf, 1e-45, 0.0, 0.0], np.float32)
    assert np.array_equal(out.view(np.int32), exp.view(np.int32))
    tail = port.relu(np.array([1.0, 1.0, 1.0, 1.0, -0.0, np.nan], np.float32))
    assert np.signbit(tail[4]) and np.isnan(tail[5])


def test_bias_act_vs_reference(port, ref):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((2, 3, 5, 7)).astype(np.float32)
    x.ravel()[:SPECIAL.size] = SPECIAL
    x.ravel()[-SPECIAL.size:] = SPECIAL
    b = rng.standard_normal(3).astype(np.float32)
    eq = lambda a, c: np.array_equal(a.view(np.int32), c.view(np.int32))
    assert eq(port.add_bias(x, b), ref.add_bias(x, b))
    assert eq(port.relu(x), ref.relu(x))
    assert eq(port.leaky_relu(x, 0.1), ref.leaky_relu(x, 0.1))
    y = x.reshape(-1)[:209]     # count % 4 == 1: exercises the scalar tail
    assert eq(port.relu(y), ref.relu(y))
    assert eq(port.leaky_relu(y, 0.1), ref.leaky_relu(y, 0.1))


def test_fused_epilogue_is_the_operator_chain(port, ref):
    rng = np.random.default_rng(10)
    n, c, h, w, cout = 3, 8, 6, 5, 6
    x = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    wt = rng.integers(-128, 128, (cout, c, 3, 3)).astype(np.int8)
    dq = rng.uniform(1e-4, 1e-3, cout).astype(np.float32)
    bias = rng.standard_normal(cout).astype(np.float32)
    qs = np.full(n, 31.0, np.float32)
    for act in (None, "relu", "leaky_relu"):
        f32, q = port.conv2d_i8_fused(x, wt, dq, bias, act, 0.1, qs, pads=(1, 1, 1, 1))
        y = ref.conv2d_quantized(x, wt, dq, pads=(1, 1, 1, 1))
        y = ref.add_bias(y, bias)
        if act == "relu":
            y = ref.relu(y)
        if act == "leaky_relu":
            y = ref.leaky_relu(y, 0.1)
        assert np.array_equal(f32.view(np.int32), y.view(np.int32)), act
        assert np.array_equal(q, ref.quantize(y, qs)), act


def test_gemm_i8_dequant_composition(port):
    rng = np.random.default_rng(11)
    m, n, k = 5, 9, 64
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    b = rng.integers(-128, 128, (k, n)).astype(np.int8)
    dqw = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    dqa = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    out, acc = port.gemm_i8_dequant(a, b, dqw, dqa, bias, return_acc=True)
    exp_acc = a.astype(np.int64) @ b.astype(np.int64)
    assert np.array_equal(acc, exp_acc)
    exp = ((exp_acc.astype(np.float32) * dqw[None, :]) * dqa[:, None]) + bias[None, :]
    assert np.array_equal(out.view(np.int32), exp.view(np.int32))
