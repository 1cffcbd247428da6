"""GPU parity of the int8 path through the C ABI (libtsx_hip.so) against the CPU oracle.

Bar: bit-exact -- int32 accumulators, int8 (re)quantized values and the fp32 bit patterns of
the dequant + bias + activation epilogue.
"""
import numpy as np
import pytest

from _util import bits, c2_like

pytestmark = pytest.mark.gpu


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


# ---------------------------------------------------------------- quantize

@pytest.mark.parametrize("shape,ns", [((1, 11), 1), ((2, 11), 2), ((1, 3, 7, 9), 1), ((5, 3, 7, 9), 5),
                                      ((32, 77), 32), ((1, 4096), 1), ((7, 1000), 7), ((3, 64, 28, 28), 3)])
def test_quantize(tsx, port, shape, ns):
    rng = np.random.default_rng(100)
    x = (rng.standard_normal(shape) * 50).astype(np.float32)
    x.ravel()[::3] = np.round(x.ravel()[::3]) + 0.5          # exact ties
    x.ravel()[:8] = [np.inf, -np.inf, np.nan, 3e9, -3e9, 127.5, -128.5, 1e20][:min(8, x.size)]
    s = np.ones(ns, np.float32) if ns <= 2 else rng.uniform(0.25, 2, ns).astype(np.float32)
    got = tsx.quantize(_dev(x), _dev(s)).cpu().numpy()
    assert np.array_equal(got, port.quantize(x, s))


def test_quantize_known_answers(tsx):
    kat = np.array([.5, 1.5, 2.5, -.5, -1.5, 3.5, 4.5, 5.5, .5, 1.5, 2.5], np.float32)
    one = tsx.quantize(_dev(kat.reshape(1, 11)), _dev(np.ones(1, np.float32))).cpu().numpy()
    assert one.ravel().tolist() == [0, 2, 2, 0, -2, 4, 4, 6, 1, 2, 3]
    two = tsx.quantize(_dev(np.stack([kat, kat])), _dev(np.ones(2, np.float32))).cpu().numpy()
    assert two.tolist() == [[1, 2, 3, -1, -2, 4, 5, 6, 1, 2, 3]] * 2


def _tie_neighbourhood():
    """Every x.5 from -131.5 to 131.5 with the float just below and just above it, the float below 0.5 (which
    v + 0.5 would round up to 1), and values around 2^23 where a float has no fraction bits left."""
    half = np.arange(-132, 132, dtype=np.float32) + np.float32(0.5)
    vals = [half, np.nextafter(half, np.float32(np.inf)), np.nextafter(half, np.float32(-np.inf)),
            np.array([0.49999997, -0.49999997, 0.0, -0.0, 8388607.5, -8388607.5, 8388609.0, -8388609.0,
                      4194303.5, -4194303.5, 126.99999, -127.99999, 1e-30, -1e-30], np.float32)]
    return np.concatenate(vals).astype(np.float32)


@pytest.mark.parametrize("ns", [1, 2])
def test_quantize_tie_neighbourhood(tsx, port, ns):
    """Round-half-away (several scales, and the tail of the single-scale case) and round-half-even (its body) on the
    values where the two differ from each other and from truncation of v + 0.5."""
    v = _tie_neighbourhood()
    x = np.stack([np.resize(v, 811)] * ns)                   # 811 = 8 * 101 + 3: a body and a tail
    s = np.ones(ns, np.float32)
    got = tsx.quantize(_dev(x), _dev(s)).cpu().numpy()
    assert np.array_equal(got, port.quantize(x, s))
    if ns == 2:   # half away from zero, stated without the oracle: sign(v) * floor(|v| + 0.5) in exact arithmetic
        want = np.clip(np.sign(x) * np.floor(np.abs(x).astype(np.float64) + 0.5), -128, 127).astype(np.int8)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("n", [1, 2])
def test_staged_quantize_tie_neighbourhood(tsx, port, n):
    """The same values through the quantize fused into the staging kernel: a 1x1 convolution with identity weights
    and unit scales hands the quantized input back as fp32."""
    v = _tie_neighbourhood()
    c, h, w = 8, 9, 12                                          # 864 elements per image
    x = np.stack([np.resize(np.roll(v, 5 * i), c * h * w).reshape(c, h, w) for i in range(n)])
    wq = np.eye(c, dtype=np.int8).reshape(c, c, 1, 1)
    s = np.ones(n, np.float32)
    conv = tsx.Conv2dI8(_dev(wq), (0, 0, 0, 0))
    out, _, _ = conv(_dev(x), dq=_dev(np.ones(c, np.float32)), x_scales=_dev(s))
    assert np.array_equal(out.cpu().numpy(), port.quantize(x, s).astype(np.float32))


def test_quantize_unaligned_view(tsx, port):
    import torch
    rng = np.random.default_rng(101)
    x = (rng.standard_normal(1003) * 30).astype(np.float32)
    base = _dev(np.concatenate([[0.0], x]).astype(np.float32))
    view = base[1:].view(1, 1003)                          # 4-byte aligned only
    got = tsx.quantize(view, _dev(np.array([1.5], np.float32))).cpu().numpy()
    assert np.array_equal(got, port.quantize(x.reshape(1, 1003), [1.5]))


# ---------------------------------------------------------------- conv2d int8

CONV_CASES = [
    # n, c, h, w, cout, kh, kw, pads(t,b,l,r), strides, dilations
    (2, 8, 6, 6, 4, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (1, 3, 9, 7, 5, 3, 3, (0, 0, 0, 0), (2, 2), (1, 1)),
    (2, 16, 5, 5, 8, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),
    (1, 4, 8, 8, 3, 1, 1, (0, 0, 0, 0), (2, 2), (1, 1)),
    (1, 5, 10, 9, 6, 3, 2, (2, 1, 0, 1), (1, 2), (2, 1)),
    (3, 2, 7, 7, 7, 7, 7, (3, 3, 3, 3), (2, 2), (1, 1)),
    (2, 64, 14, 14, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (1, 130, 9, 9, 200, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # ragged channels / cout > one tile
    (5, 96, 7, 7, 129, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),
    (2, 256, 28, 28, 256, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),   # two images of BASELINE config 2
    (1, 16, 5, 300, 40, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # rows wider than a tile: column tiles
    (2, 16, 7, 301, 72, 3, 3, (1, 1, 1, 1), (2, 2), (1, 1)),     # ... with stride 2
    (2, 16, 9, 50, 24, 3, 3, (1, 0, 2, 1), (1, 1), (1, 1)),      # at most 32 output channels: one wavefront along cout
    (3, 70, 15, 13, 96, 3, 3, (1, 1, 1, 1), (2, 2), (1, 1)),     # stride 2, tiles straddling images
    (3, 40, 14, 14, 130, 1, 1, (0, 0, 0, 0), (2, 2), (1, 1)),    # 1x1 stride 2 (a projection shortcut)
    (2, 24, 11, 12, 33, 3, 3, (2, 2, 2, 2), (2, 1), (2, 2)),     # mixed strides with dilation
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_i8_accumulators_and_dequant(tsx, port, case):
    n, c, h, w, cout, kh, kw, pads, st, dl = case
    rng = np.random.default_rng(200)
    x = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    wt = rng.integers(-128, 128, (cout, c, kh, kw)).astype(np.int8)
    dq = rng.uniform(1e-4, 1e-2, cout).astype(np.float32)
    conv = tsx.Conv2dI8(_dev(wt), pads, st, dl)
    out, _, acc = conv(_dev(x), dq=_dev(dq), want_acc=True)
    exp, exp_acc = port.conv2d_quantized(x, wt, dq, pads, st, dl, return_acc=True)
    assert np.array_equal(acc.cpu().numpy(), exp_acc)
    assert np.array_equal(bits(out.cpu().numpy()), bits(exp))


def _random_conv_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        kh, kw = (int(v) for v in rng.choice([1, 2, 3, 5], 2))
        st = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        dl = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pads = tuple(int(rng.integers(0, k // 2 + 2)) for k in (kh, kh, kw, kw))
        n, c, cout = int(rng.integers(1, 4)), int(rng.choice([3, 16, 40, 64, 70, 130])), int(rng.choice([8, 24, 32, 33, 64, 96, 130]))
        h, w = int(rng.integers(5, 34)), int(rng.integers(5, 70))
        if h + pads[0] + pads[1] < dl[0] * (kh - 1) + 1 or w + pads[2] + pads[3] < dl[1] * (kw - 1) + 1:
            continue
        cases.append((n, c, h, w, cout, kh, kw, pads, st, dl))
    return cases


@pytest.mark.parametrize("case", _random_conv_cases(24, 419))
def test_conv2d_i8_random_geometries_with_every_output(tsx, port, case):
    """Seeded random geometries (kernel 1..5, strides, dilations, asymmetric padding, ragged channel counts, maps wider
    than a tile) through the full epilogue -- dequantize, bias, LeakyReLU, fp32 out, requantized int8 out, raw
    accumulators -- against the oracle bit for bit: the tile / window / fragment arithmetic of whichever kernel the
    planner picks."""
    n, c, h, w, cout, kh, kw, pads, st, dl = case
    rng = np.random.default_rng(hash(case) % (1 << 31))
    x = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    wt = rng.integers(-127, 128, (cout, c, kh, kw)).astype(np.int8)
    dq = rng.uniform(1e-4, 1e-3, cout).astype(np.float32)
    bias = rng.standard_normal(cout).astype(np.float32)
    qs = np.full(n, 6.0, np.float32)
    conv = tsx.Conv2dI8(_dev(wt), pads, st, dl)
    out, q, acc = conv(_dev(x), dq=_dev(dq), bias=_dev(bias), act="leaky_relu", slope=0.1, q_scales=_dev(qs), want_acc=True)
    exp, exp_q = port.conv2d_i8_fused(x, wt, dq, bias, "leaky_relu", 0.1, qs, pads, st, dl)
    assert np.array_equal(acc.cpu().numpy(), port.conv2d_quantized(x, wt, dq, pads, st, dl, return_acc=True)[1])
    assert np.array_equal(bits(out.cpu().numpy()), bits(exp))
    assert np.array_equal(q.cpu().numpy(), exp_q)
    # the same without the raw accumulators: the fragment-wise epilogue instead of the per-element one
    out2, q2, _ = conv(_dev(x), dq=_dev(dq), bias=_dev(bias), act="leaky_relu", slope=0.1, q_scales=_dev(qs))
    assert np.array_equal(bits(out2.cpu().numpy()), bits(exp)) and np.array_equal(q2.cpu().numpy(), exp_q)


def test_conv2d_i8_padding_value(tsx, port):
    rng = np.random.default_rng(201)
    x = rng.integers(-128, 128, (2, 5, 6, 7)).astype(np.int8)
    wt = rng.integers(-128, 128, (9, 5, 3, 3)).astype(np.int8)
    dq = np.ones(9, np.float32)
    conv = tsx.Conv2dI8(_dev(wt), (1, 2, 2, 1), (1, 1), (1, 1), padding_value=-3.9)
    _, _, acc = conv(_dev(x), dq=_dev(dq), want_acc=True)
    _, exp = port.conv2d_quantized(x, wt, dq, (1, 2, 2, 1), padding_value=-3.9, return_acc=True)
    assert np.array_equal(acc.cpu().numpy(), exp)


def test_conv2d_i8_extreme_operands(tsx, port):
    # -128 * -128 over K = 2304: the largest accumulator magnitude the layer can produce
    x = np.full((1, 256, 3, 3), -128, np.int8)
    wt = np.full((2, 256, 3, 3), -128, np.int8)
    wt[1] = 127
    dq = np.array([1.0, 0.5], np.float32)
    conv = tsx.Conv2dI8(_dev(wt))
    out, _, acc = conv(_dev(x), dq=_dev(dq), want_acc=True)
    exp, exp_acc = port.conv2d_quantized(x, wt, dq, return_acc=True)
    assert acc.cpu().numpy().ravel().tolist() == [128 * 128 * 2304, -128 * 127 * 2304]
    assert np.array_equal(acc.cpu().numpy(), exp_acc)
    assert np.array_equal(bits(out.cpu().numpy()), bits(exp))


@pytest.mark.parametrize("act", [None, "relu", "leaky_relu"])
@pytest.mark.parametrize("n", [1, 3])
def test_conv2d_i8_fused_epilogue(tsx, port, act, n):
    rng = np.random.default_rng(202)
    x, x_scales, wq, dq, bias = c2_like(rng, n, 24, 9, 11, 40)
    xq = port.quantize(x, x_scales)
    qs = np.full(n, 9.0, np.float32)
    bias[3] = -0.0
    conv = tsx.Conv2dI8(_dev(wq), (1, 1, 1, 1))
    out, q, _ = conv(_dev(xq), dq=_dev(dq), bias=_dev(bias), act=act, slope=0.1, q_scales=_dev(qs))
    exp, exp_q = port.conv2d_i8_fused(xq, wq, dq, bias, act, 0.1, qs, pads=(1, 1, 1, 1))
    assert np.array_equal(bits(out.cpu().numpy()), bits(exp))
    assert np.array_equal(q.cpu().numpy(), exp_q)


def test_conv2d_i8_epilogue_signed_zero_and_tail(tsx, port):
    # all-zero accumulators with a negative dequant scale give -0.0; bias -0.0 keeps it; the
    # reference's relu turns it into +0.0 in its SIMD body but not in its scalar tail.
    x = np.zeros((1, 8, 3, 3), np.int8)
    wt = np.ones((3, 8, 1, 1), np.int8)
    dq = np.array([-1.0, 1.0, -2.0], np.float32)
    bias = np.array([-0.0, -0.0, -0.0], np.float32)
    conv = tsx.Conv2dI8(_dev(wt))
    for act in ("relu", "leaky_relu"):
        out, _, _ = conv(_dev(x), dq=_dev(dq), bias=_dev(bias), act=act, slope=0.1)
        exp, _ = port.conv2d_i8_fused(x, wt, dq, bias, act, 0.1)
        assert np.array_equal(bits(out.cpu().numpy()), bits(exp)), act
    assert np.signbit(exp.ravel()[-1])        # 27 elements: the last three are the scalar tail


@pytest.mark.parametrize("case", [
    # n, cin, h, w, cout, k, pad, consumer kernel (its halo decides whether the producer's rows are flat pixel lists)
    (3, 768, 7, 9, 130, 1, 0, 3),      # 12 channel blocks -> windows of 4; consumer with halo
    (2, 384, 5, 6, 64, 1, 0, 1),       # 6 blocks -> windows of 2; 64 output channels; flat consumer
    (2, 192, 6, 5, 24, 1, 0, 3),       # 3 blocks -> single-block windows; one wavefront along cout
    (1, 40, 4, 300, 72, 3, 1, 3),      # column tiles
    (2, 24, 9, 37, 20, 3, 1, 1),       # <= 32 output channels, 3x3
])
@pytest.mark.parametrize("after", [False, True])      # residual in front of / behind the activation
def test_conv2d_i8_all_epilogue_terms_on_every_tiling(tsx, port, case, after):
    """Residual join + fp32 output + requantized staged output together, on the tilings the plan picks for
    1x1 layers (flat pixel lists, multi-block windows), few output channels and column tiles; the staged
    output is checked through a consumer convolution."""
    n, cin, h, w, cout, k, pad, ck = case
    rng = np.random.default_rng(207)
    xq = rng.integers(-128, 128, (n, cin, h, w)).astype(np.int8)
    wa = rng.integers(-127, 128, (cout, cin, k, k)).astype(np.int8)
    dqa = rng.uniform(1e-5, 3e-5, cout).astype(np.float32)
    ba = rng.standard_normal(cout).astype(np.float32)
    qs = np.full(n, 7.0, np.float32)
    A = tsx.Conv2dI8(_dev(wa), (pad,) * 4)
    plain = port.conv2d_i8_fused(xq, wa, dqa, ba, None, pads=(pad,) * 4)[0]
    res = (rng.standard_normal(plain.shape) * np.abs(plain).mean()).astype(np.float32)
    exp = port.add(port.leaky_relu(plain, 0.1), res) if after else port.leaky_relu(port.add(plain, res), 0.1)
    exp_q = port.quantize(exp, qs)
    wb = rng.integers(-127, 128, (40, cout, ck, ck)).astype(np.int8)
    dqb = rng.uniform(1e-4, 3e-4, 40).astype(np.float32)
    B = tsx.Conv2dI8(_dev(wb), (ck // 2,) * 4)
    sb = tsx.StagedInput(B, tuple(plain.shape))
    sa = tsx.StagedInput(A, tuple(xq.shape))
    A.stage(_dev(xq), sa)
    f = A.run_staged(sa, _dev(dqa), _dev(ba), "leaky_relu", 0.1, q_scales=_dev(qs), residual=_dev(res), staged_out=sb,
                     residual_after_act=after)[0]
    assert np.array_equal(bits(f.cpu().numpy()), bits(exp))
    got = B.run_staged(sb, _dev(dqb))[0].cpu().numpy()
    assert np.array_equal(bits(got), bits(port.conv2d_quantized(exp_q, wb, dqb, (ck // 2,) * 4)))


@pytest.mark.parametrize("strides", [(1, 1), (2, 2)])
def test_conv2d_i8_residual_join_in_epilogue(tsx, port, strides):
    """conv -> add_bias -> add(residual) -> relu (-> quantize) fused, against the separate operators."""
    rng = np.random.default_rng(204)
    x, _, wq, dq, bias = c2_like(rng, 3, 70, 12, 11, 37)
    xq = rng.integers(-128, 128, x.shape).astype(np.int8)
    conv = tsx.Conv2dI8(_dev(wq), (1, 1, 1, 1), strides)
    plain = port.conv2d_i8_fused(xq, wq, dq, bias, None, pads=(1, 1, 1, 1), strides=strides)[0]
    res = (rng.standard_normal(plain.shape) * np.abs(plain).mean()).astype(np.float32)
    res.ravel()[::5] = -plain.ravel()[::5]                    # exact zeros before the activation
    qs = np.full(3, 0.05, np.float32)
    for act in (None, "relu"):
        out, q, _ = conv(_dev(xq), dq=_dev(dq), bias=_dev(bias), act=act, q_scales=_dev(qs), residual=_dev(res))
        exp = port.add(plain, res)
        if act:
            exp = port.relu(exp)
        assert np.array_equal(bits(out.cpu().numpy()), bits(exp)), act
        assert np.array_equal(q.cpu().numpy(), port.quantize(exp, qs))
    with pytest.raises(tsx.TsxError):
        conv(_dev(xq), dq=_dev(dq), residual=_dev(res[:, :, :-1]))


@pytest.mark.parametrize("cmid", [64, 37])          # packed dword stores / per-element path (cout not a multiple of 32)
@pytest.mark.parametrize("a_strides", [(1, 1), (2, 2)])   # producer: window-stationary kernel / generic implicit GEMM
def test_conv2d_i8_staged_hand_over(tsx, port, cmid, a_strides):
    """Producer writes its requantized output straight into the consumers' staged input; results must equal
    the NCHW int8 hand-over (and the oracle) bit for bit.  Two consumers share one staged buffer: a 3x3 p1
    convolution and -- through its own padded buffer's interior being a superset -- a strided 1x1."""
    import torch
    rng = np.random.default_rng(205)
    n, cin, h, w = 3, 70, 13, 12
    xq = rng.integers(-128, 128, (n, cin, h, w)).astype(np.int8)
    wa = rng.integers(-127, 128, (cmid, cin, 3, 3)).astype(np.int8)
    dqa = rng.uniform(1e-4, 3e-4, cmid).astype(np.float32)
    ba = rng.standard_normal(cmid).astype(np.float32)
    qs = np.full(n, 3.0, np.float32)
    A = tsx.Conv2dI8(_dev(wa), (1, 1, 1, 1), a_strides)
    ya_f, ya_q, _ = A(_dev(xq), dq=_dev(dqa), bias=_dev(ba), act="relu", q_scales=_dev(qs))
    exp_f, exp_q = port.conv2d_i8_fused(xq, wa, dqa, ba, "relu", 0.0, qs, (1, 1, 1, 1), a_strides)
    assert np.array_equal(ya_q.cpu().numpy(), exp_q)

    wb = rng.integers(-127, 128, (48, cmid, 3, 3)).astype(np.int8)
    wc = rng.integers(-127, 128, (40, cmid, 1, 1)).astype(np.int8)
    dqb = rng.uniform(1e-4, 3e-4, 48).astype(np.float32)
    dqc = rng.uniform(1e-4, 3e-4, 40).astype(np.float32)
    B = tsx.Conv2dI8(_dev(wb), (1, 1, 1, 1))
    C1 = tsx.Conv2dI8(_dev(wc))                      # 1x1 stride 1: owns the un-padded staged buffer
    C2 = tsx.Conv2dI8(_dev(wc), strides=(2, 2))      # 1x1 stride 2 reading C1's buffer
    sb = tsx.StagedInput(B, tuple(ya_q.shape))
    sc = tsx.StagedInput(C1, tuple(ya_q.shape))
    for staged in (sb, sc):
        f, q, _ = A(_dev(xq), dq=_dev(dqa), bias=_dev(ba), act="relu", q_scales=_dev(qs), staged_out=staged)
        assert q is None and np.array_equal(bits(f.cpu().numpy()), bits(exp_f))
    got_b = B.run_staged(sb, _dev(dqb))[0].cpu().numpy()
    assert np.array_equal(bits(got_b), bits(port.conv2d_quantized(exp_q, wb, dqb, (1, 1, 1, 1))))
    got_c1 = C1.run_staged(sc, _dev(dqc))[0].cpu().numpy()
    assert np.array_equal(bits(got_c1), bits(port.conv2d_quantized(exp_q, wc, dqc)))
    sc2 = tsx.StagedInput.__new__(tsx.StagedInput)   # C2's view of C1's buffer
    sc2.__dict__.update(sc.__dict__)
    got_c2 = C2.run_staged(sc2, _dev(dqc))[0].cpu().numpy()
    assert np.array_equal(bits(got_c2), bits(port.conv2d_quantized(exp_q, wc, dqc, strides=(2, 2))))
    # a second run overwrites only the interior: the halo written once stays valid
    A(_dev((xq // 2).astype(np.int8)), dq=_dev(dqa), bias=_dev(ba), act="relu", q_scales=_dev(qs), staged_out=sb)
    exp_q2 = port.conv2d_i8_fused((xq // 2).astype(np.int8), wa, dqa, ba, "relu", 0.0, qs, (1, 1, 1, 1), a_strides)[1]
    got_b2 = B.run_staged(sb, _dev(dqb))[0].cpu().numpy()
    assert np.array_equal(bits(got_b2), bits(port.conv2d_quantized(exp_q2, wb, dqb, (1, 1, 1, 1))))
    # fresh memory with only halo and channel padding set, then the producer: the same bytes as the full fill
    for consumer, full in ((B, sb), (C1, sc)):
        part = tsx.StagedInput(consumer, tuple(ya_q.shape), halo_only=True)
        A(_dev((xq // 2).astype(np.int8)), dq=_dev(dqa), bias=_dev(ba), act="relu", q_scales=_dev(qs), staged_out=part)
        A(_dev((xq // 2).astype(np.int8)), dq=_dev(dqa), bias=_dev(ba), act="relu", q_scales=_dev(qs), staged_out=full)
        assert torch.equal(part.buf, full.buf)
    with pytest.raises(tsx.TsxError):                # a buffer too small for the producer's output
        small = tsx.StagedInput(tsx.Conv2dI8(_dev(wb)), (n, cmid, 4, 4))
        A(_dev(xq), dq=_dev(dqa), q_scales=_dev(qs), staged_out=small)


@pytest.mark.parametrize("cmid", [64, 48])                # 32-channel fragments whole / the per-element path for the last 16
@pytest.mark.parametrize("producer", ["1x1", "3x3", "3x3s2"])   # window-stationary 1x1 (flat pixel rows) / 3x3 / generic kernel
def test_conv2d_i8_staged_hand_over_upsampled_into_a_channel_slice(tsx, port, cmid, producer):
    """convolution -> nearest-neighbour resize x2 -> concatenation with a second convolution's output -> convolution,
    without an fp32 tensor in between: the first producer writes every requantized pixel to the 2 x 2 staged pixels
    it becomes (staged_upsample = 2) in its run of channels of the consumer's staged input, the second producer its own
    run; the consumer's output equals the operator chain's (oracle) bit for bit."""
    rng = np.random.default_rng(411)
    n, cin, h, w = 2, 40, 7, 5
    k, pads, strides = {"1x1": (1, (0,) * 4, (1, 1)), "3x3": (3, (1,) * 4, (1, 1)), "3x3s2": (3, (1,) * 4, (2, 2))}[producer]
    hin, win = (h * 2 - 1, w * 2 - 1) if producer == "3x3s2" else (h, w)
    xa = rng.integers(-128, 128, (n, cin, hin, win)).astype(np.int8)
    xb = rng.integers(-128, 128, (n, cin, 2 * h, 2 * w)).astype(np.int8)
    wa = rng.integers(-127, 128, (cmid, cin, k, k)).astype(np.int8)
    wb = rng.integers(-127, 128, (32, cin, 1, 1)).astype(np.int8)
    dqa = rng.uniform(1e-4, 3e-4, cmid).astype(np.float32)
    dqb = rng.uniform(1e-4, 3e-4, 32).astype(np.float32)
    ba = rng.standard_normal(cmid).astype(np.float32)
    qs = np.full(n, 2.5, np.float32)
    A = tsx.Conv2dI8(_dev(wa), pads, strides)
    B = tsx.Conv2dI8(_dev(wb))
    wc = rng.integers(-127, 128, (24, cmid + 32, 3, 3)).astype(np.int8)
    dqc = rng.uniform(1e-4, 3e-4, 24).astype(np.float32)
    C = tsx.Conv2dI8(_dev(wc), (1, 1, 1, 1))
    whole = tsx.StagedInput(C, (n, cmid + 32, 2 * h, 2 * w))
    A(_dev(xa), dq=_dev(dqa), bias=_dev(ba), act="leaky_relu", slope=0.1, q_scales=_dev(qs), want_f32=False,
      staged_out=tsx.StagedSlice(whole, 0, cmid, upsample=2))
    B(_dev(xb), dq=_dev(dqb), q_scales=_dev(qs), want_f32=False, staged_out=tsx.StagedSlice(whole, cmid, 32))
    got = C.run_staged(whole, _dev(dqc))[0].cpu().numpy()
    fa = port.leaky_relu(port.add_bias(port.conv2d_quantized(xa, wa, dqa, pads, strides), ba), 0.1)
    assert fa.shape == (n, cmid, h, w)
    cat = port.concat([port.resize_nearest(fa, 2 * h, 2 * w), port.conv2d_quantized(xb, wb, dqb)], 1)
    exp = port.conv2d_quantized(port.quantize(cat, qs), wc, dqc, (1, 1, 1, 1))
    assert np.array_equal(bits(got), bits(exp))
    # the checker's view of the slice is the producer's own map
    q = tsx.staged_interior(tsx.StagedSlice(whole, 0, cmid, upsample=2), range(n)).cpu().numpy()
    assert np.array_equal(q, port.quantize(fa, qs))
    with pytest.raises(tsx.TsxError):                # an upsampled map larger than the staged one
        A(_dev(xa), dq=_dev(dqa), q_scales=_dev(qs), want_f32=False,
          staged_out=tsx.StagedSlice(tsx.StagedInput(C, (n, cmid + 32, 2 * h - 2, 2 * w)), 0, cmid, upsample=2))


@pytest.mark.parametrize("k,stride,pad,size", [(7, 2, 3, (30, 44)), (3, 1, 1, (9, 12)), (5, 2, 2, (17, 40))])
def test_conv2d_i8_stem_as_pairs_of_output_columns(tsx, port, k, stride, pad, size):
    """A few-channel stem computed as pairs of output columns (a k x (k + stride) window at twice the column stride,
    2 x cout channels, pair_outputs_weights) writes the very bytes the plain stem writes into a pixel-major int8
    buffer: fused input quantize, bias, ReLU, requantize; values = the operator chain's (oracle)."""
    import torch
    rng = np.random.default_rng(433)
    n, (h, w) = 2, size
    x = rng.uniform(-1, 1, (n, 3, h, w)).astype(np.float32)
    wa = rng.integers(-127, 128, (64, 3, k, k)).astype(np.int8)
    sx = np.full(n, 127.0, np.float32)
    dqa = (rng.uniform(0.5, 1.5, 64) / (127.0 * 127.0 * k)).astype(np.float32)
    ba = (0.1 * rng.standard_normal(64)).astype(np.float32)
    qs = np.full(n, 40.0, np.float32)
    ho, wo = (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
    assert wo % 2 == 0
    plain, paired = tsx.StagedPlain((n, 64, ho, wo), "cuda:0"), tsx.StagedPlain((n, 64, ho, wo), "cuda:0")
    A = tsx.Conv2dI8(_dev(wa), (pad,) * 4, (stride, stride))
    A(_dev(x), dq=_dev(dqa), bias=_dev(ba), act="relu", x_scales=_dev(sx), q_scales=_dev(qs), want_f32=False, staged_out=plain)
    A2 = tsx.Conv2dI8(tsx.pair_outputs_weights(_dev(wa), stride), (pad,) * 4, (stride, 2 * stride))
    A2(_dev(x), dq=_dev(np.tile(dqa, 2)), bias=_dev(np.tile(ba, 2)), act="relu", x_scales=_dev(sx), q_scales=_dev(qs),
       want_f32=False, staged_out=paired.column_pairs())
    assert torch.equal(plain.buf, paired.buf)
    f = port.relu(port.add_bias(port.conv2d_quantized(port.quantize(x, sx), wa, dqa, (pad,) * 4, (stride, stride)), ba))
    q = port.quantize(f, qs)
    assert len(np.unique(q)) > 20
    assert np.array_equal(tsx.staged_interior(paired, range(n)).cpu().numpy(), q)


# im2col-staged stem / the same computed as pairs of output columns / window-stationary 1x1 / 3x3
@pytest.mark.parametrize("producer", ["stem", "stem-pairs", "1x1", "3x3"])
@pytest.mark.parametrize("size", [(9, 12), (32, 70)])
def test_conv2d_i8_staged_hand_over_in_column_pairs(tsx, port, producer, size):
    """A 32-channel producer followed by a 3x3 convolution of stride 2: the producer writes pairs of columns as one
    64-channel pixel (no channel padding in the staged buffer) and the consumer runs as a 3x2 convolution of stride
    (2, 1) over the pairs with rearranged weights.  Output = the operator chain's (oracle, original weights and
    geometry) bit for bit."""
    rng = np.random.default_rng(431)
    n, (h, w) = 2, size
    cin, k, pads = {"stem": (3, 3, (1,) * 4), "stem-pairs": (3, 3, (1,) * 4), "1x1": (48, 1, (0,) * 4), "3x3": (64, 3, (1,) * 4)}[producer]
    xa = rng.integers(-128, 128, (n, cin, h, w)).astype(np.int8)
    wa = rng.integers(-127, 128, (32, cin, k, k)).astype(np.int8)
    dqa = rng.uniform(1e-4, 3e-4, 32).astype(np.float32) * (20 if cin == 3 else 1)
    ba = rng.standard_normal(32).astype(np.float32)
    qs = np.full(n, 3.0, np.float32)
    wb = rng.integers(-127, 128, (40, 32, 3, 3)).astype(np.int8)
    dqb = rng.uniform(1e-4, 3e-4, 40).astype(np.float32)
    A = tsx.Conv2dI8(_dev(wa), pads)
    B = tsx.Conv2dI8(tsx.pair_columns_weights(_dev(wb)), (1, 1, 1, 0), (2, 1))
    st = tsx.StagedPairs(tsx.StagedInput(B, (n, 64, h, w // 2)))
    if producer == "stem-pairs":
        # 2 x 32 output channels per pair of columns from a 3x4 window at column stride 2: the same bytes
        A2 = tsx.Conv2dI8(tsx.pair_outputs_weights(_dev(wa)), pads, (1, 2))
        A2(_dev(xa), dq=_dev(np.tile(dqa, 2)), bias=_dev(np.tile(ba, 2)), act="leaky_relu", slope=0.1, q_scales=_dev(qs),
           want_f32=False, staged_out=st.pairs)
    else:
        A(_dev(xa), dq=_dev(dqa), bias=_dev(ba), act="leaky_relu", slope=0.1, q_scales=_dev(qs), want_f32=False, staged_out=st)
    got = B.run_staged(st.pairs, _dev(dqb))[0].cpu().numpy()
    fa = port.leaky_relu(port.add_bias(port.conv2d_quantized(xa, wa, dqa, pads), ba), 0.1)
    qa = port.quantize(fa, qs)
    assert np.array_equal(tsx.staged_interior(st, range(n)).cpu().numpy(), qa)       # the checker sees the 32-channel map
    assert len(np.unique(qa)) > 20
    exp = port.conv2d_quantized(qa, wb, dqb, (1, 1, 1, 1), (2, 2))
    assert got.shape == exp.shape and np.array_equal(bits(got), bits(exp))
    with pytest.raises(tsx.TsxError):                # pairs need whole 64-channel blocks
        tsx.StagedPairs(tsx.StagedInput(tsx.Conv2dI8(_dev(wb)), (n, 32, h, w)))


@pytest.mark.parametrize("geom", [((3, 3), (2, 2), (0, 1, 0, 1)), ((2, 2), (2, 2), (0, 0, 0, 0)), ((3, 3), (1, 1), (1, 1, 1, 1)),
                                  ((5, 5), (1, 1), (2, 2, 2, 2))])
@pytest.mark.parametrize("few_channels", [False, True])   # producer = window-stationary kernel / im2col-staged stem
def test_max_pooling_on_staged_int8(tsx, port, geom, few_channels):
    """producer (requantized, pixel-major int8) -> max pooling on int8 -> consumer convolution must equal the
    operator chain conv -> bias -> relu -> pooling2d(fp32) -> quantize -> conv2d_quantized bit for bit."""
    ksize, strides, pads = geom
    rng = np.random.default_rng(206)
    n, cin, h, w, cmid = (2, 3, 23, 21, 64) if few_channels else (2, 40, 13, 15, 70)
    k = 7 if few_channels else 3
    x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
    x_scales = np.full(n, 40.0, np.float32)
    wa = rng.integers(-127, 128, (cmid, cin, k, k)).astype(np.int8)
    dqa = rng.uniform(1e-4, 3e-4, cmid).astype(np.float32)
    ba = rng.standard_normal(cmid).astype(np.float32)
    qs = np.full(n, 5.0, np.float32)
    a_strides = (2, 2) if few_channels else (1, 1)
    A = tsx.Conv2dI8(_dev(wa), (k // 2,) * 4, a_strides)
    xq = port.quantize(x, x_scales)
    exp_f = port.conv2d_i8_fused(xq, wa, dqa, ba, "relu", 0.0, None, (k // 2,) * 4, a_strides)[0]
    pooled = port.pooling2d(exp_f, "max", ksize, strides, pads)
    pooled_q = port.quantize(pooled, qs)
    wb = rng.integers(-127, 128, (48, cmid, 3, 3)).astype(np.int8)
    dqb = rng.uniform(1e-4, 3e-4, 48).astype(np.float32)
    B = tsx.Conv2dI8(_dev(wb), (1, 1, 1, 1))
    s_mid = tsx.StagedPlain(tuple(exp_f.shape), "cuda")
    f, q, _ = A(_dev(x), dq=_dev(dqa), bias=_dev(ba), act="relu", x_scales=_dev(x_scales), q_scales=_dev(qs), want_f32=False,
                staged_out=s_mid)
    assert f is None and q is None
    s_b = tsx.StagedInput(B, tuple(pooled.shape))
    tsx.max_pooling2d_staged(s_mid, s_b, ksize, strides, pads)
    got = B.run_staged(s_b, _dev(dqb))[0].cpu().numpy()
    assert np.array_equal(bits(got), bits(port.conv2d_quantized(pooled_q, wb, dqb, (1, 1, 1, 1))))
    with pytest.raises(tsx.TsxError):                # windows that start outside the map
        bad = tsx.StagedInput(B, (n, cmid, pooled.shape[2] + 3, pooled.shape[3]))
        a, b = tsx._staged_map(s_mid), tsx._staged_map(bad)
        import ctypes
        tsx.check(tsx.lib().tsx_max_pooling2d_i8_staged(ctypes.byref(a), ctypes.byref(b), ksize[0], ksize[1], pads[0], pads[2],
                                                        strides[0], strides[1], None))


def test_max_pooling_on_a_channel_slice_of_staged_int8(tsx, port):
    """An SPP block on int8: a convolution writes its requantized output into the last 64 channels of the consumer's
    staged input, stride-1 max poolings go from one run of 64 channels into the next (5x5 of the convolution's run, then
    5x5 of that = 9x9), and the consumer's output equals the operator chain conv -> pooling2d(fp32) x2 -> concat ->
    quantize -> conv2d_quantized bit for bit."""
    rng = np.random.default_rng(412)
    n, cin, h, w, f = 2, 40, 11, 9, 64
    xq = rng.integers(-128, 128, (n, cin, h, w)).astype(np.int8)
    wa = rng.integers(-127, 128, (f, cin, 1, 1)).astype(np.int8)
    dqa = rng.uniform(1e-3, 3e-3, f).astype(np.float32)
    ba = rng.standard_normal(f).astype(np.float32)
    qs = np.full(n, 4.0, np.float32)
    A = tsx.Conv2dI8(_dev(wa))
    wc = rng.integers(-127, 128, (24, 3 * f, 1, 1)).astype(np.int8)
    dqc = rng.uniform(1e-4, 3e-4, 24).astype(np.float32)
    C = tsx.Conv2dI8(_dev(wc))
    whole = tsx.StagedInput(C, (n, 3 * f, h, w))
    A(_dev(xq), dq=_dev(dqa), bias=_dev(ba), act="leaky_relu", slope=0.1, q_scales=_dev(qs), want_f32=False,
      staged_out=tsx.StagedSlice(whole, 2 * f, f))
    tsx.max_pooling2d_staged(tsx.StagedSlice(whole, 2 * f, f), tsx.StagedSlice(whole, f, f), (5, 5), (1, 1), (2, 2, 2, 2))
    tsx.max_pooling2d_staged(tsx.StagedSlice(whole, f, f), tsx.StagedSlice(whole, 0, f), (5, 5), (1, 1), (2, 2, 2, 2))
    got = C.run_staged(whole, _dev(dqc))[0].cpu().numpy()
    fa = port.leaky_relu(port.add_bias(port.conv2d_quantized(xq, wa, dqa), ba), 0.1)
    cat = port.concat([port.pooling2d(fa, "max", (9, 9), (1, 1), (4, 4, 4, 4)), port.pooling2d(fa, "max", (5, 5), (1, 1), (2, 2, 2, 2)), fa], 1)
    assert np.array_equal(bits(got), bits(port.conv2d_quantized(port.quantize(cat, qs), wc, dqc)))
    # a run that is no whole number of 64-channel blocks would pool into its neighbour's channels: refused
    with pytest.raises(tsx.TsxError, match="whole 64-channel blocks"):
        tsx.max_pooling2d_staged(tsx.StagedSlice(whole, 2 * f, 48), tsx.StagedSlice(whole, f, 48), (5, 5), (1, 1), (2, 2, 2, 2))


def test_quantize_conv2d_fused_input(tsx, port):
    rng = np.random.default_rng(203)
    for n in (1, 4):
        x, x_scales, wq, dq, bias = c2_like(rng, n, 70, 10, 9, 33)
        x.ravel()[::5] = (np.round(x.ravel()[::5] * x_scales[0]) + 0.5) / x_scales[0]   # near-ties
        conv = tsx.Conv2dI8(_dev(wq), (1, 1, 1, 1))
        out, _, acc = conv(_dev(x), dq=_dev(dq), bias=_dev(bias), act="relu", x_scales=_dev(x_scales), want_acc=True)
        xq = port.quantize(x, x_scales)
        exp, _ = port.conv2d_i8_fused(xq, wq, dq, bias, "relu", pads=(1, 1, 1, 1))
        assert np.array_equal(bits(out.cpu().numpy()), bits(exp))


def test_conv2d_i8_baseline_config2_full(tsx, port):
    """BASELINE config 2 at full size: 32x256x28x28, 256x256x3x3, s1 p1, dequant + bias + ReLU."""
    rng = np.random.default_rng(1234)
    x, x_scales, wq, dq, bias = c2_like(rng, 32, 256, 28, 28, 256)
    conv = tsx.Conv2dI8(_dev(wq), (1, 1, 1, 1))
    xq_dev = tsx.quantize(_dev(x), _dev(x_scales))
    xq = port.quantize(x, x_scales)
    assert np.array_equal(xq_dev.cpu().numpy(), xq)
    out, _, acc = conv(xq_dev, dq=_dev(dq), bias=_dev(bias), act="relu", want_acc=True)
    exp_acc = port.conv2d_quantized(xq, wq, dq, (1, 1, 1, 1), return_acc=True)[1]
    assert np.array_equal(acc.cpu().numpy(), exp_acc)
    exp, _ = port.epilogue(exp_acc, dq, bias, "relu")
    assert np.array_equal(bits(out.cpu().numpy()), bits(exp))
    # size-independent property: the convolution is linear in x, exactly, in integers
    _, _, acc2 = conv(_dev((xq // 2).astype(np.int8)), want_acc=True)
    _, _, acc3 = conv(_dev((xq - xq // 2).astype(np.int8)), want_acc=True)
    assert np.array_equal((acc2 + acc3).cpu().numpy(), exp_acc)
    # ... and a zero input leaves exactly the activation of the bias in every position of a channel
    out0, _, _ = conv(_dev(np.zeros_like(xq)), dq=_dev(dq), bias=_dev(bias), act="relu")
    exp0 = np.broadcast_to(np.maximum(bias, 0)[None, :, None, None], exp.shape)
    assert np.array_equal(out0.cpu().numpy(), exp0)


def test_conv2d_i8_rejects_bad_arguments(tsx):
    import torch
    wt = torch.zeros((4, 8, 3, 3), dtype=torch.int8, device="cuda")
    conv = tsx.Conv2dI8(wt)
    with pytest.raises(tsx.TsxError):
        conv(torch.zeros((1, 8, 2, 2), dtype=torch.int8, device="cuda"), want_acc=True)   # empty output
    with pytest.raises(tsx.TsxError):
        conv(torch.zeros((1, 7, 5, 5), dtype=torch.int8, device="cuda"), want_acc=True)   # channel mismatch
    with pytest.raises(tsx.TsxError):   # consumer scales must match the batch (base_quantize.cpp:26)
        conv(torch.zeros((2, 8, 5, 5), dtype=torch.int8, device="cuda"), dq=torch.ones(4, device="cuda"),
             q_scales=torch.ones(3, device="cuda"))


# ---------------------------------------------------------------- int8 GEMM

@pytest.mark.parametrize("m,k,n", [(1, 64, 32), (3, 70, 33), (32, 1024, 1024), (256, 1024, 1024), (130, 200, 260),
                                   (1, 2048, 2048)])
@pytest.mark.parametrize("transpose", [False, True])
def test_gemm_i8(tsx, port, m, k, n, transpose):
    rng = np.random.default_rng(300)
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    b = rng.integers(-128, 128, (k, n)).astype(np.int8)
    dqw = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    dqa = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    g = tsx.GemmI8(_dev(b.T.copy() if transpose else b), transpose=transpose)
    out, _, acc = g(_dev(a), dq=_dev(dqw), row_scale=_dev(dqa), bias=_dev(bias), want_acc=True)
    exp, exp_acc = port.gemm_i8_dequant(a, b, dqw, dqa, bias, return_acc=True)
    assert np.array_equal(acc.cpu().numpy(), exp_acc)
    assert np.array_equal(bits(out.cpu().numpy()), bits(exp))


@pytest.mark.parametrize("m,k,n", [(33, 64, 128), (256, 1024, 1024), (130, 200, 260), (257, 320, 96), (100, 512, 30),
                                   (64, 128, 64), (500, 192, 1000)])
@pytest.mark.parametrize("act", [None, "relu"])
def test_gemm_i8_f32_output_only(tsx, port, m, k, n, act):
    """More than 32 rows and only the fp32 output wanted: the window-stationary kernel's row-major epilogue
    (16-byte stores; scalar stores when n is not a multiple of 4), with and without the per-row scale."""
    rng = np.random.default_rng(310 + m)
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    b = rng.integers(-128, 128, (k, n)).astype(np.int8)
    dqw = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    dqa = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    g = tsx.GemmI8(_dev(b))
    for row_scale in (dqa, None):
        out, _, _ = g(_dev(a), dq=_dev(dqw), row_scale=None if row_scale is None else _dev(row_scale), bias=_dev(bias), act=act)
        exp = port.gemm_i8_dequant(a, b, dqw, np.ones(m, np.float32) if row_scale is None else row_scale, bias)
        if act == "relu":
            exp = port.relu(exp)
        assert np.array_equal(bits(out.cpu().numpy()), bits(exp)), (m, k, n, act, row_scale is None)


@pytest.mark.parametrize("m,k,n", [(33, 64, 128), (256, 1024, 1024), (130, 200, 260), (257, 320, 96), (100, 512, 30),
                                   (64, 4096, 192), (500, 192, 1000), (65, 2048, 66), (100, 2500, 72)])
@pytest.mark.parametrize("mode", ["force", "forcereg"])
def test_gemm_i8_k_split_kernel(tsx, port, monkeypatch, m, k, n, mode):
    """The K-split kernels by themselves (TSX_GEMM_I8_KSPLIT=force gives them every GEMM of more than 32 rows; by
    itself the planner takes them for up to 512 rows against 8 MiB of weights): activations through LDS for K of
    2048 and more, straight into registers below (and everywhere with "forcereg").  The 16-byte fp32 epilogue with
    and without row scale, bias and ReLU, and the per-element epilogue with the raw accumulators, requantized rows
    and LeakyReLU; rows and columns that end inside a 64 x 64 tile, K-steps that do not divide by the 8 wavefronts
    or fill the last chunk of 16."""
    if mode == "forcereg" and k < 2048:
        pytest.skip("below K = 2048 both modes run the same kernel")
    monkeypatch.setenv("TSX_GEMM_I8_KSPLIT", mode)
    rng = np.random.default_rng(330 + m + n)
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    b = rng.integers(-128, 128, (k, n)).astype(np.int8)
    dqw = rng.uniform(1e-4, 1e-3, n).astype(np.float32)
    dqa = rng.uniform(0.5, 2.0, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    qs = rng.uniform(5, 20, m).astype(np.float32)
    g = tsx.GemmI8(_dev(b))
    for row_scale, with_bias, act in ((dqa, True, "relu"), (None, True, None), (dqa, False, None)):
        out, _, _ = g(_dev(a), dq=_dev(dqw), row_scale=None if row_scale is None else _dev(row_scale),
                      bias=_dev(bias) if with_bias else None, act=act)
        exp = port.gemm_i8_dequant(a, b, dqw, row_scale, bias if with_bias else None)
        if act == "relu":
            exp = port.relu(exp)
        assert np.array_equal(bits(out.cpu().numpy()), bits(exp)), (m, k, n, act, row_scale is None, with_bias)
    out, q, acc = g(_dev(a), dq=_dev(dqw), row_scale=_dev(dqa), bias=_dev(bias), act="leaky_relu", slope=0.1, q_scales=_dev(qs),
                    want_acc=True)
    exp, exp_acc = port.gemm_i8_dequant(a, b, dqw, dqa, bias, return_acc=True)
    exp = port.leaky_relu(exp, 0.1)
    assert np.array_equal(acc.cpu().numpy(), exp_acc)
    assert np.array_equal(bits(out.cpu().numpy()), bits(exp))
    assert np.array_equal(q.cpu().numpy(), port.quantize(exp, qs))


def test_gemm_i8_requantized_rows(tsx, port):
    """int8 output with one consumer scale per row (base_quantize.cpp:26 groups by the first extent)."""
    rng = np.random.default_rng(320)
    m, k, n = 70, 256, 136
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    b = rng.integers(-128, 128, (k, n)).astype(np.int8)
    dqw = rng.uniform(1e-4, 1e-3, n).astype(np.float32)
    qs = rng.uniform(5, 20, m).astype(np.float32)
    g = tsx.GemmI8(_dev(b))
    out, q, _ = g(_dev(a), dq=_dev(dqw), q_scales=_dev(qs))
    exp = port.gemm_i8_dequant(a, b, dqw, np.ones(m, np.float32), np.zeros(n, np.float32))
    assert np.array_equal(bits(out.cpu().numpy()), bits(exp))
    assert np.array_equal(q.cpu().numpy(), port.quantize(exp, qs))


def test_gemm_i8_largest_sweep_shape_by_rows(tsx, port):
    """M=4096, K=N=4096 (largest shape of the GEMM sweep): rows are independent, so a random
    subset of rows is checked against the oracle, all columns."""
    rng = np.random.default_rng(301)
    m = k = n = 4096
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    b = rng.integers(-128, 128, (k, n)).astype(np.int8)
    dqw = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    dqa = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    g = tsx.GemmI8(_dev(b))
    out, _, acc = g(_dev(a), dq=_dev(dqw), row_scale=_dev(dqa), bias=_dev(bias), want_acc=True)
    rows = np.sort(rng.choice(m, 48, replace=False))
    exp, exp_acc = port.gemm_i8_dequant(a[rows], b, dqw, dqa[rows], bias, return_acc=True)
    assert np.array_equal(acc.cpu().numpy()[rows], exp_acc)
    assert np.array_equal(bits(out.cpu().numpy()[rows]), bits(exp))
    # checksum of checksums over the whole product: column sums of acc = (sum of rows of a) . b
    colsum = acc.cpu().numpy().astype(np.int64).sum(axis=0)
    assert np.array_equal(colsum, a.astype(np.int64).sum(axis=0) @ b.astype(np.int64))


@pytest.mark.parametrize("k", [1024, 2048, 4096])
@pytest.mark.parametrize("m", [1, 32, 256, 4096])
def test_gemm_i8_whole_sweep(tsx, port, m, k):
    """Every shape of the GEMM sweep (M in {1, 32, 256, 4096}, K = N in {1024, 2048, 4096}) as the bench calls
    it: per-row and per-channel dequantize scales, bias, fp32 output only (the kernel each shape takes is the
    one it takes there).  All rows up to 256; above, 64 random rows against the oracle plus a checksum of the
    whole output against the rows' sum in float64 (rows are independent)."""
    n = k
    rng = np.random.default_rng(400 + m + k)
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    b = rng.integers(-128, 128, (k, n)).astype(np.int8)
    dqw = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
    dqa = rng.uniform(1e-3, 1e-2, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    g = tsx.GemmI8(_dev(b))
    out, _, _ = g(_dev(a), dq=_dev(dqw), row_scale=_dev(dqa), bias=_dev(bias))
    got = out.cpu().numpy()
    rows = np.arange(m) if m <= 256 else np.sort(rng.choice(m, 64, replace=False))
    exp = port.gemm_i8_dequant(a[rows], b, dqw, dqa[rows], bias)
    assert np.array_equal(bits(got[rows]), bits(exp))
    if m > 256:
        # every row: the exact integer products through numpy, then the same three roundings
        acc = a.astype(np.float64) @ b.astype(np.float64)          # exact: |acc| < 2^53
        ref = ((acc.astype(np.float32) * dqw[None, :]) * dqa[:, None] + bias[None, :]).astype(np.float32)
        assert np.array_equal(bits(got), bits(ref))
