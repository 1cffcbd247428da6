"""GPU parity of the fp32 path (im2col-GEMM conv2d, inner_prod, Winograd F(6,3)) through the C ABI.

Tolerance of the floating-point paths, from the path's contract: |gpu - ref| <= 1e-5 + 1e-4*|ref|
(1e-4 relative / 1e-5 absolute).  Winograd additionally restates the reference's arithmetic
operation for operation and is held to bit-exactness against the oracle."""
import numpy as np
import pytest

from _util import bits

pytestmark = pytest.mark.gpu

REL, ABS = 1e-4, 1e-5


def _close(a, b):
    return np.all(np.abs(a.astype(np.float64) - b) <= ABS + REL * np.abs(b))


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


CONV_CASES = [
    # n, c, h, w, cout, kh, kw, pads(t,b,l,r), strides, dilations
    (1, 8, 12, 12, 8, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (2, 5, 9, 7, 6, 3, 3, (0, 0, 0, 0), (2, 2), (1, 1)),
    (2, 16, 8, 8, 8, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1)),
    (1, 3, 10, 11, 4, 3, 2, (2, 1, 0, 1), (1, 2), (2, 1)),
    (3, 2, 7, 7, 7, 7, 7, (3, 3, 3, 3), (2, 2), (1, 1)),
    (2, 70, 13, 9, 90, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),       # ragged in every GEMM dimension
    (4, 128, 28, 28, 128, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),    # large enough for the 64x64 tiles
    (1, 64, 56, 56, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # BASELINE config 1
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_f32(tsx, port, case):
    n, c, h, w, cout, kh, kw, pads, st, dl = case
    rng = np.random.default_rng(400)
    x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, c, kh, kw)) * np.sqrt(2.0 / (c * kh * kw))).astype(np.float32)
    got = tsx.conv2d_f32(_dev(x), _dev(wt), pads, st, dl).cpu().numpy()
    exp = port.conv2d_f32(x, wt, pads, st, dl)
    assert got.shape == exp.shape
    assert _close(got, exp), np.abs(got - exp).max()


def test_conv2d_f32_config1_bias_relu(tsx, port):
    """BASELINE config 1: 1x64x56x56, 64x64x3x3 Kaiming-normal, bias N(0,0.01), s1 p1, then ReLU."""
    rng = np.random.default_rng(1234)
    x = rng.uniform(-1, 1, (1, 64, 56, 56)).astype(np.float32)
    wt = (rng.standard_normal((64, 64, 3, 3)) * np.sqrt(2.0 / 576)).astype(np.float32)
    bias = (rng.standard_normal(64) * 0.01).astype(np.float32)
    got = tsx.conv2d_f32(_dev(x), _dev(wt), (1, 1, 1, 1), bias=_dev(bias), act="relu").cpu().numpy()
    exp = port.relu(port.add_bias(port.conv2d_f32(x, wt, (1, 1, 1, 1)), bias))
    assert _close(got, exp), np.abs(got - exp).max()
    assert (got >= 0).all()


def small_layer_cases(count, seed):
    """Seeded 3x3 layers of the kind the small-layer kernel admits (a multiple of 4 channels, up to 64): strides,
    dilations, asymmetric padding, output channels and positions that end inside a 32 x 32 tile, several images."""
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        c = int(rng.choice([4, 8, 16, 28, 32, 36, 48, 60, 64]))
        cout = int(rng.choice([1, 7, 32, 33, 64, 70, 100]))
        n, h, w = int(rng.integers(1, 4)), int(rng.integers(3, 24)), int(rng.integers(3, 30))
        st = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        dl = (int(rng.choice([1, 1, 2, 3])), int(rng.choice([1, 1, 2])))
        pads = tuple(int(rng.integers(0, 4)) for _ in range(4))
        if h + pads[0] + pads[1] < 2 * dl[0] + 1 or w + pads[2] + pads[3] < 2 * dl[1] + 1:
            continue
        cases.append((n, c, h, w, cout, 3, 3, pads, st, dl))
    return cases


SMALL_FIXED = [
    (1, 64, 56, 56, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # BASELINE config 1
    (2, 64, 28, 28, 128, 3, 3, (1, 0, 2, 1), (2, 1), (1, 1)),
    (1, 60, 30, 30, 70, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),
    (3, 32, 5, 5, 48, 3, 3, (3, 3, 3, 3), (1, 1), (2, 2)),        # more padding than map
    (1, 4, 3, 3, 1, 3, 3, (0, 0, 0, 0), (1, 1), (1, 1)),          # one output value
]


@pytest.mark.parametrize("case", small_layer_cases(16, 411) + SMALL_FIXED)
def test_conv2d_f32_small_layer_kernel(tsx, port, monkeypatch, case):
    """The small-layer 3x3 kernel by itself (TSX_CONV_F32_SMALL=force puts layers of any size on it, and
    tsx_conv2d_f32_plan_info confirms it), with a padding value, bias and LeakyReLU, and without any of them."""
    n, c, h, w, cout, kh, kw, pads, st, dl = case
    monkeypatch.setenv("TSX_CONV_F32_SMALL", "force")
    rng = np.random.default_rng(hash(case) % (1 << 31))
    x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, c, kh, kw)) * np.sqrt(2.0 / (c * kh * kw))).astype(np.float32)
    bias = (rng.standard_normal(cout) * 0.1).astype(np.float32)
    wd = _dev(wt)
    assert tsx.conv2d_f32_plan_info(x.shape, wd, pads, st, dl)["kernel"] == "small_3x3"
    got = tsx.conv2d_f32(_dev(x), wd, pads, st, dl, padding_value=0.75, bias=_dev(bias), act="leaky_relu", slope=0.1).cpu().numpy()
    exp = port.add_bias(port.conv2d_f32(x, wt, pads, st, dl, padding_value=0.75), bias)
    exp = np.where(exp > 0, exp, np.float32(0.1) * exp)
    assert got.shape == exp.shape
    assert _close(got, exp), np.abs(got - exp).max()
    got = tsx.conv2d_f32(_dev(x), wd, pads, st, dl).cpu().numpy()
    assert _close(got, port.conv2d_f32(x, wt, pads, st, dl)), case


def test_conv2d_f32_small_layer_kernel_exact_integers(tsx, port, monkeypatch):
    """Small-integer data (every product and partial sum exact in fp32): equal bits whatever the summation order,
    so a wrong tap, channel or padding element cannot hide inside the tolerance."""
    monkeypatch.setenv("TSX_CONV_F32_SMALL", "force")
    rng = np.random.default_rng(412)
    for (n, c, h, w, cout, pads, st, dl) in ((2, 8, 9, 10, 5, (1, 2, 2, 1), (1, 1), (1, 1)), (1, 64, 20, 33, 40, (1, 1, 1, 1), (1, 1), (1, 1)),
                                             (3, 36, 11, 7, 66, (2, 0, 1, 3), (2, 1), (1, 2))):
        x = rng.integers(-8, 9, (n, c, h, w)).astype(np.float32)
        wt = rng.integers(-4, 5, (cout, c, 3, 3)).astype(np.float32)
        wd = _dev(wt)
        assert tsx.conv2d_f32_plan_info(x.shape, wd, pads, st, dl)["kernel"] == "small_3x3"
        got = tsx.conv2d_f32(_dev(x), wd, pads, st, dl, padding_value=3.0).cpu().numpy()
        assert np.array_equal(bits(got), bits(port.conv2d_f32(x, wt, pads, st, dl, padding_value=3.0)))


def test_conv2d_f32_kernel_choice(tsx, monkeypatch):
    """What the planner picks by itself: the small-layer kernel for config 1, the register-fed kernel for a small
    layer it does not admit (128 channels), staged tiles for large layers; "0" switches either off."""
    import torch
    w64 = torch.zeros((64, 64, 3, 3), device="cuda")
    assert tsx.conv2d_f32_plan_info((1, 64, 56, 56), w64, (1, 1, 1, 1))["kernel"] == "small_3x3"
    assert tsx.conv2d_f32_plan_info((32, 64, 56, 56), w64, (1, 1, 1, 1))["kernel"] == "staged_64x64"
    assert tsx.conv2d_f32_plan_info((1, 128, 28, 28), torch.zeros((128, 128, 3, 3), device="cuda"), (1, 1, 1, 1))["kernel"] == "register_fed"
    monkeypatch.setenv("TSX_CONV_F32_SMALL", "0")
    assert tsx.conv2d_f32_plan_info((1, 64, 56, 56), w64, (1, 1, 1, 1))["kernel"] == "register_fed"
    monkeypatch.setenv("TSX_GEMM_F32_REGFED", "0")
    assert tsx.conv2d_f32_plan_info((1, 64, 56, 56), w64, (1, 1, 1, 1))["kernel"] == "staged_32x32_ksplit"


@pytest.mark.parametrize("case", CONV_CASES + small_layer_cases(6, 413))
def test_conv2d_f32_register_fed_kernel(tsx, port, monkeypatch, case):
    """The register-fed kernel by itself (TSX_GEMM_F32_REGFED=force; it needs K a multiple of 4 and at least one
    32-deep chunk, other cases are skipped), bias + ReLU and a padding value."""
    n, c, h, w, cout, kh, kw, pads, st, dl = case
    monkeypatch.setenv("TSX_CONV_F32_SMALL", "0")
    monkeypatch.setenv("TSX_GEMM_F32_REGFED", "force")
    rng = np.random.default_rng(hash(case) % (1 << 31))
    x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, c, kh, kw)) * np.sqrt(2.0 / (c * kh * kw))).astype(np.float32)
    bias = (rng.standard_normal(cout) * 0.1).astype(np.float32)
    wd = _dev(wt)
    if tsx.conv2d_f32_plan_info(x.shape, wd, pads, st, dl)["kernel"] != "register_fed":
        assert (c * kh * kw) % 4 != 0 or c * kh * kw < 32, case
        pytest.skip("K = %d: the register-fed kernel takes multiples of 4 from 32 up" % (c * kh * kw))
    got = tsx.conv2d_f32(_dev(x), wd, pads, st, dl, padding_value=-0.5, bias=_dev(bias), act="relu").cpu().numpy()
    exp = port.relu(port.add_bias(port.conv2d_f32(x, wt, pads, st, dl, padding_value=-0.5), bias))
    assert _close(got, exp), np.abs(got - exp).max()


@pytest.mark.parametrize("transpose", [False, True])
def test_inner_prod_f32_register_fed_kernel(tsx, port, monkeypatch, transpose):
    monkeypatch.setenv("TSX_GEMM_F32_REGFED", "force")
    rng = np.random.default_rng(414)
    for m, k, n in ((130, 200, 260), (65, 64, 33), (200, 1024, 96)):
        lhs = rng.standard_normal((m, k)).astype(np.float32)
        rhs = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
        arg = np.ascontiguousarray(rhs.T) if transpose else rhs
        got = tsx.inner_prod_f32(_dev(lhs), _dev(arg), transpose).cpu().numpy()
        assert _close(got, port.inner_prod_f32(lhs, arg, transpose)), (m, k, n)


def test_conv2d_f32_padding_value_and_exact_integers(tsx, port):
    # small-integer data: every product and partial sum is exact in fp32, so any order gives equal bits
    rng = np.random.default_rng(401)
    x = rng.integers(-8, 9, (2, 6, 9, 10)).astype(np.float32)
    wt = rng.integers(-4, 5, (5, 6, 3, 3)).astype(np.float32)
    got = tsx.conv2d_f32(_dev(x), _dev(wt), (1, 2, 2, 1), (1, 1), (1, 1), padding_value=3.0).cpu().numpy()
    exp = port.conv2d_f32(x, wt, (1, 2, 2, 1), padding_value=3.0)
    assert np.array_equal(bits(got), bits(exp))


@pytest.mark.parametrize("m,k,n", [(1, 64, 32), (3, 70, 33), (32, 1024, 1000), (130, 200, 260), (12, 2048, 1000),
                                   (17, 301, 45), (64, 259, 16), (5, 1000, 7), (33, 4096, 130)])   # the few-rows kernel's edges
@pytest.mark.parametrize("transpose", [False, True])
def test_inner_prod_f32(tsx, port, m, k, n, transpose):
    rng = np.random.default_rng(402)
    lhs = rng.standard_normal((m, k)).astype(np.float32)
    rhs = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    arg = np.ascontiguousarray(rhs.T) if transpose else rhs
    got = tsx.inner_prod_f32(_dev(lhs), _dev(arg), transpose).cpu().numpy()
    exp = port.inner_prod_f32(lhs, arg, transpose)
    assert _close(got, exp), np.abs(got - exp).max()


WINO_CASES = [
    (1, 8, 12, 12, 8, (1, 1, 1, 1)),
    (2, 16, 9, 11, 8, (1, 1, 1, 1)),
    (1, 8, 10, 10, 16, (0, 0, 0, 0)),
    (1, 5, 7, 7, 3, (2, 1, 1, 2)),
    (2, 70, 20, 17, 36, (1, 1, 1, 1)),
    (1, 64, 56, 56, 64, (1, 1, 1, 1)),      # BASELINE config 1 through F(6,3)
]


@pytest.mark.parametrize("mode", ["f63", "f23"])
@pytest.mark.parametrize("case", WINO_CASES)
def test_winograd(tsx, port, case, mode):
    n, c, h, w, cout, pads = case
    rng = np.random.default_rng(403)
    x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, c, 3, 3)) * np.sqrt(2.0 / (c * 9))).astype(np.float32)
    op = tsx.Winograd(_dev(wt), pads, mode=mode)
    got = op(_dev(x)).cpu().numpy()
    exp = getattr(port, "winograd_" + mode)(x, wt, pads)
    assert _close(got, exp), np.abs(got - exp).max()
    # same operations in the same order as the reference's AVX2/FMA build: equal bits
    assert np.array_equal(bits(got), bits(exp)), (bits(got) != bits(exp)).mean()


@pytest.mark.parametrize("case", WINO_CASES + [(3, 20, 31, 13, 50, (1, 0, 2, 1)), (2, 64, 28, 28, 96, (1, 1, 1, 1))])
def test_winograd_f63_fast_path(tsx, port, case):
    """The MFMA form of F(6,3) against the reference's F(6,3) values (the oracle is bit-exact to them),
    with bias, activation and a non-zero padding value; channel counts and tile counts that are not multiples of the
    kernel's 16-wide blocks included.  Two F(6,3) evaluations that sum the channel products in different orders
    differ by the method's own fp32 noise (its transforms multiply by up to 32 and cancel again), ~1e-5 absolute on
    O(1) outputs, so the bar is the one TenniS's own backend test applies between devices (tools/run_test/
    test_case.hpp:491-503): max |diff| <= 1e-4 and mean |diff| <= 1e-5; on top of it, all but a small share of the
    elements must meet the strict per-element bar 1e-4 |exp| + 1e-5."""
    n, c, h, w, cout, pads = case
    rng = np.random.default_rng(405)
    x = rng.uniform(-1, 1, (n, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, c, 3, 3)) * np.sqrt(2.0 / (c * 9))).astype(np.float32)
    bias = (rng.standard_normal(cout) * 0.1).astype(np.float32)
    op = tsx.Winograd(_dev(wt), pads, padding_value=0.25, mode="f63")
    got = op(_dev(x), bias=_dev(bias), act="relu", fast=True).cpu().numpy()
    exp = port.relu(port.add_bias(port.winograd_f63(x, wt, pads, padding_value=0.25), bias))
    assert got.shape == exp.shape
    diff = np.abs(got.astype(np.float64) - exp)
    assert diff.max() <= 1e-4 and diff.mean() <= 1e-5, (diff.max(), diff.mean())
    strict = diff <= ABS + REL * np.abs(exp)
    assert strict.mean() >= 0.999, (1.0 - strict.mean(), diff.max())
    # and against the direct convolution in fp64, to see that the tolerance is not hiding a wrong transform
    exact = port.relu(port.add_bias(port.conv2d_f32(x, wt, pads, padding_value=0.25), bias))
    assert np.abs(got - exact).max() < 2e-4


@pytest.mark.parametrize("mode", ["f63", "f23"])
def test_winograd_padding_value_bias_relu(tsx, port, mode):
    rng = np.random.default_rng(404)
    x = rng.uniform(-1, 1, (2, 8, 9, 9)).astype(np.float32)
    wt = (rng.standard_normal((8, 8, 3, 3)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(8).astype(np.float32) * 0.1
    op = tsx.Winograd(_dev(wt), (1, 1, 1, 1), padding_value=0.5, mode=mode)
    got = op(_dev(x), bias=_dev(bias), act="relu").cpu().numpy()
    exp = port.relu(port.add_bias(getattr(port, "winograd_" + mode)(x, wt, (1, 1, 1, 1), padding_value=0.5), bias))
    assert np.array_equal(bits(got), bits(exp))


def test_winograd_rejects_non_3x3(tsx):
    import torch
    with pytest.raises(tsx.TsxError):
        op = tsx.WinogradF63(torch.zeros((4, 4, 3, 3), device="cuda"))
        op.w = torch.zeros((4, 4, 5, 5), device="cuda")
        op(torch.zeros((1, 4, 9, 9), device="cuda"))
