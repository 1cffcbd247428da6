"""The flat-tile and the weight-stationary int8 MFMA kernels each by themselves, against the CPU oracle bit for bit.

The planner gives these kernels large layers only (160 workgroups and more), which the small seeded cases of
tests/test_gpu_int8.py never are; here TSX_CONV_I8_FLAT=force / TSX_CONV_I8_RS=force (read at every plan) put small
layers on them, and tsx_conv2d_i8_plan_info confirms which kernel the plan launches before anything is compared.
Covered: kernels of 2..5 taps a side, strides, dilations, asymmetric padding, ragged channel counts and output
channels that are no multiple of 32 or 64, tiles that span several images and end inside one, windows that do and
do not fit LDS whole (resident / double-buffered with remainder K-steps), rows that wrap backwards (stride 2 on an
unpadded map), staged buffers wider than the layer needs, and every epilogue term: raw accumulators, fp32, bias,
ReLU / LeakyReLU / Mish, residual in front of and behind the activation, requantized NCHW and staged int8 output.
"""
import numpy as np
import pytest

from _util import bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tsx():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from tennis_amd import capi
    capi.lib()
    return capi


@pytest.fixture
def force(monkeypatch):
    def choose(kernel, tile=""):
        """tile: for the flat-tile kernel "43" = tiles of 4 + 3 fragments only (default: the largest tile that fits);
        for the weight-stationary kernel "6" = tiles of 6 fragments (default: at most 5)."""
        monkeypatch.setenv("TSX_CONV_I8_FLAT", "force" + tile if kernel == "flat_tile" else "0")
        monkeypatch.setenv("TSX_CONV_I8_RS", "force" + tile if kernel == "weight_stationary" else "0")
    return choose


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _plan(tsx, conv, x_shape):
    return tsx.conv2d_i8_plan_info(conv._plan(tuple(x_shape))[0])


def flat_cases(count, seed):
    """Seeded geometries of the kind the flat-tile kernel admits: more than one tap, more than 64 output channels, a
    tile's window of at most 512 pixels (large dilated kernels on wide strided maps exceed it and are declined)."""
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        kh, kw = (int(v) for v in rng.choice([1, 2, 3, 3, 5], 2))
        if kh * kw == 1:
            continue
        st = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        dl = (int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2])))
        pads = tuple(int(rng.integers(0, k // 2 + 2)) for k in (kh, kh, kw, kw))
        n, c = int(rng.integers(1, 5)), int(rng.choice([3, 16, 40, 64, 70, 130, 200]))
        cout = int(rng.choice([65, 96, 100, 128, 130, 200]))
        h, w = int(rng.integers(5, 30)), int(rng.integers(5, 46))
        if h + pads[0] + pads[1] < dl[0] * (kh - 1) + 1 or w + pads[2] + pads[3] < dl[1] * (kw - 1) + 1:
            continue
        cases.append((n, c, h, w, cout, kh, kw, pads, st, dl))
    return cases


FLAT_FIXED = [
    # n, c, h, w, cout, kh, kw, pads, strides, dilations
    (5, 64, 7, 7, 96, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),        # 49 positions an image: every tile spans images
    (2, 40, 20, 21, 130, 1, 3, (0, 0, 1, 1), (2, 1), (1, 1)),     # rows wrap backwards: hs < ho * stride
    (1, 600, 12, 60, 72, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # 10 channel blocks of wide rows: windows double-buffered,
                                                                  # 90 K-steps (a remainder of the ring of 4)
    (2, 330, 9, 40, 100, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),     # 6 channel blocks, 54 K-steps
    (3, 256, 14, 14, 256, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),    # a ResNet stage-4 layer
    (1, 16, 3, 160, 65, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1)),      # rows longer than a tile
]


@pytest.mark.parametrize("case", flat_cases(24, 977) + FLAT_FIXED)
def test_flat_tile_kernel_every_output(tsx, port, force, case):
    n, c, h, w, cout, kh, kw, pads, st, dl = case
    force("flat_tile")
    rng = np.random.default_rng(hash(case) % (1 << 31))
    x = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    wt = rng.integers(-127, 128, (cout, c, kh, kw)).astype(np.int8)
    dq = rng.uniform(1e-4, 1e-3, cout).astype(np.float32)
    bias = rng.standard_normal(cout).astype(np.float32)
    qs = np.full(n, 6.0, np.float32)
    conv = tsx.Conv2dI8(_dev(wt), pads, st, dl)
    info = _plan(tsx, conv, x.shape)
    if info["kernel"] != "flat_tile":
        assert case not in FLAT_FIXED, info
        pytest.skip("the flat-tile plan declines this geometry: %r" % (info,))
    exp, exp_q = port.conv2d_i8_fused(x, wt, dq, bias, "leaky_relu", 0.1, qs, pads, st, dl)
    # with the raw accumulators (the per-element epilogue) ...
    out, q, acc = conv(_dev(x), dq=_dev(dq), bias=_dev(bias), act="leaky_relu", slope=0.1, q_scales=_dev(qs), want_acc=True)
    assert np.array_equal(acc.cpu().numpy(), port.conv2d_quantized(x, wt, dq, pads, st, dl, return_acc=True)[1])
    assert np.array_equal(bits(out.cpu().numpy()), bits(exp))
    assert np.array_equal(q.cpu().numpy(), exp_q)
    # ... and without them (the fragment-wise one)
    out2, q2, _ = conv(_dev(x), dq=_dev(dq), bias=_dev(bias), act="leaky_relu", slope=0.1, q_scales=_dev(qs))
    assert np.array_equal(bits(out2.cpu().numpy()), bits(exp)) and np.array_equal(q2.cpu().numpy(), exp_q)
    # fp32 output alone, no bias, ReLU: the streaming-store path of plain outputs
    out3 = conv(_dev(x), dq=_dev(dq), act="relu")[0]
    assert np.array_equal(bits(out3.cpu().numpy()), bits(port.conv2d_i8_fused(x, wt, dq, None, "relu", 0.0, None, pads, st, dl)[0]))


def test_flat_tile_kernel_is_taken(tsx, force):
    """Most seeded cases and every fixed one run on the kernel under test (a declined geometry is skipped above, not
    silently run on another kernel), on tiles of several sizes and with both window schedules -- every channel
    block's window resident in LDS, or two windows double-buffered."""
    force("flat_tile")
    taken, tiles, resident = 0, set(), set()
    for case in flat_cases(24, 977) + FLAT_FIXED:
        n, c, h, w, cout, kh, kw, pads, st, dl = case
        conv = tsx.Conv2dI8(_dev(np.zeros((cout, c, kh, kw), np.int8)), pads, st, dl)
        info = _plan(tsx, conv, (n, c, h, w))
        if info["kernel"] == "flat_tile":
            taken += 1
            tiles.add(info["fragments_per_tile"])
            resident.add(info["resident"])
    assert taken >= 22 and len(tiles) >= 4 and resident == {"0", "1"}, (taken, tiles, resident)


@pytest.mark.parametrize("split", ["11", "21", "22", "32", "33", "43", "44"])
def test_flat_tile_kernel_every_tile_size(tsx, port, force, split):
    """One layer (two images of a 30x40 map, 3x3, 100 channels in, 130 out; stride 1 and column stride 2) on every
    instantiated tile size, full epilogue."""
    force("flat_tile", split)
    rng = np.random.default_rng(977)
    n, c, h, w, cout = 2, 100, 30, 40, 130
    x = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    wt = rng.integers(-127, 128, (cout, c, 3, 3)).astype(np.int8)
    dq = rng.uniform(1e-4, 1e-3, cout).astype(np.float32)
    bias = rng.standard_normal(cout).astype(np.float32)
    qs = np.full(n, 5.0, np.float32)
    for st in ((1, 1), (1, 2)):
        conv = tsx.Conv2dI8(_dev(wt), (1, 1, 1, 1), st)
        info = _plan(tsx, conv, x.shape)
        if st == (1, 2) and info["kernel"] != "flat_tile":
            continue                       # the larger tiles' windows of a strided layer exceed the kernel's 512 pixels
        assert info["kernel"] == "flat_tile" and info["fragments_per_tile"] == str(int(split[0]) + int(split[1])), info
        out, q, _ = conv(_dev(x), dq=_dev(dq), bias=_dev(bias), act="relu", q_scales=_dev(qs))
        exp, exp_q = port.conv2d_i8_fused(x, wt, dq, bias, "relu", 0.0, qs, (1, 1, 1, 1), st)
        assert np.array_equal(bits(out.cpu().numpy()), bits(exp)) and np.array_equal(q.cpu().numpy(), exp_q)


@pytest.mark.parametrize("case", [
    # n, cin, h, w, cout, stride, consumer kernel
    (3, 70, 9, 11, 130, 1, 3),
    (2, 130, 12, 13, 96, 2, 1),
    (4, 64, 7, 7, 200, 1, 3),
])
@pytest.mark.parametrize("after", [False, True])
@pytest.mark.parametrize("act", ["leaky_relu", "mish"])
def test_flat_tile_kernel_all_epilogue_terms(tsx, port, force, case, after, act):
    """Residual join + fp32 output + requantized staged output together; the staged output is checked through a
    consumer convolution.  Mish is the exact form: the values of the operator chain."""
    n, cin, h, w, cout, s, ck = case
    force("flat_tile")
    rng = np.random.default_rng(311)
    xq = rng.integers(-128, 128, (n, cin, h, w)).astype(np.int8)
    wa = rng.integers(-127, 128, (cout, cin, 3, 3)).astype(np.int8)
    dqa = rng.uniform(1e-5, 3e-5, cout).astype(np.float32)
    ba = rng.standard_normal(cout).astype(np.float32)
    qs = np.full(n, 7.0, np.float32)
    A = tsx.Conv2dI8(_dev(wa), (1, 1, 1, 1), (s, s))
    assert _plan(tsx, A, xq.shape)["kernel"] == "flat_tile"
    plain = port.conv2d_i8_fused(xq, wa, dqa, ba, None, pads=(1, 1, 1, 1), strides=(s, s))[0]
    res = (rng.standard_normal(plain.shape) * np.abs(plain).mean()).astype(np.float32)
    f_act = (lambda t: port.leaky_relu(t, 0.1)) if act == "leaky_relu" else port.mish
    exp = port.add(f_act(plain), res) if after else f_act(port.add(plain, res))
    exp_q = port.quantize(exp, qs)
    wb = rng.integers(-127, 128, (40, cout, ck, ck)).astype(np.int8)
    dqb = rng.uniform(1e-4, 3e-4, 40).astype(np.float32)
    B = tsx.Conv2dI8(_dev(wb), (ck // 2,) * 4)
    sb = tsx.StagedInput(B, tuple(plain.shape))
    sa = tsx.StagedInput(A, tuple(xq.shape))
    A.stage(_dev(xq), sa)
    f = A.run_staged(sa, _dev(dqa), _dev(ba), act, 0.1, q_scales=_dev(qs), residual=_dev(res), staged_out=sb,
                     residual_after_act=after)[0]
    assert np.array_equal(bits(f.cpu().numpy()), bits(exp))
    got = B.run_staged(sb, _dev(dqb))[0].cpu().numpy()
    assert np.array_equal(bits(got), bits(port.conv2d_quantized(exp_q, wb, dqb, (ck // 2,) * 4)))


@pytest.mark.parametrize("kernel", ["window_stationary", "flat_tile", "igemm"])
@pytest.mark.parametrize("after", [None, False, True])
def test_exact_mish_where_only_int8_leaves(tsx, port, force, kernel, after):
    """A layer that hands over nothing but requantized int8 values (no fp32 output) evaluates the exact Mish only
    where it decides a rounding and the one-exponential form elsewhere: the bytes must be those of the operator
    chain all the same.  Checked through a consumer convolution on each kernel family, without a residual, with one
    in front of the activation (the exact form throughout) and with one behind it; consumer scales of 20 to 60 put
    some thousand of the 10^5..10^6 values within 10^-4 of a rounding boundary."""
    n, cin, h, w, cout, s = (4, 70, 24, 26, 130, 1) if kernel != "igemm" else (4, 70, 24, 26, 130, 2)
    k = 3 if kernel != "igemm" else 1
    force(kernel)
    rng = np.random.default_rng(977 + (0 if after is None else 1 + int(after)))
    xq = rng.integers(-128, 128, (n, cin, h, w)).astype(np.int8)
    wa = rng.integers(-127, 128, (cout, cin, k, k)).astype(np.int8)
    dqa = rng.uniform(2e-5, 6e-5, cout).astype(np.float32)
    ba = rng.standard_normal(cout).astype(np.float32)
    qs = rng.uniform(20.0, 60.0, n).astype(np.float32)
    A = tsx.Conv2dI8(_dev(wa), (k // 2,) * 4, (s, s))
    assert _plan(tsx, A, xq.shape)["kernel"] == kernel
    plain = port.conv2d_i8_fused(xq, wa, dqa, ba, None, pads=(k // 2,) * 4, strides=(s, s))[0]
    res = None if after is None else (rng.standard_normal(plain.shape) * 0.5).astype(np.float32)
    exp = port.mish(plain) if after is None else port.add(port.mish(plain), res) if after else port.mish(port.add(plain, res))
    exp_q = port.quantize(exp, qs)
    wb = rng.integers(-127, 128, (40, cout, 3, 3)).astype(np.int8)
    dqb = rng.uniform(1e-4, 3e-4, 40).astype(np.float32)
    B = tsx.Conv2dI8(_dev(wb), (1, 1, 1, 1))
    sb = tsx.StagedInput(B, tuple(plain.shape))
    sa = tsx.StagedInput(A, tuple(xq.shape))
    A.stage(_dev(xq), sa)
    A.run_staged(sa, _dev(dqa), _dev(ba), "mish", 0.0, q_scales=_dev(qs), staged_out=sb, want_f32=False,
                 residual=None if res is None else _dev(res), residual_after_act=bool(after))
    got = B.run_staged(sb, _dev(dqb))[0].cpu().numpy()
    assert np.array_equal(bits(got), bits(port.conv2d_quantized(exp_q, wb, dqb, (1, 1, 1, 1))))
    # the same layer's NCHW int8 output
    q = A.run_staged(sa, _dev(dqa), _dev(ba), "mish", 0.0, q_scales=_dev(qs), want_f32=False,
                     residual=None if res is None else _dev(res), residual_after_act=bool(after))[1]
    assert np.array_equal(q.cpu().numpy(), exp_q)


def test_flat_tile_kernel_reads_a_wider_staged_buffer(tsx, port, force):
    """A 3x3 convolution without padding reading the staged input of a padded one (tsx_conv2d_i8_staged_at: the
    buffer's row and image pitch are larger than the layer's own)."""
    force("flat_tile")
    rng = np.random.default_rng(312)
    n, c, h, w = 3, 70, 11, 13
    xq = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    wa = rng.integers(-127, 128, (96, c, 3, 3)).astype(np.int8)
    wb = rng.integers(-127, 128, (130, c, 3, 3)).astype(np.int8)
    dqa = rng.uniform(1e-4, 3e-4, 96).astype(np.float32)
    dqb = rng.uniform(1e-4, 3e-4, 130).astype(np.float32)
    A = tsx.Conv2dI8(_dev(wa), (2, 2, 2, 2), dilations=(2, 2))       # owner: halo of 2
    B = tsx.Conv2dI8(_dev(wb), (1, 1, 0, 0))                          # reads it with halo (1, 0)
    assert _plan(tsx, A, xq.shape)["kernel"] == "flat_tile" and _plan(tsx, B, xq.shape)["kernel"] == "flat_tile"
    sa = tsx.StagedInput(A, xq.shape)
    A.stage(_dev(xq), sa)
    got_a = A.run_staged(sa, _dev(dqa))[0].cpu().numpy()
    assert np.array_equal(bits(got_a), bits(port.conv2d_quantized(xq, wa, dqa, (2, 2, 2, 2), (1, 1), (2, 2))))
    got_b = B.run_staged(tsx.StagedView(sa, 1, 0), _dev(dqb))[0].cpu().numpy()
    assert np.array_equal(bits(got_b), bits(port.conv2d_quantized(xq, wb, dqb, (1, 1, 0, 0))))


# ---------------------------------------------------------------- weight-stationary kernel

def rs_cases(count, seed):
    """Seeded geometries of the kind the weight-stationary kernel admits: 3x3 taps, stride 1, on 193..256 channels,
    more than 64 output channels, maps 16 to 30 pixels wide (window rows of at most 32 pixels; a fragment then
    covers at most two rows, which is what the kernel's ring takes in per fragment), asymmetric padding."""
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        pads = tuple(int(rng.integers(0, 3)) for _ in range(4))
        n, c = int(rng.integers(1, 5)), int(rng.choice([193, 200, 224, 255, 256]))
        cout = int(rng.choice([65, 96, 100, 128, 130, 200, 256]))
        h, w = int(rng.integers(5, 30)), int(rng.integers(16, 29))
        cases.append((n, c, h, w, cout, pads, (1, 1), (1, 1), ""))
    return cases


RS_FIXED = [
    # n, c, h, w, cout, pads, strides, dilations, fragments per tile ("": at most 5)
    (2, 256, 28, 28, 256, (1, 1, 1, 1), (1, 1), (1, 1), ""),      # two images of BASELINE config 2
    (2, 256, 28, 28, 256, (1, 1, 1, 1), (1, 1), (1, 1), "9"),     # ... in tiles of 9 fragments (odd: the loop's tail)
    (3, 256, 17, 20, 128, (1, 1, 1, 1), (1, 1), (1, 1), "4"),     # 10.6 fragments an image: tiles that span two images
    (1, 200, 9, 30, 65, (0, 0, 0, 0), (1, 1), (1, 1), "3"),       # no padding, a second 64-channel tile with one channel
    (2, 224, 12, 30, 100, (2, 0, 0, 2), (1, 1), (1, 1), "6"),     # asymmetric padding
    (1, 256, 6, 6, 72, (1, 1, 1, 1), (1, 1), (1, 1), ""),         # a small map: the whole of it in the ring
    (1, 256, 12, 30, 96, (1, 1, 1, 1), (2, 1), (1, 1), "3"),      # stride 2 down the rows
    (1, 256, 9, 29, 96, (1, 1, 1, 1), (1, 2), (1, 1), "3"),       # stride 2 along the rows
    (1, 256, 5, 29, 96, (1, 1, 1, 1), (2, 2), (1, 1), ""),        # both
    (1, 224, 9, 28, 80, (2, 2, 1, 1), (1, 1), (2, 1), "3"),       # dilated rows
]


@pytest.mark.parametrize("act", [None, "relu", "leaky_relu", "mish_fast"])
@pytest.mark.parametrize("case", rs_cases(10, 4242) + RS_FIXED)
def test_weight_stationary_kernel(tsx, port, force, case, act):
    n, c, h, w, cout, pads, st, dl, frags = case
    force("weight_stationary", frags)
    rng = np.random.default_rng(hash(case[:-1]) % (1 << 31))
    x = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    wt = rng.integers(-127, 128, (cout, c, 3, 3)).astype(np.int8)
    dq = rng.uniform(1e-5, 1e-4, cout).astype(np.float32)
    dq[1] = -dq[1]                                         # zero sums times a negative scale: -0.0 into the activation
    bias = rng.standard_normal(cout).astype(np.float32) if act != "relu" else None
    if bias is not None:
        bias[3] = -0.0
    x[:, :, :2] = 0                                        # rows of exact zero sums
    conv = tsx.Conv2dI8(_dev(wt), pads, st, dl)
    info = _plan(tsx, conv, x.shape)
    if info["fp32_kernel"] != "weight_stationary":
        assert case not in RS_FIXED, info
        pytest.skip("the weight-stationary plan declines this geometry: %r" % (info,))
    assert not frags or info["fragments_per_tile"] == frags, info
    out = conv(_dev(x), dq=_dev(dq), bias=None if bias is None else _dev(bias), act=act, slope=0.1)[0].cpu().numpy()
    if act == "mish_fast":
        exp = port.mish(port.conv2d_i8_fused(x, wt, dq, bias, None, 0.0, None, pads, st, dl)[0])
        assert np.all(np.abs(out.astype(np.float64) - exp) <= 1e-4 * np.abs(exp) + 1e-5)     # the fast form's bar
    else:
        exp = port.conv2d_i8_fused(x, wt, dq, bias, act, 0.1, None, pads, st, dl)[0]
        assert np.array_equal(bits(out), bits(exp))


def test_weight_stationary_kernel_is_taken(tsx, force):
    """Most of the seeded cases run on the kernel under test (a declined geometry is skipped above, not silently run
    on another kernel; the fixed ones must all be taken)."""
    taken = 0
    for n, c, h, w, cout, pads, st, dl, frags in rs_cases(10, 4242):
        force("weight_stationary", frags)
        conv = tsx.Conv2dI8(_dev(np.zeros((cout, c, 3, 3), np.int8)), pads, st, dl)
        taken += _plan(tsx, conv, (n, c, h, w))["fp32_kernel"] == "weight_stationary"
    assert taken >= 8, taken


def test_config2_takes_the_weight_stationary_kernel_by_default(tsx, monkeypatch):
    monkeypatch.delenv("TSX_CONV_I8_FLAT", raising=False)
    monkeypatch.delenv("TSX_CONV_I8_RS", raising=False)
    conv = tsx.Conv2dI8(_dev(np.zeros((256, 256, 3, 3), np.int8)), (1, 1, 1, 1))
    info = _plan(tsx, conv, (32, 256, 28, 28))
    assert info["kernel"] == "flat_tile" and info["fp32_kernel"] == "weight_stationary", info
