"""YOLOv4-shaped int8 network: the device runner (tennis_amd/yolov4.py) against the CPU oracle interpreting
the same layer list operator by operator.

Every operator on the path is bit-exact, Mish in its default (exact) form included: the heads of the small network
match the oracle's bit for bit, and at full size every layer's fp32 output and int8 hand-over is the operator
chain's -- the frozen bar allows 2 differing int8 values over the 190 M of the pass (none has been seen).  With the
opt-in fast Mish (mish="fast": one hardware exponential and reciprocal, 1e-7 relative) a value now and then lands
on the other side of a rounding boundary of the next quantize: at most 200 of the 190 M, each by one step.
"""
import numpy as np
import pytest

from _util import bits

pytestmark = pytest.mark.gpu


def oracle_forward(port, L, heads, srcs, params, scales, x):
    n = x.shape[0]
    outs = []
    for i, l in enumerate(L):
        src = [x if j < 0 else outs[j] for j in srcs[i]]
        if l["type"] == "conv":
            p, s = params[i], np.float32(scales[i])
            tq = port.quantize(src[0], np.full(n, s, np.float32))
            dq = (np.float32(1.0) / (s * p["sw"])).astype(np.float32)
            pad = l["size"] // 2
            y = port.add_bias(port.conv2d_quantized(tq, p["wq"], dq, (pad,) * 4, (l["stride"],) * 2), p["bias"])
            if l["act"] == "mish":
                y = port.mish(y)
            elif l["act"] == "leaky_relu":
                y = port.leaky_relu(y, 0.1)
        elif l["type"] == "route":
            y = src[0] if len(src) == 1 else port.concat(src, 1)
        elif l["type"] == "shortcut":
            y = port.add(src[0], src[1])
        elif l["type"] == "maxpool":
            k = l["size"]
            y = port.pooling2d(src[0], "max", (k, k), (1, 1), (k // 2,) * 4)
        elif l["type"] == "upsample":
            y = port.resize_nearest(src[0], src[0].shape[2] * 2, src[0].shape[3] * 2)
        outs.append(y)
    return [outs[h] for h in heads]


@pytest.mark.parametrize("mish", ["exact", "fast", None])
def test_yolov4_shaped_network(port, mish):
    import torch
    from tennis_amd import yolov4
    L, heads = yolov4.layers(width=0.125, classes=3)
    if mish is None:
        for l in L:
            if l["type"] == "conv" and l["act"] == "mish":
                l["act"] = "leaky_relu"
    params = yolov4.make_parameters(L, seed=5)
    net = yolov4.YoloV4Int8(L, heads, params, mish=mish or "exact")
    x = np.random.default_rng(6).uniform(0, 1, (2, 3, 64, 64)).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    scales = net.calibrate(xd)
    got = [t.cpu().numpy() for t in net.forward(xd)]                      # chained: int8 hand-over, folded shortcuts
    plain = [t.cpu().numpy() for t in net.forward(xd, chained=False)]      # one operator per layer, fp32 in between
    for g, q in zip(got, plain):
        assert np.array_equal(bits(g), bits(q))
    srcs, _ = yolov4.resolve(L)
    exp = oracle_forward(port, L, heads, srcs, params, scales, x)
    assert [g.shape for g in got] == [(2, 24, 8, 8), (2, 24, 4, 4), (2, 24, 2, 2)]
    for g, e in zip(got, exp):
        assert g.shape == e.shape and np.isfinite(e).all() and np.abs(e).max() > 0
        if mish == "fast":
            assert np.abs(g - e).max() <= 2e-3 * np.abs(e).max()
        else:
            assert np.array_equal(bits(g), bits(e))


@pytest.mark.parametrize("mish", ["exact", "fast"])
def test_full_size_network_every_layer(port, capsys, mish):
    """BASELINE config 5 at its real size (batch 8, 3x608x608, full width): every convolution of the chained
    pass checked by itself for the first and the last image -- the oracle runs the operator chain on the very
    tensor the device kernel read, so one layer's result does not depend on another's.  Bar for LeakyReLU / linear
    layers: bit-exact fp32 outputs and int8 hand-overs.  Mish layers, exact form (the default): fp32 outputs bit for
    bit, and at most 2 differing int8 hand-over values over the whole pass; fast form (only its Mish layers are
    checked): fp32 within 1e-4 relative + 1e-5 absolute, int8 hand-over values that differ differ by one step and
    number at most 200 over the whole pass."""
    import torch
    from tennis_amd import yolov4
    n = 8
    L, heads = yolov4.layers()
    params = yolov4.make_parameters(L, seed=0)
    net = yolov4.YoloV4Int8(L, heads, params, mish=mish)
    x = torch.rand((n, 3, 608, 608), device="cuda", generator=torch.Generator(device="cuda").manual_seed(12))
    scales = net.calibrate(x)
    imgs = (0, n - 1)
    net.trace = (imgs, [])
    outs = net.forward(x)
    torch.cuda.synchronize()
    rows, net.trace = net.trace[1], None
    assert all(torch.isfinite(o).all() for o in outs)
    report, checked, worst_f32, f32_bits_off = [], 0, 0.0, 0
    for row in rows:
        i = row["layer"]
        l, p, s = L[i], params[i], np.float32(scales[i])
        is_mish = l["act"] == "mish"
        checked += 1
        if mish == "fast" and not is_mish:
            continue                                   # the other layers are the exact run's, checked there
        xq = row["in_q"] if row["in_q"] is not None else port.quantize(row["in_f32"], np.full(len(imgs), s, np.float32))
        dq = (np.float32(1.0) / (s * p["sw"])).astype(np.float32)
        pad = l["size"] // 2
        y = port.add_bias(port.conv2d_quantized(xq, p["wq"], dq, (pad,) * 4, (l["stride"],) * 2), p["bias"])
        if is_mish:
            y = port.mish(y)
        elif l["act"] == "leaky_relu":
            y = port.leaky_relu(y, 0.1)
        if row["residual"] is not None:
            y = port.add(y, row["residual"])          # darknet's shortcut joins behind the activation
        loose = is_mish and mish == "fast"
        if row["out_f32"] is not None:
            if loose:
                err = np.abs(row["out_f32"].astype(np.float64) - y)
                assert (err <= 1e-4 * np.abs(y) + 1e-5).all(), "layer %d" % i
                worst_f32 = max(worst_f32, float((err / (np.abs(y) + 1e-3)).max()))
            else:
                off = int(np.count_nonzero(bits(row["out_f32"]) != bits(y)))
                assert off == 0, "layer %d: %d fp32 values differ" % (i, off)
        if row["out_q"] is not None:
            q = port.quantize(y, np.full(len(imgs), np.float32(scales[row["q_layer"]]), np.float32))
            diff = row["out_q"].astype(np.int32) - q.astype(np.int32)
            bad = int(np.count_nonzero(diff))
            if not is_mish:
                assert bad == 0, "layer %d: %d int8 values differ" % (i, bad)
            else:
                report.append((i, bad, diff.size))
                assert np.abs(diff).max() <= 1, "layer %d" % i
    assert checked == 110
    total, values = sum(b for _, b, _ in report), sum(c for _, _, c in report)
    with capsys.disabled():
        print("\nMish (%s) layers, int8 hand-over values that differ from the host's (layer: differing / values): " % mish
              + (", ".join("%d: %d/%d" % r for r in report if r[1]) or "none")
              + "; total %d of %d; largest fp32 deviation %.2e of |value| + 1e-3" % (total, values, worst_f32))
    assert total <= (2 if mish == "exact" else 200), "%d int8 hand-over values of the Mish layers differ" % total


def test_layer_list_matches_yolov4():
    from tennis_amd import yolov4
    L, heads = yolov4.layers()
    assert sum(1 for l in L if l["type"] == "conv") == 110          # the 110 convolutions of yolov4.cfg
    macs = yolov4.total_macs(L, 1, 608)
    assert 60e9 < macs < 68e9                                        # ~64 GMAC per 608x608 image


def test_fast_mish_error_bound_every_float():
    """|mish_short(x) - mish_value(x)| <= 5.21 * 2^-24 |x| for every float x (measured maximum, at x = 0.768): the
    bound the int8-only epilogues rely on (with 8 * 2^-24 |x|) when they evaluate the exact form only next to a
    rounding boundary.  All 2^32 bit patterns, both forms through the C ABI (tsx_add_f32 with the fast activation
    on x + 0, tsx_mish_f32), compared in float64 on the device; non-finite results must coincide."""
    import torch
    from tennis_amd import capi
    dev = torch.device("cuda:0")
    chunk = 1 << 26
    zeros = torch.zeros(chunk, device=dev)
    worst = 0.0
    for first in range(0, 1 << 32, chunk):
        b = torch.arange(first, first + chunk, device=dev, dtype=torch.int64)
        x = torch.where(b >= (1 << 31), b - (1 << 32), b).to(torch.int32).view(torch.float32)
        fast = capi.add(x, zeros, act="mish_fast")
        exact = capi.mish(x)
        finite = torch.isfinite(x) & (x != 0)
        assert bool((torch.isfinite(fast) == torch.isfinite(exact))[finite].all()), first
        both = finite & torch.isfinite(exact)
        ratio = (fast.double() - exact.double()).abs() / (x.double().abs() * 2.0 ** -24)
        worst = max(worst, float(torch.where(both, ratio, torch.zeros_like(ratio)).max()))
    assert worst <= 6.0, worst
