"""ResNet-50-shaped int8 network: the device runner (tennis_amd/resnet50.py) against the CPU oracle
evaluating the same layer description operator by operator (quantize -> conv2d_quantized -> add_bias ->
relu, add, pooling2d, global_pooling2d, quantize -> int8 gemm -> dequant -> add_bias).

Bar: bit-exact logits (every operator on the path is bit-exact and the fused epilogues reproduce the
separate operators' roundings), on a narrow/short network the oracle finishes in seconds, for the eager
path and for replays of a captured HIP graph.
"""
import numpy as np
import pytest

from _util import bits

pytestmark = pytest.mark.gpu


def oracle_forward(port, desc, params, scales, x):
    stem, net, fc = desc
    n = x.shape[0]

    def conv(spec, t):
        p = params[spec.name]
        s = np.float32(scales[spec.name])
        tq = port.quantize(t, np.full(n, s, np.float32))
        dq = (np.float32(1.0) / (s * p["sw"])).astype(np.float32)
        y = port.conv2d_quantized(tq, p["wq"], dq, (spec.pad,) * 4, (spec.stride, spec.stride))
        y = port.add_bias(y, p["bias"])
        return port.relu(y) if spec.relu else y

    y = conv(stem, x)
    y = port.pooling2d(y, "max", (3, 3), (2, 2), (0, 1, 0, 1))
    for c1, c2, c3, proj in net:
        c = conv(c3, conv(c2, conv(c1, y)))
        sc = conv(proj, y) if proj is not None else y
        y = port.relu(port.add(c, sc))
    pooled = port.global_pooling2d(y, "avg").reshape(n, fc[0])
    s = np.float32(scales["fc"])
    p8 = port.quantize(pooled, np.full(n, s, np.float32))
    dq = (np.float32(1.0) / (s * params["fc"]["sw"])).astype(np.float32)
    return port.gemm_i8_dequant(p8, params["fc"]["wq"], dq, None, params["fc"]["bias"])


def test_resnet_shaped_network_bit_exact(port):
    import torch
    from tennis_amd import resnet50
    desc, params = resnet50.make_parameters(seed=3, width=0.25, blocks=(2, 1, 1, 1), classes=40)
    net = resnet50.ResNet50Int8(desc, params)
    rng = np.random.default_rng(4)
    x = rng.uniform(0, 1, (2, 3, 64, 64)).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    scales = net.calibrate(xd)
    net.set_scales(scales, 2)
    got = net.forward(xd).cpu().numpy()
    exp = oracle_forward(port, desc, params, scales, x)
    assert got.shape == exp.shape == (2, 40)
    assert np.isfinite(exp).all() and np.abs(exp).max() > 0
    assert np.array_equal(bits(got), bits(exp)), np.abs(got - exp).max()

    # a different batch through the same calibrated network
    x2 = rng.uniform(0, 1, (2, 3, 64, 64)).astype(np.float32)
    got2 = net.forward(torch.from_numpy(x2).cuda()).cpu().numpy()
    assert np.array_equal(bits(got2), bits(oracle_forward(port, desc, params, scales, x2)))

    # captured HIP graph: replayed several times with eager work and synchronisation in between,
    # every replay checked against the eager result
    static_x = xd.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        net.forward(static_x)          # warm-up on the capture stream: packs weights, sizes workspaces
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = net.forward(static_x)
    for batch, want in ((x2, got2), (x, got), (x2, got2)):
        static_x.copy_(torch.from_numpy(batch).cuda())
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bits(static_out.cpu().numpy()), bits(want))
        net.forward(xd)                # eager work between replays
        torch.cuda.synchronize()


def test_full_size_network_every_layer(port):
    """BASELINE config 4 at its real size (batch 32, 3x224x224, full width and depth): the tile plans the
    kernels pick here differ from the small network's.  Every convolution of the chained pass is checked by
    itself for the first and the last image of the batch: the oracle runs the operator chain on the very
    tensor the device kernel read (its staged int8 input), so one layer's result does not depend on another's.
    Bar: bit-exact fp32 outputs and int8 hand-overs."""
    import torch
    from tennis_amd import resnet50
    n = 32
    desc, params = resnet50.make_parameters(seed=0)
    net = resnet50.ResNet50Int8(desc, params)
    x = torch.rand((n, 3, 224, 224), device="cuda", generator=torch.Generator(device="cuda").manual_seed(11))
    scales = net.calibrate(x)
    net.set_scales(scales, n)
    imgs = (0, n - 1)
    net.trace = (imgs, [])
    logits = net.forward(x)
    torch.cuda.synchronize()
    rows, net.trace = net.trace[1], None
    assert torch.isfinite(logits).all()
    checked, prev_q = 0, None
    for row in rows:
        spec = row["spec"]
        if spec == "pool":
            pooled = port.pooling2d(prev_q.astype(np.float32), "max", (3, 3), (2, 2), (0, 1, 0, 1)).astype(np.int8)
            assert np.array_equal(row["out_q"], pooled), "max pooling on int8"
            continue
        p = params[spec.name]
        s = np.float32(scales[spec.name])
        xq = row["in_q"] if row["in_q"] is not None else port.quantize(row["in_f32"], np.full(len(imgs), s, np.float32))
        dq = (np.float32(1.0) / (s * p["sw"])).astype(np.float32)
        y = port.add_bias(port.conv2d_quantized(xq, p["wq"], dq, (spec.pad,) * 4, (spec.stride, spec.stride)), p["bias"])
        if row["residual"] is not None:
            y = port.relu(port.add(y, row["residual"]))
        elif spec.relu:
            y = port.relu(y)
        if row["out_f32"] is not None:
            assert np.array_equal(bits(row["out_f32"]), bits(y)), spec.name
        if row["out_q"] is not None:
            q = port.quantize(y, np.full(len(imgs), np.float32(scales[row["q_name"]]), np.float32))
            assert np.array_equal(row["out_q"], q), spec.name
            prev_q = row["out_q"]
        checked += 1
    assert checked == 53      # 1 stem + 16 blocks x 3 + 4 projections


def test_mac_count_of_the_full_network():
    from tennis_amd import resnet50
    desc = resnet50.layers()
    macs = resnet50.total_macs(desc, 1, 224)
    assert 4.0e9 < macs < 4.2e9      # the ResNet-50 v1.5 figure, 4.09 GMAC per image
