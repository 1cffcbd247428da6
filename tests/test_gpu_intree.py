"""The "hip" backend inside the real TenniS runtime: tennis_amd/backend/intree/intree.mk compiles
tennis_amd/backend/hip/*.cpp against TenniS's own headers and links them into the TenniS library, as TenniS does
with its own device backends (tennis_amd/lib/intree/libtennis_hip.so, driven through tennis_amd/intree.py).  Each
operator is then created and run by TenniS's Workbench on ComputingDevice("hip") and on ComputingDevice("cpu") --
same process, same operator factory, same Tensor/SyncMemory machinery -- and the two outputs compared.

Bar: bitwise for the int8 operators, the elementwise operators and Winograd F(6,3); 1e-4
relative + 1e-5 absolute for the fp32 MFMA GEMM paths.  Skipped where the in-tree build is absent
(it needs the TenniS source tree at build time).

A "hip" class hands inputs its kernel does not cover to the host operator of the same name.  So that a comparison
of "hip" with "cpu" cannot quietly become one of "cpu" with "cpu", every test here runs under a check that the
library's count of such hand-overs did not move -- except the tests marked `delegates`, which are about exactly
those inputs and must see it rise.
"""
import numpy as np
import pytest

from _util import bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ts():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from tennis_amd import intree
    if not intree.available():
        pytest.skip("tennis_amd/lib/intree/libtennis_hip_driver.so not built in this tree")
    intree.lib()
    return intree


@pytest.fixture(autouse=True)
def host_delegate_watch(request, ts):
    """Yields a dict; a test that hands some operator runs to the host on purpose sets watch["expected"] to their
    number (tests marked `delegates` are about such inputs throughout and only need to see the count rise)."""
    watch = {"expected": 0}
    before = ts.host_delegate_count()
    yield watch
    moved = ts.host_delegate_count() - before
    if request.node.get_closest_marker("delegates"):
        assert moved > 0, "no operator run was handed to the host operator"
    else:
        assert moved == watch["expected"], "%d operator runs on \"hip\" were handed to the host operator, %d expected" % (
            moved, watch["expected"])


def conv_params(ts, pads, strides=(1, 1), dil=(1, 1), pv=0.0):
    return {
        "format": "NCHW",
        "padding": np.array([[0, 0], [0, 0], [pads[0], pads[1]], [pads[2], pads[3]]], np.int32),
        "padding_value": np.array([pv], np.float32),
        "stride": np.array([1, 1, strides[0], strides[1]], np.int32),
        "dilation": np.array([1, 1, dil[0], dil[1]], np.int32),
    }


def both(ts, op, params, inputs, out_bytes):
    cpu = ts.run_op("cpu", op, params, inputs, out_bytes)
    hip = ts.run_op("hip", op, params, inputs, out_bytes)
    assert cpu.shape == hip.shape and cpu.dtype == hip.dtype
    return cpu, hip


def close(a, b):
    return np.all(np.abs(a.astype(np.float64) - b) <= 1e-4 * np.abs(b) + 1e-5)


def test_quantized_chain_in_tennis_workbench(ts):
    rng = np.random.default_rng(900)
    n, c, h, w, cout = 3, 70, 12, 11, 37
    x = (rng.standard_normal((n, c, h, w)) * 30).astype(np.float32)
    scales = np.array([1.3, 0.7, 2.1], np.float32)
    cpu, hip = both(ts, "quantize", {"quantize_scale": scales}, [x], x.size)
    assert np.array_equal(cpu, hip)
    xq = cpu
    wq = rng.integers(-127, 128, (cout, c, 3, 3)).astype(np.int8)
    dq = rng.uniform(1e-4, 1e-3, cout).astype(np.float32)
    for pads, strides, dil, pv in (((1, 1, 1, 1), (1, 1), (1, 1), 0.0), ((2, 0, 1, 2), (2, 1), (1, 2), 3.0)):
        p = conv_params(ts, pads, strides, dil, pv)
        p["dequantize_scales"] = dq
        cpu, hip = both(ts, "conv2d_quantized", p, [xq, wq], 4 * n * cout * (h + 4) * (w + 4))
        assert np.array_equal(bits(cpu), bits(hip)), (pads, strides, dil)
    bias = rng.standard_normal(cout).astype(np.float32)
    y = cpu
    cpu, hip = both(ts, "add_bias", {"dim": np.array([1], np.int32)}, [y, bias], y.nbytes)
    assert np.array_equal(bits(cpu), bits(hip))
    yb = cpu
    cpu, hip = both(ts, "relu", {}, [yb], yb.nbytes)
    assert np.array_equal(bits(cpu), bits(hip))
    cpu, hip = both(ts, "leaky_relu", {"scale": np.array([0.1], np.float32)}, [yb], yb.nbytes)
    assert np.array_equal(bits(cpu), bits(hip))


def test_fp32_operators_in_tennis_workbench(ts):
    rng = np.random.default_rng(901)
    x = rng.uniform(-1, 1, (2, 16, 20, 19)).astype(np.float32)
    w = (rng.standard_normal((24, 16, 3, 3)) * 0.1).astype(np.float32)
    p = conv_params(ts, (1, 1, 1, 1))
    cpu, hip = both(ts, "conv2d", p, [x, w], 4 * 2 * 24 * 20 * 19)
    assert close(hip, cpu)
    # TenniS's skeleton picks F(2,3) for this shape and F(6,3) for the 256x256-channel one
    # (src/kernels/common/function.cpp:154-173); both are bit-exact restatements on the device
    wp = {"format": "NCHW", "padding": p["padding"], "padding_value": p["padding_value"]}
    cpu, hip = both(ts, "conv2d_winograd", wp, [x, w], 4 * 2 * 24 * 20 * 19)
    assert np.array_equal(bits(cpu), bits(hip))
    xb = rng.uniform(-1, 1, (1, 256, 18, 17)).astype(np.float32)
    wb = (rng.standard_normal((256, 256, 3, 3)) * 0.02).astype(np.float32)
    cpu, hip = both(ts, "conv2d_winograd", wp, [xb, wb], 4 * 256 * 18 * 17)
    assert np.array_equal(bits(cpu), bits(hip))
    a = rng.standard_normal((5, 70)).astype(np.float32)
    b = rng.standard_normal((70, 33)).astype(np.float32)
    cpu, hip = both(ts, "inner_prod", {"transpose": np.array([False], np.bool_)}, [a, b], 4 * 5 * 33)
    assert close(hip, cpu)


def test_glue_operators_in_tennis_workbench(ts):
    """pooling2d / global_pooling2d / add / depthwise_conv2d run by TenniS's Workbench with strict device
    lookup, so the "hip" classes are the ones created, and (host_delegate_watch) none of them hands its inputs to the
    host operator: the device produces the result; bitwise against the host operators."""
    rng = np.random.default_rng(902)
    x = rng.standard_normal((2, 6, 14, 12)).astype(np.float32)

    def strict_both(op, params, inputs, out_bytes):
        cpu = ts.run_op("cpu", op, params, inputs, out_bytes)
        hip = ts.run_op("hip", op, params, inputs, out_bytes, strict=True)
        assert cpu.shape == hip.shape
        assert np.array_equal(bits(cpu), bits(hip)), (op, params)

    for kind, k, s, pads, white in ((0, (3, 3), (2, 2), (0, 1, 0, 1), False), (1, (2, 2), (2, 2), (0, 0, 0, 0), False),
                                    (1, (3, 3), (1, 1), (1, 1, 1, 1), True), (0, (5, 5), (1, 1), (2, 2, 2, 2), False)):
        p = {"format": "NCHW", "type": np.array([kind], np.int32),
             "padding": np.array([[0, 0], [0, 0], [pads[0], pads[1]], [pads[2], pads[3]]], np.int32),
             "padding_type": np.array([3 if white else 0], np.int32),
             "ksize": np.array([1, 1, k[0], k[1]], np.int32), "stride": np.array([1, 1, s[0], s[1]], np.int32)}
        strict_both("pooling2d", p, [x], x.nbytes + 4096)
    for kind in (0, 1):
        strict_both("global_pooling2d", {"format": "NCHW", "type": np.array([kind], np.int32)}, [x], 4 * 12)
    for shape in ((2, 6, 14, 12), (1,), (1, 6, 1, 1), (2, 1, 14, 1), (14, 12)):
        b = rng.standard_normal(shape).astype(np.float32)
        strict_both("add", {}, [x, b], x.nbytes)
        strict_both("add", {}, [b, x], x.nbytes)
    w = rng.standard_normal((1, 6, 3, 3)).astype(np.float32)
    for pads, strides, dil, pv in (((1, 1, 1, 1), (1, 1), (1, 1), 0.0), ((0, 2, 1, 0), (2, 1), (1, 2), 0.5)):
        strict_both("depthwise_conv2d", conv_params(ts, pads, strides, dil, pv), [x, w], x.nbytes + 8192)


def test_unregistered_operator_falls_back_to_cpu(ts):
    """An operator the backend does not register runs through TenniS's device -> cpu lookup order
    (src/global/operator_factory.cpp:60-81) on a "hip" Workbench, with the tensors copied by the
    backend's converters."""
    x = np.linspace(-3, 3, 24, dtype=np.float32).reshape(2, 3, 4)
    with pytest.raises(RuntimeError):
        ts.run_op("hip", "sigmoid", {}, [x], x.nbytes, strict=True)
    cpu = ts.run_op("cpu", "sigmoid", {}, [x], x.nbytes)
    hip = ts.run_op("hip", "sigmoid", {}, [x], x.nbytes, strict=False)
    assert np.array_equal(bits(cpu), bits(hip))


def test_v2_wrappers_in_tennis_workbench(ts):
    """The dynamic-padding wrappers registered for "hip" against TenniS's own (cpu) ones, both inside its Workbench."""
    rng = np.random.default_rng(905)
    x = rng.standard_normal((2, 6, 12, 10)).astype(np.float32)
    w = (rng.standard_normal((7, 6, 3, 3)) * 0.2).astype(np.float32)
    full = conv_params(ts, (0, 2, 1, 0), (2, 1), (1, 1), 0.5)
    v2 = {k: v for k, v in full.items() if k != "padding"}
    cpu, hip = both(ts, "conv2d_v2", v2, [x, full["padding"], w], 1 << 20)
    assert close(hip, cpu)
    cpu, hip = both(ts, "depthwise_conv2d_v2", v2, [x, full["padding"], w[:1].copy()], 1 << 20)
    assert close(hip, cpu)
    cpu, hip = both(ts, "pooling2d_v2", {"format": "NCHW", "type": np.array([1], np.int32)},
                    [x, conv_params(ts, (0, 1, 1, 0))["padding"], np.array([1, 1, 3, 2], np.int32), np.array([1, 1, 2, 1], np.int32)],
                    1 << 20)
    assert np.array_equal(bits(cpu), bits(hip))
    cpu, hip = both(ts, "conv2d_winograd_v2", {"format": "NCHW"}, [x, conv_params(ts, (1, 1, 1, 1))["padding"], w], 1 << 20)
    assert np.array_equal(bits(cpu), bits(hip))


def test_concat_and_resize2d_in_tennis_workbench(ts):
    rng = np.random.default_rng(906)
    a, b = rng.standard_normal((2, 5, 7, 6)).astype(np.float32), rng.standard_normal((2, 3, 7, 6)).astype(np.float32)
    cpu, hip = both(ts, "concat", {"dim": np.array([1], np.int32)}, [a, b], 1 << 20)
    assert np.array_equal(bits(cpu), bits(hip))
    cpu, hip = both(ts, "_resize2d", {"type": np.array([2], np.int32)}, [a, np.array([-1, -1, 14, 12], np.int32)], 1 << 20)
    assert np.array_equal(bits(cpu), bits(hip))


def test_module_file_in_tennis_workbench_on_hip(ts):
    """A `.tsm` module loaded by TenniS's own Module::Load, compiled by its graph compiler and run by its Workbench on
    ComputingDevice("hip"): the whole drop-in path (quantize, conv2d_quantized x2, add_bias, relu, pooling2d, concat
    served by this backend).  Same values as on TenniS's CPU device and as the committed expected output."""
    import os
    from tennis_amd import tensor_file
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "modules")
    path = os.path.join(root, "quantized_block.tsm")
    x = tensor_file.read_tensor(os.path.join(root, "quantized_block.input_0.t"))
    want = tensor_file.read_tensor(os.path.join(root, "quantized_block.output_0.t"))
    fused0 = ts.fused_chain_count()
    cpu = ts.run_module("cpu", path, [x])
    assert ts.fused_chain_count() == fused0        # the zipper option is for device "hip" only
    hip = ts.run_module("hip", path, [x])
    # TenniS's compiler, walking the graph with this backend's zipper option, has replaced both chains of the
    # module (quantize -> conv -> add_bias -> relu and quantize -> conv) by conv2d_quantized_fused nodes
    assert ts.fused_chain_count() == fused0 + 2
    assert np.array_equal(bits(cpu), bits(want))
    assert hip.shape == want.shape and np.array_equal(bits(hip), bits(want))


def test_resnet_shaped_module_in_tennis_workbench_on_hip(ts, tmp_path):
    """A ResNet-50-shaped int8 network (quarter width, 2 + 1 + 2 + 1 bottlenecks: 23 quantized convolutions, 6
    residual joins, pooling, global pooling, classifier) written as a `.tsm` module and run (a) by TenniS's own
    runtime on its CPU device, (b) by TenniS's own runtime on ComputingDevice("hip"), (c) by this repository's
    operator-by-operator module runner, plain and with the chain-fusing rewrite.  Everything up to the fp32
    classifier is exact arithmetic shared by all four; the classifier's MFMA summation order differs from the
    host's, hence the fp32 tolerance of 1e-4 relative + 1e-5 absolute on the logits."""
    from tennis_amd import module_file as mf, resnet50
    desc, params = resnet50.make_parameters(seed=3, width=0.25, blocks=(2, 1, 2, 1), classes=10)
    module = resnet50.to_module(desc, params, batch=2)
    path = str(tmp_path / "resnet_shaped.tsm")
    mf.write_module(path, module)
    x = np.random.default_rng(1).random((2, 3, 64, 64), dtype=np.float32)
    cpu = ts.run_module("cpu", path, [x])
    fused0 = ts.fused_chain_count()
    hand0, dual0 = ts.handover_counts()
    hip = ts.run_module("hip", path, [x])
    assert ts.fused_chain_count() == fused0 + 23   # every quantized convolution of the network, fused by TenniS's compiler
    # int8 hand-overs: c1 -> c2 -> c3 inside each of the 6 blocks (12), and each join that another block reads
    # (5: the last one feeds the pooling), plus the stem through its max pooling (2).  The joins in front of the two identity blocks are read by the next
    # block's first convolution AND its residual add, so they return both forms (dual output); the ones in front
    # of a projection block are read by two convolutions of different stride sharing one staged tensor.
    hand, dual = ts.handover_counts()
    assert (hand - hand0, dual - dual0) == (19, 2)
    assert cpu.shape == (2, 10) and hip.shape == (2, 10) and np.abs(cpu).max() > 0.1
    assert close(hip, cpu)
    (own,) = mf.run_module(module, [x])
    (fused,) = mf.run_module(mf.fuse_quantized_chains(module), [x])
    assert np.array_equal(bits(own), bits(hip))          # the same device operators, with or without TenniS around them
    assert np.array_equal(bits(fused), bits(own))


def test_cloned_workbenches_on_hip_one_per_host_thread(ts, tmp_path):
    """TenniS's threading contract on "hip": one Workbench per thread, the further ones made by Workbench::clone
    (src/runtime/workbench.cpp; every instruction's operator is re-created with the same parameters,
    src/runtime/instruction.cpp:91-103; the thread-local contexts of include/utils/ctxmgr_lite_support.h:47-95 are
    bound by each Workbench's own entry points).  The ResNet-50-shaped module -- fused nodes that keep their staged
    int8 output from run to run, packed weights per operator instance, scratch per device context -- is loaded
    once, cloned twice, and the three Workbenches run three times each on three different batches from three host
    threads at once: every thread's logits must be, bit for bit, what a single Workbench gives for its batch."""
    from tennis_amd import module_file as mf, resnet50
    desc, params = resnet50.make_parameters(seed=3, width=0.25, blocks=(2, 1, 2, 1), classes=10)
    path = str(tmp_path / "resnet_shaped.tsm")
    mf.write_module(path, resnet50.to_module(desc, params, batch=2))
    rng = np.random.default_rng(31)
    batches = [rng.random((2, 3, 64, 64), dtype=np.float32) for _ in range(3)]
    alone = [ts.run_module("hip", path, [x]) for x in batches]
    assert not np.array_equal(alone[0], alone[1])
    together = ts.run_module_cloned("hip", path, [[x] for x in batches], runs=3)
    for t, (a, b) in enumerate(zip(alone, together)):
        assert a.shape == b.shape == (2, 10) and np.array_equal(bits(a), bits(b)), "thread %d" % t
    # a control of the driver entry by itself: one thread, the host device of the same library
    (cpu,) = ts.run_module_cloned("cpu", path, [[batches[0]]], runs=1)
    assert np.array_equal(bits(cpu), bits(ts.run_module("cpu", path, [batches[0]])))


def test_full_width_stem_as_column_pairs_in_tennis_workbench_on_hip(ts, tmp_path):
    """The same at full width (one bottleneck per stage): with 64 output channels and an even number of output
    columns the fused stem node runs as pairs of output columns (rearranged weights, half the im2col rows) into the
    staged max pooling.  Bitwise equal to the operator-by-operator run of the same device operators, which has no
    such form, and within the classifier's tolerance of TenniS's CPU device."""
    from tennis_amd import module_file as mf, resnet50
    desc, params = resnet50.make_parameters(seed=5, width=1.0, blocks=(1, 1, 1, 1), classes=10)
    module = resnet50.to_module(desc, params, batch=2)
    path = str(tmp_path / "resnet_full_width.tsm")
    mf.write_module(path, module)
    x = np.random.default_rng(2).random((2, 3, 64, 64), dtype=np.float32)
    cpu = ts.run_module("cpu", path, [x])
    hand0, _ = ts.handover_counts()
    hip = ts.run_module("hip", path, [x])
    assert ts.handover_counts()[0] > hand0
    assert cpu.shape == (2, 10) and np.abs(cpu).max() > 0.1 and close(hip, cpu)
    (own,) = mf.run_module(module, [x])
    assert np.array_equal(bits(own), bits(hip))


def test_zipper_option_leaky_relu_and_shared_convolution(ts, tmp_path):
    """The graph compiler's rewrite on the cases the fixtures do not hold: a chain that ends in leaky_relu behind an
    add_bias given by `dim`, and a convolution whose output has two readers (a relu and an add_bias), where only
    quantize + convolution may fold and both readers must stay.  Two chains fused; values as on TenniS's CPU device."""
    import sys, os
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    from make_modules import conv_params
    from tennis_amd import module_file as mf
    rng = np.random.default_rng(77)
    n, c, h, w, ca, cb = 2, 16, 9, 11, 12, 20
    wa = rng.integers(-127, 128, (ca, c, 3, 3)).astype(np.int8)
    wb = rng.integers(-127, 128, (cb, c, 1, 1)).astype(np.int8)
    N = mf.Node
    nodes = [
        N(mf.PARAMETER, "x"),                                                                                   # 0
        N("quantize", "q", {"quantize_scale": np.array([7.5, 12.0], np.float32)}, [0]),                          # 1
        N(mf.CONST, "wa", {"value": wa}),                                                                       # 2
        N("conv2d_quantized", "conv_a", dict(conv_params((1, 1, 1, 1)),
                                             dequantize_scales=rng.uniform(1e-4, 1e-3, ca).astype(np.float32)), [1, 2]),   # 3
        N(mf.CONST, "ba", {"value": rng.standard_normal(ca).astype(np.float32)}),                               # 4
        N("add_bias", "bias_a", {"dim": np.array([1], np.int32)}, [3, 4]),                                      # 5
        N("leaky_relu", "act_a", {"scale": np.array([0.1], np.float32)}, [5]),                                  # 6
        N(mf.CONST, "wb", {"value": wb}),                                                                       # 7
        N("conv2d_quantized", "conv_b", dict(conv_params((0, 0, 0, 0)),
                                             dequantize_scales=rng.uniform(1e-3, 1e-2, cb).astype(np.float32)), [1, 7]),   # 8
        N("relu", "relu_b", {}, [8]),                                                                           # 9
        N(mf.CONST, "bb", {"value": rng.standard_normal(cb).astype(np.float32)}),                               # 10
        N("add_bias", "bias_b", {"format": "NCHW"}, [8, 10]),                                                   # 11
        N("concat", "join", {"dim": np.array([1], np.int32)}, [6, 9, 11]),                                      # 12
    ]
    module = mf.Module(nodes, [0], [12])
    path = str(tmp_path / "zipper_cases.tsm")
    mf.write_module(path, module)
    x = (rng.standard_normal((n, c, h, w)) * 6).astype(np.float32)
    cpu = ts.run_module("cpu", path, [x])
    fused0 = ts.fused_chain_count()
    hip = ts.run_module("hip", path, [x])
    assert ts.fused_chain_count() == fused0 + 2
    assert cpu.shape == (n, ca + 2 * cb, h, w)
    assert np.array_equal(bits(hip), bits(cpu))
    (own,) = mf.run_module(mf.fuse_quantized_chains(module), [x])     # the same rewrite outside TenniS
    assert np.array_equal(bits(own), bits(cpu))


@pytest.mark.delegates
def test_inputs_a_hip_class_does_not_cover_run_the_host_operator(ts):
    """A registered "hip" class that meets a data type or mode its kernel does not take hands the call to the
    host operator of the same name (TenniS itself falls back only for operators a device does not register):
    graphs that ran on "cpu" keep running on "hip", with the host's results bit for bit.  Strict device
    lookup, so it is the "hip" class that is created and delegates."""
    rng = np.random.default_rng(905)

    def same(op, params, inputs, out_bytes):
        cpu = ts.run_op("cpu", op, params, inputs, out_bytes)
        hip = ts.run_op("hip", op, params, inputs, out_bytes, strict=True)
        assert cpu.shape == hip.shape and cpu.dtype == hip.dtype, (op, cpu.dtype, hip.dtype)
        assert np.array_equal(cpu.view(np.uint8), hip.view(np.uint8)), op
        return cpu

    a = rng.integers(-1000, 1000, (2, 3, 5, 7)).astype(np.int32)
    b = rng.integers(-1000, 1000, (1, 3, 1, 1)).astype(np.int32)
    assert same("add", {}, [a, b], a.nbytes).dtype == np.int32
    assert same("mul", {}, [a, a], a.nbytes).dtype == np.int32
    d = rng.standard_normal((2, 3, 5, 7))
    assert same("add", {}, [d, d[::-1].copy()], d.nbytes).dtype == np.float64
    # interpolating resize (type 0 = LINEAR, 1 = CUBIC): the device kernel is nearest-neighbour only
    x = rng.standard_normal((2, 3, 9, 8)).astype(np.float32)
    size = np.array([-1, -1, 17, 13], np.int32)
    for kind in (0, 1, 2):
        out = same("_resize2d", {"type": np.array([kind], np.int32)}, [x, size], 4 * 2 * 3 * 17 * 13)
        assert out.shape == (2, 3, 17, 13)
    # fp64 convolution and inner product
    xd = rng.uniform(-1, 1, (2, 5, 9, 8))
    wd = rng.standard_normal((7, 5, 3, 3)) * 0.1
    out = same("conv2d", conv_params(ts, (1, 1, 1, 1)), [xd, wd], 8 * 2 * 7 * 9 * 8)
    assert out.dtype == np.float64 and out.shape == (2, 7, 9, 8)
    # (no fp64 inner_prod here: the reference's own leaves parts of its output unwritten on any device)
    bd = rng.standard_normal(7)
    assert same("add_bias", {"dim": np.array([1], np.int32)}, [out, bd], out.nbytes).dtype == np.float64
    # int8 concat (1-byte elements)
    q1 = rng.integers(-128, 128, (2, 3, 4, 5)).astype(np.int8)
    q2 = rng.integers(-128, 128, (2, 6, 4, 5)).astype(np.int8)
    assert same("concat", {"dim": np.array([1], np.int32)}, [q1, q2], 2 * 9 * 4 * 5).shape == (2, 9, 4, 5)
    # fp64 activations
    assert same("relu", {}, [d], d.nbytes).dtype == np.float64
    # a case neither side supports fails the same way on both: NHWC pooling (pooling2d_core.cpp:234)
    p = {"format": "NHWC", "type": np.array([0], np.int32),
         "padding": np.array([[0, 0], [0, 0], [0, 0], [0, 0]], np.int32), "padding_type": np.array([0], np.int32),
         "ksize": np.array([1, 2, 2, 1], np.int32), "stride": np.array([1, 2, 2, 1], np.int32)}
    xn = rng.standard_normal((1, 8, 8, 3)).astype(np.float32)
    errors = []
    for device in ("cpu", "hip"):
        with pytest.raises(RuntimeError) as e:
            ts.run_op(device, "pooling2d", p, [xn], xn.nbytes)
        errors.append(str(e.value).split("only support")[-1])
    assert errors[0] == errors[1] and "NCHW" in errors[0]


def test_zipper_option_resolves_the_bias_axis_like_add_bias(ts, tmp_path):
    """add_bias with format NCHW AND dim 3: AddBias::init lets dim override the format (base_add_bias.cpp:27-40), so
    the bias runs along W.  The rewrite must not take it for a channel bias: it folds quantize + convolution only
    and leaves the add_bias node in the graph; values as on TenniS's CPU device."""
    import sys, os
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    from make_modules import conv_params
    from tennis_amd import module_file as mf
    rng = np.random.default_rng(78)
    n, c, h, w, co = 2, 8, 6, 10, 10          # cout == w: a channel bias would have the same length
    wq = rng.integers(-127, 128, (co, c, 3, 3)).astype(np.int8)
    N = mf.Node
    nodes = [N(mf.PARAMETER, "x"), N("quantize", "q", {"quantize_scale": np.array([9.0, 11.0], np.float32)}, [0]),
             N(mf.CONST, "w", {"value": wq}),
             N("conv2d_quantized", "conv", dict(conv_params((1, 1, 1, 1)),
                                                dequantize_scales=rng.uniform(1e-4, 1e-3, co).astype(np.float32)), [1, 2]),
             N(mf.CONST, "b", {"value": rng.standard_normal(w).astype(np.float32)}),
             N("add_bias", "bias_w", {"format": "NCHW", "dim": np.array([3], np.int32)}, [3, 4]),
             N("relu", "act", {}, [5])]
    module = mf.Module(nodes, [0], [6])
    path = str(tmp_path / "bias_axis.tsm")
    mf.write_module(path, module)
    x = (rng.standard_normal((n, c, h, w)) * 6).astype(np.float32)
    cpu = ts.run_module("cpu", path, [x])
    fused0 = ts.fused_chain_count()
    hip = ts.run_module("hip", path, [x])
    assert ts.fused_chain_count() == fused0 + 1
    assert np.array_equal(bits(hip), bits(cpu))
    fused = mf.fuse_quantized_chains(module)
    assert [m.op for m in fused.nodes].count("add_bias") == 1
    (own,) = mf.run_module(fused, [x])
    assert np.array_equal(bits(own), bits(cpu))


def test_batch_norm_family_in_tennis_workbench(ts, host_delegate_watch):
    """batch_norm / batch_scale / fused_batch_norm created with strict device lookup, so the "hip" classes run:
    bitwise against TenniS's CPU operators; fp64 inputs go through the host delegate."""
    rng = np.random.default_rng(907)
    for shape, dim in (((2, 6, 7, 9), 1), ((3, 5, 4, 4), 1), ((4, 10), 1), ((2, 3, 5, 6), 3)):
        c = shape[dim]
        x = (rng.standard_normal(shape) * 3).astype(np.float32)
        mean, var = rng.standard_normal(c).astype(np.float32), rng.uniform(1e-3, 4, c).astype(np.float32)
        scale, bias = rng.standard_normal(c).astype(np.float32), rng.standard_normal(c).astype(np.float32)
        d = {"dim": np.array([dim], np.int32)}
        e = dict(d, epsilon=np.array([1e-3], np.float32))
        for op, params, inputs in (("batch_norm", e, [x, mean, var]), ("batch_norm", d, [x, mean, var]),
                                   ("batch_scale", d, [x, scale, bias]), ("fused_batch_norm", e, [x, mean, var, scale, bias])):
            cpu = ts.run_op("cpu", op, params, inputs, x.nbytes)
            hip = ts.run_op("hip", op, params, inputs, x.nbytes, strict=True)
            assert np.array_equal(bits(cpu), bits(hip)), (op, shape)
    xd = rng.standard_normal((2, 4, 3, 3))
    vd = rng.uniform(0.5, 2, 4)
    d = {"dim": np.array([1], np.int32)}
    cpu = ts.run_op("cpu", "batch_scale", d, [xd, vd, vd], xd.nbytes)
    host_delegate_watch["expected"] = 1        # fp64: the one run of this test the device hands to the host operator
    hip = ts.run_op("hip", "batch_scale", d, [xd, vd, vd], xd.nbytes, strict=True)
    assert hip.dtype == np.float64 and np.array_equal(cpu.view(np.uint8), hip.view(np.uint8))


def test_zipper_option_folds_residual_joins(ts, tmp_path):
    """add + relu behind a chain (a residual block's join, the other operand another chain's output), a darknet-style
    shortcut behind an activated chain, and an add whose other operand broadcasts: TenniS's compiler folds all three
    into conv2d_quantized_fused nodes, values as on its CPU device bit for bit."""
    import sys, os
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    from make_modules import conv_params
    from tennis_amd import module_file as mf
    rng = np.random.default_rng(79)
    n, c, h, w, co = 2, 16, 9, 11, 12
    N = mf.Node
    nodes = [N(mf.PARAMETER, "x")]

    def chain(name, src, k, pad, act=None):
        wq = rng.integers(-127, 128, (co, c, k, k)).astype(np.int8)
        nodes.append(N("quantize", name + ".q", {"quantize_scale": np.array([7.5, 12.0], np.float32)}, [src]))
        nodes.append(N(mf.CONST, name + ".w", {"value": wq}))
        nodes.append(N("conv2d_quantized", name, dict(conv_params((pad,) * 4),
                                                      dequantize_scales=rng.uniform(1e-4, 1e-3, co).astype(np.float32)),
                       [len(nodes) - 2, len(nodes) - 1]))
        nodes.append(N(mf.CONST, name + ".b", {"value": rng.standard_normal(co).astype(np.float32)}))
        nodes.append(N("add_bias", name + ".bias", {"format": "NCHW"}, [len(nodes) - 2, len(nodes) - 1]))
        if act:
            nodes.append(N(act, name + ".act", {"scale": np.array([0.1], np.float32)} if act == "leaky_relu" else {},
                           [len(nodes) - 1]))
        return len(nodes) - 1

    a = chain("main", 0, 3, 1)
    b = chain("proj", 0, 1, 0)
    nodes.append(N("add", "join", {}, [a, b]))
    nodes.append(N("relu", "join.relu", {}, [len(nodes) - 1]))
    join = len(nodes) - 1
    d = chain("dark", 0, 3, 1, "leaky_relu")
    nodes.append(N("add", "shortcut", {}, [join, d]))
    shortcut = len(nodes) - 1
    e = chain("scaled", 0, 1, 0)
    nodes.append(N(mf.CONST, "offsets", {"value": rng.standard_normal((1, co, 1, 1)).astype(np.float32)}))
    nodes.append(N("add", "offset", {}, [e, len(nodes) - 1]))
    nodes.append(N("concat", "out", {"dim": np.array([1], np.int32)}, [shortcut, len(nodes) - 1]))
    module = mf.Module(nodes, [0], [len(nodes) - 1])
    path = str(tmp_path / "residual_cases.tsm")
    mf.write_module(path, module)
    x = (rng.standard_normal((n, c, h, w)) * 6).astype(np.float32)
    cpu = ts.run_module("cpu", path, [x])
    fused0 = ts.fused_chain_count()
    hip = ts.run_module("hip", path, [x])
    assert ts.fused_chain_count() == fused0 + 4     # main (+ join), proj, dark (+ shortcut), scaled (+ offset)
    assert cpu.shape == (n, 2 * co, h, w)
    assert np.array_equal(bits(hip), bits(cpu))
    fused = mf.fuse_quantized_chains(module)
    assert "add" not in [m.op for m in fused.nodes]
    (own,) = mf.run_module(fused, [x])
    assert np.array_equal(bits(own), bits(cpu))


def test_zipper_option_residuals_that_broadcast_keep_running(ts, tmp_path):
    """An `add` the zipper folds into a fused node whose operands do not have one shape: (a) the convolution's
    [n, c, 1, 1] output added to an [n, c, h, w] tensor -- the convolution's result is the one that repeats -- and
    (b) a per-channel [1, c, 1, 1] operand, each followed by another quantized chain, so the fused node also has to
    hand its sum over as staged int8.  Both ran as separate operators before the rewrite and must keep running, with
    the host device's values bit for bit."""
    import sys, os
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    from make_modules import conv_params
    from tennis_amd import module_file as mf
    rng = np.random.default_rng(83)
    n, c, h, w, co = 2, 16, 7, 9, 16
    N = mf.Node
    nodes = [N(mf.PARAMETER, "x")]

    def chain(name, src, cin, kh, kw, pads, act=None):
        wq = rng.integers(-127, 128, (co, cin, kh, kw)).astype(np.int8)
        nodes.append(N("quantize", name + ".q", {"quantize_scale": np.array([7.5, 12.0], np.float32)}, [src]))
        nodes.append(N(mf.CONST, name + ".w", {"value": wq}))
        nodes.append(N("conv2d_quantized", name, dict(conv_params(pads),
                                                      dequantize_scales=rng.uniform(1e-4, 1e-3, co).astype(np.float32)),
                       [len(nodes) - 2, len(nodes) - 1]))
        nodes.append(N(mf.CONST, name + ".b", {"value": rng.standard_normal(co).astype(np.float32)}))
        nodes.append(N("add_bias", name + ".bias", {"format": "NCHW"}, [len(nodes) - 2, len(nodes) - 1]))
        if act:
            nodes.append(N(act, name + ".act", {}, [len(nodes) - 1]))
        return len(nodes) - 1

    g = chain("global", 0, c, h, w, (0, 0, 0, 0))                      # [n, co, 1, 1]
    nodes.append(N(mf.CONST, "map", {"value": rng.standard_normal((n, co, h, w)).astype(np.float32)}))
    nodes.append(N("add", "grown", {}, [g, len(nodes) - 1]))           # [n, co, h, w]
    nodes.append(N("relu", "grown.relu", {}, [len(nodes) - 1]))
    a = chain("behind_grown", len(nodes) - 1, co, 3, 3, (1, 1, 1, 1))
    e = chain("scaled", 0, c, 1, 1, (0, 0, 0, 0), "relu")
    nodes.append(N(mf.CONST, "offsets", {"value": rng.standard_normal((1, co, 1, 1)).astype(np.float32)}))
    nodes.append(N("add", "offset", {}, [e, len(nodes) - 1]))
    b = chain("behind_offset", len(nodes) - 1, co, 3, 3, (1, 1, 1, 1))
    nodes.append(N("concat", "out", {"dim": np.array([1], np.int32)}, [a, b]))
    module = mf.Module(nodes, [0], [len(nodes) - 1])
    path = str(tmp_path / "broadcast_residuals.tsm")
    mf.write_module(path, module)
    x = (rng.standard_normal((n, c, h, w)) * 6).astype(np.float32)
    cpu = ts.run_module("cpu", path, [x])
    fused0 = ts.fused_chain_count()
    hip = ts.run_module("hip", path, [x])
    assert ts.fused_chain_count() == fused0 + 4
    assert cpu.shape == (n, 2 * co, h, w)
    assert np.array_equal(bits(hip), bits(cpu))
