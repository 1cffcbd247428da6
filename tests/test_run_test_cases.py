"""TenniS `.t` tensor files and run_test-style operator case directories (tools/run_test/test_case.hpp).

The fixtures under tests/golden/cases were written by the reference's own serializer and hold the
reference CPU operators' outputs (tests/golden/make_cases.py)."""
import glob
import io
import os

import numpy as np
import pytest

from tennis_amd import run_test, tensor_file

CASES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cases")
ALL_T = sorted(glob.glob(os.path.join(CASES, "**", "*.t"), recursive=True))


def test_reader_decodes_the_reference_serializers_files():
    rd = lambda n: tensor_file.read_tensor(os.path.join(CASES, "sample.%s.t" % n), with_dtype=True)
    code, v = rd("int8")
    assert code == tensor_file.INT8 and v.dtype == np.int8 and v.shape == (3, 4) and v.any()
    code, v = rd("uint8")
    assert code == tensor_file.UINT8 and v.dtype == np.uint8 and v.shape == (5,)
    code, v = rd("int32")
    assert code == tensor_file.INT32 and v.dtype == np.int32 and v.shape == (2, 1, 3)
    code, v = rd("float32")
    assert code == tensor_file.FLOAT32 and v.dtype == np.float32 and v.shape == (2, 3, 4) and np.isfinite(v).all()
    code, v = rd("float64")
    assert code == tensor_file.FLOAT64 and v.dtype == np.float64 and v.shape == (4, 2)
    code, v = rd("bool")
    assert code == tensor_file.BOOLEAN and v.dtype == np.bool_ and v.tolist() == [True, False, True]
    code, v = rd("string")
    assert code == tensor_file.CHAR8 and v == "NCHW"


def test_known_bytes():
    """The layout spelled out: fields, dtype, ndims, sizes, data (src/core/tensor.cpp:314-389)."""
    raw = bytes([1, 0, 0, 0, 5, 2, 0, 0, 0, 1, 0, 0, 0, 2, 0, 0, 0, 0xFF, 0xFF, 0xFF, 0xFF, 7, 0, 0, 0])
    (code, arr), = tensor_file.parse_fields(raw)
    assert code == tensor_file.INT32 and arr.tolist() == [[-1, 7]]
    assert tensor_file.serialize(np.array([[-1, 7]], np.int32)) == raw
    scalar = bytes([1, 0, 0, 0, 10, 0, 0, 0, 0, 0, 0, 0x60, 0x40])      # FLOAT32, no sizes, one element: 3.5
    (code, arr), = tensor_file.parse_fields(scalar)
    assert code == tensor_file.FLOAT32 and arr.shape == () and float(arr) == 3.5
    assert tensor_file.serialize(np.float32(3.5)) == scalar


@pytest.mark.parametrize("path", ALL_T, ids=[os.path.relpath(p, CASES) for p in ALL_T])
def test_writer_reproduces_the_reference_serializers_bytes(path):
    with open(path, "rb") as fh:
        raw = fh.read()
    assert tensor_file.serialize(tensor_file.read_tensor(path)) == raw


def test_packed_and_broken_files(tmp_path):
    p = tmp_path / "packed.t"
    tensor_file.write_tensor(p, [np.arange(3, dtype=np.int32), "ab"])
    a, b = tensor_file.read_tensor(p)
    assert a.tolist() == [0, 1, 2] and b == "ab"
    raw = tensor_file.serialize(np.zeros((2, 2), np.float32))
    with pytest.raises(tensor_file.TensorFileError, match="truncated"):
        tensor_file.parse_fields(raw[:-1])
    with pytest.raises(tensor_file.TensorFileError, match="behind"):
        tensor_file.parse_fields(raw + b"\0")
    with pytest.raises(tensor_file.TensorFileError, match="dtype code"):
        tensor_file.parse_fields(bytes([1, 0, 0, 0, 12, 0, 0, 0, 0]))   # PTR has no portable element


def test_case_loader():
    tc = run_test.TestCase.load(os.path.join(CASES, "conv2d_quantized", "3x3_pad1"))
    assert tc.op == "conv2d_quantized" and tc.input_count == 2 and tc.output_count == 1
    assert set(tc.param) == {"format", "padding", "padding_value", "stride", "dilation", "dequantize_scales"}
    assert tc.param["format"][1] == "NCHW" and tc.input[0][1].dtype == np.int8
    assert tc.output[0][0] == tensor_file.FLOAT32 and tc.output[0][1].shape == (2, 12, 7, 7)
    assert run_test.TestCase.load(CASES) is None            # sample files only: not a case
    found = [d for d in run_test.find_cases(CASES) if run_test.TestCase.load(os.path.join(CASES, d))]
    assert len(found) == 34


def test_broken_cases_are_reported(tmp_path):
    src = os.path.join(CASES, "relu", "4d")
    for name in os.listdir(src):
        if not name.startswith("2."):
            (tmp_path / name).write_bytes(open(os.path.join(src, name), "rb").read())
    with pytest.raises(run_test.CaseError, match="Input count mismatch"):
        run_test.TestCase.load(str(tmp_path))
    (tmp_path / "0.relu.txt").write_text("zero one\n")
    with pytest.raises(run_test.CaseError, match="format error"):
        run_test.TestCase.load(str(tmp_path))


def test_unregistered_operator_is_skipped():
    """Host-only: the registry lookup needs no device (test_case.hpp:441-443 reports SKIP the same way)."""
    tc = run_test.TestCase.load(os.path.join(CASES, "softmax", "not_on_device"))
    assert tc.run("hip") == run_test.SKIP and "Not supported operator" in tc.log[0]


@pytest.fixture(scope="module")
def hip_device():
    """torch initialises its HIP runtime before the operator library loads its own, as in the other GPU tests."""
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return "hip"


@pytest.mark.gpu
def test_reference_cases_pass_on_hip(hip_device):
    out = io.StringIO()
    results = run_test.run_tree(CASES, "hip", 0, out=out)
    text = out.getvalue()
    assert not results[run_test.FAILED] and not results[run_test.WARNING], text
    assert results[run_test.SKIP] == [os.path.join("softmax", "not_on_device")], text
    assert len(results[run_test.OK]) == 33, text
    assert "[OK]: 33, [SKIP]: 1, [WARNING]: 0, [FAILED]: 0" in text


@pytest.mark.gpu
def test_integer_and_bit_exact_cases_match_exactly(hip_device):
    """The runner's tolerance is the reference's; the operators that are exact by construction are held to 0."""
    from tennis_amd import operators
    for sub in ("quantize/per_image", "quantize/single_scale", "conv2d_quantized/3x3_pad1", "conv2d_quantized/1x1_s2",
                "relu/4d", "add_bias/nchw", "add/broadcast", "pooling2d/max_3x3_s2", "conv2d_winograd/auto_mode",
                "conv2d_winograd_v2/auto_mode", "pooling2d_v2/avg_3x2", "concat/channels", "concat/last_axis",
                "_resize2d/nearest_up", "_resize2d/nearest_odd", "mul/broadcast", "mul/same_shape", "batch_norm/nchw",
                "batch_scale/nchw", "fused_batch_norm/nchw"):
        tc = run_test.TestCase.load(os.path.join(CASES, *sub.split("/")))
        got = operators.run_op(tc.op, {k: v for k, (_, v) in tc.param.items()}, [tc.input[i][1] for i in range(tc.input_count)])
        want = tc.output[0][1]
        assert got.dtype == want.dtype and np.array_equal(got, want), sub


@pytest.mark.gpu
def test_wrong_expected_output_fails(tmp_path, hip_device):
    src = os.path.join(CASES, "relu", "4d")
    for name in os.listdir(src):
        (tmp_path / name).write_bytes(open(os.path.join(src, name), "rb").read())
    want = tensor_file.read_tensor(str(tmp_path / "3.output_0.t"))
    want = want.copy()
    want[0, 0, 0, 0] += 0.5
    tensor_file.write_tensor(str(tmp_path / "3.output_0.t"), want)
    tc = run_test.TestCase.load(str(tmp_path))
    assert tc.run("hip") == run_test.FAILED and "[FAILED] Diff output 0" in tc.log[-1]
    tensor_file.write_tensor(str(tmp_path / "3.output_0.t"), want[:, :, :, :4].copy())
    tc = run_test.TestCase.load(str(tmp_path))
    assert tc.run("hip") == run_test.FAILED and tc.log[-1].startswith("Infer:")


def test_reference_reader_accepts_this_writers_files(ref, tmp_path):
    """The compiled reference's own tensor::load reads what write_tensor wrote (where oracle/_ref is built)."""
    rng = np.random.default_rng(7)
    for i, v in enumerate((rng.standard_normal((2, 3, 4)).astype(np.float32), rng.integers(-128, 128, (5, 2)).astype(np.int8),
                           rng.integers(-9, 9, (4,)).astype(np.int32), rng.standard_normal((3,)))):
        path = str(tmp_path / ("w%d.t" % i))
        tensor_file.write_tensor(path, v)
        code, back = ref.load_tensor(path)
        assert code == tensor_file._NP2TS[v.dtype] and back.dtype == v.dtype and np.array_equal(back, v)
        ref.save_tensor(path + ".ref", v)
        assert open(path, "rb").read() == open(path + ".ref", "rb").read()
