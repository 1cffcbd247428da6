"""Glue operators between convolutions (residual add, pooling2d, global_pooling2d).

CPU part: the oracle against the compiled reference operators (bitwise) and against numpy closed
forms.  GPU part (marked gpu): the HIP kernels through the C ABI against the oracle, bitwise
(max is exact; the average keeps the reference's sequential fp32 summation order).
"""
import numpy as np
import pytest

from _util import bits

POOL_CASES = [
    # ksize, strides, pads (top, bottom, left, right), white
    ((3, 3), (2, 2), (1, 1, 1, 1), False),     # ceil mode: 13x14 -> 7x8
    ((3, 3), (2, 2), (0, 1, 0, 1), False),     # the ResNet stem pool as used by the network runner
    ((2, 2), (2, 2), (0, 0, 0, 0), False),
    ((3, 2), (1, 2), (1, 0, 1, 0), True),
    ((5, 5), (1, 1), (2, 2, 2, 2), False),     # SPP-style same-size pooling
    ((3, 3), (2, 2), (0, 0, 0, 0), True),
]


def _x(seed=7, shape=(2, 5, 13, 14)):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


@pytest.mark.parametrize("kind", ["max", "avg"])
@pytest.mark.parametrize("case", POOL_CASES)
def test_oracle_pooling_vs_reference(port, ref, kind, case):
    k, s, p, white = case
    x = _x()
    a, b = port.pooling2d(x, kind, k, s, p, white), ref.pooling2d(x, kind, k, s, p, white)
    assert a.shape == b.shape and np.array_equal(bits(a), bits(b))


def test_oracle_global_pooling_and_add_vs_reference(port, ref):
    x, y = _x(), _x(8)
    for kind in ("max", "avg"):
        a = port.global_pooling2d(x, kind)
        assert np.array_equal(bits(a), bits(ref.global_pooling2d(x, kind).reshape(a.shape)))
    assert np.array_equal(bits(port.add(x, y)), bits(ref.add(x, y)))


def test_oracle_pooling_closed_forms(port):
    """Reference-independent: max over the clipped window; mean over valid elements (BLACK) with a
    fp64 bound; a constant map averages to the constant under BLACK and to const*valid/k^2 under WHITE."""
    x = _x(9, (1, 2, 9, 9))
    got = port.pooling2d(x, "max", (3, 3), (2, 2), (1, 1, 1, 1))
    assert got.shape == (1, 2, 5, 5)
    for oh in range(5):
        for ow in range(5):
            win = x[:, :, max(2 * oh - 1, 0):min(2 * oh + 2, 9), max(2 * ow - 1, 0):min(2 * ow + 2, 9)]
            assert np.array_equal(got[:, :, oh, ow], win.max(axis=(2, 3)))
    avg = port.pooling2d(x, "avg", (3, 3), (2, 2), (1, 1, 1, 1))
    win = x[:, :, 0:2, 0:2].astype(np.float64).mean(axis=(2, 3))
    assert np.allclose(avg[:, :, 0, 0], win, rtol=1e-6, atol=1e-7)
    ones = np.full((1, 1, 4, 4), 3.0, np.float32)
    assert np.array_equal(port.pooling2d(ones, "avg", (3, 3), (2, 2), (1, 1, 1, 1)), np.full((1, 1, 3, 3), 3.0, np.float32))
    white = port.pooling2d(ones, "avg", (3, 3), (2, 2), (1, 1, 1, 1), white=True)
    assert white[0, 0, 0, 0] == np.float32(12.0) / np.float32(9.0) and white[0, 0, 1, 1] == np.float32(3.0)
    assert np.array_equal(port.global_pooling2d(ones, "avg"), np.full((1, 1, 1, 1), 3.0, np.float32))


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
@pytest.mark.parametrize("kind", ["max", "avg"])
@pytest.mark.parametrize("case", POOL_CASES)
def test_hip_pooling2d(tsx, port, kind, case):
    k, s, p, white = case
    for shape in ((2, 5, 13, 14), (3, 70, 28, 28)):
        x = _x(11, shape)
        got = tsx.pooling2d(_dev(x), kind, k, s, p, white).cpu().numpy()
        exp = port.pooling2d(x, kind, k, s, p, white)
        assert got.shape == exp.shape and np.array_equal(bits(got), bits(exp))


@pytest.mark.gpu
def test_hip_global_pooling_resnet_tail(tsx, port):
    x = np.maximum(_x(12, (4, 2048, 7, 7)), 0)
    for kind in ("avg", "max"):
        got = tsx.global_pooling2d(_dev(x), kind).cpu().numpy()
        assert np.array_equal(bits(got), bits(port.global_pooling2d(x, kind)))


@pytest.mark.gpu
@pytest.mark.parametrize("act", [None, "relu", "leaky_relu"])
def test_hip_add_with_activation(tsx, port, act):
    for count_shape in ((2, 3, 5, 7), (1, 3, 3, 3), (4, 64, 28, 28)):
        a, b = _x(13, count_shape), _x(14, count_shape)
        a.ravel()[::7] = -b.ravel()[::7]          # exact zeros of both signs in the sum
        a.ravel()[-1], b.ravel()[-1] = -0.0, -0.0   # -0 in the activation's scalar tail
        got = tsx.add(_dev(a), _dev(b), act, 0.1).cpu().numpy()
        exp = port.add(a, b)
        if act == "relu":
            exp = port.relu(exp)
        elif act == "leaky_relu":
            exp = port.leaky_relu(exp, 0.1)
        assert np.array_equal(bits(got), bits(exp))


@pytest.mark.gpu
def test_hip_pooling_rejects_bad_arguments(tsx):
    import torch
    x = torch.zeros((1, 1, 4, 4), device="cuda")
    out = torch.zeros((1, 1, 9, 9), device="cuda")
    rc = tsx.lib().tsx_pooling2d_f32(x.data_ptr(), 1, 4, 4, 0, 0, 0, 3, 3, 2, 2, 0, out.data_ptr(), 9, 9, None)
    assert rc < 0 and b"outside" in tsx.lib().tsx_last_error()
    rc = tsx.lib().tsx_pooling2d_f32(x.data_ptr(), 1, 4, 4, 2, 0, 0, 3, 3, 2, 2, 0, out.data_ptr(), 2, 2, None)
    assert rc < 0


# ---------------------------------------------------------------- batch_norm / batch_scale / fused_batch_norm

@pytest.mark.parametrize("shape,dim", [((2, 5, 7, 9), 1), ((3, 6, 4, 4), 1), ((2, 3, 1, 1), 1), ((4, 10), 1), ((2, 3, 5, 6), 3),
                                       ((1, 8, 13, 3), 2), ((6,), 0)])
def test_batch_norm_family_against_the_compiled_reference(port, ref, shape, dim):
    """Bitwise against cpu::BatchNorm / BatchScale / FusedBatchNorm, on inner extents that are and are not
    multiples of their 4-wide body (body and tail contract x * scale + bias to one fma alike), with variances whose
    reciprocal root differs between float and double evaluation (the reference's is the double one)."""
    rng = np.random.default_rng(700 + len(shape) + dim)
    c = shape[dim]
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    mean, var = rng.standard_normal(c).astype(np.float32), rng.uniform(1e-3, 4, c).astype(np.float32)
    scale, bias = rng.standard_normal(c).astype(np.float32), rng.standard_normal(c).astype(np.float32)
    d = {"dim": np.array([dim], np.int32)}
    for eps in (1e-5, 1e-3):
        e = dict(d, epsilon=np.array([eps], np.float32))
        assert np.array_equal(bits(port.batch_norm(x, mean, var, eps, dim)), bits(ref.run_op("batch_norm", e, [x, mean, var], x.nbytes)))
        assert np.array_equal(bits(port.fused_batch_norm(x, mean, var, scale, bias, eps, dim)),
                              bits(ref.run_op("fused_batch_norm", e, [x, mean, var, scale, bias], x.nbytes)))
    assert np.array_equal(bits(port.batch_scale(x, scale, bias, dim)), bits(ref.run_op("batch_scale", d, [x, scale, bias], x.nbytes)))
    # the default epsilon (include/backend/base/base_batch_norm.h:33)
    assert np.array_equal(bits(port.batch_norm(x, mean, var, 1e-5, dim)), bits(ref.run_op("batch_norm", d, [x, mean, var], x.nbytes)))


def test_batch_norm_family_closed_forms(port):
    """Without the reference: the definitions in float64 bound the fp32 results, batch_scale is exactly one fused
    multiply-add per element, and fused_batch_norm is batch_scale applied to batch_norm."""
    rng = np.random.default_rng(710)
    x = (rng.standard_normal((3, 7, 5, 6)) * 2).astype(np.float32)
    mean, var = rng.standard_normal(7).astype(np.float32), rng.uniform(0.05, 3, 7).astype(np.float32)
    scale, bias = rng.standard_normal(7).astype(np.float32), rng.standard_normal(7).astype(np.float32)
    sh = (1, 7, 1, 1)
    bn = port.batch_norm(x, mean, var, 1e-3)
    exact = (x.astype(np.float64) - mean.reshape(sh)) / np.sqrt(var.reshape(sh).astype(np.float64) + np.float32(1e-3))
    assert np.abs(bn - exact).max() <= 4e-7 * np.abs(exact).max()
    bs = port.batch_scale(x, scale, bias)
    fma = (x.astype(np.float64) * scale.reshape(sh).astype(np.float64) + bias.reshape(sh).astype(np.float64)).astype(np.float32)
    assert np.count_nonzero(bits(bs) != bits(fma)) <= 2      # float64 evaluation rounds twice in rare ties
    assert np.array_equal(bits(port.fused_batch_norm(x, mean, var, scale, bias, 1e-3)), bits(port.batch_scale(bn, scale, bias)))
    assert np.array_equal(bits(port.batch_norm(x, np.zeros(7, np.float32), np.ones(7, np.float32), 0.0)), bits(x))


@pytest.mark.gpu
@pytest.mark.parametrize("shape,dim", [((2, 5, 7, 9), 1), ((3, 6, 4, 4), 1), ((2, 3, 1, 1), 1), ((4, 10), 1), ((2, 3, 5, 6), 3),
                                       ((32, 64, 56, 56), 1), ((3, 1000), 1)])
def test_hip_batch_norm_family(tsx, port, shape, dim):
    """tsx_batch_norm_f32 / tsx_batch_scale_f32 / tsx_fused_batch_norm_f32 through the C ABI: bit-exact against the
    oracle (which is bit-exact against the compiled reference), inner extents with and without whole 4-element
    groups, an unaligned view of the input."""
    rng = np.random.default_rng(720 + len(shape) + dim)
    c = shape[dim]
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    mean, var = rng.standard_normal(c).astype(np.float32), rng.uniform(1e-3, 4, c).astype(np.float32)
    scale, bias = rng.standard_normal(c).astype(np.float32), rng.standard_normal(c).astype(np.float32)
    xd, md, vd, sd, bd = (_dev(a) for a in (x, mean, var, scale, bias))
    for eps in (1e-5, 1e-3):
        assert np.array_equal(bits(tsx.batch_norm(xd, md, vd, eps, dim).cpu().numpy()), bits(port.batch_norm(x, mean, var, eps, dim)))
        assert np.array_equal(bits(tsx.fused_batch_norm(xd, md, vd, sd, bd, eps, dim).cpu().numpy()),
                              bits(port.fused_batch_norm(x, mean, var, scale, bias, eps, dim)))
    assert np.array_equal(bits(tsx.batch_scale(xd, sd, bd, dim).cpu().numpy()), bits(port.batch_scale(x, scale, bias, dim)))


@pytest.mark.gpu
def test_hip_batch_norm_rejects_bad_arguments(tsx):
    import torch
    x = torch.zeros((2, 3, 4), device="cuda")
    v = torch.ones(3, device="cuda")
    L = tsx.lib()
    assert L.tsx_batch_norm_f32(tsx._ptr(x), 2, 0, 4, tsx._ptr(v), tsx._ptr(v), 1e-5, tsx._ptr(x), None) == -1
    assert L.tsx_batch_scale_f32(tsx._ptr(x), 2, 3, 4, None, tsx._ptr(v), tsx._ptr(x), None) == -1
    assert b"batch_scale" in L.tsx_last_error()
