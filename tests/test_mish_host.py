"""The exact Mish arithmetic of the kernels (tennis_amd/csrc/tsx_mish.hpp) pinned on the CPU: the header is compiled
for the host as it stands and swept over the floats against the C library's chain -- the chain the reference's
operators evaluate (src/kernels/cpu/softplus.cpp:30-39, tanh.cpp:14-23, mul).  The bar is the one the device tests
hold the kernels to: expf, tanh and Mish bit for bit; softplus bit for bit but for at most one float of the sweep
(the whole range of 2.26e9 floats in (-200, 200) holds one float whose softplus lies within 2^-50 of a rounding
boundary and comes out one ulp apart; Mish of it is the host's all the same)."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

from _util import bits

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "tennis_amd", "csrc")


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    so = str(tmp_path_factory.mktemp("mish") / "mish_host_check.so")
    subprocess.run(["g++", "-O2", "-ffp-contract=off", "-fopenmp", "-mfma", "-shared", "-fPIC", "-I", CSRC,
                    os.path.join(HERE, "mish_host_check.cpp"), "-o", so], check=True)
    L = ctypes.CDLL(so)
    L.mish_sweep.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_float, ctypes.POINTER(ctypes.c_longlong)]
    L.mish_values.argtypes = [ctypes.c_void_p, ctypes.c_longlong] + [ctypes.c_void_p] * 4
    return L


@pytest.mark.parametrize("first,stride,limit", [(0, 61, 200.0), (17, 97, 200.0), (5, 4099, 3.4e38)])
def test_sweep_against_the_c_library(model, first, stride, limit):
    out = (ctypes.c_longlong * 5)()
    model.mish_sweep(first, stride, limit, out)
    checked, mish, softplus, tanh, expf = list(out)
    assert checked > 1_000_000
    assert (mish, tanh, expf) == (0, 0, 0) and softplus <= 1, (checked, mish, softplus, tanh, expf)


def test_limits_against_the_oracle(model, port):
    x = np.float32([0.0, -0.0, 1.0, -1.0, 17.0, -17.0, 30.0, -30.0, 88.0, 88.7, 88.8, 89.0, 100.0, -87.0, -88.0, -103.0,
                    -104.0, -150.0, -1000.0, 1000.0, 1e-30, -1e-30, 1e-45, np.inf, -np.inf, np.nan, 3.4e38, -3.4e38])
    outs = [np.empty_like(x) for _ in range(4)]
    model.mish_values(x.ctypes.data, x.size, *[o.ctypes.data for o in outs])
    with np.errstate(all="ignore"):
        exp = [port.mish(x), port.softplus(x), port.tanh(x)]
    for name, g, e in zip(("mish", "softplus", "tanh"), outs, exp):
        both_nan = np.isnan(g) & np.isnan(e)
        assert np.array_equal(bits(g)[~both_nan], bits(e)[~both_nan]), (name, g, e)
