#!/usr/bin/env python3
"""Writes tests/golden/hotpath_vectors.npz: inputs and the outputs the *compiled TenniS reference*
(oracle/_ref, built from the reference's own sources by oracle/ref.mk) gives for them.

    python tests/golden/make_golden.py          # needs oracle/_ref (make -C oracle ref)

The fixture is data only (seeded inputs + reference outputs); tests/test_golden.py checks the CPU
oracle and the HIP path against it, so parity stays anchored where the compiled reference is not
present.  One thread everywhere: the reference's dequant loop is only correct at one thread.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import ref  # noqa: E402


def main():
    if not ref.available():
        sys.exit("oracle/_ref is not built: run `make -C oracle ref` where the reference tree is present")
    rng = np.random.default_rng(20240607)
    v = {}

    # quantize (quantize.cpp:70-125): ties, NaN/inf, overflow; one scale (half-even bulk of 8, half-away
    # tail) and one scale per leading index (half-away everywhere)
    base = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, -127.5, -128.5, 300.0, -300.0, np.nan, np.inf,
                     -np.inf, 0.49999997, -0.49999997, 3.5, -3.5], np.float32)
    v["q1_x"] = base.reshape(1, 19)
    v["q1_s"] = np.array([1.0], np.float32)
    v["q1_y"] = ref.quantize(v["q1_x"], v["q1_s"])
    v["q2_x"] = np.concatenate([base, base[::-1] * np.float32(0.5), [7.5]]).astype(np.float32).reshape(3, 13)
    v["q2_s"] = np.array([1.0, 2.0, 0.5], np.float32)
    v["q2_y"] = ref.quantize(v["q2_x"], v["q2_s"])
    x = (rng.standard_normal((2, 3, 5, 7)) * 40).astype(np.float32)
    v["q3_x"], v["q3_s"] = x, np.array([1.7, 0.9], np.float32)
    v["q3_y"] = ref.quantize(x, v["q3_s"])

    # conv2d_quantized -> add_bias -> relu / leaky_relu (conv2d_quantized_core.cpp:18-147, add_bias.cpp,
    # relu.cpp, leaky_relu.cpp): 3x3 s1 p1, a strided/dilated asymmetric case, and the 1x1 bypass
    def qconv(tag, n, c, h, w, cout, k, pads, strides, dil, pv):
        xq = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
        wq = rng.integers(-127, 128, (cout, c, k, k)).astype(np.int8)
        dq = rng.uniform(1e-4, 1e-3, cout).astype(np.float32)
        bias = rng.standard_normal(cout).astype(np.float32)
        y = ref.conv2d_quantized(xq, wq, dq, pads, strides, dil, pv)
        yb = ref.add_bias(y, bias)
        v[tag + "_x"], v[tag + "_w"], v[tag + "_dq"], v[tag + "_b"] = xq, wq, dq, bias
        v[tag + "_geom"] = np.array(list(pads) + list(strides) + list(dil), np.int32)
        v[tag + "_pv"] = np.array([pv], np.float32)
        v[tag + "_y"], v[tag + "_yb"] = y, yb
        v[tag + "_relu"] = ref.relu(yb)
        v[tag + "_leaky"] = ref.leaky_relu(yb, 0.1)
        qs = np.full(n, 9.0, np.float32)
        v[tag + "_qs"] = qs
        v[tag + "_requant"] = ref.quantize(v[tag + "_relu"], qs)

    qconv("c3", 2, 70, 9, 10, 37, 3, (1, 1, 1, 1), (1, 1), (1, 1), 0.0)
    qconv("cs", 3, 5, 11, 9, 6, 3, (2, 0, 1, 2), (2, 1), (1, 2), 3.0)
    qconv("c1", 1, 19, 6, 5, 9, 1, (0, 0, 0, 0), (1, 1), (1, 1), 0.0)

    # fp32 conv2d (conv2d_core.cpp, math_cpu.cpp gemm incl. remainder paths) and inner_prod
    x = rng.uniform(-1, 1, (2, 5, 9, 11)).astype(np.float32)
    w = (rng.standard_normal((13, 5, 3, 3)) * 0.2).astype(np.float32)
    v["f_x"], v["f_w"] = x, w
    v["f_y"] = ref.conv2d(x, w, (1, 1, 1, 1))
    v["f_y_s2"] = ref.conv2d(x, w, (0, 1, 2, 0), (2, 2), (1, 1), 0.5)
    a = rng.standard_normal((5, 70)).astype(np.float32)
    b = rng.standard_normal((70, 33)).astype(np.float32)
    v["ip_a"], v["ip_b"] = a, b
    v["ip_y"] = ref.inner_prod(a, b, False)
    v["ip_yt"] = ref.inner_prod(a, np.ascontiguousarray(b.T), True)

    # Winograd F(6,3) (winograd_algorithm.cpp:504-947): sizes that are not multiples of the 6x6 tile
    x = rng.uniform(-1, 1, (2, 5, 13, 10)).astype(np.float32)
    w = (rng.standard_normal((7, 5, 3, 3)) * 0.2).astype(np.float32)
    v["wg_x"], v["wg_w"] = x, w
    v["wg_y"] = ref.winograd(x, w, (1, 1, 1, 1), True, 0.0)
    v["wg_y_pv"] = ref.winograd(x, w, (1, 1, 1, 1), True, 0.25)
    # ... and F(2,3) (:57-459) on the same input
    v["wg23_y"] = ref.winograd(x, w, (1, 1, 1, 1), False, 0.0)
    v["wg23_y_pv"] = ref.winograd(x, w, (1, 1, 1, 1), False, 0.25)

    # int8 GEMM (math_cpu.cpp:143-244)
    a8 = rng.integers(-128, 128, (7, 45)).astype(np.int8)
    b8 = rng.integers(-128, 128, (45, 19)).astype(np.int8)
    v["g8_a"], v["g8_b"] = a8, b8
    v["g8_c"] = ref.gemm_i8(a8, b8)

    out = os.path.join(HERE, "hotpath_vectors.npz")
    np.savez_compressed(out, **v)
    print("wrote", out, os.path.getsize(out), "bytes,", len(v), "arrays")


if __name__ == "__main__":
    main()
