"""Seeded synthetic inputs shared by the parity tests (and mirrored by bench.py)."""
import numpy as np


def quantize_weights_per_channel(w):
    """Offline per-output-channel symmetric int8 weights: s_c = 127/max|w_c|, round half away."""
    flat = np.abs(w.reshape(w.shape[0], -1)).max(axis=1).astype(np.float32)
    s = (np.float32(127.0) / np.maximum(flat, np.float32(1e-30))).astype(np.float32)
    q = w * s.reshape((-1,) + (1,) * (w.ndim - 1))
    q = np.clip(np.sign(q) * np.floor(np.abs(q) + 0.5), -127, 127).astype(np.int8)
    return q, s


def c2_like(rng, n, c, h, w, cout, k=3):
    """BASELINE config 2 shaped inputs: x ~ N(0,1), w ~ N(0,0.05), per-tensor activation scale."""
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, c, k, k)) * 0.05).astype(np.float32)
    bias = (rng.standard_normal(cout) * 0.1).astype(np.float32)
    s_x = np.float32(127.0) / np.abs(x).max().astype(np.float32)
    x_scales = np.full(n, s_x, np.float32)          # len == batch, as base::Quantize requires
    wq, s_w = quantize_weights_per_channel(wt)
    dq = (np.float32(1.0) / (s_x * s_w)).astype(np.float32)
    return x, x_scales, wq, dq, bias


def bits(a):
    return np.ascontiguousarray(a).view(np.int32)
