"""The allocation-free entry point tsx_quantize_conv2d_i8_nchw_noalloc against the entry point it is a
variant of (tsx_quantize_conv2d_i8_nchw with a caller workspace), through the C ABI.

Bar: bit-exact (same kernels; only the staging workspace differs).  Two calls in a row on the same GPU,
the second with a smaller input: the built-in scratch keeps the first call's bytes, and the second
result must not depend on them.  A layer too large for the scratch is rejected, not truncated.
"""
import ctypes

import numpy as np
import pytest

from _util import bits, c2_like

pytestmark = pytest.mark.gpu


def _run_both(tsx, torch, rng, n, c, h, w, cout, k, pads, act):
    L = tsx.lib()
    x, x_scales, wq, dq, bias = c2_like(rng, n, c, h, w, cout, k)
    dev = torch.device("cuda:0")
    xd = torch.from_numpy(x).to(dev)
    xsd = torch.from_numpy(x_scales).to(dev)
    conv = tsx.Conv2dI8(torch.from_numpy(wq).to(dev), pads)
    geom, packed, ws_bytes = conv._plan(tuple(x.shape))
    assert ws_bytes <= L.tsx_noalloc_scratch_bytes()
    ho, wo = tsx.conv_out_size(geom)
    ep = tsx._EpilogueArgs(torch.from_numpy(dq).to(dev), torch.from_numpy(bias).to(dev), act)
    ref_out = torch.empty((n, cout, ho, wo), dtype=torch.float32, device=dev)
    ref_acc = torch.empty((n, cout, ho, wo), dtype=torch.int32, device=dev)
    workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    stream = tsx._stream()
    tsx.check(L.tsx_quantize_conv2d_i8_nchw(ctypes.byref(geom), tsx._ptr(xd), tsx._ptr(xsd), n, tsx._ptr(packed), 0.0,
                                            ctypes.byref(ep.c), tsx._ptr(ref_out), None, tsx._ptr(ref_acc),
                                            tsx._ptr(workspace), ws_bytes, stream))
    got_out = torch.full((n, cout, ho, wo), float("nan"), dtype=torch.float32, device=dev)
    got_acc = torch.full((n, cout, ho, wo), -1, dtype=torch.int32, device=dev)
    tsx.check(L.tsx_quantize_conv2d_i8_nchw_noalloc(ctypes.byref(geom), tsx._ptr(xd), tsx._ptr(xsd), n, tsx._ptr(packed),
                                                    0.0, ctypes.byref(ep.c), tsx._ptr(got_out), None, tsx._ptr(got_acc),
                                                    stream))
    torch.cuda.synchronize()
    assert np.array_equal(got_acc.cpu().numpy(), ref_acc.cpu().numpy())
    assert np.array_equal(bits(got_out.cpu().numpy()), bits(ref_out.cpu().numpy()))


def test_noalloc_matches_workspace_entry_point_twice():
    import torch
    assert torch.cuda.is_available(), "this test needs the MI355X"
    from tennis_amd import capi as tsx
    tsx.lib()
    rng = np.random.default_rng(2024)
    print("noalloc call 1: 4x96x28x28 -> 128, 3x3 p1", flush=True)
    _run_both(tsx, torch, rng, 4, 96, 28, 28, 128, 3, (1, 1, 1, 1), "relu")
    print("noalloc call 2 (smaller): 2x40x9x11 -> 48, 3x3 p1", flush=True)
    _run_both(tsx, torch, rng, 2, 40, 9, 11, 48, 3, (1, 1, 1, 1), "relu")


def test_noalloc_rejects_layers_beyond_the_scratch():
    import torch
    assert torch.cuda.is_available(), "this test needs the MI355X"
    from tennis_amd import capi as tsx
    L = tsx.lib()
    # 64x256x30x30 staged bytes = 14.7 MB > 8 MiB: no launch, a clear error
    geom = tsx.make_geom((64, 256, 28, 28), (256, 256, 3, 3), (1, 1, 1, 1))
    assert L.tsx_conv2d_i8_workspace_bytes(ctypes.byref(geom)) > L.tsx_noalloc_scratch_bytes()
    one = torch.zeros(16, dtype=torch.float32, device="cuda:0")
    ep = tsx._EpilogueArgs(one)
    rc = L.tsx_quantize_conv2d_i8_nchw_noalloc(ctypes.byref(geom), tsx._ptr(one), tsx._ptr(one), 64, tsx._ptr(one), 0.0,
                                               ctypes.byref(ep.c), tsx._ptr(one), None, None, tsx._stream())
    assert rc == -2
    assert b"scratch" in L.tsx_last_error()
