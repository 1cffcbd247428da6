"""A YOLOv4-shaped int8 network (CSPDarknet53 backbone with Mish, SPP 5/9/13, PANet neck with LeakyReLU 0.1,
route/concat, 2x nearest upsample, three linear heads) on the MI355X convolution path.

The network is a darknet-style layer list (`layers()`), pure data, so that the device runner here and a
CPU checker interpret the same description.  Every convolution is the TenniS operator chain
    quantize(x, s) -> conv2d_quantized(w_q, dq) -> add_bias -> activation
with per-output-channel int8 weights (BN folded: conv + bias) and a per-tensor activation scale calibrated
on a batch; shortcut = add, route = concat on channels, maxpool = pooling2d MAX stride 1 with k//2 padding,
upsample = resize2d NEAREST.  Mish is the composition softplus -> tanh -> mul.
"""
import numpy as np
import torch

from . import capi
from .resnet50 import quantize_weights


def layers(width=1.0, classes=80):
    """Darknet-style list of dicts.  conv: (filters, size, stride, act); route: layers (negative = relative);
    shortcut: from; maxpool: size; upsample.  Returns (list, indices of the three head outputs)."""
    ch = lambda c: max(8, int(c * width))
    L = []

    def conv(f, k, s=1, act="mish"):
        L.append({"type": "conv", "filters": f, "size": k, "stride": s, "act": act})

    def csp(f, blocks, first=False):
        """downsample to f channels, then a cross-stage-partial group of `blocks` residual units."""
        half = f if first else f // 2
        conv(f, 3, 2)
        conv(half, 1)                                   # partial A
        L.append({"type": "route", "layers": [-2]})
        conv(half, 1)                                   # partial B
        for _ in range(blocks):
            conv(half // 2 if first else half, 1)
            conv(half, 3)
            L.append({"type": "shortcut", "from": -3})
        conv(half, 1)
        L.append({"type": "route", "layers": [-1, -(3 * blocks + 4)]})
        conv(f, 1)

    conv(ch(32), 3)
    csp(ch(64), 1, first=True)
    csp(ch(128), 2)
    csp(ch(256), 8)
    c3 = len(L) - 1
    csp(ch(512), 8)
    c4 = len(L) - 1
    csp(ch(1024), 4)
    lk = "leaky_relu"
    conv(ch(512), 1, act=lk)
    conv(ch(1024), 3, act=lk)
    conv(ch(512), 1, act=lk)
    L.append({"type": "maxpool", "size": 5})
    L.append({"type": "route", "layers": [-2]})
    L.append({"type": "maxpool", "size": 9})
    L.append({"type": "route", "layers": [-4]})
    L.append({"type": "maxpool", "size": 13})
    L.append({"type": "route", "layers": [-1, -3, -5, -6]})
    conv(ch(512), 1, act=lk)
    conv(ch(1024), 3, act=lk)
    conv(ch(512), 1, act=lk)
    p5 = len(L) - 1

    def up_merge(f, lateral):
        conv(f, 1, act=lk)
        L.append({"type": "upsample"})
        L.append({"type": "route", "layers": [lateral]})
        conv(f, 1, act=lk)
        L.append({"type": "route", "layers": [-1, -3]})
        for i in range(5):
            conv(f if i % 2 == 0 else 2 * f, 1 if i % 2 == 0 else 3, act=lk)

    up_merge(ch(256), c4)
    p4 = len(L) - 1
    up_merge(ch(128), c3)
    p3 = len(L) - 1
    heads = []
    out_ch = 3 * (classes + 5)

    def head(f):
        conv(f, 3, act=lk)
        conv(out_ch, 1, act=None)
        heads.append(len(L) - 1)

    def down_merge(f, src, lateral):
        L.append({"type": "route", "layers": [src]})
        conv(f, 3, 2, act=lk)
        L.append({"type": "route", "layers": [-1, lateral]})
        for i in range(5):
            conv(f if i % 2 == 0 else 2 * f, 1 if i % 2 == 0 else 3, act=lk)

    head(ch(256))
    down_merge(ch(256), p3, p4)
    n4 = len(L) - 1
    head(ch(512))
    down_merge(ch(512), n4, p5)
    head(ch(1024))
    return L, heads


def resolve(L):
    """Absolute source indices and channel counts of every layer (input = index -1 with 3 channels)."""
    chans, srcs = [], []
    for i, l in enumerate(L):
        ab = lambda r: r if r >= 0 else i + r
        cin = lambda j: 3 if j < 0 else chans[j]
        if l["type"] == "conv":
            srcs.append([i - 1])
            chans.append(l["filters"])
        elif l["type"] == "route":
            s = [ab(r) for r in l["layers"]]
            srcs.append(s)
            chans.append(sum(cin(j) for j in s))
        elif l["type"] == "shortcut":
            srcs.append([i - 1, ab(l["from"])])
            chans.append(cin(i - 1))
        else:
            srcs.append([i - 1])
            chans.append(cin(i - 1))
    return srcs, chans


def make_parameters(L, seed=0):
    rng = np.random.default_rng(seed)
    srcs, chans = resolve(L)
    params = {}
    for i, l in enumerate(L):
        if l["type"] != "conv":
            continue
        cin = 3 if srcs[i][0] < 0 else chans[srcs[i][0]]
        k = l["size"]
        w = (rng.standard_normal((l["filters"], cin, k, k)) * np.sqrt(2.0 / (cin * k * k))).astype(np.float32)
        wq, sw = quantize_weights(w)
        params[i] = {"wq": wq, "sw": sw, "bias": (rng.standard_normal(l["filters"]) * 0.05).astype(np.float32)}
    return params


def total_macs(L, batch, size):
    srcs, chans = resolve(L)
    hw, macs = [], 0
    for i, l in enumerate(L):
        src = srcs[i][0]
        h = size if src < 0 else hw[src]
        if l["type"] == "conv":
            h = (h + 2 * (l["size"] // 2) - l["size"]) // l["stride"] + 1
            cin = 3 if src < 0 else chans[src]
            macs += batch * l["filters"] * h * h * cin * l["size"] ** 2
        elif l["type"] == "upsample":
            h *= 2
        hw.append(h)
    return macs


class YoloV4Int8:
    """The network on the device: calibrate(x) fixes one activation scale per convolution input, forward(x)
    returns the three head tensors (fp32 NCHW)."""

    def __init__(self, L, heads, params, device="cuda:0"):
        self.L, self.heads, self.host = L, heads, params
        self.srcs, self.chans = resolve(L)
        self.dev = torch.device(device)
        self.conv, self.bias, self.dq, self.sx = {}, {}, {}, {}
        for i, p in params.items():
            l = L[i]
            self.conv[i] = capi.Conv2dI8(torch.from_numpy(p["wq"]).to(self.dev), (l["size"] // 2,) * 4, (l["stride"],) * 2)
            self.bias[i] = torch.from_numpy(p["bias"]).to(self.dev)
        self.scales = None

    def set_scales(self, scales, n):
        self.scales = dict(scales)
        for i, s in self.scales.items():
            self.dq[i] = torch.from_numpy((np.float32(1.0) / (np.float32(s) * self.host[i]["sw"])).astype(np.float32)).to(self.dev)
            self.sx[i] = torch.full((n,), s, dtype=torch.float32, device=self.dev)

    def calibrate(self, x):
        self.scales = {}
        self._run(x, calibrating=True)
        self.set_scales(self.scales, x.shape[0])
        return dict(self.scales)

    def forward(self, x):
        assert self.scales is not None
        return self._run(x, calibrating=False)

    def _run(self, x, calibrating):
        n = x.shape[0]
        outs = []
        last_use = {}
        for i, s in enumerate(self.srcs):
            for j in s:
                last_use[j] = i
        for i, l in enumerate(self.L):
            get = lambda j: x if j < 0 else outs[j]
            src = [get(j) for j in self.srcs[i]]
            if l["type"] == "conv":
                t = src[0]
                if calibrating:
                    m = float(t.abs().max().item())
                    self.scales[i] = float(np.float32(127.0) / np.float32(m if m > 0 else 1.0))
                    sx = torch.full((n,), self.scales[i], dtype=torch.float32, device=self.dev)
                    dq = torch.from_numpy((np.float32(1.0) / (np.float32(self.scales[i]) * self.host[i]["sw"])).astype(np.float32)).to(self.dev)
                else:
                    sx, dq = self.sx[i], self.dq[i]
                y = self.conv[i](t, dq=dq, bias=self.bias[i], act=l["act"], slope=0.1, x_scales=sx)[0]
            elif l["type"] == "route":
                y = src[0] if len(src) == 1 else capi.concat_channels(src)
            elif l["type"] == "shortcut":
                y = capi.add(src[0], src[1])
            elif l["type"] == "maxpool":
                k = l["size"]
                y = capi.pooling2d(src[0], "max", (k, k), (1, 1), (k // 2,) * 4)
            elif l["type"] == "upsample":
                y = capi.resize_nearest(src[0], src[0].shape[2] * 2, src[0].shape[3] * 2)
            outs.append(y)
            for j in self.srcs[i]:            # free activations nothing reads any more
                if j >= 0 and last_use[j] == i and j not in self.heads:
                    outs[j] = None
        return [outs[h] for h in self.heads]
