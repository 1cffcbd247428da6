"""A ResNet-50-shaped int8 network on the MI355X convolution path.

Topology (random-init; the shape is what matters): 7x7/2 stem -> 3x3/2 max pool -> [3, 4, 6, 3]
bottleneck blocks (1x1 -> 3x3 -> 1x1, stride 2 on the 3x3 of the first block of stages 2-4, 1x1
projection shortcuts) with 64..2048 channels, BN folded into conv (so conv + bias), ReLU, residual
add, global average pool, FC 2048 -> 1000.  Per-output-channel int8 weights, per-tensor int8
activations calibrated on a batch.

Every layer is the TenniS operator chain the reference would run for a quantized graph --
    quantize(x, s) -> conv2d_quantized(w_q, dq) -> add_bias -> relu        (src/kernels/cpu/quantize.cpp,
    quantized/conv2d_quantized_core.cpp, add_bias.cpp, relu.cpp)
    add -> relu (residual join), pooling2d, global_pooling2d, and for the classifier
    quantize -> int8 gemm -> dequant -> add_bias
-- executed with the chain fused into the kernels' epilogues, which reproduce the separate operators
rounding for rounding.  `layers()` describes the network independently of the device so that the same
description can be evaluated by a CPU checker.

Activation scales follow the reference's quantize operator: `quantize_scale` holds one multiplier per
image (its length must equal the batch); per-tensor calibration passes N equal values.
"""
import numpy as np
import torch

from . import capi

STAGES = ((64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2))   # (mid channels, blocks, stride of the first block)


class ConvSpec:
    def __init__(self, name, cin, cout, k, stride, pad, relu):
        self.name, self.cin, self.cout, self.k, self.stride, self.pad, self.relu = name, cin, cout, k, stride, pad, relu


def layers(width=1.0, blocks=None, classes=1000):
    """The network as data: stem spec, list of blocks (conv1, conv2, conv3, projection-or-None), fc (cin, cout).
    `width` scales every channel count and `blocks` overrides the per-stage block counts (small test nets)."""
    ch = lambda c: max(8, int(c * width))
    stem = ConvSpec("stem", 3, ch(64), 7, 2, 3, True)
    net, cin = [], ch(64)
    for si, (mid, count, stride) in enumerate(STAGES):
        count = blocks[si] if blocks else count
        for bi in range(count):
            s = stride if bi == 0 else 1
            m, cout = ch(mid), ch(mid * 4)
            name = "s%db%d" % (si + 1, bi)
            proj = ConvSpec(name + ".proj", cin, cout, 1, s, 0, False) if bi == 0 else None
            net.append((ConvSpec(name + ".c1", cin, m, 1, 1, 0, True), ConvSpec(name + ".c2", m, m, 3, s, 1, True),
                        ConvSpec(name + ".c3", m, cout, 1, 1, 0, False), proj))
            cin = cout
    return stem, net, (cin, classes)


def quantize_weights(w):
    """Per-output-channel symmetric int8, round half away from zero (offline weight quantization)."""
    flat = w.reshape(w.shape[0], -1)
    s = (np.float32(127.0) / np.maximum(np.abs(flat).max(axis=1), np.float32(1e-12))).astype(np.float32)
    q = flat * s[:, None]
    q = np.clip(np.sign(q) * np.floor(np.abs(q) + np.float32(0.5)), -127, 127).astype(np.int8)
    return q.reshape(w.shape), s


def make_parameters(seed=0, width=1.0, blocks=None, classes=1000):
    """Random Kaiming-normal weights quantized per channel; small random biases.  Host arrays only."""
    rng = np.random.default_rng(seed)
    stem, net, fc = layers(width, blocks, classes)
    params = {}

    def conv(spec):
        fan_in = spec.cin * spec.k * spec.k
        w = (rng.standard_normal((spec.cout, spec.cin, spec.k, spec.k)) * np.sqrt(2.0 / fan_in)).astype(np.float32)
        wq, sw = quantize_weights(w)
        params[spec.name] = {"wq": wq, "sw": sw, "bias": (rng.standard_normal(spec.cout) * 0.05).astype(np.float32)}

    conv(stem)
    for c1, c2, c3, proj in net:
        for spec in (c1, c2, c3, proj):
            if spec is not None:
                conv(spec)
    w = (rng.standard_normal((fc[0], fc[1])) * np.sqrt(1.0 / fc[0])).astype(np.float32)   # [k][n]
    wq_t, sw = quantize_weights(np.ascontiguousarray(w.T))                                  # per output column
    params["fc"] = {"wq": np.ascontiguousarray(wq_t.T), "sw": sw, "bias": (rng.standard_normal(fc[1]) * 0.05).astype(np.float32)}
    return (stem, net, fc), params


def total_macs(desc, batch, size):
    """Multiply-accumulates of one forward pass (convolutions + classifier)."""
    stem, net, fc = desc

    def out(h, spec):
        return (h + 2 * spec.pad - spec.k) // spec.stride + 1

    h = out(size, stem)
    macs = batch * stem.cout * h * h * stem.cin * stem.k * stem.k
    h = int(np.ceil((h + 1 - 3) / 2.0 + 1))
    for c1, c2, c3, proj in net:
        h2 = out(h, c2)
        macs += batch * c1.cout * h * h * c1.cin
        macs += batch * c2.cout * h2 * h2 * c2.cin * 9
        macs += batch * c3.cout * h2 * h2 * c3.cin
        if proj is not None:
            macs += batch * proj.cout * h2 * h2 * proj.cin
        h = h2
    return macs + batch * fc[0] * fc[1]


class ResNet50Int8:
    """The network on the device.  calibrate(x) fixes the activation scales; forward(x) runs the fused path."""

    POOL = ((3, 3), (2, 2), (0, 1, 0, 1))   # ksize, stride, pads: 112 -> 56 under TenniS's ceil-mode size rule

    def __init__(self, desc, params, device="cuda:0"):
        self.desc, self.host = desc, params
        self.dev = torch.device(device)
        self.conv, self.bias, self.sw = {}, {}, {}
        stem, net, fc = desc
        specs = [stem] + [s for blk in net for s in blk if s is not None]
        for spec in specs:
            p = params[spec.name]
            self.conv[spec.name] = capi.Conv2dI8(torch.from_numpy(p["wq"]).to(self.dev), (spec.pad,) * 4,
                                                 (spec.stride, spec.stride))
            self.bias[spec.name] = torch.from_numpy(p["bias"]).to(self.dev)
            self.sw[spec.name] = p["sw"]
        self.fc = capi.GemmI8(torch.from_numpy(params["fc"]["wq"]).to(self.dev))
        self.bias["fc"] = torch.from_numpy(params["fc"]["bias"]).to(self.dev)
        self.sw["fc"] = params["fc"]["sw"]
        self.scales = None      # name -> python float (multiplier applied before rounding)
        self._dq, self._sx = {}, {}
        self._staged = {}      # (conv name, input shape) -> StagedInput
        # set to (images, list) to record, per convolution of the chained pass, the tensors it read and wrote for
        # those images of the batch (copies; for per-layer checks against the operator chain)
        self.trace = None

    def _rec(self, spec, s_in=None, x=None, residual=None, out_f32=None, s_out=None, q_name=None):
        if self.trace is None:
            return
        imgs, rows = self.trace
        idx = list(imgs)
        rows.append({"spec": spec, "in_q": None if s_in is None else capi.staged_interior(s_in, idx).cpu().numpy(),
                     "in_f32": None if x is None else x[idx].cpu().numpy(),
                     "residual": None if residual is None else residual[idx].cpu().numpy(),
                     "out_f32": None if out_f32 is None else out_f32[idx].cpu().numpy(),
                     "out_q": None if s_out is None else capi.staged_interior(s_out, idx).cpu().numpy(),
                     "q_name": q_name})

    # ---- calibration: per-tensor scale = 127 / max|input of the layer| on this batch, measured on the
    # activations of the quantized network itself, layer by layer
    @staticmethod
    def _scale_of(t):
        m = float(t.abs().max().item())
        return float(np.float32(127.0) / np.float32(m if m > 0 else 1.0))

    def calibrate(self, x):
        n = x.shape[0]
        self.scales = {}
        self._forward(x, n, calibrating=True)
        self._dq = {k: torch.from_numpy((np.float32(1.0) / (np.float32(s) * self.sw[k])).astype(np.float32)).to(self.dev)
                    for k, s in self.scales.items()}
        return dict(self.scales)

    def set_scales(self, scales, n):
        self.scales = dict(scales)
        self._dq = {k: torch.from_numpy((np.float32(1.0) / (np.float32(s) * self.sw[k])).astype(np.float32)).to(self.dev)
                    for k, s in self.scales.items()}
        self._sx = {}
        self._batch_scales(n)

    def _batch_scales(self, n):
        """quantize_scale tensors: one equal multiplier per image (base_quantize.cpp:26)."""
        if self._sx.get("_n") != n:
            self._sx = {k: torch.full((n,), s, dtype=torch.float32, device=self.dev) for k, s in self.scales.items()}
            self._sx["_n"] = n
        return self._sx

    def forward(self, x):
        assert self.scales is not None, "calibrate() or set_scales() first"
        return self._forward_chained(x)

    def _staged_input(self, spec, x_shape):
        key = (spec.name, tuple(x_shape))
        if key not in self._staged:
            self._staged[key] = capi.StagedInput(self.conv[spec.name], x_shape)
        return self._staged[key]

    def _forward_chained(self, x):
        """Inference path: between quantized convolutions the activations stay int8 in the consumer's staged
        layout (written by the producer's epilogue); block outputs are also kept as fp32 NCHW, which the
        residual join of the next block reads.  Values are those of the operator chain in _forward."""
        stem, net, fc = self.desc
        n = x.shape[0]
        sxs = self._batch_scales(n)
        relu = lambda spec: "relu" if spec.relu else None

        c1 = net[0][0]
        if net[0][3] is not None:
            # Nothing reads the pooled tensor in fp32 (the first block's shortcut is a projection), and quantize
            # commutes with max: the stem requantizes for layer 1 in its epilogue and the pooling runs on int8,
            # from the stem's pixel-major output straight into layer 1's staged input.
            h1 = (x.shape[2] + 2 * stem.pad - stem.k) // stem.stride + 1
            w1 = (x.shape[3] + 2 * stem.pad - stem.k) // stem.stride + 1
            key = ("stem_out", n, h1, w1)
            if key not in self._staged:
                self._staged[key] = capi.StagedPlain((n, stem.cout, h1, w1), self.dev)
            s_stem = self._staged[key]
            if w1 % 2 == 0 and stem.cout % 64 == 0 and stem.cin * stem.k * (stem.k + stem.stride) <= 512:
                # the stem computed as pairs of output columns (a k x (k + stride) window at twice the column stride,
                # 2 x cout channels): the same staged bytes from half as many im2col rows of the same padded length
                dq1 = self._dq[stem.name]
                if "stem_pairs" not in self._staged or self._staged["stem_pairs"][1] is not dq1:   # new scales: new dq
                    pconv = (self._staged["stem_pairs"][0] if "stem_pairs" in self._staged else
                             capi.Conv2dI8(capi.pair_outputs_weights(self.conv[stem.name].w, stem.stride), (stem.pad,) * 4,
                                           (stem.stride, 2 * stem.stride)))
                    self._staged["stem_pairs"] = (pconv, dq1, torch.cat([dq1] * 2), torch.cat([self.bias[stem.name]] * 2))
                pconv, _, dq2, bias2 = self._staged["stem_pairs"]
                pconv(x, dq=dq2, bias=bias2, act=relu(stem), x_scales=sxs[stem.name], q_scales=sxs[c1.name],
                      want_f32=False, staged_out=s_stem.column_pairs())
            else:
                self.conv[stem.name](x, dq=self._dq[stem.name], bias=self.bias[stem.name], act=relu(stem),
                                     x_scales=sxs[stem.name], q_scales=sxs[c1.name], want_f32=False, staged_out=s_stem)
            hp, wp = capi.pool_out_size(h1, w1, self.POOL[0], self.POOL[2], self.POOL[1])
            s_in = self._staged_input(c1, (n, stem.cout, hp, wp))
            capi.max_pooling2d_staged(s_stem, s_in, *self.POOL)
            self._rec(stem, x=x, s_out=s_stem, q_name=c1.name)
            if self.trace is not None:
                self.trace[1].append({"spec": "pool", "out_q": capi.staged_interior(s_in, list(self.trace[0])).cpu().numpy()})
            y = None
        else:
            y = self.conv[stem.name](x, dq=self._dq[stem.name], bias=self.bias[stem.name], act=relu(stem),
                                     x_scales=sxs[stem.name])[0]
            y = capi.pooling2d(y, "max", *self.POOL)
            s_in = self._staged_input(c1, y.shape)
            self.conv[c1.name].stage(y, s_in, x_scales=sxs[c1.name])     # the only staging pass after the stem
        for bi, (c1, c2, c3, proj) in enumerate(net):
            conv1, conv2, conv3 = self.conv[c1.name], self.conv[c2.name], self.conv[c3.name]
            in_shape = s_in.x_shape
            sc = y if proj is None else self.conv[proj.name].run_staged(s_in, self._dq[proj.name], self.bias[proj.name])[0]
            if proj is not None:
                self._rec(proj, s_in=s_in, out_f32=sc)
            s2 = self._staged_input(c2, (n, c1.cout, in_shape[2], in_shape[3]))
            conv1.run_staged(s_in, self._dq[c1.name], self.bias[c1.name], relu(c1), q_scales=sxs[c2.name], want_f32=False,
                             staged_out=s2)
            self._rec(c1, s_in=s_in, s_out=s2, q_name=c2.name)
            h2 = (in_shape[2] + 2 * c2.pad - c2.k) // c2.stride + 1
            w2 = (in_shape[3] + 2 * c2.pad - c2.k) // c2.stride + 1
            s3 = self._staged_input(c3, (n, c2.cout, h2, w2))
            conv2.run_staged(s2, self._dq[c2.name], self.bias[c2.name], relu(c2), q_scales=sxs[c3.name], want_f32=False,
                             staged_out=s3)
            self._rec(c2, s_in=s2, s_out=s3, q_name=c3.name)
            if bi + 1 < len(net):
                nxt = net[bi + 1][0]
                s_next = self._staged_input(nxt, (n, c3.cout, h2, w2))
                y = conv3.run_staged(s3, self._dq[c3.name], self.bias[c3.name], "relu", q_scales=sxs[nxt.name],
                                     residual=sc, staged_out=s_next)[0]
                self._rec(c3, s_in=s3, residual=sc, out_f32=y, s_out=s_next, q_name=nxt.name)
                s_in = s_next
            else:
                y = conv3.run_staged(s3, self._dq[c3.name], self.bias[c3.name], "relu", residual=sc)[0]
                self._rec(c3, s_in=s3, residual=sc, out_f32=y)
        pooled = capi.global_pooling2d(y, "avg").reshape(n, fc[0])
        p8 = capi.quantize(pooled, sxs["fc"])
        return self.fc(p8, dq=self._dq["fc"], bias=self.bias["fc"])[0]

    def _forward(self, x, n, calibrating):
        stem, net, fc = self.desc

        def dq_of(name, s):
            return torch.from_numpy((np.float32(1.0) / (np.float32(s) * self.sw[name])).astype(np.float32)).to(self.dev)

        def conv_from_f32(spec, t, out_scale_name=None):
            """quantize(t) -> conv -> bias -> relu?; int8 requantized output when the consumer's scale is known."""
            if calibrating:
                self.scales[spec.name] = self._scale_of(t)
                sx = torch.full((n,), self.scales[spec.name], dtype=torch.float32, device=self.dev)
                dq = dq_of(spec.name, self.scales[spec.name])
                return self.conv[spec.name](t, dq=dq, bias=self.bias[spec.name], act="relu" if spec.relu else None, x_scales=sx)[0]
            sxs = self._batch_scales(n)
            qs = sxs[out_scale_name] if out_scale_name else None
            f, q, _ = self.conv[spec.name](t, dq=self._dq[spec.name], bias=self.bias[spec.name],
                                           act="relu" if spec.relu else None, x_scales=sxs[spec.name], q_scales=qs,
                                           want_f32=qs is None)
            return q if qs is not None else f

        def conv_from_i8(spec, t8, out_scale_name=None, residual=None):
            """conv -> bias (-> + residual -> relu: the block's join, fused behind the last convolution)."""
            sxs = self._batch_scales(n)
            qs = sxs[out_scale_name] if out_scale_name else None
            act = "relu" if (spec.relu or residual is not None) else None
            f, q, _ = self.conv[spec.name](t8, dq=self._dq[spec.name], bias=self.bias[spec.name], act=act, q_scales=qs,
                                           want_f32=qs is None, residual=residual)
            return q if qs is not None else f

        y = conv_from_f32(stem, x)
        y = capi.pooling2d(y, "max", *self.POOL)
        for c1, c2, c3, proj in net:
            if calibrating:
                a = conv_from_f32(c1, y)
                b = conv_from_f32(c2, a)
                c = conv_from_f32(c3, b)
                sc = conv_from_f32(proj, y) if proj is not None else y
                y = capi.add(c, sc, "relu")
            else:
                sc = conv_from_f32(proj, y) if proj is not None else y
                a8 = conv_from_f32(c1, y, out_scale_name=c2.name)
                b8 = conv_from_i8(c2, a8, out_scale_name=c3.name)
                y = conv_from_i8(c3, b8, residual=sc)
        pooled = capi.global_pooling2d(y, "avg").reshape(n, fc[0])
        if calibrating:
            self.scales["fc"] = self._scale_of(pooled)
            sx = torch.full((n,), self.scales["fc"], dtype=torch.float32, device=self.dev)
            dq = dq_of("fc", self.scales["fc"])
        else:
            sx, dq = self._batch_scales(n)["fc"], self._dq["fc"]
        p8 = capi.quantize(pooled, sx)
        return self.fc(p8, dq=dq, bias=self.bias["fc"])[0]


def to_module(desc, params, batch, act_scale=16.0):
    """The network as a TenniS module graph (tennis_amd.module_file.Module) for a fixed batch size: per convolution
    quantize -> conv2d_quantized -> add_bias [-> relu], max pooling behind the stem, `add` + relu at every residual
    join, global average pooling and an fp32 inner_prod + add_bias classifier (TenniS has no quantized inner_prod).
    Every activation is quantized with the same multiplier `act_scale` (a module for exercising runtimes, not a
    calibrated model).  The graph a TenniS front end would hand to Workbench::Load."""
    from . import module_file as mf
    stem, net, fc = desc
    nodes = []

    def add(op, name, p=None, inputs=()):
        nodes.append(mf.Node(op, name, p or {}, list(inputs)))
        return len(nodes) - 1

    def conv(spec, x, relu):
        p = params[spec.name]
        scales = np.full(batch, act_scale, np.float32)
        q = add("quantize", spec.name + ".q", {"quantize_scale": scales}, [x])
        w = add(mf.CONST, spec.name + ".w", {"value": p["wq"]})
        cp = {"format": "NCHW",
              "padding": np.array([[0, 0], [0, 0], [spec.pad, spec.pad], [spec.pad, spec.pad]], np.int32),
              "padding_value": np.array([0.0], np.float32),
              "stride": np.array([1, 1, spec.stride, spec.stride], np.int32),
              "dilation": np.array([1, 1, 1, 1], np.int32),
              "dequantize_scales": (np.float32(1.0) / (np.float32(act_scale) * p["sw"])).astype(np.float32)}
        c = add("conv2d_quantized", spec.name, cp, [q, w])
        b = add(mf.CONST, spec.name + ".b", {"value": p["bias"]})
        y = add("add_bias", spec.name + ".bias", {"format": "NCHW"}, [c, b])
        return add("relu", spec.name + ".relu", {}, [y]) if relu else y

    x = add(mf.PARAMETER, "x")
    y = conv(stem, x, True)
    (kh, kw), (sh, sw_), pads = ResNet50Int8.POOL
    y = add("pooling2d", "pool", {"format": "NCHW", "type": np.array([0], np.int32),
                                  "padding": np.array([[0, 0], [0, 0], [pads[0], pads[1]], [pads[2], pads[3]]], np.int32),
                                  "padding_type": np.array([0], np.int32), "ksize": np.array([1, 1, kh, kw], np.int32),
                                  "stride": np.array([1, 1, sh, sw_], np.int32)}, [y])
    for c1, c2, c3, proj in net:
        sc = y if proj is None else conv(proj, y, False)
        z = conv(c3, conv(c2, conv(c1, y, True), True), False)
        y = add("relu", c3.name + ".out", {}, [add("add", c3.name + ".join", {}, [z, sc])])
    y = add("global_pooling2d", "gap", {"format": "NCHW", "type": np.array([1], np.int32)}, [y])
    wf = add(mf.CONST, "fc.w", {"value": (params["fc"]["wq"].astype(np.float32) / params["fc"]["sw"][None, :]).astype(np.float32)})
    y = add("inner_prod", "fc", {}, [y, wf])
    bf = add(mf.CONST, "fc.b", {"value": params["fc"]["bias"]})
    y = add("add_bias", "fc.bias", {"dim": np.array([1], np.int32)}, [y, bf])
    return mf.Module(nodes, [x], [y])
