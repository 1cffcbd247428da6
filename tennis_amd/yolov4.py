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
    returns the three head tensors (fp32 NCHW).  mish: "exact" -- the Mish layers give the values of the operator
    chain softplus -> tanh -> mul bit for bit -- or "fast", the one-exponential form (1e-7 relative; about one
    requantized int8 value in a million differs)."""

    def __init__(self, L, heads, params, device="cuda:0", mish="exact"):
        if mish not in ("exact", "fast"):
            raise ValueError("mish: 'exact' or 'fast'")
        if mish == "fast":
            L = [dict(l, act="mish_fast") if l.get("act") == "mish" else l for l in L]
        self.L, self.heads, self.host = L, heads, params
        self.srcs, self.chans = resolve(L)
        self.dev = torch.device(device)
        self.conv, self.bias, self.dq, self.sx = {}, {}, {}, {}
        for i, p in params.items():
            l = L[i]
            self.conv[i] = capi.Conv2dI8(torch.from_numpy(p["wq"]).to(self.dev), (l["size"] // 2,) * 4, (l["stride"],) * 2)
            self.bias[i] = torch.from_numpy(p["bias"]).to(self.dev)
        self.scales = None
        self._shapes = {}
        # set to (images, list) to record, per convolution of the chained pass, the tensors it read and wrote for
        # those images of the batch (copies; for per-layer checks against the operator chain)
        self.trace = None

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

    def forward(self, x, chained=True):
        assert self.scales is not None
        return self._run_chained(x) if chained else self._run(x, calibrating=False)

    # ---------------------------------------------------------------- chained inference
    def _chain_plan(self):
        """Who reads what, with single-source routes looked through and `conv -> shortcut` pairs folded into the
        convolution's epilogue (darknet's shortcut adds behind the activation).  Returns per layer: the resolved
        sources, the consumers of each tensor, and for folded shortcuts the convolution that absorbs them."""
        L = self.L

        def root(j):
            while j >= 0 and L[j]["type"] == "route" and len(self.srcs[j]) == 1:
                j = self.srcs[j][0]
            return j

        rsrcs = [[root(j) for j in s] for s in self.srcs]
        identity = [l["type"] == "route" and len(self.srcs[i]) == 1 for i, l in enumerate(L)]
        consumers = {i: [] for i in range(-1, len(L))}
        for i, s in enumerate(rsrcs):
            if not identity[i]:
                for j in s:
                    consumers[j].append(i)
        heads = {root(h) for h in self.heads}
        folded = {}      # shortcut layer -> the convolution whose epilogue performs it
        for i, l in enumerate(L):
            if l["type"] == "shortcut":
                a, b = rsrcs[i]
                if L[a]["type"] == "conv" and consumers[a] == [i] and a not in heads and a != b:
                    folded[i] = a
        # Channel concatenations (routes with several sources) whose sources are all convolution outputs that nothing
        # else reads and whose one consumer is a convolution that can read a staged buffer: every source convolution
        # writes its requantized output into its run of channels of that consumer's staged input (the CSP stages'
        # two-branch joins).  concat_of: source convolution -> (route, consumer, first channel, total channels).
        self._concat_of, self._concat_routes, self._concat_channels, self._folded_upsamples = {}, {}, {}, set()
        self._spp_pools = {}   # max pooling layer -> (consumer, total channels, source run, own run, channels, window)
        for i, l in enumerate(L):
            if l["type"] != "route" or len(self.srcs[i]) < 2 or i in heads:
                continue
            cons = consumers[i]
            if len(cons) != 1 or L[cons[0]]["type"] != "conv" or not self._stageable(cons[0]):
                continue
            s = rsrcs[i]
            # An SPP block: one convolution and stride-1 "same" max poolings of its output, nothing else reading any
            # of them.  quantize commutes with max, so the convolution writes its requantized output into its run of
            # the consumer's staged channels and every pooling goes from one run of int8 channels into the next
            # (cascaded: the k x k maximum is the (k - k' + 1)-maximum of the k' x k' maxima).
            convs = [j for j in s if j >= 0 and L[j]["type"] == "conv"]
            pools = [j for j in s if j >= 0 and L[j]["type"] == "maxpool"]
            if len(convs) == 1 and pools and len(convs) + len(pools) == len(s) and len(set(s)) == len(s):
                c = convs[0]
                f = L[c]["filters"]
                ok = (f % 64 == 0 and c not in heads and c not in folded.values() and sorted(consumers[c]) == sorted(pools + [i])
                      and all(rsrcs[j] == [c] and consumers[j] == [i] and j not in heads and L[j]["size"] % 2 == 1 for j in pools)
                      and len({L[j]["size"] for j in pools}) == len(pools))
                if ok:
                    total = f * len(s)
                    self._concat_of[c] = (i, cons[0], s.index(c) * f, total, 1)
                    self._concat_routes[i] = cons[0]
                    self._concat_channels[i] = total
                    prev_k, prev_off = 1, s.index(c) * f
                    for j in sorted(pools, key=lambda j: L[j]["size"]):
                        self._spp_pools[j] = (cons[0], total, prev_off, s.index(j) * f, f, L[j]["size"] - prev_k + 1)
                        prev_k, prev_off = L[j]["size"], s.index(j) * f
                    continue
            # a source is a convolution, or the 2x upsampling of one that nothing else reads (the convolution then
            # writes every pixel to the 2 x 2 pixels it becomes: capi.StagedSlice(upsample=2))
            prod = []
            for j in s:
                if j >= 0 and L[j]["type"] == "upsample" and consumers[j] == [i] and j not in heads:
                    c = rsrcs[j][0]
                    prod.append((c, 2) if c >= 0 and L[c]["type"] == "conv" and consumers[c] == [j] else None)
                else:
                    # read by this route once; further readers get the fp32 copy the convolution then also writes
                    prod.append((j, 1) if j >= 0 and L[j]["type"] == "conv" and consumers[j].count(i) == 1
                                and j not in self._concat_of else None)
            ok = all(pr is not None and pr[0] not in heads and pr[0] not in folded.values() for pr in prod) and \
                len({pr[0] for pr in prod if pr}) == len(prod)
            if not ok:
                continue
            filters = [L[pr[0]]["filters"] for pr in prod]
            offsets = [sum(filters[:m]) for m in range(len(prod))]
            if any(o % 16 for o in offsets):
                continue
            total = sum(filters)
            for (c, up), o in zip(prod, offsets):
                self._concat_of[c] = (i, cons[0], o, total, up)
            self._concat_routes[i] = cons[0]
            self._concat_channels[i] = total
            for j in s:
                if L[j]["type"] == "upsample":
                    self._folded_upsamples.add(j)
        return rsrcs, consumers, heads, folded

    def _run_chained(self, x):
        """Inference with int8 hand-over: a convolution whose output feeds convolutions writes it requantized
        straight into their staged input (one buffer per consumer geometry; consumers of one tensor share its
        calibrated scale), keeps an fp32 copy only if something else reads it (route, shortcut, pooling,
        upsample, a head), and performs a following shortcut in its epilogue.  Values equal the
        operator-by-operator path (_run)."""
        n = x.shape[0]
        if not hasattr(self, "_plan"):
            self._plan = self._chain_plan()
            self._staged, self._pair_conv, self._pair_prod = {}, {}, {}
        rsrcs, consumers, heads, folded = self._plan
        absorbed = {a: s for s, a in folded.items()}
        L = self.L
        outs = [None] * len(L)            # fp32 tensors
        staged_for = {}                   # consumer conv -> StagedInput holding its input (written by the producer)
        last_use = {}
        for i, s in enumerate(rsrcs):
            for j in s:
                last_use[j] = i
        get = lambda j: x if j < 0 else outs[j]

        def staged_input(k, shape):
            key = (k, tuple(shape))
            if key not in self._staged:
                l = L[k]
                if shape[1] == 32 and l["size"] == 3 and l["stride"] == 2 and shape[3] % 2 == 0:
                    # 32 channels would be staged with 32 bytes of padding per pixel: stage pairs of columns as one
                    # 64-channel pixel instead and run the 3x3 stride-2 layer as a 3x2 stride-(2, 1) one over the pairs
                    # (equal accumulators; half the bytes written and read, 6 K-steps instead of 9)
                    if k not in self._pair_conv:
                        self._pair_conv[k] = capi.Conv2dI8(capi.pair_columns_weights(self.conv[k].w), (1, 1, 1, 0), (2, 1))
                    pairs = capi.StagedInput(self._pair_conv[k], (shape[0], 64, shape[2], shape[3] // 2))
                    self._staged[key] = capi.StagedPairs(pairs)
                else:
                    self._staged[key] = capi.StagedInput(self.conv[k], shape)
            return self._staged[key]

        for i, l in enumerate(L):
            t = l["type"]
            if t == "conv":
                out_id = absorbed.get(i, i)                     # the tensor this kernel produces
                conv = self.conv[i]
                src = rsrcs[i][0]
                in_shape = tuple(x.shape) if src < 0 else self._shapes[src]
                ho = (in_shape[2] + 2 * (l["size"] // 2) - l["size"]) // l["stride"] + 1
                wo = (in_shape[3] + 2 * (l["size"] // 2) - l["size"]) // l["stride"] + 1
                shape = (n, l["filters"], ho, wo)
                self._shapes[out_id] = shape
                self._shapes[i] = shape
                # consumers of the produced tensor
                conv_cons = [k for k in consumers[out_id] if L[k]["type"] == "conv"]
                others = [k for k in consumers[out_id] if L[k]["type"] != "conv"]
                # one staged buffer -- the consumer's with the largest halo -- serves every consumer whose own staged
                # input fits inside it (less halo, fewer rows: a 1x1 or a strided convolution beside a 3x3 one)
                target, served = None, []
                branch = i in self._concat_of and out_id == i
                own = {} if branch else {k: staged_input(k, shape) for k in conv_cons if self._stageable(k)}
                if own:
                    owner = max(own, key=lambda k: (own[k].pad_top, own[k].pad_left, own[k].hs, own[k].ws))
                    target = own[owner]
                    for k, st in own.items():
                        if k == owner or (st.hs, st.ws, st.cp, st.pad_top, st.pad_left) == (target.hs, target.ws, target.cp, target.pad_top, target.pad_left):
                            served.append(k)
                            staged_for[k] = target
                        elif (st.cp == target.cp and st.pad_top <= target.pad_top and st.pad_left <= target.pad_left
                              and st.hs + target.pad_top - st.pad_top <= target.hs and st.ws + target.pad_left - st.pad_left <= target.ws):
                            served.append(k)
                            staged_for[k] = capi.StagedView(target, st.pad_top, st.pad_left)
                for k in served:
                    assert self.scales[k] == self.scales[served[0]]   # calibrated on the same tensor
                want_f32 = bool(others) or out_id in heads or any(k not in served for k in conv_cons)
                q_layer = served[0] if served else None
                if branch:
                    # one branch of a channel concatenation: straight into its channels of the consumer's staged input,
                    # requantized with that consumer's scale; any other reader (a convolution with a scale of its own
                    # included) takes the fp32 copy
                    route, k, c0, total, up = self._concat_of[i]
                    whole = staged_input(k, (n, total, ho * up, wo * up))
                    target = capi.StagedSlice(whole, c0, l["filters"], upsample=up)
                    staged_for[k] = whole
                    want_f32 = bool(conv_cons) or any(o != route for o in others) or out_id in heads
                    q_layer = k
                kw = dict(dq=self.dq[i], bias=self.bias[i], act=l["act"], slope=0.1, want_f32=want_f32)
                if target is not None:
                    kw.update(q_scales=self.sx[q_layer], staged_out=target)
                if i in absorbed:
                    kw.update(residual=outs[rsrcs[absorbed[i]][1]], residual_after_act=True)
                cin = self.conv[i].w.shape[1]
                if (isinstance(target, capi.StagedPairs) and not want_f32 and i not in absorbed and i not in staged_for
                        and l["size"] == 3 and l["stride"] == 1 and cin * 3 * 4 <= 64):
                    # the stem in front of a pair-staged layer: computed as pairs of output columns (a 3x4 window at column
                    # stride 2, 2 x 32 output channels; its K still fits one 64-byte step), so that its im2col rows are
                    # per pair -- half the staged bytes
                    if i not in self._pair_prod or self._pair_prod[i][1] is not self.dq[i]:      # new scales: new dq
                        pconv = (self._pair_prod[i][0] if i in self._pair_prod else
                                 capi.Conv2dI8(capi.pair_outputs_weights(self.conv[i].w), (1, 1, 1, 1), (1, 2)))
                        self._pair_prod[i] = (pconv, self.dq[i], torch.cat([self.dq[i]] * 2), torch.cat([self.bias[i]] * 2))
                    pconv, _, dq2, bias2 = self._pair_prod[i]
                    pconv(get(src), x_scales=self.sx[i], dq=dq2, bias=bias2, act=l["act"], slope=0.1, want_f32=False,
                          q_scales=self.sx[q_layer], staged_out=target.pairs)
                    y = None
                elif i in staged_for and isinstance(staged_for[i], capi.StagedPairs):
                    y = self._pair_conv[i].run_staged(staged_for[i].pairs, **kw)[0]
                elif i in staged_for:
                    y = conv.run_staged(staged_for[i], **kw)[0]
                else:
                    y = conv(get(src), x_scales=self.sx[i], **kw)[0]
                if self.trace is not None:
                    idx = list(self.trace[0])
                    res = kw.get("residual")
                    self.trace[1].append({
                        "layer": i, "in_q": capi.staged_interior(staged_for[i], idx).cpu().numpy() if i in staged_for else None,
                        "in_f32": None if i in staged_for else get(src)[idx].cpu().numpy(),
                        "residual": None if res is None else res[idx].cpu().numpy(),
                        "out_f32": None if y is None else y[idx].cpu().numpy(),
                        "out_q": None if target is None else capi.staged_interior(target, idx).cpu().numpy(),
                        "q_layer": q_layer})
                outs[out_id] = y
                if out_id != i:
                    outs[i] = None
            elif t == "shortcut":
                if i not in folded:
                    a, b = rsrcs[i]
                    outs[i] = capi.add(outs[a], outs[b])
                    self._shapes[i] = self._shapes[a]
            elif t == "route":
                s = rsrcs[i]
                if len(self.srcs[i]) == 1:
                    outs[i] = None                                 # looked through
                    self._shapes[i] = self._shapes[s[0]]
                elif i in self._concat_routes:
                    outs[i] = None                                 # its sources wrote the consumer's staged input
                    first = self._shapes[s[0]]
                    self._shapes[i] = (first[0], self._concat_channels[i], first[2], first[3])
                else:
                    outs[i] = capi.concat_channels([outs[j] for j in s])
                    self._shapes[i] = tuple(outs[i].shape)
            elif t == "maxpool" and i in self._spp_pools:
                k1, total, src_off, dst_off, f, win = self._spp_pools[i]
                sh = self._shapes[rsrcs[i][0]]
                whole = staged_input(k1, (n, total, sh[2], sh[3]))
                capi.max_pooling2d_staged(capi.StagedSlice(whole, src_off, f), capi.StagedSlice(whole, dst_off, f),
                                          (win, win), (1, 1), (win // 2,) * 4)
                outs[i] = None
                self._shapes[i] = sh
            elif t == "maxpool":
                k = l["size"]
                # An SPP block pools one map with growing odd windows at stride 1: the k x k maximum is the
                # (k - k' + 1)-maximum of the k' x k' maxima already computed (windows clipped to the map on both
                # levels; equal for finite values -- a tie between +0 and -0 may keep the other sign), so 9 and 13
                # cost a 5 x 5 pass each instead of 81 and 169 elements per output.
                src, kk = outs[rsrcs[i][0]], k
                for m in range(i):
                    if (L[m]["type"] == "maxpool" and rsrcs[m][0] == rsrcs[i][0] and outs[m] is not None
                            and L[m]["size"] % 2 == 1 and k % 2 == 1 and L[m]["size"] < k and k - L[m]["size"] + 1 <= kk):
                        src, kk = outs[m], k - L[m]["size"] + 1
                outs[i] = capi.pooling2d(src, "max", (kk, kk), (1, 1), (kk // 2,) * 4)
                self._shapes[i] = tuple(outs[i].shape)
            elif t == "upsample":
                if i in self._folded_upsamples:
                    outs[i] = None                                 # the producing convolution wrote the upsampled pixels
                    sh = self._shapes[rsrcs[i][0]]
                    self._shapes[i] = (sh[0], sh[1], sh[2] * 2, sh[3] * 2)
                else:
                    src = outs[rsrcs[i][0]]
                    outs[i] = capi.resize_nearest(src, src.shape[2] * 2, src.shape[3] * 2)
                    self._shapes[i] = tuple(outs[i].shape)
            for j in rsrcs[i]:                                     # free activations nothing reads any more
                if j >= 0 and last_use.get(j) == i and j not in heads:
                    outs[j] = None
        res = []
        for h in self.heads:
            j = h
            while L[j]["type"] == "route" and len(self.srcs[j]) == 1:
                j = self.srcs[j][0]
            res.append(outs[j])
        return res

    def _stageable(self, k):
        """True when convolution k can read a staged buffer a producer wrote (not an im2col-staged layer)."""
        l = self.L[k]
        cin = self.host[k]["wq"].shape[1]
        return not (l["size"] > 1 and cin <= 8 and cin * l["size"] ** 2 <= 512)

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
