"""Host logic of the YOLOv4-shaped network runner (no GPU): the layer list, and which tensors the chained pass
keeps int8 between quantized convolutions (tennis_amd/yolov4.py, YoloV4Int8._chain_plan).  The plan is a pure
function of the layer list and the weight shapes, so it is built here on an object without device state.
"""
import numpy as np

from tennis_amd import yolov4


def planned(width=1.0, classes=80):
    L, heads = yolov4.layers(width=width, classes=classes)
    srcs, chans = yolov4.resolve(L)
    net = object.__new__(yolov4.YoloV4Int8)
    net.L, net.heads, net.srcs, net.chans = L, heads, srcs, chans
    net.host = {}
    for i, l in enumerate(L):
        if l["type"] == "conv":
            cin = 3 if srcs[i][0] < 0 else chans[srcs[i][0]]
            net.host[i] = {"wq": np.broadcast_to(np.int8(0), (l["filters"], cin, l["size"], l["size"]))}
    return net, L, net._chain_plan()


def test_layer_list():
    L, heads = yolov4.layers()
    assert sum(1 for l in L if l["type"] == "conv") == 110          # the 110 convolutions of yolov4.cfg
    assert sum(1 for l in L if l["type"] == "shortcut") == 23
    assert sum(1 for l in L if l["type"] == "maxpool") == 3 and sum(1 for l in L if l["type"] == "upsample") == 2
    assert len(heads) == 3
    assert 60e9 < yolov4.total_macs(L, 1, 608) < 68e9               # ~64 GMAC per 608x608 image


def test_every_join_is_handed_over_in_int8_at_full_width():
    net, L, (rsrcs, consumers, heads, folded) = planned()
    joins = [i for i, l in enumerate(L) if l["type"] == "route" and len(net.srcs[i]) > 1]
    assert len(joins) == 10 and sorted(net._concat_routes) == joins          # no fp32 concatenation left
    assert len(folded) == 23                                                 # every shortcut sits in an epilogue
    assert all(L[a]["type"] == "conv" and consumers[a] == [s] for s, a in folded.items())
    assert len(net._folded_upsamples) == 2 and all(L[j]["type"] == "upsample" for j in net._folded_upsamples)
    assert sorted(L[j]["size"] for j in net._spp_pools) == [5, 9, 13]
    # SPP: each pooling is a 5 x 5 maximum of the next smaller window's run of channels
    assert all(v[5] == 5 for v in net._spp_pools.values())
    by_size = sorted(net._spp_pools, key=lambda j: L[j]["size"])
    for a, b in zip(by_size, by_size[1:]):
        assert net._spp_pools[b][2] == net._spp_pools[a][3]                  # reads what the smaller window wrote


def test_channel_runs_tile_each_consumer():
    for width in (1.0, 0.125):
        net, L, (rsrcs, consumers, heads, folded) = planned(width, 3)
        per_route = {}
        for c, (route, k, c0, total, up) in net._concat_of.items():
            assert L[c]["type"] == "conv" and L[k]["type"] == "conv" and consumers[route] == [k]
            assert c not in heads and c not in folded.values() and c0 % 16 == 0 and up in (1, 2)
            per_route.setdefault(route, []).append((c0, L[c]["filters"], total))
        for j, (k, total, src_off, dst_off, f, win) in net._spp_pools.items():
            route = [r for r, kk in net._concat_routes.items() if kk == k][0]
            per_route[route].append((dst_off, f, total))
        for route, runs in per_route.items():
            runs.sort()
            total = runs[0][2]
            assert all(r[2] == total for r in runs) and net._concat_channels[route] == total
            pos = 0
            for c0, f, _ in runs:                                            # the runs cover [0, total) without overlap
                assert c0 == pos
                pos += f
            assert pos == total == net.chans[route]


def test_a_branch_with_other_readers_keeps_its_fp32_copy():
    """PANet's downsampling joins: the lateral branch is also read by a 3x3 convolution with a scale of its own."""
    net, L, (rsrcs, consumers, heads, folded) = planned()
    shared = {c: consumers[c] for c, v in net._concat_of.items() if len(consumers[c]) > 1 and L[v[0]]["type"] == "route"
              and all(L[j]["type"] != "maxpool" for j in consumers[c])}
    assert len(shared) == 2
    for c, cons in shared.items():
        route = net._concat_of[c][0]
        assert cons.count(route) == 1 and all(L[k]["type"] == "conv" for k in cons if k != route)
