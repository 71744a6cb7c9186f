"""The chained int8 network of benchmark configuration 3: MobileNetV1, width 0.5, 128x128x3
input: a 3x3 stride-2 stem to 16 channels, 13 depthwise-3x3 + pointwise-1x1 blocks, global
average pooling and a 512 -> 1000 linear layer with int32 output.

Everything runs through the C API: pulp_nn_conv_Ho_parallel, pulp_nn_depthwise_generic,
pulp_nn_pointwise_HoWo_parallel, pulp_nn_avgpool, pulp_nn_linear_out_32, plus
pulp_nn_hip_hwc_to_chw between a pointwise output (HWC) and the next depthwise input (CHW)
(or, where the library has a kernel for it, the two fused: pulp_nn_hip_depthwise_hwc),
a step the reference leaves to the application.

Parameters are seeded like configuration 0 (int8 weights and bias, 32-bit k in [256, 1024],
lambda in [-2^16, 2^16]); every conv / depthwise / pointwise layer uses batch-norm + ReLU
with out_shift = floor(log2(max |acc * k|)) - 7 over the whole batch.  The shifts depend on
the data flowing through the chain, so they are calibrated once by
tests/golden/make_cfg3_shifts.py and stored next to this file.
"""
import json
import os

import numpy as np

from . import network

WIDTHS = (32, 64, 64, 128, 128, 256, 256, 256, 256, 256, 256, 512, 512)
STRIDE2_BLOCKS = (2, 4, 6, 12)   # 1-based
SEED = 20243
SHIFTS_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mobilenet_cfg3_shifts.json")


def layer_table():
    """[(kind, name, cin, cout, stride, in_hw, out_hw)] for the conv-like layers."""
    layers = [("conv", "stem", 3, 16, 2, 128, 64)]
    hw, cin = 64, 16
    for i, cout in enumerate(WIDTHS, start=1):
        s = 2 if i in STRIDE2_BLOCKS else 1
        layers.append(("dw", "b%d_dw" % i, cin, cin, s, hw, hw // s))
        hw //= s
        layers.append(("pw", "b%d_pw" % i, cin, cout, 1, hw, hw))
        cin = cout
    return layers


def build(batch=256, shifts=None):
    """Seeded parameters and input.  `shifts`: {layer name: out_shift}; by default the
    calibrated values stored in mobilenet_cfg3_shifts.json (valid for batch 256)."""
    r = np.random.Generator(np.random.PCG64(SEED))
    net = {"batch": batch, "layers": []}
    net["x"] = r.integers(0, 256, size=(batch, 128, 128, 3), dtype=np.uint8)
    if shifts is None:
        if not os.path.exists(SHIFTS_FILE):
            raise FileNotFoundError("%s missing: run tests/golden/make_cfg3_shifts.py" % SHIFTS_FILE)
        rec = json.load(open(SHIFTS_FILE))
        if rec["batch"] != batch:
            raise ValueError("stored shifts were calibrated for batch %d" % rec["batch"])
        shifts = rec["shifts"]
    for kind, name, cin, cout, stride, hin, hout in layer_table():
        if kind == "conv":
            w = r.integers(-128, 128, size=(cout, 3, 3, cin), dtype=np.int8)
        elif kind == "dw":
            w = r.integers(-128, 128, size=(cout, 3, 3), dtype=np.int8)
        else:
            w = r.integers(-128, 128, size=(cout, 1, 1, cin), dtype=np.int8)
        net["layers"].append(dict(
            kind=kind, name=name, cin=cin, cout=cout, stride=stride, hin=hin, hout=hout, w=w,
            bias=r.integers(-128, 128, size=cout, dtype=np.int8),
            k=r.integers(256, 1025, size=cout).astype(np.int32),
            lam=r.integers(-2 ** 16, 2 ** 16 + 1, size=cout).astype(np.int32),
            shift=shifts.get(name) if shifts else None))
    net["fc_w"] = r.integers(-128, 128, size=(1000, 512), dtype=np.int8)
    net["fc_bias"] = r.integers(-2 ** 12, 2 ** 12 + 1, size=1000).astype(np.int32)
    ops = 0
    for L in net["layers"]:
        taps = 9 if L["kind"] in ("conv", "dw") else 1
        cin_eff = 1 if L["kind"] == "dw" else L["cin"]
        ops += 2 * batch * L["hout"] ** 2 * L["cout"] * taps * cin_eff
    net["ops"] = ops + 2 * batch * 512 * 1000
    return net


def descriptor(net):
    """The chain as a layer table for network.Runner (see network.py for the format)."""
    layers, prev = [], "input"
    for L in net["layers"]:
        s = L["stride"]
        common = dict(name=L["name"], w=L["w"], bias=L["bias"], k=L["k"], lam=L["lam"], relu=1, bn=1, mult=0,
                      shift=L["shift"])
        common["in"] = prev
        if L["kind"] == "conv":
            layers.append(dict(op="conv", pads=(1, 1, 1, 1), strides=(s, s), out_hw=(L["hout"], L["hout"]), **common))
        elif L["kind"] == "dw":
            layers.append(dict(op="depthwise", pads=(1, 1, 1, 1), strides=(s, s), out_hw=(L["hout"], L["hout"]), **common))
        else:
            layers.append(dict(op="pointwise", **common))
        prev = L["name"]
    layers.append({"op": "avgpool", "name": "pool", "in": prev, "kernel": (4, 4), "strides": (4, 4), "out_hw": (1, 1)})
    layers.append({"op": "linear_out_32", "name": "fc", "in": "pool", "w": net["fc_w"], "bias32": net["fc_bias"]})
    return layers


class Runner(network.Runner):
    """The configuration-3 chain on the generic runner.  fused: depthwise layers read the HWC
    output of the previous layer directly (pulp_nn_hip_depthwise_hwc) where the library has a
    kernel for it; otherwise, and with fused=False, the chain is the reference's:
    pulp_nn_hip_hwc_to_chw + pulp_nn_depthwise_generic.  fuse_blocks: a depthwise layer and the
    pointwise layer behind it run as one launch (pulp_nn_hip_dw_pw_hwc); the depthwise results are
    then not materialised (self.activations holds stale buffers for them).  chain_blocks: the run of
    five identical blocks on 8 x 8 x 256 is one launch (pulp_nn_hip_dw_pw_chain_hwc); only its last
    output is materialised."""

    def __init__(self, nn, net, fused=True, fuse_blocks="auto", chain_blocks=True):
        self.net = net
        super().__init__(nn, descriptor(net), (128, 128, 3), net["batch"], fused=fused, fuse_blocks=fuse_blocks,
                         chain_blocks=chain_blocks)
        self.logits = self.act["fc"].view(net["batch"], 1000)
        self.activations = [self.act[L["name"]] for L in net["layers"]]

    def run(self, x):
        """x: device tensor B,128,128,3 uint8.  Returns the int32 logits tensor (B,1000)."""
        super().run(x)
        return self.logits
