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

from .api import PulpNNError

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


class Runner:
    """Uploads the parameters once and runs the chain on the GPU through the C API."""

    def __init__(self, nn, net, fused=True):
        import torch
        self.nn, self.net, self.torch = nn, net, torch
        # fused: depthwise layers read the HWC output of the previous layer directly
        # (pulp_nn_hip_depthwise_hwc) where the library has a kernel for it; otherwise, and with
        # fused=False, the chain is the reference's: pulp_nn_hip_hwc_to_chw + pulp_nn_depthwise_generic
        self.fused, self.unfused = fused, set()
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        self.params = [dict(w=dev(L["w"]), bias=dev(L["bias"]), k=dev(L["k"]), lam=dev(L["lam"]))
                       for L in net["layers"]]
        self.fc_w, self.fc_bias = dev(net["fc_w"]), dev(net["fc_bias"])
        B = net["batch"]
        u8 = lambda *shape: torch.empty(shape, dtype=torch.uint8, device="cuda")
        self.act = [u8(B, L["hout"], L["hout"], L["cout"]) for L in net["layers"]]
        self.chw = {i: u8(B, L["cin"], L["hin"], L["hin"]) for i, L in enumerate(net["layers"]) if L["kind"] == "dw"}
        self.pooled = u8(B, 512)
        self.logits = torch.empty((B, 1000), dtype=torch.int32, device="cuda")

    def run(self, x):
        """x: device tensor B,128,128,3 uint8.  Returns the int32 logits tensor (B,1000)."""
        nn, B = self.nn, self.net["batch"]
        nn.set_batch(B)
        cur = x
        for i, (L, P) in enumerate(zip(self.net["layers"], self.params)):
            out = self.act[i]
            hi, ho, ci, co, s = L["hin"], L["hout"], L["cin"], L["cout"], L["stride"]
            if L["kind"] == "conv":
                nn.pulp_nn_conv_Ho_parallel(cur, None, P["bias"], out, P["w"], P["k"], P["lam"], 0, L["shift"],
                                            hi, hi, ci, ho, ho, co, 3, 3, 1, 1, 1, 1, s, s, 1, 1)
            elif L["kind"] == "dw":
                if self.fused and i not in self.unfused:
                    try:
                        # layout change fused into the depthwise kernel
                        nn.depthwise_hwc(cur, P["bias"], out, P["w"], P["k"], P["lam"], 0, L["shift"],
                                         hi, hi, ci, ho, ho, s, 1, 1)
                        cur = out
                        continue
                    except PulpNNError as err:
                        if err.code != 2:
                            raise
                        self.unfused.add(i)   # no fused kernel for this geometry
                chw = self.chw[i]
                nn.hwc_to_chw(cur, chw, hi, hi, ci)
                nn.pulp_nn_depthwise_generic(chw, None, P["bias"], out, P["w"], None, P["k"], P["lam"], 0, L["shift"],
                                             hi, hi, ci, ho, ho, co, 3, 3, 1, 1, 1, 1, s, s, 1, 1)
            else:
                nn.pulp_nn_pointwise_HoWo_parallel(cur, None, P["bias"], out, P["w"], P["k"], P["lam"], 0, L["shift"],
                                                   hi, hi, ci, ho, ho, co, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1)
            cur = out
        nn.pulp_nn_avgpool(cur, self.pooled, 0, 0, 0, 4, 4, 512, 1, 1, 4, 4, 0, 0, 0, 0, 4, 4, 0)
        nn.pulp_nn_linear_out_32(self.pooled, self.fc_bias, self.logits, self.fc_w, 512, 1000)
        return self.logits
