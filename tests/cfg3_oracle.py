"""The configuration-3 chain evaluated with the CPU oracle (test infrastructure)."""
import numpy as np

import oracle


def layer_acc(L, x):
    """int32 accumulators (bias included) of one conv-like layer; x is B,H,W,C (HWC)."""
    s = L["stride"]
    if L["kind"] == "conv":
        return oracle.conv_acc(x, L["w"], L["bias"], (1, 1, 1, 1), (s, s), out_hw=(L["hout"], L["hout"]))
    if L["kind"] == "pw":
        return oracle.conv_acc(x, L["w"], L["bias"], (0, 0, 0, 0), (1, 1))
    # depthwise: one input channel per output channel -> a conv per channel; use the generic
    # oracle with k = 1, lambda = 0 is not possible (clipped), so accumulate in numpy
    xp = np.pad(x.astype(np.int32), ((0, 0), (1, 1), (1, 1), (0, 0)))
    ho = L["hout"]
    acc = np.zeros((x.shape[0], ho, ho, L["cout"]), np.int32) + L["bias"].astype(np.int32)
    for fy in range(3):
        for fx in range(3):
            acc += xp[:, fy:fy + s * ho:s, fx:fx + s * ho:s, :] * L["w"][:, fy, fx].astype(np.int32)
    return acc


def layer_forward(L, x):
    s = L["stride"]
    if L["kind"] == "conv":
        return oracle.conv(x, L["w"], L["bias"], L["k"], L["lam"], 0, L["shift"], (1, 1, 1, 1), (s, s), 1, 1, 32,
                           out_hw=(L["hout"], L["hout"]))
    if L["kind"] == "pw":
        return oracle.pointwise(x, L["w"], L["bias"], L["k"], L["lam"], 0, L["shift"], 1, 1, 32)
    chw = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    return oracle.depthwise_generic(chw, L["w"], L["bias"], L["k"], L["lam"], 0, L["shift"], (1, 1, 1, 1), (s, s), 1, 1,
                                    32, out_hw=(L["hout"], L["hout"]))


def tail_forward(net, x):
    pooled = oracle.avgpool(x, (4, 4), (4, 4))
    return oracle.linear_out_32(pooled.reshape(x.shape[0], 512), net["fc_w"], net["fc_bias"])


def forward(net, x=None, keep=False):
    cur = net["x"] if x is None else x
    outs = []
    for L in net["layers"]:
        cur = layer_forward(L, cur)
        if keep:
            outs.append(cur)
    logits = tail_forward(net, cur)
    return (logits, outs) if keep else logits
