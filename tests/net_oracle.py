"""A layer table (pulp_nn_amd/network.py format) evaluated with the CPU oracle (test infrastructure)."""
import numpy as np

import oracle


def dw_acc(x, w, bias, pads, strides, out_hw):
    """int32 accumulators of a depthwise layer on an HWC batch (numpy, zero padding)."""
    pt, pb, pl, pr = pads
    sx, sy = strides
    ky, kx = w.shape[1:3]
    Ho, Wo = out_hw
    # enough zero rows / columns for every window, whatever pad_bottom / pad_right say
    need_h, need_w = (Ho - 1) * sy + ky, (Wo - 1) * sx + kx
    xp = np.pad(x.astype(np.int32), ((0, 0), (pt, max(need_h - pt - x.shape[1], 0)),
                                     (pl, max(need_w - pl - x.shape[2], 0)), (0, 0)))
    acc = np.zeros((x.shape[0], Ho, Wo, x.shape[3]), np.int32)
    if bias is not None:
        acc += bias.astype(np.int32)
    for fy in range(ky):
        for fx in range(kx):
            acc += xp[:, fy:fy + sy * Ho:sy, fx:fx + sx * Wo:sx, :] * w[:, fy, fx].astype(np.int32)
    return acc


def layer_acc(L, x, out_hw):
    """Accumulators (bias included) of a conv-like layer; x is B,H,W,C."""
    if L["op"] == "conv":
        return oracle.conv_acc(x, L["w"], L.get("bias"), L["pads"], L["strides"], out_hw=out_hw)
    if L["op"] == "pointwise":
        return oracle.conv_acc(x, L["w"], L.get("bias"), (0, 0, 0, 0), (1, 1))
    if L["op"] == "depthwise":
        return dw_acc(x, L["w"], L.get("bias"), L["pads"], L["strides"], out_hw)
    if L["op"] == "linear":
        flat = x.reshape(x.shape[0], -1).astype(np.int64)
        acc = flat @ L["w"].astype(np.int64).T
        if L.get("bias") is not None:
            acc += L["bias"].astype(np.int64)
        return acc.astype(np.int32).reshape(x.shape[0], 1, 1, -1)
    raise ValueError(L["op"])


def absmax(L, x, out_hw):
    acc = layer_acc(L, x, out_hw).astype(np.int64)
    return int(np.abs(acc * np.asarray(L["k"], np.int64)).max())


def shift_from(m):
    return max(int(m).bit_length() - 1 - 7, 0) if m else 0


def forward(layers, shapes, x, bn_bits=32, keep=False):
    """Every layer through the oracle.  Returns the last tensor (or {name: tensor} with keep)."""
    t = {"input": x}
    for L in layers:
        op = L["op"]
        Ho, Wo, Co = shapes[L["name"]]
        q = (L.get("k"), L.get("lam"), L.get("mult", 0), L.get("shift", 0) or 0)
        fl = (L.get("relu", 0), L.get("bn", 0), bn_bits)
        if op == "add":
            t[L["name"]] = oracle.add(t[L["in"][0]], t[L["in"][1]], L["m1"], L["m2"], L["shift"])
            continue
        cur = t[L["in"]]
        if op == "conv":
            out = oracle.conv(cur, L["w"], L.get("bias"), *q, L["pads"], L["strides"], *fl, out_hw=(Ho, Wo))
        elif op == "pointwise":
            out = oracle.pointwise(cur, L["w"], L.get("bias"), *q, *fl)
        elif op == "depthwise":
            chw = np.ascontiguousarray(cur.transpose(0, 3, 1, 2))
            out = oracle.depthwise_generic(chw, L["w"], L.get("bias"), *q, L["pads"], L["strides"], *fl, out_hw=(Ho, Wo))
        elif op == "maxpool":
            out = oracle.maxpool(cur, L["kernel"], L["strides"], L.get("pads", (0, 0, 0, 0)), out_hw=(Ho, Wo))
        elif op == "avgpool":
            out = oracle.avgpool(cur, L["kernel"], L["strides"], L.get("pads", (0, 0, 0, 0)), (Ho, Wo), L.get("lam", 0),
                                 L.get("shift", 0), L.get("add", 0), L.get("requant", 0), bn_bits)
        elif op == "linear":
            out = oracle.linear(cur.reshape(cur.shape[0], -1), L["w"], L.get("bias"), *q, *fl).reshape(-1, 1, 1, Co)
        elif op == "linear_out_32":
            out = oracle.linear_out_32(cur.reshape(cur.shape[0], -1), L["w"], L.get("bias32")).reshape(-1, 1, 1, Co)
        else:
            raise ValueError(op)
        t[L["name"]] = out
    return t if keep else t[layers[-1]["name"]]
