#!/usr/bin/env python3
"""Calibrates the per-layer out_shift of the configuration-3 network with the CPU oracle
(out_shift = floor(log2(max |acc * k|)) - 7 over the whole batch, layer by layer), writes
pulp_nn_amd/mobilenet_cfg3_shifts.json and adds the digest of the oracle's logits to
tests/golden/config_digests.json.

    python tests/golden/make_cfg3_shifts.py
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(HERE))

import oracle  # noqa: E402
from pulp_nn_amd import mobilenet  # noqa: E402
from cfg3_oracle import layer_acc, layer_forward, tail_forward  # noqa: E402


def main():
    batch = 256
    net = mobilenet.build(batch, shifts={})
    cur = net["x"]
    shifts = {}
    for L in net["layers"]:
        acc = layer_acc(L, cur).astype(np.int64)                      # B,Ho,Wo,Co incl. bias
        m = int(np.abs(acc * L["k"].astype(np.int64)).max())
        L["shift"] = shifts[L["name"]] = max(int(np.floor(np.log2(m))) - 7, 0)
        cur = layer_forward(L, cur)
        print("%-8s shift %2d  mean out %.1f" % (L["name"], L["shift"], cur.mean()), flush=True)
    logits = tail_forward(net, cur)
    json.dump({"batch": batch, "seed": mobilenet.SEED, "shifts": shifts}, open(mobilenet.SHIFTS_FILE, "w"), indent=1)
    dig = os.path.join(HERE, "config_digests.json")
    d = json.load(open(dig))
    d["cfg3_b256_logits"] = {"sha256": hashlib.sha256(np.ascontiguousarray(logits).tobytes()).hexdigest(),
                             "shape": list(logits.shape), "mean": float(logits.mean())}
    json.dump(d, open(dig, "w"), indent=1, sort_keys=True)
    print("wrote", mobilenet.SHIFTS_FILE, "and", dig)


if __name__ == "__main__":
    main()
