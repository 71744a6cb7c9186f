#!/usr/bin/env python3
"""Writes config_digests.json: SHA-256 of the CPU oracle's outputs on the benchmark
configurations at full size (minutes of CPU work, done once here so that the GPU
tests can check full-size outputs by digest).

    python tests/golden/make_config_digests.py

The inputs are the seeded tensors of pulp_nn_amd/workloads.py; the digests cover
the raw bytes of each output tensor in C order.
"""
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from pulp_nn_amd import workloads  # noqa: E402


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def config4_chain(c4, conv_out):
    """maxpool 2x2 s2 (63 -> 32, ceil mode through the window clamp), mean over the 256
    channels of every pooled pixel as a 1-output-channel pointwise conv with unit weights
    and out_shift 8, then the 1024 -> 4096 linear layer with 64-bit batch-norm."""
    pooled = oracle.maxpool(conv_out, (2, 2), (2, 2), out_hw=(32, 32))
    ones = np.ones((1, 256), np.int8)
    means = oracle.pointwise(pooled, ones, None, None, None, 0, 8, 0, 0, 64)       # B,32,32,1
    vec = means.reshape(means.shape[0], 1024)
    lin = oracle.linear(vec, c4["lin_w"], c4["lin_bias"], c4["lin_k"], c4["lin_lam"], 0, c4["lin_shift"], 1, 1, 64)
    return pooled, vec, lin


def main():
    out = {}
    t0 = time.time()
    for batch in (1, 256):
        c = workloads.config0(batch)
        y = oracle.conv(c["x"], c["w"], c["bias"], c["k"], c["lam"], 0, c["out_shift"], c["pads"], c["strides"], 1, 1, 32)
        out["cfg0_b%d" % batch] = {"sha256": sha(y), "shape": list(y.shape), "mean": float(y.mean())}
    c = workloads.config1(256)
    y = oracle.pointwise(c["x"], c["w"], c["bias"], None, None, c["out_mult"], c["out_shift"], 1, 0, 32)
    out["cfg1_b256"] = {"sha256": sha(y), "shape": list(y.shape), "mean": float(y.mean())}
    c = workloads.config2(256, 1)
    xpad = np.pad(c["x"], ((0, 0), (0, 0), (1, 1), (0, 0)))
    y = oracle.depthwise_3x3_s1(xpad, c["w"], c["k"], c["lam"], 0, c["out_shift"], 1, 1, 1, 1, 32)
    out["cfg2_s1_b256"] = {"sha256": sha(y), "shape": list(y.shape), "mean": float(y.mean())}
    c = workloads.config2(256, 2)
    y = oracle.depthwise_generic(c["x"], c["w"], c["bias"], c["k"], c["lam"], 0, c["out_shift"], (1, 1, 1, 1), (2, 2),
                                 1, 1, 32)
    out["cfg2_s2_b256"] = {"sha256": sha(y), "shape": list(y.shape), "mean": float(y.mean())}
    print("configs 0-2 done in %.0f s" % (time.time() - t0), flush=True)
    # flag_relu = 0 is not digested: with out_shift = 38 the reference's raw branch is
    # `sum >> 38` on a 32-bit int, undefined behaviour in C; the HIP library rejects it.
    for relu in (1,):
        c = workloads.config4(64, relu)
        y = oracle.conv(c["x"], c["w"], c["bias"], c["k"], c["lam"], 0, c["out_shift"], c["pads"], c["strides"],
                        relu, 1, 64, out_hw=(63, 63))
        tag = "cfg4_b64_relu%d" % relu
        out[tag + "_conv"] = {"sha256": sha(y), "shape": list(y.shape), "mean": float(y.mean())}
        if relu:
            pooled, vec, lin = config4_chain(c, y)
            out[tag + "_maxpool"] = {"sha256": sha(pooled), "shape": list(pooled.shape), "mean": float(pooled.mean())}
            out[tag + "_chmean"] = {"sha256": sha(vec), "shape": list(vec.shape), "mean": float(vec.mean())}
            out[tag + "_linear"] = {"sha256": sha(lin), "shape": list(lin.shape), "mean": float(lin.mean())}
        print(tag, "done at %.0f s" % (time.time() - t0), flush=True)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config_digests.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print("wrote", path)


if __name__ == "__main__":
    main()
