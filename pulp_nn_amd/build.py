"""Compiles the HIP library for gfx950: one shared object per batch-norm width.

    python -m pulp_nn_amd.build          # both libraries
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def lib_path(bn_bits):
    return os.path.join(LIBDIR, "libpulpnn_hip%d.so" % bn_bits)


def build(bn_bits, verbose=False):
    os.makedirs(LIBDIR, exist_ok=True)
    out = lib_path(bn_bits)
    cmd = [HIPCC] + FLAGS + ["-DPULPNN_BN_BITS=%d" % bn_bits, os.path.join(CSRC, "pulp_nn_hip.hip"), "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    log = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)
    return out


def build_all(verbose=False):
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(2) as ex:
        return list(ex.map(lambda b: build(b, verbose), (32, 64)))


if __name__ == "__main__":
    for p in build_all(verbose=True):
        print("built", p)
