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


TOOLS = ("mfma_ceiling", "conv_phases", "hbm_ceiling")


def tool_path(name="mfma_ceiling"):
    return os.path.join(LIBDIR, name)


def build_tool(name="mfma_ceiling", verbose=False):
    """The measurement tools: the matrix-core yardstick (csrc/mfma_ceiling.hip) and the phase / ablation trace of
    the large convolution (csrc/conv_phases.hip), the plain-copy memory yardstick (csrc/hbm_ceiling.hip).  Stand-alone executables, no part of the libraries."""
    os.makedirs(LIBDIR, exist_ok=True)
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", os.path.join(CSRC, name + ".hip"), "-o", tool_path(name)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + res.stdout)
    return tool_path(name)


def demo_path():
    return os.path.join(LIBDIR, "capi_demo")


def build_demo(verbose=False):
    """The plain C caller (csrc/capi_demo.c), compiled by gcc as C99 against include/ and linked with the 32-bit
    library: what a reference-side application's build does.  Needs libpulpnn_hip32.so to exist."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["gcc", "-std=c99", "-O2", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(os.path.dirname(HERE), "include"),
           "-I", os.path.join(rocm, "include"), os.path.join(CSRC, "capi_demo.c"), "-o", demo_path(),
           "-L", LIBDIR, "-lpulpnn_hip32", "-L", os.path.join(rocm, "lib"), "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("gcc failed:\n" + res.stdout)
    return demo_path()


def build_all(verbose=False):
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(4) as ex:
        libs = [ex.submit(build, b, verbose) for b in (32, 64)]
        tools = [ex.submit(build_tool, t, verbose) for t in TOOLS]
        out = [f.result() for f in libs] + [f.result() for f in tools]
    return out + [build_demo(verbose)]


if __name__ == "__main__":
    for p in build_all(verbose=True):
        print("built", p)
