"""CPU-only checks of the C-ABI boundary: both libraries load and export every entry point
that include/*.h declares; the headers compile as C; no compute is attempted without a GPU."""
import ctypes
import os
import re
import subprocess

import pytest

from pulp_nn_amd import build as hip_build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INC = os.path.join(ROOT, "include")


def declared_symbols():
    names = set()
    for fn in ("pulp_nn_kernels_decl.h", "pulp_nn_hip.h"):
        text = open(os.path.join(INC, fn)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(pulp_nn_[A-Za-z0-9_]+)\s*\(", text))
    return sorted(names)


@pytest.fixture(scope="module")
def libs():
    out = {}
    for bits in (32, 64):
        path = hip_build.lib_path(bits)
        if not os.path.exists(path):
            hip_build.build(bits)
        out[bits] = ctypes.CDLL(path)
    return out


def test_header_declares_the_reference_api():
    names = declared_symbols()
    for n in ("pulp_nn_add", "pulp_nn_avgpool", "pulp_nn_conv_Ho_parallel", "pulp_nn_conv_Co_parallel",
              "pulp_nn_conv_HoWo_parallel", "pulp_nn_pointwise_HoWo_parallel", "pulp_nn_pointwise_Ho_parallel",
              "pulp_nn_pointwise_Co_parallel", "pulp_nn_linear", "pulp_nn_linear_out_32", "pulp_nn_matmul",
              "pulp_nn_maxpool", "pulp_nn_depthwise_generic", "pulp_nn_depthwise_generic_less_4_weights",
              "pulp_nn_depthwise_3x3_s1", "pulp_nn_hip_set_batch"):
        assert n in names, n


@pytest.mark.parametrize("bits", [32, 64])
def test_library_exports_every_declared_symbol(libs, bits):
    lib = libs[bits]
    for name in declared_symbols():
        assert hasattr(lib, name), "%s missing from libpulpnn_hip%d.so" % (name, bits)
    lib.pulp_nn_hip_bn_bits.restype = ctypes.c_int
    assert lib.pulp_nn_hip_bn_bits() == bits


@pytest.mark.parametrize("bits", [32, 64])
def test_host_state_without_gpu(libs, bits):
    lib = libs[bits]
    lib.pulp_nn_hip_get_batch.restype = ctypes.c_uint
    lib.pulp_nn_hip_set_batch(7)
    assert lib.pulp_nn_hip_get_batch() == 7
    lib.pulp_nn_hip_set_batch(0)          # 0 is treated as 1
    assert lib.pulp_nn_hip_get_batch() == 1
    lib.pulp_nn_hip_last_error.restype = ctypes.c_int
    lib.pulp_nn_hip_clear_error()
    assert lib.pulp_nn_hip_last_error() == 0
    # argument validation happens before any GPU work: a null pointer is reported, not launched
    lib.pulp_nn_add.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_uint16] * 6
    lib.pulp_nn_add(None, None, None, 1, 1, 1, 2, 2, 2)
    assert lib.pulp_nn_hip_last_error() == 1
    lib.pulp_nn_hip_last_error_string.restype = ctypes.c_char_p
    assert b"pulp_nn_add" in lib.pulp_nn_hip_last_error_string()
    lib.pulp_nn_hip_clear_error()


@pytest.mark.parametrize("bits", [32, 64])
def test_headers_compile_as_c(tmp_path, bits):
    src = tmp_path / "t.c"
    src.write_text('#include "%dbit/pulp_nn_kernels.h"\nint main(void) { return pulp_nn_hip_bn_bits() == %d ? 0 : 1; }\n'
                   % (bits, bits))
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", INC, "-c", str(src), "-o", str(tmp_path / "t.o")])


def test_python_front_end_refuses_to_run_without_the_library(monkeypatch):
    import pulp_nn_amd.api as api
    monkeypatch.setattr(api, "lib_path", lambda bits: "/nonexistent/libpulpnn_hip%d.so" % bits)
    with pytest.raises(ImportError):
        api.PulpNN(32)
