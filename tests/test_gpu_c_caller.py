"""The library called from plain C (pulp_nn_amd/csrc/capi_demo.c, compiled by gcc as C99 against include/): the
call sequence of a PULP-NN application -- pointwise layer, layout change, 3x3 depthwise layer -- with device
buffers from the HIP runtime.  The program runs as a child process; its two outputs are compared byte for byte
with the CPU oracle's."""
import os
import subprocess

import numpy as np
import pytest

import oracle
from gpu_helpers import rand_s8, rand_u8, rng_for
from pulp_nn_amd import build as hip_build

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("geom", [(3, 12, 20, 24, 64), (130, 28, 28, 32, 64)], ids=lambda g: "x".join(map(str, g)))
def test_c_program_matches_oracle(tmp_path, geom):
    exe = hip_build.demo_path()
    assert os.path.exists(exe), "build the C caller first: python -m pulp_nn_amd.build"
    B, H, W, Ci, Co = geom
    r = rng_for(606 + B)
    x, w, bias = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, Ci)), rand_s8(r, (Co,))
    dw_w = rand_s8(r, (Co, 3, 3))
    k = r.integers(2 ** 12, 2 ** 14, Co).astype(np.int32)
    lam = r.integers(-2 ** 16, 2 ** 16, Co).astype(np.int32)
    pw_mult, pw_shift, dw_shift = 700, 20, 16
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(fin, "wb") as f:
        f.write(np.array([B, H, W, Ci, Co, pw_mult, pw_shift, dw_shift], dtype=np.int32).tobytes())
        for a in (x, w, bias, dw_w, k, lam):
            f.write(np.ascontiguousarray(a).tobytes())
    res = subprocess.run([exe, str(fin), str(fout)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert res.returncode == 0, res.stdout
    got = np.fromfile(fout, dtype=np.uint8)
    n = B * H * W * Co
    got_pw, got_dw = got[:n].reshape(B, H, W, Co), got[n:].reshape(B, H, W, Co)
    want_pw = oracle.pointwise(x, w, bias, None, None, pw_mult, pw_shift, 1, 0)
    assert np.array_equal(got_pw, want_pw), "pointwise from C"
    want_dw = oracle.depthwise_generic(np.ascontiguousarray(want_pw.transpose(0, 3, 1, 2)), dw_w, None, k, lam, 0, dw_shift,
                                       (1, 1, 1, 1), (1, 1), 1, 1)
    assert np.array_equal(got_dw, want_dw), "depthwise from C"
    assert want_pw.max() > 0 and (want_pw < 255).any() and want_dw.max() > 0 and (want_dw < 255).any(), "degenerate case"
