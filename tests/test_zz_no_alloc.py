"""The allocation-free calibration entry point (pulp_nn_hip_calib_conv_static) against the
workspace one and against the exact integers of the layer's accumulators, through the C ABI:
two calls in a row, the second on a smaller input; and the device's free memory does not move
across such a call."""
import numpy as np
import pytest
import torch

import net_oracle
from gpu_helpers import bn_dev, dev, nn, rand_s8, rand_u8, rng_for

pytestmark = pytest.mark.gpu


def both(L, bn_bits, x, w, b, k, geom):
    H, W, Ci, Ho, Wo, Co, kx, ky, pt, pl, sx, sy = geom
    B = x.shape[0]
    xd, wd, bd, kd = dev(x), dev(w), dev(b), bn_dev(k, bn_bits)
    nbytes = L.calib_workspace_bytes(B * Ho * Wo * Co)
    ws = torch.zeros(nbytes // 8 + 1, dtype=torch.int64, device="cuda")
    res_ws = torch.zeros(2, dtype=torch.int64, device="cuda")
    res_st = torch.full((2,), -1, dtype=torch.int64, device="cuda")
    L.set_batch(B)
    try:
        L.calib_conv(xd, bd, wd, kd, W, H, Ci, Wo, Ho, Co, kx, ky, pt, pl, sx, sy, ws, nbytes, res_ws)
        L.calib_conv_static(xd, bd, wd, kd, W, H, Ci, Wo, Ho, Co, kx, ky, pt, pl, sx, sy, res_st)
        L.sync()
    finally:
        L.set_batch(1)
    return res_ws.cpu().numpy(), res_st.cpu().numpy()


@pytest.mark.parametrize("bn_bits", [32, 64])
def test_static_scratch_calibration_matches_workspace_calibration(bn_bits):
    r = rng_for(24000 + bn_bits)
    L = nn(bn_bits)
    # first call: 20 * 48 * 48 * 32 = 1.47 M outputs (23 slots); second: 3 * 9 * 7 * 6 = 1134 outputs (1 slot),
    # so stale partial maxima of the first call sit in the scratch array during the second
    cases = [(20, 48, 48, 16, 32, 3, 3, 1, 1, 1, 1), (3, 9, 7, 5, 6, 3, 3, 1, 1, 1, 1)]
    results = []
    for B, H, W, Ci, Co, ky, kx, pt, pl, sx, sy in cases:
        x, w, b = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, ky, kx, Ci)), rand_s8(r, (Co,))
        if B == 3:
            x //= 16                  # the smaller layer also has the smaller maximum
        k = r.integers(256, 1025, Co)
        a, s = both(L, bn_bits, x, w, b, k, (H, W, Ci, H, W, Co, kx, ky, pt, pl, sx, sy))
        np.testing.assert_array_equal(s, a)
        assert a[0] > 0
        # the static path against the layer's accumulators in exact integers (numpy)
        layer = dict(op="conv", w=w, bias=b, k=k, pads=(pt, pt, pl, pl), strides=(sx, sy))
        want = net_oracle.absmax(layer, x, (H, W))
        assert int(s[0]) == want and int(s[1]) == net_oracle.shift_from(want)
        results.append(int(a[0]))
    assert results[1] < results[0]


def test_static_scratch_calibration_allocates_nothing():
    r = rng_for(24100)
    L = nn(32)
    B, H, W, Ci, Co = 6, 20, 20, 8, 16
    x, w, b = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, 3, 3, Ci)), rand_s8(r, (Co,))
    xd, wd, bd, kd = dev(x), dev(w), dev(b), bn_dev(r.integers(256, 1025, Co), 32)
    res = torch.zeros(2, dtype=torch.int64, device="cuda")
    L.set_batch(B)
    try:
        L.calib_conv_static(xd, bd, wd, kd, W, H, Ci, W, H, Co, 3, 3, 1, 1, 1, 1, res)   # first call on this device: looks the array up
        L.sync()
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        for _ in range(3):
            L.calib_conv_static(xd, bd, wd, kd, W, H, Ci, W, H, Co, 3, 3, 1, 1, 1, 1, res)
        L.sync()
        assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the device's free memory"
    finally:
        L.set_batch(1)
    assert int(res[0]) > 0


def test_static_scratch_calibration_rejects_a_layer_beyond_its_slots():
    from pulp_nn_amd import PulpNNError
    L = nn(32)
    x = torch.zeros(16, dtype=torch.uint8, device="cuda")
    w = torch.zeros(16, dtype=torch.int8, device="cuda")
    k = torch.ones(1, dtype=torch.int32, device="cuda")
    res = torch.full((2,), 7, dtype=torch.int64, device="cuda")
    L.set_batch(2 ** 31 - 1)          # 2^31 - 1 images x 1 output: more than 8192 slots of 65536 outputs
    try:
        with pytest.raises(PulpNNError) as ei:
            L.calib_conv_static(x, None, w, k, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0, 1, 1, res)
        assert ei.value.code == 1
    finally:
        L.set_batch(1)
    L.sync()
    assert res.tolist() == [7, 7]
