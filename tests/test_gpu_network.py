"""GPU tests of the product-side network layer: out_shift calibration on the GPU
(pulp_nn_hip_calib_conv / pulp_nn_hip_calib_depthwise), the generic layer-table runner, a
ResNet-style block (conv -> conv -> pulp_nn_add with the block input -> pulp_nn_avgpool with
requantisation) and padded pulp_nn_maxpool, all through the C ABI and against the oracle."""
import json

import numpy as np
import pytest
import torch

import net_oracle
import oracle
from gpu_helpers import assert_same, bn_dev, dev, maxpool, nn, rand_s8, rand_u8, rng_for
from pulp_nn_amd import mobilenet, network

pytestmark = pytest.mark.gpu


def gpu_absmax(L, bn_bits, op, x, w, bias, k, geom, hwc=1):
    """(max, shift) from the calibration entry points; geom = (H, W, Ci, Ho, Wo, Co, kx, ky, pt, pl, sx, sy)."""
    H, W, Ci, Ho, Wo, Co, kx, ky, pt, pl, sx, sy = geom
    B = x.shape[0]
    nbytes = L.calib_workspace_bytes(B * Ho * Wo * Co)
    ws = torch.full((nbytes // 8 + 1,), -1, dtype=torch.int64, device="cuda")     # stale contents must not matter
    res = torch.zeros(2, dtype=torch.int64, device="cuda")
    L.set_batch(B)
    try:
        if op == "dw":
            L.calib_depthwise(dev(x), dev(bias), dev(w), bn_dev(k, bn_bits), W, H, Ci, Wo, Ho, kx, ky, pt, pl, sx, sy,
                              hwc, ws, nbytes, res)
        else:
            L.calib_conv(dev(x), dev(bias), dev(w), bn_dev(k, bn_bits), W, H, Ci, Wo, Ho, Co, kx, ky, pt, pl, sx, sy,
                         ws, nbytes, res)
        L.sync()
    finally:
        L.set_batch(1)
    m, s = (int(v) for v in res.cpu().numpy().view(np.uint64))
    return m, s


@pytest.mark.parametrize("bn_bits", [32, 64])
def test_calibration_matches_exact_integers(bn_bits):
    r = rng_for(21000 + bn_bits)
    L = nn(bn_bits)
    kmax = 2 ** 14 if bn_bits == 32 else 2 ** 30
    # conv: ragged sizes, asymmetric padding, stride 2; more than one 65536-output chunk
    for B, H, W, Ci, Co, ky, kx, pads, strides in [(3, 9, 7, 5, 6, 3, 3, (1, 1, 1, 1), (1, 1)),
                                                    (2, 11, 13, 3, 7, 3, 3, (1, 0, 1, 0), (2, 2)),
                                                    (5, 40, 40, 16, 24, 1, 1, (0, 0, 0, 0), (1, 1)),
                                                    (2, 6, 6, 64, 10, 5, 3, (2, 2, 1, 1), (1, 1))]:
        x, w, b = rand_u8(r, (B, H, W, Ci)), rand_s8(r, (Co, ky, kx, Ci)), rand_s8(r, (Co,))
        k = r.integers(-kmax, kmax, Co)
        Ld = dict(op="conv", w=w, bias=b, k=k, pads=pads, strides=strides)
        Ho, Wo = network.out_size(H, ky, strides[1], pads[0], pads[1]), network.out_size(W, kx, strides[0], pads[2], pads[3])
        want = net_oracle.absmax(Ld, x, (Ho, Wo))
        got = gpu_absmax(L, bn_bits, "conv", x, w, b, k, (H, W, Ci, Ho, Wo, Co, kx, ky, pads[0], pads[2]) + strides)
        assert got == (want, net_oracle.shift_from(want)), ("conv", got, want)
        Ld["bias"] = None
        want = net_oracle.absmax(Ld, x, (Ho, Wo))
        got = gpu_absmax(L, bn_bits, "conv", x, w, None, k, (H, W, Ci, Ho, Wo, Co, kx, ky, pads[0], pads[2]) + strides)
        assert got[0] == want
    # depthwise, both input layouts
    for B, CH, H, W, ky, kx, pads, strides in [(2, 70, 9, 11, 3, 3, (1, 1, 1, 1), (2, 2)),
                                               (3, 16, 64, 64, 3, 3, (1, 1, 1, 1), (1, 1)),
                                               (1, 3, 10, 8, 5, 5, (2, 2, 2, 2), (1, 1))]:
        x, w, b = rand_u8(r, (B, H, W, CH)), rand_s8(r, (CH, ky, kx)), rand_s8(r, (CH,))
        k = r.integers(-kmax, kmax, CH)
        Ho, Wo = network.out_size(H, ky, strides[1], pads[0], pads[1]), network.out_size(W, kx, strides[0], pads[2], pads[3])
        want = net_oracle.absmax(dict(op="depthwise", w=w, bias=b, k=k, pads=pads, strides=strides), x, (Ho, Wo))
        geom = (H, W, CH, Ho, Wo, CH, kx, ky, pads[0], pads[2]) + strides
        assert gpu_absmax(L, bn_bits, "dw", x, w, b, k, geom, hwc=1) == (want, net_oracle.shift_from(want))
        x_chw = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
        assert gpu_absmax(L, bn_bits, "dw", x_chw, w, b, k, geom, hwc=0) == (want, net_oracle.shift_from(want))
    # an all-zero layer reports shift 0
    z = np.zeros((1, 4, 4, 8), np.uint8)
    assert gpu_absmax(L, bn_bits, "conv", z, rand_s8(r, (4, 1, 1, 8)), None, np.ones(4), (4, 4, 8, 4, 4, 4, 1, 1, 0, 0, 1, 1)) == (0, 0)


def test_calibration_rejects_a_short_workspace():
    from pulp_nn_amd import PulpNNError
    L = nn(32)
    x, w, k = torch.zeros(90000, dtype=torch.uint8, device="cuda"), torch.zeros(8, dtype=torch.int8, device="cuda"), \
        torch.ones(1, dtype=torch.int32, device="cuda")
    ws, res = torch.zeros(1, dtype=torch.int64, device="cuda"), torch.full((2,), 7, dtype=torch.int64, device="cuda")
    with pytest.raises(PulpNNError):     # 300 x 300 outputs need two slots
        L.calib_conv(x, None, w, k, 300, 300, 1, 300, 300, 1, 1, 1, 0, 0, 1, 1, ws, 8, res)
    L.sync()
    assert res.tolist() == [7, 7]


def test_config3_shifts_calibrated_on_the_gpu():
    """The whole configuration-3 chain calibrated layer by layer on the GPU gives the out_shift
    table that the CPU oracle produced (pulp_nn_amd/mobilenet_cfg3_shifts.json), and with those
    shifts the logits digest."""
    import hashlib
    import os
    stored = json.load(open(mobilenet.SHIFTS_FILE))["shifts"]
    net = mobilenet.build(256, shifts={})
    assert all(Ld["shift"] is None for Ld in net["layers"])
    L = nn(32)
    runner = mobilenet.Runner(L, net)
    x = torch.from_numpy(net["x"]).cuda()
    chosen = runner.calibrate(x)
    assert chosen == stored
    logits = runner.run(x)
    L.sync()
    L.set_batch(1)
    dig = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "config_digests.json")))["cfg3_b256_logits"]
    assert hashlib.sha256(np.ascontiguousarray(logits.cpu().numpy()).tobytes()).hexdigest() == dig["sha256"]


def resnet_block(r, C=64, bn_bits=32):
    """stem conv + maxpool(3x3, stride 2, padding 1) -> [conv3x3 -> conv3x3] + skip -> avgpool (requant) -> linear."""
    kr = (256, 1025) if bn_bits == 32 else (2 ** 20, 2 ** 24)
    lr = 2 ** 16 if bn_bits == 32 else 2 ** 36

    def bnp(n):
        return dict(k=r.integers(kr[0], kr[1], n), lam=r.integers(-lr, lr + 1, n), relu=1, bn=1, shift=None)

    return [
        dict(op="conv", name="stem", **{"in": "input"}, w=rand_s8(r, (C, 3, 3, 3)), bias=rand_s8(r, (C,)),
             pads=(1, 1, 1, 1), strides=(1, 1), **bnp(C)),
        dict(op="maxpool", name="pool0", **{"in": "stem"}, kernel=(3, 3), strides=(2, 2), pads=(1, 1, 1, 1), out_hw=(16, 16)),
        dict(op="conv", name="c1", **{"in": "pool0"}, w=rand_s8(r, (C, 3, 3, C)), bias=rand_s8(r, (C,)),
             pads=(1, 1, 1, 1), strides=(1, 1), **bnp(C)),
        dict(op="conv", name="c2", **{"in": "c1"}, w=rand_s8(r, (C, 3, 3, C)), bias=rand_s8(r, (C,)),
             pads=(1, 1, 1, 1), strides=(1, 1), **bnp(C)),
        dict(op="add", name="sum", **{"in": ("c2", "pool0")}, m1=3, m2=2, shift=2),
        dict(op="avgpool", name="gap", **{"in": "sum"}, kernel=(4, 4), strides=(4, 4), out_hw=(4, 4), lam=3, shift=1, add=5,
             requant=1),
        dict(op="linear", name="fc", **{"in": "gap"}, w=rand_s8(r, (100, 4 * 4 * C)), bias=rand_s8(r, (100,)), **bnp(100)),
    ]


@pytest.mark.parametrize("bn_bits", [32, 64])
def test_resnet_style_block_batch256(bn_bits):
    r = rng_for(22000 + bn_bits)
    B = 256
    layers = resnet_block(r, 64, bn_bits)
    x = rand_u8(r, (B, 32, 32, 3))
    L = nn(bn_bits)
    runner = network.Runner(L, layers, (32, 32, 3), B)
    xd = torch.from_numpy(x).cuda()
    chosen = runner.calibrate(xd)
    assert set(chosen) == {"stem", "c1", "c2", "fc"}
    out = runner.run(xd)
    L.sync()
    L.set_batch(1)
    # the shifts the GPU chose are the ones exact integers give, layer by layer along the oracle's chain
    want = net_oracle.forward(layers, runner.shapes, x, bn_bits, keep=True)
    for Ld in layers:
        if Ld["name"] in chosen:
            m = net_oracle.absmax(Ld, want[Ld["in"]], runner.shapes[Ld["name"]][:2])
            assert chosen[Ld["name"]] == net_oracle.shift_from(m), Ld["name"]
    for Ld in layers:
        assert_same(runner.act[Ld["name"]].cpu().numpy(), want[Ld["name"]], "resnet block layer %s" % Ld["name"])
    assert want["sum"].max() > 0 and (want["sum"] < 255).any() and want["fc"].std() > 0
    assert out.data_ptr() == runner.act["fc"].data_ptr()


def test_fusion_choice_on_a_table_that_is_not_a_mobilenet():
    """The ResNet-style block with two depthwise + pointwise pairs put in front of its tail: the runner's default
    rule and the timed choice of tune() each pick one form per pair, and either way every layer equals the oracle."""
    r = rng_for(22500)
    B, C = 64, 64
    layers = resnet_block(r, C, 32)[:5]

    def bnp(n):
        return dict(k=r.integers(256, 1025, n), lam=r.integers(-2 ** 16, 2 ** 16 + 1, n), relu=1, bn=1, shift=None)

    layers += [
        dict(op="depthwise", name="dw1", **{"in": "sum"}, w=rand_s8(r, (C, 3, 3)), bias=rand_s8(r, (C,)), pads=(1, 1, 1, 1),
             strides=(1, 1), **bnp(C)),                                   # 16 x 16 planes at stride 1: 16 x 16 out
        dict(op="pointwise", name="pw1", **{"in": "dw1"}, w=rand_s8(r, (2 * C, 1, 1, C)), bias=rand_s8(r, (2 * C,)), **bnp(2 * C)),
        dict(op="depthwise", name="dw2", **{"in": "pw1"}, w=rand_s8(r, (2 * C, 3, 3)), bias=rand_s8(r, (2 * C,)),
             pads=(1, 1, 1, 1), strides=(2, 2), **bnp(2 * C)),            # 16 x 16 planes at stride 2: 8 x 8 out
        dict(op="pointwise", name="pw2", **{"in": "dw2"}, w=rand_s8(r, (2 * C, 1, 1, 2 * C)), bias=None, **bnp(2 * C)),
        dict(op="avgpool", name="gap", **{"in": "pw2"}, kernel=(4, 4), strides=(4, 4), out_hw=(2, 2), lam=3, shift=1, add=5,
             requant=1),
        dict(op="linear", name="fc", **{"in": "gap"}, w=rand_s8(r, (50, 2 * 2 * 2 * C)), bias=rand_s8(r, (50,)), **bnp(50)),
    ]
    x = rand_u8(r, (B, 32, 32, 3))
    L = nn(32)
    runner = network.Runner(L, layers, (32, 32, 3), B)
    xd = torch.from_numpy(x).cuda()
    runner.calibrate(xd)
    i1, i2 = [i for i, Ld in enumerate(layers) if Ld["op"] == "depthwise"]
    # the rule: one launch for the pair with an 8 x 8 output plane only
    assert not runner._block_fusable(i1) and runner._block_fusable(i2)
    runner.run(xd)
    L.sync()
    assert runner.launches == len(layers) - 1
    want = net_oracle.forward(layers, runner.shapes, x, 32, keep=True)
    check = [Ld["name"] for Ld in layers if Ld["name"] != "dw2"]          # dw2 is not materialised when its pair is fused
    for name in check:
        assert_same(runner.act[name].cpu().numpy(), want[name], "rule-based path, layer %s" % name)
    # the timed choice: whatever it picks, the results stay those of the oracle
    chosen = runner.tune(xd)
    assert set(chosen) == {"dw1", "dw2"} and all(isinstance(v, bool) for v in chosen.values())
    for Ld in layers:
        runner.act[Ld["name"]].zero_()
    runner.run(xd)
    L.sync()
    L.set_batch(1)
    assert runner.launches == len(layers) - sum(chosen.values())
    for Ld in layers:
        fused_away = Ld["op"] == "depthwise" and chosen[Ld["name"]]
        if not fused_away:
            assert_same(runner.act[Ld["name"]].cpu().numpy(), want[Ld["name"]], "timed path, layer %s" % Ld["name"])


@pytest.mark.parametrize("case", [
    # B, H, W, C, kernel(kx,ky), strides(sx,sy), pads(t,b,l,r), out_hw
    (2, 32, 32, 64, (3, 3), (2, 2), (1, 1, 1, 1), (16, 16)),     # ResNet stem pooling
    (3, 9, 11, 3, (3, 3), (2, 2), (1, 1, 1, 1), (5, 6)),          # odd sizes, byte path
    (2, 63, 63, 16, (3, 3), (2, 2), (1, 0, 1, 0), (32, 32)),
    (1, 7, 7, 20, (2, 3), (2, 2), (1, 1, 1, 1), (4, 4)),          # kx != ky
    (2, 8, 8, 16, (5, 5), (3, 3), (2, 2, 2, 2), (3, 3)),          # padding 2 with stride 3
])
def test_maxpool_padded(case):
    B, H, W, Cc, kernel, strides, pads, out_hw = case
    r = rng_for(23000 + H)
    x = rand_u8(r, (B, H, W, Cc))
    got, xin_after = maxpool(x, kernel, strides, out_hw, pads)
    assert_same(got, oracle.maxpool(x, kernel, strides, pads, out_hw=out_hw), "padded maxpool")
    assert_same(xin_after, x, "maxpool input must stay intact")
