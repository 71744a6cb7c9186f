"""GPU parity of pulp_nn_hip_dw_pw_hwc (3x3 depthwise + pointwise in one launch) against the oracle's
two-layer chain: depthwise_generic (on the CHW view of the HWC input) followed by pointwise."""
import numpy as np
import pytest
import torch

import oracle
from gpu_helpers import bn_dev, dev, nn, rand_s8, rand_u8, rng_for
from pulp_nn_amd import PulpNNError

pytestmark = pytest.mark.gpu

# B, H, W, C, Co, stride: every geometry variant of the kernel, channel counts below / at / above one 64-channel
# group, channel counts that are not a multiple of 64, batches that leave the last tile partly empty
GEOMS = [
    (5, 64, 64, 16, 32, 1),
    (3, 64, 64, 32, 64, 2),
    (3, 32, 64, 64, 48, 1),      # H != W
    (6, 32, 32, 64, 64, 1),
    (5, 32, 32, 64, 128, 2),
    (7, 16, 16, 128, 128, 1),
    (9, 16, 16, 128, 256, 2),
    (11, 8, 8, 256, 256, 1),
    (13, 8, 8, 256, 512, 2),
    (10, 4, 4, 512, 512, 1),
    (4, 16, 16, 192, 80, 1),     # three channel groups, output channels not a multiple of 64
    (300, 8, 8, 64, 16, 1),      # many small images, a single 16-channel output group
    (9, 8, 16, 320, 96, 2),      # H = 8, W = 16, five K slices (two passes over the weights)
    (4, 8, 8, 64, 2048, 1),      # 2048 output channels: legal because so few images are split over workgroups by channels
]
FLAGS = [((1, 1), (1, 1)), ((1, 0), (1, 1)), ((1, 1), (1, 0)), ((0, 0), (0, 0)), ((2, 0), (0, 1))]


def fused(x, dw, pw, stride, bn_bits):
    B, H, W, C = x.shape
    Co = pw["w"].shape[0]
    Ho, Wo = (H - 1) // stride + 1, (W - 1) // stride + 1
    L = nn(bn_bits)
    out = torch.full((B, Ho, Wo, Co), 0xA5, dtype=torch.uint8, device="cuda")
    L.set_batch(B)
    try:
        L.dw_pw_hwc(dev(x), out, W, H, C, Wo, Ho, Co, stride, dev(dw["w"]), dev(dw["bias"]), bn_dev(dw["k"], bn_bits),
                    bn_dev(dw["lam"], bn_bits), dw["mult"], dw["shift"], dw["relu"], dw["bn"], dev(pw["w"]), dev(pw["bias"]),
                    bn_dev(pw["k"], bn_bits), bn_dev(pw["lam"], bn_bits), pw["mult"], pw["shift"], pw["relu"], pw["bn"])
        L.sync()
    finally:
        L.set_batch(1)
    return out.cpu().numpy()


def layer_params(r, ch, flags, bn_bits):
    relu, bn = flags
    if bn_bits == 64:
        k, lam = r.integers(2 ** 20, 2 ** 24, ch), r.integers(-2 ** 36, 2 ** 36, ch)
    else:
        k, lam = r.integers(256, 1025, ch), r.integers(-2 ** 16, 2 ** 16, ch)
    return dict(k=k, lam=lam, mult=int(r.integers(256, 1025)), relu=relu, bn=bn)


def pick_shift(P, acc_absmax):
    """out_shift that brings the layer's largest value to about 2^8 (the calibration rule of the chain)."""
    if P["relu"] and P["bn"]:
        top = acc_absmax * int(np.abs(P["k"]).max())
    elif P["relu"]:
        top = acc_absmax * P["mult"]
    else:
        top = acc_absmax
    return max(int(np.log2(max(top, 1))) - 7, 0)


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", FLAGS, ids=lambda f: "dw%d%d_pw%d%d" % (f[0] + f[1]))
@pytest.mark.parametrize("geom", GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_fused_block(geom, flags, bn_bits):
    B, H, W, C, Co, stride = geom
    r = rng_for(31337 + bn_bits + 7 * flags[0][0] + flags[1][1])
    x = rand_u8(r, (B, H, W, C))
    dw = dict(w=rand_s8(r, (C, 3, 3)), bias=rand_s8(r, (C,)), **layer_params(r, C, flags[0], bn_bits))
    pw = dict(w=rand_s8(r, (Co, 1, 1, C)), bias=rand_s8(r, (Co,)) if flags[1][0] else None,
              **layer_params(r, Co, flags[1], bn_bits))
    sample = sorted({0, B // 2, B - 1})
    # shifts from the layers' own accumulators on the sample (numpy), so that both layers produce real values
    dw["shift"] = pick_shift(dw, int(9 ** 0.5 * 128 * 74 * 2))
    xc = np.ascontiguousarray(x[sample].transpose(0, 3, 1, 2))
    mid = oracle.depthwise_generic(xc, dw["w"], dw["bias"], dw["k"], dw["lam"], dw["mult"], dw["shift"], (1, 1, 1, 1),
                                   (stride, stride), dw["relu"], dw["bn"], bn_bits)
    acc = mid.reshape(-1, C).astype(np.int64) @ pw["w"].reshape(Co, C).astype(np.int64).T
    pw["shift"] = pick_shift(pw, int(np.abs(acc).max()))
    got = fused(x, dw, pw, stride, bn_bits)
    # the oracle chain on the sample: depthwise (CHW in, HWC out), then pointwise
    want = oracle.pointwise(mid, pw["w"], pw["bias"], pw["k"], pw["lam"], pw["mult"], pw["shift"], pw["relu"], pw["bn"], bn_bits)
    assert got.shape[1:] == want.shape[1:]
    assert np.array_equal(got[sample], want), "fused block differs from the two-layer oracle chain"
    assert mid.max() > 0 and (mid < 255).any() and want.max() > 0 and (want < 255).any(), "degenerate case"


def test_fused_block_rejects_what_it_cannot_do():
    L = nn(32)
    x = torch.zeros((1, 12, 12, 64), dtype=torch.uint8, device="cuda")      # width 12: no kernel
    out = torch.zeros((1, 12, 12, 64), dtype=torch.uint8, device="cuda")
    w9 = torch.zeros((64, 9), dtype=torch.int8, device="cuda")
    pw = torch.zeros((64, 64), dtype=torch.int8, device="cuda")
    with pytest.raises(PulpNNError) as err:
        L.dw_pw_hwc(x, out, 12, 12, 64, 12, 12, 64, 1, w9, None, None, None, 300, 15, 1, 0, pw, None, None, None, 300, 15, 1, 0)
    assert err.value.code == 2
    with pytest.raises(PulpNNError):                                           # wrong output size
        L.dw_pw_hwc(x, out, 16, 16, 64, 15, 16, 64, 1, w9, None, None, None, 300, 15, 1, 0, pw, None, None, None, 300, 15, 1, 0)
    # more than 1024 output channels in one workgroup: a batch large enough that the tiles are not split by channels
    B = 1024
    xb = torch.zeros((B, 8, 8, 64), dtype=torch.uint8, device="cuda")
    ob = torch.zeros((B, 8, 8, 2048), dtype=torch.uint8, device="cuda")
    pwb = torch.zeros((2048, 64), dtype=torch.int8, device="cuda")
    L.set_batch(B)
    try:
        with pytest.raises(PulpNNError) as err:
            L.dw_pw_hwc(xb, ob, 8, 8, 64, 8, 8, 2048, 1, w9, None, None, None, 300, 15, 1, 0, pwb, None, None, None, 300, 15, 1, 0)
        assert err.value.code == 2
    finally:
        L.set_batch(1)


# ---- several blocks of one shape in one launch (pulp_nn_hip_dw_pw_chain_hwc) --------------------------------------
# B, H, W, C, number of blocks.  Whole images per workgroup: 8 x 8 x 256 (one image), 4 x 4 x 512 (two images, so
# an even batch), 16 x 16 x 64 (one image), 8 x 8 x 64 with 16-channel-multiple counts
CHAINS = [
    (7, 8, 8, 256, 5),       # the run of five identical blocks of the MobileNet chain
    (6, 4, 4, 512, 3),
    (5, 16, 16, 64, 2),
    (4, 8, 8, 128, 8),       # the most blocks one launch takes
    (9, 8, 8, 64, 1),        # a single block through the chain entry point
]


@pytest.mark.parametrize("bn_bits", [32, 64])
@pytest.mark.parametrize("flags", [((1, 1), (1, 1)), ((1, 0), (1, 1)), ((1, 1), (1, 0))], ids=lambda f: "dw%d%d_pw%d%d" % (f[0] + f[1]))
@pytest.mark.parametrize("geom", CHAINS, ids=lambda g: "x".join(map(str, g)))
def test_block_chain(geom, flags, bn_bits):
    B, H, W, C, nb = geom
    r = rng_for(4711 + bn_bits + 5 * flags[0][1] + flags[1][1] + nb)
    x = rand_u8(r, (B, H, W, C))
    cur = x
    blocks, keep = [], []
    for j in range(nb):
        dw = dict(w=rand_s8(r, (C, 3, 3)), bias=rand_s8(r, (C,)) if j % 2 == 0 else None, **layer_params(r, C, flags[0], bn_bits))
        pw = dict(w=rand_s8(r, (C, 1, 1, C)), bias=rand_s8(r, (C,)) if j % 2 else None, **layer_params(r, C, flags[1], bn_bits))
        # shifts from the layers' own accumulators (the oracle walks the chain), so that every layer produces real values
        dw["shift"] = pick_shift(dw, int(9 ** 0.5 * 128 * 74 * 2))
        mid = oracle.depthwise_generic(np.ascontiguousarray(cur.transpose(0, 3, 1, 2)), dw["w"], dw["bias"], dw["k"], dw["lam"],
                                       dw["mult"], dw["shift"], (1, 1, 1, 1), (1, 1), dw["relu"], dw["bn"], bn_bits)
        acc = mid.reshape(-1, C).astype(np.int64) @ pw["w"].reshape(C, C).astype(np.int64).T
        pw["shift"] = pick_shift(pw, int(np.abs(acc).max()))
        cur = oracle.pointwise(mid, pw["w"], pw["bias"], pw["k"], pw["lam"], pw["mult"], pw["shift"], pw["relu"], pw["bn"], bn_bits)
        assert cur.max() > 0 and (cur < 255).any(), "degenerate block %d" % j
        dev_args = (dev(dw["w"]), dev(dw["bias"]), bn_dev(dw["k"], bn_bits), bn_dev(dw["lam"], bn_bits), dw["mult"], dw["shift"],
                    dw["relu"], dw["bn"], dev(pw["w"]), dev(pw["bias"]), bn_dev(pw["k"], bn_bits), bn_dev(pw["lam"], bn_bits),
                    pw["mult"], pw["shift"], pw["relu"], pw["bn"])
        keep.append(dev_args)
        blocks.append(dev_args)
    L = nn(bn_bits)
    out = torch.full((B, H, W, C), 0xA5, dtype=torch.uint8, device="cuda")
    L.set_batch(B)
    try:
        L.dw_pw_chain_hwc(dev(x), out, W, H, C, blocks)
        L.sync()
    finally:
        L.set_batch(1)
    assert np.array_equal(out.cpu().numpy(), cur), "chain of %d blocks differs from the oracle's 2 x %d layers" % (nb, nb)


def test_block_chain_rejects_what_it_cannot_do():
    L = nn(32)
    z = lambda *s: torch.zeros(s, dtype=torch.int8, device="cuda")
    blk = lambda C: (z(C, 9), None, None, None, 300, 15, 1, 0, z(C, C), None, None, None, 300, 15, 1, 0)
    x = torch.zeros((3, 4, 4, 512), dtype=torch.uint8, device="cuda")
    L.set_batch(3)                      # two 4 x 4 images per workgroup: an odd batch cannot be chained
    try:
        with pytest.raises(PulpNNError) as err:
            L.dw_pw_chain_hwc(x, torch.zeros_like(x), 4, 4, 512, [blk(512)] * 2)
        assert err.value.code == 2
        x = torch.zeros((3, 32, 32, 64), dtype=torch.uint8, device="cuda")   # 32 x 32 x 64 x 2 bytes: too large for LDS
        with pytest.raises(PulpNNError) as err:
            L.dw_pw_chain_hwc(x, torch.zeros_like(x), 32, 32, 64, [blk(64)] * 2)
        assert err.value.code == 2
        with pytest.raises(PulpNNError) as err:                                 # more blocks than one launch takes
            L.dw_pw_chain_hwc(x, torch.zeros_like(x), 32, 32, 64, [blk(64)] * 9)
        assert err.value.code == 1
    finally:
        L.set_batch(1)
