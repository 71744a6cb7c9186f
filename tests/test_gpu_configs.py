"""GPU parity on the five benchmark configurations at full size.

Full-size outputs are compared with SHA-256 digests of the CPU oracle's outputs
(tests/golden/config_digests.json, written by tests/golden/make_config_digests.py and
make_cfg3_shifts.py); a slice of every output is also compared element by element with
the oracle run here, so that a mismatch is located and not just detected."""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

import cfg3_oracle
import oracle
from gpu_helpers import assert_same, bn_dev, conv, depthwise_3x3_s1, depthwise_generic, dev, linear, maxpool, nn
from pulp_nn_amd import PulpNNError, mobilenet, workloads

pytestmark = pytest.mark.gpu

DIGESTS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "config_digests.json")))


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def check_digest(name, got):
    want = DIGESTS[name]
    assert list(got.shape) == want["shape"], name
    assert sha(got) == want["sha256"], "%s: digest differs (mean %.4f, oracle mean %.4f)" % (name, got.mean(), want["mean"])


@pytest.mark.parametrize("batch", [1, 256])
def test_config0_conv3x3(batch):
    c = workloads.config0(batch)
    got = conv(c["x"], c["w"], c["bias"], c["k"], c["lam"], 0, c["out_shift"], c["pads"], c["strides"], 1, 1, 32)
    n = min(batch, 4)
    assert_same(got[:n], oracle.conv(c["x"][:n], c["w"], c["bias"], c["k"], c["lam"], 0, c["out_shift"], c["pads"],
                                     c["strides"], 1, 1, 32), "config 0")
    check_digest("cfg0_b%d" % batch, got)


def test_config1_pointwise_batch256():
    c = workloads.config1(256)
    got = conv(c["x"], c["w"], c["bias"], None, None, c["out_mult"], c["out_shift"], (0, 0, 0, 0), (1, 1), 1, 0, 32,
               out_hw=(28, 28), fn="pulp_nn_pointwise_HoWo_parallel")
    assert_same(got[-3:], oracle.pointwise(c["x"][-3:], c["w"], c["bias"], None, None, c["out_mult"], c["out_shift"],
                                           1, 0, 32), "config 1")
    check_digest("cfg1_b256", got)


def test_config2_depthwise_stride1_batch256():
    c = workloads.config2(256, 1)
    xpad = np.pad(c["x"], ((0, 0), (0, 0), (1, 1), (0, 0)))
    got = depthwise_3x3_s1(xpad, c["w"], c["k"], c["lam"], 0, c["out_shift"], 1, 1, 32)
    assert_same(got[:2], oracle.depthwise_3x3_s1(xpad[:2], c["w"], c["k"], c["lam"], 0, c["out_shift"], 1, 1, 1, 1, 32),
                "config 2 stride 1")
    check_digest("cfg2_s1_b256", got)
    # the same layer through the generic entry point (no bias) must agree
    got2 = depthwise_generic(c["x"], c["w"], None, c["k"], c["lam"], 0, c["out_shift"], (1, 1, 1, 1), (1, 1), 1, 1, 32)
    assert sha(got2) == sha(got)


def test_config2_depthwise_stride2_batch256():
    c = workloads.config2(256, 2)
    got = depthwise_generic(c["x"], c["w"], c["bias"], c["k"], c["lam"], 0, c["out_shift"], (1, 1, 1, 1), (2, 2), 1, 1, 32)
    assert_same(got[:2], oracle.depthwise_generic(c["x"][:2], c["w"], c["bias"], c["k"], c["lam"], 0, c["out_shift"],
                                                  (1, 1, 1, 1), (2, 2), 1, 1, 32), "config 2 stride 2")
    check_digest("cfg2_s2_b256", got)


def test_config3_mobilenet_batch256():
    net = mobilenet.build(256)
    L = nn(32)
    x = torch.from_numpy(net["x"]).cuda()
    # two images through the oracle chain, every intermediate layer kept
    want_logits, want_layers = cfg3_oracle.forward(net, net["x"][:2], keep=True)
    # 1. every depthwise + pointwise block as one launch: 16 launches, the depthwise results never materialised
    runner = mobilenet.Runner(L, net, fuse_blocks=True, chain_blocks=False)
    got = runner.run(x)
    L.sync()
    L.set_batch(1)
    got = got.cpu().numpy()
    assert not runner.unfused_blocks, "blocks without a fused kernel: %s" % sorted(runner.unfused_blocks)
    assert runner.launches == 16, runner.launches
    for i, (Ld, w) in enumerate(zip(net["layers"], want_layers)):
        if Ld["kind"] != "dw":
            assert_same(runner.activations[i][:2].cpu().numpy(), w, "config 3 layer %s (blocks fused)" % Ld["name"])
    assert_same(got[:2], want_logits, "config 3 logits (blocks fused)")
    check_digest("cfg3_b256_logits", got)
    # 2. one launch per layer (the layout change fused into the depthwise layers): every layer compared
    runner = mobilenet.Runner(L, net, fuse_blocks=False)
    got = runner.run(x)
    L.sync()
    L.set_batch(1)
    got = got.cpu().numpy()
    assert runner.launches == 29, runner.launches
    for i, (Ld, w) in enumerate(zip(net["layers"], want_layers)):
        assert_same(runner.activations[i][:2].cpu().numpy(), w, "config 3 layer %s" % Ld["name"])
    assert_same(got[:2], want_logits, "config 3 logits")
    check_digest("cfg3_b256_logits", got)
    assert not runner.unfused, "depthwise layers without a fused kernel: %s" % sorted(runner.unfused)
    # 3. the runner's default: the five identical blocks on 8 x 8 x 256 as one launch, of the others those fused
    # that are not slower that way (one here)
    auto = mobilenet.Runner(L, net)
    got3 = auto.run(x)
    L.sync()
    L.set_batch(1)
    assert auto.launches == 19, auto.launches
    assert not auto.unchained
    check_digest("cfg3_b256_logits", got3.cpu().numpy())
    # ... and with every block fused: 12 launches
    allf = mobilenet.Runner(L, net, fuse_blocks=True)
    got4 = allf.run(x)
    L.sync()
    L.set_batch(1)
    assert allf.launches == 12, allf.launches
    check_digest("cfg3_b256_logits", got4.cpu().numpy())
    # 4. the same chain with the layout changes as separate launches (the reference's call sequence)
    plain = mobilenet.Runner(L, net, fused=False)
    got2 = plain.run(x)
    L.sync()
    L.set_batch(1)
    check_digest("cfg3_b256_logits", got2.cpu().numpy())


def test_config3_chain_in_a_hip_graph():
    """The library allocates nothing, clears nothing and queues on the stream it is given, so a
    caller can capture the whole chain in a HIP graph.  Replays, with eager work and
    synchronisations between them, must all reproduce the eager logits."""
    net = mobilenet.build(256)
    L = nn(32)
    runner = mobilenet.Runner(L, net)
    x = torch.from_numpy(net["x"]).cuda()
    eager = runner.run(x).clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        L.use_torch_stream()
        runner.run(x)
    L.use_torch_stream()
    try:
        for i in range(3):
            runner.logits.fill_(-1)
            for a in runner.activations:
                a.random_(0, 255)      # eager work between the replays; every activation is rewritten by the graph
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert bool((runner.logits == eager).all()), "replay %d differs from the eager run" % i
    finally:
        L.set_batch(1)


def test_config4_bn64_chain_batch64():
    c = workloads.config4(64, relu=1)
    y = conv(c["x"], c["w"], c["bias"], c["k"], c["lam"], 0, c["out_shift"], c["pads"], c["strides"], 1, 1, 64,
             out_hw=(63, 63))
    want1 = oracle.conv(c["x"][:1], c["w"], c["bias"], c["k"], c["lam"], 0, c["out_shift"], c["pads"], c["strides"],
                        1, 1, 64, out_hw=(63, 63))
    assert_same(y[:1], want1, "config 4 conv")
    check_digest("cfg4_b64_relu1_conv", y)
    pooled, _ = maxpool(y, (2, 2), (2, 2), (32, 32), bn_bits=64)
    check_digest("cfg4_b64_relu1_maxpool", pooled)
    # mean over the 256 channels of every pooled pixel: a pointwise conv with one output
    # channel, unit weights and out_shift 8 in the plain-shift branch
    ones = np.ones((1, 1, 1, 256), np.int8)
    means = conv(pooled, ones, None, None, None, 0, 8, (0, 0, 0, 0), (1, 1), 0, 0, 64, out_hw=(32, 32),
                 fn="pulp_nn_pointwise_HoWo_parallel")
    vec = means.reshape(64, 1024)
    check_digest("cfg4_b64_relu1_chmean", vec)
    out = linear(vec, c["lin_w"], c["lin_bias"], c["lin_k"], c["lin_lam"], 0, c["lin_shift"], 1, 1, 64)
    check_digest("cfg4_b64_relu1_linear", out)


def test_config4_literal_flags_are_rejected():
    """relu off with out_shift = 38 selects the reference's `sum >> 38` on a 32-bit int:
    undefined behaviour in C, reported as an argument error here."""
    c = workloads.config4(1, relu=0)
    with pytest.raises(PulpNNError):
        conv(c["x"], c["w"], c["bias"], c["k"], c["lam"], 0, c["out_shift"], c["pads"], c["strides"], 0, 1, 64,
             out_hw=(63, 63))
    nn(64).set_batch(1)


def test_linearity_property_at_full_size():
    """Size-independent check: with the plain-shift branch at shift 0 and inputs small enough
    not to clip, conv(x1 + x2) == conv(x1) + conv(x2) - conv(0) element-wise."""
    r = np.random.Generator(np.random.PCG64(5))
    B, H, W, Ci, Co = 64, 28, 28, 128, 256
    w = r.integers(-1, 2, size=(Co, 1, 1, Ci), dtype=np.int8)
    bias = np.full(Co, 100, np.int8)
    x1 = r.integers(0, 2, size=(B, H, W, Ci), dtype=np.uint8)
    x2 = r.integers(0, 2, size=(B, H, W, Ci), dtype=np.uint8)
    f = lambda x: conv(x, w, bias, None, None, 0, 0, (0, 0, 0, 0), (1, 1), 0, 0, 32, out_hw=(H, W),
                       fn="pulp_nn_pointwise_HoWo_parallel").astype(np.int32)
    y1, y2, y12, y0 = f(x1), f(x2), f(x1 + x2), f(np.zeros_like(x1))
    assert y12.max() < 255 and y12.min() > 0, "inputs must stay clear of the clip"
    np.testing.assert_array_equal(y12, y1 + y2 - y0)
