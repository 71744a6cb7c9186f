"""Pins the oracle's requantisation epilogue (oracle_bn_quant_u8, oracle_quant_u8,
oracle_add_quant_u8, branch selection) against hand-derived known answers and
against exact-integer arithmetic on random values."""
import json
import os

import numpy as np
import pytest

import npref
import oracle

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "epilogue_kats.json")))


@pytest.mark.parametrize("v", KATS["bn"], ids=lambda v: v["why"][:40])
def test_bn_kat(v):
    assert oracle.bn_quant_u8(v["phi"], v["k"], v["lambda"], v["d"], v["bits"]) == v["out"]
    # the numpy model used elsewhere in the tests is held to the same answers
    assert int(npref.epilogue([v["phi"]], [v["k"]], [v["lambda"]], 0, v["d"], 1, 1, v["bits"])[0]) == v["out"]


@pytest.mark.parametrize("v", KATS["quant"], ids=lambda v: v["why"][:40])
def test_quant_kat(v):
    assert oracle.quant_u8(v["phi"], v["m"], v["d"]) == v["out"]
    assert int(npref.epilogue([v["phi"]], None, None, v["m"], v["d"], 1, 0)[0]) == v["out"]


@pytest.mark.parametrize("v", KATS["add"], ids=lambda v: v["why"][:40])
def test_add_kat(v):
    assert oracle.add_quant_u8(v["p1"], v["p2"], v["m1"], v["m2"], v["d"]) == v["out"]
    out = oracle.add(np.array([v["p1"]], np.uint8), np.array([v["p2"]], np.uint8), v["m1"], v["m2"], v["d"])
    assert int(out[0]) == v["out"]


@pytest.mark.parametrize("v", KATS["branch"], ids=lambda v: v["why"][:40])
def test_branch_kat(v):
    for bits in (32, 64):
        got = oracle.epilogue(v["acc"], v["k"], v["lambda"], v["mult"], v["shift"], v["relu"], v["bn"],
                              bits, bool(v["relu_eq1"]))
        assert got == v["out"]
        ref = npref.epilogue([v["acc"]], [v["k"]], [v["lambda"]], v["mult"], v["shift"], v["relu"], v["bn"],
                             bits, bool(v["relu_eq1"]))
        assert int(ref[0]) == v["out"]


def test_bn_random_against_exact_integers():
    rng = np.random.Generator(np.random.PCG64(11))
    for bits in (32, 64):
        lim = 2 ** (31 if bits == 32 else 62)
        for _ in range(3000):
            phi = int(rng.integers(-2 ** 31, 2 ** 31))
            mag = int(rng.integers(1, 31 if bits == 32 else 62))
            k = int(rng.integers(-2 ** mag, 2 ** mag))
            lam = int(rng.integers(-lim, lim))
            d = int(rng.integers(0, 32 if bits == 32 else 64))
            v = npref.wrap(k * phi + lam, bits) >> d
            if bits == 64:
                v = npref.wrap(v, 32)
            want = min(max(int(v), 0), 255)
            assert oracle.bn_quant_u8(phi, k, lam, d, bits) == want, (bits, phi, k, lam, d)


def test_quant_random_against_exact_integers():
    rng = np.random.Generator(np.random.PCG64(12))
    for _ in range(5000):
        phi = int(rng.integers(-2 ** 31, 2 ** 31)) >> int(rng.integers(0, 24))
        m = int(rng.integers(0, 65536))
        d = int(rng.integers(0, 32))
        x = npref.wrap(npref.wrap(npref.as_i16(m) * phi, 32) >> d, 16)
        assert oracle.quant_u8(phi, m, d) == min(max(int(x), 0), 255), (phi, m, d)


def test_add_random_against_exact_integers():
    rng = np.random.Generator(np.random.PCG64(13))
    for _ in range(3000):
        p1, p2 = int(rng.integers(0, 256)), int(rng.integers(0, 256))
        m1, m2 = int(rng.integers(0, 65536)), int(rng.integers(0, 65536))
        d = int(rng.integers(0, 32))
        v = (p1 * npref.as_i16(m1) + p2 * npref.as_i16(m2)) % (1 << 32)
        want = min(((v >> d) & 0xFFFF), 255)
        assert oracle.add_quant_u8(p1, p2, m1, m2, d) == want
