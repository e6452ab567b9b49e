"""Pins for the oracle's constant tables and 16-bit conversions.

Sources of truth that are independent of the oracle's own code:
  * the reference's literals (tests/golden/tq4_tables.json, extracted from
    csrc/tq/tq4_codebook.cuh:46-101 by tests/golden/make_table_fixture.py);
  * the mathematics: the centroids are the Lloyd-Max fixed point of the coordinate density
    of a uniformly random unit vector in R^256, f(x) ~ (1-x^2)^((256-3)/2)
    (tq4_codebook.cuh:1-5,45), boundaries are midpoints of adjacent centroids;
  * numpy's IEEE fp16 conversions for the scalar converters
    (crates/warp34-host/src/cuda/tests.rs:3-71 tests the same property exhaustively).
"""
import json
import os

import numpy as np
from scipy import integrate

import oracle

HERE = os.path.dirname(os.path.abspath(__file__))
FIX = json.load(open(os.path.join(HERE, "golden", "tq4_tables.json")))


def test_tables_equal_reference_literals():
    c = np.array([np.float32(s) for s in FIX["d256_centroids"]], dtype=np.float32)
    b = np.array([np.float32(s) for s in FIX["d256_boundaries"]], dtype=np.float32)
    assert oracle.centroids().tobytes() == c.tobytes()
    assert oracle.boundaries().tobytes() == b.tobytes()
    s = np.array(FIX["signs256"], dtype=np.float32)
    assert oracle.signs().tobytes() == s.tobytes()


def test_sign_fingerprint():
    s = oracle.signs()
    assert set(np.unique(s)) == {-1.0, 1.0}
    assert int((s < 0).sum()) == 134 == FIX["signs256_negative_count"]
    mask = 0
    for i, v in enumerate(s):
        if v < 0:
            mask |= 1 << i
    assert "%064x" % mask == FIX["signs256_negative_mask_hex"]
    assert "%064x" % mask == "36b5bda1fde0ee14e2eb25d0ba639274f1297e2aeebc0de44897475229e1d357"


def test_codebook_antisymmetric_and_midpoints():
    c, b = oracle.centroids().astype(np.float64), oracle.boundaries().astype(np.float64)
    assert np.all(np.diff(c) > 0) and np.all(np.diff(b) > 0)
    assert np.array_equal(c, -c[::-1])
    assert np.array_equal(b, -b[::-1]) and b[7] == 0.0
    assert np.max(np.abs(b - 0.5 * (c[:-1] + c[1:]))) < 1e-8


def test_codebook_is_lloyd_max_fixed_point_of_beta256():
    """centroid_k == E[x | b_{k-1} < x <= b_k] under f(x) ~ (1-x^2)^(253/2)."""
    c, b = oracle.centroids().astype(np.float64), oracle.boundaries().astype(np.float64)
    f = lambda x: (1.0 - x * x) ** ((256 - 3) / 2.0)
    edges = np.concatenate([[-1.0], b, [1.0]])
    total = 0.0
    mse = 0.0
    for k in range(16):
        m0 = integrate.quad(f, edges[k], edges[k + 1], epsabs=1e-14, epsrel=1e-12)[0]
        m1 = integrate.quad(lambda x: x * f(x), edges[k], edges[k + 1], epsabs=1e-14, epsrel=1e-12)[0]
        assert abs(m1 / m0 - c[k]) < 5e-7, (k, m1 / m0, c[k])
        mse += integrate.quad(lambda x: (x - c[k]) ** 2 * f(x), edges[k], edges[k + 1],
                              epsabs=1e-16, epsrel=1e-12)[0]
        total += m0
    # header comment: d * C(f,4) = 0.009408 for d = 256 (tq4_codebook.cuh:45)
    assert abs(256 * mse / total - 0.009408) < 2e-6


def test_f16_converters_match_ieee_exhaustively():
    L = oracle.lib()
    allbits = np.arange(65536, dtype=np.uint16)
    ref = allbits.view(np.float16).astype(np.float32)
    got = np.array([L.tq4o_f16_to_f32(int(h)) for h in allbits], dtype=np.float32)
    fin = np.isfinite(ref)
    assert got[fin].tobytes() == ref[fin].tobytes()
    assert np.all(np.isnan(got[np.isnan(ref)]))
    # f32 -> f16: every finite half round-trips, plus midpoints / overflow / subnormal ties
    back = np.array([L.tq4o_f32_to_f16(float(v)) for v in ref[fin]], dtype=np.uint16)
    assert np.array_equal(back, allbits[fin])
    rng = np.random.default_rng(1)
    probes = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([65504.0, 65519.99, 65520.0, 1e6, -1e6, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)),
                  2.0 ** -24, 1.5 * 2.0 ** -24, 2.5 * 2.0 ** -24, 2.0 ** -14, 0.0, -0.0, 6.1e-5], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        want = probes.astype(np.float16).view(np.uint16)
    got = np.array([L.tq4o_f32_to_f16(float(v)) for v in probes], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16_converters():
    L = oracle.lib()
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(20000) * 10.0 ** rng.integers(-20, 20, 20000)).astype(np.float32)
    # RNE by exact arithmetic: candidates are the two neighbouring bf16 values
    u = x.view(np.uint32)
    lo = (u & 0xFFFF0000).view(np.float32).astype(np.float64)
    hi = ((u & 0xFFFF0000) + 0x10000).view(np.float32).astype(np.float64)
    xd = x.astype(np.float64)
    pick_hi = (np.abs(hi - xd) < np.abs(xd - lo)) | ((np.abs(hi - xd) == np.abs(xd - lo)) & (((u >> 16) & 1) == 1))
    want = np.where(pick_hi, (u >> 16) + 1, u >> 16).astype(np.uint16)
    got = np.array([L.tq4o_f32_to_bf16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(oracle.f32_to_bf16_bits(x), want)
    for h in (0x3F80, 0xC000, 0x0001, 0x7F7F):
        assert L.tq4o_bf16_to_f32(h) == np.array([h << 16], dtype=np.uint32).view(np.float32)[0]
