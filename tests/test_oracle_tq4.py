"""Pins for the oracle's WHT-256, TQ4 encode and dequant.

Independent checks (none of them re-types the oracle's loops):
  * WHT: multiplication by scipy's Sylvester Hadamard matrix / 16 -- exact equality on
    integer-valued inputs (all intermediate sums are exact in fp32), involution, Parseval,
    impulse response (csrc/tq/tq4_kv_common.cuh:75-107);
  * encode: a straight-line fp64 restatement by matrix algebra -- rotation = H/16 @ (s*x),
    per-128 RMS normalisation, NEAREST centroid (argmin) instead of the boundary count,
    numpy least-squares for the scale (op_kv_cache.cu:152-218);
  * special cases the mathematics fixes (all-zero row, scaling covariance, LSQ optimality);
  * layout: 132-byte rows, fp16 scale at byte 0 / 66, low nibble = even element
    (csrc/tq/tq4_kv_common.cuh:21-26, op_kv_cache.cu:192-198 vs :303-305).
"""
import numpy as np
from scipy.linalg import hadamard

import oracle

H = hadamard(256).astype(np.float64)


def rows(seed, n, outliers=True):
    bits = oracle.fill_kv_rows(n, 1, 256, seed, oracle.DT_BF16, 3 if outliers else 0)
    return oracle.bf16_bits_to_f32(bits.reshape(n, 256))


def test_wht_equals_sylvester_matrix_exact_on_integers():
    rng = np.random.default_rng(0)
    for _ in range(20):
        x = rng.integers(-64, 65, 256).astype(np.float32)
        want = (H @ x.astype(np.float64)) / 16.0
        got = oracle.wht256(x)
        assert np.array_equal(got.astype(np.float64), want)


def test_wht_impulse_involution_parseval():
    for k in (0, 1, 37, 128, 255):
        e = np.zeros(256, dtype=np.float32)
        e[k] = 1.0
        assert np.array_equal(oracle.wht256(e).astype(np.float64), H[:, k] / 16.0)
    x = rows(3, 4)
    for r in x:
        y = oracle.wht256(r)
        assert abs(float(np.dot(y.astype(np.float64), y.astype(np.float64))) /
                   float(np.dot(r.astype(np.float64), r.astype(np.float64))) - 1.0) < 1e-6
        assert np.max(np.abs(oracle.wht256(y) - r)) < 1e-4 * np.max(np.abs(r))
        assert np.max(np.abs(y.astype(np.float64) - H @ r.astype(np.float64) / 16.0)) < 1e-4 * np.max(np.abs(r))


def unpack(row):
    """Independent reader of the 132-byte row: returns (codes[256], d[2])."""
    row = np.asarray(row, dtype=np.uint8)
    d = np.array([row[0:2].view(np.float16)[0], row[66:68].view(np.float16)[0]], dtype=np.float32)
    qs = np.concatenate([row[2:66], row[68:132]])
    codes = np.empty(256, dtype=np.int64)
    codes[0::2] = qs & 0x0F
    codes[1::2] = qs >> 4
    return codes, d


def encode_fp64(x):
    """Straight-line restatement in fp64 matrix algebra."""
    c = oracle.centroids().astype(np.float64)
    s = oracle.signs().astype(np.float64)
    y = H @ (s * x.astype(np.float64)) / 16.0
    codes = np.empty(256, dtype=np.int64)
    d = np.empty(2)
    margin = np.empty(256)
    for h in range(2):
        yh = y[128 * h:128 * (h + 1)]
        n2 = float(yh @ yh)
        rv = yh * (np.sqrt(0.5) / np.sqrt(n2)) if n2 > 1e-20 else np.zeros(128)
        dist = np.abs(rv[:, None] - c[None, :])
        k = np.argmin(dist, axis=1)
        part = np.sort(dist, axis=1)
        margin[128 * h:128 * (h + 1)] = part[:, 1] - part[:, 0]
        codes[128 * h:128 * (h + 1)] = k
        ch = c[k]
        d[h] = np.linalg.lstsq(ch[:, None], yh, rcond=None)[0][0]
    return y, codes, d, margin


def test_encode_matches_fp64_restatement():
    x = rows(11, 64)
    n_checked = 0
    for r in x:
        row = oracle.encode_row(r)
        codes, d = unpack(row)
        y, codes64, d64, margin = encode_fp64(r)
        safe = margin > 1e-5  # exclude elements within rounding distance of a boundary
        assert safe.sum() > 250
        assert np.array_equal(codes[safe], codes64[safe])
        n_checked += int(safe.sum())
        if np.array_equal(codes, codes64):
            # scale: fp16 rounding of the least-squares optimum
            want = d64.astype(np.float32).astype(np.float16).astype(np.float32)
            ulp = np.maximum(np.abs(want) * 2.0 ** -10, 2.0 ** -24)
            assert np.all(np.abs(d - want) <= ulp)
    assert n_checked > 64 * 250


def test_encode_scale_is_least_squares_optimum():
    """The residual y - d*c must be orthogonal to c in each 128-half (up to fp16 rounding of d)."""
    c = oracle.centroids().astype(np.float64)
    s = oracle.signs().astype(np.float64)
    for r in rows(5, 16):
        codes, d = unpack(oracle.encode_row(r))
        y = H @ (s * r.astype(np.float64)) / 16.0
        for h in range(2):
            ch, yh = c[codes[128 * h:128 * (h + 1)]], y[128 * h:128 * (h + 1)]
            d_opt = float(yh @ ch) / float(ch @ ch)
            assert abs(d[h] - d_opt) <= abs(d_opt) * 2.0 ** -10


def test_encode_zero_row():
    """s_sq = 0 -> inv_norm = 0 -> rv = 0 -> exactly the 7 negative boundaries satisfy rv > b
    (b[7] = 0 is a strict compare) -> every code 7; sum v*c = 0 -> d = +-0."""
    row = oracle.encode_row(np.zeros(256, dtype=np.float32))
    codes, d = unpack(row)
    assert np.all(codes == 7)
    assert np.all(d == 0.0)
    assert np.all(row[2:66] == 0x77) and np.all(row[68:132] == 0x77)
    assert np.all(oracle.dequant_row(row) == 0.0)


def test_encode_power_of_two_scaling_covariance():
    """Multiplying the input by 2^k is exact in every fp32 step, so codes are identical and
    the scale is multiplied by 2^k."""
    for r in rows(9, 8, outliers=False):
        a = oracle.encode_row(r)
        b = oracle.encode_row(r * np.float32(4.0))
        ca, da = unpack(a)
        cb, db = unpack(b)
        assert np.array_equal(ca, cb)
        assert np.array_equal(db, da * 4.0)


def test_row_layout_and_dequant_reader():
    r = rows(21, 1)[0]
    row = oracle.encode_row(r)
    assert row.shape == (132,)
    codes, d = unpack(row)
    assert codes.min() >= 0 and codes.max() <= 15
    c = oracle.centroids()
    want = np.concatenate([d[0] * c[codes[:128]], d[1] * c[codes[128:]]]).astype(np.float32)
    assert oracle.dequant_row(row).tobytes() == want.tobytes()


def test_rotation_preserves_inner_products_and_quality():
    """<Q', K_rot> = <Q, K>; relative MSE of the round trip ~ codebook distortion 0.0094."""
    x = rows(33, 32)
    s = oracle.signs()
    q = rows(34, 1, outliers=False)[0]
    qrot = oracle.wht256(q * s)
    errs = []
    for r in x:
        row = oracle.encode_row(r)
        yhat = oracle.dequant_row(row)
        y = oracle.wht256(r * s)
        errs.append(float(np.sum((yhat - y) ** 2) / np.sum(y ** 2)))
        assert abs(float(qrot @ y) - float(q @ r)) < 1e-3 * np.linalg.norm(q) * np.linalg.norm(r)
        xhat = oracle.unrotate_row(yhat)
        assert abs(float(np.sum((xhat - r) ** 2) / np.sum(r ** 2)) - errs[-1]) < 1e-4
    assert 0.005 < np.mean(errs) < 0.015, np.mean(errs)


# ---- TQ4 without the rotation (op_kv_cache.cu:219-264): the same block quantiser on the raw
# 128-element blocks of a row of any head dimension that is a multiple of 128 ----

def unpack_blocks(row):
    """Independent reader: 66-byte blocks {fp16 scale, 64 bytes of nibbles} -> (codes, scales)."""
    row = np.asarray(row, dtype=np.uint8).reshape(-1, 66)
    d = row[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1)
    codes = np.empty((row.shape[0], 128), dtype=np.int64)
    codes[:, 0::2] = row[:, 2:] & 0x0F
    codes[:, 1::2] = row[:, 2:] >> 4
    return codes.reshape(-1), d


def encode_plain_fp64(x):
    c = oracle.centroids().astype(np.float64)
    x = x.astype(np.float64)
    nb = x.shape[0] // 128
    codes = np.empty(x.shape[0], dtype=np.int64)
    d = np.empty(nb)
    margin = np.empty(x.shape[0])
    for b in range(nb):
        xb = x[128 * b:128 * (b + 1)]
        n = np.sqrt(float(xb @ xb))
        u = xb * (np.sqrt(0.5) / n) if n > 1e-12 else np.zeros(128)
        dist = np.abs(u[:, None] - c[None, :])
        k = np.argmin(dist, axis=1)
        part = np.sort(dist, axis=1)
        margin[128 * b:128 * (b + 1)] = part[:, 1] - part[:, 0]
        codes[128 * b:128 * (b + 1)] = k
        ck = c[k]
        d[b] = np.linalg.lstsq(ck[:, None], xb, rcond=None)[0][0]
    return codes, d, margin


def test_plain_encode_matches_fp64_restatement():
    n_checked = 0
    for hd in (128, 256):
        bits = oracle.fill_kv_rows(48, 1, hd, 21 + hd, oracle.DT_BF16, 3)
        for r in oracle.bf16_bits_to_f32(bits.reshape(48, hd)):
            row = oracle.encode_row_plain(r)
            assert row.shape == (66 * (hd // 128),)
            codes, d = unpack_blocks(row)
            codes64, d64, margin = encode_plain_fp64(r)
            safe = margin > 1e-5
            assert safe.sum() > hd - 6
            assert np.array_equal(codes[safe], codes64[safe])
            n_checked += int(safe.sum())
            if np.array_equal(codes, codes64):
                want = d64.astype(np.float32).astype(np.float16).astype(np.float32)
                ulp = np.maximum(np.abs(want) * 2.0 ** -10, 2.0 ** -24)
                assert np.all(np.abs(d - want) <= ulp)
    assert n_checked > 96 * 120


def test_plain_encode_special_rows():
    """Zero block: inv_norm = 0 -> u = 0 -> code 7 (the strict compare stops at b[7] = 0), x.c = 0 -> d = 0.
    A block that is a multiple of a centroid pattern: the codes reproduce the pattern and the
    scale is that multiple (every element then dequantises to itself up to the fp16 scale)."""
    codes, d = unpack_blocks(oracle.encode_row_plain(np.zeros(256, dtype=np.float32)))
    assert np.all(codes == 7) and np.all(d == 0)
    c = oracle.centroids().astype(np.float64)
    rng = np.random.default_rng(5)
    pattern = rng.integers(0, 16, 128)
    x = np.concatenate([3.0 * c[pattern], np.zeros(128)]).astype(np.float32)
    codes, d = unpack_blocks(oracle.encode_row_plain(x))
    # the normalisation maps the block onto the unit-variance codebook only if its RMS matches;
    # what must hold for ANY scale: the quantiser is monotone, so equal inputs get equal codes
    # and larger inputs never get smaller codes
    order = np.argsort(x[:128], kind="stable")
    assert np.all(np.diff(codes[:128][order]) >= 0)
    for v in np.unique(x[:128]):
        assert len(set(codes[:128][x[:128] == v])) == 1
    assert np.all(codes[128:] == 7) and d[1] == 0
    # least-squares optimality of the scale
    ck = c[codes[:128]]
    d_opt = float(x[:128].astype(np.float64) @ ck) / float(ck @ ck)
    assert abs(d[0] - d_opt) <= abs(d_opt) * 2.0 ** -10


def test_plain_encode_power_of_two_scaling_covariance():
    """x -> 4x: same codes, scale x 4 (exact in fp32; the fp16 scale stays in range)."""
    bits = oracle.fill_kv_rows(8, 1, 256, 77, oracle.DT_BF16, 0)
    for r in oracle.bf16_bits_to_f32(bits.reshape(8, 256)):
        c1, d1 = unpack_blocks(oracle.encode_row_plain(r))
        c4, d4 = unpack_blocks(oracle.encode_row_plain(4.0 * r))
        assert np.array_equal(c1, c4) and np.array_equal(4.0 * d1, d4)
