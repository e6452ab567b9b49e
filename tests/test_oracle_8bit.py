"""Oracle pins for the 8-bit tail-anchor formats (FP8 E4M3 rows of 264 B, Q8_0 rows of 272 B).

The conversion is pinned by brute force against the definition of the OCP E4M3 format
(sign, 4 exponent bits with bias 7, 3 mantissa bits, no infinities, largest finite value 448):
every code decodes to the value the definition gives, and encoding any float gives the nearest
finite code, ties to the code with an even mantissa, saturating at +-448.  The row encoders are
pinned by their closed forms (scale = amax / 448 or amax / 127 in fp32, elementwise conversion of
x * (1 / scale)), by the layouts the reference declares
(csrc/tq/tq4_kv_common.cuh:28-46) and by round-trip error bounds.
"""
import numpy as np
import pytest

import oracle
from oracle import DT_BF16, FMT_FP8, FMT_Q8_0


def _e4m3_value(c):
    e, m = (c >> 3) & 15, c & 7
    if e == 15 and m == 7:
        return float("nan")
    v = m * 2.0 ** -9 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
    return -v if c & 0x80 else v


def test_e4m3_decode_matches_the_format_definition():
    for c in range(256):
        want = _e4m3_value(c)
        got = oracle.e4m3_to_f32(c)
        assert (np.isnan(want) and np.isnan(got)) or got == want, c
    assert oracle.e4m3_to_f32(0x7e) == 448.0 and oracle.e4m3_to_f32(0x08) == 2.0 ** -6


def test_e4m3_encode_is_nearest_even_and_saturating():
    finite = [(c, _e4m3_value(c)) for c in range(0x7f)]  # positive finite codes, ascending values
    vals = np.array([v for _, v in finite])
    rng = np.random.default_rng(3)
    probes = list(vals)                                   # exact values
    probes += list((vals[:-1] + vals[1:]) / 2)            # exact midpoints: ties
    probes += list(np.nextafter(((vals[:-1] + vals[1:]) / 2).astype(np.float32), np.float32(0)))
    probes += list(np.nextafter(((vals[:-1] + vals[1:]) / 2).astype(np.float32), np.float32(1e9)))
    probes += list(np.exp(rng.uniform(np.log(1e-4), np.log(600.0), size=4000)))
    for p in probes:
        p = float(np.float32(p))
        d = np.abs(vals - p)
        best = np.flatnonzero(d == d.min())
        want = best[0] if len(best) == 1 else [b for b in best if b % 2 == 0][0]  # tie -> even mantissa
        if p >= 448.0:
            want = 0x7e
        assert oracle.f32_to_e4m3(p) == want, (p, want)
        assert oracle.f32_to_e4m3(-p) == (want | 0x80) or p == 0.0
    assert oracle.f32_to_e4m3(float("inf")) == 0x7e and oracle.f32_to_e4m3(float("-inf")) == 0xfe
    assert oracle.f32_to_e4m3(float("nan")) & 0x7f == 0x7f


def _rows(seed, n=8):
    x = oracle.bits_to_f32(oracle.fill_kv_rows(n, 1, 256, seed, DT_BF16, 3), DT_BF16)
    return x.reshape(n, 256).astype(np.float32)


def test_fp8_row_closed_form_layout_and_round_trip():
    for x in _rows(11):
        row = oracle.encode_row_fmt(x, FMT_FP8)
        assert row.shape == (264,)
        d = row[256:264].view(np.float32)
        for h in range(2):
            xh = x[128 * h:128 * h + 128]
            want_d = np.float32(np.abs(xh).max()) * np.float32(1.0 / 448.0)
            assert d[h] == want_d
            inv = np.float32(1.0) / want_d
            codes = [oracle.f32_to_e4m3(float(np.float32(v) * inv)) for v in xh]
            assert list(row[128 * h:128 * h + 128]) == codes
        y = oracle.dequant_row_fmt(row, FMT_FP8)
        # 3 mantissa bits: relative error <= 2^-4 in the normal range, absolute <= d * 2^-10 below it
        bound = np.maximum(np.abs(x) * 2.0 ** -4, np.repeat(d, 128) * 2.0 ** -10) * (1 + 1e-6)
        assert (np.abs(y - x) <= bound).all()
    z = oracle.encode_row_fmt(np.zeros(256, np.float32), FMT_FP8)
    assert not z.any()


def test_q8_row_closed_form_layout_and_round_trip():
    for x in _rows(12):
        row = oracle.encode_row_fmt(x, FMT_Q8_0)
        assert row.shape == (272,)
        for sb in range(4):
            xb = x[64 * sb:64 * sb + 64]
            d = row[68 * sb:68 * sb + 4].view(np.float32)[0]
            want_d = np.float32(np.abs(xb).max()) / np.float32(127.0)
            assert d == want_d
            inv = np.float32(1.0) / want_d
            t = (xb * inv).astype(np.float32)
            q = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -127, 127).astype(np.int8)
            assert (row[68 * sb + 4:68 * sb + 68].view(np.int8) == q).all()
        y = oracle.dequant_row_fmt(row, FMT_Q8_0)
        dd = np.repeat([row[68 * sb:68 * sb + 4].view(np.float32)[0] for sb in range(4)], 64)
        assert (np.abs(y - x) <= dd * 0.5 * (1 + 1e-5)).all()
    z = oracle.encode_row_fmt(np.zeros(256, np.float32), FMT_Q8_0)
    assert not z.any()


@pytest.mark.parametrize("fmt", [FMT_FP8, FMT_Q8_0])
def test_paged_write_and_attention_over_8bit_rows(fmt):
    """Append through the paged write, then attention == brute-force softmax over the rows the
    row dequantiser gives (identity transform, as the default policy uses for these layers)."""
    from cases import make_case

    seq_lens, q_lens = [70, 33], [3, 1]
    pool, bt, k, v, q, aq, ctx = make_case(fmt, 16, seq_lens, q_lens, 13, DT_BF16)
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx)
    got = oracle.paged_attention(pool, hb, q, DT_BF16, 8)
    tok = pool.tok
    qf = oracle.bits_to_f32(q, DT_BF16).astype(np.float64)
    start = 0
    for r, (s, ql) in enumerate(zip(seq_lens, q_lens)):
        for h in range(2):
            rows_k = np.zeros((s, 256))
            rows_v = np.zeros((s, 256))
            for t in range(s):
                base = int(bt[r, t // 16]) * pool.page + h * pool.head + (t % 16) * tok
                rows_k[t] = oracle.dequant_row_fmt(pool.k[base:base + tok], fmt)
                rows_v[t] = oracle.dequant_row_fmt(pool.v[base:base + tok], fmt)
            # the stored rows are the appended rows, re-encoded
            want_row = oracle.encode_row_fmt(oracle.bits_to_f32(k[sum(seq_lens[:r]) + 5, h], DT_BF16), fmt)
            base5 = int(bt[r, 0]) * pool.page + h * pool.head + 5 * tok
            assert bytes(pool.k[base5:base5 + tok]) == bytes(want_row)
            for i in range(ql):
                n_vis = s - ql + i + 1
                for a in range(4):
                    qv = qf[start + i, 4 * h + a]
                    sc = rows_k[:n_vis] @ qv * 0.0625
                    p = np.exp(sc - sc.max())
                    want = (p / p.sum()) @ rows_v[:n_vis]
                    assert np.abs(got[start + i, 4 * h + a] - want).max() < 1e-4
        start += ql
