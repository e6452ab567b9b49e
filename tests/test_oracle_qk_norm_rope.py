"""Pins of the oracle's QK RMSNorm + RoPE (+ paged KV write) restatement
(ops/op_dflash2.cu:338-418).  The reference's golden tensors for this operator are LFS pointers
only (tools/oracle/goldens/sglang_dflash_bf16.safetensors is 132 bytes), so the checks are what
the mathematics fixes: an independent float64 restatement within one bf16 ulp, the identity
rotation, norm preservation of the rotated pairs, untouched V, skip rules, and the equality of
the fused cache write with the un-fused composition (operator, then append)."""
import numpy as np
import pytest

import oracle
from oracle import DT_BF16, FMT_BF16, FMT_FP8, FMT_Q8_0, FMT_TQ4, XF_IDENTITY, XF_WHT256

Q_HEADS, KV_HEADS, DIM = 4, 2, 256


def _case(rows, seed, dim=DIM, q_heads=Q_HEADS, kv_heads=KV_HEADS, table_rows=64):
    rng = np.random.default_rng(seed)
    qkv = oracle.f32_to_bf16_bits(rng.standard_normal((rows, (q_heads + 2 * kv_heads) * dim)).astype(np.float32) * 1.7)
    qw = oracle.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(dim)).astype(np.float32))
    kw = oracle.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(dim)).astype(np.float32))
    pos = rng.integers(0, table_rows, size=rows).astype(np.int32)
    half = dim // 2
    inv_freq = 1.0 / (10000.0 ** (np.arange(half) / half))
    ang = np.arange(table_rows)[:, None] * inv_freq[None, :]
    table = np.concatenate([np.cos(ang), np.sin(ang)], axis=1).astype(np.float32)
    return qkv, qw, kw, pos, table


def _reference_f64(qkv_bits, qw, kw, pos, table, q_heads, kv_heads, dim, eps):
    """float64 restatement written from the operator's definition: y = x / sqrt(mean(x^2) + eps) * w,
    rounded to bf16, then (a, b) -> (a cos - b sin, b cos + a sin) on the pairs (c, c + dim/2)."""
    x = oracle.bf16_bits_to_f32(qkv_bits).astype(np.float64).reshape(qkv_bits.shape[0], q_heads + 2 * kv_heads, dim)
    out = x.copy()
    half = dim // 2
    for h in range(q_heads + kv_heads):
        w = oracle.bf16_bits_to_f32(qw if h < q_heads else kw).astype(np.float64)
        xs = x[:, h, :]
        y = xs / np.sqrt((xs * xs).mean(axis=1, keepdims=True) + eps) * w
        y = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(y.astype(np.float32))).astype(np.float64)
        c, s = table[pos, :half].astype(np.float64), table[pos, half:].astype(np.float64)
        a, b = y[:, :half], y[:, half:]
        out[:, h, :half] = a * c - b * s
        out[:, h, half:] = b * c + a * s
    return out.reshape(qkv_bits.shape[0], -1)


def _ulp_bf16(x):
    return np.maximum(np.abs(x), 2.0 ** -126) * 2.0 ** -7


@pytest.mark.parametrize("dim", [256, 128])
def test_matches_float64_restatement_within_one_bf16_ulp(dim):
    qkv, qw, kw, pos, table = _case(24, 1, dim=dim)
    want = _reference_f64(qkv, qw, kw, pos, table, Q_HEADS, KV_HEADS, dim, 1e-6)
    got_bits, _ = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, table, Q_HEADS, KV_HEADS, dim, 1e-6)
    got = oracle.bf16_bits_to_f32(got_bits).astype(np.float64)
    # the normalised value is rounded to bf16 before the rotation in both; a one-ulp difference of that
    # intermediate moves the result by at most (|cos| + |sin|) ulp(y) <= 1.5 ulp of the larger input
    y_mag = np.abs(want).reshape(24, -1, dim)
    bound = 2.5 * _ulp_bf16(np.maximum(y_mag, np.roll(y_mag, dim // 2, axis=2))).reshape(24, -1)
    qk = (Q_HEADS + KV_HEADS) * dim
    assert (np.abs(got - want)[:, :qk] <= bound[:, :qk]).all()
    assert (np.abs(got - want)[:, :qk] <= 0.5 * _ulp_bf16(want)[:, :qk] + 1e-30).mean() > 0.97
    # V columns are bit-identical
    assert (got_bits[:, qk:] == qkv[:, qk:]).all()


def test_bf16_table_equals_f32_table_of_the_same_values():
    qkv, qw, kw, pos, table = _case(8, 2)
    tb = oracle.f32_to_bf16_bits(table)
    t32 = oracle.bf16_bits_to_f32(tb).astype(np.float32)
    a, _ = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, tb, Q_HEADS, KV_HEADS, DIM, 1e-6)
    b, _ = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, t32, Q_HEADS, KV_HEADS, DIM, 1e-6)
    assert (a == b).all()


def test_identity_rotation_and_unit_rms():
    """cos = 1, sin = 0 and unit weights: the output is bf16(x / rms(x)), its RMS is 1."""
    qkv, qw, kw, pos, table = _case(6, 3)
    table[:, :DIM // 2] = 1.0
    table[:, DIM // 2:] = 0.0
    one = oracle.f32_to_bf16_bits(np.ones(DIM, np.float32))
    got_bits, _ = oracle.qk_norm_rope_bf16(qkv.copy(), pos, one, one, table, Q_HEADS, KV_HEADS, DIM, 1e-6)
    got = oracle.bf16_bits_to_f32(got_bits).reshape(6, -1, DIM)[:, :Q_HEADS + KV_HEADS]
    x = oracle.bf16_bits_to_f32(qkv).astype(np.float64).reshape(6, -1, DIM)[:, :Q_HEADS + KV_HEADS]
    want = x / np.sqrt((x * x).mean(axis=2, keepdims=True) + 1e-6)
    assert (np.abs(got - want) <= 0.5 * _ulp_bf16(want) * 1.001).all()
    assert np.allclose(np.sqrt((got.astype(np.float64) ** 2).mean(axis=2)), 1.0, atol=3e-3)


def test_rotation_preserves_pair_norms():
    qkv, qw, kw, pos, table = _case(10, 4)
    got_bits, _ = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, table, Q_HEADS, KV_HEADS, DIM, 1e-6)
    zero_rot = table.copy()
    zero_rot[:, :DIM // 2], zero_rot[:, DIM // 2:] = 1.0, 0.0
    base_bits, _ = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, zero_rot, Q_HEADS, KV_HEADS, DIM, 1e-6)
    g = oracle.bf16_bits_to_f32(got_bits).astype(np.float64).reshape(10, -1, 2, DIM // 2)[:, :Q_HEADS + KV_HEADS]
    b = oracle.bf16_bits_to_f32(base_bits).astype(np.float64).reshape(10, -1, 2, DIM // 2)[:, :Q_HEADS + KV_HEADS]
    n_g, n_b = np.hypot(g[:, :, 0], g[:, :, 1]), np.hypot(b[:, :, 0], b[:, :, 1])
    assert np.allclose(n_g, n_b, rtol=2.0 ** -7, atol=1e-6)


def test_sum_of_squares_follows_the_32_lane_tree():
    """Squares 2^24, 1, 1 at elements 0, 128, 64: the tree of op_dflash2.cu:30-39 adds
    (v0 + v128) first, which rounds the 1 away, then (v64 + v192) = 1 is rounded away as well:
    2^24.  An order that meets the two ones first gives 2^24 + 2.  eps is searched so that this
    difference flips a bf16 rounding of the output; the oracle must give the tree's bits."""
    x = np.zeros(DIM, np.float32)
    x[0], x[128], x[64] = 4096.0, 1.0, 1.0

    def out_bits(sum_sq, eps):
        mean = np.float32(np.float32(sum_sq) / np.float32(DIM)) + np.float32(eps)
        inv = np.float32(1.0 / np.sqrt(np.float64(np.float32(mean))))
        return oracle.f32_to_bf16_bits(np.array([np.float32(4096.0) * inv], np.float32))[0]

    # aim at the bf16 rounding midpoint 15.96875 of the output 4096 / sqrt(mean): the mean has
    # a spacing of 2^-7 there, which is exactly what the two sums differ by after the division
    target = (4096.0 / 15.96875) ** 2 - 65536.0
    found = None
    for k in range(-4000, 4000):
        eps = np.float32(target + k * 2.0 ** -7)
        if out_bits(16777216.0, eps) != out_bits(16777218.0, eps):
            found = float(eps)
            break
    assert found is not None
    qkv = np.zeros((1, (Q_HEADS + 2 * KV_HEADS) * DIM), np.uint16)
    qkv[0, :DIM] = oracle.f32_to_bf16_bits(x)
    one = oracle.f32_to_bf16_bits(np.ones(DIM, np.float32))
    table = np.zeros((1, DIM), np.float32)
    table[:, :DIM // 2] = 1.0
    got_bits, _ = oracle.qk_norm_rope_bf16(qkv.copy(), [0], one, one, table, Q_HEADS, KV_HEADS, DIM, found)
    assert got_bits[0, 0] == out_bits(16777216.0, found)
    assert got_bits[0, 0] != out_bits(16777218.0, found)


def test_positions_outside_the_table_skip_the_row_and_q_out():
    qkv, qw, kw, pos, table = _case(5, 5)
    pos[1], pos[3] = -1, table.shape[0]
    q_out = np.full((5, Q_HEADS * DIM), 0x7E7E, np.uint16)
    got, q_out = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, table, Q_HEADS, KV_HEADS, DIM, 1e-6, q_out=q_out)
    in_place, _ = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, table, Q_HEADS, KV_HEADS, DIM, 1e-6)
    for r in (1, 3):
        assert (got[r] == qkv[r]).all() and (q_out[r] == 0x7E7E).all()
    for r in (0, 2, 4):
        assert (q_out[r] == in_place[r, :Q_HEADS * DIM]).all()           # Q went to q_out ...
        assert (got[r, :Q_HEADS * DIM] == qkv[r, :Q_HEADS * DIM]).all()   # ... and the packed Q is untouched
        assert (got[r, Q_HEADS * DIM:] == in_place[r, Q_HEADS * DIM:]).all()


@pytest.mark.parametrize("fmt,xf", [(FMT_BF16, XF_IDENTITY), (FMT_TQ4, XF_WHT256), (FMT_FP8, XF_IDENTITY),
                                    (FMT_Q8_0, XF_IDENTITY), (FMT_Q8_0, XF_WHT256)])
def test_fused_cache_write_equals_operator_then_append(fmt, xf):
    """tests/dflash_proposer.rs:371-520: reversed page table, one negative slot."""
    rows, bs = 20, 16
    qkv, qw, kw, pos, table = _case(rows, 6, dim=256)
    bt = np.array([2, 1, 0], np.int32)
    slots = oracle.slot_mapping(bt, 0, rows, bs)
    slots[7] = -1
    fused = oracle.HostPool(3, KV_HEADS, 256, bs, fmt, xf)
    fused.k[:], fused.v[:] = 0x7E, 0x7E
    q_out = np.zeros((rows, Q_HEADS * 256), np.uint16)
    got, q_out = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, table, Q_HEADS, KV_HEADS, 256, 1e-6, q_out=q_out,
                                          pool=fused, write_slot_mapping=slots)
    # un-fused: operator in place, then append of the K and V columns
    plain, _ = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, table, Q_HEADS, KV_HEADS, 256, 1e-6)
    ref = oracle.HostPool(3, KV_HEADS, 256, bs, fmt, xf)
    ref.k[:], ref.v[:] = 0x7E, 0x7E
    stride = (Q_HEADS + 2 * KV_HEADS) * 256
    hb = oracle.HostBatch([0, rows], [rows], bt.reshape(1, -1), context_lens_before=[0], write_slot_mapping=slots)
    k_cols = np.ascontiguousarray(plain[:, Q_HEADS * 256:(Q_HEADS + KV_HEADS) * 256])
    v_cols = np.ascontiguousarray(plain[:, (Q_HEADS + KV_HEADS) * 256:])
    oracle.kv_cache_write(ref, hb, k_cols, v_cols, DT_BF16)
    assert fused.k.tobytes() == ref.k.tobytes() and fused.v.tobytes() == ref.v.tobytes()
    assert (q_out == plain[:, :Q_HEADS * 256]).all()
    # the packed K of a written row stays as it was; the skipped slot's K is rotated in place
    kq = slice(Q_HEADS * 256, (Q_HEADS + KV_HEADS) * 256)
    for r in range(rows):
        if r == 7:
            assert (got[r, kq] == plain[r, kq]).all()
        else:
            assert (got[r, kq] == qkv[r, kq]).all()
    assert stride == qkv.shape[1]
