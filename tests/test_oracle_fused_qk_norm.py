"""Pins of the oracle's restatement of the target model's fused Gemma RMSNorm + interleaved mRoPE +
gate split (ops/op_norms_rope_act.cu:524-689).  No vector of this operator is in the reference
tree, so the restatement is checked against what the arithmetic fixes: an independent float64
implementation written from the formulas (within one fp16 ulp), position 0 = the normed row,
rotation preserves pair norms, the un-rotated tail and the gate are copies, three equal position
planes give plain RoPE, the plane pattern of the interleaved sections, strides, masks."""
import numpy as np

import oracle
from oracle import DT_F16

HD, ROT, MROPE, THETA, EPS = 256, 64, (11, 11, 10), 1.0e7, 1.0e-6


def _inputs(n, qh, kh, seed, q_stride=None, k_stride=None):
    q_stride = qh * 2 * HD if q_stride is None else q_stride
    k_stride = kh * HD if k_stride is None else k_stride
    qg = oracle.fill_normal(n * q_stride, seed, DT_F16).reshape(n, q_stride)
    k = oracle.fill_normal(n * k_stride, seed + 1, DT_F16).reshape(n, k_stride)
    qw = oracle.f32_to_f16_bits(0.1 * oracle.f16_bits_to_f32(oracle.fill_normal(HD, seed + 2, DT_F16)))
    kw = oracle.f32_to_f16_bits(0.1 * oracle.f16_bits_to_f32(oracle.fill_normal(HD, seed + 3, DT_F16)))
    return qg, k, qw, kw


def _plane(i):
    if i % 3 == 1 and i < 3 * MROPE[1]:
        return 1
    if i % 3 == 2 and i < 3 * MROPE[2]:
        return 2
    return 0


def _ref64(x, w, pos3):
    """float64 restatement of one head: x fp16 values [HD], w fp16 values [HD], pos3 = the token's three positions"""
    x = x.astype(np.float64)
    inv = 1.0 / np.sqrt((x * x).mean() + EPS)
    normed = x * inv * (1.0 + w.astype(np.float64))
    out = normed.copy()
    half = ROT // 2
    for i in range(half):
        ang = np.float64(np.float32(pos3[_plane(i)]) * np.float32(1.0 / np.float32(THETA ** (np.float32(2 * i) / np.float32(ROT)))))
        c, s = np.cos(ang), np.sin(ang)
        out[i] = normed[i] * c - normed[i + half] * s
        out[i + half] = normed[i + half] * c + normed[i] * s
    return out


def _ulp16(x):
    return np.maximum(np.spacing(np.abs(x).astype(np.float16)).astype(np.float64), 2.0 ** -24)


def test_against_float64_restatement():
    n, qh, kh = 5, 4, 2
    qg, k, qw, kw = _inputs(n, qh, kh, 100)
    pos = np.array([[0, 7, 300, 5000, 131071], [0, 3, 300, 17, 9], [0, 11, 300, 4999, 262143]], dtype=np.int32)
    q_out, k_out, gate = oracle.fused_qk_rmsnorm_rope_gate_f16(qg, k, qw, kw, pos, qh, kh, HD, ROT, MROPE, THETA, EPS)
    qf, kf = oracle.f16_bits_to_f32(q_out), oracle.f16_bits_to_f32(k_out)
    qgf, kin = oracle.f16_bits_to_f32(qg).reshape(n, qh, 2, HD), oracle.f16_bits_to_f32(k).reshape(n, kh, HD)
    wq, wk = oracle.f16_bits_to_f32(qw), oracle.f16_bits_to_f32(kw)
    for t in range(n):
        for h in range(qh):
            want = _ref64(qgf[t, h, 0], wq, pos[:, t])
            # two fp16 roundings (normed, result) and fp16 sine / cosine: a few ulp of the larger pair element
            tol = 3.0 * _ulp16(np.maximum(np.abs(want), 1e-3)) + 2.0 ** -10 * np.abs(want).max() * (np.arange(HD) < ROT)
            assert (np.abs(qf[t, h] - want) <= tol).all(), (t, h)
        for h in range(kh):
            want = _ref64(kin[t, h], wk, pos[:, t])
            tol = 3.0 * _ulp16(np.maximum(np.abs(want), 1e-3)) + 2.0 ** -10 * np.abs(want).max() * (np.arange(HD) < ROT)
            assert (np.abs(kf[t, h] - want) <= tol).all(), (t, h)
    # the gate half of every Q head is copied bit for bit
    assert gate.tobytes() == np.ascontiguousarray(qg.reshape(n, qh, 2, HD)[:, :, 1]).tobytes()


def test_position_zero_is_the_normed_row_and_rotation_preserves_pair_norms():
    n, qh, kh = 2, 2, 1
    qg, k, qw, kw = _inputs(n, qh, kh, 200)
    zero = np.zeros((3, n), dtype=np.int32)
    q0, k0, _ = oracle.fused_qk_rmsnorm_rope_gate_f16(qg, k, qw, kw, zero, qh, kh, HD, ROT, MROPE, THETA, EPS)
    pos = np.array([[12345, 77]] * 3, dtype=np.int32)
    q1, k1, _ = oracle.fused_qk_rmsnorm_rope_gate_f16(qg, k, qw, kw, pos, qh, kh, HD, ROT, MROPE, THETA, EPS)
    f0, f1 = oracle.f16_bits_to_f32(k0).astype(np.float64), oracle.f16_bits_to_f32(k1).astype(np.float64)
    # cos 0 = 1, sin 0 = 0: the output is the normed row (mean square 1 before the weight)
    x = oracle.f16_bits_to_f32(k).reshape(n, kh, HD).astype(np.float64)
    normed = x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + EPS) * (1.0 + oracle.f16_bits_to_f32(kw))
    assert np.abs(f0 - normed).max() <= 2.0 ** -10 * np.abs(normed).max()
    # the tail behind rotary_dim does not depend on the position
    assert k0[..., ROT:].tobytes() == k1[..., ROT:].tobytes() and q0[..., ROT:].tobytes() == q1[..., ROT:].tobytes()
    # a rotation keeps the norm of every pair (i, i + ROT / 2)
    half = ROT // 2
    n0 = f0[..., :half] ** 2 + f0[..., half:ROT] ** 2
    n1 = f1[..., :half] ** 2 + f1[..., half:ROT] ** 2
    assert np.abs(n0 - n1).max() <= 4e-3 * max(n0.max(), 1.0)


def test_interleaved_sections_select_the_position_planes():
    # one plane at a time set to a non-zero position: exactly the pairs of that plane move
    n, qh, kh = 1, 1, 1
    qg, k, qw, kw = _inputs(n, qh, kh, 300)
    base = oracle.fused_qk_rmsnorm_rope_gate_f16(qg, k, qw, kw, np.zeros((3, 1), np.int32), qh, kh, HD, ROT, MROPE,
                                                 THETA, EPS)[1]
    half = ROT // 2
    for plane in range(3):
        pos = np.zeros((3, 1), dtype=np.int32)
        pos[plane, 0] = 1000
        out = oracle.fused_qk_rmsnorm_rope_gate_f16(qg, k, qw, kw, pos, qh, kh, HD, ROT, MROPE, THETA, EPS)[1]
        moved = {i for i in range(half) if out[0, 0, i] != base[0, 0, i] or out[0, 0, i + half] != base[0, 0, i + half]}
        expect = {i for i in range(half) if _plane(i) == plane}
        assert moved <= expect and len(moved) >= len(expect) - 2, (plane, sorted(expect - moved))
    assert [_plane(i) for i in range(8)] == [0, 1, 2, 0, 1, 2, 0, 1] and _plane(31) == 1 and _plane(29) == 2 and _plane(32) == 0


def test_strides_and_token_mask():
    n, qh, kh = 4, 2, 2
    qs, ks = qh * 2 * HD + 512, kh * HD + 256  # K rows inside a wider packed buffer
    qg, k, qw, kw = _inputs(n, qh, kh, 400, qs, ks)
    pos = np.arange(3 * n, dtype=np.int32).reshape(3, n)
    a = oracle.fused_qk_rmsnorm_rope_gate_f16(qg, k, qw, kw, pos, qh, kh, HD, ROT, MROPE, THETA, EPS)
    qg_c = np.ascontiguousarray(qg[:, :qh * 2 * HD])
    k_c = np.ascontiguousarray(k[:, :kh * HD])
    b = oracle.fused_qk_rmsnorm_rope_gate_f16(qg_c, k_c, qw, kw, pos, qh, kh, HD, ROT, MROPE, THETA, EPS)
    for x, y in zip(a, b):
        assert x.tobytes() == y.tobytes()
    mask = np.array([1, 0, 1, 0], dtype=np.uint8)
    sent = [np.full_like(x, 0x5555) for x in a]
    m = oracle.fused_qk_rmsnorm_rope_gate_f16(qg, k, qw, kw, pos, qh, kh, HD, ROT, MROPE, THETA, EPS, valid_token_mask=mask,
                                              q_out=sent[0], k_out=sent[1], gate_out=sent[2])
    for x, y in zip(m, a):
        assert x[0].tobytes() == y[0].tobytes() and x[2].tobytes() == y[2].tobytes()
        assert (x[1] == 0x5555).all() and (x[3] == 0x5555).all()
