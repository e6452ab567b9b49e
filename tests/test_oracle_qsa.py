"""Pins of the oracle's QSA sparse paged attention (ops/op_qsa.cu:716-1158,1446-1571).

  * the reference test's known answer: V = 0.25 everywhere, gate 0 -> 0.125
    (crates/warp34-host/src/ple/gpu_tests.rs:653-681)
  * every group of a sequence selected = dense causal attention of the last token (the dense
    oracle is pinned on its own)
  * brute-force fp64 softmax over independently dequantised rows, with skipped groups (phys < 0),
    keys behind the token's position, a partial tail group, fewer groups than the list holds,
    masked tokens and tokens without any visible key
  * the per-64 output transform is the Sylvester matrix H64 / 8 (exact on small integers) and an
    involution (ops/hadamard_inline.cuh:11-50)
"""
import numpy as np
import pytest
from scipy.linalg import hadamard

import oracle
from oracle import DT_F16, FMT_FP16, FMT_FP8, FMT_Q8_0, FMT_TQ4, XF_IDENTITY, XF_WHT256
from cases import make_case, qsa_groups_of


def f16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16).view(np.uint16)


def test_known_answer_uniform_values_and_zero_gate():
    # two tokens, 2 q heads over 1 kv head, pages of 16 tokens, groups as the reference's selector
    # returned them for this fixture: sel_phys[0..6] = 8, 9, 10, 11, 4, 5
    pool = oracle.HostPool(4, 1, 256, 16, FMT_FP16, XF_IDENTITY)
    pool.k.view(np.uint16)[:] = f16(0.1)
    pool.v.view(np.uint16)[:] = f16(0.25)
    sel_phys = np.array([[8, 9, 10, 11, 4, 5, -1, -1]] * 2, dtype=np.int32)
    sel_log = np.array([[0, 1, 2, 3, 4, 5, 0, 0]] * 2, dtype=np.int32)
    q = np.full((2, 2, 256), f16(0.1), dtype=np.uint16)
    gate = np.full((2, 2, 256), f16(0.0), dtype=np.uint16)
    out = oracle.qsa_sparse_paged_attn_f16(pool, q, sel_phys, sel_log, [6, 6], [20, 21], 2, gate=gate)
    assert np.all(out == f16(0.125))
    # without the gate: 0.25
    out = oracle.qsa_sparse_paged_attn_f16(pool, q, sel_phys, sel_log, [6, 6], [20, 21], 2)
    assert np.all(out == f16(0.25))


@pytest.mark.parametrize("fmt,xf", [(FMT_TQ4, XF_WHT256), (FMT_FP16, XF_IDENTITY), (FMT_Q8_0, XF_WHT256),
                                    (FMT_FP8, XF_IDENTITY)])
def test_all_groups_selected_is_dense_decode(fmt, xf):
    seq = [203, 64]
    pool, bt, k, v, q, aq, ctx = make_case(fmt, 16, seq, [1, 1], 501, DT_F16, xf=xf)
    hb = oracle.HostBatch(aq, seq, bt, context_lens_before=ctx)
    dense = oracle.paged_attention(pool, hb, q, DT_F16, 8)
    sel_phys, sel_log, num_sel = qsa_groups_of(bt, seq, 16, select_k=64)
    out = oracle.qsa_sparse_paged_attn_f16(pool, q, sel_phys, sel_log, num_sel, [s - 1 for s in seq], 8)
    got = oracle.f16_bits_to_f32(out)
    want = dense.astype(np.float16).astype(np.float32)
    # both round the same fp64-accumulated value once: at most one fp16 ulp apart (fp32 un-rotation)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-3)) < 2e-3


def _brute(pool, q, sel_phys, sel_log, num_sel, seq_pos, heads, gate, mask, sm_scale):
    n_tok = q.shape[0]
    g = heads // pool.kv_heads
    gpp = pool.block_size // 4
    kk = pool.k.reshape(pool.num_pages, pool.kv_heads, pool.block_size, pool.tok)
    vv = pool.v.reshape(pool.num_pages, pool.kv_heads, pool.block_size, pool.tok)
    out = np.zeros((n_tok, heads, 256))

    cent = oracle.centroids().astype(np.float64)
    Hs = hadamard(256).astype(np.float64) / 16.0 * oracle.signs().astype(np.float64)[:, None]

    def row(slab, page, h, r, xf):
        raw = slab[page, h, r]
        if pool.fmt == FMT_TQ4:    # two blocks of {fp16 d, 64 bytes of nibbles, low nibble first}
            y = np.zeros(256)
            for blk in range(2):
                d = float(raw[66 * blk:66 * blk + 2].view(np.float16)[0])
                qs = raw[66 * blk + 2:66 * blk + 66]
                y[128 * blk:128 * blk + 128:2] = d * cent[qs & 15]
                y[128 * blk + 1:128 * blk + 128:2] = d * cent[qs >> 4]
        elif pool.fmt == FMT_Q8_0:  # four blocks of {fp32 d, 64 int8}
            y = np.concatenate([float(raw[68 * b:68 * b + 4].view(np.float32)[0]) *
                                raw[68 * b + 4:68 * b + 68].view(np.int8).astype(np.float64) for b in range(4)])
        else:
            y = raw.view(np.float16).astype(np.float64)
        return Hs @ y if xf == XF_WHT256 else y  # x = sign * (H / 16) y

    for t in range(n_tok):
        if mask is not None and not mask[t]:
            continue
        for h in range(pool.kv_heads):
            ks, vs = [], []
            for j in range(min(int(num_sel[t]), sel_phys.shape[1])):
                for off in range(4):
                    if sel_phys[t, j] < 0 or sel_log[t, j] * 4 + off > seq_pos[t]:
                        continue
                    page, r = sel_phys[t, j] // gpp, (sel_phys[t, j] % gpp) * 4 + off
                    ks.append(row(kk, page, h, r, pool.transform))
                    vs.append(row(vv, page, h, r, pool.transform))
            if not ks:
                continue
            K, V = np.array(ks), np.array(vs)
            for a in range(g):
                qq = oracle.f16_bits_to_f32(q[t, h * g + a]).astype(np.float64)
                s = K @ qq * sm_scale
                p = np.exp(s - s.max())
                o = p @ V / p.sum()
                if gate is not None:
                    o = o / (1.0 + np.exp(-oracle.f16_bits_to_f32(gate[t, h * g + a]).astype(np.float64)))
                out[t, h * g + a] = o
    return out


@pytest.mark.parametrize("fmt,xf", [(FMT_TQ4, XF_WHT256), (FMT_FP16, XF_IDENTITY), (FMT_Q8_0, XF_IDENTITY)])
def test_brute_force_sparse_selection(fmt, xf):
    seq = [150]
    pool, bt, k, v, _, _, _ = make_case(fmt, 16, seq, [1], 511, DT_F16, xf=xf)
    n_tok, heads, select_k = 5, 4, 9
    rng = np.random.default_rng(3)
    q = oracle.fill_normal(n_tok * heads * 256, 512, DT_F16).reshape(n_tok, heads, 256)
    gate = oracle.fill_normal(n_tok * heads * 256, 513, DT_F16).reshape(n_tok, heads, 256)
    all_phys, all_log, _ = qsa_groups_of(bt, seq, 16, select_k=64)
    n_groups = (seq[0] + 3) // 4
    sel_phys = np.full((n_tok, select_k), -7, dtype=np.int32)
    sel_log = np.zeros((n_tok, select_k), dtype=np.int32)
    num_sel = np.zeros(n_tok, dtype=np.int32)
    seq_pos = np.array([149, 120, 77, 3, 149], dtype=np.int32)
    for t in range(n_tok):
        pick = rng.permutation(n_groups)[:select_k]
        sel_phys[t] = all_phys[0, pick]
        sel_log[t] = all_log[0, pick]
        num_sel[t] = select_k
    sel_phys[0, 2] = -1            # a skipped group
    sel_log[1, 0] = 120 // 4       # a group cut by the token position
    sel_phys[1, 0] = all_phys[0, 120 // 4]
    num_sel[2] = 4                 # fewer groups than the list holds
    sel_log[3, :] = 30             # every key behind the position: zero row
    mask = np.array([1, 1, 1, 1, 0], dtype=np.uint8)
    out = oracle.qsa_sparse_paged_attn_f16(pool, q, sel_phys, sel_log, num_sel, seq_pos, heads, gate=gate,
                                           valid_token_mask=mask)
    want = _brute(pool, q, sel_phys, sel_log, num_sel, seq_pos, heads, gate, mask, 0.0625)
    got = oracle.f16_bits_to_f32(out).astype(np.float64)
    assert np.all(got[3] == 0) and np.all(got[4] == 0)
    assert np.max(np.abs(got - want)) <= 1e-3 * np.max(np.abs(want)) + 1e-6


def test_hadamard64_output_transform():
    pool = oracle.HostPool(2, 1, 256, 16, FMT_FP16, XF_IDENTITY)
    rng = np.random.default_rng(9)
    vals = rng.integers(-8, 9, size=(32, 256)).astype(np.float32)
    pool.v.view(np.uint16).reshape(32, 256)[:] = vals.astype(np.float16).view(np.uint16)
    # one key per token: the attention output is that key's value row
    n_tok = 8
    sel_phys = np.arange(n_tok, dtype=np.int32).reshape(n_tok, 1)
    sel_log = np.arange(n_tok, dtype=np.int32).reshape(n_tok, 1)
    seq_pos = 4 * np.arange(n_tok, dtype=np.int32)  # only the first key of each group is visible
    q = np.zeros((n_tok, 1, 256), dtype=np.uint16)
    plain = oracle.qsa_sparse_paged_attn_f16(pool, q, sel_phys, sel_log, [1] * n_tok, seq_pos, 1)
    assert np.array_equal(oracle.f16_bits_to_f32(plain)[:, 0], vals[0:32:4])
    had = oracle.qsa_sparse_paged_attn_f16(pool, q, sel_phys, sel_log, [1] * n_tok, seq_pos, 1, hadamard64=True)
    H = hadamard(64).astype(np.float64) / 8.0
    want = (vals[0:32:4].reshape(n_tok, 4, 64).astype(np.float64) @ H.T).reshape(n_tok, 256)
    assert np.array_equal(oracle.f16_bits_to_f32(had)[:, 0].astype(np.float64), want.astype(np.float16).astype(np.float64))
    # an involution: feeding multiples of 8 keeps every intermediate exact
    pool.v.view(np.uint16).reshape(32, 256)[:] = (8 * vals).astype(np.float16).view(np.uint16)
    once = oracle.qsa_sparse_paged_attn_f16(pool, q, sel_phys, sel_log, [1] * n_tok, seq_pos, 1, hadamard64=True)
    pool.v.view(np.uint16).reshape(32, 256)[0:32:4] = once[:, 0]
    twice = oracle.qsa_sparse_paged_attn_f16(pool, q, sel_phys, sel_log, [1] * n_tok, seq_pos, 1, hadamard64=True)
    assert np.array_equal(oracle.f16_bits_to_f32(twice)[:, 0], 8 * vals[0:32:4])


def test_gate_limits():
    pool = oracle.HostPool(1, 1, 256, 16, FMT_FP16, XF_IDENTITY)
    pool.v.view(np.uint16)[:] = f16(1.0)
    q = np.zeros((1, 1, 256), dtype=np.uint16)
    for g, want in ((0.0, 0.5), (30.0, 1.0), (-30.0, 0.0), (1.0, 1.0 / (1.0 + np.exp(-1.0)))):
        gate = np.full((1, 1, 256), f16(g), dtype=np.uint16)
        out = oracle.qsa_sparse_paged_attn_f16(pool, q, [[0]], [[0]], [1], [3], 1, gate=gate)
        assert np.allclose(oracle.f16_bits_to_f32(out), want, atol=5e-4)
