"""Shared builders of synthetic paged-KV cases for the oracle and the GPU parity tests."""
import numpy as np

import oracle
from oracle import FMT_TQ4, XF_IDENTITY, XF_WHT256


def make_case(fmt, block_size, seq_lens, q_lens, seed, dtype, kv_heads=2, q_heads=8, perm_seed=5,
              extra_pages=3, xf=None, head_dim=256, v_xf=None):
    """Append seq_len tokens per request through the oracle's write, return everything."""
    if xf is None:
        xf = XF_WHT256 if fmt == FMT_TQ4 else XF_IDENTITY
    pages_per = [(s + block_size - 1) // block_size for s in seq_lens]
    num_pages = sum(pages_per) + extra_pages
    perm = oracle.permutation(num_pages, perm_seed)
    pool = oracle.HostPool(num_pages, kv_heads, head_dim, block_size, fmt, xf, v_xf)
    mb = max(pages_per)
    bt = np.zeros((len(seq_lens), mb), dtype=np.int32)
    at = 0
    slots, qsl = [], [0]
    for r, s in enumerate(seq_lens):
        bt[r, :pages_per[r]] = perm[at:at + pages_per[r]]
        at += pages_per[r]
        slots.append(oracle.slot_mapping(bt[r], 0, s, block_size))
        qsl.append(qsl[-1] + s)
    total = qsl[-1]
    k = oracle.fill_kv_rows(total, kv_heads, head_dim, seed, dtype, 3)
    v = oracle.fill_kv_rows(total, kv_heads, head_dim, seed + 1, dtype, 3)
    wb = oracle.HostBatch(qsl, seq_lens, bt, context_lens_before=[0] * len(seq_lens),
                          write_slot_mapping=np.concatenate(slots))
    oracle.kv_cache_write(pool, wb, k, v, dtype)
    # attention batch: last q_len tokens of each request are the queries
    aq = [0]
    for ql in q_lens:
        aq.append(aq[-1] + ql)
    q = oracle.fill_normal(aq[-1] * q_heads * head_dim, seed + 2, dtype).reshape(aq[-1], q_heads, head_dim)
    ctx = [s - ql for s, ql in zip(seq_lens, q_lens)]
    return pool, bt, k, v, q, aq, ctx


def qsa_groups_of(bt, seq_lens, block_size, select_k):
    """Every 4-token group of each sequence in logical order, as the selection lists of the QSA
    sparse attention (ops/op_qsa.cu:812-822): physical group = page * (block_size / 4) + group in
    page, logical group = position / 4; unused entries are -1."""
    gpp = block_size // 4
    n = len(seq_lens)
    sel_phys = np.full((n, select_k), -1, dtype=np.int32)
    sel_log = np.zeros((n, select_k), dtype=np.int32)
    num_sel = np.zeros(n, dtype=np.int32)
    for r, s in enumerate(seq_lens):
        groups = (s + 3) // 4
        assert groups <= select_k
        lg = np.arange(groups)
        sel_phys[r, :groups] = np.asarray(bt[r])[lg * 4 // block_size] * gpp + (lg * 4 % block_size) // 4
        sel_log[r, :groups] = lg
        num_sel[r] = groups
    return sel_phys, sel_log, num_sel
