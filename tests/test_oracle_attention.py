"""Pins for the oracle's paged append addressing and paged GQA attention.

Closed forms and brute force, mirroring the reference's own GPU invariant tests:
  * Q = K = 0  ->  causal running mean of V through a permuted table (tests/paged_fa2.rs:108-127)
  * single visible key -> output is that V row
  * brute-force fp64 softmax over independently gathered / dequantised rows
    (tests/backbone_and_collectives.rs:574-681), incl. non-causal window and sliding window
  * bit-identical output under page permutation (tests/backbone_and_collectives.rs:455-572)
  * masked rows untouched (cuda/tests.rs sentinel 0x5500; tests/paged_fa2.rs:618-691)
  * split-KV merge equals single pass (tests/tq4_vision_and_moe.rs:1652-1660)
  * slot mapping KAT (model/graph_io.rs:1279-1306)
"""
import numpy as np
import pytest
from scipy.linalg import hadamard

import oracle
from cases import make_case
from oracle import DT_BF16, DT_F16, FMT_BF16, FMT_FP16, FMT_TQ4, XF_IDENTITY, XF_WHT256

H = hadamard(256).astype(np.float64)


def gather_rows(pool, which, table, kv_head, n):
    """Independent gather + dequant (numpy) of logical rows 0..n-1 -> fp64 [n, 256] in the
    ORIGINAL (un-rotated) domain."""
    slab = pool.k if which == "k" else pool.v
    out = np.empty((n, pool.head_dim))
    c = oracle.centroids().astype(np.float64)
    s = oracle.signs().astype(np.float64)
    for pos in range(n):
        off = int(table[pos // pool.block_size]) * pool.page + kv_head * pool.head + (pos % pool.block_size) * pool.tok
        raw = slab[off:off + pool.tok]
        if pool.fmt == FMT_TQ4:
            d = [float(raw[0:2].view(np.float16)[0]), float(raw[66:68].view(np.float16)[0])]
            qs = np.concatenate([raw[2:66], raw[68:132]]).astype(np.int64)
            codes = np.empty(256, dtype=np.int64)
            codes[0::2], codes[1::2] = qs & 15, qs >> 4
            y = np.concatenate([d[0] * c[codes[:128]], d[1] * c[codes[128:]]])
            out[pos] = s * (H @ y / 16.0)
        elif pool.fmt == FMT_FP16:
            out[pos] = raw.view(np.float16).astype(np.float64)
        else:
            out[pos] = oracle.bf16_bits_to_f32(raw.view(np.uint16)).astype(np.float64)
    return out


def brute(qf, K, V, lo, hi, scale):
    if hi < lo:
        return np.zeros(V.shape[1])
    sc = (K[lo:hi + 1] @ qf) * scale
    p = np.exp(sc - sc.max())
    return (p[:, None] * V[lo:hi + 1]).sum(0) / p.sum()


@pytest.mark.parametrize("fmt,dtype", [(FMT_TQ4, DT_BF16), (FMT_TQ4, DT_F16), (FMT_FP16, DT_F16), (FMT_BF16, DT_BF16)])
@pytest.mark.parametrize("block_size", [16, 64])
def test_attention_matches_bruteforce(fmt, dtype, block_size):
    seq_lens, q_lens = [70, 33, 129], [1, 4, 3]
    pool, bt, k, v, q, aq, ctx = make_case(fmt, block_size, seq_lens, q_lens, 100 + block_size, dtype)
    batch = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx)
    out = oracle.paged_attention(pool, batch, q, dtype, 8)
    qf = oracle.bits_to_f32(q, dtype).astype(np.float64)
    for r in range(3):
        for h in range(2):
            K = gather_rows(pool, "k", bt[r], h, seq_lens[r])
            V = gather_rows(pool, "v", bt[r], h, seq_lens[r])
            for t in range(q_lens[r]):
                tok = aq[r] + t
                for a in range(4):
                    want = brute(qf[tok, 4 * h + a], K, V, 0, ctx[r] + t, 0.0625)
                    assert np.max(np.abs(out[tok, 4 * h + a] - want)) < 2e-5 * max(1.0, np.max(np.abs(want)))


@pytest.mark.parametrize("fmt,dtype", [(FMT_FP16, DT_F16), (FMT_BF16, DT_BF16)])
def test_attention_matches_bruteforce_at_head_dim_128(fmt, dtype):
    """16-bit pages at the reference's other head dimension (ops/op_kv_cache.cu:1227)."""
    seq_lens, q_lens = [70, 33, 129], [1, 4, 3]
    pool, bt, k, v, q, aq, ctx = make_case(fmt, 16, seq_lens, q_lens, 117, dtype, head_dim=128)
    batch = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx)
    out = oracle.paged_attention(pool, batch, q, dtype, 8)
    assert out.shape == (8, 8, 128)
    qf = oracle.bits_to_f32(q, dtype).astype(np.float64)
    for r in range(3):
        for h in range(2):
            K = gather_rows(pool, "k", bt[r], h, seq_lens[r])
            V = gather_rows(pool, "v", bt[r], h, seq_lens[r])
            for t in range(q_lens[r]):
                tok = aq[r] + t
                for a in range(4):
                    want = brute(qf[tok, 4 * h + a], K, V, 0, ctx[r] + t, 0.0625)
                    assert np.max(np.abs(out[tok, 4 * h + a] - want)) < 2e-5 * max(1.0, np.max(np.abs(want)))


def test_written_fp16_rows_are_the_inputs():
    pool, bt, k, v, q, aq, ctx = make_case(FMT_FP16, 16, [40], [1], 7, DT_F16)
    K = gather_rows(pool, "k", bt[0], 1, 40)
    assert np.array_equal(K, oracle.f16_bits_to_f32(k[:, 1, :]).astype(np.float64))


@pytest.mark.parametrize("mask_mode,window", [(0, 5), (1, 0), (1, 7), (0, 1000)])
def test_windows_and_noncausal(mask_mode, window):
    seq_lens, q_lens = [50], [6]
    pool, bt, k, v, q, aq, ctx = make_case(FMT_FP16, 16, seq_lens, q_lens, 31, DT_F16)
    batch = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=None, mask_mode=mask_mode,
                             sliding_window=window)  # ctx derived from seq_after - q_len
    out = oracle.paged_attention(pool, batch, q, DT_F16, 8)
    qf = oracle.f16_bits_to_f32(q).astype(np.float64)
    K = gather_rows(pool, "k", bt[0], 0, 50)
    V = gather_rows(pool, "v", bt[0], 0, 50)
    for t in range(6):
        hi = 49 if mask_mode == 1 else 44 + t
        lo = max(0, 44 + t - window + 1) if window > 0 else 0
        want = brute(qf[t, 2], K, V, lo, hi, 0.0625)
        assert np.max(np.abs(out[t, 2] - want)) < 2e-5


def test_zero_qk_gives_running_mean_of_v():
    seq_lens, q_lens = [37], [8]
    pool, bt, k, v, q, aq, ctx = make_case(FMT_FP16, 16, seq_lens, q_lens, 41, DT_F16)
    pool.k[:] = 0
    q[:] = 0
    batch = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx)
    out = oracle.paged_attention(pool, batch, q, DT_F16, 8)
    vf = oracle.f16_bits_to_f32(v).astype(np.float64)  # [37, 2, 256]
    for t in range(8):
        n = 29 + t + 1
        for qh in range(8):
            assert np.max(np.abs(out[t, qh] - vf[:n, qh // 4].mean(0))) < 1e-6


@pytest.mark.parametrize("fmt,dtype", [(FMT_TQ4, DT_BF16), (FMT_BF16, DT_BF16)])
def test_single_key_returns_that_v_row(fmt, dtype):
    pool, bt, k, v, q, aq, ctx = make_case(fmt, 64, [1], [1], 51, dtype)
    batch = oracle.HostBatch(aq, [1], bt, context_lens_before=[0])
    out = oracle.paged_attention(pool, batch, q, dtype, 8)
    for h in range(2):
        V = gather_rows(pool, "v", bt[0], h, 1)
        for a in range(4):
            assert np.max(np.abs(out[0, 4 * h + a] - V[0])) < 1e-5 * max(1.0, np.abs(V[0]).max())


@pytest.mark.parametrize("fmt,dtype", [(FMT_TQ4, DT_BF16), (FMT_FP16, DT_F16)])
def test_page_permutation_invariance_is_bit_exact(fmt, dtype):
    outs = []
    for perm_seed in (1, 2):
        pool, bt, k, v, q, aq, ctx = make_case(fmt, 16, [100, 45], [2, 1], 61, dtype, perm_seed=perm_seed)
        batch = oracle.HostBatch(aq, [100, 45], bt, context_lens_before=ctx)
        outs.append((bt.copy(), oracle.paged_attention(pool, batch, q, dtype, 8)))
    assert not np.array_equal(outs[0][0], outs[1][0])
    assert outs[0][1].tobytes() == outs[1][1].tobytes()


def test_masked_rows_untouched_and_threads_do_not_change_bits():
    seq_lens, q_lens = [40, 24, 3000], [2, 3, 1]
    pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 64, seq_lens, q_lens, 71, DT_BF16)
    tmask = np.array([1, 0, 1, 1, 1, 1], dtype=np.uint8)
    rmask = np.array([1, 0, 1], dtype=np.uint8)
    batch = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx, valid_token_mask=tmask, valid_req_mask=rmask)
    out1 = np.full((6, 8, 256), 12345.0, dtype=np.float32)
    oracle.paged_attention(pool, batch, q, DT_BF16, 8, n_threads=1, out=out1)
    out4 = np.full((6, 8, 256), 12345.0, dtype=np.float32)
    oracle.paged_attention(pool, batch, q, DT_BF16, 8, n_threads=4, out=out4)
    assert out1.tobytes() == out4.tobytes()
    for tok in (1, 2, 3, 4):
        assert np.all(out1[tok] == 12345.0)
    for tok in (0, 5):
        assert not np.any(out1[tok] == 12345.0)


@pytest.mark.parametrize("n_splits", [2, 5, 64])
def test_split_merge_equals_single_pass(n_splits):
    seq_lens, q_lens = [300, 17], [4, 1]
    pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 16, seq_lens, q_lens, 81, DT_F16)
    batch = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx)
    single = oracle.paged_attention(pool, batch, q, DT_F16, 8)
    split = oracle.paged_attention(pool, batch, q, DT_F16, 8, n_splits=n_splits)
    assert np.max(np.abs(single - split)) < 2e-5


def test_slot_mapping_kat_and_append_masks():
    # model/graph_io.rs:1279-1306: ctx 15, table [7, 3], 2 tokens -> [7*16+15, 3*16]
    assert list(oracle.slot_mapping([7, 3], 15, 2, 16)) == [7 * 16 + 15, 3 * 16]
    pool = oracle.HostPool(8, 2, 256, 16, FMT_FP16, XF_IDENTITY)
    k = oracle.fill_kv_rows(4, 2, 256, 5, DT_F16, 0)
    v = oracle.fill_kv_rows(4, 2, 256, 6, DT_F16, 0)
    slots = np.array([7 * 16 + 15, 3 * 16, -1, 5 * 16 + 2], dtype=np.int32)
    wb = oracle.HostBatch([0, 2, 4], [16, 17], np.zeros((2, 2), np.int32), write_slot_mapping=slots,
                          valid_token_mask=[1, 0, 1, 1], valid_req_mask=[1, 1])
    oracle.kv_cache_write(pool, wb, k, v, DT_F16)
    def row(slab, page, head, off):
        o = page * pool.page + head * pool.head + off * pool.tok
        return slab[o:o + 512].view(np.uint16)
    assert np.array_equal(row(pool.k, 7, 1, 15), k[0, 1])
    assert np.array_equal(row(pool.v, 5, 0, 2), v[3, 0])
    written = np.zeros_like(pool.k, dtype=bool)
    for page, off in ((7, 15), (5, 2)):
        for h in range(2):
            o = page * pool.page + h * pool.head + off * pool.tok
            written[o:o + 512] = True
    assert not pool.k[~written].any() and not pool.v[~written].any()
    # request mask
    pool2 = oracle.HostPool(8, 2, 256, 16, FMT_FP16, XF_IDENTITY)
    wb2 = oracle.HostBatch([0, 2, 4], [16, 17], np.zeros((2, 2), np.int32), write_slot_mapping=np.abs(slots),
                           valid_req_mask=[0, 1])
    oracle.kv_cache_write(pool2, wb2, k, v, DT_F16)
    assert not row(pool2.k, 7, 0, 15).any() and row(pool2.k, 5, 0, 2).any()
    # strided source: V read out of a packed [K | V] buffer
    packed = np.concatenate([k.reshape(4, 512), v.reshape(4, 512)], axis=1)
    pool3 = oracle.HostPool(8, 2, 256, 16, FMT_FP16, XF_IDENTITY)
    wb3 = oracle.HostBatch([0, 4], [4], np.zeros((1, 1), np.int32), write_slot_mapping=[0, 1, 2, 3])
    L, B = pool3.layout(), wb3.struct()
    import ctypes as C
    flat = np.ascontiguousarray(packed)
    rc = oracle.lib().tq4o_kv_cache_write(C.byref(L), C.byref(B), flat.ctypes.data, flat.ctypes.data + 1024,
                                          1024, 1024, DT_F16)
    assert rc == 0
    assert np.array_equal(row(pool3.v, 0, 1, 3), v[3, 1]) and np.array_equal(row(pool3.k, 0, 0, 2), k[2, 0])
