"""GPU parity: paged GQA decode / verify attention through the C ABI vs the CPU oracle.

Tolerance (gpu_harness.assert_close): |got - want| <= 2e-3 + 1e-2 |want| against the fp64-accumulating
oracle on every channel of unit-scale data; only on the x20 outlier channels of the benchmark inputs
(three per head) is the absolute part taken relative to the channel's magnitude, 2e-3 * max|V|.  Every
call logs its worst excess over the plain bound on ALL channels (pytest's terminal summary).
Invariants follow the reference's GPU tests: page-permutation 0-ULP
(tests/backbone_and_collectives.rs:455-572), split vs single pass < 2e-3 and graph-bucket
bound independence (tests/tq4_vision_and_moe.rs:1355-1663), masked rows untouched
(cuda/tests.rs sentinel 0x5500), scratch canaries (tests/paged_fa2.rs:171-200).
"""
import numpy as np
import pytest

import oracle
from cases import make_case
from oracle import DT_BF16, DT_F16, FMT_BF16, FMT_FP8, FMT_FP16, FMT_Q8_0, FMT_TQ4, XF_IDENTITY, XF_WHT256

pytestmark = pytest.mark.gpu

SCRATCH = 16 << 20


def _dev_pool(pool):
    import gpu_harness as G

    d = G.DevPool(pool)
    d.upload()
    return d


def _check(fmt, dtype, block_size, seq_lens, q_lens, seed, scratch=SCRATCH, q_heads=8, kv_heads=2,
           mask_mode=0, window=0, ctx_null=False, xf=None, head_dim=256, v_xf=None, plain_excess=0.0, **kw):
    import gpu_harness as G

    pool, bt, k, v, q, aq, ctx = make_case(fmt, block_size, seq_lens, q_lens, seed, dtype, kv_heads=kv_heads,
                                           q_heads=q_heads, xf=xf, head_dim=head_dim, v_xf=v_xf)
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=None if ctx_null else ctx, mask_mode=mask_mode,
                          sliding_window=window)
    want = oracle.paged_attention(pool, hb, q, dtype, q_heads, n_threads=4)
    dpool = _dev_pool(pool)
    rc, got, _ = G.dev_attention(dpool, hb, q, dtype, q_heads, scratch_bytes=scratch, **kw)
    assert rc == 0
    err = G.assert_close(got, dtype, want, what="fmt=%d bs=%d seq=%s q=%s" % (fmt, block_size, seq_lens, q_lens),
                         scale=G.channel_scale(v, dtype, hb, q_heads), plain_excess=plain_excess)
    return got, want, err


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F16])
@pytest.mark.parametrize("block_size", [16, 64])
def test_tq4_decode_small_batch(dtype, block_size):
    _check(FMT_TQ4, dtype, block_size, [70, 33, 129, 1, 32], [1, 1, 1, 1, 1], 11)


@pytest.mark.parametrize("scratch", [0, SCRATCH])
def test_tq4_decode_gqa8_long(scratch):
    """16 q heads / 2 kv heads (GQA 8), one sequence of 5000 tokens, with and without scratch."""
    _check(FMT_TQ4, DT_BF16, 64, [5000], [1], 21, scratch=scratch, q_heads=16)


def test_tq4_decode_split_vs_single_pass():
    import gpu_harness as G

    pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 64, [20000, 777], [1, 1], 31, DT_BF16, q_heads=16)
    hb = oracle.HostBatch(aq, [20000, 777], bt, context_lens_before=ctx)
    dpool = _dev_pool(pool)
    rc0, single, _ = G.dev_attention(dpool, hb, q, DT_BF16, 16, scratch_bytes=0)
    rc1, split, ws = G.dev_attention(dpool, hb, q, DT_BF16, 16, scratch_bytes=SCRATCH)
    assert rc0 == 0 and rc1 == 0
    # split vs single pass (tests/tq4_vision_and_moe.rs:1652-1660: < 2e-3 on unit-scale data);
    # both are bf16 here, so allow the same row-scaled bound as against the oracle
    G.assert_close(split, DT_BF16, oracle.bf16_bits_to_f32(single), what="split vs single")
    want = oracle.paged_attention(pool, hb, q, DT_BF16, 16, n_threads=8)
    G.assert_close(split, DT_BF16, want, what="split")
    G.assert_close(single, DT_BF16, want, what="single")
    # a scratch that is too small or misaligned must be left untouched (single pass instead)
    rc2, small, ws2 = G.dev_attention(dpool, hb, q, DT_BF16, 16, scratch_bytes=4096)
    assert rc2 == 0 and bool((ws2 == 0x5A).all())
    assert small.tobytes() == single.tobytes()


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F16])
def test_tq4_decode_batch_balanced_shares(dtype):
    """Decode batches whose requests differ widely in length: the work is cut into equal shares
    of 32-token units across workgroups, so long requests are split over many workgroups and a
    workgroup may work on several short requests in turn (one of them empty-keyed, one masked)."""
    import gpu_harness as G

    seq = [5000, 300, 9000, 64, 2500, 33, 1, 7777]
    _check(FMT_TQ4, dtype, 64, seq, [1] * len(seq), 181, q_heads=16)
    _check(FMT_TQ4, dtype, 16, seq, [1] * len(seq), 182, q_heads=8, window=0, mask_mode=1)
    # two query tokens per request (one tile at 8 q heads per kv head), a masked request
    pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 64, [700, 40, 3000], [2, 2, 2], 183, dtype, q_heads=16)
    rmask = np.array([1, 0, 1], np.uint8)
    hb = oracle.HostBatch(aq, [700, 40, 3000], bt, context_lens_before=ctx, valid_req_mask=rmask)
    want = oracle.paged_attention(pool, hb, q, dtype, 16, n_threads=4)
    rc, got, _ = G.dev_attention(_dev_pool(pool), hb, q, dtype, 16, scratch_bytes=SCRATCH)
    assert rc == 0
    assert (got[2:4] == 0x5500).all()  # rows of the masked request keep the sentinel
    live = np.array([0, 1, 4, 5])
    G.assert_close(got[live], dtype, want[live], what="masked request", scale=G.channel_scale(v, dtype, hb, 16)[live])


@pytest.mark.parametrize("q_lens", [[4, 4], [2, 3], [16]])
def test_tq4_verify_multi_token_causal(q_lens):
    seq = [300 + 7 * i for i in range(len(q_lens))]
    _check(FMT_TQ4, DT_BF16, 64, seq, q_lens, 41, q_heads=16)
    _check(FMT_TQ4, DT_F16, 16, seq, q_lens, 42, q_heads=8, scratch=0)


@pytest.mark.parametrize("mask_mode,window", [(0, 40), (1, 0), (1, 100), (0, 5)])
def test_tq4_windows(mask_mode, window):
    _check(FMT_TQ4, DT_BF16, 16, [333, 90], [3, 2], 51, mask_mode=mask_mode, window=window, ctx_null=True)


def test_page_permutation_and_bounds_do_not_change_bits():
    import gpu_harness as G

    outs = []
    for perm_seed in (1, 2):
        pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 16, [1500, 200], [1, 1], 61, DT_F16, perm_seed=perm_seed)
        hb = oracle.HostBatch(aq, [1500, 200], bt, context_lens_before=ctx)
        dpool = _dev_pool(pool)
        for bound in (None, 4096):
            rc, out, _ = G.dev_attention(dpool, hb, q, DT_F16, 8, scratch_bytes=SCRATCH, max_seq_len=bound)
            assert rc == 0
            outs.append(out)
    for o in outs[1:]:
        assert o.tobytes() == outs[0].tobytes()


def test_masked_rows_are_untouched():
    import gpu_harness as G

    seq_lens, q_lens = [40, 24, 300], [2, 3, 1]
    pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 64, seq_lens, q_lens, 71, DT_BF16)
    tmask = np.array([1, 0, 1, 1, 1, 1], dtype=np.uint8)
    rmask = np.array([1, 0, 1], dtype=np.uint8)
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx, valid_token_mask=tmask, valid_req_mask=rmask)
    want = oracle.paged_attention(pool, hb, q, DT_BF16, 8)
    dpool = _dev_pool(pool)
    for scratch in (0, SCRATCH):
        rc, got, _ = G.dev_attention(dpool, hb, q, DT_BF16, 8, scratch_bytes=scratch, sentinel=0x5500)
        assert rc == 0
        for tok in (1, 2, 3, 4):
            assert (got[tok] == 0x5500).all()
        for tok in (0, 5):
            G.assert_close(got[tok], DT_BF16, want[tok], what="tok %d" % tok)


def test_empty_key_range_gives_zeros():
    """A sliding window that ends before the first key -> zeros (op_kv_cache.cu:939-946)."""
    import gpu_harness as G

    pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 16, [50], [1], 81, DT_BF16)
    hb = oracle.HostBatch(aq, [10], bt, context_lens_before=[60], sliding_window=4)  # window [57, 60], seq 10
    dpool = _dev_pool(pool)
    rc, got, _ = G.dev_attention(dpool, hb, q, DT_BF16, 8, scratch_bytes=SCRATCH)
    assert rc == 0 and not oracle.bf16_bits_to_f32(got).any()  # +-0 everywhere


def test_force_kernel_selector_agrees():
    import gpu_harness as G

    pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 16, [260], [8], 91, DT_F16)
    hb = oracle.HostBatch(aq, [260], bt, context_lens_before=ctx)
    want = oracle.paged_attention(pool, hb, q, DT_F16, 8)
    dpool = _dev_pool(pool)
    outs = {}
    for sel in (0, 1, 2):
        rc, got, _ = G.dev_attention(dpool, hb, q, DT_F16, 8, force_kernel=sel)
        assert rc == 0
        G.assert_close(got, DT_F16, want, what="selector %d" % sel)
        outs[sel] = got.tobytes()
    # 0 = the decode / verify kernel as one pass, anything else = the 128-row tile kernel: two
    # kernels that add the same products in different orders, so the bytes differ
    assert outs[1] == outs[2]
    assert outs[0] != outs[1]


# ---- TQ4 pages stored without the rotation, or with one slab rotated (ops/op_kv_cache.cu:219-264;
# ops/op_paged_attn.cu:347,570: the query is rotated for rotated keys, the output for rotated values) ----

TQ4_XF = [(XF_IDENTITY, XF_IDENTITY), (XF_WHT256, XF_IDENTITY), (XF_IDENTITY, XF_WHT256)]


@pytest.mark.parametrize("k_xf,v_xf", TQ4_XF)
@pytest.mark.parametrize("dtype", [DT_BF16, DT_F16])
def test_tq4_plain_slabs_decode_and_verify(k_xf, v_xf, dtype):
    _check(FMT_TQ4, dtype, 16, [70, 33, 129, 1, 32], [1, 1, 1, 1, 1], 301, xf=k_xf, v_xf=v_xf)
    _check(FMT_TQ4, dtype, 64, [300, 307], [4, 3], 302, q_heads=16, xf=k_xf, v_xf=v_xf)


@pytest.mark.parametrize("k_xf,v_xf", TQ4_XF)
@pytest.mark.parametrize("scratch", [0, SCRATCH])
def test_tq4_plain_slabs_long_decode(k_xf, v_xf, scratch):
    """Split-K with the merge kernel (rotation there follows the V slab) and the single pass."""
    _check(FMT_TQ4, DT_BF16, 64, [20000, 777], [1, 1], 303, scratch=scratch, q_heads=16, xf=k_xf, v_xf=v_xf)


@pytest.mark.parametrize("k_xf,v_xf", TQ4_XF)
def test_tq4_plain_slabs_batched_decode_and_prefill(k_xf, v_xf):
    """The balanced decode kernel (equal shares of a batch) and the 128-row tile kernel."""
    _check(FMT_TQ4, DT_BF16, 64, [9000, 3000, 5000, 700], [1, 1, 1, 1], 304, scratch=64 << 20, q_heads=16,
           xf=k_xf, v_xf=v_xf)
    # Tolerance: the contract bound plus 2.5e-3 absolute on the plain channels.  Without the rotation
    # the three x20 channels of a key row carry most of a score, so the rounding of the query's fp16
    # MFMA operand on those three channels does not average out over 256 channels as it does in the
    # rotated domain: about five times the score error from the same operand types (the decode kernel
    # and the tile kernel, two independent implementations, land on the same values here: worst
    # element +1.6e-3 over the literal bound, 18 of 13 million elements over it).
    _check(FMT_TQ4, DT_BF16, 64, [1400, 1100], [1200, 900], 305, scratch=0, q_heads=16, xf=k_xf, v_xf=v_xf,
           plain_excess=2.5e-3)


# ---- 16-bit pages (FP16 pages with the f16 entry point, BF16 pages with the bf16 one) ----

KV16 = [(FMT_FP16, DT_F16), (FMT_BF16, DT_BF16)]


@pytest.mark.parametrize("fmt,dtype", KV16)
@pytest.mark.parametrize("block_size", [16, 64])
def test_kv16_decode_small_batch(fmt, dtype, block_size):
    _check(fmt, dtype, block_size, [70, 33, 129, 1, 32], [1, 1, 1, 1, 1], 111)


@pytest.mark.parametrize("fmt,dtype", KV16)
@pytest.mark.parametrize("scratch", [0, SCRATCH])
def test_kv16_decode_gqa8_long(fmt, dtype, scratch):
    _check(fmt, dtype, 64, [5000], [1], 121, scratch=scratch, q_heads=16)


def test_kv16_bf16_decode_ctx32k():
    """Benchmark bf16 decode shape: ctx 32768, 16 q / 2 kv heads, 64-token pages."""
    _check(FMT_BF16, DT_BF16, 64, [32768], [1], 131, scratch=64 << 20, q_heads=16)


@pytest.mark.parametrize("fmt,dtype", KV16)
@pytest.mark.parametrize("q_lens", [[4, 4], [2, 3], [16]])
def test_kv16_verify_multi_token_causal(fmt, dtype, q_lens):
    seq = [300 + 7 * i for i in range(len(q_lens))]
    _check(fmt, dtype, 64, seq, q_lens, 141, q_heads=16)
    _check(fmt, dtype, 16, seq, q_lens, 142, q_heads=8, scratch=0)


@pytest.mark.parametrize("mask_mode,window", [(0, 40), (1, 0), (1, 100), (0, 5)])
def test_kv16_windows(mask_mode, window):
    _check(FMT_BF16, DT_BF16, 16, [333, 90], [3, 2], 151, mask_mode=mask_mode, window=window, ctx_null=True)


# ---- head dimension 128 (16-bit pages only, ops/op_kv_cache.cu:873,1227) ----

@pytest.mark.parametrize("fmt,dtype", KV16)
@pytest.mark.parametrize("block_size", [16, 64])
def test_kv16_head_dim_128_decode(fmt, dtype, block_size):
    _check(fmt, dtype, block_size, [70, 33, 129, 1, 32], [1, 1, 1, 1, 1], 181, head_dim=128)


@pytest.mark.parametrize("fmt,dtype", KV16)
@pytest.mark.parametrize("scratch", [0, SCRATCH])
def test_kv16_head_dim_128_decode_gqa8_long(fmt, dtype, scratch):
    """Split-K (partial records keep their 256-float stride) and the single pass."""
    _check(fmt, dtype, 64, [5000], [1], 182, scratch=scratch, q_heads=16, head_dim=128)
    _check(fmt, dtype, 16, [20000, 777], [1, 1], 183, scratch=scratch, q_heads=16, head_dim=128)


@pytest.mark.parametrize("fmt,dtype", KV16)
@pytest.mark.parametrize("q_lens", [[4, 4], [2, 3], [16], [200]])
def test_kv16_head_dim_128_verify_and_prefill(fmt, dtype, q_lens):
    """Several query tokens per request, up to a prefill chunk: every shape runs the decode / verify kernel."""
    seq = [300 + 7 * i for i in range(len(q_lens))]
    _check(fmt, dtype, 64, seq, q_lens, 184, q_heads=16, head_dim=128)
    _check(fmt, dtype, 16, seq, q_lens, 185, q_heads=8, scratch=0, head_dim=128)


@pytest.mark.parametrize("mask_mode,window", [(0, 40), (1, 0), (1, 100), (0, 5)])
def test_kv16_head_dim_128_windows(mask_mode, window):
    _check(FMT_BF16, DT_BF16, 16, [333, 90], [3, 2], 186, mask_mode=mask_mode, window=window, ctx_null=True, head_dim=128)


def test_kv16_head_dim_128_gqa_shapes():
    """One and four q heads per kv head, and more than sixteen (two q subgroups)."""
    _check(FMT_BF16, DT_BF16, 16, [90, 41], [1, 2], 187, q_heads=2, kv_heads=2, head_dim=128)
    _check(FMT_BF16, DT_BF16, 16, [90, 41], [1, 2], 188, q_heads=4, kv_heads=1, head_dim=128)
    _check(FMT_FP16, DT_F16, 32, [150], [3], 189, q_heads=32, kv_heads=1, head_dim=128)


def test_kv16_head_dim_128_8bit_and_tq4_pages_are_refused():
    """Only 16-bit rows exist at head dimension 128: the other formats answer "not supported"."""
    import gpu_harness as G

    pool, bt, k, v, q, aq, ctx = make_case(FMT_BF16, 16, [40], [1], 190, DT_BF16, head_dim=128)
    hb = oracle.HostBatch(aq, [40], bt, context_lens_before=ctx)
    dpool = _dev_pool(pool)
    for fmt in (FMT_TQ4, FMT_FP8, FMT_Q8_0):
        rc, got, _ = G.dev_attention(dpool, hb, q, DT_BF16, 8, layout=dpool.layout(fmt))
        assert rc == 801 and (got == 0x5500).all()


def test_kv16_unwritten_pool_bytes_do_not_leak():
    """Rows beyond the sequence hold 0xFF bytes (NaN patterns): they must not reach the output."""
    import gpu_harness as G

    pool, bt, k, v, q, aq, ctx = make_case(FMT_FP16, 64, [37, 100], [1, 2], 161, DT_F16)
    hb = oracle.HostBatch(aq, [37, 100], bt, context_lens_before=ctx)
    want = oracle.paged_attention(pool, hb, q, DT_F16, 8)
    # poison every row the oracle's write did not touch
    kk = pool.k.reshape(-1, pool.kv_heads, pool.block_size, 512)
    vv = pool.v.reshape(-1, pool.kv_heads, pool.block_size, 512)
    for r, s in enumerate([37, 100]):
        last = bt[r, (s - 1) // 64]
        kk[last, :, s % 64:, :] = 0xFF
        vv[last, :, s % 64:, :] = 0xFF
    dpool = _dev_pool(pool)
    for scratch in (0, SCRATCH):
        rc, got, _ = G.dev_attention(dpool, hb, q, DT_F16, 8, scratch_bytes=scratch)
        assert rc == 0
        G.assert_close(got, DT_F16, want, what="poisoned tail", scale=G.channel_scale(v, DT_F16, hb, 8))


def test_kv16_mismatched_query_type_is_refused():
    import gpu_harness as G

    pool, bt, k, v, q, aq, ctx = make_case(FMT_BF16, 16, [40], [1], 171, DT_BF16)
    hb = oracle.HostBatch(aq, [40], bt, context_lens_before=ctx)
    dpool = _dev_pool(pool)
    rc, got, _ = G.dev_attention(dpool, hb, q, DT_F16, 8)
    assert rc == 801 and (got == 0x5500).all()


# ---- 8-bit pages: FP8-E4M3-256 and Q8_0-64 rows (tail layers of the default TQ4 policy) ----

KV8 = [FMT_FP8, FMT_Q8_0]


@pytest.mark.parametrize("fmt", KV8)
@pytest.mark.parametrize("dtype", [DT_F16, DT_BF16])
@pytest.mark.parametrize("block_size", [16, 64])
def test_kv8_decode_small_batch(fmt, dtype, block_size):
    _check(fmt, dtype, block_size, [70, 33, 129, 1, 32], [1, 1, 1, 1, 1], 211)


@pytest.mark.parametrize("fmt", KV8)
@pytest.mark.parametrize("scratch", [0, SCRATCH])
def test_kv8_decode_gqa8_long(fmt, scratch):
    _check(fmt, DT_F16, 64, [5000], [1], 221, scratch=scratch, q_heads=16)


@pytest.mark.parametrize("fmt", KV8)
def test_kv8_decode_ctx32k(fmt):
    _check(fmt, DT_BF16, 64, [32768], [1], 231, scratch=64 << 20, q_heads=16)


@pytest.mark.parametrize("fmt", KV8)
@pytest.mark.parametrize("q_lens", [[4, 4], [2, 3], [16]])
def test_kv8_verify_multi_token_causal(fmt, q_lens):
    seq = [300 + 7 * i for i in range(len(q_lens))]
    _check(fmt, DT_F16, 64, seq, q_lens, 241, q_heads=16)
    _check(fmt, DT_BF16, 16, seq, q_lens, 242, q_heads=8, scratch=0)


@pytest.mark.parametrize("fmt", KV8)
@pytest.mark.parametrize("mask_mode,window", [(0, 40), (1, 0), (1, 100), (0, 5)])
def test_kv8_windows(fmt, mask_mode, window):
    _check(fmt, DT_F16, 16, [333, 90], [3, 2], 251, mask_mode=mask_mode, window=window, ctx_null=True)


@pytest.mark.parametrize("fmt,dtype,xf", [(FMT_FP8, DT_BF16, XF_IDENTITY), (FMT_Q8_0, DT_F16, XF_WHT256),
                                          (FMT_BF16, DT_BF16, XF_IDENTITY), (FMT_FP16, DT_F16, XF_IDENTITY)])
def test_rows_decode_batch_balanced_shares(fmt, dtype, xf):
    """Decode batches with very different request lengths over 16-bit and 8-bit pages: equal
    shares of units per workgroup, long requests cut into many pieces, several short requests
    worked off by one workgroup."""
    seq = [5000, 300, 9000, 64, 2500, 33, 1, 7777]
    _check(fmt, dtype, 64, seq, [1] * len(seq), 281, q_heads=16, xf=xf)
    _check(fmt, dtype, 16, seq[:5], [2, 1, 2, 1, 2], 282, q_heads=8, xf=xf)


@pytest.mark.parametrize("fmt", KV8)
@pytest.mark.parametrize("scratch", [0, SCRATCH])
def test_kv8_rotated_rows(fmt, scratch):
    """Rows stored after sign + WHT256 (op_kv_cache.cu:36-44,71-99): the kernel rotates the query
    rows and rotates the output back."""
    _check(fmt, DT_F16, 64, [700, 130], [1, 3], 261, scratch=scratch, q_heads=16, xf=XF_WHT256)
    _check(fmt, DT_BF16, 16, [45], [2], 262, scratch=scratch, xf=XF_WHT256)


@pytest.mark.parametrize("fmt", KV8)
def test_kv8_unwritten_pool_bytes_do_not_leak(fmt):
    """Rows beyond the sequence hold 0xFF bytes (NaN codes and NaN scales): they must not reach
    the output."""
    import gpu_harness as G

    pool, bt, k, v, q, aq, ctx = make_case(fmt, 64, [37, 100], [1, 2], 271, DT_F16)
    hb = oracle.HostBatch(aq, [37, 100], bt, context_lens_before=ctx)
    want = oracle.paged_attention(pool, hb, q, DT_F16, 8)
    kk = pool.k.reshape(-1, pool.kv_heads, pool.block_size, pool.tok)
    vv = pool.v.reshape(-1, pool.kv_heads, pool.block_size, pool.tok)
    for r, s in enumerate([37, 100]):
        last = bt[r, (s - 1) // 64]
        kk[last, :, s % 64:, :] = 0xFF
        vv[last, :, s % 64:, :] = 0xFF
    dpool = _dev_pool(pool)
    for scratch in (0, SCRATCH):
        rc, got, _ = G.dev_attention(dpool, hb, q, DT_F16, 8, scratch_bytes=scratch)
        assert rc == 0
        G.assert_close(got, DT_F16, want, what="poisoned tail", scale=G.channel_scale(v, DT_F16, hb, 8))


# ---- chunked prefill over TQ4 pages (128-row tile kernel) ----

def _prefill_case(dtype, block_size, seq_lens, q_lens, seed, q_heads=16, force=None, fmt=FMT_TQ4, xf=None,
                  mask_mode=0, window=0, plain_excess=0.0, **kw):
    import gpu_harness as G

    pool, bt, k, v, q, aq, ctx = make_case(fmt, block_size, seq_lens, q_lens, seed, dtype, q_heads=q_heads, xf=xf)
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx, mask_mode=mask_mode, sliding_window=window, **kw)
    want = oracle.paged_attention(pool, hb, q, dtype, q_heads, n_threads=8)
    dpool = _dev_pool(pool)
    rc, got, _ = G.dev_attention(dpool, hb, q, dtype, q_heads, scratch_bytes=SCRATCH, force_kernel=force)
    assert rc == 0
    G.assert_close(got, dtype, want, what="prefill bs=%d seq=%s q=%s" % (block_size, seq_lens, q_lens),
                   scale=G.channel_scale(v, dtype, hb, q_heads), plain_excess=plain_excess)
    return pool, hb, q, got, want


@pytest.mark.parametrize("block_size", [16, 64])
def test_prefill_tile_kernel_forced_small(block_size):
    """Ragged tiles: chunk lengths that are not multiples of the 16-token tile, one request with
    no prefix, one whose chunk starts in the middle of a page."""
    _prefill_case(DT_F16, block_size, [300, 77, 45], [150, 77, 3], 201, force=2)
    _prefill_case(DT_F16, block_size, [33, 700], [1, 37], 202, q_heads=8, force=1)


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F16])
def test_prefill_tile_kernel_auto_dispatch(dtype):
    """Large enough for the dispatcher to pick the tile kernel by itself: 4 x 300 query tokens."""
    _prefill_case(dtype, 64, [900, 300, 1300, 512], [300, 300, 300, 300], 211)


@pytest.mark.parametrize("mask_mode,window", [(0, 100), (1, 0), (1, 64)])
def test_prefill_tile_kernel_windows(mask_mode, window):
    _prefill_case(DT_F16, 16, [400, 130], [90, 130], 221, force=1, mask_mode=mask_mode, window=window)


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F16])
def test_prefill_tile_kernel_long_chunks(dtype):
    """The TQ4 tile kernel on chunks of a thousand tokens and more, through the automatic dispatch:
    causal chunks on a prefix with ragged last tiles, 4, 8 and 16 q heads per kv head, 16- and
    64-token pages, a sliding window, the non-causal window mode, a token mask, and
    page-permutation invariance."""
    import gpu_harness as G

    _prefill_case(dtype, 64, [1500, 900], [1100, 650], 361)                       # gqa 8: 16-token tiles, ragged tails
    _prefill_case(dtype, 16, [2100, 131], [2100, 90], 362, q_heads=8)             # gqa 4: 32-token tiles, no prefix
    _prefill_case(dtype, 64, [700, 1300], [700, 530], 363, q_heads=32)            # gqa 16: 8-token tiles
    _prefill_case(dtype, 16, [1301, 77], [1301, 40], 364, mask_mode=0, window=200)
    _prefill_case(dtype, 64, [1100], [1100], 365, mask_mode=1, window=96)
    # token mask + two page permutations of the same data
    seq_lens, q_lens = [1400, 300], [1200, 300]
    outs = []
    for perm_seed in (1, 2):
        pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 16, seq_lens, q_lens, 366, dtype, q_heads=16, perm_seed=perm_seed)
        tmask = np.ones(sum(q_lens), dtype=np.uint8)
        tmask[5:40] = 0
        tmask[1199] = 0
        hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx, valid_token_mask=tmask)
        rc, got, _ = G.dev_attention(_dev_pool(pool), hb, q, dtype, 16, scratch_bytes=SCRATCH, sentinel=0x5500)
        assert rc == 0
        outs.append(got)
        if perm_seed == 1:
            want = oracle.paged_attention(pool, hb, q, dtype, 16, n_threads=8)
            live = tmask.astype(bool)
            # fp16 centroid table on rotated outlier rows (mechanism 1 of assert_close): one element
            # of 6 million is 2.8e-4 over the plain bound
            G.assert_close(got[live], dtype, want[live], what="long chunks, token mask",
                           scale=G.channel_scale(v, dtype, hb, 16)[live], plain_excess=4e-4)
            assert np.all(got[~live] == 0x5500), "masked rows must stay untouched"
    assert outs[0].tobytes() == outs[1].tobytes(), "result depends on the physical page numbering"


@pytest.mark.parametrize("fmt", [FMT_FP8, FMT_Q8_0])
@pytest.mark.parametrize("xf", [XF_IDENTITY, XF_WHT256])
@pytest.mark.parametrize("dtype", [DT_BF16, DT_F16])
def test_prefill_tile_kernel_8bit_pages(xf, dtype, fmt):
    """The tile kernel over FP8-E4M3 pages (same row shape as TQ4: two scale blocks of 128) and
    Q8_0 pages (four blocks of 64, dequantised into both tiles), plain and rotated, through the
    automatic dispatch and the test selector."""
    # The value tile holds fp16(d * code) and the probabilities are fp16, as in the reference's MMA
    # kernels (op_paged_attn.cu:59-105): mechanism 2 of assert_close leaves single elements of
    # millions up to 3e-4 over the plain bound.  Rotated value rows keep the codes exact and carry
    # the block scales in two-operand fp16 weights, so they need no more than plain rows.
    ex = 4e-4
    _prefill_case(dtype, 64, [1500, 900], [1100, 650], 331, fmt=fmt, xf=xf, plain_excess=ex)
    if dtype == DT_F16:  # the test selector is an f16 entry point
        _prefill_case(dtype, 16, [300, 77], [130, 40], 332, fmt=fmt, xf=xf, force=1, plain_excess=ex)
        _prefill_case(dtype, 64, [700], [333], 333, fmt=fmt, xf=xf, mask_mode=1, window=64, force=1, plain_excess=ex)


@pytest.mark.parametrize("dtype", [DT_BF16, DT_F16])
def test_prefill_tile_kernel_16bit_pages(dtype):
    """The tile kernel over FP16 / BF16 pages (rows copied as stored, MFMAs in the storage type; BF16
    probabilities split into two bf16 operands), through the automatic dispatch: causal chunks on a
    prefix, a sliding window, and 0xFF-filled rows behind the sequence ends."""
    import gpu_harness as G

    fmt = FMT_BF16 if dtype == DT_BF16 else FMT_FP16
    _prefill_case(dtype, 64, [1500, 900], [1100, 650], 351, fmt=fmt)
    _prefill_case(dtype, 16, [1301, 77], [1301, 40], 352, fmt=fmt, mask_mode=0, window=200)
    seq_lens, q_lens = [1500, 901], [1100, 650]
    pool, bt, k, v, q, aq, ctx = make_case(fmt, 64, seq_lens, q_lens, 353, dtype, q_heads=16)
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx)
    want = oracle.paged_attention(pool, hb, q, dtype, 16, n_threads=8)
    kk = pool.k.reshape(-1, pool.kv_heads, pool.block_size, pool.tok)
    vv = pool.v.reshape(-1, pool.kv_heads, pool.block_size, pool.tok)
    for r, s_ in enumerate(seq_lens):
        last = bt[r, (s_ - 1) // 64]
        kk[last, :, s_ % 64:, :] = 0xFF
        vv[last, :, s_ % 64:, :] = 0xFF
    rc, got, _ = G.dev_attention(_dev_pool(pool), hb, q, dtype, 16, scratch_bytes=SCRATCH)
    assert rc == 0
    G.assert_close(got, dtype, want, what="poisoned tail, 16-bit tile kernel", scale=G.channel_scale(v, dtype, hb, 16))


@pytest.mark.parametrize("fmt", [FMT_FP8, FMT_Q8_0])
def test_prefill_tile_kernel_8bit_unwritten_rows_do_not_leak(fmt):
    """Rows beyond the sequence hold 0xFF bytes (NaN codes, NaN scales) in the last page of each
    request: the tile kernel must keep them out of the P V product."""
    import gpu_harness as G

    seq_lens, q_lens = [1500, 901], [1100, 650]
    pool, bt, k, v, q, aq, ctx = make_case(fmt, 64, seq_lens, q_lens, 341, DT_F16, q_heads=16)
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx)
    want = oracle.paged_attention(pool, hb, q, DT_F16, 16, n_threads=8)
    kk = pool.k.reshape(-1, pool.kv_heads, pool.block_size, pool.tok)
    vv = pool.v.reshape(-1, pool.kv_heads, pool.block_size, pool.tok)
    for r, s in enumerate(seq_lens):
        last = bt[r, (s - 1) // 64]
        kk[last, :, s % 64:, :] = 0xFF
        vv[last, :, s % 64:, :] = 0xFF
    dpool = _dev_pool(pool)
    for force in (None, 1):
        rc, got, _ = G.dev_attention(dpool, hb, q, DT_F16, 16, scratch_bytes=SCRATCH, force_kernel=force)
        assert rc == 0
        G.assert_close(got, DT_F16, want, what="poisoned tail, tile kernel", scale=G.channel_scale(v, DT_F16, hb, 16))


def test_prefill_tile_kernel_masks_and_page_permutation():
    import gpu_harness as G

    seq_lens, q_lens = [200, 120, 64], [40, 50, 64]
    outs = []
    for perm_seed in (1, 2):
        pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 16, seq_lens, q_lens, 231, DT_F16, perm_seed=perm_seed)
        tmask = np.ones(sum(q_lens), dtype=np.uint8)
        tmask[[0, 17, 41, 153]] = 0
        rmask = np.array([1, 0, 1], dtype=np.uint8)
        hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx, valid_token_mask=tmask, valid_req_mask=rmask)
        want = oracle.paged_attention(pool, hb, q, DT_F16, 8)
        dpool = _dev_pool(pool)
        rc, got, _ = G.dev_attention(dpool, hb, q, DT_F16, 8, force_kernel=1, sentinel=0x5500)
        assert rc == 0
        dead = np.zeros(sum(q_lens), dtype=bool)
        dead[[0, 17, 41, 153]] = True
        dead[40:90] = True  # masked request
        assert (got[dead] == 0x5500).all()
        G.assert_close(got[~dead], DT_F16, want[~dead], what="prefill masks",
                       scale=G.channel_scale(v, DT_F16, hb, 8)[~dead])
        outs.append(got)
    assert outs[0].tobytes() == outs[1].tobytes()


def test_verify_with_shared_prefix_pages():
    """MTP-style verify: three requests share the block-table entries of a 640-token prefix
    (whole pages, as the prefix cache hands them out), each has a private suffix and verifies
    4 query tokens with causal masking among them."""
    import gpu_harness as G

    bs, prefix, suffixes, ql, q_heads, kv_heads = 64, 640, [130, 71, 200], 4, 16, 2
    n_prefix_pages = prefix // bs
    priv_pages = [(prefix + s + bs - 1) // bs - n_prefix_pages for s in suffixes]
    num_pages = n_prefix_pages + sum(priv_pages) + 2
    perm = oracle.permutation(num_pages, 9)
    pool = oracle.HostPool(num_pages, kv_heads, 256, bs, FMT_TQ4, oracle.XF_WHT256)
    mb = n_prefix_pages + max(priv_pages)
    bt = np.zeros((len(suffixes), mb), dtype=np.int32)
    at = n_prefix_pages
    for r, pp in enumerate(priv_pages):
        bt[r, :n_prefix_pages] = perm[:n_prefix_pages]
        bt[r, n_prefix_pages:n_prefix_pages + pp] = perm[at:at + pp]
        at += pp
    # the prefix is appended once (through request 0's table), every suffix separately
    k = oracle.fill_kv_rows(prefix, kv_heads, 256, 301, DT_BF16, 3)
    v = oracle.fill_kv_rows(prefix, kv_heads, 256, 302, DT_BF16, 3)
    wb = oracle.HostBatch([0, prefix], [prefix], bt[:1], context_lens_before=[0],
                          write_slot_mapping=oracle.slot_mapping(bt[0], 0, prefix, bs))
    oracle.kv_cache_write(pool, wb, k, v, DT_BF16)
    v_rows = []
    for r, s in enumerate(suffixes):
        ks = oracle.fill_kv_rows(s, kv_heads, 256, 310 + r, DT_BF16, 3)
        vs = oracle.fill_kv_rows(s, kv_heads, 256, 320 + r, DT_BF16, 3)
        v_rows += [v, vs]
        wb = oracle.HostBatch([0, s], [prefix + s], bt[r:r + 1], context_lens_before=[prefix],
                              write_slot_mapping=oracle.slot_mapping(bt[r], prefix, s, bs))
        oracle.kv_cache_write(pool, wb, ks, vs, DT_BF16)
    seq = [prefix + s for s in suffixes]
    aq = [0, ql, 2 * ql, 3 * ql]
    q = oracle.fill_normal(3 * ql * q_heads * 256, 330, DT_BF16).reshape(3 * ql, q_heads, 256)
    hb = oracle.HostBatch(aq, seq, bt, context_lens_before=[s - ql for s in seq])
    want = oracle.paged_attention(pool, hb, q, DT_BF16, q_heads, n_threads=4)
    dpool = _dev_pool(pool)
    for scratch in (0, SCRATCH):
        rc, got, _ = G.dev_attention(dpool, hb, q, DT_BF16, q_heads, scratch_bytes=scratch)
        assert rc == 0
        G.assert_close(got, DT_BF16, want, what="shared prefix, scratch %d" % scratch,
                       scale=G.channel_scale(np.concatenate(v_rows), DT_BF16, hb, q_heads))
