"""Verify batches whose requests share their leading pages: the shared keys go through the tile
kernel once for all query rows of the batch, the private rest through the decode kernel, one merge
(no counterpart in the reference, which runs such a batch without any split,
op_paged_attn.cu:1399-1415).  The pass is chosen from the batch shape and the scratch size only;
what is shared is found on the device."""
import numpy as np
import pytest

import oracle
from oracle import DT_BF16

pytestmark = pytest.mark.gpu

Q_HEADS, D = 16, 256
BIG = 96 << 20    # scratch that admits the wide partial records of the pass
SMALL = 8 << 20   # scratch that does not: the plain split-K path


def _case(ctx, q_len, shared, seed):
    from test_gpu_full_size import BS, BigPool

    R = len(ctx)
    pages = sum((c + BS - 1) // BS for c in ctx) + 8
    pool = BigPool(ctx, pages, seed=seed, shared_prefix=shared)
    q = oracle.fill_normal(R * q_len * Q_HEADS * D, seed + 1, DT_BF16).reshape(R * q_len, Q_HEADS, D)
    hb = oracle.HostBatch(np.arange(R + 1) * q_len, pool.ctx, pool.bt, context_lens_before=[c - q_len for c in pool.ctx])
    return pool, hb, q


def _run(pool, hb, q, scratch):
    rc, got, _ = pool.G.dev_attention(pool.dev, hb, q, DT_BF16, Q_HEADS, scratch_bytes=scratch)
    assert rc == 0
    return got


@pytest.mark.parametrize("q_len", [4, 2])
def test_shared_prefix_verify_matches_oracle(q_len):
    """Requests of different lengths over a 32 768-token common prefix (the pass wants at least 16 query tokens)."""
    ctx = [40000, 40037, 41111, 39000, 40960, 40001] if q_len == 4 else [40000, 40037, 41111, 39000, 40960, 40001, 38000, 42000]
    pool, hb, q = _case(ctx, q_len, 32768, seed=901 + q_len)
    want = oracle.paged_attention(pool.host, hb, q, DT_BF16, Q_HEADS, n_threads=oracle.hw_threads())
    got = _run(pool, hb, q, BIG)
    pool.G.assert_close(got, DT_BF16, want, what="shared prefix, pass taken", scale=pool.scale_for(hb))
    plain = _run(pool, hb, q, SMALL)
    pool.G.assert_close(plain, DT_BF16, want, what="shared prefix, plain path", scale=pool.scale_for(hb))
    # the two paths add the same products in different orders: were the bytes equal, the pass was not taken
    assert got.tobytes() != plain.tobytes()


def test_shared_prefix_limited_by_the_shortest_request():
    """One request ends inside the common pages: only the keys below ITS first query position count
    as shared (its later positions are not visible to its own queries)."""
    ctx = [40000, 20010, 40500, 39990]
    pool, hb, q = _case(ctx, 4, 20000 // 64 * 64, seed=911)
    want = oracle.paged_attention(pool.host, hb, q, DT_BF16, Q_HEADS, n_threads=oracle.hw_threads())
    got = _run(pool, hb, q, BIG)
    pool.G.assert_close(got, DT_BF16, want, what="shared prefix, short request", scale=pool.scale_for(hb))


def test_nothing_shared_gives_the_plain_path_bits():
    """Same batch shape, unrelated block tables: the probe finds no common run, the tile kernel's
    records are empty and the result has the bits of the plain split-K path."""
    ctx = [33000, 34000, 35000, 36000]
    pool, hb, q = _case(ctx, 4, 0, seed=921)
    got = _run(pool, hb, q, BIG)
    plain = _run(pool, hb, q, SMALL)
    assert got.tobytes() == plain.tobytes()
    want = oracle.paged_attention(pool.host, hb, q, DT_BF16, Q_HEADS, n_threads=oracle.hw_threads())
    pool.G.assert_close(got, DT_BF16, want, what="nothing shared", scale=pool.scale_for(hb))


def test_one_kv_head_layouts_give_the_same_bytes():
    """The pass on a rank that holds one kv head computes the bits of a rank that holds both
    (op_paged_attn.cu:1301-1304): same parts, same records, same merge order."""
    from warp34_amd import ffi

    ctx = [40000, 40037, 41111, 39000]
    pool, hb, q = _case(ctx, 4, 32768, seed=931)
    full = _run(pool, hb, q, BIG)
    assert full.tobytes() != _run(pool, hb, q, SMALL).tobytes()  # the pass is taken
    d, h = pool.dev, pool.dev.h
    for head in range(2):
        lay = ffi.Warp34KvLayerLayout(d.k.data_ptr() + head * h.head, d.v.data_ptr() + head * h.head, h.page, h.head, h.tok,
                                      h.page, h.head, h.tok, 0, 0, 1, h.head_dim, h.block_size, h.fmt, h.fmt,
                                      h.transform, h.transform, 0)
        q_h = np.ascontiguousarray(q[:, head * 8:(head + 1) * 8])
        rc, part, _ = pool.G.dev_attention(pool.dev, hb, q_h, DT_BF16, 8, scratch_bytes=BIG, layout=lay)
        assert rc == 0
        assert part.tobytes() == np.ascontiguousarray(full[:, head * 8:(head + 1) * 8]).tobytes()


def test_gated_entry_through_the_pass():
    """The gate of warp34_paged_attention_gated_f16 is applied where the merged rows are stored, so through
    the pass too it equals attention followed by warp34_apply_attn_output_gate_f16, byte for byte
    (model/forward.rs:1192-1211 makes the two calls)."""
    from oracle import DT_F16
    from test_gpu_full_size import BS, BigPool
    from test_gpu_output_gate import _run as gate_op

    ctx, q_len = [40000, 40037, 41111, 39000], 4
    R = len(ctx)
    pool = BigPool(ctx, sum((c + BS - 1) // BS for c in ctx) + 8, seed=951, shared_prefix=32768)
    n = R * q_len
    q = oracle.fill_normal(n * Q_HEADS * D, 952, DT_F16).reshape(n, Q_HEADS, D)
    hb = oracle.HostBatch(np.arange(R + 1) * q_len, pool.ctx, pool.bt, context_lens_before=[c - q_len for c in pool.ctx])
    gate = oracle.f32_to_f16_bits(3.0 * oracle.f16_bits_to_f32(oracle.fill_normal(n * Q_HEADS * D, 953, DT_F16)))
    gate = gate.reshape(n, Q_HEADS * D)
    rc, plain, _ = pool.G.dev_attention(pool.dev, hb, q, DT_F16, Q_HEADS, scratch_bytes=BIG)
    assert rc == 0
    rc, small, _ = pool.G.dev_attention(pool.dev, hb, q, DT_F16, Q_HEADS, scratch_bytes=SMALL)
    assert rc == 0 and plain.tobytes() != small.tobytes()  # the pass is taken
    rc, want = gate_op(plain.reshape(n, Q_HEADS * D), gate)
    assert rc == 0
    rc, got, _ = pool.G.dev_attention(pool.dev, hb, q, DT_F16, Q_HEADS, scratch_bytes=BIG, gate=gate)
    assert rc == 0
    assert got.reshape(n, Q_HEADS * D).tobytes() == want.tobytes()
    ref = oracle.paged_attention(pool.host, hb, q, DT_F16, Q_HEADS, n_threads=oracle.hw_threads())
    pool.G.assert_close(plain, DT_F16, ref, what="shared prefix, fp16 queries", scale=pool.scale_for(hb))
