"""Outputs must not depend on how many kv heads a rank holds: a tensor-parallel rank that owns
one kv head computes each of its rows with exactly the bits a rank that owns all of them does
(op_paged_attn.cu:1301-1304: the split count depends only on TP-invariant batch geometry;
crates/warp34-host/tests/tq4_vision_and_moe.rs:1336-1351 compares TP=1 with TP=2 at 0 ULP).

One GPU is enough: the batch is run once over the two-kv-head layout and once per kv head over a
one-kv-head layout that addresses the same slabs (base + head * head_stride, same page stride),
with that head's query rows, and the output BYTES are compared.  Split-K (long single request,
where the chunk cap binds), balanced decode shares, verify tiles, single pass (no scratch)."""
import numpy as np
import pytest

import oracle
from oracle import DT_BF16, DT_F16, FMT_BF16, FMT_FP8, FMT_TQ4
from cases import make_case
from warp34_amd import ffi

pytestmark = pytest.mark.gpu
SCRATCH = 16 << 20
KV_HEADS, GQA = 2, 8


def _head_layout(dpool, head):
    h = dpool.h
    return ffi.Warp34KvLayerLayout(
        dpool.k.data_ptr() + head * h.head, dpool.v.data_ptr() + head * h.head, h.page, h.head, h.tok, h.page,
        h.head, h.tok, 0, 0, 1, h.head_dim, h.block_size, h.fmt, h.fmt, h.transform, h.transform, 0)


CASES = [
    # format, query type, page tokens, sequence lengths, query lengths
    (FMT_TQ4, DT_BF16, 64, [70000], [1]),                  # split-K, more units than the chunk cap allows
    (FMT_TQ4, DT_F16, 16, [9000, 300, 4100, 77], [1, 1, 1, 1]),  # balanced shares
    (FMT_TQ4, DT_BF16, 64, [5000, 2100], [4, 3]),          # verify tiles
    (FMT_BF16, DT_BF16, 64, [40000], [1]),                 # row-format kernel, split-K
    (FMT_FP8, DT_F16, 32, [6000, 900, 2500], [1, 1, 1]),   # row-format kernel, balanced shares
]


@pytest.mark.parametrize("scratch", [0, SCRATCH])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "fmt%d-seq%d-q%d" % (c[0], c[3][0], c[4][0]))
def test_one_kv_head_layouts_give_the_same_bytes(case, scratch):
    import gpu_harness as G

    fmt, dtype, block_size, seq_lens, q_lens = case
    q_heads = KV_HEADS * GQA
    pool, bt, k, v, q, aq, ctx = make_case(fmt, block_size, seq_lens, q_lens, 4242, dtype, kv_heads=KV_HEADS,
                                           q_heads=q_heads)
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx)
    dpool = G.DevPool(pool)
    dpool.upload()
    rc, full, _ = G.dev_attention(dpool, hb, q, dtype, q_heads, scratch_bytes=scratch)
    assert rc == 0
    for head in range(KV_HEADS):
        q_h = np.ascontiguousarray(q[:, head * GQA:(head + 1) * GQA])
        rc, part, _ = G.dev_attention(dpool, hb, q_h, dtype, GQA, scratch_bytes=scratch,
                                      layout=_head_layout(dpool, head))
        assert rc == 0
        assert part.tobytes() == np.ascontiguousarray(full[:, head * GQA:(head + 1) * GQA]).tobytes(), \
            "kv head %d differs between the two-head and the one-head layout" % head


@pytest.mark.parametrize("fmt,dtype", [(FMT_TQ4, DT_BF16), (FMT_BF16, DT_BF16)])
def test_split_k_does_not_depend_on_the_sequence_bound(fmt, dtype):
    """One long request (per-request chunks, not balanced shares) under two host bounds
    max_seq_len: the bound shapes the launch and the partial layout, never a chunk."""
    import gpu_harness as G

    seq = 20000 if fmt == FMT_TQ4 else 12000
    pool, bt, k, v, q, aq, ctx = make_case(fmt, 64, [seq], [1], 4343, dtype, kv_heads=KV_HEADS, q_heads=16)
    hb = oracle.HostBatch(aq, [seq], bt, context_lens_before=ctx)
    dpool = G.DevPool(pool)
    dpool.upload()
    outs = []
    for bound in (None, seq + 1, 65536, 262144):
        rc, out, _ = G.dev_attention(dpool, hb, q, dtype, 16, scratch_bytes=SCRATCH, max_seq_len=bound)
        assert rc == 0
        outs.append(out.tobytes())
    assert all(o == outs[0] for o in outs[1:])
