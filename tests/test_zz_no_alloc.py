"""warp34_paged_attention_bf16_static_scratch: the attention entry point that allocates nothing
(split-K partials in a device array inside the library).  Called through the C ABI with an exec
that carries no scratch, and compared byte for byte with warp34_paged_attention_bf16 given an
8 MiB scratch, on two calls in a row, the second with a smaller input (the array keeps the first
call's contents); batches whose full split wants more than the array run as they do with an 8 MiB
scratch; a batch with more query rows than the entry point's limit is refused."""
import ctypes as C

import numpy as np
import pytest

import oracle
from oracle import DT_BF16, FMT_BF16, FMT_TQ4
from cases import make_case

pytestmark = pytest.mark.gpu
STATIC_BYTES = 8 << 20


def _both(fmt, block_size, seq_lens, q_lens, seed, q_heads=16):
    import torch

    import gpu_harness as G

    pool, bt, k, v, q, aq, ctx = make_case(fmt, block_size, seq_lens, q_lens, seed, DT_BF16, q_heads=q_heads)
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx)
    dpool = G.DevPool(pool)
    dpool.upload()
    rc, want, _ = G.dev_attention(dpool, hb, q, DT_BF16, q_heads, scratch_bytes=STATIC_BYTES)
    assert rc == 0
    L = dpool.layout()
    db = G.DevBatch(hb)
    B = db.struct()
    ex, _ = G.make_exec(0)  # no scratch
    qd = G.to_dev(q)
    out = torch.full((hb.total_tokens, q_heads, 256), 0x5500, dtype=torch.int16, device=G.DEV)
    rc = G.lib().warp34_paged_attention_bf16_static_scratch(C.byref(ex), C.byref(L), C.byref(B), G.ptr(qd), G.ptr(out),
                                                            q_heads)
    torch.cuda.synchronize()
    assert rc == 0
    got = out.cpu().numpy().view(np.uint16)
    assert got.tobytes() == want.tobytes(), "static-scratch entry point differs from warp34_paged_attention_bf16"
    # and both are the oracle's answer
    ref = oracle.paged_attention(pool, hb, q, DT_BF16, q_heads, n_threads=8)
    G.assert_close(got, DT_BF16, ref, what="static scratch seq=%s" % seq_lens, scale=G.channel_scale(v, DT_BF16, hb, q_heads))


def test_static_scratch_entry_point_matches_on_two_calls_in_a_row():
    _both(FMT_TQ4, 64, [20000], [1], 9101)               # split-K: 79 chunks of partials in the array
    _both(FMT_TQ4, 64, [3000, 700], [1, 1], 9102)        # smaller, balanced shares: the array holds stale partials
    _both(FMT_TQ4, 16, [900], [4], 9103)                 # verify tile
    _both(FMT_BF16, 64, [5000], [1], 9104)               # row-format kernel


def test_static_scratch_entry_point_degrades_like_an_8mib_scratch():
    """Shapes whose full split wants more than the array (a verify batch that may take the
    shared-prefix pass: 38 slots per row; a decode batch of 200 requests: 328 shares) run as
    warp34_paged_attention_bf16 runs them with 8 MiB, byte for byte."""
    _both(FMT_TQ4, 64, [33000, 33100, 34000, 32900], [4, 4, 4, 4], 9106)
    _both(FMT_TQ4, 16, [40] * 200, [1] * 200, 9107)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    import torch

    import gpu_harness as G

    n_req = 260  # 260 x 16 = 4160 query rows: two records per row no longer fit in 8 MiB
    seq_lens = [40] * n_req
    pool, bt, k, v, q, aq, ctx = make_case(FMT_TQ4, 16, seq_lens, [1] * n_req, 9105, DT_BF16, q_heads=16)
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx)
    dpool = G.DevPool(pool)
    dpool.upload()
    L = dpool.layout()
    assert n_req * 16 * 2 * 1040 > STATIC_BYTES
    db = G.DevBatch(hb)
    B = db.struct()
    ex, _ = G.make_exec(0)
    qd = G.to_dev(q)
    out = torch.full((n_req, 16, 256), 0x5500, dtype=torch.int16, device=G.DEV)
    rc = G.lib().warp34_paged_attention_bf16_static_scratch(C.byref(ex), C.byref(L), C.byref(B), G.ptr(qd), G.ptr(out), 16)
    torch.cuda.synchronize()
    assert rc == 2  # hipErrorOutOfMemory: refused, nothing launched
    assert bool((out == 0x5500).all())
