"""GPU parity over shapes the other attention tests do not use: 32- and 128-token pages, 1 and 4 kv
heads, 1, 2 and 16 q heads per kv head, every page format, decode / verify / prefill / mixed
batches with windows and both mask modes, with no, a too small and a large scratch.

The cases are fixed (drawn once from a randomised soak of the entry points against the oracle);
the tolerance is the one of tests/test_gpu_attention.py (gpu_harness.assert_close)."""
import numpy as np
import pytest

import oracle
from cases import make_case

pytestmark = pytest.mark.gpu

# (format, transform, query type, page tokens, kv heads, q heads per kv head, sequence lengths, query lengths,
#  mask mode, sliding window, scratch bytes, seed)
CASES = [
    (0, 0, 0, 32, 1, 2, [5194, 3110, 11, 204, 4656], [1, 1, 1, 1, 1], 1, 226, 0, 48739),  # decode
    (0, 0, 0, 128, 1, 1, [1823, 2839, 352], [6, 8, 2], 0, 77, 4096, 231294),  # verify
    (0, 0, 0, 128, 1, 2, [1106, 1015, 1501, 268, 427], [852, 798, 1112, 228, 172], 1, 0, 0, 130220),  # prefill
    (0, 0, 0, 128, 1, 16, [498, 520], [74, 25], 1, 118, 4096, 886463),  # mixed
    (1, 0, 1, 32, 1, 2, [120, 2182, 3668, 5], [1, 1, 1, 1], 1, 196, 16777216, 872035),  # decode
    (1, 0, 1, 128, 1, 16, [2603, 1351, 409, 986], [3, 6, 1, 5], 1, 308, 16777216, 880060),  # verify
    (1, 0, 1, 32, 1, 16, [87, 373], [79, 132], 1, 0, 0, 400047),  # prefill
    (1, 0, 1, 32, 1, 1, [2376, 1524, 2222], [175, 300, 222], 0, 399, 16777216, 341381),  # mixed
    (2, 1, 1, 128, 4, 16, [3243, 3412, 1192, 2391], [1, 1, 1, 1], 1, 44, 16777216, 21611),  # decode
    (2, 1, 1, 32, 1, 2, [3757, 5744], [1, 1], 0, 128, 0, 70672),  # decode
    (2, 1, 0, 32, 4, 16, [484, 1186], [8, 6], 1, 38, 0, 482816),  # verify
    (2, 1, 0, 128, 1, 2, [780, 2935, 2823], [4, 3, 5], 0, 174, 16777216, 329588),  # verify
    (2, 1, 1, 128, 4, 1, [1301, 258, 402], [547, 204, 278], 0, 299, 16777216, 693265),  # prefill
    (2, 1, 1, 16, 1, 2, [1456], [841], 1, 166, 16777216, 768210),  # prefill
    (2, 1, 1, 16, 4, 2, [1733, 2166, 1663, 1568], [183, 9, 14, 136], 1, 24, 16777216, 190647),  # mixed
    (2, 1, 0, 32, 4, 2, [365, 865, 1305, 973, 877], [198, 37, 119, 31, 212], 0, 150, 0, 862798),  # mixed
    (3, 0, 0, 32, 1, 1, [4168, 2669, 3768], [1, 1, 1], 1, 0, 0, 927363),  # decode
    (3, 0, 0, 16, 1, 2, [551], [5], 1, 244, 0, 680572),  # verify
    (3, 1, 0, 16, 1, 2, [891, 661, 1081, 454, 1451], [882, 630, 880, 330, 1342], 1, 52, 16777216, 489762),  # prefill
    (3, 1, 0, 128, 4, 16, [2352], [24], 0, 293, 16777216, 615901),  # mixed
    (4, 0, 1, 128, 1, 2, [3484], [1], 0, 181, 4096, 663741),  # decode
    (4, 0, 1, 128, 1, 16, [2405, 1897], [5, 8], 1, 0, 16777216, 93091),  # verify
    (4, 0, 0, 32, 4, 1, [336, 1772], [258, 1649], 1, 285, 16777216, 253449),  # prefill
    (4, 1, 1, 128, 1, 2, [2380, 1283, 1542, 2473, 321], [175, 250, 51, 57, 94], 1, 55, 4096, 266641),  # mixed
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "fmt%d-bs%d-kv%dx%d-seed%d" % (c[0], c[3], c[4], c[5], c[11]))
def test_attention_shape(case):
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
    G.assert_close(got, dtype, want, what="fmt=%d bs=%d seq=%s q=%s" % (fmt, block_size, seq_lens, q_lens),
                   scale=G.channel_scale(v, dtype, hb, q_heads))
