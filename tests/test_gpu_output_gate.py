"""GPU parity: output gate through the C ABI vs the CPU oracle.  Both compute in fp32 with their
own expf (each within one fp32 ulp of the true value), so the fp16 results agree except where the
product sits on a rounding boundary: at most one fp16 ulp apart, and equal in all but a few
elements per million (the sign of a zero product and the double rounding fp32 -> fp16 included).
The attention entry point that applies the gate itself is held to the bytes of the two calls."""
import ctypes as C

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu


def _run(a_bits, g_bits, mask=None, sentinel=0x5500):
    import gpu_harness as G
    import torch

    l = G.lib()
    ex, _ = G.make_exec()
    da, dg = G.to_dev(a_bits), G.to_dev(g_bits)
    out = torch.full(a_bits.shape, sentinel, dtype=torch.int16, device=G.DEV)
    dm = None if mask is None else G.to_dev(np.asarray(mask, np.uint8))
    rc = l.warp34_apply_attn_output_gate_f16(C.byref(ex), G.ptr(da), G.ptr(dg), C.c_void_p(out.data_ptr()),
                                             None if dm is None else G.ptr(dm), a_bits.shape[0], a_bits.shape[1])
    torch.cuda.synchronize()
    return rc, out.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("tokens,dim", [(37, 4096), (5, 4100), (3, 7), (2048, 4096)])
def test_output_gate_matches_oracle(tokens, dim):
    rng = np.random.default_rng(tokens)
    a = (rng.standard_normal((tokens, dim)) * 2).astype(np.float16).view(np.uint16)
    g = (rng.standard_normal((tokens, dim)) * 3).astype(np.float16).view(np.uint16)
    rc, got = _run(a, g)
    assert rc == 0
    want = oracle.apply_attn_output_gate_f16(a, g)
    gf, wf = got.view(np.float16).astype(np.float64), want.view(np.float16).astype(np.float64)
    ulp = np.maximum(np.abs(wf), 2.0 ** -14) * 2.0 ** -10
    assert (np.abs(gf - wf) <= ulp * 1.001).all()
    print("output gate %dx%d: %d of %d elements differ from the oracle" % (tokens, dim, int((got != want).sum()), got.size))
    assert (got == want).mean() > 0.9999


def test_output_gate_mask_and_validation():
    from warp34_amd import ffi
    import gpu_harness as G

    rng = np.random.default_rng(9)
    a = rng.standard_normal((6, 256)).astype(np.float16).view(np.uint16)
    g = rng.standard_normal((6, 256)).astype(np.float16).view(np.uint16)
    mask = [1, 0, 1, 1, 0, 1]
    rc, got = _run(a, g, mask=mask)
    assert rc == 0
    want = oracle.apply_attn_output_gate_f16(a, g, out=np.full((6, 256), 0x5500, np.uint16), valid_token_mask=mask)
    assert (got[1] == 0x5500).all() and (got[4] == 0x5500).all()
    assert (got == want).mean() > 0.9999
    l = G.lib()
    ex, _ = G.make_exec()
    d = G.to_dev(a)
    assert l.warp34_apply_attn_output_gate_f16(C.byref(ex), None, G.ptr(d), G.ptr(d), None, 6, 256) == ffi.HIP_ERROR_INVALID_VALUE
    assert l.warp34_apply_attn_output_gate_f16(C.byref(ex), G.ptr(d), G.ptr(d), G.ptr(d), None, 0, 256) == 0


# (format, transform, page tokens, kv heads, q heads per kv head, sequence lengths, query lengths, scratch bytes,
#  masked token, masked request): one case per kernel that stores output rows
GATED_CASES = [
    (oracle.FMT_TQ4, 1, 16, 2, 8, [700], [1], 0, None, None),                      # decode kernel, one pass
    (oracle.FMT_TQ4, 1, 16, 2, 8, [9000], [1], 1 << 24, None, None),               # split-K + merge
    (oracle.FMT_TQ4, 1, 16, 2, 8, [3000, 40, 1500, 0 + 7], [1, 1, 1, 1], 1 << 24, None, 1),  # balanced shares + merge
    (oracle.FMT_TQ4, 1, 16, 1, 16, [600, 900], [3, 4], 1 << 24, 2, None),          # verify tiles, a masked token
    (oracle.FMT_TQ4, 1, 16, 2, 8, [300, 520], [260, 500], 0, None, None),          # tile kernel (prefill)
    (oracle.FMT_FP16, 0, 32, 2, 4, [2500, 130], [1, 1], 1 << 24, None, None),      # 16-bit rows, balanced
    (oracle.FMT_FP16, 0, 16, 1, 8, [5000], [2], 1 << 24, None, None),              # 16-bit rows, split-K
    (oracle.FMT_FP8, 1, 16, 2, 8, [800, 90], [5, 1], 0, None, None),               # rotated 8-bit rows
    (oracle.FMT_Q8_0, 0, 16, 2, 8, [200, 420], [180, 400], 0, None, None),         # 8-bit pages, tile kernel
]


@pytest.mark.parametrize("case", GATED_CASES, ids=lambda c: "fmt%d-seq%s-q%s-ws%d" % (c[0], "_".join(map(str, c[5])), "_".join(map(str, c[6])), c[7]))
def test_gated_attention_equals_attention_then_gate(case):
    """warp34_paged_attention_gated_f16 == warp34_paged_attention_f16 + warp34_apply_attn_output_gate_f16, byte
    for byte (model/forward.rs:1192-1211 makes the two calls), rows of masked tokens and requests untouched."""
    import gpu_harness as G
    from cases import make_case

    fmt, xf, bs, kv_heads, gqa, seq_lens, q_lens, scratch, masked_tok, masked_req = case
    q_heads = kv_heads * gqa
    pool, bt, k, v, q, aq, ctx = make_case(fmt, bs, seq_lens, q_lens, 4000 + fmt + len(seq_lens), oracle.DT_F16,
                                           kv_heads=kv_heads, q_heads=q_heads, xf=xf)
    n = aq[-1]
    tmask = rmask = None
    if masked_tok is not None:
        tmask = np.ones(n, np.uint8)
        tmask[masked_tok] = 0
    if masked_req is not None:
        rmask = np.ones(len(seq_lens), np.uint8)
        rmask[masked_req] = 0
    hb = oracle.HostBatch(aq, seq_lens, bt, context_lens_before=ctx, valid_token_mask=tmask, valid_req_mask=rmask)
    gate = oracle.f32_to_f16_bits(3.0 * oracle.f16_bits_to_f32(oracle.fill_normal(n * q_heads * 256, 77, oracle.DT_F16)))
    gate = gate.reshape(n, q_heads * 256)
    gate[0, :8] = [0x7C00, 0xFC00, 0x7E00, 0x0000, 0x8000, 0x7BFF, 0xFBFF, 0x0001]  # inf, -inf, nan, zeros, extremes
    dpool = G.DevPool(pool)
    dpool.upload()
    rc, plain, _ = G.dev_attention(dpool, hb, q, oracle.DT_F16, q_heads, scratch_bytes=scratch)
    assert rc == 0
    rc, want = _run(plain.reshape(n, q_heads * 256), gate, mask=tmask)
    assert rc == 0
    rc, got, _ = G.dev_attention(dpool, hb, q, oracle.DT_F16, q_heads, scratch_bytes=scratch, gate=gate)
    assert rc == 0
    got = got.reshape(n, q_heads * 256)
    untouched = (plain.reshape(n, q_heads * 256) == 0x5500).all(axis=1)  # rows the attention left alone
    if masked_tok is not None or masked_req is not None:
        assert untouched.any()
    want[untouched] = 0x5500  # the separate gate op would process a masked request's sentinel rows; the fused one never sees them
    nan = lambda a: (a & 0x7C00 == 0x7C00) & (a & 0x3FF != 0)
    assert (nan(got) == nan(want)).all()
    bad = np.argwhere((got != want) & ~nan(got))
    ow = oracle.apply_attn_output_gate_f16(plain.reshape(n, q_heads * 256), gate)
    pl = plain.reshape(n, q_heads * 256)
    assert len(bad) == 0, "%d differ, first %s: got %s want %s oracle %s attn %s gate %s" % (
        len(bad), bad[:4].tolist(), [hex(got[tuple(b)]) for b in bad[:4]], [hex(want[tuple(b)]) for b in bad[:4]],
        [hex(ow[tuple(b)]) for b in bad[:4]], [hex(pl[tuple(b)]) for b in bad[:4]], [hex(gate[tuple(b)]) for b in bad[:4]])
    # and the plain output agrees with the oracle's gate applied to it (one ulp where expf differs)
    ow = oracle.apply_attn_output_gate_f16(plain.reshape(n, q_heads * 256), gate)
    live = ~untouched
    assert (got[live] == ow[live]).mean() > 0.9999
