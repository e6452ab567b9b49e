"""GPU parity: QK RMSNorm + RoPE (+ fused paged KV write) through the C ABI vs the CPU oracle --
bit-exact (bf16 outputs, cache rows in every page format), and fused == operator + append, the
reference's own check (tests/dflash_proposer.rs:371-520: reversed page table, a negative slot,
0x7E7E sentinels)."""
import ctypes as C

import numpy as np
import pytest

import oracle
from oracle import DT_BF16, FMT_BF16, FMT_FP8, FMT_Q8_0, FMT_TQ4, XF_IDENTITY, XF_WHT256

pytestmark = pytest.mark.gpu


def _case(rows, seed, dim, q_heads, kv_heads, table_rows=96):
    rng = np.random.default_rng(seed)
    qkv = oracle.f32_to_bf16_bits(rng.standard_normal((rows, (q_heads + 2 * kv_heads) * dim)).astype(np.float32) * 1.7)
    qw = oracle.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(dim)).astype(np.float32))
    kw = oracle.f32_to_bf16_bits((1.0 + 0.2 * rng.standard_normal(dim)).astype(np.float32))
    pos = rng.integers(0, table_rows, size=rows).astype(np.int32)
    half = dim // 2
    inv_freq = 1.0 / (10000.0 ** (np.arange(half) / half))
    ang = np.arange(table_rows)[:, None] * inv_freq[None, :]
    table = np.concatenate([np.cos(ang), np.sin(ang)], axis=1).astype(np.float32)
    return qkv, qw, kw, pos, table


def _dev_call(name, qkv, pos, qw, kw, table, q_heads, kv_heads, dim, eps, q_out=None, dpool=None, slots=None,
              layout=None, rows=None):
    import gpu_harness as G
    import torch

    l = G.lib()
    ex, _ = G.make_exec()
    d_qkv, d_pos, d_qw, d_kw, d_tab = G.to_dev(qkv), G.to_dev(pos), G.to_dev(qw), G.to_dev(kw), G.to_dev(table)
    d_qout = None if q_out is None else G.to_dev(q_out)
    rows, table_rows = qkv.shape[0] if rows is None else rows, table.shape[0]
    fn = getattr(l, name)
    if name == "warp34_dflash_qk_norm_rope_kv_write_bf16_f32_table":
        L = dpool.layout() if layout is None else layout
        d_slots = G.to_dev(slots)
        rc = fn(C.byref(ex), G.ptr(d_qkv), None if d_qout is None else G.ptr(d_qout), G.ptr(d_pos), G.ptr(d_qw),
                G.ptr(d_kw), G.ptr(d_tab), C.byref(L), G.ptr(d_slots), rows, q_heads, kv_heads, dim, table_rows, eps)
    elif name == "warp34_dflash_qk_norm_rope_bf16_f32_table_qout":
        rc = fn(C.byref(ex), G.ptr(d_qkv), None if d_qout is None else G.ptr(d_qout), G.ptr(d_pos), G.ptr(d_qw),
                G.ptr(d_kw), G.ptr(d_tab), rows, q_heads, kv_heads, dim, table_rows, eps)
    else:
        rc = fn(C.byref(ex), G.ptr(d_qkv), G.ptr(d_pos), G.ptr(d_qw), G.ptr(d_kw), G.ptr(d_tab), rows, q_heads,
                kv_heads, dim, table_rows, eps)
    torch.cuda.synchronize()
    got = d_qkv.cpu().numpy().view(np.uint16).reshape(qkv.shape)
    got_q = None if d_qout is None else d_qout.cpu().numpy().view(np.uint16).reshape(q_out.shape)
    return rc, got, got_q


@pytest.mark.parametrize("dim,q_heads,kv_heads", [(256, 16, 4), (128, 8, 2), (256, 3, 1), (64, 4, 4), (96, 2, 2)])
def test_operator_in_place_bit_exact(dim, q_heads, kv_heads):
    """fp32-table and bf16-table entry points, Q in place; head sizes below 256, an odd number of
    Q heads, a head size whose halves are not a multiple of the 32 lanes."""
    qkv, qw, kw, pos, table = _case(37, 11, dim, q_heads, kv_heads)
    pos[5], pos[20] = -3, table.shape[0]
    want, _ = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, table, q_heads, kv_heads, dim, 1e-6)
    rc, got, _ = _dev_call("warp34_dflash_qk_norm_rope_bf16_f32_table", qkv, pos, qw, kw, table, q_heads, kv_heads,
                           dim, 1e-6)
    assert rc == 0 and (got == want).all()
    tb = oracle.f32_to_bf16_bits(table)
    want_b, _ = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, tb, q_heads, kv_heads, dim, 1e-6)
    rc, got_b, _ = _dev_call("warp34_dflash_qk_norm_rope_bf16", qkv, pos, qw, kw, tb, q_heads, kv_heads, dim, 1e-6)
    assert rc == 0 and (got_b == want_b).all()
    # skipped rows and every V column are untouched
    assert (got[5] == qkv[5]).all() and (got[20] == qkv[20]).all()
    assert (got[:, (q_heads + kv_heads) * dim:] == qkv[:, (q_heads + kv_heads) * dim:]).all()


def test_operator_q_out_bit_exact():
    dim, q_heads, kv_heads = 256, 16, 4
    qkv, qw, kw, pos, table = _case(16, 12, dim, q_heads, kv_heads)
    q_out = np.full((16, q_heads * dim), 0x7E7E, np.uint16)
    want, want_q = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, table, q_heads, kv_heads, dim, 1e-6,
                                            q_out=q_out.copy())
    rc, got, got_q = _dev_call("warp34_dflash_qk_norm_rope_bf16_f32_table_qout", qkv, pos, qw, kw, table, q_heads,
                               kv_heads, dim, 1e-6, q_out=q_out)
    assert rc == 0 and (got == want).all() and (got_q == want_q).all()
    assert (got[:, :q_heads * dim] == qkv[:, :q_heads * dim]).all()  # packed Q untouched


@pytest.mark.parametrize("fmt,xf", [(FMT_BF16, XF_IDENTITY), (FMT_TQ4, XF_WHT256), (FMT_TQ4, XF_IDENTITY), (FMT_FP8, XF_IDENTITY),
                                    (FMT_Q8_0, XF_IDENTITY), (FMT_FP8, XF_WHT256), (FMT_Q8_0, XF_WHT256)])
def test_fused_kv_write_bit_exact_and_equal_to_operator_then_append(fmt, xf):
    import gpu_harness as G

    dim, q_heads, kv_heads, rows, bs = 256, 16, 4, 40, 16
    qkv, qw, kw, pos, table = _case(rows, 13, dim, q_heads, kv_heads)
    pos[3] = -1  # skipped row: nothing written anywhere
    bt = np.array([2, 1, 0], np.int32)  # reversed page table
    slots = oracle.slot_mapping(bt, 0, rows, bs)
    slots[7] = -1
    # oracle
    hpool = oracle.HostPool(3, kv_heads, dim, bs, fmt, xf)
    hpool.k[:], hpool.v[:] = 0x7E, 0x7E
    q_out = np.full((rows, q_heads * dim), 0x7E7E, np.uint16)
    want, want_q = oracle.qk_norm_rope_bf16(qkv.copy(), pos, qw, kw, table, q_heads, kv_heads, dim, 1e-6,
                                            q_out=q_out.copy(), pool=hpool, write_slot_mapping=slots)
    # fused on the device
    dpool = G.DevPool(hpool, fill=0x7E)
    rc, got, got_q = _dev_call("warp34_dflash_qk_norm_rope_kv_write_bf16_f32_table", qkv, pos, qw, kw, table,
                               q_heads, kv_heads, dim, 1e-6, q_out=q_out, dpool=dpool, slots=slots)
    assert rc == 0
    gk, gv = dpool.download()
    assert (got == want).all() and (got_q == want_q).all()
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()
    # un-fused on the device: operator in place, then the strided append of the K and V columns
    rc, plain, _ = _dev_call("warp34_dflash_qk_norm_rope_bf16_f32_table", qkv, pos, qw, kw, table, q_heads,
                             kv_heads, dim, 1e-6)
    assert rc == 0
    ref_pool = oracle.HostPool(3, kv_heads, dim, bs, fmt, xf)
    dref = G.DevPool(ref_pool, fill=0x7E)
    stride = (q_heads + 2 * kv_heads) * dim
    live = slots.copy()
    live[3] = -1  # the fused call skips the row whose position is outside the table
    hb = oracle.HostBatch([0, rows], [rows], bt.reshape(1, -1), context_lens_before=[0], write_slot_mapping=live)
    k_cols = plain[:, q_heads * dim:].copy()            # K columns first, row stride = the rest of the row
    v_cols = plain[:, (q_heads + kv_heads) * dim:].copy()
    pad_k = np.zeros((rows, stride), np.uint16)
    pad_v = np.zeros((rows, stride), np.uint16)
    pad_k[:, :k_cols.shape[1]] = k_cols
    pad_v[:, :v_cols.shape[1]] = v_cols
    assert G.dev_write(dref, hb, pad_k, pad_v, DT_BF16, stride, stride) == 0
    rk, rv = dref.download()
    assert rk.tobytes() == gk.tobytes() and rv.tobytes() == gv.tobytes()


def test_argument_validation():
    """Error convention of op_dflash2.cu:1263-1268,1326-1335."""
    import gpu_harness as G
    from warp34_amd import ffi

    dim, q_heads, kv_heads, rows = 256, 8, 2, 4
    qkv, qw, kw, pos, table = _case(rows, 14, dim, q_heads, kv_heads)
    inval = ffi.HIP_ERROR_INVALID_VALUE
    name = "warp34_dflash_qk_norm_rope_bf16_f32_table"
    assert _dev_call(name, qkv, pos, qw, kw, table, q_heads, 3, dim, 1e-6)[0] == inval      # q_heads % kv_heads
    assert _dev_call(name, qkv, pos, qw, kw, table, q_heads, kv_heads, 255, 1e-6)[0] == inval  # odd dim
    assert _dev_call(name, qkv, pos, qw, kw, table, q_heads, kv_heads, dim, 0.0)[0] == inval
    assert _dev_call(name, qkv, pos, qw, kw, table, q_heads, kv_heads, dim, float("inf"))[0] == inval
    rc, got, _ = _dev_call(name, qkv, pos, qw, kw, table, q_heads, kv_heads, dim, 1e-6, rows=0)
    assert rc == 0 and (got == qkv).all()
    # fused write: layout must describe the same heads / head size, FP16 pages are refused,
    # K and V must share format and transform
    hpool = oracle.HostPool(2, kv_heads, dim, 16, FMT_TQ4, XF_WHT256)
    dpool = G.DevPool(hpool)
    slots = np.arange(rows, dtype=np.int32)
    fused = "warp34_dflash_qk_norm_rope_kv_write_bf16_f32_table"
    for mutate in (lambda L: setattr(L, "local_kv_heads", kv_heads + 1), lambda L: setattr(L, "head_dim", 128),
                   lambda L: setattr(L, "k_format", ffi.WARP34_KV_FORMAT_FP16),
                   lambda L: setattr(L, "v_format", ffi.WARP34_KV_FORMAT_Q8_0),
                   lambda L: setattr(L, "v_transform", ffi.WARP34_KV_TRANSFORM_IDENTITY),
                   lambda L: setattr(L, "block_size", 0)):
        L = dpool.layout()
        mutate(L)
        rc, _, _ = _dev_call(fused, qkv, pos, qw, kw, table, q_heads, kv_heads, dim, 1e-6, dpool=dpool, slots=slots,
                             layout=L)
        assert rc == inval
    gk, gv = dpool.download()
    assert not gk.any() and not gv.any()
