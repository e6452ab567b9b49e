"""GPU parity of the target model's Q/K producer (Gemma RMSNorm + interleaved mRoPE + gate split,
ops/op_norms_rope_act.cu:524-689,1201-1272) against the oracle, bit for bit, and of the variant
fused with the append against operator + warp34_kv_cache_write_strided, byte for byte."""
import ctypes as C

import numpy as np
import pytest

import oracle
from oracle import DT_F16, FMT_FP8, FMT_FP16, FMT_Q8_0, FMT_TQ4, XF_IDENTITY, XF_WHT256

pytestmark = pytest.mark.gpu

MROPE, THETA, EPS = (11, 11, 10), 1.0e7, 1.0e-6


def _inputs(n, qh, kh, hd, seed, q_stride=None, k_stride=None):
    q_stride = qh * 2 * hd if q_stride is None else q_stride
    k_stride = kh * hd if k_stride is None else k_stride
    qg = oracle.fill_normal(n * q_stride, seed, DT_F16).reshape(n, q_stride)
    k = oracle.fill_normal(n * k_stride, seed + 1, DT_F16).reshape(n, k_stride)
    qw = oracle.f32_to_f16_bits(0.1 * oracle.f16_bits_to_f32(oracle.fill_normal(hd, seed + 2, DT_F16)))
    kw = oracle.f32_to_f16_bits(0.1 * oracle.f16_bits_to_f32(oracle.fill_normal(hd, seed + 3, DT_F16)))
    return qg, k, qw, kw


def _positions(n, seed, plane_stride=None):
    rng = np.random.default_rng(seed)
    plane_stride = n if plane_stride is None else plane_stride
    pos = rng.integers(0, 262144, size=(3, plane_stride)).astype(np.int32)
    pos[:, 0] = 0
    if n > 1:
        pos[:, 1] = 262143
    return pos


def _dev_operator(qg, k, qw, kw, pos, qh, kh, hd, rot, mask=None, strided=True, fill=0x7E7E, mrope=MROPE,
                  theta=THETA, eps=EPS, num_tokens=None):
    import torch
    import gpu_harness as G

    n = qg.shape[0]
    d = dict(qg=G.to_dev(qg), k=G.to_dev(k), qw=G.to_dev(qw), kw=G.to_dev(kw), pos=G.to_dev(pos),
             mask=G.to_dev(mask),
             q=G.to_dev(np.full((n, qh, hd), fill, np.uint16)), ko=G.to_dev(np.full((n, kh, hd), fill, np.uint16)),
             g=G.to_dev(np.full((n, qh, hd), fill, np.uint16)))
    ex, _ = G.make_exec()
    head = [C.byref(ex), G.ptr(d["qg"]), G.ptr(d["k"]), G.ptr(d["qw"]), G.ptr(d["kw"]), G.ptr(d["pos"]),
            G.ptr(d["mask"]), G.ptr(d["q"]), G.ptr(d["ko"]), G.ptr(d["g"]), n if num_tokens is None else num_tokens,
            pos.shape[1], qh, kh, hd, rot, mrope[0], mrope[1], mrope[2]]
    if strided:
        rc = G.lib().warp34_fused_qk_rmsnorm_rope_gate_strided_f16(*head, qg.shape[1], k.shape[1], theta, eps)
    else:
        rc = G.lib().warp34_fused_qk_rmsnorm_rope_gate_f16(*head, theta, eps)
    torch.cuda.synchronize()
    out = [d[x].cpu().numpy().view(np.uint16) for x in ("q", "ko", "g")]
    return rc, out


# (tokens, q heads, kv heads, head_dim, rotary_dim, q stride or None, k stride or None, masked, seed)
OPERATOR_CASES = [
    (37, 16, 2, 256, 64, None, None, False, 11),       # the target model's layer shape, dense rows
    (64, 8, 1, 256, 64, 8 * 512 + 2 * 256 + 64, 2 * 256 + 8, True, 12),  # rows inside a wider projection, masked
    (5, 3, 1, 256, 64, None, None, False, 13),          # odd Q head count: a half wave without a head
    (9, 4, 4, 128, 128, None, None, True, 14),          # full rotation, smaller head
    (3, 2, 2, 256, 256, None, None, False, 15),         # the widest rotation
    (4, 5, 3, 64, 32, 5 * 128 + 16, 3 * 64 + 8, False, 16),
    (2, 2, 1, 256, 0, None, None, False, 17),           # no rotation at all
]


@pytest.mark.parametrize("case", OPERATOR_CASES, ids=lambda c: "n%d-q%d-kv%d-d%d-rot%d-seed%d" % (c[0], c[1], c[2], c[3], c[4], c[8]))
def test_operator_bits(case):
    n, qh, kh, hd, rot, qs, ks, masked, seed = case
    qg, k, qw, kw = _inputs(n, qh, kh, hd, seed, qs, ks)
    pos = _positions(n, seed, plane_stride=n + 3)
    mask = None
    if masked:
        mask = (np.arange(n) % 3 != 1).astype(np.uint8)
    fill = 0x7E7E
    want = oracle.fused_qk_rmsnorm_rope_gate_f16(
        qg, k, qw, kw, pos, qh, kh, hd, rot, MROPE, THETA, EPS, valid_token_mask=mask,
        q_out=np.full((n, qh, hd), fill, np.uint16), k_out=np.full((n, kh, hd), fill, np.uint16),
        gate_out=np.full((n, qh, hd), fill, np.uint16))
    rc, got = _dev_operator(qg, k, qw, kw, pos, qh, kh, hd, rot, mask=mask, fill=fill)
    assert rc == 0
    for name, g, w in zip(("q_out", "k_out", "gate_out"), got, want):
        assert g.reshape(w.shape).tobytes() == w.tobytes(), name


def test_dense_wrapper_equals_strided():
    n, qh, kh, hd, rot = 12, 16, 2, 256, 64
    qg, k, qw, kw = _inputs(n, qh, kh, hd, 21)
    pos = _positions(n, 21)
    rc_a, a = _dev_operator(qg, k, qw, kw, pos, qh, kh, hd, rot, strided=False)
    rc_b, b = _dev_operator(qg, k, qw, kw, pos, qh, kh, hd, rot, strided=True)
    assert rc_a == 0 and rc_b == 0
    for x, y in zip(a, b):
        assert x.tobytes() == y.tobytes()
    # other section sizes and another base: the plane pattern and the frequencies follow the arguments
    for mrope, theta in (((24, 20, 20), 1.0e6), ((32, 0, 0), 10000.0)):
        want = oracle.fused_qk_rmsnorm_rope_gate_f16(qg, k, qw, kw, pos, qh, kh, hd, rot, mrope, theta, 1e-5)
        rc, got = _dev_operator(qg, k, qw, kw, pos, qh, kh, hd, rot, mrope=mrope, theta=theta, eps=1e-5)
        assert rc == 0
        for g, w in zip(got, want):
            assert g.reshape(w.shape).tobytes() == w.tobytes()


def _dev_fused_write(dpool, qg, k, v, qw, kw, pos, slots, qh, kh, hd, rot, mask=None, with_k_out=True, layout=None):
    import torch
    import gpu_harness as G

    n = qg.shape[0]
    fill = 0x7E7E
    d = dict(qg=G.to_dev(qg), k=G.to_dev(k), v=G.to_dev(v), qw=G.to_dev(qw), kw=G.to_dev(kw), pos=G.to_dev(pos),
             mask=G.to_dev(mask), slots=G.to_dev(slots),
             q=G.to_dev(np.full((n, qh, hd), fill, np.uint16)), ko=G.to_dev(np.full((n, kh, hd), fill, np.uint16)),
             g=G.to_dev(np.full((n, qh, hd), fill, np.uint16)))
    ex, _ = G.make_exec()
    L = dpool.layout() if layout is None else layout
    rc = G.lib().warp34_fused_qk_rmsnorm_rope_gate_kv_write_f16(
        C.byref(ex), G.ptr(d["qg"]), G.ptr(d["k"]), G.ptr(d["v"]), G.ptr(d["qw"]), G.ptr(d["kw"]), G.ptr(d["pos"]),
        G.ptr(d["mask"]), G.ptr(d["q"]), G.ptr(d["ko"]) if with_k_out else None, G.ptr(d["g"]), C.byref(L),
        G.ptr(d["slots"]), n, pos.shape[1], qh, kh, hd, rot, MROPE[0], MROPE[1], MROPE[2], qg.shape[1], k.shape[1],
        v.shape[1], THETA, EPS)
    torch.cuda.synchronize()
    return rc, [d[x].cpu().numpy().view(np.uint16) for x in ("q", "ko", "g")]


@pytest.mark.parametrize("fmt,xf", [(FMT_TQ4, XF_WHT256), (FMT_TQ4, XF_IDENTITY), (FMT_FP8, XF_WHT256), (FMT_Q8_0, XF_WHT256),
                                    (FMT_FP8, XF_IDENTITY), (FMT_Q8_0, XF_IDENTITY), (FMT_FP16, XF_IDENTITY)])
@pytest.mark.parametrize("with_k_out", [True, False])
def test_fused_append_equals_operator_then_append(fmt, xf, with_k_out):
    import gpu_harness as G

    n, qh, kh, hd, rot, bs = 45, 16, 2, 256, 64, 16
    # the rows of one fused projection: [q_gate | k | v] per token
    width = qh * 2 * hd + 2 * kh * hd
    row = oracle.fill_normal(n * width, 31 + fmt, DT_F16).reshape(n, width)
    qg, k, v = row, row[:, qh * 2 * hd:], row[:, qh * 2 * hd + kh * hd:]
    k = np.ascontiguousarray(np.pad(k, ((0, 0), (0, width - k.shape[1]))))
    v = np.ascontiguousarray(np.pad(v, ((0, 0), (0, width - v.shape[1]))))
    _, _, qw, kw = _inputs(1, qh, kh, hd, 32)
    pos = _positions(n, 33)
    bt = np.array([2, 0, 1], np.int32)
    slots = oracle.slot_mapping(bt, 0, n, bs)
    slots[7] = -1
    mask = np.ones(n, np.uint8)
    mask[11] = 0

    # oracle: operator, then the append of its K rows and of the V columns
    fill = 0x7E7E
    want_q, want_k, want_g = oracle.fused_qk_rmsnorm_rope_gate_f16(
        qg, k, qw, kw, pos, qh, kh, hd, rot, MROPE, THETA, EPS, valid_token_mask=mask,
        q_out=np.full((n, qh, hd), fill, np.uint16), k_out=np.full((n, kh, hd), fill, np.uint16),
        gate_out=np.full((n, qh, hd), fill, np.uint16))
    hpool = oracle.HostPool(3, kh, hd, bs, fmt, xf)
    hpool.k[:], hpool.v[:] = 0x7E, 0x7E
    hb = oracle.HostBatch([0, n], [n], bt.reshape(1, -1), context_lens_before=[0], write_slot_mapping=slots,
                          valid_token_mask=mask)
    oracle.kv_cache_write(hpool, hb, want_k.reshape(n, kh * hd), v, DT_F16, kh * hd, width)

    dpool = G.DevPool(hpool, fill=0x7E)
    rc, (got_q, got_k, got_g) = _dev_fused_write(dpool, qg, k, v, qw, kw, pos, slots, qh, kh, hd, rot, mask=mask,
                                                 with_k_out=with_k_out)
    assert rc == 0
    gk, gv = dpool.download()
    assert got_q.tobytes() == want_q.tobytes() and got_g.tobytes() == want_g.tobytes()
    if with_k_out:
        assert got_k.tobytes() == want_k.tobytes()
    else:
        assert (got_k == fill).all()
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()

    # the un-fused sequence on the device lands on the same bytes
    rc, (_, dk, _) = _dev_operator(qg, k, qw, kw, pos, qh, kh, hd, rot, mask=mask, fill=fill)
    assert rc == 0
    ref_pool = oracle.HostPool(3, kh, hd, bs, fmt, xf)
    dref = G.DevPool(ref_pool, fill=0x7E)
    assert G.dev_write(dref, hb, dk.reshape(n, kh * hd), v, DT_F16, kh * hd, width) == 0
    rk, rv = dref.download()
    assert rk.tobytes() == gk.tobytes() and rv.tobytes() == gv.tobytes()


def test_argument_validation():
    """Error convention of ops/op_norms_rope_act.cu:1201-1246 (null pointers, strides shorter than a row:
    invalid value; zero tokens: success, nothing touched) and this build's documented restrictions."""
    import gpu_harness as G
    from warp34_amd import ffi

    n, qh, kh, hd, rot = 4, 4, 2, 256, 64
    qg, k, qw, kw = _inputs(n, qh, kh, hd, 41)
    pos = _positions(n, 41)
    inval, unsup = ffi.HIP_ERROR_INVALID_VALUE, ffi.HIP_ERROR_NOT_SUPPORTED
    rc, out = _dev_operator(qg, k, qw, kw, pos, qh, kh, hd, rot, num_tokens=0)
    assert rc == 0 and all((o == 0x7E7E).all() for o in out)
    # strides shorter than the heads they hold
    short_q = np.ascontiguousarray(qg[:, :qh * 2 * hd - 8])
    assert _dev_operator(short_q, k, qw, kw, pos, qh, kh, hd, rot)[0] == inval
    short_k = np.ascontiguousarray(k[:, :kh * hd - 8])
    assert _dev_operator(qg, short_k, qw, kw, pos, qh, kh, hd, rot)[0] == inval
    # outside this build's lane mapping: loud, nothing written
    rc, out = _dev_operator(qg, k, qw, kw, pos, qh, kh, 252, rot)
    assert rc in (inval, unsup) and all((o == 0x7E7E).all() for o in out)
    rc, out = _dev_operator(qg, k, qw, kw, pos, qh, kh, hd, 63)
    assert rc == unsup and all((o == 0x7E7E).all() for o in out)
    # fused append: layout must describe the same heads, K and V pages of one kind
    hpool = oracle.HostPool(2, kh, hd, 16, FMT_TQ4, XF_WHT256)
    dpool = G.DevPool(hpool)
    slots = np.arange(n, dtype=np.int32)
    v = k.copy()
    for mutate, code in ((lambda L: setattr(L, "local_kv_heads", kh + 1), inval),
                         (lambda L: setattr(L, "head_dim", 128), inval),
                         (lambda L: setattr(L, "block_size", 0), inval),
                         (lambda L: setattr(L, "v_format", ffi.WARP34_KV_FORMAT_Q8_0), unsup),
                         (lambda L: setattr(L, "v_transform", ffi.WARP34_KV_TRANSFORM_IDENTITY), unsup)):
        L = dpool.layout()
        mutate(L)
        rc, _ = _dev_fused_write(dpool, qg, k, v, qw, kw, pos, slots, qh, kh, hd, rot, layout=L)
        assert rc == code
    gk, gv = dpool.download()
    assert not gk.any() and not gv.any()
