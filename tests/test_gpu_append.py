"""GPU parity: quantize-on-append through the C ABI vs the CPU oracle -- bit-exact.

Cases follow the reference's write tests (tests/backbone_and_collectives.rs:455-572 page
placement and 132-byte strides, tests/paged_fa2.rs:618-691 mask contract) and benchmark
config 1 (4096 tokens, 2 kv heads, 64-token pages in a seeded random physical order,
1 % outlier channels).
"""
import ctypes as C

import numpy as np
import pytest

import oracle
from oracle import DT_BF16, DT_F16, FMT_BF16, FMT_FP8, FMT_FP16, FMT_Q8_0, FMT_TQ4, XF_IDENTITY, XF_WHT256

pytestmark = pytest.mark.gpu


def _run_append(fmt, xf, block_size, n_tokens, in_dtype, seed, kv_heads=2, tmask=None, rmask=None,
                neg_slots=(), stride=None, head_dim=256):
    import gpu_harness as G

    n_pages = (n_tokens + block_size - 1) // block_size
    perm = oracle.permutation(n_pages + 2, seed + 100)
    bt = perm[:n_pages].reshape(1, -1)
    slots = oracle.slot_mapping(bt[0], 0, n_tokens, block_size)
    for i in neg_slots:
        slots[i] = -1
    k = oracle.fill_kv_rows(n_tokens, kv_heads, head_dim, seed, in_dtype, 3)
    v = oracle.fill_kv_rows(n_tokens, kv_heads, head_dim, seed + 1, in_dtype, 3)
    if stride is not None:
        pad = stride - kv_heads * head_dim
        filler = oracle.fill_normal(n_tokens * pad, seed + 2, in_dtype).reshape(n_tokens, pad)
        k_src = np.concatenate([k.reshape(n_tokens, -1), filler], axis=1)
        v_src = np.concatenate([v.reshape(n_tokens, -1), filler[:, ::-1]], axis=1)
    else:
        k_src, v_src = k, v
    hpool = oracle.HostPool(n_pages + 2, kv_heads, head_dim, block_size, fmt, xf)
    hb = oracle.HostBatch([0, n_tokens], [n_tokens], bt, context_lens_before=[0], write_slot_mapping=slots,
                          valid_token_mask=tmask, valid_req_mask=rmask)
    oracle.kv_cache_write(hpool, hb, k_src, v_src, in_dtype, stride, stride)
    dpool = G.DevPool(hpool)
    rc = G.dev_write(dpool, hb, k_src, v_src, in_dtype, stride, stride)
    assert rc == 0
    gk, gv = dpool.download()
    return hpool, gk, gv


@pytest.mark.parametrize("in_dtype", [DT_BF16, DT_F16])
def test_config1_tq4_append_bit_exact(in_dtype):
    """Benchmark configuration 1: 4096 tokens x 2 kv heads, 64-token pages, permuted physical order."""
    hpool, gk, gv = _run_append(FMT_TQ4, XF_WHT256, 64, 4096, in_dtype, seed=0)
    assert hpool.tok == 132 and hpool.head == 64 * 132 and hpool.page == 2 * 64 * 132
    assert gk.tobytes() == hpool.k.tobytes()
    assert gv.tobytes() == hpool.v.tobytes()
    # dequant round trip of what the GPU wrote (reference quality gate ~ codebook distortion)
    row = gk[:132]
    y = oracle.dequant_row(row)
    assert np.isfinite(y).all()


@pytest.mark.parametrize("block_size,n_tokens", [(16, 40), (16, 1), (64, 65), (128, 300)])
def test_tq4_append_ragged_pages(block_size, n_tokens):
    hpool, gk, gv = _run_append(FMT_TQ4, XF_WHT256, block_size, n_tokens, DT_BF16, seed=3)
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()


def test_tq4_append_special_rows():
    """all-zero rows, tiny rows (below the 1e-20 energy threshold), huge rows."""
    import gpu_harness as G

    n = 8
    k = np.zeros((n, 2, 256), dtype=np.float32)
    rng = np.random.default_rng(0)
    k[1] = rng.standard_normal((2, 256)) * 1e-12
    k[2] = rng.standard_normal((2, 256)) * 1e4
    k[3, :, 7] = 1.0
    k[4] = 1.0
    k[5] = rng.standard_normal((2, 256)) * 1e-30
    k[6] = -rng.random((2, 256))
    k[7] = rng.standard_normal((2, 256))
    kb = oracle.f32_to_bf16_bits(k)
    vb = kb[::-1].copy()
    hpool = oracle.HostPool(2, 2, 256, 16, FMT_TQ4, XF_WHT256)
    hb = oracle.HostBatch([0, n], [n], np.array([[1, 0]], np.int32), context_lens_before=[0],
                          write_slot_mapping=oracle.slot_mapping([1, 0], 0, n, 16))
    oracle.kv_cache_write(hpool, hb, kb, vb, DT_BF16)
    dpool = G.DevPool(hpool)
    assert G.dev_write(dpool, hb, kb, vb, DT_BF16) == 0
    gk, gv = dpool.download()
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()


def test_append_masks_and_negative_slots_write_nothing():
    n = 24
    tmask = np.ones(n, np.uint8)
    tmask[[2, 17]] = 0
    hpool, gk, gv = _run_append(FMT_TQ4, XF_WHT256, 16, n, DT_F16, seed=5, tmask=tmask, neg_slots=(0, 9))
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()
    # masked request: nothing at all is written
    hpool2, gk2, gv2 = _run_append(FMT_TQ4, XF_WHT256, 16, n, DT_F16, seed=5, rmask=np.zeros(1, np.uint8))
    assert not gk2.any() and not gv2.any() and not hpool2.k.any()


@pytest.mark.parametrize("fmt,in_dtype", [(FMT_FP16, DT_F16), (FMT_BF16, DT_BF16), (FMT_BF16, DT_F16)])
def test_16bit_formats_and_strided_source(fmt, in_dtype):
    hpool, gk, gv = _run_append(fmt, XF_IDENTITY, 16, 50, in_dtype, seed=7, stride=2 * 256 + 64)
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()


@pytest.mark.parametrize("fmt,in_dtype", [(FMT_FP16, DT_F16), (FMT_BF16, DT_BF16), (FMT_BF16, DT_F16)])
def test_16bit_formats_at_head_dim_128(fmt, in_dtype):
    """The 16-bit row formats exist at every head dimension up to 256 (ops/op_kv_cache.cu:860-865)."""
    hpool, gk, gv = _run_append(fmt, XF_IDENTITY, 16, 50, in_dtype, seed=8, head_dim=128)
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()
    hpool, gk, gv = _run_append(fmt, XF_IDENTITY, 64, 130, in_dtype, seed=9, stride=2 * 128 + 24, head_dim=128)
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()


@pytest.mark.parametrize("in_dtype", [DT_BF16, DT_F16])
@pytest.mark.parametrize("head_dim", [128, 256])
def test_tq4_plain_append_bit_exact(in_dtype, head_dim):
    """TQ4 without the rotation: one 66-byte block per 128 elements (ops/op_kv_cache.cu:219-264)."""
    hpool, gk, gv = _run_append(FMT_TQ4, XF_IDENTITY, 64, 1500, in_dtype, seed=31, head_dim=head_dim)
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()
    hpool, gk, gv = _run_append(FMT_TQ4, XF_IDENTITY, 16, 77, in_dtype, seed=32, head_dim=head_dim,
                                stride=2 * head_dim + 3)
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()


def test_tq4_plain_append_at_head_dim_128_ignores_the_transform():
    """Rotated rows exist at head dimension 256 only: at 128 the WHT-256 transform value selects the
    same plain block quantiser (ops/op_kv_cache.cu:152)."""
    a, gk_a, gv_a = _run_append(FMT_TQ4, XF_WHT256, 16, 50, DT_F16, seed=33, head_dim=128)
    b, gk_b, gv_b = _run_append(FMT_TQ4, XF_IDENTITY, 16, 50, DT_F16, seed=33, head_dim=128)
    assert gk_a.tobytes() == a.k.tobytes() and gk_a.tobytes() == gk_b.tobytes() and gv_a.tobytes() == gv_b.tobytes()


def test_tq4_plain_append_special_rows():
    """Zero blocks (codes 7, scale 0), tiny, huge and negative-zero rows."""
    import gpu_harness as G

    rng = np.random.default_rng(2)
    n = 8
    k = np.zeros((n, 2, 256), dtype=np.float32)
    k[1] = rng.standard_normal((2, 256)) * 1e-12
    k[2] = rng.standard_normal((2, 256)) * 1e4
    k[3, :, :128] = rng.standard_normal((2, 128))
    k[4] = -0.0
    k[5] = rng.standard_normal((2, 256)) * 1e-30
    k[6] = -rng.random((2, 256))
    k[7] = rng.standard_normal((2, 256))
    kb = oracle.f32_to_f16_bits(k)
    hpool = oracle.HostPool(2, 2, 256, 16, FMT_TQ4, XF_IDENTITY)
    bt = np.array([[1, 0]], dtype=np.int32)
    slots = oracle.slot_mapping(bt[0], 0, n, 16)
    hb = oracle.HostBatch([0, n], [n], bt, context_lens_before=[0], write_slot_mapping=slots)
    oracle.kv_cache_write(hpool, hb, kb, kb[::-1].copy(), DT_F16)
    dpool = G.DevPool(hpool)
    assert G.dev_write(dpool, hb, kb, kb[::-1].copy(), DT_F16) == 0
    gk, gv = dpool.download()
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()


def test_tq4_strided_source_bf16():
    hpool, gk, gv = _run_append(FMT_TQ4, XF_WHT256, 64, 130, DT_BF16, seed=9, stride=3 * 512)
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()


@pytest.mark.parametrize("in_dtype", [DT_BF16, DT_F16])
@pytest.mark.parametrize("pad", [2, 4, 6])
def test_tq4_source_rows_not_16_byte_aligned(in_dtype, pad):
    """A source row stride of 2 * 256 + pad elements: every second row (or more) starts off the
    16-byte boundary the vector load wants, so those rows take the element-wise loads."""
    hpool, gk, gv = _run_append(FMT_TQ4, XF_WHT256, 32, 77, in_dtype, seed=21 + pad, stride=2 * 256 + pad)
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()


@pytest.mark.parametrize("fmt", [FMT_FP8, FMT_Q8_0])
@pytest.mark.parametrize("xf", [XF_IDENTITY, XF_WHT256])
@pytest.mark.parametrize("in_dtype", [DT_BF16, DT_F16])
def test_8bit_formats_append_bit_exact(fmt, xf, in_dtype):
    """FP8-E4M3 (264-byte) and Q8_0 (272-byte) rows, un-rotated as the default policy's tail layers
    store them and rotated (op_kv_cache.cu:32-140); 1 % outlier channels, ragged last page."""
    hpool, gk, gv = _run_append(fmt, xf, 64, 1000, in_dtype, seed=11)
    assert hpool.tok == (264 if fmt == FMT_FP8 else 272)
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()
    assert gk.any()


@pytest.mark.parametrize("fmt", [FMT_FP8, FMT_Q8_0])
def test_8bit_formats_special_rows_masks_and_strided_source(fmt):
    """Zero rows (d = 0 -> codes 0), rows below the scale thresholds, saturating rows, a source
    whose row stride breaks the 16-byte alignment of the vector load, masks and negative slots."""
    import gpu_harness as G

    n = 8
    k = np.zeros((n, 2, 256), dtype=np.float32)
    rng = np.random.default_rng(1)
    k[1] = rng.standard_normal((2, 256)) * 1e-12
    k[2] = rng.standard_normal((2, 256)) * 3e4
    k[3, :, 7] = 1.0
    k[4] = 1.0
    k[5] = rng.standard_normal((2, 256)) * 1e-30
    k[6] = -rng.random((2, 256))
    k[7, :, :128] = rng.standard_normal((2, 128)) * 100.0
    for dt, to_bits in ((DT_BF16, oracle.f32_to_bf16_bits), (DT_F16, lambda a: np.clip(a, -6e4, 6e4).astype(np.float16).view(np.uint16))):
        kb = to_bits(k)
        vb = kb[::-1].copy()
        hpool = oracle.HostPool(2, 2, 256, 16, fmt, XF_IDENTITY)
        hb = oracle.HostBatch([0, n], [n], np.array([[1, 0]], np.int32), context_lens_before=[0],
                              write_slot_mapping=oracle.slot_mapping([1, 0], 0, n, 16))
        oracle.kv_cache_write(hpool, hb, kb, vb, dt)
        dpool = G.DevPool(hpool)
        assert G.dev_write(dpool, hb, kb, vb, dt) == 0
        gk, gv = dpool.download()
        assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()
    hpool, gk, gv = _run_append(fmt, XF_IDENTITY, 16, 50, DT_F16, seed=13, stride=2 * 256 + 4)
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()
    tmask = np.ones(24, np.uint8)
    tmask[[2, 17]] = 0
    hpool, gk, gv = _run_append(fmt, XF_IDENTITY, 16, 24, DT_BF16, seed=15, tmask=tmask, neg_slots=(0, 9))
    assert gk.tobytes() == hpool.k.tobytes() and gv.tobytes() == hpool.v.tobytes()


def test_write_argument_validation():
    """Error convention of op_kv_cache.cu:836-845,1174-1177."""
    import gpu_harness as G
    from warp34_amd import ffi

    l = G.lib()
    hpool = oracle.HostPool(2, 2, 256, 16, FMT_TQ4, XF_WHT256)
    dpool = G.DevPool(hpool)
    hb = oracle.HostBatch([0, 4], [4], np.array([[0, 1]], np.int32), context_lens_before=[0],
                          write_slot_mapping=[0, 1, 2, 3])
    db = G.DevBatch(hb)
    L, B = dpool.layout(), db.struct()
    ex, _ = G.make_exec()
    k = G.to_dev(np.zeros((4, 512), np.uint16))
    inval, nosup = ffi.HIP_ERROR_INVALID_VALUE, ffi.HIP_ERROR_NOT_SUPPORTED
    assert l.warp34_kv_cache_write(None, C.byref(L), C.byref(B), G.ptr(k), G.ptr(k)) == inval
    assert l.warp34_kv_cache_write(C.byref(ex), None, C.byref(B), G.ptr(k), G.ptr(k)) == inval
    assert l.warp34_kv_cache_write(C.byref(ex), C.byref(L), C.byref(B), None, G.ptr(k)) == inval
    assert l.warp34_kv_cache_write_strided(C.byref(ex), C.byref(L), C.byref(B), G.ptr(k), G.ptr(k), 511, 512) == inval
    B0 = db.struct(total_tokens=0)
    assert l.warp34_kv_cache_write(C.byref(ex), C.byref(L), C.byref(B0), G.ptr(k), G.ptr(k)) == 0
    # FP8 needs head_dim 256 (op_kv_cache.cu:839-842); 8-bit rows carry fp32 scales: 4-byte aligned
    Lf8 = dpool.layout(fmt=ffi.WARP34_KV_FORMAT_FP8_E4M3)
    Lf8.head_dim = 128
    assert l.warp34_kv_cache_write(C.byref(ex), C.byref(Lf8), C.byref(B), G.ptr(k), G.ptr(k)) == inval
    Lf8 = dpool.layout(fmt=ffi.WARP34_KV_FORMAT_FP8_E4M3)
    Lf8.k_token_stride_bytes = 266
    assert l.warp34_kv_cache_write(C.byref(ex), C.byref(Lf8), C.byref(B), G.ptr(k), G.ptr(k)) == inval
    # TQ4 rows exist at head dimensions 128 and 256 only (rotated at 256 + WHT256, else plain)
    Lt = dpool.layout()
    Lt.head_dim = 64
    assert l.warp34_kv_cache_write_strided(C.byref(ex), C.byref(Lt), C.byref(B), G.ptr(k), G.ptr(k), 512, 512) == nosup
    # bf16 entry points: FP16 storage is rejected like in the reference
    Lh = dpool.layout(fmt=ffi.WARP34_KV_FORMAT_FP16)
    assert l.warp34_kv_cache_write_bf16(C.byref(ex), C.byref(Lh), C.byref(B), G.ptr(k), G.ptr(k)) == inval
    assert l.warp34_kv_cache_write_strided_bf16(C.byref(ex), C.byref(L), C.byref(B), G.ptr(k), G.ptr(k), 100) == inval
    gk, gv = dpool.download()
    assert not gk.any() and not gv.any()
