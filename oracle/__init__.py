"""ctypes view of the CPU oracle (oracle/libtq4_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py as the checker / the timed CPU baseline.  The product
package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libtq4_oracle.so")

FMT_FP16, FMT_BF16, FMT_TQ4, FMT_Q8_0, FMT_FP8 = 0, 1, 2, 3, 4
XF_IDENTITY, XF_WHT256 = 0, 1
DT_F16, DT_BF16 = 0, 1


class Layout(C.Structure):
    _fields_ = [
        ("k_base", C.c_void_p), ("v_base", C.c_void_p),
        ("k_page_stride", C.c_uint64), ("k_head_stride", C.c_uint64), ("k_token_stride", C.c_uint64),
        ("v_page_stride", C.c_uint64), ("v_head_stride", C.c_uint64), ("v_token_stride", C.c_uint64),
        ("local_kv_heads", C.c_int32), ("head_dim", C.c_int32), ("block_size", C.c_int32),
        ("k_format", C.c_int32), ("v_format", C.c_int32),
        ("k_transform", C.c_int32), ("v_transform", C.c_int32),
    ]


class Batch(C.Structure):
    _fields_ = [
        ("query_start_loc", C.c_void_p), ("context_lens_before", C.c_void_p),
        ("seq_lens_after", C.c_void_p), ("block_tables", C.c_void_p),
        ("write_slot_mapping", C.c_void_p), ("valid_token_mask", C.c_void_p),
        ("valid_req_mask", C.c_void_p),
        ("num_reqs", C.c_int32), ("total_tokens", C.c_int32), ("max_blocks_per_req", C.c_int32),
        ("mask_mode", C.c_int32), ("sliding_window", C.c_int32), ("sm_scale", C.c_float),
    ]


def build(force=False):
    """Compile the oracle with the Makefile beside it."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        fp = C.POINTER(C.c_float)
        L.tq4o_centroids256.restype = fp
        L.tq4o_boundaries256.restype = fp
        L.tq4o_signs256.restype = fp
        L.tq4o_f16_to_f32.restype = C.c_float
        L.tq4o_f16_to_f32.argtypes = [C.c_uint16]
        L.tq4o_f32_to_f16.restype = C.c_uint16
        L.tq4o_f32_to_f16.argtypes = [C.c_float]
        L.tq4o_bf16_to_f32.restype = C.c_float
        L.tq4o_bf16_to_f32.argtypes = [C.c_uint16]
        L.tq4o_f32_to_bf16.restype = C.c_uint16
        L.tq4o_f32_to_bf16.argtypes = [C.c_float]
        L.tq4o_wht256.argtypes = [C.c_void_p]
        L.tq4o_encode_row.argtypes = [C.c_void_p, C.c_void_p]
        L.tq4o_encode_row_plain.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
        L.tq4o_encode_row_plain.restype = None
        L.tq4o_dequant_row.argtypes = [C.c_void_p, C.c_void_p]
        for name in ("tq4o_encode_row_fp8", "tq4o_encode_row_q8", "tq4o_dequant_row_fp8", "tq4o_dequant_row_q8"):
            getattr(L, name).argtypes = [C.c_void_p, C.c_void_p]
        L.tq4o_f32_to_e4m3.restype = C.c_uint8
        L.tq4o_f32_to_e4m3.argtypes = [C.c_float]
        L.tq4o_e4m3_to_f32.restype = C.c_float
        L.tq4o_e4m3_to_f32.argtypes = [C.c_uint8]
        L.tq4o_unrotate_row.argtypes = [C.c_void_p, C.c_void_p]
        L.tq4o_kv_cache_write.restype = C.c_int
        L.tq4o_kv_cache_write.argtypes = [C.POINTER(Layout), C.POINTER(Batch), C.c_void_p, C.c_void_p,
                                          C.c_int, C.c_int, C.c_int]
        L.tq4o_paged_attention.restype = C.c_int
        L.tq4o_paged_attention.argtypes = [C.POINTER(Layout), C.POINTER(Batch), C.c_void_p, C.c_int,
                                           C.c_void_p, C.c_int, C.c_int]
        L.tq4o_paged_attention_split.restype = C.c_int
        L.tq4o_paged_attention_split.argtypes = [C.POINTER(Layout), C.POINTER(Batch), C.c_void_p, C.c_int,
                                                 C.c_void_p, C.c_int, C.c_int]
        L.tq4o_qk_norm_rope_bf16.restype = C.c_int
        L.tq4o_qk_norm_rope_bf16.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                             C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float,
                                             C.POINTER(Layout), C.c_void_p]
        L.tq4o_fused_qk_rmsnorm_rope_gate_f16.restype = C.c_int
        L.tq4o_fused_qk_rmsnorm_rope_gate_f16.argtypes = [C.c_void_p] * 9 + [C.c_int] * 11 + [C.c_float, C.c_float]
        L.tq4o_fill_normal.argtypes = [C.c_void_p, C.c_size_t, C.c_uint64, C.c_int]
        L.tq4o_fill_kv_rows.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_uint64, C.c_int, C.c_int]
        L.tq4o_permutation.argtypes = [C.c_void_p, C.c_int, C.c_uint64]
        L.tq4o_hw_threads.restype = C.c_int
        _lib = L
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data


# ---- tables ----------------------------------------------------------------------------
def centroids():
    return np.ctypeslib.as_array(lib().tq4o_centroids256(), (16,)).copy()


def boundaries():
    return np.ctypeslib.as_array(lib().tq4o_boundaries256(), (15,)).copy()


def signs():
    return np.ctypeslib.as_array(lib().tq4o_signs256(), (256,)).copy()


# ---- row level -------------------------------------------------------------------------
def wht256(x):
    y = np.ascontiguousarray(x, dtype=np.float32).copy()
    assert y.shape == (256,)
    lib().tq4o_wht256(y.ctypes.data)
    return y


def encode_row(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.shape == (256,)
    out = np.zeros(132, dtype=np.uint8)
    lib().tq4o_encode_row(x.ctypes.data, out.ctypes.data)
    return out


def encode_row_plain(x):
    """head_dim fp32 values (a multiple of 128) -> a TQ4 row without the rotation."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.ndim == 1 and x.shape[0] % 128 == 0
    out = np.zeros(66 * (x.shape[0] // 128), dtype=np.uint8)
    lib().tq4o_encode_row_plain(x.ctypes.data, x.shape[0], out.ctypes.data)
    return out


def encode_row_fmt(x, fmt):
    """256 fp32 values (already transformed) -> one stored row of an 8-bit format."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.shape == (256,)
    out = np.zeros(row_bytes(fmt, 256), dtype=np.uint8)
    fn = lib().tq4o_encode_row_fp8 if fmt == FMT_FP8 else lib().tq4o_encode_row_q8
    fn(x.ctypes.data, out.ctypes.data)
    return out


def dequant_row_fmt(row, fmt):
    row = np.ascontiguousarray(row, dtype=np.uint8)
    out = np.zeros(256, dtype=np.float32)
    fn = lib().tq4o_dequant_row_fp8 if fmt == FMT_FP8 else lib().tq4o_dequant_row_q8
    fn(row.ctypes.data, out.ctypes.data)
    return out


def f32_to_e4m3(f):
    return int(lib().tq4o_f32_to_e4m3(float(f)))


def e4m3_to_f32(c):
    return float(lib().tq4o_e4m3_to_f32(int(c)))


def dequant_row(row):
    row = np.ascontiguousarray(row, dtype=np.uint8)
    assert row.shape == (132,)
    y = np.zeros(256, dtype=np.float32)
    lib().tq4o_dequant_row(row.ctypes.data, y.ctypes.data)
    return y


def unrotate_row(y):
    y = np.ascontiguousarray(y, dtype=np.float32)
    x = np.zeros(256, dtype=np.float32)
    lib().tq4o_unrotate_row(y.ctypes.data, x.ctypes.data)
    return x


# ---- 16-bit helpers (vectorised through numpy; the C scalars are tested against these) ---
def f32_to_bf16_bits(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)
    nan = np.isnan(a)
    if nan.any():
        r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f16_bits_to_f32(b):
    return np.ascontiguousarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)


def f32_to_f16_bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).astype(np.float16).view(np.uint16)


def bits_to_f32(b, dtype):
    return bf16_bits_to_f32(b) if dtype == DT_BF16 else f16_bits_to_f32(b)


# ---- generators ------------------------------------------------------------------------
def fill_normal(n, seed, dtype):
    out = np.zeros(n, dtype=np.uint16)
    lib().tq4o_fill_normal(out.ctypes.data, n, seed, dtype)
    return out


def fill_kv_rows(rows, kv_heads, head_dim, seed, dtype, n_outliers=3):
    out = np.zeros((rows, kv_heads, head_dim), dtype=np.uint16)
    lib().tq4o_fill_kv_rows(out.ctypes.data, rows, kv_heads, head_dim, seed, dtype, n_outliers)
    return out


def permutation(n, seed):
    out = np.zeros(n, dtype=np.int32)
    lib().tq4o_permutation(out.ctypes.data, n, seed)
    return out


def hw_threads():
    return lib().tq4o_hw_threads()


# ---- paged pool + batch on the host ------------------------------------------------------
def row_bytes(fmt, head_dim):
    """crates/warp34-host/src/cache.rs:157-165"""
    if fmt in (FMT_FP16, FMT_BF16):
        return head_dim * 2
    if fmt == FMT_TQ4:
        return 66 * (head_dim // 128)
    if fmt == FMT_Q8_0:
        return 68 * (head_dim // 64)
    if fmt == FMT_FP8:
        return head_dim + 4 * (head_dim // 128)
    raise ValueError(fmt)


class HostPool:
    """One layer's K and V slabs in host memory with KvPool strides
    (crates/warp34-host/src/cache.rs:304-335)."""

    def __init__(self, num_pages, kv_heads, head_dim, block_size, fmt, transform, v_transform=None):
        self.num_pages, self.kv_heads, self.head_dim, self.block_size = num_pages, kv_heads, head_dim, block_size
        self.fmt, self.transform = fmt, transform
        self.v_transform = transform if v_transform is None else v_transform  # the V slab's, if it differs
        self.tok = row_bytes(fmt, head_dim)
        self.head = block_size * self.tok
        self.page = kv_heads * self.head
        self.k = np.zeros(num_pages * self.page, dtype=np.uint8)
        self.v = np.zeros(num_pages * self.page, dtype=np.uint8)

    def layout(self):
        return Layout(self.k.ctypes.data, self.v.ctypes.data, self.page, self.head, self.tok,
                      self.page, self.head, self.tok, self.kv_heads, self.head_dim, self.block_size,
                      self.fmt, self.fmt, self.transform, self.v_transform)


class HostBatch:
    """Keeps the numpy index arrays alive and exposes the C struct."""

    def __init__(self, query_start_loc, seq_lens_after, block_tables, context_lens_before=None,
                 write_slot_mapping=None, valid_token_mask=None, valid_req_mask=None,
                 mask_mode=0, sliding_window=0, sm_scale=0.0625, total_tokens=None):
        i32 = lambda a: None if a is None else np.ascontiguousarray(a, dtype=np.int32)
        u8 = lambda a: None if a is None else np.ascontiguousarray(a, dtype=np.uint8)
        self.qsl = i32(query_start_loc)
        self.ctx = i32(context_lens_before)
        self.seq = i32(seq_lens_after)
        self.bt = i32(block_tables)
        assert self.bt.ndim == 2
        self.slots = i32(write_slot_mapping)
        self.tmask = u8(valid_token_mask)
        self.rmask = u8(valid_req_mask)
        self.num_reqs = len(self.seq)
        self.total_tokens = int(self.qsl[-1]) if total_tokens is None else int(total_tokens)
        self.mask_mode, self.sliding_window, self.sm_scale = mask_mode, sliding_window, sm_scale

    def struct(self):
        return Batch(_ptr(self.qsl), _ptr(self.ctx), _ptr(self.seq), _ptr(self.bt), _ptr(self.slots),
                     _ptr(self.tmask), _ptr(self.rmask), self.num_reqs, self.total_tokens,
                     self.bt.shape[1], self.mask_mode, self.sliding_window, self.sm_scale)


def kv_cache_write(pool, batch, k_in, v_in, in_dtype, k_row_stride=None, v_row_stride=None):
    k_in = np.ascontiguousarray(k_in, dtype=np.uint16)
    v_in = np.ascontiguousarray(v_in, dtype=np.uint16)
    dflt = pool.kv_heads * pool.head_dim
    L, B = pool.layout(), batch.struct()
    rc = lib().tq4o_kv_cache_write(C.byref(L), C.byref(B), k_in.ctypes.data, v_in.ctypes.data,
                                   k_row_stride or dflt, v_row_stride or dflt, in_dtype)
    if rc:
        raise RuntimeError("oracle kv_cache_write: unsupported layout")


def paged_attention(pool, batch, q_bits, q_dtype, num_q_heads, n_threads=1, out=None, n_splits=0):
    q_bits = np.ascontiguousarray(q_bits, dtype=np.uint16)
    if out is None:
        out = np.zeros((batch.total_tokens, num_q_heads, pool.head_dim), dtype=np.float32)
    L, B = pool.layout(), batch.struct()
    if n_splits:
        rc = lib().tq4o_paged_attention_split(C.byref(L), C.byref(B), q_bits.ctypes.data, q_dtype,
                                              out.ctypes.data, num_q_heads, n_splits)
    else:
        rc = lib().tq4o_paged_attention(C.byref(L), C.byref(B), q_bits.ctypes.data, q_dtype,
                                        out.ctypes.data, num_q_heads, n_threads)
    if rc:
        raise RuntimeError("oracle paged_attention: unsupported shape")
    return out


def qk_norm_rope_bf16(qkv, positions, qw, kw, table, q_heads, kv_heads, dim, eps, q_out=None, pool=None,
                      write_slot_mapping=None):
    """ops/op_dflash2.cu:338-418.  qkv: uint16 [rows, (q_heads + 2 kv_heads) * dim], modified in
    place; table: float32 or uint16 (bf16 bits) [table_rows, dim]; with pool + write_slot_mapping the
    rotated K and the V rows go to the pool instead.  Returns (qkv, q_out)."""
    assert qkv.dtype == np.uint16 and qkv.flags.c_contiguous
    rows = qkv.shape[0]
    positions = np.ascontiguousarray(positions, dtype=np.int32)
    qw = np.ascontiguousarray(qw, dtype=np.uint16)
    kw = np.ascontiguousarray(kw, dtype=np.uint16)
    table = np.ascontiguousarray(table)
    assert table.dtype in (np.float32, np.uint16)
    slots = None if write_slot_mapping is None else np.ascontiguousarray(write_slot_mapping, dtype=np.int32)
    L = pool.layout() if pool is not None else None
    rc = lib().tq4o_qk_norm_rope_bf16(qkv.ctypes.data, None if q_out is None else q_out.ctypes.data,
                                      positions.ctypes.data, qw.ctypes.data, kw.ctypes.data, table.ctypes.data,
                                      1 if table.dtype == np.float32 else 0, rows, q_heads, kv_heads, dim,
                                      table.shape[0], eps, None if L is None else C.byref(L),
                                      None if slots is None else slots.ctypes.data)
    if rc:
        raise RuntimeError("oracle qk_norm_rope_bf16: rc=%d" % rc)
    return qkv, q_out


def fused_qk_rmsnorm_rope_gate_f16(q_gate, k, q_norm_w, k_norm_w, positions, num_q_heads, num_kv_heads, head_dim,
                                   rotary_dim, mrope, rope_theta, rms_eps, valid_token_mask=None, q_out=None,
                                   k_out=None, gate_out=None):
    """ops/op_norms_rope_act.cu:524-689.  q_gate: uint16 (fp16 bits) [tokens, q_gate_row_stride], k: uint16
    [tokens, k_row_stride] (row strides taken from the arrays), positions: int32 [3, plane_stride],
    mrope: the three section sizes.  Returns (q_out, k_out, gate_out) as uint16 [tokens, heads, head_dim];
    buffers passed in keep their bytes where a token is masked."""
    n = q_gate.shape[0]
    assert q_gate.dtype == np.uint16 and k.dtype == np.uint16 and q_gate.flags.c_contiguous and k.flags.c_contiguous
    positions = np.ascontiguousarray(positions, dtype=np.int32)
    assert positions.ndim == 2 and positions.shape[0] == 3
    q_out = np.zeros((n, num_q_heads, head_dim), dtype=np.uint16) if q_out is None else q_out
    k_out = np.zeros((n, num_kv_heads, head_dim), dtype=np.uint16) if k_out is None else k_out
    gate_out = np.zeros((n, num_q_heads, head_dim), dtype=np.uint16) if gate_out is None else gate_out
    mask = None if valid_token_mask is None else np.ascontiguousarray(valid_token_mask, dtype=np.uint8)
    qw = np.ascontiguousarray(q_norm_w, dtype=np.uint16)
    kw = np.ascontiguousarray(k_norm_w, dtype=np.uint16)
    rc = lib().tq4o_fused_qk_rmsnorm_rope_gate_f16(
        q_gate.ctypes.data, k.ctypes.data, qw.ctypes.data, kw.ctypes.data, positions.ctypes.data,
        None if mask is None else mask.ctypes.data, q_out.ctypes.data, k_out.ctypes.data, gate_out.ctypes.data,
        n, positions.shape[1], num_q_heads, num_kv_heads, head_dim, rotary_dim, mrope[0], mrope[1], mrope[2],
        q_gate.shape[1], k.shape[1], rope_theta, rms_eps)
    if rc:
        raise RuntimeError("oracle fused_qk_rmsnorm_rope_gate_f16: rc=%d" % rc)
    return q_out, k_out, gate_out


def apply_attn_output_gate_f16(attn_out, gate, out=None, valid_token_mask=None):
    """ops/op_norms_rope_act.cu:742-759 on uint16 (fp16 bits) [num_tokens, total_dim] arrays."""
    attn_out = np.ascontiguousarray(attn_out, dtype=np.uint16)
    gate = np.ascontiguousarray(gate, dtype=np.uint16)
    if out is None:
        out = np.zeros_like(attn_out)
    mask = None if valid_token_mask is None else np.ascontiguousarray(valid_token_mask, dtype=np.uint8)
    fn = lib().tq4o_apply_attn_output_gate_f16
    fn.restype = C.c_int
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int]
    rc = fn(attn_out.ctypes.data, gate.ctypes.data, out.ctypes.data, None if mask is None else mask.ctypes.data,
            attn_out.shape[0], attn_out.shape[1])
    if rc:
        raise RuntimeError("oracle apply_attn_output_gate_f16: rc=%d" % rc)
    return out


def qsa_sparse_paged_attn_f16(pool, q_bits, sel_phys, sel_log, num_sel, seq_pos, num_q_heads, sm_scale=0.0625,
                              gate=None, valid_token_mask=None, hadamard64=False):
    """ops/op_qsa.cu:716-1158,1446-1571: fp16 bits in, fp16 bits out [tokens, q heads, 256]."""
    q_bits = np.ascontiguousarray(q_bits, dtype=np.uint16)
    sel_phys = np.ascontiguousarray(sel_phys, dtype=np.int32)
    sel_log = np.ascontiguousarray(sel_log, dtype=np.int32)
    num_sel = np.ascontiguousarray(num_sel, dtype=np.int32)
    seq_pos = np.ascontiguousarray(seq_pos, dtype=np.int32)
    n_tok, select_k = sel_phys.shape
    assert sel_log.shape == sel_phys.shape and num_sel.shape == (n_tok,) and seq_pos.shape == (n_tok,)
    g = None if gate is None else np.ascontiguousarray(gate, dtype=np.uint16)
    mask = None if valid_token_mask is None else np.ascontiguousarray(valid_token_mask, dtype=np.uint8)
    out = np.zeros((n_tok, num_q_heads, 256), dtype=np.uint16)
    fn = lib().tq4o_qsa_sparse_paged_attn_f16
    fn.restype = C.c_int
    fn.argtypes = [C.c_void_p] * 9 + [C.c_int, C.c_int, C.c_int, C.c_float, C.c_int]
    L = pool.layout()
    rc = fn(C.addressof(L), q_bits.ctypes.data, None if g is None else g.ctypes.data, sel_phys.ctypes.data,
            sel_log.ctypes.data, num_sel.ctypes.data, seq_pos.ctypes.data,
            None if mask is None else mask.ctypes.data, out.ctypes.data, n_tok, num_q_heads, select_k,
            sm_scale, 1 if hadamard64 else 0)
    if rc:
        raise RuntimeError("oracle qsa_sparse_paged_attn_f16: rc=%d" % rc)
    return out


def slot_mapping(block_table, ctx_before, n_tokens, block_size):
    """crates/warp34-host/src/model/execution.rs:382-388"""
    pos = np.arange(ctx_before, ctx_before + n_tokens)
    bt = np.asarray(block_table, dtype=np.int64)
    return (bt[pos // block_size] * block_size + pos % block_size).astype(np.int32)
