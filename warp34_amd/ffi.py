"""ctypes binding of libwarp34_kernels.so -- the Python view of include/warp34_kv.h.

Mirrors the reference's Rust FFI module (crates/warp34-kernels/src/ffi.rs:6-90,701-760):
same struct layouts, constants and function signatures.  There is no fallback: when the
shared library has not been built, importing a symbol raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libwarp34_kernels.so")

WARP34_KV_NAMESPACE_TARGET_FULL_ATTN = 0
WARP34_KV_NAMESPACE_MTP_FULL_ATTN = 1
WARP34_KV_NAMESPACE_DFLASH_DRAFT_CTX = 2

WARP34_KV_FORMAT_FP16 = 0
WARP34_KV_FORMAT_BF16 = 1
WARP34_KV_FORMAT_TQ4 = 2
WARP34_KV_FORMAT_Q8_0 = 3
WARP34_KV_FORMAT_FP8_E4M3 = 4

WARP34_KV_TRANSFORM_IDENTITY = 0
WARP34_KV_TRANSFORM_RADEMACHER_WHT256 = 1

WARP34_ATTN_MASK_CAUSAL = 0
WARP34_ATTN_MASK_SYMMETRIC_WINDOW = 1
WARP34_ATTN_MASK_NONCAUSAL_WINDOW = 1

HIP_SUCCESS = 0
HIP_ERROR_INVALID_VALUE = 1
HIP_ERROR_NOT_SUPPORTED = 801


class Warp34Exec(C.Structure):
    _fields_ = [
        ("stream", C.c_size_t),
        ("scratch_ptr", C.c_uint64),
        ("scratch_size", C.c_size_t),
        ("flags", C.c_uint64),
    ]


class Warp34KvLayerLayout(C.Structure):
    _fields_ = [
        ("k_base", C.c_uint64),
        ("v_base", C.c_uint64),
        ("k_page_stride_bytes", C.c_uint64),
        ("k_head_stride_bytes", C.c_uint64),
        ("k_token_stride_bytes", C.c_uint64),
        ("v_page_stride_bytes", C.c_uint64),
        ("v_head_stride_bytes", C.c_uint64),
        ("v_token_stride_bytes", C.c_uint64),
        ("namespace_id", C.c_int32),
        ("layer_id", C.c_int32),
        ("local_kv_heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("block_size", C.c_int32),
        ("k_format", C.c_int32),
        ("v_format", C.c_int32),
        ("k_transform", C.c_int32),
        ("v_transform", C.c_int32),
        ("reserved", C.c_int32),
    ]


class Warp34AttentionBatch(C.Structure):
    _fields_ = [
        ("query_start_loc", C.c_void_p),
        ("context_lens_before", C.c_void_p),
        ("seq_lens_after", C.c_void_p),
        ("block_tables", C.c_void_p),
        ("write_slot_mapping", C.c_void_p),
        ("valid_token_mask", C.c_void_p),
        ("valid_req_mask", C.c_void_p),
        ("num_reqs", C.c_int32),
        ("total_tokens", C.c_int32),
        ("max_blocks_per_req", C.c_int32),
        ("max_q_len", C.c_int32),
        ("max_seq_len", C.c_int32),
        ("mask_mode", C.c_int32),
        ("sliding_window", C.c_int32),
        ("sm_scale", C.c_float),
        ("reserved", C.c_int32),
    ]


assert C.sizeof(Warp34Exec) == 32
assert C.sizeof(Warp34KvLayerLayout) == 104
assert C.sizeof(Warp34AttentionBatch) == 96

_EX = C.POINTER(Warp34Exec)
_LAY = C.POINTER(Warp34KvLayerLayout)
_BAT = C.POINTER(Warp34AttentionBatch)

# name -> (restype, argtypes); every symbol the headers under include/ declare
SIGNATURES = {
    # deterministic synthetic inputs (include/warp34_synth.h)
    "warp34_synth_normal_bf16": (None, [C.c_void_p, C.c_size_t, C.c_size_t, C.c_uint64]),
    "warp34_synth_kv_rows_bf16": (None, [C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, C.c_int, C.c_uint64, C.c_int]),
    "warp34_synth_permutation": (None, [C.c_void_p, C.c_int, C.c_uint64]),
    "warp34_synth_uniform_i32": (None, [C.c_void_p, C.c_int, C.c_int32, C.c_int32, C.c_uint64]),
    "warp34_kv_cache_write": (C.c_int, [_EX, _LAY, _BAT, C.c_void_p, C.c_void_p]),
    "warp34_kv_cache_write_strided": (C.c_int, [_EX, _LAY, _BAT, C.c_void_p, C.c_void_p, C.c_int, C.c_int]),
    "warp34_kv_cache_write_bf16": (C.c_int, [_EX, _LAY, _BAT, C.c_void_p, C.c_void_p]),
    "warp34_kv_cache_write_strided_bf16": (C.c_int, [_EX, _LAY, _BAT, C.c_void_p, C.c_void_p, C.c_int]),
    "warp34_paged_attention_f16": (C.c_int, [_EX, _LAY, _BAT, C.c_void_p, C.c_void_p, C.c_int]),
    "warp34_paged_attention_bf16": (C.c_int, [_EX, _LAY, _BAT, C.c_void_p, C.c_void_p, C.c_int]),
    "warp34_paged_attention_f16_force_kernel_for_test":
        (C.c_int, [_EX, _LAY, _BAT, C.c_void_p, C.c_void_p, C.c_int, C.c_int]),
    "warp34_paged_attention_scratch_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int]),
    "warp34_paged_attention_gated_f16": (C.c_int, [_EX, _LAY, _BAT, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]),
    "warp34_paged_attention_bf16_static_scratch": (C.c_int, [_EX, _LAY, _BAT, C.c_void_p, C.c_void_p, C.c_int]),
    "warp34_paged_attention_scratch_bytes_for_layout": (C.c_size_t, [_LAY, C.c_int, C.c_int, C.c_int, C.c_int]),
    # QK RMSNorm + RoPE on packed bf16 rows, optionally fused with the paged KV write
    "warp34_dflash_qk_norm_rope_bf16":
        (C.c_int, [_EX, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                   C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]),
    "warp34_dflash_qk_norm_rope_bf16_f32_table":
        (C.c_int, [_EX, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                   C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]),
    "warp34_dflash_qk_norm_rope_bf16_f32_table_qout":
        (C.c_int, [_EX, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                   C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]),
    "warp34_dflash_qk_norm_rope_kv_write_bf16_f32_table":
        (C.c_int, [_EX, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, _LAY, C.c_void_p,
                   C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float]),
    "warp34_fused_qk_rmsnorm_rope_gate_strided_f16":
        (C.c_int, [_EX] + [C.c_void_p] * 9 + [C.c_int] * 11 + [C.c_float, C.c_float]),
    "warp34_fused_qk_rmsnorm_rope_gate_f16":
        (C.c_int, [_EX] + [C.c_void_p] * 9 + [C.c_int] * 9 + [C.c_float, C.c_float]),
    "warp34_fused_qk_rmsnorm_rope_gate_kv_write_f16":
        (C.c_int, [_EX] + [C.c_void_p] * 10 + [_LAY, C.c_void_p] + [C.c_int] * 12 + [C.c_float, C.c_float]),
    "warp34_host_decode_graph_bucket": (C.c_int, [C.c_int]),
    "warp34_host_pack_batched_decode_blob":
        (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p]),
    "warp34_host_batched_decode_batch_at":
        (None, [C.c_uint64, C.c_uint64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, _BAT]),
    "warp34_apply_attn_output_gate_f16":
        (C.c_int, [_EX, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int]),
    # QSA sparse paged attention over selected 4-token groups (plain, and with the per-64 output transform)
    "warp34_qsa_sparse_paged_attn_f16":
        (C.c_int, [_EX, C.c_void_p, C.c_void_p, _LAY, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                   C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float]),
    "warp34_qsa_sparse_paged_attn_hadamard_f16":
        (C.c_int, [_EX, C.c_void_p, C.c_void_p, _LAY, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                   C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float]),
    "warp34_cuda_error_string": (C.c_char_p, [C.c_int]),
    "warp34_get_device_count": (C.c_int, [C.POINTER(C.c_int)]),
    "warp34_set_device": (C.c_int, [C.c_int]),
    "warp34_device_synchronize": (C.c_int, []),
    "warp34_get_mem_info": (C.c_int, [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "warp34_malloc": (C.c_int, [C.POINTER(C.c_void_p), C.c_size_t]),
    "warp34_free": (C.c_int, [C.c_void_p]),
    "warp34_memcpy_h2d_async": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]),
    "warp34_memcpy_d2h_async": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]),
    "warp34_memcpy_d2d_async": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]),
    "warp34_memset_async": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t, C.c_size_t]),
    "warp34_stream_create": (C.c_int, [C.POINTER(C.c_size_t)]),
    "warp34_stream_destroy": (C.c_int, [C.c_size_t]),
    "warp34_stream_synchronize": (C.c_int, [C.c_size_t]),
    "warp34_event_create": (C.c_int, [C.POINTER(C.c_size_t), C.c_int]),
    "warp34_event_destroy": (C.c_int, [C.c_size_t]),
    "warp34_event_record": (C.c_int, [C.c_size_t, C.c_size_t]),
    "warp34_stream_wait_event": (C.c_int, [C.c_size_t, C.c_size_t]),
    "warp34_event_synchronize": (C.c_int, [C.c_size_t]),
    "warp34_event_elapsed_ms": (C.c_int, [C.POINTER(C.c_float), C.c_size_t, C.c_size_t]),
}

_lib = None


def load():
    """Load the shared library (raises if it has not been built) and set the prototypes."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libwarp34_kernels.so is missing: build it with `python -m warp34_amd.build` "
                "(there is no CPU fallback for the KV-cache kernels)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class Warp34Error(RuntimeError):
    """Mirror of CudaError / check_rc (crates/warp34-host/src/cuda.rs:45-123)."""

    def __init__(self, code, context):
        self.code = code
        try:
            msg = load().warp34_cuda_error_string(code).decode()
        except Exception:
            msg = "?"
        super().__init__("%s failed: code %d (%s)" % (context, code, msg))


def check_rc(rc, context):
    if rc != 0:
        raise Warp34Error(rc, context)


# ---- deterministic synthetic inputs (include/warp34_synth.h) as numpy arrays ----

def synth_normal_bf16(n, seed, first=0):
    """Elements first .. first + n of the N(0,1) stream of `seed`, bf16 bits (uint16)."""
    import numpy as np

    out = np.empty(n, dtype=np.uint16)
    load().warp34_synth_normal_bf16(out.ctypes.data, first, n, seed)
    return out


def synth_kv_rows_bf16(rows, kv_heads, head_dim, seed, n_outliers=3, first_row=0):
    """Rows first_row .. first_row + rows of the K / V tensor of `seed`: [rows, kv_heads, head_dim] bf16 bits."""
    import numpy as np

    out = np.empty((rows, kv_heads, head_dim), dtype=np.uint16)
    load().warp34_synth_kv_rows_bf16(out.ctypes.data, first_row, rows, kv_heads, head_dim, seed, n_outliers)
    return out


def synth_permutation(n, seed):
    import numpy as np

    out = np.empty(n, dtype=np.int32)
    load().warp34_synth_permutation(out.ctypes.data, n, seed)
    return out


def synth_uniform_i32(n, lo, hi, seed):
    import numpy as np

    out = np.empty(n, dtype=np.int32)
    load().warp34_synth_uniform_i32(out.ctypes.data, n, lo, hi, seed)
    return out
