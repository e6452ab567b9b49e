/*
 * warp34_kv.h -- C ABI of the MI355X (gfx950) KV-cache hot path.
 *
 * This is the drop-in boundary: the descriptor structs, enum values, symbol names,
 * argument lists and the int error convention are those of the reference's kernel
 * crate for this path, so warp34-host binds to libwarp34_kernels built from this
 * repository without source changes:
 *
 *   reference C header : crates/warp34-kernels/csrc/warp34_cuda.h:20-44   (enums)
 *                        crates/warp34-kernels/csrc/warp34_cuda.h:50-101  (structs)
 *                        crates/warp34-kernels/csrc/warp34_cuda.h:142-164 (runtime shims)
 *                        crates/warp34-kernels/csrc/warp34_cuda.h:353-373 (KV write + attention)
 *   reference Rust view: crates/warp34-kernels/src/ffi.rs:6-90,701-760
 *
 * Conventions (all entry points):
 *   - return 0 on success; a positive value is a hipError_t; nothing is synchronised
 *     inside a call, all work is enqueued on ex->stream and is stream-capturable;
 *   - the caller owns every buffer; the library allocates nothing.  Temporary space
 *     comes only from ex->scratch_ptr / ex->scratch_size.  When the scratch is null,
 *     misaligned (16 B) or too small the attention calls run a single-pass kernel and
 *     do not touch it;
 *   - every index array in warp34_attention_batch is a DEVICE pointer; the scalar
 *     fields max_q_len / max_seq_len / max_blocks_per_req are host-known upper bounds
 *     used only for launch geometry -- results do not depend on them;
 *   - masked tokens / requests (valid_token_mask[tok]==0, valid_req_mask[req]==0,
 *     write slot < 0) write nothing and leave the output row untouched.
 */
#ifndef WARP34_KV_H
#define WARP34_KV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* warp34_cuda.h:20-24 */
enum {
    WARP34_KV_NAMESPACE_TARGET_FULL_ATTN = 0,
    WARP34_KV_NAMESPACE_MTP_FULL_ATTN    = 1,
    WARP34_KV_NAMESPACE_DFLASH_DRAFT_CTX = 2,
};

/* warp34_cuda.h:26-32 */
enum {
    WARP34_KV_FORMAT_FP16     = 0, /* 2 B / element                                   */
    WARP34_KV_FORMAT_BF16     = 1, /* 2 B / element                                   */
    WARP34_KV_FORMAT_TQ4      = 2, /* 66 B per 128 elements: fp16 scale + 64 B nibbles */
    WARP34_KV_FORMAT_Q8_0     = 3, /* 68 B per 64 elements: fp32 scale + 64 int8       */
    WARP34_KV_FORMAT_FP8_E4M3 = 4, /* 264 B per 256 elements: 256 E4M3 + 2 fp32 scales */
};

/* warp34_cuda.h:34-37 */
enum {
    WARP34_KV_TRANSFORM_IDENTITY          = 0,
    WARP34_KV_TRANSFORM_RADEMACHER_WHT256 = 1,
};

/* warp34_cuda.h:39-44 */
enum {
    WARP34_ATTN_MASK_CAUSAL           = 0,
    WARP34_ATTN_MASK_SYMMETRIC_WINDOW = 1, /* legacy name */
    WARP34_ATTN_MASK_NONCAUSAL_WINDOW = 1,
};

/* warp34_cuda.h:50-57 -- 32 bytes */
typedef struct {
    uintptr_t stream;       /* hipStream_t */
    uint64_t  scratch_ptr;  /* device workspace, may be 0 */
    size_t    scratch_size; /* bytes */
    uint64_t  flags;
} warp34_exec;

/* warp34_cuda.h:59-80 -- 104 bytes */
typedef struct {
    uint64_t k_base;
    uint64_t v_base;
    uint64_t k_page_stride_bytes;
    uint64_t k_head_stride_bytes;
    uint64_t k_token_stride_bytes;
    uint64_t v_page_stride_bytes;
    uint64_t v_head_stride_bytes;
    uint64_t v_token_stride_bytes;
    int32_t  namespace_id;
    int32_t  layer_id;
    int32_t  local_kv_heads;
    int32_t  head_dim;
    int32_t  block_size;
    int32_t  k_format;
    int32_t  v_format;
    int32_t  k_transform;
    int32_t  v_transform;
    int32_t  reserved;
} warp34_kv_layer_layout;

/* warp34_cuda.h:82-101 -- 96 bytes */
typedef struct {
    const int32_t* query_start_loc;     /* [num_reqs + 1] */
    const int32_t* context_lens_before; /* [num_reqs] or NULL (= seq_lens_after - q_len) */
    const int32_t* seq_lens_after;      /* [num_reqs] */
    const int32_t* block_tables;        /* [num_reqs, max_blocks_per_req] physical page ids */
    const int32_t* write_slot_mapping;  /* [total_tokens] page*block_size + offset, <0 = skip */
    const uint8_t* valid_token_mask;    /* [total_tokens] or NULL */
    const uint8_t* valid_req_mask;      /* [num_reqs] or NULL */
    int32_t        num_reqs;
    int32_t        total_tokens;
    int32_t        max_blocks_per_req;
    int32_t        max_q_len;
    int32_t        max_seq_len;
    int32_t        mask_mode;
    int32_t        sliding_window;
    float          sm_scale;
    int32_t        reserved;
} warp34_attention_batch;

#if defined(__cplusplus)
static_assert(sizeof(warp34_exec) == 32, "warp34_exec ABI size");
static_assert(sizeof(warp34_kv_layer_layout) == 104, "warp34_kv_layer_layout ABI size");
static_assert(sizeof(warp34_attention_batch) == 96, "warp34_attention_batch ABI size");
#else
_Static_assert(sizeof(warp34_exec) == 32, "warp34_exec ABI size");
_Static_assert(sizeof(warp34_kv_layer_layout) == 104, "warp34_kv_layer_layout ABI size");
_Static_assert(sizeof(warp34_attention_batch) == 96, "warp34_attention_batch ABI size");
#endif

/* ------------------------------------------------------------------------------------
 * Quantize-on-append (replaces op_kv_cache.cu:325-368,828-858).
 *
 * k_in / v_in: [total_tokens, row_stride] fp16 elements, head h of token t at
 * t*row_stride + h*head_dim.  Row strides are in ELEMENTS and must be
 * >= local_kv_heads*head_dim.  Destination row:
 *   base + (slot / block_size)*page_stride + head*head_stride + (slot % block_size)*token_stride.
 * Formats built: FP16, BF16 (converted from fp16), TQ4 (rotated rows at head_dim 256 with the
 * WHT256 transform; every other TQ4 layout at head_dim 128 or 256 is the plain block quantiser,
 * one 66-byte block per 128 elements, op_kv_cache.cu:219-264), Q8_0 and FP8_E4M3 (head_dim 256,
 * identity or WHT256 transform, rows 4-byte aligned).
 * TQ4, Q8_0 and FP8 rows are bit-exact with the declared-numerics CPU restatement of
 * op_kv_cache.cu:32-264.
 * ------------------------------------------------------------------------------------ */
int warp34_kv_cache_write(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                          const warp34_attention_batch* batch,
                          const void* k_in, const void* v_in);               /* warp34_cuda.h:353-355 */
int warp34_kv_cache_write_strided(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                  const warp34_attention_batch* batch,
                                  const void* k_in, const void* v_in,
                                  int k_row_stride, int v_row_stride);       /* warp34_cuda.h:356-359 */

/* bf16 source rows (replaces op_kv_cache.cu:798-824,1172-1190).  The reference accepts
 * only BF16-format identity layouts here; this library additionally accepts the TQ4 layouts
 * and, at head_dim 256, Q8_0 and FP8_E4M3 (bf16 -> fp32 is exact, the encode is the same
 * arithmetic). */
int warp34_kv_cache_write_bf16(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                               const warp34_attention_batch* batch,
                               const void* k_in, const void* v_in);          /* warp34_cuda.h:362-363 */
int warp34_kv_cache_write_strided_bf16(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                       const warp34_attention_batch* batch,
                                       const void* k_in, const void* v_in,
                                       int row_stride_elems);                /* warp34_cuda.h:364-365 */

/* ------------------------------------------------------------------------------------
 * Paged GQA attention (replaces op_paged_attn.cu:1266-1448 and op_kv_cache.cu:1192-1241).
 *
 * q_in / attn_out: [total_tokens, num_q_heads, head_dim] contiguous, fp16 for _f16 and
 * bf16 for _bf16.  kv_head = q_head / (num_q_heads / local_kv_heads).  Visible keys of
 * token t of request r: [min_kv, max_kv] with
 *   max_kv = (mask_mode == NONCAUSAL_WINDOW ? seq_after-1 : ctx_before + q_off), clamped to seq_after-1
 *   min_kv = sliding_window > 0 ? max(0, ctx_before + q_off - sliding_window + 1) : 0
 * Output = softmax(sm_scale * q.K^T) V in fp32 accumulation; an empty key range gives zeros.
 * _f16 accepts FP16, TQ4, Q8_0 and FP8_E4M3 layouts (TQ4 and the 8-bit ones with each slab
 * plain or WHT256, op_paged_attn.cu:347,570; K and V in the same format); _bf16 accepts BF16
 * (reference) and, additionally,
 * the TQ4 and 8-bit layouts.  head_dim must be 256 -- or, for the 16-bit layouts, 128
 * (op_kv_cache.cu:873,1227) --, block_size a multiple of 16, and the token stride the row size
 * (2 * head_dim / 132 / 272 / 264 bytes) with 16-byte aligned slabs.
 * ------------------------------------------------------------------------------------ */
int warp34_paged_attention_f16(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                               const warp34_attention_batch* batch,
                               const void* q_in, void* attn_out, int num_q_heads);  /* warp34_cuda.h:369-372 */
int warp34_paged_attention_bf16(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                const warp34_attention_batch* batch,
                                const void* q_in, void* attn_out, int num_q_heads); /* warp34_cuda.h:366-367 */

/* Test-only kernel selector (op_paged_attn.cu:1451-1519): use_64q == 0 runs the decode / verify
 * kernel as a single pass (no split, scratch untouched), any other value the 128-row MFMA tile
 * kernel (when the layout admits it: a power-of-two number of q heads per kv head; otherwise as 0).
 * Both compute the same function, with different summation orders. */
int warp34_paged_attention_f16_force_kernel_for_test(
    const warp34_exec* ex, const warp34_kv_layer_layout* layout,
    const warp34_attention_batch* batch,
    const void* q_in, void* attn_out, int num_q_heads, int use_64q);

/* ------------------------------------------------------------------------------------
 * Producer side of the path: per-head RMSNorm + RoPE over packed bf16 rows
 * [rows, (q_heads + 2 kv_heads) * dim] (replaces ops/op_dflash2.cu:338-418,1251-1410).
 *
 * For each Q and K head: y = bf16(x * rsqrt(mean(x^2) + eps) * w), then the pairs
 * (c, c + dim/2) are rotated with cos = table[pos][c], sin = table[pos][dim/2 + c]
 * (table: [table_rows, dim], bf16 for the first entry point, fp32 for the others).  Rows
 * whose position is outside [0, table_rows) are skipped.  Q goes to q_out
 * [rows, q_heads * dim] when q_out != NULL, otherwise it is rotated in place; V is never
 * modified.  dim <= 256 and even, q_heads % kv_heads == 0, eps > 0 and finite, q_out != qkv.
 *
 * _kv_write_: rows with write_slot_mapping[row] >= 0 store the rotated K and the V row in
 * the paged cache (same addressing as the append entry points) and leave the packed K as it
 * was; rows with a negative slot are rotated in place.  The reference accepts BF16 pages
 * only (op_dflash2.cu:1326-1333); this library also takes TQ4 + WHT256, FP8_E4M3 and Q8_0
 * pages at dim 256 (K and V in the same format and transform), written with the encoders
 * of the append entry points: a fused call equals operator + append bit for bit.
 * ------------------------------------------------------------------------------------ */
int warp34_dflash_qk_norm_rope_bf16(const warp34_exec* ex, void* qkv, const int32_t* positions,
                                    const void* qw, const void* kw, const void* table,
                                    int rows, int q_heads, int kv_heads, int dim,
                                    int table_rows, float eps);               /* warp34_cuda.h:635-637 */
int warp34_dflash_qk_norm_rope_bf16_f32_table(const warp34_exec* ex, void* qkv,
                                              const int32_t* positions, const void* qw,
                                              const void* kw, const void* table,
                                              int rows, int q_heads, int kv_heads, int dim,
                                              int table_rows, float eps);     /* warp34_cuda.h:619-621 */
int warp34_dflash_qk_norm_rope_bf16_f32_table_qout(const warp34_exec* ex, void* qkv, void* q_out,
                                                   const int32_t* positions, const void* qw,
                                                   const void* kw, const void* table,
                                                   int rows, int q_heads, int kv_heads, int dim,
                                                   int table_rows, float eps); /* warp34_cuda.h:622-624 */
int warp34_dflash_qk_norm_rope_kv_write_bf16_f32_table(
    const warp34_exec* ex, void* qkv, void* q_out, const int32_t* positions,
    const void* qw, const void* kw, const void* table,
    const warp34_kv_layer_layout* kv_layout, const int32_t* write_slot_mapping,
    int rows, int q_heads, int kv_heads, int dim, int table_rows, float eps);  /* warp34_cuda.h:625-628 */

/* Producer side of the target model's gated full-attention layers (model/forward.rs:1105-1148):
 * Gemma RMSNorm (weight 1 + w) over every Q head of q_gate_in ([tokens, q_gate_row_stride], head h
 * at h * 2 * head_dim: head_dim query elements, then head_dim gate elements) and every K head of
 * k_in ([tokens, k_row_stride]), interleaved mRoPE over the first rotary_dim elements (pair
 * (i, i + rotary_dim / 2), position plane i % 3 for i below 3 * s1 / 3 * s2, plane 0 otherwise;
 * positions = three planes pos_plane_stride apart), and the gate halves copied to gate_out; all
 * fp16, outputs dense [tokens, heads, head_dim].  Tokens whose valid_token_mask byte is 0 are
 * skipped (mask may be NULL).  Replaces ops/op_norms_rope_act.cu:524-689,1201-1272.  This build
 * wants head_dim % 8 == 0 and <= 256, rotary_dim <= 256, strides % 8 == 0 and 16-byte aligned
 * pointers (hipErrorNotSupported otherwise). */
int warp34_fused_qk_rmsnorm_rope_gate_strided_f16(
    const warp34_exec* ex, const void* q_gate_in, const void* k_in, const void* q_norm_w,
    const void* k_norm_w, const int32_t* positions, const uint8_t* valid_token_mask, void* q_out,
    void* k_out, void* gate_out, int num_tokens, int pos_plane_stride, int num_q_heads,
    int num_kv_heads, int head_dim, int rotary_dim, int mrope_s0, int mrope_s1, int mrope_s2,
    int q_gate_row_stride, int k_row_stride, float rope_theta, float rms_eps); /* warp34_cuda.h:264-287 */
int warp34_fused_qk_rmsnorm_rope_gate_f16(
    const warp34_exec* ex, const void* q_gate_in, const void* k_in, const void* q_norm_w,
    const void* k_norm_w, const int32_t* positions, const uint8_t* valid_token_mask, void* q_out,
    void* k_out, void* gate_out, int num_tokens, int pos_plane_stride, int num_q_heads,
    int num_kv_heads, int head_dim, int rotary_dim, int mrope_s0, int mrope_s1, int mrope_s2,
    float rope_theta, float rms_eps);                                         /* warp34_cuda.h:241-262 */
/* The same operator fused with the append.  No counterpart in the reference, which runs the
 * operator and then warp34_kv_cache_write_strided (model/forward.rs:1128-1148): here the finished K
 * rows and the V rows of v_in ([tokens, v_row_stride], fp16) go straight to the pages of kv_layout
 * at write_slot_mapping[token] (negative: no cache write for that token), with bits equal to that
 * sequence's.  k_out may be NULL.  head_dim 256, K and V pages of one format and transform. */
int warp34_fused_qk_rmsnorm_rope_gate_kv_write_f16(
    const warp34_exec* ex, const void* q_gate_in, const void* k_in, const void* v_in,
    const void* q_norm_w, const void* k_norm_w, const int32_t* positions,
    const uint8_t* valid_token_mask, void* q_out, void* k_out, void* gate_out,
    const warp34_kv_layer_layout* kv_layout, const int32_t* write_slot_mapping, int num_tokens,
    int pos_plane_stride, int num_q_heads, int num_kv_heads, int head_dim, int rotary_dim,
    int mrope_s0, int mrope_s1, int mrope_s2, int q_gate_row_stride, int k_row_stride,
    int v_row_stride, float rope_theta, float rms_eps);

/* Consumer side of the path: out = attn_out * sigmoid(gate) over fp16 [num_tokens, total_dim]
 * (replaces ops/op_norms_rope_act.cu:742-759,1329-1344; called right after
 * warp34_paged_attention_f16 in the gated layers, model/forward.rs:1192-1211).  Rows whose
 * valid_token_mask byte is 0 are left untouched; the mask may be NULL. */
int warp34_apply_attn_output_gate_f16(const warp34_exec* ex, const void* attn_out, const void* gate,
                                      void* out, const uint8_t* valid_token_mask,
                                      int num_tokens, int total_dim);             /* warp34_cuda.h:297-300 */

/* warp34_paged_attention_f16 followed by warp34_apply_attn_output_gate_f16 in one call, with the
 * bits of that sequence; the ungated output never goes to memory.  No counterpart in the reference
 * (model/forward.rs:1192-1211 makes the two calls).  gate: fp16 [total_tokens, num_q_heads, 256],
 * 8-byte aligned.  Rows of masked tokens and requests stay untouched. */
int warp34_paged_attention_gated_f16(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                     const warp34_attention_batch* batch, const void* q_in,
                                     const void* gate, void* attn_out, int num_q_heads);

/* QSA sparse paged attention: query token t attends over its own list of selected 4-token groups
 * (replaces ops/op_qsa.cu:716-1158,1446-1571,1711-1751).  Group j of token t is rows
 * (phys % (block_size / 4)) * 4 .. + 3 of page phys / (block_size / 4), phys =
 * selected_phys_blocks[t * select_k_blocks + j]; its keys sit at positions
 * 4 * selected_logical_blocks[..] + 0..3.  Groups with phys < 0, groups at or behind
 * num_selected_blocks[t] and keys behind token_seq_pos[t] are skipped.  out = fp16(attention *
 * sigmoid(gate)) (gate may be NULL); the hadamard form then applies H64 / 8 to every 64-element
 * block of the rounded row (ops/hadamard_inline.cuh:11-50).  Rows of masked tokens and of tokens
 * without a visible key are written as zeros.  q, gate, out: fp16 [num_tokens, local_q_heads, 256].
 * Page formats: rotated TQ4, FP16, FP8-E4M3 and Q8_0 (8-bit rows plain or rotated), K and V alike;
 * other layouts return hipErrorNotSupported.  Uses ex->scratch for split partials when it is large
 * enough (num_tokens * local_q_heads * splits * 1040 bytes, splits <= 16). */
int warp34_qsa_sparse_paged_attn_f16(const warp34_exec* ex, const void* q, const void* gate,
                                     const warp34_kv_layer_layout* kv_layout,
                                     const int32_t* selected_phys_blocks,
                                     const int32_t* selected_logical_blocks,
                                     const int32_t* num_selected_blocks, const int32_t* token_seq_pos,
                                     const uint8_t* valid_token_mask, void* out, int num_tokens,
                                     int local_q_heads, int select_k_blocks, float sm_scale);  /* warp34_cuda.h:851-859 */
int warp34_qsa_sparse_paged_attn_hadamard_f16(
    const warp34_exec* ex, const void* q, const void* gate, const warp34_kv_layer_layout* kv_layout,
    const int32_t* selected_phys_blocks, const int32_t* selected_logical_blocks,
    const int32_t* num_selected_blocks, const int32_t* token_seq_pos, const uint8_t* valid_token_mask,
    void* out, int num_tokens, int local_q_heads, int select_k_blocks, float sm_scale);  /* warp34_cuda.h:860-865 */

/* Bytes of scratch the attention entry points can make use of for a batch of this shape
 * (split-K partials).  No counterpart in the reference, whose engine simply guarantees
 * >= 8 MiB (op_paged_attn.cu:1301-1304); provided so a host can size ex->scratch. */
size_t warp34_paged_attention_scratch_bytes(int total_tokens, int num_q_heads, int max_seq_len);
/* The same for a known layout and request count: the exact figure the launchers use (the form
 * above does not know local_kv_heads and returns the largest need over all layouts).
 * num_reqs < 0: unknown, total_tokens is assumed.  No counterpart in the reference. */
size_t warp34_paged_attention_scratch_bytes_for_layout(const warp34_kv_layer_layout* layout, int total_tokens,
                                                       int num_reqs, int num_q_heads, int max_seq_len);

/* warp34_paged_attention_bf16 for callers that cannot allocate or provide a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  The split-K partials go to a WARP34_STATIC_SCRATCH_BYTES array inside the library,
 * one copy per device, held until the process ends; ex->scratch_ptr / scratch_size are ignored and
 * nothing is allocated or freed.  Results equal warp34_paged_attention_bf16 with an 8 MiB scratch
 * bit for bit: like that call, a batch whose full split wants more than the array holds
 * (warp34_paged_attention_scratch_bytes_for_layout) runs with fewer chunks, or without the
 * shared-prefix pass.  Limit: a batch of more than 4032 query rows (total_tokens x num_q_heads;
 * two 1040-byte records per row no longer fit) is refused with hipErrorOutOfMemory (2) and nothing
 * is launched.  All calls on one device share the array: calls that overlap in time on one device (two
 * streams) race on it and must be ordered by the caller.  The first call on a device looks up the
 * array's address; make it outside stream capture. */
#define WARP34_STATIC_SCRATCH_BYTES (8u << 20)
int warp34_paged_attention_bf16_static_scratch(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                               const warp34_attention_batch* batch, const void* q_in,
                                               void* attn_out, int num_q_heads);

/* ------------------------------------------------------------------------------------
 * Runtime shims a standalone harness needs (replace op_init.cu; warp34_cuda.h:135,142-164).
 * ------------------------------------------------------------------------------------ */
const char* warp34_cuda_error_string(int code);
int warp34_get_device_count(int* out_count);
int warp34_set_device(int device_id);
int warp34_device_synchronize(void);
int warp34_get_mem_info(size_t* out_free, size_t* out_total);
int warp34_malloc(void** out_ptr, size_t bytes);
int warp34_free(void* ptr);
int warp34_memcpy_h2d_async(void* dst, const void* src, size_t bytes, uintptr_t stream);
int warp34_memcpy_d2h_async(void* dst, const void* src, size_t bytes, uintptr_t stream);
int warp34_memcpy_d2d_async(void* dst, const void* src, size_t bytes, uintptr_t stream);
int warp34_memset_async(void* dst, int value, size_t bytes, uintptr_t stream);
int warp34_stream_create(uintptr_t* out_stream);
int warp34_stream_destroy(uintptr_t stream);
int warp34_stream_synchronize(uintptr_t stream);
int warp34_event_create(uintptr_t* out_event, int enable_timing);
int warp34_event_destroy(uintptr_t event);
int warp34_event_record(uintptr_t event, uintptr_t stream);
int warp34_stream_wait_event(uintptr_t stream, uintptr_t event);
int warp34_event_synchronize(uintptr_t event);
int warp34_event_elapsed_ms(float* out_ms, uintptr_t start_event, uintptr_t end_event);

#ifdef __cplusplus
}
#endif
#endif /* WARP34_KV_H */
