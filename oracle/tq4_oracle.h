/*
 * tq4_oracle.h -- CPU restatement of the reference's KV-cache hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product library links, loads or calls this
 * code: it exists so that tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
 * can check (and time) the HIP path against the reference's algorithm.
 *
 * The reference has no CPU implementation of this path and cannot be compiled here
 * (CUDA kernels + a Rust host), so there is no oracle/_ref build; every function below
 * restates the reference source it cites, with the numerics the CUDA source leaves to
 * nvcc's -use_fast_math fixed as follows (declared oracle numerics):
 *   - fp32 arithmetic in source order, no FMA contraction (build with -ffp-contract=off);
 *   - 32-lane warp sums as the xor butterfly with offsets 16,8,4,2,1
 *     (csrc/tq/tq4_kv_common.cuh:54-60);
 *   - rsqrtf(x)  := (float)(1.0 / sqrt((double)x));
 *   - a / b      := IEEE-754 fp32 division, round to nearest even;
 *   - float -> fp16 / bf16 conversions round to nearest even;
 *   - attention: fp32 dequantisation (scale * centroid), fp64 dot products, softmax and
 *     accumulation (the tolerance of the parity tests covers the fp32/fp16 differences of
 *     the kernels).
 *
 * Pins (what each function is checked against, see tests/test_oracle_*.py):
 *   tables            reference literals (tests/golden/tq4_tables.json) + Lloyd-Max fixed
 *                     point of the Beta(256) coordinate density by numeric integration
 *   tq4o_wht256       Sylvester Hadamard matrix / 16, exact on integer inputs; involution
 *   tq4o_encode_row   independent fp64 nearest-centroid + least-squares restatement,
 *                     zero-row special case, layout pins (132 B stride, nibble order)
 *                     -- exact code/scale BYTES for general inputs are pinned by no
 *                     reference-held vector (none exists): "parity unpinned" beyond that
 *   tq4o_encode_row_plain  (TQ4 without the rotation) the same fp64 restatement on the raw
 *                     128-element blocks, zero-block special case, one-centroid rows reproduced
 *                     exactly -- exact BYTES for general inputs: "parity unpinned" as above
 *   tq4o_attention    closed forms (Q=K=0 -> running mean of V, single key -> that V row),
 *                     brute-force fp64 softmax over independently dequantised rows
 *   tq4o_split_merge  equality with the single-pass result
 *   fp8 e4m3 / q8_0   conversion: brute force over all 256 codes (nearest finite code, ties to
 *                     the even code, saturation at 448); rows: scale = amax / 448 (amax / 127),
 *                     round trip error bounds, layout pins (264 B: codes then two fp32 scales;
 *                     272 B: four {fp32 scale, 64 int8}) -- exact BYTES for general inputs are
 *                     pinned by no reference-held vector: "parity unpinned" beyond that
 *   tq4o_qk_norm_rope independent fp64 restatement (RMS norm, weight, rotation of the (c, c + dim/2)
 *                     pairs) within one bf16 ulp; identity rotation at cos = 1, sin = 0; pair norms
 *                     preserved; V bit-identical; cache rows = append of the rotated K.  The
 *                     reference's golden tensors for this operator are not in its tree (LFS
 *                     pointers only), so exact bf16 bits are "parity unpinned"
 *   tq4o_fused_qk_rmsnorm_rope_gate  independent fp64 restatement (Gemma norm, plane selection,
 *                     partial rotation) within one fp16 ulp; position 0 -> the normed row itself;
 *                     pair norms preserved; un-rotated tail and gate copied bit for bit; text-only
 *                     positions (three equal planes) = plain RoPE; masked tokens untouched.  No
 *                     vector of this operator is in the reference tree: exact fp16 bits are
 *                     "parity unpinned"
 *   tq4o_qsa_sparse   the reference test's known answer (V = 0.25, gate 0 -> 0.125, ple/gpu_tests.rs:677-681);
 *                     all groups of a sequence selected = dense causal attention of the last token;
 *                     brute-force fp64 softmax over independently dequantised rows with skipped groups,
 *                     keys behind the token position and masked tokens; per-64 transform = Sylvester
 *                     H64 / 8, exact on small integers, an involution
 */
#ifndef TQ4_ORACLE_H
#define TQ4_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { TQ4O_FMT_FP16 = 0, TQ4O_FMT_BF16 = 1, TQ4O_FMT_TQ4 = 2, TQ4O_FMT_Q8_0 = 3, TQ4O_FMT_FP8 = 4 };
enum { TQ4O_XF_IDENTITY = 0, TQ4O_XF_WHT256 = 1 };
enum { TQ4O_DT_F16 = 0, TQ4O_DT_BF16 = 1 };

/* Host-pointer mirror of warp34_kv_layer_layout (csrc/warp34_cuda.h:59-80). */
typedef struct {
    uint8_t* k_base;
    uint8_t* v_base;
    uint64_t k_page_stride, k_head_stride, k_token_stride;
    uint64_t v_page_stride, v_head_stride, v_token_stride;
    int32_t  local_kv_heads, head_dim, block_size;
    int32_t  k_format, v_format, k_transform, v_transform;
} tq4o_layout;

/* Host-pointer mirror of warp34_attention_batch (csrc/warp34_cuda.h:82-101). */
typedef struct {
    const int32_t* query_start_loc;
    const int32_t* context_lens_before;
    const int32_t* seq_lens_after;
    const int32_t* block_tables;
    const int32_t* write_slot_mapping;
    const uint8_t* valid_token_mask;
    const uint8_t* valid_req_mask;
    int32_t num_reqs, total_tokens, max_blocks_per_req;
    int32_t mask_mode, sliding_window;
    float   sm_scale;
} tq4o_batch;

/* --- tables (csrc/tq/tq4_codebook.cuh:46-101) --- */
const float* tq4o_centroids256(void);  /* [16] */
const float* tq4o_boundaries256(void); /* [15] */
const float* tq4o_signs256(void);      /* [256] */

/* --- scalar conversions (crates/warp34-host/src/cuda/half.rs:10-95 semantics) --- */
float    tq4o_f16_to_f32(uint16_t h);
uint16_t tq4o_f32_to_f16(float f);
float    tq4o_bf16_to_f32(uint16_t h);
uint16_t tq4o_f32_to_bf16(float f);

/* --- csrc/tq/tq4_kv_common.cuh:75-107 : in-place 256-point Walsh-Hadamard, scaled 1/16 --- */
void tq4o_wht256(float* x);

/* --- op_kv_cache.cu:152-218 : quantize one 256-wide row (fp32 values of the fp16/bf16
 * source) into 132 bytes --- */
void tq4o_encode_row(const float* x, uint8_t* dst132);
/* TQ4 without the rotation: head_dim / 128 blocks of 66 bytes (op_kv_cache.cu:219-264) */
void tq4o_encode_row_plain(const float* x, int head_dim, uint8_t* dst);

/* OCP FP8 E4M3 (finite-only, max 448) <-> fp32: round to nearest even, saturating
 * (__nv_cvt_float2_to_fp8x2(.., __NV_SATFINITE, __NV_E4M3) in op_kv_cache.cu:83-86). */
uint8_t tq4o_f32_to_e4m3(float f);
float tq4o_e4m3_to_f32(uint8_t c);

/* 8-bit rows of a 256-wide head (x already transformed if the layer rotates):
 *   fp8:  264 B = 256 e4m3 codes, then fp32 d0 (elements 0..127) and d1 (128..255);
 *         d = amax / 448, code = e4m3(x / d)                  (op_kv_cache.cu:64-140)
 *   q8_0: 272 B = 4 x {fp32 d, 64 int8}; d = amax / 127, q = clamp(roundf(x / d), +-127)
 *                                                             (op_kv_cache.cu:32-62) */
void tq4o_encode_row_fp8(const float* x, uint8_t* dst);
void tq4o_encode_row_q8(const float* x, uint8_t* dst);
void tq4o_dequant_row_fp8(const uint8_t* src, float* y);
void tq4o_dequant_row_q8(const uint8_t* src, float* y);

/* --- op_kv_cache.cu:298-306 : dequantise one 132-byte row into the ROTATED domain --- */
void tq4o_dequant_row(const uint8_t* src132, float* y);

/* un-rotate: x = sign * WHT(y)  (op_kv_cache.cu:775-781) */
void tq4o_unrotate_row(const float* y, float* x);

/* --- op_kv_cache.cu:325-368, 798-824 : paged append.  k_in/v_in are 16-bit rows of dtype
 * in_dtype with strides in elements.  Returns 0, or -1 for an unsupported layout. --- */
int tq4o_kv_cache_write(const tq4o_layout* L, const tq4o_batch* B,
                        const uint16_t* k_in, const uint16_t* v_in,
                        int k_row_stride, int v_row_stride, int in_dtype);

/* --- op_kv_cache.cu:373-457,619-792 : paged GQA attention, one (token, q_head) row at a
 * time.  q is 16-bit of dtype q_dtype; out is fp32 [total_tokens, num_q_heads, head_dim];
 * rows that the reference leaves untouched are left untouched here too.
 * n_threads > 1 spreads rows over pthreads (results do not depend on it). --- */
/* ops/op_dflash2.cu:338-418,1251-1410: RMSNorm over each Q and K head of packed bf16 rows
 * [rows, (q_heads + 2 kv_heads) * dim], RoPE with a [table_rows, dim] cos|sin table (fp32 or bf16),
 * Q to q_out (or in place), K in place -- or, with a layout and a slot mapping, K (rotated) and V
 * (as it is) into the paged cache in the layout's formats.  Rows whose position is outside the
 * table are skipped. */
int tq4o_qk_norm_rope_bf16(uint16_t* qkv, uint16_t* q_out, const int32_t* positions, const uint16_t* qw,
                           const uint16_t* kw, const void* table, int table_is_f32, int rows, int q_heads,
                           int kv_heads, int dim, int table_rows, float eps, const tq4o_layout* L,
                           const int32_t* write_slot_mapping);

/* ops/op_norms_rope_act.cu:524-689,1201-1246: the fused Gemma RMSNorm + interleaved mRoPE + gate split
 * of the target model's full-attention layers, fp16.  q_gate_in [tokens, q_gate_row_stride]: per Q
 * head head_dim query elements then head_dim gate elements; k_in [tokens, k_row_stride]; positions
 * [3, pos_plane_stride]; outputs contiguous.  Masked tokens are skipped.  Returns -1 for the
 * arguments the reference rejects, -2 for head sizes outside the restated summation order
 * (head_dim a multiple of 8, at most 1024). */
int tq4o_fused_qk_rmsnorm_rope_gate_f16(const uint16_t* q_gate_in, const uint16_t* k_in, const uint16_t* q_norm_w,
                                        const uint16_t* k_norm_w, const int32_t* positions,
                                        const uint8_t* valid_token_mask, uint16_t* q_out, uint16_t* k_out,
                                        uint16_t* gate_out, int num_tokens, int pos_plane_stride, int num_q_heads,
                                        int num_kv_heads, int head_dim, int rotary_dim, int mrope_s0, int mrope_s1,
                                        int mrope_s2, int q_gate_row_stride, int k_row_stride, float rope_theta,
                                        float rms_eps);

/* ops/op_norms_rope_act.cu:742-759: out = attn_out * sigmoid(gate), fp16 [num_tokens, total_dim];
 * rows with a zero mask byte are skipped.  Pinned by the float64 sigmoid within one fp16 ulp,
 * g = 0 -> a / 2 exactly, saturation at large |g|. */
int tq4o_apply_attn_output_gate_f16(const uint16_t* attn_out, const uint16_t* gate, uint16_t* out,
                                    const uint8_t* valid_token_mask, int num_tokens, int total_dim);

/* QSA sparse paged attention over selected 4-token groups (op_qsa.cu:716-1158,1446-1571;
 * hadamard_inline.cuh:11-50); fp16 query, gate and output bits. */
int tq4o_qsa_sparse_paged_attn_f16(const tq4o_layout* L, const uint16_t* q, const uint16_t* gate,
                                   const int32_t* selected_phys_blocks, const int32_t* selected_logical_blocks,
                                   const int32_t* num_selected_blocks, const int32_t* token_seq_pos,
                                   const uint8_t* valid_token_mask, uint16_t* out, int num_tokens,
                                   int local_q_heads, int select_k_blocks, float sm_scale, int hadamard64);

int tq4o_paged_attention(const tq4o_layout* L, const tq4o_batch* B,
                         const uint16_t* q, int q_dtype, float* out, int num_q_heads,
                         int n_threads);

/* Same, but the key range of every row is cut into n_splits contiguous page ranges whose
 * partial (acc, m, l) states are merged as op_paged_attn.cu:1132-1218 does. */
int tq4o_paged_attention_split(const tq4o_layout* L, const tq4o_batch* B,
                               const uint16_t* q, int q_dtype, float* out, int num_q_heads,
                               int n_splits);

/* --- deterministic synthetic inputs: SplitMix64 -> Box-Muller (fp64) -> RNE bf16/fp16 --- */
uint64_t tq4o_splitmix64(uint64_t* state);
/* fills n values ~ N(0,1) rounded to dtype; channels listed in outlier_cols (period
 * head_dim within every row of row_elems) are multiplied by 20 before rounding */
void tq4o_fill_normal(uint16_t* dst, size_t n, uint64_t seed, int dtype);
void tq4o_fill_kv_rows(uint16_t* dst, size_t rows, int kv_heads, int head_dim,
                       uint64_t seed, int dtype, int n_outliers);
void tq4o_permutation(int32_t* dst, int n, uint64_t seed);

/* number of hardware threads the timed baseline may use */
int tq4o_hw_threads(void);

#ifdef __cplusplus
}
#endif
#endif
