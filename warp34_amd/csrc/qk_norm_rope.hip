// QK RMSNorm + RoPE over packed bf16 rows for gfx950, optionally fused with the append of the
// rotated K row and the V row into the paged KV cache: the producer side of the KV path, one
// HBM round trip instead of two (operator, then append).
//
// Replaces qk_norm_rope_bf16_warp and its four entry points (ops/op_dflash2.cu:338-418,
// 1251-1410).  The reference's fused cache write takes BF16 pages only (op_dflash2.cu:1326-1333);
// here the cache may also be TQ4 + WHT256, FP8-E4M3 or Q8_0 at head_dim 256, encoded by the same
// row encoders as the append kernel, so a fused write equals operator + append bit for bit.
//
// Mapping: one wave per work item, two items' worth of lanes: lanes 0-31 and lanes 32-63 each
// play the reference's 32-thread warp.  A Q item handles two Q heads; a KV item handles one K
// head (lanes 0-31: norm, rotation, cache row or in-place store) and, when the cache is
// written, the V row of the same kv head (lanes 32-63).
//
// Numerics (bit-exact contract with the CPU restatement, file built with -ffp-contract=off):
// fp32 in source order; sum of squares in the order of reduce_sum256_exact_warp
// (op_dflash2.cu:30-39); rsqrt(x) computed as (float)(1.0 / sqrt((double)x)); bf16 RNE.
#include "kv_encode.h"

namespace w34 {

struct NormRopeParams {
    uint16_t* qkv;         // [rows, (q_heads + 2 kv_heads) * dim] bf16
    uint16_t* q_out;       // [rows, q_heads * dim] or null (Q in place)
    const int32_t* positions;
    const uint16_t* qw;
    const uint16_t* kw;
    const void* table;     // [table_rows, dim]: cos (dim/2) | sin (dim/2)
    const int32_t* write_slot_mapping;  // null: no cache write
    warp34_kv_layer_layout L;
    int rows, q_heads, kv_heads, dim, table_rows;
    float eps;
};

// D256: head size 256 known at compile time (no bounds tests, the second pass reuses the
// values of the first instead of loading them again).
template <bool TABLE_F32, bool D256>
__global__ __launch_bounds__(256) void qk_norm_rope_kernel(const NormRopeParams P) {
    __shared__ __align__(8) uint8_t rows_lds[4][2][272];
    __shared__ __align__(16) float xpose_lds[4][2][256];  // register layout of the rotation -> the encoder's
    const int wave = (int)(threadIdx.x >> 6);
    const int lane = lane_id();
    const int half_id = lane >> 5;
    const int l32 = lane & 31;
    // Items are ordered KV items of all rows first, then the Q items: the long items (norm +
    // two row encodes) start first and every workgroup holds items of one kind.
    const int q_items = (P.q_heads + 1) >> 1;
    const long long item = (long long)blockIdx.x * 4 + wave;
    const long long n_kv_items = (long long)P.rows * P.kv_heads;
    int row, it;
    if (item < n_kv_items) {
        row = (int)(item / P.kv_heads);
        it = q_items + (int)(item - (long long)row * P.kv_heads);
    } else {
        const long long qi = item - n_kv_items;
        row = q_items > 0 ? (int)(qi / q_items) : P.rows;
        it = q_items > 0 ? (int)(qi - (long long)row * q_items) : 0;
    }
    if (row >= P.rows) return;
    const int pos = P.positions[row];
    if (pos < 0 || pos >= P.table_rows) return;  // op_dflash2.cu:356

    const int dim = D256 ? 256 : P.dim, half = dim >> 1;
    const size_t row_elems = (size_t)(P.q_heads + 2 * P.kv_heads) * dim;
    uint16_t* row_base = P.qkv + (size_t)row * row_elems;

    // Both halves of the wave run the same instruction stream (the cross-lane steps want the
    // whole wave): the half without a head of its own (the V half of a KV item, the second half
    // of the last Q item when q_heads is odd) computes on a row it may read and stores nothing.
    const bool is_q = it < q_items;
    const bool is_v_half = !is_q && half_id == 1;
    const int kv_head = is_q ? 0 : it - q_items;
    int head = is_q ? 2 * it + half_id : P.q_heads + kv_head;
    const bool has_head = is_q ? head < P.q_heads : !is_v_half;
    if (is_q && head >= P.q_heads) head = P.q_heads - 1;
    const int slot = (!is_q && P.write_slot_mapping != nullptr) ? P.write_slot_mapping[row] : -1;
    const bool to_cache = slot >= 0;  // wave-uniform
    uint8_t* row_lds = rows_lds[wave][half_id];

    // V half: its "head" is the V row of the kv head (read-only)
    uint16_t* src = row_base + (size_t)(is_v_half ? P.q_heads + P.kv_heads + kv_head : head) * dim;
    const uint16_t* w = is_q ? P.qw : P.kw;

    // sum of squares, element c = l32 + 32 k in register k (op_dflash2.cu:362-380)
    float raw[8], sq[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const int c = l32 + 32 * k;
        raw[k] = (D256 || c < dim) ? BF16::to_f32(src[c]) : 0.0f;
        sq[k] = raw[k] * raw[k];
    }
    float s = ((sq[0] + sq[4]) + (sq[2] + sq[6])) + ((sq[1] + sq[5]) + (sq[3] + sq[7]));
    s = half_wave_sum(s, lane);
    const float mean = s / (float)dim + P.eps;
    const float inv = (float)(1.0 / sqrt((double)mean));

    // rotated values of this lane: out[c] and out[half + c] for c = l32, l32 + 32, ... < half
    float lo[4], hi[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int c = l32 + 32 * k;
        lo[k] = hi[k] = 0.0f;
        if (D256 || c < half) {
            const float x_lo = D256 ? raw[k] : BF16::to_f32(src[c]);
            const float x_hi = D256 ? raw[k + 4] : BF16::to_f32(src[half + c]);
            const float a = BF16::to_f32(BF16::from_f32(x_lo * inv * BF16::to_f32(w[c])));
            const float b = BF16::to_f32(BF16::from_f32(x_hi * inv * BF16::to_f32(w[half + c])));
            float cosine, sine;
            if constexpr (TABLE_F32) {
                const float* t = reinterpret_cast<const float*>(P.table) + (size_t)pos * dim;
                cosine = t[c];
                sine = t[half + c];
            } else {
                const uint16_t* t = reinterpret_cast<const uint16_t*>(P.table) + (size_t)pos * dim;
                cosine = BF16::to_f32(t[c]);
                sine = BF16::to_f32(t[half + c]);
            }
            const float ac = a * cosine, bs = b * sine, bc = b * cosine, as = a * sine;
            lo[k] = BF16::to_f32(BF16::from_f32(ac - bs));
            hi[k] = BF16::to_f32(BF16::from_f32(bc + as));
        }
    }

    if (to_cache) {
        // rotated K (lanes 0-31) and the V row as it is (lanes 32-63) into the cache; the packed
        // row keeps its K (op_dflash2.cu:387-416)
        const int page = slot / P.L.block_size, off = slot - page * P.L.block_size;
        uint8_t* dst = reinterpret_cast<uint8_t*>((uintptr_t)(is_v_half ? P.L.v_base : P.L.k_base)) +
                       (size_t)page * (is_v_half ? P.L.v_page_stride_bytes : P.L.k_page_stride_bytes) +
                       (size_t)kv_head * (is_v_half ? P.L.v_head_stride_bytes : P.L.k_head_stride_bytes) +
                       (size_t)off * (is_v_half ? P.L.v_token_stride_bytes : P.L.k_token_stride_bytes);
        const int format = is_v_half ? P.L.v_format : P.L.k_format;
        const int transform = is_v_half ? P.L.v_transform : P.L.k_transform;
        if (format == WARP34_KV_FORMAT_BF16) {  // both slabs are BF16 (host check)
            uint16_t* d16 = reinterpret_cast<uint16_t*>(dst);
            if (is_v_half) {
                for (int c = l32; c < dim; c += 32) d16[c] = src[c];
            } else {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int c = l32 + 32 * k;
                    if (D256 || c < half) {
                        d16[c] = BF16::from_f32(lo[k]);
                        d16[half + c] = BF16::from_f32(hi[k]);
                    }
                }
            }
        } else {
            // Quantised pages: head_dim 256, K and V in the same format and transform (host
            // check), so both halves take the same path through the encoder.  Element
            // l32 + 32 j is lo[j] for j < 4 and hi[j - 4] above.
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = is_v_half ? raw[j] : (j < 4 ? lo[j & 3] : hi[j & 3]);
            strided_to_consecutive(v, lane, xpose_lds[wave][half_id]);
            encode_store_row(v, format, transform, lane, row_lds, dst);
        }
        return;
    }
    if (!has_head) return;
    uint16_t* dst = (is_q && P.q_out != nullptr) ? P.q_out + ((size_t)row * P.q_heads + head) * dim : src;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int c = l32 + 32 * k;
        if (D256 || c < half) {
            dst[c] = BF16::from_f32(lo[k]);
            dst[half + c] = BF16::from_f32(hi[k]);
        }
    }
}

static bool norm_rope_args_ok(const warp34_exec* ex, const void* qkv, const int32_t* positions, const void* qw,
                              const void* kw, const void* table, int rows, int q_heads, int kv_heads, int dim,
                              int table_rows, float eps) {
    return ex && qkv && positions && qw && kw && table && rows >= 0 && q_heads >= 0 && kv_heads > 0 &&
           q_heads % kv_heads == 0 && dim > 0 && dim <= 256 && dim % 2 == 0 && table_rows > 0 && eps > 0.0f &&
           eps <= 3.402823466e38f;  // finite: NaN fails the first comparison, +inf this one
}

template <bool TABLE_F32>
static int launch_norm_rope(const warp34_exec* ex, void* qkv, void* q_out, const int32_t* positions, const void* qw,
                            const void* kw, const void* table, const warp34_kv_layer_layout* layout,
                            const int32_t* write_slot_mapping, int rows, int q_heads, int kv_heads, int dim,
                            int table_rows, float eps) {
    NormRopeParams P{};
    P.qkv = (uint16_t*)qkv;
    P.q_out = (uint16_t*)q_out;
    P.positions = positions;
    P.qw = (const uint16_t*)qw;
    P.kw = (const uint16_t*)kw;
    P.table = table;
    P.write_slot_mapping = write_slot_mapping;
    if (layout != nullptr) P.L = *layout;
    P.rows = rows;
    P.q_heads = q_heads;
    P.kv_heads = kv_heads;
    P.dim = dim;
    P.table_rows = table_rows;
    P.eps = eps;
    const long long items = (long long)rows * ((q_heads + 1) / 2 + kv_heads);
    const unsigned grid = (unsigned)((items + 3) / 4);
    if (dim == 256) {
        hipLaunchKernelGGL((qk_norm_rope_kernel<TABLE_F32, true>), dim3(grid), dim3(256), 0, (hipStream_t)ex->stream, P);
    } else {
        hipLaunchKernelGGL((qk_norm_rope_kernel<TABLE_F32, false>), dim3(grid), dim3(256), 0, (hipStream_t)ex->stream, P);
    }
    return (int)hipGetLastError();
}

}  // namespace w34

using namespace w34;

// op_dflash2.cu:1251-1278 (bf16 cos|sin table)
extern "C" int warp34_dflash_qk_norm_rope_bf16(const warp34_exec* ex, void* qkv, const int32_t* positions,
                                               const void* qw, const void* kw, const void* table, int rows,
                                               int q_heads, int kv_heads, int dim, int table_rows, float eps) {
    if (!norm_rope_args_ok(ex, qkv, positions, qw, kw, table, rows, q_heads, kv_heads, dim, table_rows, eps))
        return (int)hipErrorInvalidValue;
    if (rows == 0) return 0;
    return launch_norm_rope<false>(ex, qkv, nullptr, positions, qw, kw, table, nullptr, nullptr, rows, q_heads,
                                   kv_heads, dim, table_rows, eps);
}

// op_dflash2.cu:1280-1308 (fp32 table, Q to a contiguous buffer when q_out != null)
extern "C" int warp34_dflash_qk_norm_rope_bf16_f32_table_qout(const warp34_exec* ex, void* qkv, void* q_out,
                                                              const int32_t* positions, const void* qw,
                                                              const void* kw, const void* table, int rows,
                                                              int q_heads, int kv_heads, int dim, int table_rows,
                                                              float eps) {
    if (!norm_rope_args_ok(ex, qkv, positions, qw, kw, table, rows, q_heads, kv_heads, dim, table_rows, eps) ||
        q_out == qkv)
        return (int)hipErrorInvalidValue;
    if (rows == 0) return 0;
    return launch_norm_rope<true>(ex, qkv, q_out, positions, qw, kw, table, nullptr, nullptr, rows, q_heads,
                                  kv_heads, dim, table_rows, eps);
}

// op_dflash2.cu:1395-1410
extern "C" int warp34_dflash_qk_norm_rope_bf16_f32_table(const warp34_exec* ex, void* qkv, const int32_t* positions,
                                                         const void* qw, const void* kw, const void* table,
                                                         int rows, int q_heads, int kv_heads, int dim,
                                                         int table_rows, float eps) {
    return warp34_dflash_qk_norm_rope_bf16_f32_table_qout(ex, qkv, nullptr, positions, qw, kw, table, rows, q_heads,
                                                          kv_heads, dim, table_rows, eps);
}

// op_dflash2.cu:1310-1345.  The reference accepts BF16 pages only; TQ4 + WHT256, FP8-E4M3 and
// Q8_0 pages (head_dim 256) are accepted here as well.
extern "C" int warp34_dflash_qk_norm_rope_kv_write_bf16_f32_table(
    const warp34_exec* ex, void* qkv, void* q_out, const int32_t* positions, const void* qw, const void* kw,
    const void* table, const warp34_kv_layer_layout* kv_layout, const int32_t* write_slot_mapping, int rows,
    int q_heads, int kv_heads, int dim, int table_rows, float eps) {
    if (!norm_rope_args_ok(ex, qkv, positions, qw, kw, table, rows, q_heads, kv_heads, dim, table_rows, eps) ||
        !kv_layout || !write_slot_mapping || q_out == qkv || kv_layout->k_base == 0 || kv_layout->v_base == 0 ||
        kv_layout->block_size <= 0 || kv_layout->local_kv_heads != kv_heads || kv_layout->head_dim != dim) {
        return (int)hipErrorInvalidValue;
    }
    const bool bf16_pages = kv_layout->k_format == WARP34_KV_FORMAT_BF16 && kv_layout->v_format == WARP34_KV_FORMAT_BF16;
    const int fmt = kv_layout->k_format;
    const bool quantised_pages =
        dim == 256 && (fmt == WARP34_KV_FORMAT_TQ4 || is_8bit_format(fmt)) && kv_layout->v_format == fmt &&
        kv_layout->v_transform == kv_layout->k_transform &&
        format_supported_for_write(fmt, kv_layout->k_transform, dim) && rows_aligned_for_write(kv_layout);
    if (!bf16_pages && !quantised_pages) return (int)hipErrorInvalidValue;
    if (rows == 0) return 0;
    return launch_norm_rope<true>(ex, qkv, q_out, positions, qw, kw, table, kv_layout, write_slot_mapping, rows,
                                  q_heads, kv_heads, dim, table_rows, eps);
}
