// Quantize-on-append for gfx950: writes one (token, kv head) K row and V row per wave64
// into the paged slabs described by warp34_kv_layer_layout.
//
// Replaces the reference's kv_cache_write_kernel / write_kv_row (op_kv_cache.cu:10-368) and
// kv_cache_write_bf16_kernel (op_kv_cache.cu:798-824) behind the same entry points
// (op_kv_cache.cu:828-858,1172-1190).
//
// Mapping: lanes 0-31 of a wave encode the K row, lanes 32-63 the V row, so the reference's
// 32-lane reduction tree (tq4_kv_common.cuh:54-60) is reproduced with xor shuffles that stay
// inside one half of the wave.  Element i of a row lives in lane i%32, register i/32, as in
// op_kv_cache.cu:164-167.
//
// Numerics of the TQ4 encode (bit-exact contract with the CPU restatement): fp32 in source
// order with FMA contraction disabled for this file (-ffp-contract=off), rsqrt(x) computed
// as (float)(1.0/sqrt((double)x)), IEEE fp32 division, round-to-nearest-even fp16 scale.
#include "kv_encode.h"

namespace w34 {

// One wave per (token, kv head): blockIdx.x counts groups of four tokens, blockIdx.y the kv heads;
// lanes 0-31 write K, lanes 32-63 write V.  Everything up to the row addresses is the same for
// the whole wave and is kept in scalar registers (block_magic = floor(2^32 / block_size): the
// page of a slot without a division).
template <typename TIn>
__global__ __launch_bounds__(256) void kv_append_kernel(warp34_kv_layer_layout L,
                                                        warp34_attention_batch B,
                                                        const uint16_t* __restrict__ k_in,
                                                        const uint16_t* __restrict__ v_in,
                                                        int k_row_stride, int v_row_stride,
                                                        int check_req_mask, uint32_t block_magic) {
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int tok = (int)blockIdx.x * 4 + wave;
    const int head = (int)blockIdx.y;
    if (tok >= B.total_tokens) return;
    if (B.valid_token_mask != nullptr && B.valid_token_mask[tok] == 0) return;
    if (check_req_mask) {
        int a, b;
        const int r = find_request(B, tok, a, b);
        if (r < 0 || (B.valid_req_mask != nullptr && B.valid_req_mask[r] == 0)) return;
    }
    const int32_t slot = B.write_slot_mapping[tok];
    if (slot < 0) return;
    int page = (int)__umulhi((uint32_t)slot, block_magic);  // the quotient or one less
    page += (slot - page * L.block_size >= L.block_size) ? 1 : 0;
    const int off = slot - page * L.block_size;

    const int lane = lane_id();
    const int is_v = lane >> 5;
    const int l32 = lane & 31;
    const int format = is_v ? L.v_format : L.k_format;
    const uint64_t k_dst = L.k_base + (uint64_t)page * L.k_page_stride_bytes + (uint64_t)head * L.k_head_stride_bytes +
                           (uint64_t)off * L.k_token_stride_bytes;
    const uint64_t v_dst = L.v_base + (uint64_t)page * L.v_page_stride_bytes + (uint64_t)head * L.v_head_stride_bytes +
                           (uint64_t)off * L.v_token_stride_bytes;
    const uint16_t* k_src = k_in + (size_t)tok * (size_t)k_row_stride + (size_t)head * (size_t)L.head_dim;
    const uint16_t* v_src = v_in + (size_t)tok * (size_t)v_row_stride + (size_t)head * (size_t)L.head_dim;
    uint8_t* dst = reinterpret_cast<uint8_t*>((uintptr_t)(is_v ? v_dst : k_dst));
    const uint16_t* src = is_v ? v_src : k_src;

    __shared__ __align__(8) uint8_t rows[4][2][272];
    if (format == WARP34_KV_FORMAT_FP8_E4M3 || format == WARP34_KV_FORMAT_Q8_0) {
        // host side guarantees head_dim == 256 and 4-byte aligned rows
        float v[8];
        uint8_t* row = rows[wave][is_v];
        const int n_dwords = format == WARP34_KV_FORMAT_FP8_E4M3 ? 66 : 68;
        const uint16_t* src8 = src + 8 * l32;
        if ((reinterpret_cast<uintptr_t>(src8) & 15u) == 0) {
            const uint4 raw = *reinterpret_cast<const uint4*>(src8);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[2 * j] = TIn::to_f32((uint16_t)(w[j] & 0xffffu));
                v[2 * j + 1] = TIn::to_f32((uint16_t)(w[j] >> 16));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = TIn::to_f32(src8[j]);
        }
        // rotated rows: the same encoders over the transformed row
        if ((is_v ? L.v_transform : L.k_transform) == WARP34_KV_TRANSFORM_RADEMACHER_WHT256) sign_wht256(v, lane);
        if (format == WARP34_KV_FORMAT_FP8_E4M3) {
            fp8_encode_row(v, lane, row);
        } else {
            q8_encode_row(v, lane, row);
        }
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        __builtin_amdgcn_wave_barrier();
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        const uint32_t* r32 = reinterpret_cast<const uint32_t*>(row);
        uint32_t* d32 = reinterpret_cast<uint32_t*>(dst);
        d32[l32] = r32[l32];
        d32[l32 + 32] = r32[l32 + 32];
        if (l32 + 64 < n_dwords) d32[l32 + 64] = r32[l32 + 64];
        return;
    }
    if (format == WARP34_KV_FORMAT_TQ4) {
        // host side guarantees head_dim 256 or 128.  Rotated rows exist at 256 with the WHT-256
        // transform only; everything else is the plain block quantiser (op_kv_cache.cu:152,219).
        const bool rotated = L.head_dim == 256 &&
                             (is_v ? L.v_transform : L.k_transform) == WARP34_KV_TRANSFORM_RADEMACHER_WHT256;
        // lane l32 takes elements 8 l32 .. 8 l32 + 7: one 16-byte load where the source allows it
        // (lanes beyond a 128-element row carry zeros)
        float v[8];
        const uint16_t* src8 = src + 8 * l32;
        if (8 * l32 >= L.head_dim) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = 0.0f;
        } else if ((reinterpret_cast<uintptr_t>(src8) & 15u) == 0) {
            const uint4 raw = *reinterpret_cast<const uint4*>(src8);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[2 * j] = TIn::to_f32((uint16_t)(w[j] & 0xffffu));
                v[2 * j + 1] = TIn::to_f32((uint16_t)(w[j] >> 16));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = TIn::to_f32(src8[j]);
        }
        // the row is assembled in LDS and leaves with one 32-bit store per lane (16-bit stores
        // when the destination is only 2-byte aligned, which is all the row format promises)
        uint8_t* row = rows[wave][is_v];
        if (rotated) {
            tq4_encode_row(v, lane, row);
        } else {
            tq4_encode_row_plain(v, lane, row);
        }
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        __builtin_amdgcn_wave_barrier();
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        if (L.head_dim == 256 && (reinterpret_cast<uintptr_t>(dst) & 3u) == 0) {
            const uint32_t* r32 = reinterpret_cast<const uint32_t*>(row);
            uint32_t* d32 = reinterpret_cast<uint32_t*>(dst);
            d32[l32] = r32[l32];
            if (l32 == 0) d32[32] = r32[32];
        } else {
            const uint16_t* r16 = reinterpret_cast<const uint16_t*>(row);
            uint16_t* d16 = reinterpret_cast<uint16_t*>(dst);
            const int n16 = 33 * (L.head_dim >> 7);  // 66 bytes per 128 elements
            d16[l32] = r16[l32];
            if (l32 + 32 < n16) d16[l32 + 32] = r16[l32 + 32];
            if (l32 + 64 < n16) d16[l32 + 64] = r16[l32 + 64];
        }
        return;
    }
    // 16-bit storage formats: plain copy when the storage type is the source type,
    // otherwise convert through fp32 (op_kv_cache.cu:18-31).
    uint16_t* d16 = reinterpret_cast<uint16_t*>(dst);
    const bool same = (format == TIn::kStorageFormat);
    for (int c = l32; c < L.head_dim; c += 32) {
        const uint16_t b = src[c];
        if (same) {
            d16[c] = b;
        } else {
            const float f = TIn::to_f32(b);
            d16[c] = (format == WARP34_KV_FORMAT_BF16) ? BF16::from_f32(f) : F16::from_f32(f);
        }
    }
}

static inline uint32_t append_block_magic(int block_size) {
    return block_size <= 1 ? 0xFFFFFFFFu : (uint32_t)((1ull << 32) / (uint32_t)block_size);
}

template <typename TIn>
static int launch_append(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                         const warp34_attention_batch* batch, const void* k_in, const void* v_in,
                         int k_row_stride, int v_row_stride) {
    const dim3 grid((unsigned)((batch->total_tokens + 3) / 4), (unsigned)layout->local_kv_heads);
    const int check_req = (batch->valid_req_mask != nullptr && batch->query_start_loc != nullptr &&
                           batch->num_reqs > 0)
                              ? 1
                              : 0;
    hipLaunchKernelGGL((kv_append_kernel<TIn>), grid, dim3(256), 0, (hipStream_t)ex->stream,
                       *layout, *batch, (const uint16_t*)k_in, (const uint16_t*)v_in, k_row_stride,
                       v_row_stride, check_req, append_block_magic(layout->block_size));
    return (int)hipGetLastError();
}

}  // namespace w34

using namespace w34;

// op_kv_cache.cu:828-850
extern "C" int warp34_kv_cache_write_strided(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                             const warp34_attention_batch* batch, const void* k_in,
                                             const void* v_in, int k_row_stride, int v_row_stride) {
    if (ex == nullptr || layout == nullptr || batch == nullptr || k_in == nullptr || v_in == nullptr) {
        return (int)hipErrorInvalidValue;
    }
    if (layout->k_format == WARP34_KV_FORMAT_FP8_E4M3 || layout->v_format == WARP34_KV_FORMAT_FP8_E4M3) {
        // gfx950 always has the FP8 path (the reference gates it on the device generation,
        // op_kv_cache.cu:839-842)
        if (layout->head_dim != 256) return (int)hipErrorInvalidValue;
    }
    if (batch->total_tokens <= 0 || layout->local_kv_heads <= 0) return 0;
    const int min_stride = layout->local_kv_heads * layout->head_dim;
    if (k_row_stride < min_stride || v_row_stride < min_stride) return (int)hipErrorInvalidValue;
    if (batch->write_slot_mapping == nullptr || layout->block_size <= 0 || layout->k_base == 0 ||
        layout->v_base == 0) {
        return (int)hipErrorInvalidValue;
    }
    if (!format_supported_for_write(layout->k_format, layout->k_transform, layout->head_dim) ||
        !format_supported_for_write(layout->v_format, layout->v_transform, layout->head_dim)) {
        return (int)hipErrorNotSupported;
    }
    if (!rows_aligned_for_write(layout)) return (int)hipErrorInvalidValue;
    return launch_append<F16>(ex, layout, batch, k_in, v_in, k_row_stride, v_row_stride);
}

// op_kv_cache.cu:852-858
extern "C" int warp34_kv_cache_write(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                     const warp34_attention_batch* batch, const void* k_in,
                                     const void* v_in) {
    if (layout == nullptr) return (int)hipErrorInvalidValue;
    const int stride = layout->local_kv_heads * layout->head_dim;
    return warp34_kv_cache_write_strided(ex, layout, batch, k_in, v_in, stride, stride);
}

// Layouts the bf16 entry points accept: the reference's BF16 identity layout
// (op_kv_cache.cu:860-865) plus TQ4 (rotated or plain) and, at head_dim 256, the 8-bit row formats.
static bool valid_bf16_entry_layout(const warp34_kv_layer_layout* l) {
    if (!l || l->local_kv_heads <= 0 || l->block_size <= 0 || l->head_dim <= 0 || l->head_dim > 256 ||
        !l->k_base || !l->v_base) {
        return false;
    }
    const bool bf16 = l->k_format == WARP34_KV_FORMAT_BF16 && l->v_format == WARP34_KV_FORMAT_BF16 &&
                      l->k_transform == WARP34_KV_TRANSFORM_IDENTITY &&
                      l->v_transform == WARP34_KV_TRANSFORM_IDENTITY;
    const bool tq4 = l->k_format == WARP34_KV_FORMAT_TQ4 && l->v_format == WARP34_KV_FORMAT_TQ4 &&
                     format_supported_for_write(l->k_format, l->k_transform, l->head_dim) &&
                     format_supported_for_write(l->v_format, l->v_transform, l->head_dim);
    const bool q8 = l->head_dim == 256 && is_8bit_format(l->k_format) && is_8bit_format(l->v_format) &&
                    format_supported_for_write(l->k_format, l->k_transform, 256) &&
                    format_supported_for_write(l->v_format, l->v_transform, 256) &&
                    rows_aligned_for_write(l);
    return bf16 || tq4 || q8;
}

// op_kv_cache.cu:1172-1183
extern "C" int warp34_kv_cache_write_strided_bf16(const warp34_exec* ex,
                                                  const warp34_kv_layer_layout* layout,
                                                  const warp34_attention_batch* batch, const void* k,
                                                  const void* v, int row_stride_elems) {
    if (!ex || !valid_bf16_entry_layout(layout) || !batch || !k || !v ||
        row_stride_elems < layout->local_kv_heads * layout->head_dim || batch->total_tokens < 0 ||
        batch->num_reqs <= 0 || !batch->query_start_loc || !batch->write_slot_mapping) {
        return (int)hipErrorInvalidValue;
    }
    if (!batch->total_tokens) return 0;
    // the reference's bf16 writer always resolves the owning request (op_kv_cache.cu:803-807)
    const dim3 grid((unsigned)((batch->total_tokens + 3) / 4), (unsigned)layout->local_kv_heads);
    hipLaunchKernelGGL((kv_append_kernel<BF16>), grid, dim3(256), 0, (hipStream_t)ex->stream,
                       *layout, *batch, (const uint16_t*)k, (const uint16_t*)v, row_stride_elems,
                       row_stride_elems, 1, append_block_magic(layout->block_size));
    return (int)hipGetLastError();
}

// op_kv_cache.cu:1185-1190
extern "C" int warp34_kv_cache_write_bf16(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                          const warp34_attention_batch* batch, const void* k,
                                          const void* v) {
    if (!valid_bf16_entry_layout(layout)) return (int)hipErrorInvalidValue;
    return warp34_kv_cache_write_strided_bf16(ex, layout, batch, k, v,
                                              layout->local_kv_heads * layout->head_dim);
}
