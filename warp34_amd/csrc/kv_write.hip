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
#include "kv_common.h"

namespace w34 {

// Cross-lane moves are DPP / lane-swap VALU operations (lane_xor), not LDS permutes: the encode
// of one row needs 168 of them.  They only move bits, so the arithmetic (and its order) is the
// one of the 32-lane shuffle tree it replaces.
__device__ __forceinline__ int lane_xor1_int(int x, int lane) {
    return __float_as_int(lane_xor<1>(__int_as_float(x), lane));
}

// 32-lane xor butterfly sum, offsets 16,8,4,2,1 (tq4_kv_common.cuh:54-60).
__device__ __forceinline__ float half_wave_sum(float v, int lane) {
    v += lane_xor<16>(v, lane);
    v += lane_xor<8>(v, lane);
    v += lane_xor<4>(v, lane);
    v += lane_xor<2>(v, lane);
    v += lane_xor<1>(v, lane);
    return v;
}

template <int H>
__device__ __forceinline__ float wht_lane_stage(float val, int lane) {
    const float o = lane_xor<H>(val, lane);
    return (lane & H) ? (o - val) : (val + o);
}

// 256-point Walsh-Hadamard over 32 lanes x 8 registers (tq4_kv_common.cuh:75-107):
// stages over index bits 0..4 cross lanes, bits 5..7 stay in registers; the last stage
// carries the 1/16 scale.
__device__ __forceinline__ void wht256_half_wave(float (&v)[8], int lane) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        float val = v[j];
        val = wht_lane_stage<1>(val, lane);
        val = wht_lane_stage<2>(val, lane);
        val = wht_lane_stage<4>(val, lane);
        val = wht_lane_stage<8>(val, lane);
        val = wht_lane_stage<16>(val, lane);
        v[j] = val;
    }
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
        const float a = v[j], b = v[j + 1];
        v[j] = a + b;
        v[j + 1] = a - b;
    }
#pragma unroll
    for (int g = 0; g < 8; g += 4) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float a = v[g + i], b = v[g + i + 2];
            v[g + i] = a + b;
            v[g + i + 2] = a - b;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float a = v[i], b = v[i + 4];
        v[i] = (a + b) * 0.0625f;
        v[i + 4] = (a - b) * 0.0625f;
    }
}

// TQ4 encode of one 256-wide row held as v[j] = x[l32 + 32 j] (op_kv_cache.cu:152-218).
// The 132 row bytes are assembled in `row` (LDS, private to this half-wave).
__device__ __forceinline__ void tq4_encode_row(float (&v)[8], int lane, uint8_t* row) {
    const int l32 = lane & 31;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = apply_sign(v[j], l32 + 32 * j);
    wht256_half_wave(v, lane);

    float s_sq0 = 0.0f, s_sq1 = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        s_sq0 += half_wave_sum(v[j] * v[j], lane);
        s_sq1 += half_wave_sum(v[j + 4] * v[j + 4], lane);
    }
    const float rs0 = (float)(1.0 / sqrt((double)s_sq0));
    const float rs1 = (float)(1.0 / sqrt((double)s_sq1));
    const float inv_norm0 = (s_sq0 > 1e-20f) ? (0.7071067811865475f * rs0) : 0.0f;
    const float inv_norm1 = (s_sq1 > 1e-20f) ? (0.7071067811865475f * rs1) : 0.0f;

    float vc_dot0 = 0.0f, c_sq0 = 0.0f, vc_dot1 = 0.0f, c_sq1 = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float raw_v = v[j];
        const float rv = raw_v * ((j < 4) ? inv_norm0 : inv_norm1);
        int q = 0;
#pragma unroll
        for (int i = 0; i < 15; ++i) q += (rv > kBoundaries[i]) ? 1 : 0;
        // byte m of a 64-byte block holds elements 2m (low nibble) and 2m+1 (high nibble);
        // elements l32 and l32^1 of register j are neighbours.
        const int partner = lane_xor1_int(q, lane);
        if ((l32 & 1) == 0) {
            row[66 * (j >> 2) + 2 + (((j & 3) * 32 + l32) >> 1)] = (uint8_t)(q | (partner << 4));
        }
        const float c = kCentroids[q];
        const float vc = half_wave_sum(raw_v * c, lane);
        const float cc = half_wave_sum(c * c, lane);
        if (j < 4) {
            vc_dot0 += vc;
            c_sq0 += cc;
        } else {
            vc_dot1 += vc;
            c_sq1 += cc;
        }
    }
    if (l32 == 0) {
        const float d0 = (c_sq0 > 1e-10f) ? (vc_dot0 / c_sq0) : 0.0f;
        const float d1 = (c_sq1 > 1e-10f) ? (vc_dot1 / c_sq1) : 0.0f;
        *reinterpret_cast<uint16_t*>(row) = F16::from_f32(d0);
        *reinterpret_cast<uint16_t*>(row + 66) = F16::from_f32(d1);
    }
}

// fp32 -> OCP FP8 E4M3, round to nearest even, saturating at +-448, NaN -> 0x7f
// (__nv_cvt_float2_to_fp8x2(.., __NV_SATFINITE, __NV_E4M3) in op_kv_cache.cu:83-86).  Integer
// arithmetic, so the bits do not depend on a hardware conversion mode.
__device__ __forceinline__ uint32_t f32_to_e4m3(float f) {
    const uint32_t u = __float_as_uint(f);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t ax = u & 0x7fffffffu;
    if (ax > 0x7f800000u) return sign | 0x7fu;
    const float a = __uint_as_float(ax);
    if (a >= 448.0f) return sign | 0x7eu;
    if (a < 0.015625f) return sign | (uint32_t)rintf(a * 512.0f);  // multiples of 2^-9
    uint32_t r = (ax + 0x7ffffu + ((ax >> 20) & 1u)) >> 20;
    r -= (127u - 7u) << 3;
    return sign | (r > 0x7eu ? 0x7eu : r);
}

// 8-bit rows of a 256-wide head, identity transform; lane l32 holds elements 8 l32 .. 8 l32 + 7.
//   FP8:  264 B = 256 codes, then fp32 d0 (elements 0..127) and d1; d = amax / 448
//         (op_kv_cache.cu:104-138)
//   Q8_0: 272 B = 4 x {fp32 d, 64 int8}; d = amax / 127, q = clamp(roundf(x / d))
//         (op_kv_cache.cu:32-62)
// max() is exact and order-free, so only the element-wise arithmetic has to follow the source.
__device__ __forceinline__ void fp8_encode_row(const float (&v)[8], int lane, uint8_t* row) {
    const int l32 = lane & 31;
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
    amax = fmaxf(amax, lane_xor<8>(amax, lane));
    amax = fmaxf(amax, lane_xor<4>(amax, lane));
    amax = fmaxf(amax, lane_xor<2>(amax, lane));
    amax = fmaxf(amax, lane_xor<1>(amax, lane));
    const float d = amax * (1.0f / 448.0f);
    const float inv_d = (d > 1e-30f) ? (1.0f / d) : 0.0f;
    uint32_t w0 = 0, w1 = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        w0 |= f32_to_e4m3(v[j] * inv_d) << (8 * j);
        w1 |= f32_to_e4m3(v[4 + j] * inv_d) << (8 * j);
    }
    *reinterpret_cast<uint2*>(row + 8 * l32) = uint2{w0, w1};
    if ((l32 & 15) == 0) *reinterpret_cast<float*>(row + 256 + 4 * (l32 >> 4)) = d;
}

__device__ __forceinline__ void q8_encode_row(const float (&v)[8], int lane, uint8_t* row) {
    const int l32 = lane & 31;
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
    amax = fmaxf(amax, lane_xor<4>(amax, lane));
    amax = fmaxf(amax, lane_xor<2>(amax, lane));
    amax = fmaxf(amax, lane_xor<1>(amax, lane));
    const float d = amax / 127.0f;
    const float inv_d = (d > 1e-12f) ? (1.0f / d) : 0.0f;
    uint32_t w0 = 0, w1 = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float q0 = fminf(127.0f, fmaxf(-127.0f, roundf(v[j] * inv_d)));
        const float q1 = fminf(127.0f, fmaxf(-127.0f, roundf(v[4 + j] * inv_d)));
        w0 |= ((uint32_t)(int)q0 & 0xffu) << (8 * j);
        w1 |= ((uint32_t)(int)q1 & 0xffu) << (8 * j);
    }
    uint8_t* blk = row + 68 * (l32 >> 3);
    *reinterpret_cast<uint32_t*>(blk + 4 + 8 * (l32 & 7)) = w0;
    *reinterpret_cast<uint32_t*>(blk + 8 + 8 * (l32 & 7)) = w1;
    if ((l32 & 7) == 0) *reinterpret_cast<float*>(blk) = d;
}

// The same two rows from the rotated layout v[j] = y[l32 + 32 j] (y = WHT256(sign * x)), used when
// an 8-bit layer asks for the WHT256 transform (op_kv_cache.cu:36-44,71-99).
__device__ __forceinline__ float half_wave_max(float v, int lane) {
    v = fmaxf(v, lane_xor<16>(v, lane));
    v = fmaxf(v, lane_xor<8>(v, lane));
    v = fmaxf(v, lane_xor<4>(v, lane));
    v = fmaxf(v, lane_xor<2>(v, lane));
    v = fmaxf(v, lane_xor<1>(v, lane));
    return v;
}

__device__ __forceinline__ void fp8_encode_row_rotated(const float (&v)[8], int lane, uint8_t* row) {
    const int l32 = lane & 31;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) amax = fmaxf(amax, fabsf(v[4 * b + j]));
        amax = half_wave_max(amax, lane);
        const float d = amax * (1.0f / 448.0f);
        const float inv_d = (d > 1e-30f) ? (1.0f / d) : 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            row[l32 + 32 * (4 * b + j)] = (uint8_t)f32_to_e4m3(v[4 * b + j] * inv_d);
        }
        if (l32 == 0) *reinterpret_cast<float*>(row + 256 + 4 * b) = d;
    }
}

__device__ __forceinline__ void q8_encode_row_rotated(const float (&v)[8], int lane, uint8_t* row) {
    const int l32 = lane & 31;
#pragma unroll
    for (int sb = 0; sb < 4; ++sb) {
        const float x0 = v[2 * sb], x1 = v[2 * sb + 1];
        const float amax = half_wave_max(fmaxf(fabsf(x0), fabsf(x1)), lane);
        const float d = amax / 127.0f;
        const float inv_d = (d > 1e-12f) ? (1.0f / d) : 0.0f;
        const float q0 = fminf(127.0f, fmaxf(-127.0f, roundf(x0 * inv_d)));
        const float q1 = fminf(127.0f, fmaxf(-127.0f, roundf(x1 * inv_d)));
        uint8_t* blk = row + 68 * sb;
        blk[4 + l32] = (uint8_t)(int)q0;
        blk[4 + 32 + l32] = (uint8_t)(int)q1;
        if (l32 == 0) *reinterpret_cast<float*>(blk) = d;
    }
}

// One wave per (token, kv head); lanes 0-31 write K, lanes 32-63 write V.
template <typename TIn>
__global__ __launch_bounds__(256) void kv_append_kernel(warp34_kv_layer_layout L,
                                                        warp34_attention_batch B,
                                                        const uint16_t* __restrict__ k_in,
                                                        const uint16_t* __restrict__ v_in,
                                                        int k_row_stride, int v_row_stride,
                                                        int check_req_mask) {
    const int wave = (int)(threadIdx.x >> 6);
    const int item = (int)blockIdx.x * 4 + wave;
    const int tok = item / L.local_kv_heads;
    const int head = item - tok * L.local_kv_heads;
    if (tok >= B.total_tokens) return;
    if (B.valid_token_mask != nullptr && B.valid_token_mask[tok] == 0) return;
    if (check_req_mask) {
        int a, b;
        const int r = find_request(B, tok, a, b);
        if (r < 0 || (B.valid_req_mask != nullptr && B.valid_req_mask[r] == 0)) return;
    }
    const int32_t slot = B.write_slot_mapping[tok];
    if (slot < 0) return;
    const int page = slot / L.block_size;
    const int off = slot - page * L.block_size;

    const int lane = lane_id();
    const int is_v = lane >> 5;
    const int l32 = lane & 31;
    const int format = is_v ? L.v_format : L.k_format;
    uint8_t* dst = reinterpret_cast<uint8_t*>((uintptr_t)(is_v ? L.v_base : L.k_base)) +
                   (size_t)page * (is_v ? L.v_page_stride_bytes : L.k_page_stride_bytes) +
                   (size_t)head * (is_v ? L.v_head_stride_bytes : L.k_head_stride_bytes) +
                   (size_t)off * (is_v ? L.v_token_stride_bytes : L.k_token_stride_bytes);
    const uint16_t* src = (is_v ? v_in : k_in) +
                          (size_t)tok * (size_t)(is_v ? v_row_stride : k_row_stride) +
                          (size_t)head * (size_t)L.head_dim;

    __shared__ __align__(8) uint8_t rows[4][2][272];
    if (format == WARP34_KV_FORMAT_FP8_E4M3 || format == WARP34_KV_FORMAT_Q8_0) {
        // host side guarantees head_dim == 256 and 4-byte aligned rows
        float v[8];
        uint8_t* row = rows[wave][is_v];
        const int n_dwords = format == WARP34_KV_FORMAT_FP8_E4M3 ? 66 : 68;
        const uint16_t* src8 = src + 8 * l32;
        if ((is_v ? L.v_transform : L.k_transform) == WARP34_KV_TRANSFORM_RADEMACHER_WHT256) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = apply_sign(TIn::to_f32(src[l32 + 32 * j]), l32 + 32 * j);
            wht256_half_wave(v, lane);
            if (format == WARP34_KV_FORMAT_FP8_E4M3) {
                fp8_encode_row_rotated(v, lane, row);
            } else {
                q8_encode_row_rotated(v, lane, row);
            }
        } else {
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
        if (format == WARP34_KV_FORMAT_FP8_E4M3) {
            fp8_encode_row(v, lane, row);
        } else {
            q8_encode_row(v, lane, row);
        }
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
        // host side guarantees head_dim == 256 and the WHT256 transform for TQ4
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = TIn::to_f32(src[l32 + 32 * j]);
        // the row is assembled in LDS and leaves with one 32-bit store per lane (16-bit stores
        // when the destination is only 2-byte aligned, which is all the row format promises)
        uint8_t* row = rows[wave][is_v];
        tq4_encode_row(v, lane, row);
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        __builtin_amdgcn_wave_barrier();
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        if ((reinterpret_cast<uintptr_t>(dst) & 3u) == 0) {
            const uint32_t* r32 = reinterpret_cast<const uint32_t*>(row);
            uint32_t* d32 = reinterpret_cast<uint32_t*>(dst);
            d32[l32] = r32[l32];
            if (l32 == 0) d32[32] = r32[32];
        } else {
            const uint16_t* r16 = reinterpret_cast<const uint16_t*>(row);
            uint16_t* d16 = reinterpret_cast<uint16_t*>(dst);
            d16[l32] = r16[l32];
            d16[l32 + 32] = r16[l32 + 32];
            if (l32 < 2) d16[l32 + 64] = r16[l32 + 64];
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

static bool format_supported_for_write(int format, int transform, int head_dim) {
    if (format == WARP34_KV_FORMAT_FP16 || format == WARP34_KV_FORMAT_BF16) {
        return transform == WARP34_KV_TRANSFORM_IDENTITY;
    }
    if (format == WARP34_KV_FORMAT_TQ4) {
        return head_dim == 256 && transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256;
    }
    if (format == WARP34_KV_FORMAT_Q8_0 || format == WARP34_KV_FORMAT_FP8_E4M3) {
        // the tail-anchor layers of the default policy store these un-rotated (cache.rs:87-109);
        // the rotated variant is what op_kv_cache.cu:36-44,71-99 accepts as well
        return head_dim == 256 && (transform == WARP34_KV_TRANSFORM_IDENTITY ||
                                   transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256);
    }
    return false;
}

static bool is_8bit_format(int format) {
    return format == WARP34_KV_FORMAT_Q8_0 || format == WARP34_KV_FORMAT_FP8_E4M3;
}

// Q8_0 and FP8 rows carry fp32 scales (alignof 4, tq4_kv_common.cuh:28-46) and are stored with
// 32-bit stores.
static bool rows_aligned_for_write(const warp34_kv_layer_layout* l) {
    if (is_8bit_format(l->k_format) &&
        ((l->k_base | l->k_page_stride_bytes | l->k_head_stride_bytes | l->k_token_stride_bytes) & 3u)) {
        return false;
    }
    if (is_8bit_format(l->v_format) &&
        ((l->v_base | l->v_page_stride_bytes | l->v_head_stride_bytes | l->v_token_stride_bytes) & 3u)) {
        return false;
    }
    return true;
}

template <typename TIn>
static int launch_append(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                         const warp34_attention_batch* batch, const void* k_in, const void* v_in,
                         int k_row_stride, int v_row_stride) {
    const long long items = (long long)batch->total_tokens * layout->local_kv_heads;
    const unsigned grid = (unsigned)((items + 3) / 4);
    const int check_req = (batch->valid_req_mask != nullptr && batch->query_start_loc != nullptr &&
                           batch->num_reqs > 0)
                              ? 1
                              : 0;
    hipLaunchKernelGGL((kv_append_kernel<TIn>), dim3(grid), dim3(256), 0, (hipStream_t)ex->stream,
                       *layout, *batch, (const uint16_t*)k_in, (const uint16_t*)v_in, k_row_stride,
                       v_row_stride, check_req);
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
// (op_kv_cache.cu:860-865) plus, at head_dim 256, TQ4 + WHT256 and the 8-bit row formats.
static bool valid_bf16_entry_layout(const warp34_kv_layer_layout* l) {
    if (!l || l->local_kv_heads <= 0 || l->block_size <= 0 || l->head_dim <= 0 || l->head_dim > 256 ||
        !l->k_base || !l->v_base) {
        return false;
    }
    const bool bf16 = l->k_format == WARP34_KV_FORMAT_BF16 && l->v_format == WARP34_KV_FORMAT_BF16 &&
                      l->k_transform == WARP34_KV_TRANSFORM_IDENTITY &&
                      l->v_transform == WARP34_KV_TRANSFORM_IDENTITY;
    const bool tq4 = l->head_dim == 256 && l->k_format == WARP34_KV_FORMAT_TQ4 &&
                     l->v_format == WARP34_KV_FORMAT_TQ4 &&
                     l->k_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 &&
                     l->v_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256;
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
    const long long items = (long long)batch->total_tokens * layout->local_kv_heads;
    const unsigned grid = (unsigned)((items + 3) / 4);
    hipLaunchKernelGGL((kv_append_kernel<BF16>), dim3(grid), dim3(256), 0, (hipStream_t)ex->stream,
                       *layout, *batch, (const uint16_t*)k, (const uint16_t*)v, row_stride_elems,
                       row_stride_elems, 1);
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
