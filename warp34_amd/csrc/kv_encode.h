// Row encoders of the paged KV formats for gfx950, shared by the append kernel and the fused
// QK-norm + RoPE + append kernel.  A row is encoded by one half of a wave64 (32 lanes); the
// arithmetic and its order follow the reference's 32-lane warp (op_kv_cache.cu:32-218) and are
// bit-exact with the CPU restatement when the including file is built with -ffp-contract=off.
#pragma once

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

// Encodes one 256-wide row held as v[j] = x[l32 + 32 j] (not yet transformed) in `format` /
// `transform`, assembles it in the half-wave's LDS area `row` (272 bytes, 8-byte aligned) and
// stores it at dst (nothing is stored for dst == nullptr).  16-bit formats are stored directly.  The caller guarantees what the append
// entry points check: head_dim 256, TQ4 with WHT256, 8-bit rows 4-byte aligned.
__device__ __forceinline__ void encode_store_row(float (&v)[8], int format, int transform, int lane,
                                                 uint8_t* row, uint8_t* dst) {
    const int l32 = lane & 31;
    if (format == WARP34_KV_FORMAT_FP16 || format == WARP34_KV_FORMAT_BF16) {
        uint16_t* d16 = reinterpret_cast<uint16_t*>(dst);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            d16[l32 + 32 * j] = (format == WARP34_KV_FORMAT_BF16) ? BF16::from_f32(v[j]) : F16::from_f32(v[j]);
        return;
    }
    int n_dwords = 33;
    if (format == WARP34_KV_FORMAT_TQ4) {
        tq4_encode_row(v, lane, row);
    } else {
        if (transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = apply_sign(v[j], l32 + 32 * j);
            wht256_half_wave(v, lane);
        }
        if (format == WARP34_KV_FORMAT_FP8_E4M3) {
            fp8_encode_row_rotated(v, lane, row);
            n_dwords = 66;
        } else {
            q8_encode_row_rotated(v, lane, row);
            n_dwords = 68;
        }
    }
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_wave_barrier();
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    if (dst == nullptr) return;  // a half that only keeps the other half's cross-lane steps company
    if ((reinterpret_cast<uintptr_t>(dst) & 3u) == 0) {
        const uint32_t* r32 = reinterpret_cast<const uint32_t*>(row);
        uint32_t* d32 = reinterpret_cast<uint32_t*>(dst);
        for (int i = l32; i < n_dwords; i += 32) d32[i] = r32[i];
    } else {  // TQ4 rows promise 2-byte alignment only
        const uint16_t* r16 = reinterpret_cast<const uint16_t*>(row);
        uint16_t* d16 = reinterpret_cast<uint16_t*>(dst);
        for (int i = l32; i < 2 * n_dwords; i += 32) d16[i] = r16[i];
    }
}

// ---- host-side checks shared by the entry points that write rows ----
inline bool format_supported_for_write(int format, int transform, int head_dim) {
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

inline bool is_8bit_format(int format) {
    return format == WARP34_KV_FORMAT_Q8_0 || format == WARP34_KV_FORMAT_FP8_E4M3;
}

// Q8_0 and FP8 rows carry fp32 scales (alignof 4, tq4_kv_common.cuh:28-46) and are stored with
// 32-bit stores.
inline bool rows_aligned_for_write(const warp34_kv_layer_layout* l) {
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


}  // namespace w34
