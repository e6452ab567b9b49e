// Row encoders of the paged KV formats for gfx950, shared by the append kernel and the fused
// QK-norm + RoPE + append kernels.  A row is encoded by one half of a wave64 (32 lanes); the
// arithmetic and the order of every sum follow the reference's 32-lane warp
// (op_kv_cache.cu:32-218, tq4_kv_common.cuh:54-107) and are bit-exact with the CPU restatement
// when the including file is built with -ffp-contract=off.
//
// Data layout: lane l32 holds the eight consecutive elements 8 l32 .. 8 l32 + 7 (the reference's
// lane holds l32 + 32 j).  Index bits 0-2 are then register bits and bits 3-7 lane bits.  The
// butterfly stages run in the reference's order (1, 2, 4, ..., 128, the scale on the last); its
// 32-element sums (one per register there: elements 32 j .. 32 j + 31) are four-lane groups
// here, all eight reduced by ONE pass of the same tree (xor 16, 8 across lanes; xor 4, 2, 1
// across registers); two neighbouring codes share a lane.  Every sum adds the same operands in
// the same order, so the bytes are those of the 32-lane form at half its instruction count.
#pragma once

#include "kv_common.h"

namespace w34 {

// 32-lane xor butterfly sum, offsets 16,8,4,2,1 (tq4_kv_common.cuh:54-60); cross-lane moves are
// DPP / lane-swap VALU operations (lane_xor), not LDS permutes.
__device__ __forceinline__ float half_wave_sum(float v, int lane) {
    v += lane_xor<16>(v, lane);
    v += lane_xor<8>(v, lane);
    v += lane_xor<4>(v, lane);
    v += lane_xor<2>(v, lane);
    v += lane_xor<1>(v, lane);
    return v;
}

// One butterfly stage across lanes: lanes with bit H clear take x + x[lane ^ H], the others
// x[lane ^ H] - x (tq4_kv_common.cuh:75-107).  flip = sign bit in the lanes with bit H set.
template <int H>
__device__ __forceinline__ float wht_lane_stage(float val, uint32_t flip, int lane) {
    if constexpr (H == 16) {
        // after the swap r[0] holds the even-row operand and r[1] the odd-row operand, in both rows
        const uint32_t xi = __float_as_uint(val);
        const auto r = __builtin_amdgcn_permlane16_swap(xi, xi, false, false);
        return __uint_as_float(r[0]) + __uint_as_float(r[1] ^ flip);
    } else {
        return lane_xor<H>(val, lane) + __uint_as_float(__float_as_uint(val) ^ flip);
    }
}

// sign[i] * x[i], then the 256-point Walsh-Hadamard transform with the 1/16 scale on the last
// stage; v[j] = x[8 l32 + j] on entry and y[8 l32 + j] on return.
__device__ __forceinline__ void sign_wht256(float (&v)[8], int lane) {
    const int l32 = lane & 31;
    {
        const uint32_t sb = sign_word(l32 >> 2) >> (8 * (l32 & 3));
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = __uint_as_float(__float_as_uint(v[j]) ^ (((sb >> j) & 1u) << 31));
    }
    // stages 1, 2, 4: registers
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
        v[i] = a + b;
        v[i + 4] = a - b;
    }
    // stages 8 .. 128: lanes (each stage over all eight registers: independent instructions
    // between a write and the cross-lane read of it)
    const uint32_t f1 = (uint32_t)(lane & 1) << 31, f2 = (uint32_t)(lane & 2) << 30, f4 = (uint32_t)(lane & 4) << 29;
    const uint32_t f8 = (uint32_t)(lane & 8) << 28, f16 = (uint32_t)(lane & 16) << 27;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = wht_lane_stage<1>(v[j], f1, lane);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = wht_lane_stage<2>(v[j], f2, lane);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = wht_lane_stage<4>(v[j], f4, lane);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = wht_lane_stage<8>(v[j], f8, lane);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = wht_lane_stage<16>(v[j], f16, lane) * 0.0625f;
}

// sums of the eight 32-element groups: lanes 4 g .. 4 g + 3 receive the sum of group g, added
// in the order of the 32-lane butterfly (element e with e ^ 16, then ^ 8, ^ 4, ^ 2, ^ 1)
__device__ __forceinline__ float group32_sums(const float (&p)[8], int lane) {
    float t[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) t[r] = p[r] + lane_xor<2>(p[r], lane);
#pragma unroll
    for (int r = 0; r < 8; ++r) t[r] = t[r] + lane_xor<1>(t[r], lane);
    const float a0 = t[0] + t[4], a1 = t[1] + t[5], a2 = t[2] + t[6], a3 = t[3] + t[7];
    const float b0 = a0 + a2, b1 = a1 + a3;
    return b0 + b1;
}

// (((0 + S0) + S1) + S2) + S3 over the four groups of a 16-lane row, in every lane of the row
__device__ __forceinline__ float row_sum_of_groups(float s, int lane) {
    float x = 0.0f + s;  // the reference accumulates from +0: a sum of -0 terms ends as +0
    x = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x114, 0xF, 0xF, false)) + s;  // row_shr:4
    x = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x114, 0xF, 0xF, false)) + s;
    x = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x114, 0xF, 0xF, false)) + s;
    // lanes 12-15 of the row hold the total; hand it to the whole row
    return __int_as_float(__builtin_amdgcn_ds_bpermute((lane | 12) << 2, __float_as_int(x)));
}

// TQ4 encode of one 256-wide row, v[j] = x[8 l32 + j] (op_kv_cache.cu:152-218).  The 132 row
// bytes are assembled in `row` (LDS, private to this half-wave).  Lanes 0-15 hold the first
// scale block, lanes 16-31 the second: one instruction stream computes both norms and scales.
__device__ __forceinline__ void tq4_encode_row(float (&v)[8], int lane, uint8_t* row) {
    const int l32 = lane & 31;
    // tables in lanes: entry i in every lane with lane % 16 == i (fetched with ds_bpermute)
    const int tab_b = __float_as_int(kBoundaries[(lane & 15) < 15 ? (lane & 15) : 14]);
    const int tab_c = __float_as_int(kCentroids[lane & 15]);
    sign_wht256(v, lane);

    float p[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) p[j] = v[j] * v[j];
    const float s_sq = row_sum_of_groups(group32_sums(p, lane), lane);
    const float rs = (float)(1.0 / sqrt((double)s_sq));
    const float inv_norm = (s_sq > 1e-20f) ? (0.7071067811865475f * rs) : 0.0f;

    // code = number of boundaries below the value (op_kv_cache.cu:186-189), found by binary
    // search over the sorted boundaries: same count, thresholds fetched by index
    int q[8];
    float c[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float rv = v[j] * inv_norm;
        int code = (rv > kBoundaries[7]) ? 1 : 0;
#pragma unroll
        for (int lvl = 1; lvl < 4; ++lvl) {
            // the bits so far are the top bits of the code; the next threshold is the middle of what is left
            const int idx = (code << (4 - lvl)) + (1 << (3 - lvl)) - 1;
            const float t = __int_as_float(__builtin_amdgcn_ds_bpermute(idx << 2, tab_b));
            code = 2 * code + ((rv > t) ? 1 : 0);
        }
        q[j] = code;
        c[j] = __int_as_float(__builtin_amdgcn_ds_bpermute(code << 2, tab_c));
    }
    // byte m of a 64-byte block holds elements 2m (low nibble) and 2m + 1 (high nibble):
    // elements 8 l32 .. + 7 are bytes 4 (l32 % 16) .. + 3 of block l32 / 16
    uint32_t word = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) word |= (uint32_t)(q[2 * k] | (q[2 * k + 1] << 4)) << (8 * k);
    uint8_t* wdst = row + 66 * (l32 >> 4) + 2 + 4 * (l32 & 15);
    *reinterpret_cast<uint16_t*>(wdst) = (uint16_t)word;
    *reinterpret_cast<uint16_t*>(wdst + 2) = (uint16_t)(word >> 16);

    float pv[8], pc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        pv[j] = v[j] * c[j];
        pc[j] = c[j] * c[j];
    }
    const float vc_dot = row_sum_of_groups(group32_sums(pv, lane), lane);
    const float c_sq = row_sum_of_groups(group32_sums(pc, lane), lane);
    if ((l32 & 15) == 0) {
        const float d = (c_sq > 1e-10f) ? (vc_dot / c_sq) : 0.0f;
        *reinterpret_cast<uint16_t*>(row + 66 * (l32 >> 4)) = F16::from_f32(d);
    }
}

// TQ4 without the rotation (op_kv_cache.cu:219-264): the block quantiser on the raw 128-element
// blocks of the row, v[j] = x[8 l32 + j]; lanes 0-15 hold block 0, lanes 16-31 block 1 (absent at
// head dimension 128: those lanes carry zeros and their bytes are not stored).  The reference sums
// with block_reduce_sum_128 (tq4_kv_common.cuh:109-124): the 32-lane butterfly inside each warp,
// then the same butterfly over the four warp sums in lanes 0-3 of a warp whose other lanes hold
// +0 -- three additions of +0, then (s0 + s2) + (s1 + s3).
__device__ __forceinline__ float block128_sum(const float (&p)[8], int lane) {
    float t = group32_sums(p, lane);  // lanes 4 g .. 4 g + 3: the sum of warp g of the row
    t = ((t + 0.0f) + 0.0f) + 0.0f;   // (a sum that is -0 ends as +0, as in the reference)
    t = t + lane_xor<8>(t, lane);     // s0 + s2 (lanes of warps 0, 2), s1 + s3 (warps 1, 3)
    return t + lane_xor<4>(t, lane);
}

__device__ __forceinline__ void tq4_encode_row_plain(const float (&v)[8], int lane, uint8_t* row) {
    const int l32 = lane & 31;
    const int tab_b = __float_as_int(kBoundaries[(lane & 15) < 15 ? (lane & 15) : 14]);
    const int tab_c = __float_as_int(kCentroids[lane & 15]);
    float p[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) p[j] = v[j] * v[j];
    const float norm_x = __builtin_sqrtf(block128_sum(p, lane));
    const float inv_norm = (norm_x > 1e-12f) ? (0.7071067811865475f / norm_x) : 0.0f;
    int q[8];
    float c[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        // "q = b + 1 for the last boundary b below u" over ascending boundaries = the number of
        // boundaries below u: the binary search of tq4_encode_row
        const float u = v[j] * inv_norm;
        int code = (u > kBoundaries[7]) ? 1 : 0;
#pragma unroll
        for (int lvl = 1; lvl < 4; ++lvl) {
            const int idx = (code << (4 - lvl)) + (1 << (3 - lvl)) - 1;
            const float t = __int_as_float(__builtin_amdgcn_ds_bpermute(idx << 2, tab_b));
            code = 2 * code + ((u > t) ? 1 : 0);
        }
        q[j] = code;
        c[j] = __int_as_float(__builtin_amdgcn_ds_bpermute(code << 2, tab_c));
    }
    uint32_t word = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) word |= (uint32_t)(q[2 * k] | (q[2 * k + 1] << 4)) << (8 * k);
    uint8_t* wdst = row + 66 * (l32 >> 4) + 2 + 4 * (l32 & 15);
    *reinterpret_cast<uint16_t*>(wdst) = (uint16_t)word;
    *reinterpret_cast<uint16_t*>(wdst + 2) = (uint16_t)(word >> 16);
    float pv[8], pc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        pv[j] = v[j] * c[j];
        pc[j] = c[j] * c[j];
    }
    const float xc_dot = block128_sum(pv, lane);
    const float c_sq = block128_sum(pc, lane);
    if ((l32 & 15) == 0) {
        const float d = (c_sq > 1e-12f) ? (xc_dot / c_sq) : 0.0f;
        *reinterpret_cast<uint16_t*>(row + 66 * (l32 >> 4)) = F16::from_f32(d);
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

// Encodes one 256-wide row held as v[j] = x[8 l32 + j] (not yet transformed) in `format` /
// `transform`, assembles it in the half-wave's LDS area `row` (272 bytes, 8-byte aligned) and
// stores it at dst (nothing is stored for dst == nullptr).  16-bit formats are stored directly.
// Rotated 8-bit rows are the un-rotated encoders applied to the transformed row
// (op_kv_cache.cu:36-44,71-99: the same scale and code arithmetic; max is order-free).  The
// caller guarantees what the append entry points check: head_dim 256, TQ4 with WHT256, 8-bit
// rows 4-byte aligned.
__device__ __forceinline__ void encode_store_row(float (&v)[8], int format, int transform, int lane,
                                                 uint8_t* row, uint8_t* dst) {
    const int l32 = lane & 31;
    if (format == WARP34_KV_FORMAT_FP16 || format == WARP34_KV_FORMAT_BF16) {
        if (dst == nullptr) return;
        uint16_t* d16 = reinterpret_cast<uint16_t*>(dst) + 8 * l32;
#pragma unroll
        for (int j = 0; j < 8; ++j) d16[j] = (format == WARP34_KV_FORMAT_BF16) ? BF16::from_f32(v[j]) : F16::from_f32(v[j]);
        return;
    }
    int n_dwords = 33;
    if (format == WARP34_KV_FORMAT_TQ4) {
        if (transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256) {
            tq4_encode_row(v, lane, row);
        } else {
            tq4_encode_row_plain(v, lane, row);
        }
    } else {
        if (transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256) sign_wht256(v, lane);
        if (format == WARP34_KV_FORMAT_FP8_E4M3) {
            fp8_encode_row(v, lane, row);
            n_dwords = 66;
        } else {
            q8_encode_row(v, lane, row);
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

// v[j] = x[l32 + 32 j] (one element per lane and register, as a kernel holds a row whose pairs
// (i, i + 128) it has just rotated) -> v[j] = x[8 l32 + j], through 1 KB of LDS private to the
// half-wave.  Whole-wave call.
__device__ __forceinline__ void strided_to_consecutive(float (&v)[8], int lane, float* xpose) {
    const int l32 = lane & 31;
#pragma unroll
    for (int j = 0; j < 8; ++j) xpose[l32 + 32 * j] = v[j];
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_wave_barrier();
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    const float4 a = *reinterpret_cast<const float4*>(xpose + 8 * l32);
    const float4 b = *reinterpret_cast<const float4*>(xpose + 8 * l32 + 4);
    v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w;
    v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
}

// ---- host-side checks shared by the entry points that write rows ----
inline bool format_supported_for_write(int format, int transform, int head_dim) {
    if (format == WARP34_KV_FORMAT_FP16 || format == WARP34_KV_FORMAT_BF16) {
        return transform == WARP34_KV_TRANSFORM_IDENTITY;
    }
    if (format == WARP34_KV_FORMAT_TQ4) {
        // rotated at head dimension 256 with the WHT-256 transform; every other combination is the
        // plain block quantiser, one block per 128 elements (op_kv_cache.cu:152,219)
        return head_dim == 256 || head_dim == 128;
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
