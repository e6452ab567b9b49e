// Shared definitions for the gfx950 KV-cache kernels: TQ4 tables, 16-bit conversions,
// wave64 cross-lane helpers and the request / key-range lookup every kernel uses.
#pragma once

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/warp34_kv.h"

namespace w34 {

// ---- TQ4 codebook (reference literals: csrc/tq/tq4_codebook.cuh:46-101) -----------------
// Lloyd-Max centroids of the Beta(256) unit-sphere coordinate density and the midpoints
// between them.  Kept as constexpr so device code folds them into immediates.
__device__ __constant__ constexpr float kCentroids[16] = {
    -1.694104124e-1f, -1.285881878e-1f, -1.006979993e-1f, -7.824930800e-2f,
    -5.873210384e-2f, -4.094919437e-2f, -2.420087619e-2f, -8.008373692e-3f,
    8.008373692e-3f,  2.420087619e-2f,  4.094919437e-2f,  5.873210384e-2f,
    7.824930800e-2f,  1.006979993e-1f,  1.285881878e-1f,  1.694104124e-1f,
};
__device__ __constant__ constexpr float kBoundaries[15] = {
    -1.489993001e-1f, -1.146430936e-1f, -8.947365365e-2f, -6.849070592e-2f,
    -4.984064910e-2f, -3.257503528e-2f, -1.610462494e-2f, 0.000000000e0f,
    1.610462494e-2f,  3.257503528e-2f,  4.984064910e-2f,  6.849070592e-2f,
    8.947365365e-2f,  1.146430936e-1f,  1.489993001e-1f,
};
// Seed-42 Rademacher diagonal as a bit mask: bit i of word i/32 set <=> sign[i] = -1.
__device__ __constant__ constexpr uint32_t kSignMask[8] = {
    0x29e1d357u, 0x48974752u, 0xeebc0de4u, 0xf1297e2au,
    0xba639274u, 0xe2eb25d0u, 0xfde0ee14u, 0x36b5bda1u,
};

// Word w (0..7) of the mask for an index that differs between lanes, picked from the eight
// immediates with three levels of selects.  A lookup in the constant array would be a vector
// memory load: a round trip on the spot, and a wait that also waits for every load issued before it.
__device__ __forceinline__ uint32_t sign_word(int w) {
    const uint32_t a = (w & 1) ? 0x48974752u : 0x29e1d357u;
    const uint32_t b = (w & 1) ? 0xf1297e2au : 0xeebc0de4u;
    const uint32_t c = (w & 1) ? 0xe2eb25d0u : 0xba639274u;
    const uint32_t d = (w & 1) ? 0x36b5bda1u : 0xfde0ee14u;
    const uint32_t ab = (w & 2) ? b : a;
    const uint32_t cd = (w & 2) ? d : c;
    return (w & 4) ? cd : ab;
}
static_assert(kSignMask[0] == 0x29e1d357u && kSignMask[1] == 0x48974752u && kSignMask[2] == 0xeebc0de4u &&
                  kSignMask[3] == 0xf1297e2au && kSignMask[4] == 0xba639274u && kSignMask[5] == 0xe2eb25d0u &&
                  kSignMask[6] == 0xfde0ee14u && kSignMask[7] == 0x36b5bda1u,
              "sign_word() repeats the mask");
__device__ __forceinline__ bool sign_is_negative(int i) {
    return (sign_word(i >> 5) >> (i & 31)) & 1u;
}
// multiply by the +-1 sign of element i (exact: flips the sign bit)
__device__ __forceinline__ float apply_sign(float v, int i) {
    return __uint_as_float(__float_as_uint(v) ^ (((sign_word(i >> 5) >> (i & 31)) & 1u) << 31));
}

constexpr int kHeadDim = 256;
constexpr int kTq4RowBytes = 132;   // 2 x (fp16 scale + 64 bytes of nibbles), tq4_kv_common.cuh:21-26
constexpr int kTq4RowDwords = 33;

// ---- 16-bit element types ----------------------------------------------------------------
struct F16 {
    static constexpr int kStorageFormat = WARP34_KV_FORMAT_FP16;
    __device__ static __forceinline__ float to_f32(uint16_t b) {
        return __half2float(__ushort_as_half(b));
    }
    __device__ static __forceinline__ uint16_t from_f32(float f) {
        return __half_as_ushort(__float2half_rn(f));
    }
    // The same conversion for results whose bits are part of a contract: the value passes through
    // an empty asm statement, so the compiler cannot fold the fp32 operation that produced it and
    // the conversion into one mixed-precision FMA (which rounds once where the reference rounds
    // twice, to fp32 and then to fp16).
    __device__ static __forceinline__ uint16_t from_f32_of_fp32_result(float f) {
        asm("" : "+v"(f));
        return __half_as_ushort(__float2half_rn(f));
    }
};
struct BF16 {
    static constexpr int kStorageFormat = WARP34_KV_FORMAT_BF16;
    __device__ static __forceinline__ float to_f32(uint16_t b) {
        return __uint_as_float((uint32_t)b << 16);
    }
    // round to nearest even: gfx950 converts in hardware (v_cvt_pk_bf16_f32); a NaN comes out
    // as a quiet NaN whose payload is the hardware's choice
    __device__ static __forceinline__ uint16_t from_f32(float f) {
        return __builtin_bit_cast(uint16_t, (__bf16)f);
    }
};

// attn * sigmoid(gate) as the gate operator computes it (ops/op_norms_rope_act.cu:742-759): an
// fp32 product, which the caller then rounds to 16 bits.  The empty asm statement keeps the
// compiler from folding the multiply and that conversion into one mixed-precision FMA, which
// rounds once instead of twice and turns a product of -0 into +0.
__device__ __forceinline__ float gate_product(float attn, float gate) {
#pragma clang fp contract(off)
    const float sig = 1.0f / (1.0f + expf(-gate));
    float r = attn * sig;
    asm volatile("" : "+v"(r));
    return r;
}

// ---- request / visible-key-range lookup (op_kv_cache.cu:385-424) ------------------------
struct RowRange {
    int req;     // owning request, -1 when the row is skipped
    int min_kv;  // first visible key
    int max_kv;  // last visible key (may be < min_kv: empty)
};

__device__ __forceinline__ int find_request(const warp34_attention_batch& b, int tok, int& q_start,
                                            int& q_end) {
    for (int r = 0; r < b.num_reqs; ++r) {
        const int lo = b.query_start_loc[r];
        const int hi = b.query_start_loc[r + 1];
        if (tok >= lo && tok < hi) {
            q_start = lo;
            q_end = hi;
            return r;
        }
    }
    return -1;
}

__device__ __forceinline__ RowRange row_range(const warp34_attention_batch& b, int tok) {
    RowRange rr{-1, 0, -1};
    if (tok < 0 || tok >= b.total_tokens) return rr;
    if (b.valid_token_mask != nullptr && b.valid_token_mask[tok] == 0) return rr;
    int q_start = 0, q_end = 0;
    const int r = find_request(b, tok, q_start, q_end);
    if (r < 0) return rr;
    if (b.valid_req_mask != nullptr && b.valid_req_mask[r] == 0) return rr;
    const int q_off = tok - q_start;
    const int seq_after = b.seq_lens_after[r];
    const int ctx_before =
        b.context_lens_before != nullptr ? b.context_lens_before[r] : seq_after - (q_end - q_start);
    int mx = (b.mask_mode == WARP34_ATTN_MASK_NONCAUSAL_WINDOW) ? seq_after - 1 : ctx_before + q_off;
    if (mx >= seq_after) mx = seq_after - 1;
    int mn = 0;
    if (b.sliding_window > 0) {
        const int ws = ctx_before + q_off - b.sliding_window + 1;
        if (ws > mn) mn = ws;
    }
    rr.req = r;
    rr.min_kv = mn;
    rr.max_kv = mx;
    return rr;
}

// ---- wave64 helpers ------------------------------------------------------------------------
__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63u); }

template <int MASK>
__device__ __forceinline__ float xor_lane(float v) {
    return __shfl_xor(v, MASK, 64);
}

// value of lane (lane ^ H) for every lane of a wave, built from DPP / lane-swap VALU ops
// (no LDS round trip): quad permutes for 1 and 2, row shifts for 4, a row rotate for 8 and
// the gfx950 row / half swaps for 16 and 32.
template <int H>
__device__ __forceinline__ float lane_xor(float x, int lane) {
    const int xi = __float_as_int(x);
    if constexpr (H == 1) {
        return __int_as_float(__builtin_amdgcn_mov_dpp(xi, 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
    } else if constexpr (H == 2) {
        return __int_as_float(__builtin_amdgcn_mov_dpp(xi, 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
    } else if constexpr (H == 4) {
        // banks 0,2 (lanes 0-3, 8-11 of a row) take lane+4, banks 1,3 take lane-4
        int r = __builtin_amdgcn_update_dpp(0, xi, 0x104, 0xF, 0x5, false);  // row_shl:4
        r = __builtin_amdgcn_update_dpp(r, xi, 0x114, 0xF, 0xA, false);      // row_shr:4
        return __int_as_float(r);
    } else if constexpr (H == 8) {
        return __int_as_float(__builtin_amdgcn_mov_dpp(xi, 0x128, 0xF, 0xF, true));  // row_ror:8
    } else if constexpr (H == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap((uint32_t)xi, (uint32_t)xi, false, false);
        return __uint_as_float((lane & 16) ? r[0] : r[1]);
    } else {
        const auto r = __builtin_amdgcn_permlane32_swap((uint32_t)xi, (uint32_t)xi, false, false);
        return __uint_as_float((lane & 32) ? r[0] : r[1]);
    }
}


}  // namespace w34
