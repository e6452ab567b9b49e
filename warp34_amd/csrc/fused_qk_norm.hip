// Gemma RMSNorm + interleaved mRoPE + gate split of the target model's full-attention layers for
// gfx950, optionally fused with the append of the finished K row and of the V row into the paged
// KV cache: the producer of the KV path (model/forward.rs:1105-1148 calls the operator and then
// the strided append; fused, rotated K never makes the round trip through HBM).
//
// Replaces fused_qk_rmsnorm_rope_gate_f16_kernel and its two entry points
// (ops/op_norms_rope_act.cu:524-689,1201-1272).  The cache-writing entry point has no
// counterpart in the reference; its result equals operator + warp34_kv_cache_write_strided bit
// for bit (the same row encoders).
//
// Mapping: one workgroup (4 waves) per token.  The last wave computes the token's sine / cosine
// values (they depend on the token's three positions and on the pair index only, not on the
// head) in double precision and leaves them in LDS, fp16-rounded as the reference does, while
// the other waves normalise their first rows.  Every wave takes items in turn, one item per wave, the two 32-lane halves of the wave each
// playing the part of the reference's vector lanes: a Q item is two Q heads, a KV item is one K
// head (lanes 0-31) and, when the cache is written, the V row of the same kv head (lanes 32-63).
// Lane t of a half owns elements 8t .. 8t+7 (one 16-byte load), which is the reference's
// vectorised thread mapping and fixes the order of the sum of squares; the normalised row goes
// through LDS, where the rotation pairs (i, i + rotary / 2) and the row encoders (element
// lane + 32 j) pick their elements.
//
// Numerics (bit-exact contract with the CPU restatement, file built with -ffp-contract=off):
// fp32 in source order; the eight squares of a lane added in order, then the 32-lane xor
// butterfly 16,8,4,2,1; rsqrt, powf, sinf, cosf = the double-precision result rounded once to
// fp32 (theta^(2i/rotary) on the host, it does not depend on the token); fp16 RNE.
#include <cmath>

#include "kv_encode.h"

namespace w34 {

constexpr int kFqMaxPairs = 128;  // rotary_dim / 2

struct FusedQkParams {
    const uint16_t* q_gate_in;
    const uint16_t* k_in;
    const uint16_t* v_in;  // cache write only
    const uint16_t* qw;
    const uint16_t* kw;
    const int32_t* positions;
    const uint8_t* mask;
    uint16_t* q_out;
    uint16_t* k_out;  // may be null when the cache is written
    uint16_t* gate_out;
    const int32_t* write_slot_mapping;  // null: no cache write
    warp34_kv_layer_layout L;
    int num_tokens, pos_plane_stride, q_heads, kv_heads, head_dim, rotary_dim, s1, s2;
    int q_stride, k_stride, v_stride;
    float eps;
    float inv_freq[kFqMaxPairs];
};

__global__ __launch_bounds__(256) void fused_qk_norm_rope_gate_kernel(const FusedQkParams P) {
    __shared__ float s_cos[kFqMaxPairs], s_sin[kFqMaxPairs];
    __shared__ __align__(16) uint16_t s_row[4][2][256];
    __shared__ __align__(8) uint8_t s_enc[4][2][272];
    const int tok = (int)blockIdx.x;
    if (P.mask != nullptr && P.mask[tok] == 0) return;
    const int wave = (int)(threadIdx.x >> 6);
    const int lane = lane_id();
    const int half_id = lane >> 5;
    const int l32 = lane & 31;
    const int hd = P.head_dim, half_rot = P.rotary_dim >> 1;

    // The token's sine / cosine values: the last wave computes them (it has the fewest items),
    // the others go ahead with the first half of their first item and meet it at the barrier
    // in front of the first rotation.
    if (wave == 3) {
        for (int i = lane; i < half_rot; i += 64) {
            int plane = 0;
            if ((i % 3) == 1 && i < P.s1 * 3) {
                plane = 1;
            } else if ((i % 3) == 2 && i < P.s2 * 3) {
                plane = 2;
            }
            const float pos = (float)P.positions[(size_t)plane * P.pos_plane_stride + tok];
            const float angle = pos * P.inv_freq[i];
            s_sin[i] = F16::to_f32(F16::from_f32_of_fp32_result((float)sin((double)angle)));
            s_cos[i] = F16::to_f32(F16::from_f32_of_fp32_result((float)cos((double)angle)));
        }
    }
    bool trig_ready = false;  // wave-uniform: this wave has passed the barrier behind the sine / cosine values

    const bool to_cache_any = P.write_slot_mapping != nullptr;
    const int slot = to_cache_any ? P.write_slot_mapping[tok] : -1;
    const bool to_cache = slot >= 0;  // uniform
    const int q_items = (P.q_heads + 1) >> 1;
    const int n_items = q_items + P.kv_heads;
    uint16_t* row = s_row[wave][half_id];
    const bool owns_vec = 8 * l32 < hd;

    for (int it = wave; it < n_items; it += 4) {  // wave-uniform
        const bool is_q = it < q_items;
        const int kv_head = is_q ? 0 : it - q_items;
        const bool is_v_half = !is_q && half_id == 1;
        int q_head = 2 * it + half_id;
        // Both halves run the same instruction stream (the cross-lane steps want the whole wave):
        // a half without a head of its own (the second half of the last Q item when q_heads is odd,
        // the second half of a KV item when no V row is encoded) works on a row it may read and
        // stores nothing.
        const bool has_head = is_q ? q_head < P.q_heads : (!is_v_half || to_cache);
        if (is_q && q_head >= P.q_heads) q_head = P.q_heads - 1;
        const uint16_t* src;
        const uint16_t* w = is_q ? P.qw : P.kw;
        if (is_q) {
            src = P.q_gate_in + (size_t)tok * P.q_stride + (size_t)q_head * 2 * hd;
        } else if (is_v_half && to_cache) {
            src = P.v_in + (size_t)tok * P.v_stride + (size_t)kv_head * hd;
        } else {
            src = P.k_in + (size_t)tok * P.k_stride + (size_t)kv_head * hd;
        }

        // ---- sum of squares and normalisation: lane t owns elements 8t .. 8t+7 ----
        uint4 raw = {0u, 0u, 0u, 0u};
        uint4 wraw = {0u, 0u, 0u, 0u};
        if (owns_vec) {
            raw = *reinterpret_cast<const uint4*>(src + 8 * l32);
            wraw = *reinterpret_cast<const uint4*>(w + 8 * l32);
        }
        // (halves taken out and put together with shifts: indexing the vectors through a pointer
        // would move them to scratch memory)
        const uint32_t rw[4] = {raw.x, raw.y, raw.z, raw.w};
        const uint32_t ww[4] = {wraw.x, wraw.y, wraw.z, wraw.w};
        float x[8];
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            x[j] = F16::to_f32((uint16_t)(rw[j >> 1] >> (16 * (j & 1))));
            const float sq = x[j] * x[j];
            acc = acc + sq;
        }
        const float sum_sq = half_wave_sum(acc, lane);
        const float mean = sum_sq / (float)hd + P.eps;
        const float inv_rms = (float)(1.0 / sqrt((double)mean));
        uint32_t nw[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            uint32_t packed = 0u;
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int j = 2 * k + hh;
                const float v = x[j] * inv_rms;
                const float wt = 1.0f + F16::to_f32((uint16_t)(ww[k] >> (16 * hh)));
                packed |= (uint32_t)F16::from_f32_of_fp32_result(v * wt) << (16 * hh);
            }
            nw[k] = is_v_half ? rw[k] : packed;  // the V half keeps its row as it is
        }
        if (owns_vec) *reinterpret_cast<uint4*>(row + 8 * l32) = uint4{nw[0], nw[1], nw[2], nw[3]};
        if (!trig_ready) {  // (also orders the row buffer: a workgroup barrier includes the wave's own)
            __syncthreads();
            trig_ready = true;
        } else {
            __atomic_signal_fence(__ATOMIC_SEQ_CST);
            __builtin_amdgcn_wave_barrier();
            __atomic_signal_fence(__ATOMIC_SEQ_CST);
        }

        // ---- rotation of the pairs (i, i + rotary / 2), in place ----
        if (!is_v_half) {
            for (int i = l32; i < half_rot; i += 32) {
                const float x1 = F16::to_f32(row[i]), x2 = F16::to_f32(row[i + half_rot]);
                const float c = s_cos[i], s = s_sin[i];
                const float a = x1 * c, b = x2 * s, cc = x2 * c, d = x1 * s;
                row[i] = F16::from_f32_of_fp32_result(a - b);
                row[i + half_rot] = F16::from_f32_of_fp32_result(cc + d);
            }
        }
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        __builtin_amdgcn_wave_barrier();
        __atomic_signal_fence(__ATOMIC_SEQ_CST);

        // ---- outputs ----
        if (is_q) {
            if (has_head && owns_vec) {
                *reinterpret_cast<uint4*>(P.q_out + ((size_t)tok * P.q_heads + q_head) * hd + 8 * l32) =
                    *reinterpret_cast<const uint4*>(row + 8 * l32);
                *reinterpret_cast<uint4*>(P.gate_out + ((size_t)tok * P.q_heads + q_head) * hd + 8 * l32) =
                    *reinterpret_cast<const uint4*>(src + hd + 8 * l32);
            }
        } else {
            if (!is_v_half && P.k_out != nullptr && owns_vec) {
                *reinterpret_cast<uint4*>(P.k_out + ((size_t)tok * P.kv_heads + kv_head) * hd + 8 * l32) =
                    *reinterpret_cast<const uint4*>(row + 8 * l32);
            }
            if (to_cache) {
                const int page = slot / P.L.block_size, off = slot - page * P.L.block_size;
                uint8_t* dst = reinterpret_cast<uint8_t*>((uintptr_t)(is_v_half ? P.L.v_base : P.L.k_base)) +
                               (size_t)page * (is_v_half ? P.L.v_page_stride_bytes : P.L.k_page_stride_bytes) +
                               (size_t)kv_head * (is_v_half ? P.L.v_head_stride_bytes : P.L.k_head_stride_bytes) +
                               (size_t)off * (is_v_half ? P.L.v_token_stride_bytes : P.L.k_token_stride_bytes);
                // elements 8 l32 .. 8 l32 + 7 of the finished row (head_dim 256, host check)
                float v[8];
                {
                    const uint4 r8 = *reinterpret_cast<const uint4*>(row + 8 * l32);
                    const uint32_t w[4] = {r8.x, r8.y, r8.z, r8.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        v[2 * j] = F16::to_f32((uint16_t)(w[j] & 0xffffu));
                        v[2 * j + 1] = F16::to_f32((uint16_t)(w[j] >> 16));
                    }
                }
                encode_store_row(v, is_v_half ? P.L.v_format : P.L.k_format, is_v_half ? P.L.v_transform : P.L.k_transform,
                                 lane, s_enc[wave][half_id], dst);
            }
        }
        // the next item of this wave overwrites the row buffer
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        __builtin_amdgcn_wave_barrier();
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
    }
    if (!trig_ready) __syncthreads();  // a wave without items: every wave of the workgroup meets the barrier once
}

static int launch_fused_qk(const warp34_exec* ex, const void* q_gate_in, const void* k_in, const void* v_in,
                           const void* q_norm_w, const void* k_norm_w, const int32_t* positions,
                           const uint8_t* valid_token_mask, void* q_out, void* k_out, void* gate_out,
                           const warp34_kv_layer_layout* layout, const int32_t* write_slot_mapping, int num_tokens,
                           int pos_plane_stride, int num_q_heads, int num_kv_heads, int head_dim, int rotary_dim,
                           int mrope_s1, int mrope_s2, int q_gate_row_stride, int k_row_stride, int v_row_stride,
                           float rope_theta, float rms_eps) {
    // what this kernel's lane mapping covers: one 16-byte vector per lane of a 32-lane half
    if (head_dim <= 0 || (head_dim & 7) != 0 || head_dim > 256 || rotary_dim < 0 || (rotary_dim & 1) != 0 ||
        rotary_dim > head_dim || rotary_dim / 2 > kFqMaxPairs || num_q_heads < 0 || num_kv_heads < 0 ||
        ((q_gate_row_stride | k_row_stride | v_row_stride) & 7) != 0 ||
        (((uintptr_t)q_gate_in | (uintptr_t)k_in | (uintptr_t)v_in | (uintptr_t)q_norm_w | (uintptr_t)k_norm_w |
          (uintptr_t)q_out | (uintptr_t)k_out | (uintptr_t)gate_out) & 15u) != 0) {
        return (int)hipErrorNotSupported;
    }
    FusedQkParams P{};
    P.q_gate_in = (const uint16_t*)q_gate_in;
    P.k_in = (const uint16_t*)k_in;
    P.v_in = (const uint16_t*)v_in;
    P.qw = (const uint16_t*)q_norm_w;
    P.kw = (const uint16_t*)k_norm_w;
    P.positions = positions;
    P.mask = valid_token_mask;
    P.q_out = (uint16_t*)q_out;
    P.k_out = (uint16_t*)k_out;
    P.gate_out = (uint16_t*)gate_out;
    P.write_slot_mapping = write_slot_mapping;
    if (layout != nullptr) P.L = *layout;
    P.num_tokens = num_tokens;
    P.pos_plane_stride = pos_plane_stride;
    P.q_heads = num_q_heads;
    P.kv_heads = num_kv_heads;
    P.head_dim = head_dim;
    P.rotary_dim = rotary_dim;
    P.s1 = mrope_s1;
    P.s2 = mrope_s2;
    P.q_stride = q_gate_row_stride;
    P.k_stride = k_row_stride;
    P.v_stride = v_row_stride;
    P.eps = rms_eps;
    for (int i = 0; i < rotary_dim / 2; ++i) {
        const float expo = (float)(2 * i) / (float)rotary_dim;
        const float pw = (float)std::pow((double)rope_theta, (double)expo);
        P.inv_freq[i] = 1.0f / pw;
    }
    hipLaunchKernelGGL(fused_qk_norm_rope_gate_kernel, dim3((unsigned)num_tokens), dim3(256), 0,
                       (hipStream_t)ex->stream, P);
    return (int)hipGetLastError();
}

}  // namespace w34

using namespace w34;

// ops/op_norms_rope_act.cu:1201-1246
extern "C" int warp34_fused_qk_rmsnorm_rope_gate_strided_f16(
    const warp34_exec* ex, const void* q_gate_in, const void* k_in, const void* q_norm_w, const void* k_norm_w,
    const int32_t* positions, const uint8_t* valid_token_mask, void* q_out, void* k_out, void* gate_out,
    int num_tokens, int pos_plane_stride, int num_q_heads, int num_kv_heads, int head_dim, int rotary_dim,
    int mrope_s0, int mrope_s1, int mrope_s2, int q_gate_row_stride, int k_row_stride, float rope_theta,
    float rms_eps) {
    (void)mrope_s0;
    if (ex == nullptr || q_gate_in == nullptr || k_in == nullptr || q_norm_w == nullptr || k_norm_w == nullptr ||
        positions == nullptr || q_out == nullptr || k_out == nullptr || gate_out == nullptr) {
        return (int)hipErrorInvalidValue;
    }
    if (num_tokens <= 0) return 0;
    if (q_gate_row_stride < num_q_heads * 2 * head_dim || k_row_stride < num_kv_heads * head_dim) {
        return (int)hipErrorInvalidValue;
    }
    return launch_fused_qk(ex, q_gate_in, k_in, nullptr, q_norm_w, k_norm_w, positions, valid_token_mask, q_out, k_out,
                           gate_out, nullptr, nullptr, num_tokens, pos_plane_stride, num_q_heads, num_kv_heads,
                           head_dim, rotary_dim, mrope_s1, mrope_s2, q_gate_row_stride, k_row_stride, 0, rope_theta,
                           rms_eps);
}

// ops/op_norms_rope_act.cu:1248-1272
extern "C" int warp34_fused_qk_rmsnorm_rope_gate_f16(
    const warp34_exec* ex, const void* q_gate_in, const void* k_in, const void* q_norm_w, const void* k_norm_w,
    const int32_t* positions, const uint8_t* valid_token_mask, void* q_out, void* k_out, void* gate_out,
    int num_tokens, int pos_plane_stride, int num_q_heads, int num_kv_heads, int head_dim, int rotary_dim,
    int mrope_s0, int mrope_s1, int mrope_s2, float rope_theta, float rms_eps) {
    return warp34_fused_qk_rmsnorm_rope_gate_strided_f16(
        ex, q_gate_in, k_in, q_norm_w, k_norm_w, positions, valid_token_mask, q_out, k_out, gate_out, num_tokens,
        pos_plane_stride, num_q_heads, num_kv_heads, head_dim, rotary_dim, mrope_s0, mrope_s1, mrope_s2,
        num_q_heads * 2 * head_dim, num_kv_heads * head_dim, rope_theta, rms_eps);
}

// The operator fused with the append (no counterpart in the reference): the finished K rows and
// the V rows of v_in ([tokens, v_row_stride], fp16) go to the pages of kv_layout at
// write_slot_mapping[token] (negative slot: no cache write for that token), in the layout's
// formats; k_out may be null.  Equal to the operator followed by
// warp34_kv_cache_write_strided(k_out, v_in) for the same tokens, bit for bit.
extern "C" int warp34_fused_qk_rmsnorm_rope_gate_kv_write_f16(
    const warp34_exec* ex, const void* q_gate_in, const void* k_in, const void* v_in, const void* q_norm_w,
    const void* k_norm_w, const int32_t* positions, const uint8_t* valid_token_mask, void* q_out, void* k_out,
    void* gate_out, const warp34_kv_layer_layout* kv_layout, const int32_t* write_slot_mapping, int num_tokens,
    int pos_plane_stride, int num_q_heads, int num_kv_heads, int head_dim, int rotary_dim, int mrope_s0,
    int mrope_s1, int mrope_s2, int q_gate_row_stride, int k_row_stride, int v_row_stride, float rope_theta,
    float rms_eps) {
    (void)mrope_s0;
    if (ex == nullptr || q_gate_in == nullptr || k_in == nullptr || v_in == nullptr || q_norm_w == nullptr ||
        k_norm_w == nullptr || positions == nullptr || q_out == nullptr || gate_out == nullptr ||
        kv_layout == nullptr || write_slot_mapping == nullptr || kv_layout->k_base == 0 || kv_layout->v_base == 0 ||
        kv_layout->block_size <= 0 || kv_layout->local_kv_heads != num_kv_heads || kv_layout->head_dim != head_dim) {
        return (int)hipErrorInvalidValue;
    }
    if (num_tokens <= 0) return 0;
    if (q_gate_row_stride < num_q_heads * 2 * head_dim || k_row_stride < num_kv_heads * head_dim ||
        v_row_stride < num_kv_heads * head_dim) {
        return (int)hipErrorInvalidValue;
    }
    // the row encoders take 256-element rows, lane + 32 j; both halves of a wave go through them
    // together, so K and V share format and transform
    if (head_dim != 256 || kv_layout->k_format != kv_layout->v_format ||
        kv_layout->k_transform != kv_layout->v_transform || !format_supported_for_write(kv_layout->k_format, kv_layout->k_transform, head_dim) ||
        !format_supported_for_write(kv_layout->v_format, kv_layout->v_transform, head_dim) ||
        !rows_aligned_for_write(kv_layout)) {
        return (int)hipErrorNotSupported;
    }
    return launch_fused_qk(ex, q_gate_in, k_in, v_in, q_norm_w, k_norm_w, positions, valid_token_mask, q_out, k_out,
                           gate_out, kv_layout, write_slot_mapping, num_tokens, pos_plane_stride, num_q_heads,
                           num_kv_heads, head_dim, rotary_dim, mrope_s1, mrope_s2, q_gate_row_stride, k_row_stride,
                           v_row_stride, rope_theta, rms_eps);
}
