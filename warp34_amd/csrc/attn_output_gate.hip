// Output gate on the attention result for gfx950: out = attn_out * sigmoid(gate), the consumer of
// the paged-attention output in the gated full-attention layers (model/forward.rs:1192-1211).
// Replaces apply_attn_output_gate_f16_kernel and its entry point
// (ops/op_norms_rope_act.cu:742-759,1329-1344).  Pure streaming: 3 x 2 bytes per element.
#include "kv_common.h"

namespace w34 {

// One thread handles 8 consecutive fp16 elements (16-byte accesses) when the row length and the
// three base pointers allow it, single elements otherwise.
template <bool VEC8>
__global__ __launch_bounds__(256) void attn_output_gate_kernel(const uint16_t* __restrict__ attn_out,
                                                               const uint16_t* __restrict__ gate,
                                                               uint16_t* __restrict__ out,
                                                               const uint8_t* __restrict__ valid_token_mask,
                                                               int total_dim) {
    const int tok = (int)blockIdx.x;
    if (valid_token_mask != nullptr && valid_token_mask[tok] == 0) return;  // row untouched
    constexpr int kPer = VEC8 ? 8 : 1;
    const int col = ((int)blockIdx.y * 256 + (int)threadIdx.x) * kPer;
    if (col >= total_dim) return;
    const size_t idx = (size_t)tok * total_dim + col;
    if constexpr (VEC8) {
        const uint4 av = *reinterpret_cast<const uint4*>(attn_out + idx);
        const uint4 gv = *reinterpret_cast<const uint4*>(gate + idx);
        const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, gw[4] = {gv.x, gv.y, gv.z, gv.w};
        uint32_t ow[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float r[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const float a = F16::to_f32((uint16_t)(aw[k] >> (16 * h)));
                const float g = F16::to_f32((uint16_t)(gw[k] >> (16 * h)));
                r[h] = gate_product(a, g);
            }
            ow[k] = (uint32_t)F16::from_f32(r[0]) | ((uint32_t)F16::from_f32(r[1]) << 16);
        }
        *reinterpret_cast<uint4*>(out + idx) = uint4{ow[0], ow[1], ow[2], ow[3]};
    } else {
        const float a = F16::to_f32(attn_out[idx]);
        const float g = F16::to_f32(gate[idx]);
        out[idx] = F16::from_f32(gate_product(a, g));
    }
}

}  // namespace w34

using namespace w34;

// op_norms_rope_act.cu:1329-1344
extern "C" int warp34_apply_attn_output_gate_f16(const warp34_exec* ex, const void* attn_out, const void* gate,
                                                 void* out, const uint8_t* valid_token_mask, int num_tokens,
                                                 int total_dim) {
    if (ex == nullptr || attn_out == nullptr || gate == nullptr || out == nullptr) return (int)hipErrorInvalidValue;
    if (num_tokens <= 0 || total_dim <= 0) return 0;
    const bool vec8 = (total_dim % 8) == 0 &&
                      ((((uintptr_t)attn_out) | ((uintptr_t)gate) | ((uintptr_t)out)) & 15u) == 0;
    const int per_block = 256 * (vec8 ? 8 : 1);
    const unsigned col_blocks = (unsigned)((total_dim + per_block - 1) / per_block);
    if (col_blocks > 65535u) return (int)hipErrorInvalidValue;
    const dim3 grid((unsigned)num_tokens, col_blocks);
    hipStream_t stream = (hipStream_t)ex->stream;
    if (vec8) {
        hipLaunchKernelGGL((attn_output_gate_kernel<true>), grid, dim3(256), 0, stream, (const uint16_t*)attn_out,
                           (const uint16_t*)gate, (uint16_t*)out, valid_token_mask, total_dim);
    } else {
        hipLaunchKernelGGL((attn_output_gate_kernel<false>), grid, dim3(256), 0, stream, (const uint16_t*)attn_out,
                           (const uint16_t*)gate, (uint16_t*)out, valid_token_mask, total_dim);
    }
    return (int)hipGetLastError();
}
