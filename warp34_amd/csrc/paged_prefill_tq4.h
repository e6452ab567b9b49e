// Chunked-prefill attention over TQ4 pages for gfx950: many query rows per workgroup, every
// K/V unit dequantised ONCE per workgroup and shared by all waves through LDS.
// Replaces paged_attention_prefill_mma_f16_kernel + launch_prefill
// (op_paged_attn.cu:594-1128,1220-1259).  Included by paged_attn.hip.
//
// Workgroup = 8 waves = one tile of 128 query rows (128 / q_group consecutive tokens of ONE
// request x q_group heads of one kv head); wave w owns rows 16 w .. 16 w + 15 as the 16 columns
// of its MFMA results (S^T = K Q'^T, O^T += V^T P^T, as in the decode kernel, so the softmax
// state is one scalar pair per lane).  The workgroup walks the request's keys in 32-token
// units with a three-stage software pipeline and ONE barrier per unit:
//   load   : unit u+3, 16-byte pieces of the raw K / V rows, global -> registers
//   commit : unit u+2, registers -> raw LDS buffer
//   dequant: unit u+1, raw LDS -> fp16 centroids through the pair table, written in the
//            layouts the MFMAs read: K as [token][256] rows (528-byte stride), V transposed as
//            [dim][32 key slots] with the 16-byte pieces XOR-swizzled, scales as fp32
//   compute: unit u, 16 QK + 16 PV MFMAs per wave, operands read with 128-bit LDS loads
// Scales are not applied per element: K scales multiply the two half-row partial scores,
// V scales are folded into the probabilities, exactly as in the decode kernel.
#pragma once

namespace w34 {

constexpr int kPfWaves = 8;
constexpr int kPfRows = 128;                                  // query rows per workgroup
constexpr int kPfKStride = 528;                               // bytes per dequantised K row
constexpr int kPfKBytes = 32 * kPfKStride;                    // 16896
constexpr int kPfVBytes = 256 * 64;                           // V^T: 256 rows x 32 halves
constexpr int kPfScaleBytes = 4 * 32 * 4;                     // K d0, K d1, V d0, V d1 per token
constexpr int kPfDeqBytes = kPfKBytes + kPfVBytes + kPfScaleBytes;
constexpr int kPfRawBytes = kStageTq4;                        // 64 raw rows of 132 B
constexpr int kPfDeqBase = kLutBytes;
constexpr int kPfRawBase = kPfDeqBase + 2 * kPfDeqBytes;
constexpr int kPfDummy = kPfRawBase + 2 * kPfRawBytes;        // 256 B that absorb the writes of scale bytes
constexpr int kPfSmem = kPfDummy + 256;
static_assert(kPfSmem <= 160 * 1024, "prefill LDS budget");
static_assert(kPfWaves * 16 * 260 * 4 <= kPfSmem, "epilogue regions must fit");
static_assert(kPfWaves * 16 * 264 * 2 <= 2 * kPfDeqBytes, "query staging must fit in the dequant buffers");

typedef __attribute__((address_space(3))) uint32_t lds_u32;

template <typename TQ>
__global__ __launch_bounds__(kPfWaves * 64, 1) void paged_prefill_tq4_kernel(const AttnParams P) {
    extern __shared__ __align__(16) uint8_t smem[];
    if ((uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem != 0u) __builtin_trap();

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int b = lane >> 4;
    const warp34_kv_layer_layout& L = P.L;
    const warp34_attention_batch& B = P.B;

    // ---- tile identification: blockIdx = (tile of the request, kv head x q subgroup, request) ----
    const int req = (int)blockIdx.z;
    const int kv_sub = (int)blockIdx.y;
    const int kv_head = fast_div(kv_sub, P.q_subgroups);
    const int q_head_base = kv_head * P.gqa + (kv_sub - kv_head * P.q_subgroups) * P.q_group;
    if (B.valid_req_mask != nullptr && B.valid_req_mask[req] == 0) return;
    const int rq_start = B.query_start_loc[req];
    const int rq_end = B.query_start_loc[req + 1];
    const int seq_after = B.seq_lens_after[req];
    const int ctx_before = B.context_lens_before != nullptr ? B.context_lens_before[req]
                                                            : seq_after - (rq_end - rq_start);
    const int tile_tok = P.tok_tile;  // 128 / q_group
    const int tok0 = rq_start + (int)blockIdx.x * tile_tok;
    if (tok0 >= rq_end || tok0 >= B.total_tokens) return;
    int tile_tokens = rq_end - tok0;
    if (tile_tokens > tile_tok) tile_tokens = tile_tok;
    if (tile_tokens > B.total_tokens - tok0) tile_tokens = B.total_tokens - tok0;

    // ---- the pair table (64 lane replicas, as in the decode kernel) ----
    {
        const int e = tid >> 1;
        const uint32_t v = pack_h2(kLutGain * centroid_of_code(e & 15), kLutGain * centroid_of_code(e >> 4));
        u4 vv = {v, v, v, v};
        u4* dst = reinterpret_cast<u4*>(smem + e * 256 + (tid & 1) * 128);
#pragma unroll
        for (int k = 0; k < 8; ++k) dst[k] = vv;
    }

    // ---- key range of every column; workgroup-wide unit range ----
    const int q_off0 = tok0 - rq_start;
    auto range_hi = [&](int q_off) {
        int mx = (B.mask_mode == WARP34_ATTN_MASK_NONCAUSAL_WINDOW) ? seq_after - 1 : ctx_before + q_off;
        return mx >= seq_after ? seq_after - 1 : mx;
    };
    auto range_lo = [&](int q_off) {
        return B.sliding_window > 0 ? max(0, ctx_before + q_off - B.sliding_window + 1) : 0;
    };
    const int lo_all = range_lo(q_off0);
    const int hi_all = range_hi(q_off0 + tile_tokens - 1);
    const int u_first = lo_all >> 5;
    const int n_units = hi_all >= lo_all ? (hi_all >> 5) - u_first + 1 : 0;

    const int my_col = 16 * wave + n;
    const int my_t = fast_div(my_col, P.q_group);
    const int my_tok = tok0 + my_t;
    const bool col_ok = my_t < tile_tokens &&
                        (B.valid_token_mask == nullptr || B.valid_token_mask[min(my_tok, B.total_tokens - 1)] != 0);
    const int col_lo = col_ok ? range_lo(q_off0 + my_t) : 0;
    const int col_hi = col_ok ? range_hi(q_off0 + my_t) : -1;
    const uint32_t ok_mask = (uint32_t)(__ballot(col_ok) & 0xFFFFull);
    int i_lo = col_ok ? col_lo : 0, i_hi = col_ok ? col_hi : 0x7fffffff;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        i_lo = max(i_lo, __shfl_xor(i_lo, off, 64));
        i_hi = min(i_hi, __shfl_xor(i_hi, off, 64));
    }
    i_lo = __builtin_amdgcn_readfirstlane(i_lo);
    i_hi = __builtin_amdgcn_readfirstlane(i_hi);

    // ---- rotated, scaled queries of this wave's 16 columns -> LDS -> MFMA B operands ----
    constexpr int kQStride = 264;
    _Float16* qbuf = reinterpret_cast<_Float16*>(smem + kPfDeqBase) + wave * 16 * kQStride;
    const float q_scale = B.sm_scale * kLog2e * kLutInvGain;
    {
        uint2 q_raw[16];
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const int col = 16 * wave + c;
            const int t = fast_div(col, P.q_group);
            const int a = col - t * P.q_group;
            const int tok = min(tok0 + t, B.total_tokens - 1);
            const uint16_t* qrow = P.q + ((size_t)tok * P.num_q_heads + (size_t)(q_head_base + a)) * kHeadDim;
            q_raw[c] = *reinterpret_cast<const uint2*>(qrow + 4 * lane);
        }
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            float v[4];
            v[0] = TQ::to_f32((uint16_t)(q_raw[c].x & 0xFFFFu));
            v[1] = TQ::to_f32((uint16_t)(q_raw[c].x >> 16));
            v[2] = TQ::to_f32((uint16_t)(q_raw[c].y & 0xFFFFu));
            v[3] = TQ::to_f32((uint16_t)(q_raw[c].y >> 16));
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = apply_sign(v[k], 4 * lane + k);
            wht256_wave(v, lane);
            uint2 packed = {0u, 0u};  // dead columns: zero query
            if ((ok_mask >> c) & 1u) {
                packed.x = pack_h2(v[0] * q_scale, v[1] * q_scale);
                packed.y = pack_h2(v[2] * q_scale, v[3] * q_scale);
            }
            *reinterpret_cast<uint2*>(qbuf + c * kQStride + 4 * lane) = packed;
        }
    }
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_wave_barrier();
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    h8 bq[2][4];  // [half of the head dim][32-wide k step]: Q'[col n][128 h + 32 m + 8 b ..]
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int m = 0; m < 4; ++m)
            bq[h][m] = *reinterpret_cast<const h8*>(qbuf + n * kQStride + 128 * h + 32 * m + 8 * b);

    // ---- loader: this thread's 16-byte piece(s) of a raw unit ----
    // A unit is four runs of 16 rows (2112 B = 132 pieces): K rows 0-15, K rows 16-31, V rows
    // 0-15, V rows 16-31; piece i of the unit is piece i % 132 of run i / 132.  Threads 0-15
    // also carry pieces 512-527.
    const uint8_t* k_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.k_base) +
                            (size_t)kv_head * L.k_head_stride_bytes;
    const uint8_t* v_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.v_base) +
                            (size_t)kv_head * L.v_head_stride_bytes;
    const int32_t* req_blocks = B.block_tables + (size_t)req * B.max_blocks_per_req;
    int ld_run[2], ld_pc[2];
    ld_run[0] = tid >= 396 ? 3 : tid >= 264 ? 2 : tid >= 132 ? 1 : 0;
    ld_pc[0] = tid - 132 * ld_run[0];
    ld_run[1] = 3;
    ld_pc[1] = 116 + tid;  // only for tid < 16
    const bool two = tid < 16;
    int32_t pg_cur[2] = {-1, -1};
    u4 pf[2];
    // page ids of unit k (relative to u_first) for this thread's runs
    auto load_pages = [&](int k, int32_t (&pg)[2]) {
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            pg[x] = -1;
            if (x == 1 && !two) continue;
            const int pos = (u_first + k) * kUnit + 16 * (ld_run[x] & 1);
            const int slot = fast_div(pos, L.block_size);
            // only groups that overlap the visible key range are fetched (entries of the block
            // table beyond the request's pages are unspecified)
            const bool live = k < n_units && pos <= hi_all && pos + 15 >= lo_all && slot < B.max_blocks_per_req;
            if (live) pg[x] = req_blocks[slot];
        }
    };
    auto issue_loads = [&](int k, const int32_t (&pg)[2]) {
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            if (x == 1 && !two) continue;
            const int pos = (u_first + k) * kUnit + 16 * (ld_run[x] & 1);
            const int slot = fast_div(pos, L.block_size);
            const int in_page = pos - slot * L.block_size;
            const bool is_v = ld_run[x] >= 2;
            const uint8_t* base = is_v ? v_base : k_base;
            size_t off = 0;  // missing page: rows of page 0, every one of them is masked
            if (pg[x] >= 0)
                off = (size_t)pg[x] * (is_v ? L.v_page_stride_bytes : L.k_page_stride_bytes) +
                      (size_t)in_page * (is_v ? L.v_token_stride_bytes : L.k_token_stride_bytes);
            pf[x] = *(global_cu4*)(base + off + 16 * ld_pc[x]);
        }
    };
    auto commit_loads = [&](int buf) {
        uint8_t* raw = smem + kPfRawBase + buf * kPfRawBytes;
        *reinterpret_cast<u4*>(raw + 16 * tid) = pf[0];
        if (two) *reinterpret_cast<u4*>(raw + 16 * (512 + tid)) = pf[1];
    };

    // ---- dequantiser: this thread's items ----
    // K: dword idx of the 32 x 33 raw dwords (idx = tid, tid + 512, and tid + 1024 for tid < 32);
    // row r = idx / 33, dword w = idx % 33.  Byte q of the dword is row byte 4 w + q: bytes
    // 2..65 are code bytes 0..63 of the first half (elements 2 i, 2 i + 1), bytes 68..131 the
    // second half; the others are scale bytes, their writes go to a dummy area.
    const uint32_t lut_lane = (uint32_t)lane << 2;
    uint32_t k_src[3], k_dst[3][2];
#pragma unroll
    for (int it = 0; it < 3; ++it) {
        const int idx = tid + 512 * it;
        const int r = idx / 33;
        const int w = idx - 33 * r;
        k_src[it] = 4u * (uint32_t)idx;
        const int d0 = r * kPfKStride + 16 * w - (w <= 16 ? 8 : 16);
        k_dst[it][0] = (w == 0) ? (uint32_t)(kPfDummy + 8 * (tid & 15)) : (uint32_t)d0;
        k_dst[it][1] = (w == 16) ? (uint32_t)(kPfDummy + 8 * (tid & 15)) : (uint32_t)(d0 + 8);
    }
    // V: item = (token pair p, dword w) with p = idx & 15, w = idx >> 4 (idx = tid, and
    // tid + 512 for tid < 16).  Tokens 2p, 2p+1 sit in key slots 8 b' + 4 s + {0,1} (+2 for odd p)
    // with s = p >> 3, b' = (p >> 1) & 3; element d lives at V^T row d, 16-byte piece
    // b' ^ ((d >> 1) & 3).  Lanes whose (lane >> 4) is odd write the odd elements first so
    // that the 32 lanes of a write pass cover 32 banks.
    const int nibsel = (lane >> 4) & 1;
    uint32_t v_src[2], v_dst[2][4];
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int idx = tid + 512 * it;
        const int p = idx & 15;
        const int w = idx >> 4;
        v_src[it] = (uint32_t)(kPfRawBytes / 2 + (2 * p) * kTq4RowBytes + 4 * w);
        const int base_d = w <= 16 ? 8 * w - 4 : 8 * w - 8;
        const int bp = (p >> 1) & 3, s = p >> 3;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int d = base_d + 2 * q;  // even element of byte q
            const bool valid = !((w == 0 && q < 2) || (w == 16 && q >= 2)) && w <= 32;
            const int addr = kPfKBytes + d * 64 + 16 * (bp ^ ((d >> 1) & 3)) + 8 * s + 4 * (p & 1) + 64 * nibsel;
            v_dst[it][q] = valid ? (uint32_t)addr : (uint32_t)(kPfDummy + 128 + 4 * (tid & 15));
        }
    }
    auto dequant_unit = [&](int rawbuf, int deqbuf) {
        const uint32_t raw = (uint32_t)(kPfRawBase + rawbuf * kPfRawBytes);
        const uint32_t deq = (uint32_t)(kPfDeqBase + deqbuf * kPfDeqBytes);
        const uint32_t dummy_lo = (uint32_t)kPfDummy;
        // K
#pragma unroll
        for (int it = 0; it < 3; ++it) {
            if (it == 2 && tid >= 32) continue;
            const uint32_t word = *reinterpret_cast<lds_cu32*>((uintptr_t)(raw + k_src[it]));
            uint2 lo, hi;
            lo.x = lut_read(word, lut_lane, 0x0c0c0400u);
            lo.y = lut_read(word, lut_lane, 0x0c0c0500u);
            hi.x = lut_read(word, lut_lane, 0x0c0c0600u);
            hi.y = lut_read(word, lut_lane, 0x0c0c0700u);
            const uint32_t a0 = k_dst[it][0] >= dummy_lo ? k_dst[it][0] : deq + k_dst[it][0];
            const uint32_t a1 = k_dst[it][1] >= dummy_lo ? k_dst[it][1] : deq + k_dst[it][1];
            *reinterpret_cast<uint2*>(smem + a0) = lo;
            *reinterpret_cast<uint2*>(smem + a1) = hi;
        }
        // V
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            if (it == 1 && !two) continue;
            const uint32_t wa = *reinterpret_cast<lds_cu32*>((uintptr_t)(raw + v_src[it]));
            const uint32_t wb = *reinterpret_cast<lds_cu32*>((uintptr_t)(raw + v_src[it] + kTq4RowBytes));
            // byte q of ev / od = (even / odd element of token 2p) | (same of token 2p+1) << 4
            const uint32_t ev = (wa & 0x0F0F0F0Fu) | ((wb << 4) & 0xF0F0F0F0u);
            const uint32_t od = ((wa >> 4) & 0x0F0F0F0Fu) | (wb & 0xF0F0F0F0u);
            const uint32_t first = nibsel ? od : ev;   // element parity nibsel, written at v_dst
            const uint32_t second = nibsel ? ev : od;  // the other parity, 64 bytes away
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t sel = 0x0c0c0400u + ((uint32_t)q << 8);
                const uint32_t x0 = lut_read(first, lut_lane, sel);
                const uint32_t x1 = lut_read(second, lut_lane, sel);
                const bool dm = v_dst[it][q] >= dummy_lo;
                const uint32_t a0 = dm ? v_dst[it][q] : deq + v_dst[it][q];
                const uint32_t a1 = dm ? v_dst[it][q] : (deq + v_dst[it][q]) ^ 64u;
                *reinterpret_cast<uint32_t*>(smem + a0) = x0;
                *reinterpret_cast<uint32_t*>(smem + a1) = x1;
            }
        }
        // scales: thread x * 32 + r (x = 0: K d0, 1: K d1, 2: V d0, 3: V d1) of waves 0 and 1
        if (tid < 128) {
            const int x = tid >> 5, r = tid & 31;
            const uint8_t* src = smem + raw + (x >> 1) * (kPfRawBytes / 2) + r * kTq4RowBytes + (x & 1) * 66;
            const uint16_t bits = *reinterpret_cast<const uint16_t*>(src);
            *reinterpret_cast<float*>(smem + deq + kPfKBytes + kPfVBytes + 4 * tid) =
                (float)__builtin_bit_cast(_Float16, bits);
        }
    };

    // ---- per-wave attention state ----
    f4 o_acc[2][8];
    float m_run = kNegBig, l_run = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) o_acc[h][j] = f4{0.f, 0.f, 0.f, 0.f};

    auto compute_unit = [&](int deqbuf, int t0, const bool MASKED) {
        const uint8_t* kb = smem + kPfDeqBase + deqbuf * kPfDeqBytes;
        const uint8_t* vb = kb + kPfKBytes;
        const float* sc = reinterpret_cast<const float*>(vb + kPfVBytes);
        float score[8];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            h8 a[2][4];
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int m = 0; m < 4; ++m)
                    a[h][m] = *reinterpret_cast<const h8*>(kb + (16 * s + n) * kPfKStride + 2 * (128 * h + 32 * m + 8 * b));
            const f4 kd0 = *reinterpret_cast<const f4*>(sc + 16 * s + 4 * b);
            const f4 kd1 = *reinterpret_cast<const f4*>(sc + 32 + 16 * s + 4 * b);
            f4 s_acc[2] = {f4{0.f, 0.f, 0.f, 0.f}, f4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int h = 0; h < 2; ++h)
                    s_acc[h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[h][m], bq[h][m], s_acc[h], 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float v = kd0[i] * s_acc[0][i] + kd1[i] * s_acc[1][i];
                if (MASKED) {
                    const int pos = t0 + 16 * s + 4 * b + i;
                    score[4 * s + i] = (col_ok && pos >= col_lo && pos <= col_hi) ? v : kNegBig;
                } else {
                    score[4 * s + i] = v;
                }
            }
        }
        // online softmax, log2 domain; key slot j of this lane = token 16 (j >> 2) + 4 b + (j & 3)
        float mx = fmaxf(fmaxf(fmaxf(score[0], score[1]), fmaxf(score[2], score[3])),
                         fmaxf(fmaxf(score[4], score[5]), fmaxf(score[6], score[7])));
        mx = max_over_rows(mx);
        const float m_new = fmaxf(m_run, mx);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        float p[8];
        float psum = 0.f;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            p[t] = __builtin_amdgcn_exp2f(score[t] - m_new);
            if (MASKED) p[t] = score[t] > 0.5f * kNegBig ? p[t] : 0.f;
            psum += p[t];
        }
        l_run = l_run * alpha + psum;
        if (__ballot(alpha != 1.0f) != 0ull) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < 8; ++j) o_acc[h][j] *= alpha;
        }
        u4 pb[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const f4 da = *reinterpret_cast<const f4*>(sc + 64 + 32 * h + 4 * b);
            const f4 db = *reinterpret_cast<const f4*>(sc + 64 + 32 * h + 16 + 4 * b);
            float w[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const float d = t < 4 ? da[t] : db[t - 4];
                // select, not multiply: a garbage scale of a row beyond the sequence must not make NaN
                w[t] = MASKED ? (p[t] > 0.f ? p[t] * d : 0.f) : p[t] * d;
            }
            pb[h] = u4{pack_h2(w[0], w[1]), pack_h2(w[2], w[3]), pack_h2(w[4], w[5]), pack_h2(w[6], w[7])};
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            h8 a[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int d = 128 * h + 16 * j + n;
                a[j] = *reinterpret_cast<const h8*>(vb + d * 64 + 16 * (b ^ ((d >> 1) & 3)));
            }
#pragma unroll
            for (int j = 0; j < 8; ++j)
                o_acc[h][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j], __builtin_bit_cast(h8, pb[h]), o_acc[h][j], 0, 0, 0);
        }
    };

    // ---- pipeline ----
    __syncthreads();  // table complete; query staging (aliases the dequant buffers) consumed
    int32_t pg_next[2];
    load_pages(0, pg_cur);
    load_pages(1, pg_next);
    if (n_units > 0) issue_loads(0, pg_cur);
    for (int it = -2; it < n_units; ++it) {
        // commit unit it + 2 (loaded during the previous iteration), then start unit it + 3
        if (it + 2 < n_units) commit_loads((it + 2) & 1);
        pg_cur[0] = pg_next[0];
        pg_cur[1] = pg_next[1];
        if (it + 3 < n_units) issue_loads(it + 3, pg_cur);
        load_pages(it + 4, pg_next);
        if (it + 1 >= 0 && it + 1 < n_units) dequant_unit((it + 1) & 1, (it + 1) & 1);
        if (it >= 0) {
            const int t0 = (u_first + it) * kUnit;
            compute_unit(it & 1, t0, !(t0 >= i_lo && t0 + kUnit - 1 <= i_hi));
        }
        __syncthreads();
    }

    // ---- epilogue: normalise, transpose through LDS, rotate back, store ----
    l_run = sum_over_rows(l_run);
    float* reg = reinterpret_cast<float*>(smem) + wave * 16 * 260;
    const float inv = l_run > 0.f ? kLutInvGain / l_run : 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j)
            *reinterpret_cast<f4*>(reg + n * 260 + 128 * h + 16 * j + 4 * b) = o_acc[h][j] * inv;
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    __builtin_amdgcn_wave_barrier();
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    for (int c = 0; c < 16; ++c) {
        if (!((ok_mask >> c) & 1u)) continue;
        const int col = 16 * wave + c;
        const int t = fast_div(col, P.q_group);
        const int a = col - t * P.q_group;
        const f4 x = *reinterpret_cast<const f4*>(reg + c * 260 + 4 * lane);
        float o[4] = {x[0], x[1], x[2], x[3]};
        wht256_wave(o, lane);
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = apply_sign(o[k], 4 * lane + k);
        uint2 ob;
        ob.x = (uint32_t)TQ::from_f32(o[0]) | ((uint32_t)TQ::from_f32(o[1]) << 16);
        ob.y = (uint32_t)TQ::from_f32(o[2]) | ((uint32_t)TQ::from_f32(o[3]) << 16);
        const size_t row = (size_t)(tok0 + t) * P.num_q_heads + (size_t)(q_head_base + a);
        *reinterpret_cast<uint2*>(P.out + row * kHeadDim + 4 * lane) = ob;
    }
}

}  // namespace w34
