// Chunked-prefill attention over TQ4, FP8-E4M3, Q8_0, FP16 or BF16 pages for gfx950: many query rows per workgroup,
// every K/V unit dequantised ONCE per workgroup and shared by all waves through LDS.  (FP8 rows
// have the same shape as TQ4 rows -- two scale blocks of 128 elements -- so only the loader and
// the dequantiser differ: codes are widened with v_cvt_scalef32_pk_f16_fp8 instead of the table,
// there is no table in LDS and, for un-rotated layers, no rotation.  16-bit rows are copied into
// the same two tiles as stored and multiplied in their own type; BF16 probabilities are split
// into a high and a low bf16 part.)
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
constexpr int kPfKStride = 544;                               // bytes per dequantised K row (measured: 128-bit reads of 16 rows at this stride do not conflict; 528, 560, 576 do)
constexpr int kPfKBytes = 32 * kPfKStride;                    // 16896
constexpr int kPfVBytes = 256 * 64;                           // V^T: 256 rows x 32 halves
constexpr int kPfScaleBytes = 8 * 32 * 4;                     // per token: K d0, K d1, V d0, V d1 (Q8_0: K d0-d3, V d0-d3)
constexpr int kPfDeqBytes = kPfKBytes + kPfVBytes + kPfScaleBytes;
// LDS map per page format: [table (TQ4 only)] [2 dequantised units] [2 raw units]
template <int KVF>
struct PfLds {
    static constexpr bool kFp8 = KVF == WARP34_KV_FORMAT_FP8_E4M3;
    static constexpr bool k16 = KVF == WARP34_KV_FORMAT_FP16 || KVF == WARP34_KV_FORMAT_BF16;
    static constexpr bool kQ8 = KVF == WARP34_KV_FORMAT_Q8_0;
    static constexpr int kRowBytes = k16 ? 512 : kFp8 ? 264 : kQ8 ? 272 : kTq4RowBytes;
    static constexpr int kRun = 16 * kRowBytes;                // 16 rows: 2112 B / 4224 B / 4352 B / 8192 B
    static constexpr int kRaw = 4 * kRun;                      // K rows 0-31, V rows 0-31
    static constexpr int kDeqBase = (kFp8 || k16 || kQ8) ? 0 : kLutBytes;
    static constexpr int kRawBase = kDeqBase + 2 * kPfDeqBytes;
    static constexpr int kLoop = kRawBase + 2 * kRaw + 256;
    static constexpr int kEpilogue = kPfWaves * 16 * 260 * 4;  // the output transpose regions
    static constexpr int kSmem = kLoop > kEpilogue ? kLoop : kEpilogue;
    static_assert(kSmem <= 160 * 1024, "prefill LDS budget");
};
static_assert(PfLds<WARP34_KV_FORMAT_TQ4>::kRaw == kStageTq4, "TQ4 raw unit");
static_assert(kPfWaves * 16 * 264 * 2 <= 2 * kPfDeqBytes, "query staging must fit in the dequant buffers");

typedef __attribute__((address_space(3))) uint32_t lds_u32;

// 16x16x32 MFMA on fp16 or bf16 operands given as raw bits
template <bool IS_BF16>
__device__ __forceinline__ f4 pf_mfma32(h8 a, h8 b, f4 c) {
    if constexpr (IS_BF16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
}

// VF (8-bit rows stored rotated): the value tile holds the codes themselves (exact in fp16) and
// the block scales go into the probabilities as a high and a low fp16 operand, as for TQ4 rows.
// fp16(d * code) rounds partly alike across a scale block that holds few distinct codes, and the
// inverse rotation of the finished row would gather that common part into a single channel.
// (Q8_0 key tiles hold the codes in either form, see dequant_unit_q8.)
// PC (TQ4 pages): twelve waves.  Waves 0-7 only multiply (16 columns each, as in the eight-wave
// form); waves 8-11 load and dequantise the next unit, a whole 16-row run each.  Every SIMD then
// holds two multiplying waves and one dequantising wave whose instruction streams never wait
// for each other's results inside an iteration.
// SPLIT (with PC): blockIdx.x = tile * P.pf_split + part; a workgroup takes one of P.pf_split equal
// parts of the tile's units and leaves un-normalised partial records (slot P.pf_slot_base + part
// of every row, the decode kernels' format) for the merge kernel.
template <typename TQ, int KVF, bool VF = false, bool PC = false, bool SPLIT = false>
__global__ __launch_bounds__((PC ? 12 : kPfWaves) * 64, 1) void paged_prefill_tq4_kernel(const AttnParams P) {
    using M = PfLds<KVF>;
    constexpr bool FP8 = M::kFp8;
    constexpr bool K16 = M::k16;  // 16-bit rows, read as stored: the MFMAs run in the storage type
    constexpr bool Q8 = M::kQ8;   // Q8_0 rows: the key tile holds the codes, the value tile fp16(d * code) unless VF
    static_assert(!VF || FP8 || Q8, "scales in the probabilities: 8-bit rows only");
    static_assert(!PC || (!M::kFp8 && !M::k16 && !M::kQ8), "separate dequantising waves: TQ4 pages only");
    static_assert(!SPLIT || PC, "split form: TQ4 pages");
    // VF: the tile holds code / kVfGain (a power of two: exact) and the weights p * d * kVfGain.  The
    // block scales of 8-bit rows are small (amax / 448, amax / 127): without the gain the low-order
    // weight operand, 2^-12 of the weight, would fall into fp16's subnormal range and lose its bits.
    constexpr float kVfGain = FP8 ? 256.0f : 128.0f;
    constexpr bool TQ4F = !FP8 && !K16 && !Q8;
    constexpr bool IS_BF16 = KVF == WARP34_KV_FORMAT_BF16;
    static_assert(!K16 || KVF == TQ::kStorageFormat, "16-bit pages are read in the query type");
    constexpr int kPfDeqBase = M::kDeqBase, kPfRawBase = M::kRawBase, kPfRawBytes = M::kRaw;
    constexpr int kRowB = M::kRowBytes, kRunB = M::kRun;
    extern __shared__ __align__(16) uint8_t smem[];
    // (the pair table is addressed absolutely: the dynamic block starts at LDS address 0 because the
    // kernel has no static LDS, which the host checks before the first launch)

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int b = lane >> 4;
    const bool producer = PC && wave >= kPfWaves;  // wave-uniform
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
    const int tile_x = SPLIT ? (int)blockIdx.x / P.pf_split : (int)blockIdx.x;
    const int part_x = SPLIT ? (int)blockIdx.x - tile_x * P.pf_split : 0;
    const int tok0 = rq_start + tile_x * tile_tok;
    if (tok0 >= rq_end || tok0 >= B.total_tokens) return;
    int tile_tokens = rq_end - tok0;
    if (tile_tokens > tile_tok) tile_tokens = tile_tok;
    if (tile_tokens > B.total_tokens - tok0) tile_tokens = B.total_tokens - tok0;

    // ---- the pair table (64 lane replicas, as in the decode kernel) ----
    if (TQ4F && tid < kPfWaves * 64) {
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
    int u_first = lo_all >> 5;
    int n_units = hi_all >= lo_all ? (hi_all >> 5) - u_first + 1 : 0;
    if constexpr (SPLIT) {  // this workgroup's part of the units
        const int per_part = (n_units + P.pf_split - 1) / P.pf_split;
        const int first = part_x * per_part;
        int n = n_units - first;
        n = n < 0 ? 0 : (n > per_part ? per_part : n);
        u_first += first;
        n_units = n;
    }

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
    const float q_scale = B.sm_scale * kLog2e * (TQ4F ? kLutInvGain : 1.0f);
    const bool rot_q = !K16 && P.rot_q != 0;
    const bool rot_out = !K16 && P.rot_out != 0;
    if (!producer) {
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
            if (rot_q) {  // keys stored rotated: rotate the query rows
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] = apply_sign(v[k], 4 * lane + k);
                wht256_wave(v, lane);
            }
            uint2 packed = {0u, 0u};  // dead columns: zero query
            if ((ok_mask >> c) & 1u) {
                if constexpr (K16) {
                    packed = q_raw[c];  // as given: the scores are scaled after the MFMAs
                } else if constexpr (FP8 || Q8) {
                    // the softmax factor is applied with the fp32 key scales: an un-rotated fp16
                    // query enters the MFMAs exactly as given
                    packed.x = pack_h2(v[0], v[1]);
                    packed.y = pack_h2(v[2], v[3]);
                } else {
                    packed.x = pack_h2(v[0] * q_scale, v[1] * q_scale);
                    packed.y = pack_h2(v[2] * q_scale, v[3] * q_scale);
                }
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
            bq[h][m] = producer ? h8{} : *reinterpret_cast<const h8*>(qbuf + n * kQStride + 128 * h + 32 * m + 8 * b);

    // ---- loader ----
    // A unit is four runs of 16 rows: K rows 0-15, K rows 16-31, V rows 0-15, V rows 16-31.
    // TQ4: a run is 2112 B = 132 16-byte pieces; waves 2r and 2r+1 load pieces 0-127 of run r
    // (one piece per lane, wave-uniform base), lanes 0-3 of wave 2r also carry the tail pieces
    // 128-131.  FP8: a run is 4224 B = 264 pieces; each wave of the pair loads 132 of them
    // (two per lane and a four-lane tail).
    const uint8_t* k_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.k_base) +
                            (size_t)kv_head * L.k_head_stride_bytes;
    const uint8_t* v_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.v_base) +
                            (size_t)kv_head * L.v_head_stride_bytes;
    const int32_t* req_blocks = B.block_tables + (size_t)req * B.max_blocks_per_req;
    const int ld_run = PC ? (wave - kPfWaves) & 3 : wave >> 1;  // PC: one run per dequantising wave
    const bool ld_is_v = ld_run >= 2;
    // Q8_0: a run is 4352 B = 272 pieces; each wave of the pair loads 136 (two per lane and an eight-lane tail)
    const bool ld_tail = !K16 && (PC || FP8 || Q8 || (wave & 1) == 0);  // wave-uniform
    constexpr int kTailLanes = Q8 ? 8 : 4;
    const uint8_t* ld_base = ld_is_v ? v_base : k_base;
    const uint64_t ld_page_stride = ld_is_v ? L.v_page_stride_bytes : L.k_page_stride_bytes;
    const uint64_t ld_tok_stride = ld_is_v ? L.v_token_stride_bytes : L.k_token_stride_bytes;
    // 16-bit rows: a run is 8192 B = 512 pieces; each wave of the pair loads 256 (four per lane), no tail
    const uint32_t ld_lane_off = (uint32_t)((PC ? 0 : (wave & 1) * (K16 ? 4096 : FP8 ? 2112 : Q8 ? 2176 : 1024)) + 16 * lane);
    const uint32_t ld_tail_off = (uint32_t)((FP8 ? (wave & 1) * 2112 : Q8 ? (wave & 1) * 2176 : 0) + 2048 +
                                            16 * (lane & (kTailLanes - 1)));
    const uint32_t ld_commit0 = (uint32_t)(ld_run * kRunB) + ld_lane_off;
    const uint32_t ld_commit1 = (uint32_t)(ld_run * kRunB) + ld_tail_off;
    u4 pf[K16 ? 4 : (FP8 || Q8 || PC) ? 3 : 2];
    // page id of unit k (relative to u_first) for this wave's run; -1 = nothing to fetch.
    // Only groups that overlap the visible key range are fetched: block-table entries beyond
    // the request's pages are unspecified.
    auto load_page = [&](int k) -> int32_t {
        const int pos = (u_first + k) * kUnit + 16 * (ld_run & 1);
        const int slot = __builtin_amdgcn_readfirstlane(div_block(pos, P));
        const bool live = k < n_units && pos <= hi_all && pos + 15 >= lo_all && slot < B.max_blocks_per_req;
        int32_t pg = -1;
        if (live) pg = req_blocks[slot];
        return pg;  // wave-uniform value in a vector register: made scalar where it is used, an iteration later
    };
    auto issue_loads = [&](int k, int32_t pg) {
        const int pos = (u_first + k) * kUnit + 16 * (ld_run & 1);
        const int slot = __builtin_amdgcn_readfirstlane(div_block(pos, P));
        const int in_page = pos - slot * L.block_size;
        size_t off = 0;  // missing page: rows of page 0, every one of them is masked
        if (pg >= 0) off = (size_t)pg * ld_page_stride + (size_t)in_page * ld_tok_stride;
        const uint8_t* src = ld_base + off;
        pf[0] = *(global_cu4*)(src + ld_lane_off);
        if constexpr (K16) {
#pragma unroll
            for (int i = 1; i < 4; ++i) pf[i] = *(global_cu4*)(src + ld_lane_off + 1024 * i);
        } else {
            if (ld_tail) pf[1] = *(global_cu4*)(src + ld_tail_off);
            if constexpr (FP8 || Q8 || PC) pf[2] = *(global_cu4*)(src + ld_lane_off + 1024);
        }
    };
    auto commit_loads = [&](int buf) {
        uint8_t* raw = smem + kPfRawBase + buf * kPfRawBytes;
        *reinterpret_cast<u4*>(raw + ld_commit0) = pf[0];
        if constexpr (K16) {
#pragma unroll
            for (int i = 1; i < 4; ++i) *reinterpret_cast<u4*>(raw + ld_commit0 + 1024 * i) = pf[i];
        } else {
            if (ld_tail && lane < kTailLanes) *reinterpret_cast<u4*>(raw + ld_commit1) = pf[1];
            if constexpr (FP8 || Q8 || PC) *reinterpret_cast<u4*>(raw + ld_commit0 + 1024) = pf[2];
        }
    };

    // ---- dequantiser ----
    // A raw row is 33 dwords; dwords 0 and 16 hold two scale bytes and two code bytes each.
    // They are fused into one synthetic dword [code bytes 0,1 | code bytes 62,63], which leaves
    // exactly 32 four-code-byte items per row:
    //   item 0      : alignbit(dword 16, dword 0, 16)  -> elements 0..3 and 124..127
    //   item j 1..15: dword j                          -> elements 8 j - 4 .. 8 j + 3
    //   item j 16..31: dword j + 1                     -> elements 8 j .. 8 j + 7
    // K: 32 rows x 32 items = two per thread (item idx = tid, tid + 512: row idx >> 5, j = idx & 31);
    //    the four looked-up pairs are written as two 8-byte stores into the row-major fp16 tile.
    // V: 16 token pairs x 32 items = one per thread (pair p = tid & 15, j = tid >> 4).  Tokens
    //    2p, 2p+1 sit in key slots 8 b' + 4 s + {0,1} (+2 for odd p), s = p >> 3, b' = (p >> 1) & 3;
    //    element d lives in V^T row d, 16-byte piece b' ^ ((d >> 1) & 3).  Lanes whose
    //    (lane >> 4) is odd write the odd elements first so that a 32-lane write pass covers
    //    32 banks.
    const uint32_t lut_lane = (uint32_t)lane << 2;
    auto item_src = [](int j, uint32_t (&src)[2], uint32_t& shift) {
        // byte offsets of the two dwords inside the row, and the alignbit shift
        if (j == 0) {
            src[0] = 0;
            src[1] = 64;
            shift = 16;
        } else {
            const int w = j < 16 ? j : j + 1;
            src[0] = src[1] = 4u * (uint32_t)w;
            shift = 0;
        }
    };
    // (PC: 256 dequantising threads take twice the items)
    constexpr int kDqThreads = PC ? 256 : 512;
    constexpr int kKItems = 1024 / kDqThreads, kVItems = 512 / kDqThreads;
    const int dq_tid = PC ? (tid - kPfWaves * 64) & 255 : tid;
    uint32_t k_src[kKItems][2], k_shift[kKItems], k_dst[kKItems][2];
#pragma unroll
    for (int it = 0; it < kKItems; ++it) {
        const int idx = dq_tid + kDqThreads * it;
        const int r = idx >> 5, j = idx & 31;
        uint32_t src[2];
        item_src(j, src, k_shift[it]);
        k_src[it][0] = (uint32_t)(r * kTq4RowBytes) + src[0];
        k_src[it][1] = (uint32_t)(r * kTq4RowBytes) + src[1];
        const int d_lo = j == 0 ? 0 : j < 16 ? 8 * j - 4 : 8 * j;   // element of code byte 0
        const int d_hi = j == 0 ? 124 : d_lo + 4;                    // element of code byte 2
        k_dst[it][0] = (uint32_t)(r * kPfKStride + 2 * d_lo);
        k_dst[it][1] = (uint32_t)(r * kPfKStride + 2 * d_hi);
    }
    const int nibsel = (lane >> 4) & 1;
    uint32_t v_src[kVItems][2], v_shift[kVItems], v_dst[kVItems][4];
#pragma unroll
    for (int vi = 0; vi < kVItems; ++vi) {
        const int p = dq_tid & 15, j = (dq_tid >> 4) + (kDqThreads / 16) * vi;  // (j keeps the parity of lane >> 4)
        uint32_t src[2];
        item_src(j, src, v_shift[vi]);
        v_src[vi][0] = (uint32_t)(kPfRawBytes / 2 + (2 * p) * kTq4RowBytes) + src[0];
        v_src[vi][1] = (uint32_t)(kPfRawBytes / 2 + (2 * p) * kTq4RowBytes) + src[1];
        const int bp = (p >> 1) & 3, s = p >> 3;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int d = j == 0 ? (q < 2 ? 2 * q : 120 + 2 * q) : (j < 16 ? 8 * j - 4 : 8 * j) + 2 * q;
            v_dst[vi][q] = (uint32_t)(kPfKBytes + d * 64 + 16 * (bp ^ ((d >> 1) & 3)) + 8 * s + 4 * (p & 1) + 64 * nibsel);
        }
    }
    // ---- per-wave attention state ----
    f4 o_acc[2][8];
    float m_run = kNegBig, l_run = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) o_acc[h][j] = f4{0.f, 0.f, 0.f, 0.f};

    // Three phases, each a batch of independent LDS operations: all raw reads, all table reads,
    // all writes.  (Written item by item, every item's reads would have to wait for the previous
    // item's writes: the compiler cannot prove that they do not alias.)
    auto dequant_unit = [&](int rawbuf, int deqbuf) {
        const uint32_t raw = (uint32_t)(kPfRawBase + rawbuf * kPfRawBytes);
        const uint32_t deq = (uint32_t)(kPfDeqBase + deqbuf * kPfDeqBytes);
        // ---- phase 1: raw dwords ----
        uint32_t kw0[kKItems], kw1[kKItems];
#pragma unroll
        for (int it = 0; it < kKItems; ++it) {
            kw0[it] = *reinterpret_cast<lds_cu32*>((uintptr_t)(raw + k_src[it][0]));
            kw1[it] = *reinterpret_cast<lds_cu32*>((uintptr_t)(raw + k_src[it][1]));
        }
        uint32_t a0[kVItems], a1[kVItems], b0[kVItems], b1[kVItems];
#pragma unroll
        for (int vi = 0; vi < kVItems; ++vi) {
            a0[vi] = *reinterpret_cast<lds_cu32*>((uintptr_t)(raw + v_src[vi][0]));
            a1[vi] = *reinterpret_cast<lds_cu32*>((uintptr_t)(raw + v_src[vi][1]));
            b0[vi] = *reinterpret_cast<lds_cu32*>((uintptr_t)(raw + v_src[vi][0] + kTq4RowBytes));
            b1[vi] = *reinterpret_cast<lds_cu32*>((uintptr_t)(raw + v_src[vi][1] + kTq4RowBytes));
        }
        // scales: thread x * 32 + r (x = 0: K d0, 1: K d1, 2: V d0, 3: V d1) of the first two dequantising waves
        uint16_t scale_bits = 0;
        if (dq_tid < 128) {
            const int x = dq_tid >> 5, r = dq_tid & 31;
            scale_bits = *reinterpret_cast<const uint16_t*>(smem + raw + (x >> 1) * (kPfRawBytes / 2) +
                                                            r * kTq4RowBytes + (x & 1) * 66);
        }
        // ---- phase 2: table reads ----
        uint2 k_lo[kKItems], k_hi[kKItems];
#pragma unroll
        for (int it = 0; it < kKItems; ++it) {
            const uint32_t word = __builtin_amdgcn_alignbit(kw1[it], kw0[it], k_shift[it]);
            k_lo[it].x = lut_read(word, lut_lane, 0x0c0c0400u);
            k_lo[it].y = lut_read(word, lut_lane, 0x0c0c0500u);
            k_hi[it].x = lut_read(word, lut_lane, 0x0c0c0600u);
            k_hi[it].y = lut_read(word, lut_lane, 0x0c0c0700u);
        }
        uint32_t vx0[kVItems][4], vx1[kVItems][4];
#pragma unroll
        for (int vi = 0; vi < kVItems; ++vi) {
            const uint32_t wa = __builtin_amdgcn_alignbit(a1[vi], a0[vi], v_shift[vi]);
            const uint32_t wb = __builtin_amdgcn_alignbit(b1[vi], b0[vi], v_shift[vi]);
            // byte q of ev / od = (even / odd element of token 2p) | (same of token 2p+1) << 4
            const uint32_t ev = (wa & 0x0F0F0F0Fu) | ((wb << 4) & 0xF0F0F0F0u);
            const uint32_t od = ((wa >> 4) & 0x0F0F0F0Fu) | (wb & 0xF0F0F0F0u);
            const uint32_t first = nibsel ? od : ev;   // elements of parity nibsel, stored at v_dst
            const uint32_t second = nibsel ? ev : od;  // the other parity, one V^T row (64 B) away
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t sel = 0x0c0c0400u + ((uint32_t)q << 8);
                vx0[vi][q] = lut_read(first, lut_lane, sel);
                vx1[vi][q] = lut_read(second, lut_lane, sel);
            }
        }
        // ---- phase 3: writes ----
#pragma unroll
        for (int it = 0; it < kKItems; ++it) {
            *reinterpret_cast<uint2*>(smem + deq + k_dst[it][0]) = k_lo[it];
            *reinterpret_cast<uint2*>(smem + deq + k_dst[it][1]) = k_hi[it];
        }
#pragma unroll
        for (int vi = 0; vi < kVItems; ++vi)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t addr = deq + v_dst[vi][q];
                *reinterpret_cast<uint32_t*>(smem + addr) = vx0[vi][q];
                *reinterpret_cast<uint32_t*>(smem + (addr ^ 64u)) = vx1[vi][q];
            }
        if (dq_tid < 128) {
            *reinterpret_cast<float*>(smem + deq + kPfKBytes + kPfVBytes + 4 * dq_tid) =
                (float)__builtin_bit_cast(_Float16, scale_bits);
        }
    };

    // FP8 rows: 256 E4M3 codes, then fp32 d0, d1.  Same three phases.  K: thread (row r = tid / 16,
    // segment g = tid % 16) widens codes 16 g .. 16 g + 15 into the row-major fp16 tile (exact; the
    // scores take the fp32 scales).  V: thread (token pair p = tid % 16, group j = tid / 16) turns
    // dims 8 j .. 8 j + 7 of tokens 2p, 2p + 1 into fp16(d * code), each element rounded on its own
    // (a scale folded into the probabilities would round all 128 elements of a half the same way,
    // and the inverse rotation of rotated pages gathers such an error into a single channel), and
    // stores them as (token 2p, token 2p + 1) pairs into the transposed tile, same slots and
    // swizzle as the TQ4 path.  Value rows outside the visible key range become zeros: unwritten
    // pool memory may hold NaN codes, and 0 * NaN would poison the P V product.
    auto dequant_unit_fp8 = [&](int rawbuf, int deqbuf, int t0) {
        const uint8_t* raw = smem + kPfRawBase + rawbuf * kPfRawBytes;
        uint8_t* deq = smem + kPfDeqBase + deqbuf * kPfDeqBytes;
        const int kr = tid >> 4, kg = tid & 15;
        const int vp = tid & 15, vj = tid >> 4;
        // ---- phase 1: raw codes and scales ----
        const u2v kc0 = *reinterpret_cast<const u2v*>(raw + kr * kRowB + 16 * kg);
        const u2v kc1 = *reinterpret_cast<const u2v*>(raw + kr * kRowB + 16 * kg + 8);
        u2v va = *reinterpret_cast<const u2v*>(raw + kPfRawBytes / 2 + (2 * vp) * kRowB + 8 * vj);
        u2v vb = *reinterpret_cast<const u2v*>(raw + kPfRawBytes / 2 + (2 * vp + 1) * kRowB + 8 * vj);
        float da = *reinterpret_cast<const float*>(raw + kPfRawBytes / 2 + (2 * vp) * kRowB + 256 + 4 * (vj >> 4));
        float db = *reinterpret_cast<const float*>(raw + kPfRawBytes / 2 + (2 * vp + 1) * kRowB + 256 + 4 * (vj >> 4));
        float scale = 0.f;
        if (tid < (VF ? 128 : 64)) {
            const int x = tid >> 5, r = tid & 31;  // K d0, K d1 (VF: then V d0, V d1)
            scale = *reinterpret_cast<const float*>(raw + (x >> 1) * (kPfRawBytes / 2) + r * kRowB + 256 + 4 * (x & 1));
            if (x >= 2) scale = (t0 + r >= lo_all && t0 + r <= hi_all) ? scale * kVfGain : 0.f;
            else scale *= q_scale;  // the softmax factor rides on the key scales: the query operand stays unscaled
        }
        // ---- phase 2: widen ----
        u4 k_lo, k_hi;
        {
            uint32_t h[8];
            fp8x4_to_h4(kc0[0], h[0], h[1]);
            fp8x4_to_h4(kc0[1], h[2], h[3]);
            fp8x4_to_h4(kc1[0], h[4], h[5]);
            fp8x4_to_h4(kc1[1], h[6], h[7]);
            k_lo = u4{h[0], h[1], h[2], h[3]};
            k_hi = u4{h[4], h[5], h[6], h[7]};
        }
        {
            const int pa = t0 + 2 * vp;
            const bool a_ok = pa >= lo_all && pa <= hi_all, b_ok = pa + 1 >= lo_all && pa + 1 <= hi_all;
            va[0] = a_ok ? va[0] : 0u, va[1] = a_ok ? va[1] : 0u, da = a_ok ? da : 0.f;
            vb[0] = b_ok ? vb[0] : 0u, vb[1] = b_ok ? vb[1] : 0u, db = b_ok ? db : 0.f;
        }
        float fa[8], fb[8];
        {
            float t[4];
            codes4_to_f32<true>(va[0], t);
            fa[0] = t[0], fa[1] = t[1], fa[2] = t[2], fa[3] = t[3];
            codes4_to_f32<true>(va[1], t);
            fa[4] = t[0], fa[5] = t[1], fa[6] = t[2], fa[7] = t[3];
            codes4_to_f32<true>(vb[0], t);
            fb[0] = t[0], fb[1] = t[1], fb[2] = t[2], fb[3] = t[3];
            codes4_to_f32<true>(vb[1], t);
            fb[4] = t[0], fb[5] = t[1], fb[6] = t[2], fb[7] = t[3];
        }
        // ---- phase 3: writes ----
        *reinterpret_cast<u4*>(deq + kr * kPfKStride + 32 * kg) = k_lo;
        *reinterpret_cast<u4*>(deq + kr * kPfKStride + 32 * kg + 16) = k_hi;
        const int bp = (vp >> 1) & 3, sl = vp >> 3;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int d = 8 * vj + e;
            // (token 2p, token 2p + 1) of dim d
            *reinterpret_cast<uint32_t*>(deq + kPfKBytes + d * 64 + 16 * (bp ^ ((d >> 1) & 3)) + 8 * sl + 4 * (vp & 1)) =
                VF ? pack_h2(fa[e] * (1.0f / kVfGain), fb[e] * (1.0f / kVfGain)) : pack_h2(da * fa[e], db * fb[e]);
        }
        if (tid < (VF ? 128 : 64)) *reinterpret_cast<float*>(deq + kPfKBytes + kPfVBytes + 4 * tid) = scale;
    };

    // Q8_0 rows: four blocks of {fp32 d, 64 int8}.  The key tile receives the codes (exact in fp16)
    // and the scores take the four fp32 block scales: keys staged as fp16(d * code), as in the
    // reference's MMA kernels (op_paged_attn.cu:59-71), move a score by ~2e-3 when the row has
    // outlier channels, enough to shift the weights of two dominant keys against each other.  The
    // value tile receives fp16(d * code), every element rounded on its own from fp32 (VF: the
    // codes).  Thread roles as for FP8 rows.
    auto dequant_unit_q8 = [&](int rawbuf, int deqbuf, int t0) {
        const uint8_t* raw = smem + kPfRawBase + rawbuf * kPfRawBytes;
        uint8_t* deq = smem + kPfDeqBase + deqbuf * kPfDeqBytes;
        const int kr = tid >> 4, kg = tid & 15;
        const int vp = tid & 15, vj = tid >> 4;
        // ---- phase 1: raw codes and scales ----
        const uint8_t* krow = raw + kr * kRowB + 68 * (kg >> 2);
        float kscale = 0.f;  // scale of block tid / 32 of key row tid % 32, times the softmax factor
        if (tid < 128) kscale = *reinterpret_cast<const float*>(raw + (tid & 31) * kRowB + 68 * (tid >> 5)) * q_scale;
        uint32_t kc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) kc[i] = *reinterpret_cast<const uint32_t*>(krow + 4 + 16 * (kg & 3) + 4 * i);
        const uint8_t* va_row = raw + kPfRawBytes / 2 + (2 * vp) * kRowB + 68 * (vj >> 3);
        const uint8_t* vb_row = va_row + kRowB;
        float da = *reinterpret_cast<const float*>(va_row);
        float db = *reinterpret_cast<const float*>(vb_row);
        uint32_t va[2], vb[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            va[i] = *reinterpret_cast<const uint32_t*>(va_row + 4 + 8 * (vj & 7) + 4 * i);
            vb[i] = *reinterpret_cast<const uint32_t*>(vb_row + 4 + 8 * (vj & 7) + 4 * i);
        }
        float vscale = 0.f;  // VF: scale of block (tid - 128) / 32 of value row tid % 32
        if (VF && tid >= 128 && tid < 256) {
            const int r = tid & 31;
            vscale = *reinterpret_cast<const float*>(raw + kPfRawBytes / 2 + r * kRowB + 68 * ((tid - 128) >> 5));
            vscale = (t0 + r >= lo_all && t0 + r <= hi_all) ? vscale * kVfGain : 0.f;
        }
        // ---- phase 2: widen the key codes (exact), dequantise the values ----
        uint32_t kh[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) i8x4_to_h4(kc[i], kh[2 * i], kh[2 * i + 1]);
        {
            const int pa = t0 + 2 * vp;
            const bool a_ok = pa >= lo_all && pa <= hi_all, b_ok = pa + 1 >= lo_all && pa + 1 <= hi_all;
            va[0] = a_ok ? va[0] : 0u, va[1] = a_ok ? va[1] : 0u, da = a_ok ? da : 0.f;
            vb[0] = b_ok ? vb[0] : 0u, vb[1] = b_ok ? vb[1] : 0u, db = b_ok ? db : 0.f;
        }
        float fa[8], fb[8];
        {
            float t[4];
            codes4_to_f32<false>(va[0], t);
            fa[0] = t[0], fa[1] = t[1], fa[2] = t[2], fa[3] = t[3];
            codes4_to_f32<false>(va[1], t);
            fa[4] = t[0], fa[5] = t[1], fa[6] = t[2], fa[7] = t[3];
            codes4_to_f32<false>(vb[0], t);
            fb[0] = t[0], fb[1] = t[1], fb[2] = t[2], fb[3] = t[3];
            codes4_to_f32<false>(vb[1], t);
            fb[4] = t[0], fb[5] = t[1], fb[6] = t[2], fb[7] = t[3];
        }
        // ---- phase 3: writes ----
        *reinterpret_cast<u4*>(deq + kr * kPfKStride + 32 * kg) = u4{kh[0], kh[1], kh[2], kh[3]};
        *reinterpret_cast<u4*>(deq + kr * kPfKStride + 32 * kg + 16) = u4{kh[4], kh[5], kh[6], kh[7]};
        const int bp = (vp >> 1) & 3, sl = vp >> 3;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int d = 8 * vj + e;
            *reinterpret_cast<uint32_t*>(deq + kPfKBytes + d * 64 + 16 * (bp ^ ((d >> 1) & 3)) + 8 * sl + 4 * (vp & 1)) =
                VF ? pack_h2(fa[e] * (1.0f / kVfGain), fb[e] * (1.0f / kVfGain)) : pack_h2(da * fa[e], db * fb[e]);
        }
        if (tid < 128) *reinterpret_cast<float*>(deq + kPfKBytes + kPfVBytes + 4 * tid) = kscale;
        if (VF && tid >= 128 && tid < 256) *reinterpret_cast<float*>(deq + kPfKBytes + kPfVBytes + 4 * tid) = vscale;
    };

    // 16-bit rows: nothing to dequantise.  K: thread (row r = tid / 16, segment g = tid % 16)
    // copies elements 16 g .. 16 g + 15 into the padded row-major tile.  V: thread (token pair
    // p = tid % 16, group j = tid / 16) stores dims 8 j .. 8 j + 7 of tokens 2p, 2p + 1 as (token 2p,
    // token 2p + 1) pairs into the transposed tile.  Value rows outside the visible key range
    // become zeros (unwritten pool memory may hold NaN patterns).
    auto dequant_unit_16 = [&](int rawbuf, int deqbuf, int t0) {
        const uint8_t* raw = smem + kPfRawBase + rawbuf * kPfRawBytes;
        uint8_t* deq = smem + kPfDeqBase + deqbuf * kPfDeqBytes;
        const int kr = tid >> 4, kg = tid & 15;
        const int vp = tid & 15, vj = tid >> 4;
        const u4 k_lo = *reinterpret_cast<const u4*>(raw + kr * kRowB + 32 * kg);
        const u4 k_hi = *reinterpret_cast<const u4*>(raw + kr * kRowB + 32 * kg + 16);
        u4 ha = *reinterpret_cast<const u4*>(raw + kPfRawBytes / 2 + (2 * vp) * kRowB + 16 * vj);
        u4 hb = *reinterpret_cast<const u4*>(raw + kPfRawBytes / 2 + (2 * vp + 1) * kRowB + 16 * vj);
        {
            const int pa = t0 + 2 * vp;
            const bool a_ok = pa >= lo_all && pa <= hi_all, b_ok = pa + 1 >= lo_all && pa + 1 <= hi_all;
            if (!a_ok) ha = u4{0u, 0u, 0u, 0u};
            if (!b_ok) hb = u4{0u, 0u, 0u, 0u};
        }
        *reinterpret_cast<u4*>(deq + kr * kPfKStride + 32 * kg) = k_lo;
        *reinterpret_cast<u4*>(deq + kr * kPfKStride + 32 * kg + 16) = k_hi;
        const int bp = (vp >> 1) & 3, sl = vp >> 3;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int d = 8 * vj + e;
            const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
            const uint32_t pair = __builtin_amdgcn_perm(hb[e >> 1], ha[e >> 1], sel);
            *reinterpret_cast<uint32_t*>(deq + kPfKBytes + d * 64 + 16 * (bp ^ ((d >> 1) & 3)) + 8 * sl + 4 * (vp & 1)) = pair;
        }
    };

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
            // (the scale reads are issued with the operand reads, ahead of the MFMAs)
            f4 kd0 = {1.f, 1.f, 1.f, 1.f}, kd1 = {1.f, 1.f, 1.f, 1.f};
            if constexpr (!K16 && !Q8) {
                kd0 = *reinterpret_cast<const f4*>(sc + 16 * s + 4 * b);
                kd1 = *reinterpret_cast<const f4*>(sc + 32 + 16 * s + 4 * b);
            }
            if constexpr (Q8) {
                // one partial score per 64-element scale block (two 32-wide steps), then the fp32 scales
                f4 kd[4], s_blk[4];
#pragma unroll
                for (int blk = 0; blk < 4; ++blk) {
                    kd[blk] = *reinterpret_cast<const f4*>(sc + 32 * blk + 16 * s + 4 * b);
                    s_blk[blk] = f4{0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
                for (int m = 0; m < 4; ++m)
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        s_blk[2 * h + (m >> 1)] = pf_mfma32<false>(a[h][m], bq[h][m], s_blk[2 * h + (m >> 1)]);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    score[4 * s + i] = (kd[0][i] * s_blk[0][i] + kd[1][i] * s_blk[1][i]) +
                                       (kd[2][i] * s_blk[2][i] + kd[3][i] * s_blk[3][i]);
                continue;
            }
            f4 s_acc[2] = {f4{0.f, 0.f, 0.f, 0.f}, f4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int h = 0; h < 2; ++h) s_acc[h] = pf_mfma32<IS_BF16>(a[h][m], bq[h][m], s_acc[h]);
            if constexpr (K16) {  // rows as stored: no scales, the softmax factor comes in here
#pragma unroll
                for (int i = 0; i < 4; ++i) score[4 * s + i] = (s_acc[0][i] + s_acc[1][i]) * q_scale;
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) score[4 * s + i] = kd0[i] * s_acc[0][i] + kd1[i] * s_acc[1][i];
            }
        }
        // BF16 pages: the value operands of the first half of the head dimension are requested
        // here, ahead of the softmax arithmetic (the branches below keep the compiler from moving
        // them up itself).  Measured: -5 % with the two-operand bf16 probabilities, +3 to +5 % in
        // the fp16 forms, which therefore read them where they are used.
        h8 av0[8];
        if constexpr (IS_BF16) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int d = 16 * j + n;
                av0[j] = *reinterpret_cast<const h8*>(vb + d * 64 + 16 * (b ^ ((d >> 1) & 3)));
            }
        }
        // (the MASKED tests sit outside the unrolled loops: one wave-uniform branch per block)
        if (MASKED) {
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int pos = t0 + 16 * (t >> 2) + 4 * b + (t & 3);
                score[t] = (col_ok && pos >= col_lo && pos <= col_hi) ? score[t] : kNegBig;
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
        for (int t = 0; t < 8; ++t) p[t] = __builtin_amdgcn_exp2f(score[t] - m_new);
        if (MASKED) {
#pragma unroll
            for (int t = 0; t < 8; ++t) p[t] = score[t] > 0.5f * kNegBig ? p[t] : 0.f;
        }
#pragma unroll
        for (int t = 0; t < 8; ++t) psum += p[t];
        l_run = l_run * alpha + psum;
        if (__ballot(alpha != 1.0f) != 0ull) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < 8; ++j) o_acc[h][j] *= alpha;
        }
        u4 pb[2];
        u4 pb_lo = {0u, 0u, 0u, 0u};
        u4 pb_l2[2] = {u4{0u, 0u, 0u, 0u}, u4{0u, 0u, 0u, 0u}};  // TQ4, rotated FP8: low-order operands per half
        u4 pq[Q8 && VF ? 4 : 1], pq_lo[Q8 && VF ? 4 : 1];        // rotated Q8_0: operands per 64-element block
        if constexpr (IS_BF16) {
            // bf16 keeps 8 bits of a probability: the rest goes into a second operand (two MFMAs)
            uint32_t hi[8], lo[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                hi[t] = BF16::from_f32(p[t]);
                lo[t] = BF16::from_f32(p[t] - BF16::to_f32((uint16_t)hi[t]));
            }
            pb[0] = u4{hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16), hi[4] | (hi[5] << 16), hi[6] | (hi[7] << 16)};
            pb[1] = pb[0];
            pb_lo = u4{lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16), lo[4] | (lo[5] << 16), lo[6] | (lo[7] << 16)};
        } else if constexpr ((FP8 || K16 || Q8) && !VF) {  // the value tile already carries its scales
            pb[0] = u4{pack_h2(p[0], p[1]), pack_h2(p[2], p[3]), pack_h2(p[4], p[5]), pack_h2(p[6], p[7])};
            pb[1] = pb[0];
        } else if constexpr (Q8) {
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                const f4 da = *reinterpret_cast<const f4*>(sc + 128 + 32 * blk + 4 * b);
                const f4 db = *reinterpret_cast<const f4*>(sc + 128 + 32 * blk + 16 + 4 * b);
                float w[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) w[t] = p[t] * (t < 4 ? da[t] : db[t - 4]);
                if (MASKED) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) w[t] = p[t] > 0.f ? w[t] : 0.f;
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    uint32_t whi, wlo;
                    split_h2(w[2 * k], w[2 * k + 1], whi, wlo);
                    pq[blk][k] = whi;
                    pq_lo[blk][k] = wlo;
                }
            }
        } else {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const f4 da = *reinterpret_cast<const f4*>(sc + 64 + 32 * h + 4 * b);
                const f4 db = *reinterpret_cast<const f4*>(sc + 64 + 32 * h + 16 + 4 * b);
                float w[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) w[t] = p[t] * (t < 4 ? da[t] : db[t - 4]);
                if (MASKED) {
                    // select, not multiply: a garbage scale of a row beyond the sequence must not make NaN
#pragma unroll
                    for (int t = 0; t < 8; ++t) w[t] = p[t] > 0.f ? w[t] : 0.f;
                }
                // high and low fp16 operand (split_h2): one rounding of p * d would be shared by the
                // whole 128-element scale block
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    uint32_t whi, wlo;
                    split_h2(w[2 * k], w[2 * k + 1], whi, wlo);
                    pb[h][k] = whi;
                    pb_l2[h][k] = wlo;
                }
            }
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            h8 a[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int d = 128 * h + 16 * j + n;
                a[j] = (IS_BF16 && h == 0) ? av0[j] : *reinterpret_cast<const h8*>(vb + d * 64 + 16 * (b ^ ((d >> 1) & 3)));
            }
            if constexpr (Q8 && VF) {
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    o_acc[h][j] = pf_mfma32<false>(a[j], __builtin_bit_cast(h8, pq[2 * h + (j >> 2)]), o_acc[h][j]);
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    o_acc[h][j] = pf_mfma32<false>(a[j], __builtin_bit_cast(h8, pq_lo[2 * h + (j >> 2)]), o_acc[h][j]);
                continue;
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) o_acc[h][j] = pf_mfma32<IS_BF16>(a[j], __builtin_bit_cast(h8, pb[h]), o_acc[h][j]);
            // the low-order operands in a pass of their own: a tile's two MFMAs are then eight
            // instructions apart instead of back to back (the second waits for the first's result)
            if constexpr (IS_BF16) {
#pragma unroll
                for (int j = 0; j < 8; ++j) o_acc[h][j] = pf_mfma32<true>(a[j], __builtin_bit_cast(h8, pb_lo), o_acc[h][j]);
            }
            if constexpr (TQ4F || (FP8 && VF)) {
#pragma unroll
                for (int j = 0; j < 8; ++j) o_acc[h][j] = pf_mfma32<false>(a[j], __builtin_bit_cast(h8, pb_l2[h]), o_acc[h][j]);
            }
        }
    };

    // ---- pipeline ----
    __syncthreads();  // table complete; query staging (aliases the dequant buffers) consumed
    if constexpr (PC) {
        // Same schedule, the roles in different waves: between two barriers the dequantising
        // waves commit unit it + 2, request unit it + 3 and dequantise unit it + 1 into buffer
        // (it + 1) & 1, the multiplying waves work on unit it in buffer it & 1.
        if (producer) {
            const int32_t pg_first = __builtin_amdgcn_readfirstlane(load_page(0));
            int32_t pg_next = load_page(1);
            if (n_units > 0) issue_loads(0, pg_first);
            for (int it = -2; it < n_units; ++it) {
                if (it + 2 < n_units) commit_loads((it + 2) & 1);
                const int32_t pg_s = __builtin_amdgcn_readfirstlane(pg_next);
                pg_next = load_page(it + 4);
                if (it + 3 < n_units) issue_loads(it + 3, pg_s);
                if (it + 1 >= 0 && it + 1 < n_units) dequant_unit((it + 1) & 1, (it + 1) & 1);
                __syncthreads();
            }
            return;  // the epilogue has no workgroup barrier
        }
        __builtin_amdgcn_s_setprio(1);  // (measured: none 8.20 ms, the multiplying waves 8.04, the dequantising waves 8.65)
        for (int it = -2; it < n_units; ++it) {
            if (it >= 0) {
                const int t0 = (u_first + it) * kUnit;
                compute_unit(it & 1, t0, !(t0 >= i_lo && t0 + kUnit - 1 <= i_hi));
            }
            __syncthreads();
        }
        __builtin_amdgcn_s_setprio(0);
    } else {
        const int32_t pg_first = __builtin_amdgcn_readfirstlane(load_page(0));
        int32_t pg_next = load_page(1);
        if (n_units > 0) issue_loads(0, pg_first);
        for (int it = -2; it < n_units; ++it) {
            // commit unit it + 2 (loaded during the previous iteration), then start unit it + 3
            if (it + 2 < n_units) commit_loads((it + 2) & 1);
            // The page id of unit it + 4 is requested BEFORE the key loads of unit it + 3: a
            // write to its register after them would have to wait for all of them to return.
            const int32_t pg_s = __builtin_amdgcn_readfirstlane(pg_next);
            pg_next = load_page(it + 4);
            if (it + 3 < n_units) issue_loads(it + 3, pg_s);
            // TQ4 pages: the two waves of a SIMD (w and w + 4) take the two halves of an iteration in
            // opposite order, so that one dequantises (table reads and VALU) while the other
            // multiplies.  Both orders are valid between two barriers: the dequantiser writes buffer
            // (it + 1) & 1, the MFMAs read buffer it & 1.  (With the cheaper dequantisers of the other
            // formats the same order in all waves measured faster.)
            const bool compute_first = TQ4F && wave >= 4;  // wave-uniform
            // (TQ4: while a wave multiplies it is the one the SIMD serves first, so its MFMAs go out as
            // soon as their operands are there and the other wave's dequantiser fills the gaps: -4 %.
            // The other formats, whose waves all run the same order, measured 5 % slower with it.)
            if (compute_first && it >= 0) {
                const int t0 = (u_first + it) * kUnit;
                __builtin_amdgcn_s_setprio(1);
                compute_unit(it & 1, t0, !(t0 >= i_lo && t0 + kUnit - 1 <= i_hi));
                __builtin_amdgcn_s_setprio(0);
            }
            if (it + 1 >= 0 && it + 1 < n_units) {
                if constexpr (K16) {
                    dequant_unit_16((it + 1) & 1, (it + 1) & 1, (u_first + it + 1) * kUnit);
                } else if constexpr (Q8) {
                    dequant_unit_q8((it + 1) & 1, (it + 1) & 1, (u_first + it + 1) * kUnit);
                } else if constexpr (FP8) {
                    dequant_unit_fp8((it + 1) & 1, (it + 1) & 1, (u_first + it + 1) * kUnit);
                } else {
                    dequant_unit((it + 1) & 1, (it + 1) & 1);
                }
            }
            if (!compute_first && it >= 0) {
                const int t0 = (u_first + it) * kUnit;
                if constexpr (TQ4F) __builtin_amdgcn_s_setprio(1);
                compute_unit(it & 1, t0, !(t0 >= i_lo && t0 + kUnit - 1 <= i_hi));
                if constexpr (TQ4F) __builtin_amdgcn_s_setprio(0);
            }
            __syncthreads();
        }
    }

    // ---- epilogue: normalise, transpose through LDS, rotate back, store ----
    l_run = sum_over_rows(l_run);
    float* reg = reinterpret_cast<float*>(smem) + wave * 16 * 260;
    const float inv = SPLIT ? 1.0f : (l_run > 0.f ? (TQ4F ? kLutInvGain : 1.0f) / l_run : 0.f);
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
        if constexpr (SPLIT) {
            // un-normalised, rotated, still carrying the table gain: the merge kernel finishes
            const size_t row = (size_t)(tok0 + t) * P.num_q_heads + (size_t)(q_head_base + a);
            const size_t prow = row * P.part_stride + (size_t)(P.pf_slot_base + part_x);
            *reinterpret_cast<f4*>(P.part_acc + prow * kHeadDim + 4 * lane) = x;
            const float m_c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(m_run), c));
            const float l_c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(l_run), c));
            if (lane == 0) *reinterpret_cast<f4*>(P.part_ml + prow * 4) = f4{m_c, l_c, (float)P.pf_split, 0.f};
            continue;
        }
        if (rot_out) {  // values stored rotated: rotate the finished row back
            wht256_wave(o, lane);
#pragma unroll
            for (int k = 0; k < 4; ++k) o[k] = apply_sign(o[k], 4 * lane + k);
        }
        const size_t row = (size_t)(tok0 + t) * P.num_q_heads + (size_t)(q_head_base + a);
        store_out_row<TQ>(P, row, lane, o);
    }
}

}  // namespace w34
