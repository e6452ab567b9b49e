// Paged GQA decode / verify attention over pages whose rows are read as stored: 16-bit rows
// (FP16 or BF16 storage, identity transform) and the 8-bit rows FP8-E4M3-256 and Q8_0-64, for
// gfx950.  Same work decomposition, chunk geometry, wave merge and split-K partial format as
// the TQ4 kernel in paged_attn.hip (which includes this file); only the per-unit body differs:
//   * a 32-token unit is processed as two 16-token halves; the wave copies the 16 K rows and
//     16 V rows of a half into its private LDS area.  16-bit rows (512 B) get a row stride of
//     544 bytes (keys) or 576 bytes (values), the strides at which their 128-bit operand reads
//     are conflict-free; 8-bit rows (264 B / 272 B, codes and their fp32 block scales) 272 bytes;
//   * S^T = K Q^T: A operand = 16 K rows read from LDS, B operand = the query rows, loaded
//     once in MFMA layout.  8-bit codes are widened to fp16 in registers (exact) and the fp32
//     block scales are applied to per-block partial scores, so K is never rounded;
//   * O^T += V^T P^T with 16x16x16 MFMAs: each lane reads the 8-element slice of its 4 tokens
//     and transposes the 4x8 block in registers.  8-bit V is dequantised to fp16(d * code)
//     on the way, which is what the reference stages (op_paged_attn.cu:59-105);
//   * BF16 storage: P is split into a bf16 high and low part (two MFMAs) so that the 8-bit
//     mantissa of bf16 does not limit the accuracy of the weighted sum;
//   * 8-bit layers may be stored rotated (WHT256 transform): the query rows are then rotated
//     once per tile and the output is rotated back once (op_kv_cache.cu:443-451,763-783).
// Replaces paged_attention_gqa_bf16_kernel (op_kv_cache.cu:873-1168) and the FP16, Q8_0 and
// FP8 branches of paged_attention_gqa_mma_f16_kernel (op_paged_attn.cu:186-588).
#pragma once

namespace w34 {

typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef short s4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));

constexpr int kKv16Waves = 8;
// LDS row strides of 16-bit rows (512 B).  The key operand reads are 128 bits at (row n, piece b)
// for 16 rows x 4 pieces per instruction, the value reads 128 bits at (row 4 b + i, piece n): a
// probe of those two patterns measures the rate of a contiguous read at 544 / 608 / 672 bytes for
// the first and at 576 bytes for the second, 40 % less at 528.
constexpr int kKv16RowStride = 544;                      // key rows
constexpr int kKv16VRowStride = 576;                     // value rows
constexpr int kKv8RowStride = 272;                       // bytes: Q8_0 rows as stored, FP8 rows + 8 pad
constexpr int kKv16Stage = 16 * (kKv16RowStride + kKv16VRowStride);  // K half + V half: 17920 B per wave
constexpr int kKv16ColStride = 264;                      // dwords per column of a merge region (see kMergeColStride)
// byte offset of the (m, l) exchange table: behind both the staging areas and the merge regions
__host__ __device__ constexpr int kv16_ml_offset(int nt) {
    const int loop_bytes = kKv16Waves * kKv16Stage;
    const int region_bytes = kKv16Waves * (nt * 16 * kKv16ColStride) * 4;
    return loop_bytes > region_bytes ? loop_bytes : region_bytes;
}
__host__ __device__ constexpr int kv16_smem_bytes(int nt) {
    return kv16_ml_offset(nt) + (kKv16Waves + 1) * nt * 16 * 2 * 4 + 256;
}

// four E4M3 codes -> four fp16 values (exact)
__device__ __forceinline__ void fp8x4_to_h4(uint32_t w, uint32_t& lo, uint32_t& hi) {
    lo = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false));
    hi = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true));
}
// four int8 codes -> four fp16 values (exact): 0x6400 | (q + 128) is 1024 + (q + 128) in fp16
__device__ __forceinline__ void i8x4_to_h4(uint32_t w, uint32_t& lo, uint32_t& hi) {
    const uint32_t u = w ^ 0x80808080u;
    const h2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
    const h2 a = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u)) - bias;
    const h2 c = __builtin_bit_cast(h2, __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u)) - bias;
    lo = __builtin_bit_cast(uint32_t, a);
    hi = __builtin_bit_cast(uint32_t, c);
}
// four 8-bit codes -> fp32
template <bool FP8>
__device__ __forceinline__ void codes4_to_f32(uint32_t w, float (&f)[4]) {
    if constexpr (FP8) {
        const f2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
        const f2 c = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
        f[0] = a.x, f[1] = a.y, f[2] = c.x, f[3] = c.y;
    } else {
        f[0] = (float)(int8_t)(w & 0xFFu);
        f[1] = (float)(int8_t)((w >> 8) & 0xFFu);
        f[2] = (float)(int8_t)((w >> 16) & 0xFFu);
        f[3] = (float)(int8_t)(w >> 24);
    }
}

template <bool IS_BF16>
__device__ __forceinline__ f4 mfma_x32(u4 a, u4 b, f4 c) {
    if constexpr (IS_BF16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    }
}
template <bool IS_BF16>
__device__ __forceinline__ f4 mfma_x16(u2v a, u2v b, f4 c) {
    if constexpr (IS_BF16) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s4, a), __builtin_bit_cast(s4, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h4, a), __builtin_bit_cast(h4, b), c, 0, 0, 0);
    }
}

// KVF is the storage format of both slabs.  16-bit pages: TQ doubles as the storage type (F16
// query/output over FP16 pages, BF16 over BF16 pages).  8-bit pages: the MFMAs run in fp16 and
// a BF16 query is converted once.
// BAL: the tile and its unit range come from `item` (balanced decode, see bal_for_each_piece)
// instead of blockIdx.
// VRES (8-bit rows stored rotated): the value operand fp16(d * code) is followed by a second
// operand holding its rounding residual, and every P V tile takes a second MFMA.  A scale block
// of a rotated row with large entries holds few distinct codes, so part of the fp16 rounding of
// d * code is common to the block, and the inverse rotation of the finished row would gather
// that common part into a single channel.
// HD: the head dimension, 256 or -- 16-bit rows only (op_kv_cache.cu:1227) -- 128.  At 128 a row is
// one 128-element half: four QK operands instead of eight, eight value tiles instead of sixteen,
// and lanes 0-31 carry a finished row.  The split-K partial records keep their 256-float stride.
template <typename TQ, int NT, int KVF, bool BAL, bool VRES = false, bool STREAM = BAL, int HD = kHeadDim>
__device__ __forceinline__ void rows_tile(const AttnParams& P, uint8_t* smem, const BalItem& item) {
    static_assert(!VRES || KVF == WARP34_KV_FORMAT_FP8_E4M3 || KVF == WARP34_KV_FORMAT_Q8_0, "residual operand: 8-bit rows");
    constexpr bool K8 = KVF == WARP34_KV_FORMAT_FP8_E4M3 || KVF == WARP34_KV_FORMAT_Q8_0;
    static_assert(HD == 256 || (HD == 128 && !K8), "head dimension 128: 16-bit rows only");
    constexpr int kM = HD / 32;   // QK operands (32 elements each) per row
    constexpr int kH = HD / 128;  // 128-element halves of a row
    constexpr bool FP8 = KVF == WARP34_KV_FORMAT_FP8_E4M3;
    static_assert(K8 || KVF == TQ::kStorageFormat, "16-bit pages are read in the query type");
    constexpr bool IS_BF16 = !K8 && TQ::kStorageFormat == WARP34_KV_FORMAT_BF16;
    constexpr bool Q_BF16 = TQ::kStorageFormat == WARP34_KV_FORMAT_BF16;
    constexpr int kWaves = kKv16Waves;
    // LDS row strides (16-bit rows of 256 bytes: the row plus 32 / 64 bytes, the same bank pattern as 544 / 576)
    constexpr int kRowStride = K8 ? kKv8RowStride : (HD == 256 ? kKv16RowStride : 2 * HD + 32);    // key rows
    constexpr int kVRowStride = K8 ? kKv8RowStride : (HD == 256 ? kKv16VRowStride : 2 * HD + 64);  // value rows
    constexpr int kRowBytes = K8 ? (FP8 ? 264 : 272) : 2 * HD;       // row in memory

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int b = lane >> 4;
    const warp34_kv_layer_layout& L = P.L;
    const warp34_attention_batch& B = P.B;

    const int tile_z = BAL ? item.req : (int)blockIdx.z;  // tile index (see locate_tile)
    const int kv_sub = (int)blockIdx.y;
    const int kv_head = fast_div(kv_sub, P.q_subgroups);
    const int q_head_base = kv_head * P.gqa + (kv_sub - kv_head * P.q_subgroups) * P.q_group;
    const int chunk = BAL ? 0 : (int)blockIdx.x;

    // query rows in MFMA B layout straight from global memory: lane (n, b) holds
    // Q[column n][32 m + 8 b .. + 7] for m = 0..7 (dead columns are zeroed below).  The first
    // token of the tile is guessed so that these loads overlap the lookup; a wrong guess is
    // corrected after it.
    const int tok_guess = BAL ? item.rq_start
                              : min(P.tiles_by_request ? tile_z : tile_z * P.tok_tile, B.total_tokens - 1);
    u4 bq[NT][kM];
    auto load_q = [&](int tokbase) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int col = nt * 16 + n;
            const int t = fast_div(col, P.q_group);
            const int a = col - t * P.q_group;
            const int tok = min(tokbase + t, B.total_tokens - 1);
            const uint16_t* qrow = P.q + ((size_t)tok * P.num_q_heads + (size_t)(q_head_base + a)) * HD;
#pragma unroll
            for (int m = 0; m < kM; ++m) bq[nt][m] = *reinterpret_cast<const u4*>(qrow + 32 * m + 8 * b);
        }
    };
    // Rotated K rows: the query rows go through sign + WHT256 first (one row per wave at a time,
    // element e = 4 lane + k), are staged as fp16 in the still unused staging area and read
    // back in MFMA layout.
    constexpr int kQStride = 264;  // halves
    auto load_q_rotated = [&](int tokbase) {
        if constexpr (HD != 256) return;
        _Float16* qlds = reinterpret_cast<_Float16*>(smem);
        for (int col = wave; col < 16 * NT; col += kWaves) {
            const int t = fast_div(col, P.q_group);
            const int a = col - t * P.q_group;
            const int tok = min(tokbase + t, B.total_tokens - 1);
            const uint16_t* qrow = P.q + ((size_t)tok * P.num_q_heads + (size_t)(q_head_base + a)) * kHeadDim;
            const uint2 raw = *reinterpret_cast<const uint2*>(qrow + 4 * lane);
            float v[4] = {TQ::to_f32((uint16_t)(raw.x & 0xFFFFu)), TQ::to_f32((uint16_t)(raw.x >> 16)),
                          TQ::to_f32((uint16_t)(raw.y & 0xFFFFu)), TQ::to_f32((uint16_t)(raw.y >> 16))};
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = apply_sign(v[k], 4 * lane + k);
            wht256_wave(v, lane);
            uint2 packed;
            packed.x = pack_h2(v[0], v[1]);
            packed.y = pack_h2(v[2], v[3]);
            *reinterpret_cast<uint2*>(qlds + col * kQStride + 4 * lane) = packed;
        }
        __syncthreads();
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int m = 0; m < kM; ++m)
                bq[nt][m] = *reinterpret_cast<const u4*>(qlds + (nt * 16 + n) * kQStride + 32 * m + 8 * b);
        __syncthreads();  // the staging area is reused by the K/V rows
    };
    const bool rot_q = K8 && P.rot_q != 0;  // workgroup-uniform
    if (!rot_q) load_q(tok_guess);

    // Speculative block-table load, in flight together with the lookup: it assumes that the
    // request's length is the host's bound max_seq_len.  A wrong guess is fetched again below,
    // so it changes the latency only, never the result.
    int spec_slot_base = -1, spec_vec = -1;
    if constexpr (BAL) {
        // the piece's first unit is known: its block-table slice is requested with the query rows
        spec_slot_base = div_block(item.u_begin * kUnit, P);
        const int slot = spec_slot_base + lane;
        if (slot < B.max_blocks_per_req) spec_vec = B.block_tables[(size_t)tile_z * B.max_blocks_per_req + slot];
    } else if (P.tiles_by_request && B.sliding_window <= 0 && B.max_seq_len > 0) {
        spec_slot_base = div_block(chunk * P.spec_upc * kUnit, P);
        const int slot = spec_slot_base + lane;
        if (slot < B.max_blocks_per_req)
            spec_vec = B.block_tables[(size_t)tile_z * B.max_blocks_per_req + slot];
    }
    TileInfo ti;
    if constexpr (BAL) {
        ti = TileInfo{true, item.req, item.rq_start, item.rq_end, item.seq_after, item.ctx_before, 0};
    } else {
        ti = locate_tile(P, tile_z, lane);
    }
    if (!ti.hit) return;  // no such tile, empty or masked request: outputs untouched
    const int req = ti.req, rq_start = ti.rq_start, rq_end = ti.rq_end;
    const int seq_after = ti.seq_after, ctx_before = ti.ctx_before;
    const int tok0 = rq_start + ti.tile_in_req * P.tok_tile;
    if (rot_q) {
        load_q_rotated(tok0);  // every wave of the workgroup takes the same path up to here
    } else {
        if (tok0 != tok_guess) load_q(tok0);  // wave-uniform, rare
        if constexpr (K8 && Q_BF16) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int m = 0; m < kM; ++m)
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const uint32_t w = bq[nt][m][k];
                        bq[nt][m][k] = pack_h2(BF16::to_f32((uint16_t)(w & 0xFFFFu)), BF16::to_f32((uint16_t)(w >> 16)));
                    }
        }
    }
    bool tok_ok[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int tok = tok0 + fast_div(nt * 16 + n, P.q_group);
        tok_ok[nt] = tok < B.total_tokens &&
                     (B.valid_token_mask == nullptr || B.valid_token_mask[min(tok, B.total_tokens - 1)] != 0);
    }
    int tile_tokens = rq_end - tok0;
    if (tile_tokens > P.tok_tile) tile_tokens = P.tok_tile;

    // Column info (per lane = per query column: visible key range; tile-wide: union and intersection
    // of the ranges).  Without a token mask and a window the tile-wide values follow from scalars
    // and the per-lane part waits until the first rows have been requested (see the TQ4 kernel).
    int col_lo[NT], col_hi[NT];
    bool col_ok[NT];
    int u_lo = 0x7fffffff, u_hi = -1;
    int i_lo = 0, i_hi = 0x7fffffff;
    uint32_t ok_mask[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        col_lo[nt] = 0;
        col_hi[nt] = -1;
        col_ok[nt] = false;
        ok_mask[nt] = 0u;
    }
    const bool simple = B.valid_token_mask == nullptr && B.sliding_window <= 0;
    auto column_info = [&](bool accumulate) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int col = nt * 16 + n;
            const int t = fast_div(col, P.q_group);
            const int tok = tok0 + t;
            const bool ok = t < tile_tokens && tok_ok[nt];
            const int q_off = tok - rq_start;
            int mx = (B.mask_mode == WARP34_ATTN_MASK_NONCAUSAL_WINDOW) ? seq_after - 1 : ctx_before + q_off;
            if (mx >= seq_after) mx = seq_after - 1;
            int mn = 0;
            if (B.sliding_window > 0) mn = max(0, ctx_before + q_off - B.sliding_window + 1);
            col_ok[nt] = ok;
            col_lo[nt] = ok ? mn : 0;
            col_hi[nt] = ok ? mx : -1;
            if (ok) {
                if (accumulate) {
                    i_lo = max(i_lo, mn);
                    i_hi = min(i_hi, mx);
                    if (mn <= mx) {
                        u_lo = min(u_lo, mn);
                        u_hi = max(u_hi, mx);
                    }
                }
            } else {
#pragma unroll
                for (int m = 0; m < kM; ++m) bq[nt][m] = u4{0u, 0u, 0u, 0u};
            }
            ok_mask[nt] = (uint32_t)(__ballot(ok) & 0xFFFFull);
        }
    };
    if (simple) {
        if (tok0 >= B.total_tokens) return;  // no live column
        const int q_off0 = tok0 - rq_start;
        const bool window = B.mask_mode == WARP34_ATTN_MASK_NONCAUSAL_WINDOW;
        int hi_first = window ? seq_after - 1 : ctx_before + q_off0;
        int hi_last = window ? seq_after - 1 : ctx_before + q_off0 + tile_tokens - 1;
        if (hi_first >= seq_after) hi_first = seq_after - 1;
        if (hi_last >= seq_after) hi_last = seq_after - 1;
        u_lo = 0;
        u_hi = hi_last >= 0 ? hi_last : -1;
        i_lo = 0;
        i_hi = hi_first;
    } else {
        column_info(true);
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
            u_lo = min(u_lo, __shfl_xor(u_lo, off, 64));
            u_hi = max(u_hi, __shfl_xor(u_hi, off, 64));
            i_lo = max(i_lo, __shfl_xor(i_lo, off, 64));
            i_hi = min(i_hi, __shfl_xor(i_hi, off, 64));
        }
        uint32_t any = 0;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) any |= ok_mask[nt];
        if (any == 0u) return;
    }
    if (u_hi < 0) u_lo = 0;
    u_lo = __builtin_amdgcn_readfirstlane(u_lo);
    u_hi = __builtin_amdgcn_readfirstlane(u_hi);
    i_lo = __builtin_amdgcn_readfirstlane(i_lo);
    i_hi = __builtin_amdgcn_readfirstlane(i_hi);

    ChunkGeom g;
    int cu_first, cu_end;
    if constexpr (BAL) {
        // the plan counted the units of [0, u_hi]: the batch has no window and no token mask
        g = ChunkGeom{0, (u_hi >> 5) + 1, 0, item.n_chunks};
        cu_first = item.u_begin;
        cu_end = item.u_end;
    } else {
        if (u_lo == 0 && B.max_seq_len > 0 && u_hi == B.max_seq_len - 1) {
            g = ChunkGeom{0, P.spec_units, P.spec_upc, P.spec_chunks};  // as long as the host's bound
        } else {
            g = chunk_geom(u_lo, u_hi, P.max_chunks, P.min_upc);
        }
        if (chunk >= g.n_chunks) return;
        cu_first = g.u_first + chunk * g.upc;
        cu_end = cu_first + g.upc;
        if (cu_end > g.u_first + g.n_units) cu_end = g.u_first + g.n_units;
    }

    const uint8_t* k_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.k_base) +
                            (size_t)kv_head * L.k_head_stride_bytes;
    const uint8_t* v_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.v_base) +
                            (size_t)kv_head * L.v_head_stride_bytes;
    uint8_t* stage = smem + wave * kKv16Stage;  // [K rows 0..15][V rows 0..15], kRowStride each
    const int32_t* req_blocks = B.block_tables + (size_t)req * B.max_blocks_per_req;
    int slot_base = div_block(cu_first * kUnit, P);
    int page_vec;
    auto load_page_vec = [&]() {
        const int slot = slot_base + lane;
        page_vec = slot < B.max_blocks_per_req ? req_blocks[slot] : -1;
    };

    // A half = 16 consecutive tokens: 16 K rows and 16 V rows, each run contiguous inside one
    // page (8 KiB of 16-bit rows, 4224 B of FP8 rows, 4352 B of Q8_0 rows).  It is fetched as
    // 16-byte pieces c = lane + 64 i.
    constexpr int kPieces = 16 * kRowBytes / 16;        // 512, 264 or 272 (256 at head dimension 128)
    constexpr int kLoads = (kPieces + 63) / 64;         // 8 or 5 (4)
    u4 pf[2 * kLoads];
    auto issue_half = [&](int hidx) {  // hidx = 2 * unit + half
        const int pos = hidx * 16;
        const int page_slot = div_block(pos, P);
        const int in_page = pos - page_slot * L.block_size;
        int rel = page_slot - slot_base;
        if (rel >= 64) {
            slot_base = page_slot;
            load_page_vec();
            rel = 0;
        }
        const int32_t pg = __builtin_amdgcn_readlane(page_vec, rel);
        const bool live = pos <= u_hi && pos + 15 >= u_lo && pg >= 0;
        const uint8_t* kp = k_base + (live ? (size_t)pg * L.k_page_stride_bytes + (size_t)in_page * L.k_token_stride_bytes : 0);
        const uint8_t* vp = v_base + (live ? (size_t)pg * L.v_page_stride_bytes + (size_t)in_page * L.v_token_stride_bytes : 0);
        // STREAM: every key is read by exactly one workgroup (decode steps: no request has more
        // than one tile), and the loads carry the non-temporal hint, which is worth 8 to 13 % on a
        // plain streaming read of HBM and 3 to 8 % here.  Tiles that share a request's keys
        // (verify, prefill through this kernel) keep ordinary loads: with the hint their batches
        // measure 7 to 22 % slower, the lines are gone when the next tile asks for them.
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            // pieces beyond the run (last, partial round of the 8-bit formats) re-read piece 0
            const int c = (kPieces % 64 == 0 || lane + 64 * i < kPieces) ? lane + 64 * i : 0;
            if constexpr (STREAM) {
                pf[i] = __builtin_nontemporal_load((global_cu4*)(kp + 16 * c));
                pf[kLoads + i] = __builtin_nontemporal_load((global_cu4*)(vp + 16 * c));
            } else {
                pf[i] = *(global_cu4*)(kp + 16 * c);
                pf[kLoads + i] = *(global_cu4*)(vp + 16 * c);
            }
        }
    };
    // rows outside [u_lo, u_hi] are stored as zeros: unwritten pool memory may hold NaN
    // patterns, and 0 * NaN would poison the P V product
    auto commit_half = [&](int hidx) {
        const int pos0 = hidx * 16;
        const bool edge = pos0 < u_lo || pos0 + 15 > u_hi;
        uint8_t* k_rows = stage;
        uint8_t* v_rows = stage + 16 * kRowStride;
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            const int c = lane + 64 * i;
            if (kPieces % 64 != 0 && c >= kPieces) break;
            u4 kv = pf[i], vv = pf[kLoads + i];
            if constexpr (FP8) {
                // 264-byte rows: the two 8-byte halves of a piece may belong to different rows
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
                    const unsigned sub = 2u * (unsigned)c + hf;
                    const unsigned row = sub / 33u, col = sub - row * 33u;
                    u2v k8 = hf ? u2v{kv[2], kv[3]} : u2v{kv[0], kv[1]};
                    u2v v8 = hf ? u2v{vv[2], vv[3]} : u2v{vv[0], vv[1]};
                    if (edge && !(pos0 + (int)row >= u_lo && pos0 + (int)row <= u_hi)) {
                        k8 = u2v{0u, 0u};
                        v8 = u2v{0u, 0u};
                    }
                    *reinterpret_cast<u2v*>(k_rows + row * kRowStride + 8 * col) = k8;
                    *reinterpret_cast<u2v*>(v_rows + row * kVRowStride + 8 * col) = v8;
                }
            } else {
                constexpr int kPiecesPerRow = kRowBytes / 16;  // 32 or 17
                const int row = (int)((unsigned)c / (unsigned)kPiecesPerRow);
                const int col = c - row * kPiecesPerRow;
                if (edge) {
                    const bool vis = pos0 + row >= u_lo && pos0 + row <= u_hi;
                    if (!vis) {
                        kv = u4{0u, 0u, 0u, 0u};
                        vv = u4{0u, 0u, 0u, 0u};
                    }
                }
                *reinterpret_cast<u4*>(k_rows + row * kRowStride + 16 * col) = kv;
                *reinterpret_cast<u4*>(v_rows + row * kVRowStride + 16 * col) = vv;
            }
        }
    };

    f4 o_acc[NT][kH][8];
    float m_run[NT], l_run[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        m_run[nt] = kNegBig;
        l_run[nt] = 0.f;
#pragma unroll
        for (int h = 0; h < kH; ++h)
#pragma unroll
            for (int j = 0; j < 8; ++j) o_acc[nt][h][j] = f4{0.f, 0.f, 0.f, 0.f};
    }
    const float score_scale = B.sm_scale * kLog2e;

    auto process_half = [&](int pos0, const bool MASKED) {
        const uint8_t* k_rows = stage;
        const uint8_t* v_rows = stage + 16 * kRowStride;
        // ---- S^T = K Q^T: A row n = token n of the half ----
        f4 s_acc[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) s_acc[nt] = f4{0.f, 0.f, 0.f, 0.f};
        // V operands of the 16 P V MFMAs: a_v[h][j] = element 128 h + 8 n + j of tokens 4b..4b+3
        u2v a_v[kH][8];
        u2v a_vr[VRES ? 2 : 1][VRES ? 8 : 1];  // residuals of a_v
        if constexpr (K8 && HD == 256) {
            // Codes of row n, elements 32 m + 8 b .. + 7, widened to fp16; one partial score per
            // scale block (FP8: 2 blocks of 128 = m / 4; Q8_0: 4 blocks of 64 = m / 2), combined
            // with the fp32 scales of this lane's 4 tokens.
            constexpr int kBlocks = FP8 ? 2 : 4;
            constexpr int kMPerBlock = 8 / kBlocks;
            u4 ka[8];
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                const int off = FP8 ? 32 * m + 8 * b : 68 * (m >> 1) + 4 + 32 * (m & 1) + 8 * b;
                const uint32_t* src = reinterpret_cast<const uint32_t*>(k_rows + n * kRowStride + off);
                const uint32_t w0 = src[0], w1 = src[1];
                uint32_t h0, h1, h2_, h3;
                if constexpr (FP8) {
                    fp8x4_to_h4(w0, h0, h1);
                    fp8x4_to_h4(w1, h2_, h3);
                } else {
                    i8x4_to_h4(w0, h0, h1);
                    i8x4_to_h4(w1, h2_, h3);
                }
                ka[m] = u4{h0, h1, h2_, h3};
            }
            float dk[4][kBlocks];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int kb = 0; kb < kBlocks; ++kb)
                    dk[i][kb] = *reinterpret_cast<const float*>(k_rows + (4 * b + i) * kRowStride +
                                                                (FP8 ? 256 + 4 * kb : 68 * kb));
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int kb = 0; kb < kBlocks; ++kb) {
                    f4 part = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int mm = 0; mm < kMPerBlock; ++mm)
                        part = mfma_x32<false>(ka[kb * kMPerBlock + mm], bq[nt][kb * kMPerBlock + mm], part);
#pragma unroll
                    for (int i = 0; i < 4; ++i) s_acc[nt][i] += dk[i][kb] * part[i];
                }
            }
            // V: fp16(d * code), the value the reference stages (op_paged_attn.cu:59-105)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float vf[4][8];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint8_t* vrow = v_rows + (4 * b + i) * kVRowStride;
                    const int blk = 2 * h + (n >> 3);  // Q8_0 block of element 128 h + 8 n
                    const int off = FP8 ? 128 * h + 8 * n : 68 * blk + 4 + 8 * (n & 7);
                    const uint32_t* src = reinterpret_cast<const uint32_t*>(vrow + off);
                    const float d = *reinterpret_cast<const float*>(vrow + (FP8 ? 256 + 4 * h : 68 * blk));
                    float f0[4], f1[4];
                    codes4_to_f32<FP8>(src[0], f0);
                    codes4_to_f32<FP8>(src[1], f1);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        vf[i][k] = d * f0[k];
                        vf[i][4 + k] = d * f1[k];
                    }
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    if constexpr (VRES) {
                        uint32_t hi0, lo0, hi1, lo1;
                        split_h2(vf[0][j], vf[1][j], hi0, lo0);
                        split_h2(vf[2][j], vf[3][j], hi1, lo1);
                        a_v[h][j] = u2v{hi0, hi1};
                        a_vr[h][j] = u2v{lo0, lo1};
                    } else {
                        a_v[h][j] = u2v{pack_h2(vf[0][j], vf[1][j]), pack_h2(vf[2][j], vf[3][j])};
                    }
                }
            }
        } else {
            u4 ka[kM];
#pragma unroll
            for (int m = 0; m < kM; ++m)
                ka[m] = *reinterpret_cast<const u4*>(k_rows + n * kRowStride + 64 * m + 16 * b);
#pragma unroll
            for (int m = 0; m < kM; ++m)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) s_acc[nt] = mfma_x32<IS_BF16>(ka[m], bq[nt][m], s_acc[nt]);

            // V slices of this lane's 4 tokens (rows 4b..4b+3), both halves of the head dim; the
            // 4x8 block of 16-bit values is transposed in registers
#pragma unroll
            for (int h = 0; h < kH; ++h) {
                u4 vr[4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    vr[i] = *reinterpret_cast<const u4*>(v_rows + (4 * b + i) * kVRowStride + 256 * h + 16 * n);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    // 16-bit element j of the four token slices -> (t0,t1), (t2,t3)
                    const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
                    a_v[h][j] = u2v{__builtin_amdgcn_perm(vr[1][j >> 1], vr[0][j >> 1], sel),
                                    __builtin_amdgcn_perm(vr[3][j >> 1], vr[2][j >> 1], sel)};
                }
            }
        }

        // ---- online softmax over this lane's 4 tokens ----
        u2v pb_hi[NT], pb_lo[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            // (the MASKED tests sit outside the unrolled loops: one wave-uniform branch per block)
            float sc[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) sc[i] = s_acc[nt][i] * score_scale;
            if (MASKED) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int pos = pos0 + 4 * b + i;
                    const bool vis = col_ok[nt] && pos >= col_lo[nt] && pos <= col_hi[nt];
                    sc[i] = vis ? sc[i] : kNegBig;
                }
            }
            float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
            mx = max_over_rows(mx);
            const float m_new = fmaxf(m_run[nt], mx);
            const float alpha = __builtin_amdgcn_exp2f(m_run[nt] - m_new);
            m_run[nt] = m_new;
            float p[4];
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = __builtin_amdgcn_exp2f(sc[i] - m_new);
            if (MASKED) {
#pragma unroll
                for (int i = 0; i < 4; ++i) p[i] = sc[i] > 0.5f * kNegBig ? p[i] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) psum += p[i];
            l_run[nt] = l_run[nt] * alpha + psum;
            if (__ballot(alpha != 1.0f) != 0ull) {
#pragma unroll
                for (int h = 0; h < kH; ++h)
#pragma unroll
                    for (int j = 0; j < 8; ++j) o_acc[nt][h][j] *= alpha;
            }
            if constexpr (IS_BF16) {
                uint32_t hb[4], lb[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    hb[i] = BF16::from_f32(p[i]);
                    lb[i] = BF16::from_f32(p[i] - BF16::to_f32((uint16_t)hb[i]));
                }
                pb_hi[nt] = u2v{hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16)};
                pb_lo[nt] = u2v{lb[0] | (lb[1] << 16), lb[2] | (lb[3] << 16)};
            } else {
                pb_hi[nt] = u2v{pack_h2(p[0], p[1]), pack_h2(p[2], p[3])};
                pb_lo[nt] = u2v{0u, 0u};
            }
        }

        // ---- O^T += V^T P^T: row r = n of MFMA (h, j) is head dimension 128 h + 8 n + j ----
#pragma unroll
        for (int h = 0; h < kH; ++h) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const u2v a = a_v[h][j];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    o_acc[nt][h][j] = mfma_x16<IS_BF16>(a, pb_hi[nt], o_acc[nt][h][j]);
                    if constexpr (IS_BF16) o_acc[nt][h][j] = mfma_x16<IS_BF16>(a, pb_lo[nt], o_acc[nt][h][j]);
                }
            }
            if constexpr (VRES) {
#pragma unroll
                for (int j = 0; j < 8; ++j)
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
                        o_acc[nt][h][j] = mfma_x16<false>(a_vr[h][j], pb_hi[nt], o_acc[nt][h][j]);
            }
        }
    };

    // halves of this wave's units, in order; the next half is in flight while one is processed
    int unit = cu_first + wave;
    if (slot_base == spec_slot_base) {
        page_vec = spec_vec;
    } else {
        load_page_vec();
    }
    // Units are dealt by a fixed rule (the result must not depend on timing): round robin with
    // one extra unit for waves 0-3 after every eight rounds, because each SIMD serves its older
    // wave first (see the TQ4 kernel).
    auto nth_unit = [&](int j) -> int {
        if (wave < 4) {
            const int g = j / 9, k = j - 9 * g;
            return cu_first + 68 * g + (k < 8 ? 8 * k + wave : 64 + wave);
        }
        return cu_first + 68 * (j >> 3) + 8 * (j & 7) + wave;
    };
    static_assert(kWaves == 8, "unit deal assumes two waves per SIMD");
    int hidx = 2 * unit, unit_no = 0;
    // The query operands are touched again after the first rows have been requested (dead columns
    // are zeroed).  Loads return in order: a wait for them placed behind the row loads would wait
    // for the rows too, so the compiler is made to finish them here, where they have long landed.
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int m = 0; m < kM; ++m)
            asm volatile("" ::"v"(bq[nt][m][0]), "v"(bq[nt][m][1]), "v"(bq[nt][m][2]), "v"(bq[nt][m][3]));
    issue_half(hidx);
    if (simple) column_info(false);
    while (unit < cu_end) {
        commit_half(hidx);
        int next_h = hidx + 1, next_unit = unit;
        if (next_h & 1) {
            // second half of the same unit
        } else {
            next_unit = nth_unit(++unit_no);
            next_h = 2 * next_unit;
        }
        if (next_unit < cu_end) issue_half(next_h);
        const int pos0 = hidx * 16;
        if (pos0 <= u_hi) process_half(pos0, !(pos0 >= i_lo && pos0 + 15 <= i_hi));
        hidx = next_h;
        unit = next_unit;
    }

#pragma unroll
    for (int nt = 0; nt < NT; ++nt) l_run[nt] = sum_over_rows(l_run[nt]);

    // ---- merge of the waves' states (same scheme and region layout as the TQ4 kernel) ----
    constexpr int kColStride = kKv16ColStride;
    constexpr int kRegion = NT * 16 * kColStride;
    float* mlbuf = reinterpret_cast<float*>(smem + kv16_ml_offset(NT));
    static_assert(kv16_ml_offset(NT) >= kWaves * kRegion * 4 && kv16_ml_offset(NT) >= kWaves * kKv16Stage,
                  "(m, l) table must not alias live LDS");
    if (b == 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            mlbuf[(wave * NT * 16 + nt * 16 + n) * 2 + 0] = m_run[nt];
            mlbuf[(wave * NT * 16 + nt * 16 + n) * 2 + 1] = l_run[nt];
        }
    }
    // element e = 128 h + 8 r + j sits in slot ((h*8 + j)*4 + (r >> 2))*4 + (r & 3)
    int merge_slot[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int e = (4 * lane + k) & (HD - 1);  // (lanes beyond the row repeat its start and store nothing)
        const int h = e >> 7, r = (e >> 3) & 15, j = e & 7;
        merge_slot[k] = ((h * 8 + j) * 4 + (r >> 2)) * 4 + (r & 3);
    }
    // finishes column `col` from its sums v (element order of the head dimension) and its state
    auto finish_column = [&](int col, float (&v)[4], float m_col, float l_col) {
        const int t = fast_div(col, P.q_group);
        const int a = col - t * P.q_group;
        const size_t row = (size_t)(tok0 + t) * P.num_q_heads + (size_t)(q_head_base + a);
        if (BAL ? item.n_chunks > 1 : P.max_chunks > 1) {
            const size_t prow = BAL ? bal_partial_row(item.slot, (int)gridDim.y, kv_sub, col)
                                    : row * P.max_chunks + chunk;
            float* dst = P.part_acc + prow * kHeadDim;
            if (4 * lane < HD) *reinterpret_cast<f4*>(dst + 4 * lane) = f4{v[0], v[1], v[2], v[3]};
            if (lane == 0) {
                *reinterpret_cast<f4*>(P.part_ml + prow * 4) = f4{m_col, l_col, (float)g.n_chunks, 0.f};
            }
        } else {
            const float inv = l_col > 0.f ? 1.0f / l_col : 0.f;
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] *= inv;
            if (K8 && P.rot_out) {  // rotated V rows: one inverse rotation of the finished row
                wht256_wave(v, lane);
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] = apply_sign(v[k], 4 * lane + k);
            }
            store_out_row<TQ, HD>(P, row, lane, v);
        }
    };
    {
        static_assert(NT == 1, "the merge below is the one-tile form");
        // One 16-column tile: a wave's region fits its own staging area, which nobody else touches.
        // The wave stores its O as it stands, before the barrier; the adding wave weights the eight
        // regions by 2^(m_w - m_tot), reads one 128-bit piece per lane and region, and brings the
        // sums into element order through the 1 KB its staging area has left behind the region.
        static_assert(kRegion * 4 + 1024 <= kKv16Stage, "region and transposition buffer inside the staging area");
        float* region = reinterpret_cast<float*>(stage);
        float* tbuf = region + kRegion;
        if (col_ok[0]) {
            float* c = region + n * kColStride;
#pragma unroll
            for (int h = 0; h < kH; ++h)
#pragma unroll
                for (int j = 0; j < 8; ++j) *reinterpret_cast<f4*>(c + ((h * 8 + j) * 4 + b) * 4) = o_acc[0][h][j];
        }
        __syncthreads();
        for (int col = wave; col < 16; col += kWaves) {
            if (!((ok_mask[0] >> col) & 1u)) continue;
            float mw[kWaves], lw[kWaves];
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                const f2 r = *reinterpret_cast<const f2*>(mlbuf + (w * 16 + col) * 2);
                mw[w] = r[0];
                lw[w] = r[1];
            }
            float m_col = kNegBig, l_col = 0.f;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) m_col = fmaxf(m_col, mw[w]);
            f4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                const float wgt = __builtin_amdgcn_exp2f(mw[w] - m_col);
                l_col += lw[w] * wgt;
                // (head dimension 128: the upper lanes read what the lower ones read and drop it)
                tot += *reinterpret_cast<const f4*>(smem + w * kKv16Stage + (col * kColStride + ((4 * lane) & (HD - 1))) * 4) * wgt;
            }
            *reinterpret_cast<f4*>(tbuf + 4 * lane) = tot;
            float v[4];  // the reads follow the write of the same wave in LDS order
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = tbuf[merge_slot[k]];
            finish_column(col, v, m_col, l_col);
        }
    }
}

template <typename TQ, int NT, int KVF, bool VRES, int HD = kHeadDim>
__global__ __launch_bounds__(kKv16Waves * 64, 1) void paged_attn_rows_kernel(const AttnParams P) {
    extern __shared__ __align__(16) uint8_t smem[];
    // (one body per kind of load: a branch around the loads themselves keeps the compiler from
    // scheduling them freely and loses what the hint gains)
    if (P.tiles_by_request != 0 && P.q_subgroups == 1) {  // uniform for the grid
        rows_tile<TQ, NT, KVF, false, VRES, true, HD>(P, smem, BalItem{});
    } else {
        rows_tile<TQ, NT, KVF, false, VRES, false, HD>(P, smem, BalItem{});
    }
}

template <typename TQ, int KVF, bool VRES>
__global__ __launch_bounds__(kKv16Waves * 64, 1) void paged_attn_rows_balanced_kernel(const AttnParams P) {
    extern __shared__ __align__(16) uint8_t smem[];
    bal_for_each_piece(P, [&](const BalItem& it) { rows_tile<TQ, 1, KVF, true, VRES>(P, smem, it); });
}

}  // namespace w34
