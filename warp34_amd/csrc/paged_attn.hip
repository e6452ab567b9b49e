// Paged GQA decode / verify attention for gfx950 with split-K across workgroups.
//
// Replaces the reference's paged_attention_gqa_mma_f16_kernel, its split-KV reduce kernel and
// the dispatcher (op_paged_attn.cu:186-588,1132-1218,1266-1448), and the bf16 decode kernel
// (op_kv_cache.cu:873-1241).  The dispatch table of the reference is NOT reproduced: it is
// tuned for 84-SM GDDR parts and leaves long contexts on a handful of CTAs.
//
// Work decomposition
//   tile  = up to TT consecutive query tokens of one request x the q heads of one kv head
//           (16*NT MFMA columns; decode: 1 token x 8 heads -> 8 of 16 columns used)
//   chunk = contiguous range of 32-token "units" of the tile's visible keys; one workgroup
//           (4 waves) per (chunk, kv head, tile).  The number of chunks of a tile depends only
//           on the tile's own key range and on a host cap derived from total_tokens and the
//           scratch size -- never on max_seq_len, max_blocks_per_req, physical page numbers or
//           local_kv_heads -- so outputs are bit-identical under page permutation, graph-bucket
//           bounds and head sharding (tests/tq4_vision_and_moe.rs:1089-1663).
//   unit  = 32 consecutive tokens handled by ONE wave start to finish: the wave copies the
//           raw K and V rows of the unit into its private LDS area (flat, coalesced 16-byte
//           loads; next unit prefetched into registers), forms S^T = K Q'^T with MFMA, does the
//           online softmax in registers and accumulates O^T += V^T P^T with MFMA.  Waves never
//           synchronise inside the key loop; their (m, l, O) states are merged once at the end.
//
// TQ4 specifics (row = [fp16 d0][64 B nibbles][fp16 d1][64 B nibbles], 132 B, 33 dwords):
//   * dequantisation is a 256-entry LDS table indexed by a code BYTE that returns the two
//     centroids as packed fp16; the table is replicated once per LDS bank so random indices
//     never conflict;
//   * the per-128 scales are not applied per element: K scales multiply the two half-row
//     partial scores, V scales are folded into the probabilities (two P matrices);
//   * the first half of a row starts at byte 2, so aligned dwords straddle code words.  The
//     K path treats the row as 33 aligned dwords and zeroes the query for the 8 nibble slots
//     that hold scale bytes; the V path builds dword column 0 as [codes 0-3 | codes 124-127]
//     from dwords 0 and 16, every other column is an aligned dword;
//   * attention runs in the rotated domain: Q' = WHT(sign*q) once per tile, the output is
//     un-rotated once at the end (op_kv_cache.cu:443-451,763-783).
//
// MFMA use: v_mfma_f32_16x16x32_f16.  A = K rows (QK) or V^T (PV) so that every lane owns one
// query column: softmax state and the O rescale are per-lane scalars.
#include "kv_common.h"

namespace w34 {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));

constexpr int kWaves = 4;            // waves per workgroup
constexpr int kUnit = 32;            // tokens per wave iteration
constexpr int kLutBytes = 256 * 128; // 256 entries x 32 bank replicas x 4 B
constexpr int kStageTq4 = 2 * kUnit * kTq4RowBytes;  // K + V raw rows of one unit: 8448 B
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegBig = -1.0e30f;  // "minus infinity" that stays finite under subtraction
// The table holds fp16(kLutGain * centroid); the gain is folded back into the fp32 row scales.
// 1.908032 minimises the worst fp16 rounding error of the eight centroid magnitudes
// (9.4e-5 relative instead of 3.7e-4), which is what limits the accuracy of the scores.
constexpr float kLutGain = 1.908032f;
constexpr float kLutInvGain = 1.0f / kLutGain;

struct AttnParams {
    warp34_kv_layer_layout L;
    warp34_attention_batch B;
    const uint16_t* q;
    uint16_t* out;
    float* part_acc;  // [rows][max_chunks][256] or null
    float* part_ml;   // [rows][max_chunks][2]
    int* part_cnt;    // [rows]
    int num_q_heads;
    int gqa;          // q heads per kv head
    int q_group;      // q heads of one kv head handled by one workgroup (<= 16)
    int q_subgroups;  // gqa / q_group
    int tok_tile;     // query tokens per tile
    int max_chunks;   // cap on chunks per tile (1 = no split, scratch untouched)
    int min_upc;      // minimum units per chunk
};

// token of k-slot (s, b, i) inside a unit: spreads the four 4-row groups of an MFMA over LDS
// banks so that neither the K-row reads nor the V-column reads conflict.
__device__ __forceinline__ int unit_token(int s, int b, int i) {
    return 16 * (b & 1) + 8 * s + 4 * (b >> 1) + i;
}

// chunk geometry of a tile, identical in the attention and the merge kernel
struct ChunkGeom {
    int u_first, n_units, upc, n_chunks;
};
__device__ __forceinline__ ChunkGeom chunk_geom(int u_lo, int u_hi, int max_chunks, int min_upc) {
    ChunkGeom g;
    g.u_first = u_lo >> 5;
    g.n_units = (u_hi >= u_lo) ? ((u_hi >> 5) - g.u_first + 1) : 0;
    int nc = (g.n_units + min_upc - 1) / min_upc;
    if (nc > max_chunks) nc = max_chunks;
    if (nc < 1) nc = 1;
    g.upc = (g.n_units + nc - 1) / nc;
    if (g.upc < 1) g.upc = 1;
    g.n_chunks = (g.n_units + g.upc - 1) / g.upc;
    if (g.n_chunks < 1) g.n_chunks = 1;
    return g;
}

// 256-point WHT over one wave: element e = 4*lane + k, scaled by 1/16.
__device__ __forceinline__ void wht256_wave(float (&v)[4], int lane) {
    {
        const float a0 = v[0] + v[1], a1 = v[0] - v[1], a2 = v[2] + v[3], a3 = v[2] - v[3];
        v[0] = a0 + a2;
        v[1] = a1 + a3;
        v[2] = a0 - a2;
        v[3] = a1 - a3;
    }
#pragma unroll
    for (int h = 1; h < 64; h <<= 1) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float o = __shfl_xor(v[k], h, 64);
            v[k] = (lane & h) ? (o - v[k]) : (v[k] + o);
        }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] *= 0.0625f;
}

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    f2 f = {a, b};
    h2 h = __builtin_convertvector(f, h2);
    return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ float half_bits_to_f32(uint32_t b) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}

// element index (0..255) of nibble i of aligned dword D of a TQ4 row, -1 for scale nibbles
__device__ __forceinline__ int tq4_dword_elem(int D, int i) {
    if (D == 0) return i >= 4 ? i - 4 : -1;
    if (D < 16) return 8 * D - 4 + i;
    if (D == 16) return i < 4 ? 124 + i : -1;
    return 128 + 8 * (D - 17) + i;
}
// dword read by lane k-block bk for QK MFMA m of half h (h=0: m 0..4, h=1: m 0..3)
__device__ __forceinline__ int tq4_qk_dword(int h, int m, int bk) {
    const int base = 8 * (bk & 1) + 4 * (bk >> 1);
    if (h == 0) return m < 4 ? base + m : 16;
    return 17 + base + m;
}
// element index of V^T row r, nibble j, half h (PV MFMA output row -> head dimension)
__device__ __forceinline__ int tq4_pv_elem(int h, int j, int r) {
    if (h == 1) return 128 + 8 * r + j;
    if (r == 0) return j < 4 ? j : 120 + j;
    return 8 * r - 4 + j;
}

template <typename TQ, int NT>
__global__ __launch_bounds__(256, (NT == 1 ? 2 : 1)) void paged_attn_tq4_kernel(const AttnParams P) {
    extern __shared__ __align__(16) uint8_t smem[];
    uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
    uint8_t* stage_all = smem + kLutBytes;  // kWaves * kStageTq4 bytes, reused by prologue/epilogue

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int n = lane & 15;  // MFMA column = query row of this lane
    const int b = lane >> 4;  // MFMA k-block / output row group
    const warp34_kv_layer_layout& L = P.L;
    const warp34_attention_batch& B = P.B;

    // ---- tile identification ------------------------------------------------------------
    const int tok0 = (int)blockIdx.z;
    const int kv_sub = (int)blockIdx.y;
    const int kv_head = kv_sub / P.q_subgroups;
    const int q_head_base = kv_head * P.gqa + (kv_sub % P.q_subgroups) * P.q_group;
    const int chunk = (int)blockIdx.x;

    if (tok0 >= B.total_tokens) return;
    int rq_start = 0, rq_end = 0;
    const int req = find_request(B, tok0, rq_start, rq_end);
    if (req < 0) return;
    if (B.valid_req_mask != nullptr && B.valid_req_mask[req] == 0) return;
    if (((tok0 - rq_start) % P.tok_tile) != 0) return;  // not a tile leader
    int tile_tokens = rq_end - tok0;
    if (tile_tokens > P.tok_tile) tile_tokens = P.tok_tile;

    // per-lane column info (one column per N tile)
    int col_lo[NT], col_hi[NT], col_tok[NT], col_qh[NT];
    bool col_ok[NT];
    int u_lo = 0x7fffffff, u_hi = -1;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int col = nt * 16 + n;
        const int t = col / P.q_group;
        const int a = col - t * P.q_group;
        col_tok[nt] = tok0 + t;
        col_qh[nt] = q_head_base + a;
        col_ok[nt] = false;
        col_lo[nt] = 0;
        col_hi[nt] = -1;
        if (t < tile_tokens) {
            const RowRange rr = row_range(B, tok0 + t);
            if (rr.req >= 0) {
                col_ok[nt] = true;
                col_lo[nt] = rr.min_kv;
                col_hi[nt] = rr.max_kv;
            }
        }
        if (col_ok[nt] && col_lo[nt] <= col_hi[nt]) {
            u_lo = min(u_lo, col_lo[nt]);
            u_hi = max(u_hi, col_hi[nt]);
        }
    }
    // union over the 16 columns (lanes sharing b hold the same columns)
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        u_lo = min(u_lo, __shfl_xor(u_lo, off, 64));
        u_hi = max(u_hi, __shfl_xor(u_hi, off, 64));
    }
    bool any_ok = false;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) any_ok |= col_ok[nt];
    if (__ballot(any_ok) == 0ull) return;  // whole tile masked: outputs untouched
    if (u_hi < 0) u_lo = 0;

    const ChunkGeom g = chunk_geom(u_lo, u_hi, P.max_chunks, P.min_upc);
    if (chunk >= g.n_chunks) return;
    const int cu_first = g.u_first + chunk * g.upc;
    int cu_end = cu_first + g.upc;
    if (cu_end > g.u_first + g.n_units) cu_end = g.u_first + g.n_units;

    // ---- prologue: LUT, rotated queries ---------------------------------------------------
    {
        // thread t builds entry t: (centroid[t & 15], centroid[t >> 4]) as packed fp16
        const uint32_t e = pack_h2(kLutGain * kCentroids[tid & 15], kLutGain * kCentroids[tid >> 4]);
        u4 v = {e, e, e, e};
        u4* dst = reinterpret_cast<u4*>(lut + tid * 32);
#pragma unroll
        for (int k = 0; k < 8; ++k) dst[k] = v;
    }
    // rotated, fp16 query rows in LDS: [16*NT][264] halves (aliases the staging area)
    constexpr int kQStride = 264;
    _Float16* qlds = reinterpret_cast<_Float16*>(stage_all);
    for (int col = wave; col < 16 * NT; col += kWaves) {
        const int t = col / P.q_group;
        const int a = col - t * P.q_group;
        float v[4] = {0.f, 0.f, 0.f, 0.f};
        bool ok = false;
        if (t < tile_tokens) {
            const RowRange rr = row_range(B, tok0 + t);
            ok = rr.req >= 0;
        }
        if (ok) {
            const uint16_t* qrow =
                P.q + ((size_t)(tok0 + t) * P.num_q_heads + (size_t)(q_head_base + a)) * kHeadDim;
            const uint2 raw = *reinterpret_cast<const uint2*>(qrow + 4 * lane);
            v[0] = TQ::to_f32((uint16_t)(raw.x & 0xFFFFu));
            v[1] = TQ::to_f32((uint16_t)(raw.x >> 16));
            v[2] = TQ::to_f32((uint16_t)(raw.y & 0xFFFFu));
            v[3] = TQ::to_f32((uint16_t)(raw.y >> 16));
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = apply_sign(v[k], 4 * lane + k);
            wht256_wave(v, lane);
        }
        uint2 packed;
        packed.x = pack_h2(v[0], v[1]);
        packed.y = pack_h2(v[2], v[3]);
        *reinterpret_cast<uint2*>(qlds + col * kQStride + 4 * lane) = packed;
    }
    __syncthreads();

    // B operands of the QK MFMAs: 9 per N tile (5 for the first half-row, 4 for the second)
    h8 bq[NT][9];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int mf = 0; mf < 9; ++mf) {
            const int h = mf < 5 ? 0 : 1;
            const int m = mf < 5 ? mf : mf - 5;
            const int D = tq4_qk_dword(h, m, b);
            const bool dummy = (h == 0 && m == 4 && b != 0);
            h8 x;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int e = dummy ? -1 : tq4_dword_elem(D, i);
                x[i] = e >= 0 ? qlds[(nt * 16 + n) * kQStride + e] : (_Float16)0.0f;
            }
            bq[nt][mf] = x;
        }
    }
    __syncthreads();  // qlds is dead, the staging area may be overwritten

    // ---- per-wave state -----------------------------------------------------------------------
    uint8_t* stage = stage_all + wave * kStageTq4;  // [K rows 0..31][V rows 0..31], 132 B each
    const uint32_t lut_lane = (uint32_t)(lane & 31);
    const float score_scale = B.sm_scale * kLog2e * kLutInvGain;

    f4 o_acc[NT][2][8];
    float m_run[NT], l_run[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        m_run[nt] = kNegBig;
        l_run[nt] = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 8; ++j) o_acc[nt][h][j] = f4{0.f, 0.f, 0.f, 0.f};
    }

    const int32_t* req_blocks = B.block_tables + (size_t)req * B.max_blocks_per_req;
    const uint8_t* k_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.k_base) +
                            (size_t)kv_head * L.k_head_stride_bytes;
    const uint8_t* v_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.v_base) +
                            (size_t)kv_head * L.v_head_stride_bytes;

    // Staging copy: the unit is 4 contiguous runs of 16 rows (2112 B = 132 16-byte pieces):
    // K rows 0-15, K rows 16-31, V rows 0-15, V rows 16-31.  Piece c = lane + 64 i of the
    // 528 pieces belongs to run c / 132.
    constexpr int kPieces = 9;  // ceil(528 / 64)
    u4 pf[kPieces];
    auto issue_loads = [&](int unit) {
        const int t0 = unit * kUnit;
        const uint8_t* run_ptr[4];
#pragma unroll
        for (int gidx = 0; gidx < 2; ++gidx) {
            const int pos = t0 + 16 * gidx;
            const int page_slot = pos / L.block_size;
            const int in_page = pos - page_slot * L.block_size;
            // a run is fetched only when it overlaps the visible key range and its block
            // table entry exists; everything else keeps stale (finite-by-construction) bytes
            bool live = pos <= u_hi && pos + 15 >= u_lo && page_slot < B.max_blocks_per_req;
            const int32_t page = live ? req_blocks[page_slot] : -1;
            live = live && page >= 0;
            run_ptr[gidx] = live ? k_base + (size_t)page * L.k_page_stride_bytes +
                                       (size_t)in_page * L.k_token_stride_bytes
                                 : nullptr;
            run_ptr[2 + gidx] = live ? v_base + (size_t)page * L.v_page_stride_bytes +
                                           (size_t)in_page * L.v_token_stride_bytes
                                     : nullptr;
        }
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int c = lane + 64 * i;
            const int run = c / 132;
            const int idx = c - run * 132;
            const uint8_t* base = run == 0 ? run_ptr[0] : run == 1 ? run_ptr[1] : run == 2 ? run_ptr[2] : run_ptr[3];
            u4 v = {0u, 0u, 0u, 0u};
            if (c < 528 && base != nullptr) v = *reinterpret_cast<const u4*>(base + 16 * idx);
            pf[i] = v;
        }
    };
    auto commit_loads = [&]() {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int c = lane + 64 * i;
            if (c < 528) *reinterpret_cast<u4*>(stage + 16 * c) = pf[i];
        }
    };

    int unit = cu_first + wave;
    if (unit < cu_end) issue_loads(unit);

    for (; unit < cu_end; unit += kWaves) {
        commit_loads();
        if (unit + kWaves < cu_end) issue_loads(unit + kWaves);
        const int t0 = unit * kUnit;
        const uint8_t* k_rows = stage;
        const uint8_t* v_rows = stage + kUnit * kTq4RowBytes;

        // ---- S^T = K Q'^T for the two 16-key sub-tiles ------------------------------------
        float sc[NT][8];
        {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const int arow = unit_token(s, n >> 2, n & 3);  // A row n of sub-tile s
                const uint32_t* row32 = reinterpret_cast<const uint32_t*>(k_rows + arow * kTq4RowBytes);
                f4 s_acc[NT][2];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    s_acc[nt][0] = f4{0.f, 0.f, 0.f, 0.f};
                    s_acc[nt][1] = f4{0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
                for (int mf = 0; mf < 9; ++mf) {
                    const int h = mf < 5 ? 0 : 1;
                    const int m = mf < 5 ? mf : mf - 5;
                    const uint32_t w = row32[tq4_qk_dword(h, m, b)];
                    u4 a;
                    a[0] = lut[((w & 0xFFu) << 5) + lut_lane];
                    a[1] = lut[(((w >> 8) & 0xFFu) << 5) + lut_lane];
                    a[2] = lut[(((w >> 16) & 0xFFu) << 5) + lut_lane];
                    a[3] = lut[((w >> 24) << 5) + lut_lane];
                    const h8 av = __builtin_bit_cast(h8, a);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        s_acc[nt][h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bq[nt][mf], s_acc[nt][h], 0, 0, 0);
                    }
                }
                // rows 4b+i of the result are tokens unit_token(s, b, i); apply the K scales
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int trow = unit_token(s, b, i);
                    const uint16_t* r16 = reinterpret_cast<const uint16_t*>(k_rows + trow * kTq4RowBytes);
                    const float d0 = half_bits_to_f32(r16[0]) * score_scale;
                    const float d1 = half_bits_to_f32(r16[33]) * score_scale;
                    const int pos = t0 + trow;
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        const float v = d0 * s_acc[nt][0][i] + d1 * s_acc[nt][1][i];
                        const bool vis = col_ok[nt] && pos >= col_lo[nt] && pos <= col_hi[nt];
                        sc[nt][4 * s + i] = vis ? v : kNegBig;
                    }
                }
            }
        }

        // ---- online softmax (log2 domain), per lane = per query column --------------------
        // V scales of this lane's 8 tokens and the raw V dwords
        uint32_t vd0[8], vd16[8], vwr[8], vw1[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int trow = unit_token(t >> 2, b, t & 3);
            const uint32_t* row32 = reinterpret_cast<const uint32_t*>(v_rows + trow * kTq4RowBytes);
            vd0[t] = row32[0];
            vd16[t] = row32[16];
            vwr[t] = row32[n];       // n == 0 re-reads dword 0
            vw1[t] = row32[17 + n];
        }
        uint32_t pb[NT][2][4];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            float mx = sc[nt][0];
#pragma unroll
            for (int t = 1; t < 8; ++t) mx = fmaxf(mx, sc[nt][t]);
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run[nt], mx);
            const float alpha = __builtin_amdgcn_exp2f(m_run[nt] - m_new);
            m_run[nt] = m_new;
            float p[8];
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                p[t] = sc[nt][t] > 0.5f * kNegBig ? __builtin_amdgcn_exp2f(sc[nt][t] - m_new) : 0.f;
                psum += p[t];
            }
            l_run[nt] = l_run[nt] * alpha + psum;
            if (__ballot(alpha != 1.0f) != 0ull) {
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int j = 0; j < 8; ++j) o_acc[nt][h][j] *= alpha;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float d0a = half_bits_to_f32(vd0[2 * k] & 0xFFFFu) * kLutInvGain;
                const float d0b = half_bits_to_f32(vd0[2 * k + 1] & 0xFFFFu) * kLutInvGain;
                const float d1a = half_bits_to_f32(vd16[2 * k] >> 16) * kLutInvGain;
                const float d1b = half_bits_to_f32(vd16[2 * k + 1] >> 16) * kLutInvGain;
                // masked tokens have p == 0; select instead of multiply so that a garbage
                // scale (rows beyond the sequence end) cannot inject NaN
                pb[nt][0][k] = pack_h2(p[2 * k] > 0.f ? p[2 * k] * d0a : 0.f,
                                       p[2 * k + 1] > 0.f ? p[2 * k + 1] * d0b : 0.f);
                pb[nt][1][k] = pack_h2(p[2 * k] > 0.f ? p[2 * k] * d1a : 0.f,
                                       p[2 * k + 1] > 0.f ? p[2 * k + 1] * d1b : 0.f);
            }
        }

        // ---- O^T += V^T P^T ------------------------------------------------------------------
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                uint32_t wa, wb;
                if (h == 0) {
                    const uint32_t xa = __builtin_amdgcn_alignbit(vd16[2 * k], vd0[2 * k], 16);
                    const uint32_t xb = __builtin_amdgcn_alignbit(vd16[2 * k + 1], vd0[2 * k + 1], 16);
                    wa = n == 0 ? xa : vwr[2 * k];
                    wb = n == 0 ? xb : vwr[2 * k + 1];
                } else {
                    wa = vw1[2 * k];
                    wb = vw1[2 * k + 1];
                }
                // byte q of lo / hi = (nibble 2q / 2q+1 of token a) | (same nibble of token b) << 4
                lo[k] = (wa & 0x0F0F0F0Fu) | ((wb << 4) & 0xF0F0F0F0u);
                hi[k] = ((wa >> 4) & 0x0F0F0F0Fu) | (wb & 0xF0F0F0F0u);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                u4 a;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t src = (j & 1) ? hi[k] : lo[k];
                    const uint32_t byte = (src >> (8 * (j >> 1))) & 0xFFu;
                    a[k] = lut[(byte << 5) + lut_lane];
                }
                const h8 av = __builtin_bit_cast(h8, a);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    u4 pbv = {pb[nt][h][0], pb[nt][h][1], pb[nt][h][2], pb[nt][h][3]};
                    o_acc[nt][h][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        av, __builtin_bit_cast(h8, pbv), o_acc[nt][h][j], 0, 0, 0);
                }
            }
        }
    }

    // ---- combine the per-lane partial sums of l over the four k-block lanes of a column ------
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        l_run[nt] += __shfl_xor(l_run[nt], 16, 64);
        l_run[nt] += __shfl_xor(l_run[nt], 32, 64);
    }

    // ---- merge the waves' states through LDS (pairwise tree), result in wave 0 ----------------
    __syncthreads();  // every wave is done with its staging area
    // [2 senders][NT*16 cols][258] floats; overlays the LUT and the staging areas, both dead now
    float* xbuf = reinterpret_cast<float*>(smem);
    constexpr int kColStride = 258;
#pragma unroll
    for (int round = 0; round < 2; ++round) {
        const int senders_lo = round == 0 ? 2 : 1;  // waves [senders_lo, 2*senders_lo) send
        const int nsend = senders_lo;
        if (wave >= senders_lo && wave < 2 * senders_lo) {
            float* dst = xbuf + (size_t)(wave - senders_lo) * (NT * 16 * kColStride);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                float* c = dst + (nt * 16 + n) * kColStride;
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int j = 0; j < 8; ++j)
#pragma unroll
                        for (int i = 0; i < 4; ++i) c[tq4_pv_elem(h, j, 4 * b + i)] = o_acc[nt][h][j][i];
                if (b == 0) {
                    c[256] = m_run[nt];
                    c[257] = l_run[nt];
                }
            }
        }
        __syncthreads();
        if (wave < nsend) {
            const float* src = xbuf + (size_t)wave * (NT * 16 * kColStride);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float* c = src + (nt * 16 + n) * kColStride;
                const float m2 = c[256], l2 = c[257];
                const float m_new = fmaxf(m_run[nt], m2);
                const float w1 = __builtin_amdgcn_exp2f(m_run[nt] - m_new);
                const float w2 = __builtin_amdgcn_exp2f(m2 - m_new);
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int j = 0; j < 8; ++j)
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            o_acc[nt][h][j][i] = o_acc[nt][h][j][i] * w1 + c[tq4_pv_elem(h, j, 4 * b + i)] * w2;
                l_run[nt] = l_run[nt] * w1 + l2 * w2;
                m_run[nt] = m_new;
            }
        }
        __syncthreads();
    }

    // ---- epilogue ----------------------------------------------------------------------------
    // wave 0 publishes the tile state as [col][258] floats, then all waves either store the
    // split partial or finish the rows (normalise, un-rotate, convert).
    if (wave == 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            float* c = xbuf + (nt * 16 + n) * kColStride;
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < 8; ++j)
#pragma unroll
                    for (int i = 0; i < 4; ++i) c[tq4_pv_elem(h, j, 4 * b + i)] = o_acc[nt][h][j][i];
            if (b == 0) {
                c[256] = m_run[nt];
                c[257] = l_run[nt];
            }
        }
    }
    __syncthreads();
    for (int col = wave; col < 16 * NT; col += kWaves) {
        const int t = col / P.q_group;
        const int a = col - t * P.q_group;
        if (t >= tile_tokens) continue;
        const RowRange rr = row_range(B, tok0 + t);
        if (rr.req < 0) continue;
        const size_t row = (size_t)(tok0 + t) * P.num_q_heads + (size_t)(q_head_base + a);
        const float* c = xbuf + col * kColStride;
        float v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = c[4 * lane + k];
        if (P.max_chunks > 1) {
            float* dst = P.part_acc + (row * P.max_chunks + chunk) * kHeadDim;
            *reinterpret_cast<f4*>(dst + 4 * lane) = f4{v[0], v[1], v[2], v[3]};
            if (lane == 0) {
                P.part_ml[(row * P.max_chunks + chunk) * 2 + 0] = c[256];
                P.part_ml[(row * P.max_chunks + chunk) * 2 + 1] = c[257];
                if (chunk == 0) P.part_cnt[row] = g.n_chunks;
            }
        } else {
            const float l = c[257];
            const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] *= inv;
            wht256_wave(v, lane);
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = apply_sign(v[k], 4 * lane + k);
            uint2 o;
            o.x = (uint32_t)TQ::from_f32(v[0]) | ((uint32_t)TQ::from_f32(v[1]) << 16);
            o.y = (uint32_t)TQ::from_f32(v[2]) | ((uint32_t)TQ::from_f32(v[3]) << 16);
            *reinterpret_cast<uint2*>(P.out + row * kHeadDim + 4 * lane) = o;
        }
    }
}

// Merge of the split-K partials of one (token, q head) row per wave
// (op_paged_attn.cu:1132-1218): m_tot = max m_s, w_s = 2^(m_s - m_tot),
// out = sum acc_s w_s / sum l_s w_s, then one inverse rotation.
template <typename TQ>
__global__ __launch_bounds__(256) void split_merge_kernel(const AttnParams P, int rotate) {
    const int lane = (int)(threadIdx.x & 63);
    const int wave = (int)(threadIdx.x >> 6);
    const long long row = (long long)blockIdx.x * 4 + wave;
    const long long rows = (long long)P.B.total_tokens * P.num_q_heads;
    if (row >= rows) return;
    const int tok = (int)(row / P.num_q_heads);
    const RowRange rr = row_range(P.B, tok);
    if (rr.req < 0) return;
    const int n_chunks = P.part_cnt[row];
    const float* ml = P.part_ml + (size_t)row * P.max_chunks * 2;
    const float* acc = P.part_acc + (size_t)row * P.max_chunks * kHeadDim;
    float m_tot = kNegBig;
    for (int s = 0; s < n_chunks; ++s)
        if (ml[2 * s + 1] > 0.f) m_tot = fmaxf(m_tot, ml[2 * s]);
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    float l_tot = 0.f;
    for (int s = 0; s < n_chunks; ++s) {
        const float ls = ml[2 * s + 1];
        if (!(ls > 0.f)) continue;
        const float w = __builtin_amdgcn_exp2f(ml[2 * s] - m_tot);
        l_tot += ls * w;
        const f4 a = *reinterpret_cast<const f4*>(acc + (size_t)s * kHeadDim + 4 * lane);
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] += a[k] * w;
    }
    const float inv = l_tot > 0.f ? 1.0f / l_tot : 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] *= inv;
    if (rotate) {
        wht256_wave(v, lane);
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = apply_sign(v[k], 4 * lane + k);
    }
    uint2 o;
    o.x = (uint32_t)TQ::from_f32(v[0]) | ((uint32_t)TQ::from_f32(v[1]) << 16);
    o.y = (uint32_t)TQ::from_f32(v[2]) | ((uint32_t)TQ::from_f32(v[3]) << 16);
    *reinterpret_cast<uint2*>(P.out + (size_t)row * kHeadDim + 4 * lane) = o;
}

// ---- host side ---------------------------------------------------------------------------------
constexpr int kMaxChunksCap = 256;
constexpr int kMinUnitsPerChunk = 8;   // 256 tokens
constexpr int kTargetWorkgroupsPerHead = 512;

static size_t partial_bytes(long long rows, int max_chunks) {
    return (size_t)rows * (size_t)max_chunks * (kHeadDim + 2) * sizeof(float) + (size_t)rows * sizeof(int);
}

// Cap on chunks per tile: a function of total_tokens (tiles) and the scratch size only.
static int choose_max_chunks(const warp34_exec* ex, int total_tokens, int num_q_heads, int tok_tile) {
    if (ex->scratch_ptr == 0 || (ex->scratch_ptr & 15u) != 0u) return 1;
    const int tiles = (total_tokens + tok_tile - 1) / tok_tile;
    int want = kTargetWorkgroupsPerHead / (tiles > 0 ? tiles : 1);
    if (want > kMaxChunksCap) want = kMaxChunksCap;
    if (want < 2) return 1;
    const long long rows = (long long)total_tokens * num_q_heads;
    while (want > 1 && partial_bytes(rows, want) > ex->scratch_size) want >>= 1;
    return want < 2 ? 1 : want;
}

template <typename KernelT>
static int ensure_dynamic_lds(KernelT kernel, int bytes) {
    // one attribute call per kernel instantiation and device
    static thread_local const void* done_fn[16];
    static thread_local int done_dev[16];
    static thread_local int n_done = 0;
    int dev = 0;
    hipError_t rc = hipGetDevice(&dev);
    if (rc != hipSuccess) return (int)rc;
    for (int i = 0; i < n_done; ++i)
        if (done_fn[i] == (const void*)kernel && done_dev[i] == dev) return 0;
    rc = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (rc != hipSuccess) return (int)rc;
    if (n_done < 16) {
        done_fn[n_done] = (const void*)kernel;
        done_dev[n_done] = dev;
        ++n_done;
    }
    return 0;
}

template <typename TQ>
static int launch_tq4(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                      const warp34_attention_batch* batch, const void* q, void* out, int num_q_heads,
                      int force_single) {
    AttnParams P;
    P.L = *layout;
    P.B = *batch;
    P.q = (const uint16_t*)q;
    P.out = (uint16_t*)out;
    P.num_q_heads = num_q_heads;
    P.gqa = num_q_heads / layout->local_kv_heads;
    int q_group = P.gqa;
    if (q_group > 16) {
        for (int d = 16; d >= 1; --d)
            if (P.gqa % d == 0) {
                q_group = d;
                break;
            }
    }
    P.q_group = q_group;
    P.q_subgroups = P.gqa / q_group;
    // two N tiles when a request brings enough query rows to fill them
    const int nt = (batch->max_q_len * q_group > 16) ? 2 : 1;
    P.tok_tile = (16 * nt) / q_group;
    if (P.tok_tile < 1) P.tok_tile = 1;
    P.min_upc = kMinUnitsPerChunk;
    P.max_chunks = force_single ? 1 : choose_max_chunks(ex, batch->total_tokens, num_q_heads, P.tok_tile);
    P.part_acc = nullptr;
    P.part_ml = nullptr;
    P.part_cnt = nullptr;
    const long long rows = (long long)batch->total_tokens * num_q_heads;
    if (P.max_chunks > 1) {
        uint8_t* ws = reinterpret_cast<uint8_t*>((uintptr_t)ex->scratch_ptr);
        P.part_acc = reinterpret_cast<float*>(ws);
        P.part_ml = P.part_acc + (size_t)rows * P.max_chunks * kHeadDim;
        P.part_cnt = reinterpret_cast<int*>(P.part_ml + (size_t)rows * P.max_chunks * 2);
    }
    // grid.x: chunks that can exist given the host's upper bound on the sequence length
    int grid_x = P.max_chunks;
    if (batch->max_seq_len > 0) {
        const int units = (batch->max_seq_len + kUnit - 1) / kUnit + 1;
        const int bound = (units + P.min_upc - 1) / P.min_upc;
        if (bound < grid_x) grid_x = bound < 1 ? 1 : bound;
    }
    const dim3 grid((unsigned)grid_x, (unsigned)(layout->local_kv_heads * P.q_subgroups),
                    (unsigned)batch->total_tokens);
    const int lds = kLutBytes + kWaves * kStageTq4;
    hipStream_t stream = (hipStream_t)ex->stream;
    int rc;
    if (nt == 1) {
        rc = ensure_dynamic_lds(paged_attn_tq4_kernel<TQ, 1>, lds);
        if (rc) return rc;
        hipLaunchKernelGGL((paged_attn_tq4_kernel<TQ, 1>), grid, dim3(256), lds, stream, P);
    } else {
        rc = ensure_dynamic_lds(paged_attn_tq4_kernel<TQ, 2>, lds);
        if (rc) return rc;
        hipLaunchKernelGGL((paged_attn_tq4_kernel<TQ, 2>), grid, dim3(256), lds, stream, P);
    }
    rc = (int)hipGetLastError();
    if (rc) return rc;
    if (P.max_chunks > 1) {
        hipLaunchKernelGGL((split_merge_kernel<TQ>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream,
                           P, 1);
        rc = (int)hipGetLastError();
    }
    return rc;
}

static bool is_tq4_wht(const warp34_kv_layer_layout* l) {
    return l->head_dim == 256 && l->k_format == WARP34_KV_FORMAT_TQ4 && l->v_format == WARP34_KV_FORMAT_TQ4 &&
           l->k_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 &&
           l->v_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256;
}

static bool tq4_geometry_ok(const warp34_kv_layer_layout* l, const void* q) {
    // 16-token runs must be contiguous and 16-byte aligned for the staging copy
    return l->block_size > 0 && (l->block_size % 16) == 0 && l->k_token_stride_bytes == kTq4RowBytes &&
           l->v_token_stride_bytes == kTq4RowBytes && (l->k_base & 15u) == 0 && (l->v_base & 15u) == 0 &&
           (l->k_page_stride_bytes & 15u) == 0 && (l->k_head_stride_bytes & 15u) == 0 &&
           (l->v_page_stride_bytes & 15u) == 0 && (l->v_head_stride_bytes & 15u) == 0 &&
           (((uintptr_t)q) & 7u) == 0;
}
static_assert(kLutBytes + kWaves * kStageTq4 >= 2 * 2 * 16 * 258 * 4, "merge buffer must fit the LDS block");

static int common_checks(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                         const warp34_attention_batch* batch, const void* q, void* out, int num_q_heads) {
    if (!ex || !layout || !batch || !q || !out) return (int)hipErrorInvalidValue;
    return 0;
}

template <typename TQ>
static int attention_entry(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                           const warp34_attention_batch* batch, const void* q, void* out, int num_q_heads,
                           int force_single) {
    if (layout->local_kv_heads <= 0 || num_q_heads % layout->local_kv_heads != 0 || batch->num_reqs <= 0 ||
        !batch->query_start_loc || !batch->seq_lens_after || !batch->block_tables ||
        batch->max_blocks_per_req <= 0 || batch->sliding_window < 0 ||
        (batch->mask_mode != WARP34_ATTN_MASK_CAUSAL && batch->mask_mode != WARP34_ATTN_MASK_NONCAUSAL_WINDOW)) {
        return (int)hipErrorInvalidValue;
    }
    if (is_tq4_wht(layout)) {
        if (!tq4_geometry_ok(layout, q) || (((uintptr_t)out) & 7u) != 0) return (int)hipErrorNotSupported;
        return launch_tq4<TQ>(ex, layout, batch, q, out, num_q_heads, force_single);
    }
    return (int)hipErrorNotSupported;
}

}  // namespace w34

using namespace w34;

// op_paged_attn.cu:1266-1448
extern "C" int warp34_paged_attention_f16(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                          const warp34_attention_batch* batch, const void* q_in,
                                          void* attn_out, int num_q_heads) {
    const int rc = common_checks(ex, layout, batch, q_in, attn_out, num_q_heads);
    if (rc) return rc;
    if (layout->k_format == WARP34_KV_FORMAT_FP8_E4M3 || layout->v_format == WARP34_KV_FORMAT_FP8_E4M3) {
        if (layout->head_dim != 256) return (int)hipErrorInvalidValue;
        return (int)hipErrorNotSupported;
    }
    if (batch->total_tokens <= 0 || num_q_heads <= 0) return 0;
    return attention_entry<F16>(ex, layout, batch, q_in, attn_out, num_q_heads, 0);
}

// op_kv_cache.cu:1192-1241
extern "C" int warp34_paged_attention_bf16(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                           const warp34_attention_batch* batch, const void* q_in,
                                           void* attn_out, int num_q_heads) {
    const int rc = common_checks(ex, layout, batch, q_in, attn_out, num_q_heads);
    if (rc) return rc;
    if (num_q_heads <= 0 || batch->total_tokens < 0) return (int)hipErrorInvalidValue;
    if (!batch->total_tokens) return 0;
    return attention_entry<BF16>(ex, layout, batch, q_in, attn_out, num_q_heads, 0);
}

// op_paged_attn.cu:1451-1519
extern "C" int warp34_paged_attention_f16_force_kernel_for_test(
    const warp34_exec* ex, const warp34_kv_layer_layout* layout, const warp34_attention_batch* batch,
    const void* q_in, void* attn_out, int num_q_heads, int use_64q) {
    const int rc = common_checks(ex, layout, batch, q_in, attn_out, num_q_heads);
    if (rc) return rc;
    if (batch->total_tokens <= 0 || num_q_heads <= 0) return 0;
    (void)use_64q;
    return attention_entry<F16>(ex, layout, batch, q_in, attn_out, num_q_heads, 1);
}

extern "C" size_t warp34_paged_attention_scratch_bytes(int total_tokens, int num_q_heads, int max_seq_len) {
    (void)max_seq_len;
    if (total_tokens <= 0 || num_q_heads <= 0) return 0;
    int tiles = total_tokens;
    int want = kTargetWorkgroupsPerHead / tiles;
    if (want > kMaxChunksCap) want = kMaxChunksCap;
    if (want < 2) want = 2;
    return partial_bytes((long long)total_tokens * num_q_heads, want);
}
