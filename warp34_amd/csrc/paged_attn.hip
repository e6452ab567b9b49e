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
//           (8 waves) per (chunk, kv head, tile).  The number of chunks of a tile depends only
//           on the tile's own key range and on a host cap derived from total_tokens and the
//           scratch size -- never on max_seq_len, max_blocks_per_req, physical page numbers or
//           local_kv_heads -- so outputs are bit-identical under page permutation, graph-bucket
//           bounds and head sharding (tests/tq4_vision_and_moe.rs:1089-1663).
//   unit  = 32 consecutive tokens handled by ONE wave start to finish: the raw K and V rows of
//           the unit go straight from the pages into the wave's private LDS area (LDS-direct
//           16-byte loads from a wave-uniform base, one unit ahead), the wave forms
//           S^T = K Q'^T with MFMA, does the online softmax in registers and accumulates
//           O^T += V^T P^T with MFMA.  Waves never synchronise inside the key loop; their
//           (m, l, O) states are merged once at the end.
//
// TQ4 specifics (row = [fp16 d0][64 B nibbles][fp16 d1][64 B nibbles], 132 B, 33 dwords):
//   * dequantisation is a 256-entry LDS table indexed by a code BYTE that returns the two
//     centroids as packed fp16.  The table is replicated once per lane (entry stride 256 B) so
//     that random indices never conflict and the address is a single v_perm_b32:
//     addr = (byte << 8) | (lane << 2);
//   * the per-128 scales are not applied per element: K scales multiply the two half-row
//     partial scores, V scales are folded into the probabilities (two P matrices);
//   * LDS reads must be dword aligned (misaligned ds_read_b32 is ~15x slower on this part)
//     but the first half of a row starts at byte 2.  The K path therefore treats the row as 33
//     aligned dwords and zeroes the query for the 8 nibble slots that hold scale bytes; the V
//     path builds dword column 0 as [codes 0-3 | codes 124-127] from dwords 0 and 16, every
//     other column is an aligned dword;
//   * attention runs in the rotated domain: Q' = WHT(sign*q) once per tile, the output is
//     un-rotated once at the end (op_kv_cache.cu:443-451,763-783).
//
// MFMA use: v_mfma_f32_16x16x32_f16.  A = K rows (QK) or V^T (PV) so that every lane owns one
// query column: softmax state and the O rescale are per-lane scalars.
#include <atomic>
#include <type_traits>

#include "kv_common.h"

namespace w34 {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2v __attribute__((ext_vector_type(2)));

// waves per workgroup of the TQ4 decode kernel: eight, two per SIMD (up to 256 registers each); the
// LDS holds the table, eight staging areas, the query operand table and the (m, l) tables:
// 142 KB of 160 KB, one workgroup per CU
constexpr int kTq4Waves = 8;
__host__ __device__ constexpr int waves_for(int nt) { return nt == 1 ? kTq4Waves : 4; }
constexpr int kUnit = 32;             // tokens per wave iteration
constexpr int kLutBytes = 256 * 256;  // 256 entries x 64 lane replicas x 4 B
constexpr int kRunBytes = 16 * kTq4RowBytes;  // 16 rows = 2112 B = 132 16-byte pieces
constexpr int kStageTq4 = 4 * kRunBytes;      // K rows 0-31 then V rows 0-31: 8448 B
// column stride of a merge region in dwords: 1 056 bytes, a stride at which 128-bit accesses of
// eight columns do not collide (measured; 1 040 bytes cost 40 % more)
constexpr int kMergeColStride = 264;
__host__ __device__ constexpr int merge_floats_for(int nt) {  // one region of 8 columns per wave
    return waves_for(nt) * (nt * 8 * kMergeColStride);
}
constexpr int kQopBytes = 16 * 4 * 9 * 16;  // query operand table: 16 columns x 4 k-blocks x 9 operands
__host__ __device__ constexpr int ml_offset_for(int nt) {  // (m, l) tables of the merge: behind everything the loop uses
    return kLutBytes + waves_for(nt) * kStageTq4 + kQopBytes;
}
__host__ __device__ constexpr int smem_bytes_for(int nt) {
    return ml_offset_for(nt) + (waves_for(nt) + 1) * nt * 16 * 2 * 4;
}
static_assert(merge_floats_for(1) * 4 <= waves_for(1) * kStageTq4, "merge regions alias the staging areas only");
static_assert(smem_bytes_for(1) <= 160 * 1024, "decode LDS budget");
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegBig = -1.0e30f;  // "minus infinity" that stays finite under subtraction
// The table holds fp16(kLutGain * centroid); the gain is divided out of the query (K side)
// and of the final normalisation (V side).  1.908032 minimises the worst fp16 rounding error
// of the eight centroid magnitudes (9.4e-5 relative instead of 3.7e-4), which is what limits
// the accuracy of the scores.
constexpr float kLutGain = 1.908032f;
constexpr float kLutInvGain = 1.0f / kLutGain;

struct AttnParams {
    warp34_kv_layer_layout L;
    warp34_attention_batch B;
    const uint16_t* q;
    uint16_t* out;
    float* part_acc;  // [rows][max_chunks][256] or null
    float* part_ml;   // [rows][max_chunks][4]: m, l, chunk count, unused
    int num_q_heads;
    int gqa;          // q heads per kv head
    int q_group;      // q heads of one kv head handled by one workgroup (<= 16)
    int q_subgroups;  // gqa / q_group
    int tok_tile;     // query tokens per tile
    int max_chunks;   // cap on chunks per tile (1 = no split, scratch untouched)
    int min_upc;      // minimum units per chunk
    int tiles_by_request;  // 1: blockIdx.z is a request (no request has more than one tile)
    int rot_q;             // K rows are stored rotated (WHT-256 transform): rotate the query rows
    int rot_out;           // V rows are stored rotated: rotate the output back
    int32_t* bal_table;    // balanced decode: per query token {first partial slot, pieces, token of the tile, -}
    uint32_t block_magic;  // floor(2^32 / block_size), see div_block
    const uint16_t* gate;  // fp16 [tokens, q heads, 256] or null: out = fp16(out) * sigmoid(gate)
    // chunk geometry of a tile whose keys are exactly [0, max_seq_len): worked out on the host, so a
    // request that is as long as the host's bound needs no division on the device
    int spec_units, spec_upc, spec_chunks;
    // Partial records: part_stride slots per output row.  Slots [0, max_chunks) belong to the
    // split-K chunks of the decode kernels; a shared-prefix pass (tile kernel over the keys every
    // request of the batch has in common) owns slots [pf_slot_base, pf_slot_base + pf_split), and
    // the decode kernel then starts at key *key_floor.
    int part_stride;
    int pf_split, pf_slot_base;
    const int32_t* key_floor;
    // TQ4 decode kernels: a 32-token unit never straddles two pages (the page size is a multiple of
    // 32) and both page strides fit 32 bits, so a unit's four runs follow from ONE block-table entry
    // and two 32 x 32-bit products
    int unit_in_page;
};

// A finished output row leaves the kernels here: lane l holds channels 4 l .. 4 l + 3.  With a gate
// (the gated full-attention layers, model/forward.rs:1192-1211) the stored value is the attention
// output rounded to its 16-bit type and then passed through the gate operator's arithmetic
// (ops/op_norms_rope_act.cu:742-759), so it has the bits of the two calls in sequence.
// HD: the head dimension (lanes beyond a 128-element row store nothing).
template <typename TQ, int HD = kHeadDim>
__device__ __forceinline__ void store_out_row(const AttnParams& P, size_t row, int lane, const float (&o)[4]) {
    if (HD < 256 && 4 * lane >= HD) return;
    uint16_t h[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) h[k] = TQ::from_f32(o[k]);
    if (P.gate != nullptr) {
        const uint2 g = *reinterpret_cast<const uint2*>(P.gate + row * HD + 4 * lane);
        const uint16_t gb[4] = {(uint16_t)g.x, (uint16_t)(g.x >> 16), (uint16_t)g.y, (uint16_t)(g.y >> 16)};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            h[k] = TQ::from_f32(gate_product(TQ::to_f32(h[k]), F16::to_f32(gb[k])));
        }
    }
    uint2 ob;
    ob.x = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
    ob.y = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
    *reinterpret_cast<uint2*>(P.out + row * HD + 4 * lane) = ob;
}


// token of k-slot (s, b, i) inside a unit: spreads the four 4-row groups of an MFMA over LDS
// banks so that neither the K-row reads nor the V-column reads conflict.
__device__ __forceinline__ constexpr int unit_token(int s, int b, int i) {
    return 16 * (b & 1) + 8 * s + 4 * (b >> 1) + i;
}

// chunk geometry of a tile
// a / b for 0 <= a < 2^21 and 0 < b: the float quotient is within one of the exact result,
// one correction step makes it exact.  A runtime integer division costs ~40 dependent
// instructions on this hardware, and the prologue and the per-unit address arithmetic
// divide by block sizes and group sizes that only the descriptors know.
__device__ __forceinline__ int fast_div(int a, int b) {
    if (a >= (1 << 21)) return a / b;
    int q = (int)((float)a * __builtin_amdgcn_rcpf((float)b));
    const int r = a - q * b;
    q += r >= b ? 1 : 0;
    q -= r < 0 ? 1 : 0;
    return q;
}

// pos / block_size for 0 <= pos < 2^31 without a branch: the high word of pos * floor(2^32 / b)
// is the quotient or one less, one compare settles it.  The inner loops divide a token position
// by the page size for every group of 16 keys.
__device__ __forceinline__ int div_block(int pos, const AttnParams& P) {
    int q = (int)__umulhi((uint32_t)pos, P.block_magic);
    q += (pos - q * P.L.block_size >= P.L.block_size) ? 1 : 0;
    return q;
}
__host__ inline uint32_t block_magic_for(int block_size) {
    return block_size <= 1 ? 0xFFFFFFFFu : (uint32_t)((1ull << 32) / (uint32_t)block_size);
}

struct ChunkGeom {
    int u_first, n_units, upc, n_chunks;
};
__device__ __forceinline__ ChunkGeom chunk_geom(int u_lo, int u_hi, int max_chunks, int min_upc) {
    ChunkGeom g;
    g.u_first = u_lo >> 5;
    g.n_units = (u_hi >= u_lo) ? ((u_hi >> 5) - g.u_first + 1) : 0;
    int nc = fast_div(g.n_units + min_upc - 1, min_upc);
    if (nc > max_chunks) nc = max_chunks;
    if (nc < 1) nc = 1;
    g.upc = fast_div(g.n_units + nc - 1, nc);
    if (g.upc < 1) g.upc = 1;
    g.n_chunks = fast_div(g.n_units + g.upc - 1, g.upc);
    if (g.n_chunks < 1) g.n_chunks = 1;
    return g;
}

template <int H>
__device__ __forceinline__ void wht_stage(float (&v)[4], int lane) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float o = lane_xor<H>(v[k], lane);
        v[k] = (lane & H) ? (o - v[k]) : (v[k] + o);
    }
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
    wht_stage<1>(v, lane);
    wht_stage<2>(v, lane);
    wht_stage<4>(v, lane);
    wht_stage<8>(v, lane);
    wht_stage<16>(v, lane);
    wht_stage<32>(v, lane);
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] *= 0.0625f;
}

// centroid k as an immediate select chain (no constant-memory load on the critical path)
__device__ __forceinline__ float centroid_imm(int k) {
    const float m = (k & 4) ? ((k & 2) ? ((k & 1) ? 1.694104124e-1f : 1.285881878e-1f)
                                       : ((k & 1) ? 1.006979993e-1f : 7.824930800e-2f))
                            : ((k & 2) ? ((k & 1) ? 5.873210384e-2f : 4.094919437e-2f)
                                       : ((k & 1) ? 2.420087619e-2f : 8.008373692e-3f));
    return m;  // magnitude of centroid 8 + k; centroid[7 - k] = -m
}
__device__ __forceinline__ float centroid_of_code(int code) {
    return (code & 8) ? centroid_imm(code & 7) : -centroid_imm(7 - (code & 7));
}

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    f2 f = {a, b};
    h2 h = __builtin_convertvector(f, h2);
    return __builtin_bit_cast(uint32_t, h);
}
// Two fp16 operands for one fp32 weight pair: hi = fp16(w), lo = fp16(w - hi).  A value scale
// that is folded into the probabilities (w = p * d) reaches every element of a 128-wide scale
// block through ONE number; rounded to fp16 once, its error is the same for the whole block,
// and the inverse rotation gathers such a block-wide error into a single output channel
// (channel c ^ 128 of a channel c with large values).  With the low-order operand the weight
// carries 22 bits and that error disappears; the price is a second MFMA per value tile.
__device__ __forceinline__ void split_h2(float a, float b, uint32_t& hi, uint32_t& lo) {
    const h2 h = __builtin_convertvector(f2{a, b}, h2);
    hi = __builtin_bit_cast(uint32_t, h);
    // lo = fp16(a - hi.x) | fp16(b - hi.y) << 16: one mixed-precision FMA per half (x * 1 - h with
    // h read as fp16), the same value as widening, subtracting (exact) and rounding
    uint32_t l;
    asm("v_fma_mixlo_f16 %0, %1, 1.0, -%2 op_sel:[0,0,0] op_sel_hi:[0,0,1]" : "=v"(l) : "v"(a), "v"(hi));
    asm("v_fma_mixhi_f16 %0, %1, 1.0, -%2 op_sel:[0,0,1] op_sel_hi:[0,0,1]" : "+v"(l) : "v"(b), "v"(hi));
    lo = l;
}
// a * (fp16 half of w) as one mixed-precision FMA that reads the half in place (v_fma_mix_f32 with
// a zero addend; written as an fma so that the compiler forms it and places the wait states that
// separate it from the instruction that produced a).  A product of -0 comes out as +0.
__device__ __forceinline__ float mul_by_half_lo(float a, uint32_t w) {
    return __builtin_fmaf(a, (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xFFFFu)), 0.0f);
}
__device__ __forceinline__ float mul_by_half_hi(float a, uint32_t w) {
    return __builtin_fmaf(a, (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)), 0.0f);
}
// maximum of three finite values in one instruction (fmaxf would first quiet each operand); the
// operands must come from ordinary vector instructions: the compiler places no wait states in
// front of an assembly statement that reads the result of an MFMA
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float half_lo_to_f32(uint32_t w) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xFFFFu));
}
__device__ __forceinline__ float half_hi_to_f32(uint32_t w) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
}
// max / sum over the four 16-lane rows of a wave, result in every lane (pure VALU on gfx950)
__device__ __forceinline__ float max_over_rows(float x) {
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_over_rows(float x) {
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Table lookup: the dequantisation table sits at LDS address 0 (it is the start of the dynamic
// LDS block and the kernel has no static LDS), so the v_perm_b32 result IS the address.
typedef __attribute__((address_space(3))) const uint32_t lds_cu32;
typedef __attribute__((address_space(1))) const u4 global_cu4;
__device__ __forceinline__ uint32_t lut_read(uint32_t code_word, uint32_t lut_lane, uint32_t sel) {
    const uint32_t addr = __builtin_amdgcn_perm(code_word, lut_lane, sel);
    return *reinterpret_cast<lds_cu32*>((uintptr_t)addr);
}

// element index (0..255) of nibble i of aligned dword D of a TQ4 row, -1 for scale nibbles
__device__ __forceinline__ constexpr int tq4_dword_elem(int D, int i) {
    if (D == 0) return i >= 4 ? i - 4 : -1;
    if (D < 16) return 8 * D - 4 + i;
    if (D == 16) return i < 4 ? 124 + i : -1;
    return 128 + 8 * (D - 17) + i;
}
// dword read by k-block bk for QK MFMA m of half h (h=0: m 0..4, h=1: m 0..3).  The k-blocks of
// lanes 0-31 (bk 0,1) sit 8 dwords apart, which keeps the 32 simultaneous reads on 32 banks.
__device__ __forceinline__ constexpr int tq4_qk_dword(int h, int m, int bk) {
    const int base = 8 * (bk & 1) + 4 * (bk >> 1);
    if (h == 0) return m < 4 ? base + m : 16;
    return 17 + base + m;
}
// element index of V^T row r, nibble j, half h (PV MFMA output row -> head dimension)
__device__ __forceinline__ constexpr int tq4_pv_elem(int h, int j, int r) {
    if (h == 1) return 128 + 8 * r + j;
    if (r == 0) return j < 4 ? j : 120 + j;
    return 8 * r - 4 + j;
}

constexpr int kMergeGroups = 16;
constexpr int kMergeMaxPerGroup = 16;  // at most 256 partials per row

// ---- balanced decode ----------------------------------------------------------------------------
// A decode batch (at most one tile per request, no window, no token mask) is cut into equal
// shares of 32-token units, one share per workgroup, whatever the lengths of the requests: the
// units of all requests are laid end to end and workgroup x owns units [x S, (x + 1) S).  A share
// that crosses a request boundary is worked off piece by piece.  Piece (x, r) gets partial slot
// x + r: both grow along the pieces, so the slots are unique and those of one request are
// consecutive, first_wg(r) + r .. last_wg(r) + r.  The workgroup that owns a request's first
// piece records {first slot, number of pieces, token of the tile} for each of the request's
// query tokens in a per-token table for the merge kernel; the tokens of requests without work
// are recorded by workgroup (0, 0): pieces = 0 for a live request without visible keys (output
// zeros), -1 for a masked one and for tokens behind the last request (output untouched).
// Starting a piece (table, query rotation, first loads, merge of the waves) costs about as much
// as kBalPieceCost units of streaming, so every request is charged that many extra units in
// front of its real ones: a share that contains request boundaries gets fewer keys.
constexpr int kBalPieceCost = 32;
__host__ __device__ __forceinline__ size_t bal_partial_row(int slot, int kv_subs, int kv_sub, int col) {
    return ((size_t)slot * kv_subs + kv_sub) * 16 + col;
}

struct BalReq {  // request base + lane of a 64-request group
    int lo, hi, sa, cb, units;
    int cost;  // units + kBalPieceCost, 0 for a request without work
    int live;  // has query tokens and is not masked
};
__device__ __forceinline__ BalReq bal_load_req(const AttnParams& P, int r) {
    const warp34_attention_batch& B = P.B;
    BalReq q{0, 0, 0, 0, 0, 0, 0};
    if (r >= B.num_reqs) return q;
    q.lo = B.query_start_loc[r];
    q.hi = B.query_start_loc[r + 1];
    q.sa = B.seq_lens_after[r];
    const int q_len = q.hi - q.lo;
    q.cb = B.context_lens_before != nullptr ? B.context_lens_before[r] : q.sa - q_len;
    const bool live = q_len > 0 && (B.valid_req_mask == nullptr || B.valid_req_mask[r] != 0);
    int last = (B.mask_mode == WARP34_ATTN_MASK_NONCAUSAL_WINDOW) ? q.sa - 1 : q.cb + min(q_len, P.tok_tile) - 1;
    if (last >= q.sa) last = q.sa - 1;
    q.units = (live && last >= 0) ? (last >> 5) + 1 : 0;
    q.cost = q.units > 0 ? q.units + kBalPieceCost : 0;
    q.live = live ? 1 : 0;
    return q;
}
__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(v, off, 64);
        if (lane >= off) v += up;
    }
    return v;
}
// units per share for a batch of `total` units over `groups` workgroups
__device__ __forceinline__ int bal_share(int total, int groups, int min_share) {
    int s = (total + groups - 1) / groups;
    return s < min_share ? min_share : s;
}

// One piece of work of the balanced decode kernel: units [u_begin, u_end) of request `req`,
// the piece number `slot` (partials of a request occupy consecutive slots) and the number of
// pieces the request is cut into.
struct BalItem {
    int req, rq_start, rq_end, seq_after, ctx_before;
    int u_begin, u_end, n_chunks, slot;
};

// Tile lookup shared by the kernels that do not split it around other work (see the TQ4
// decode kernel for the scheme): blockIdx.z counts tiles; request z when no request can have
// two tiles, a prefix sum over the requests' tile counts otherwise.
struct TileInfo {
    bool hit;
    int req, rq_start, rq_end, seq_after, ctx_before, tile_in_req;
};
__device__ __forceinline__ TileInfo locate_tile(const AttnParams& P, int tile_z, int lane) {
    const warp34_attention_batch& B = P.B;
    TileInfo t{false, -1, 0, 0, 0, 0, 0};
    if (P.tiles_by_request) {
        t.req = tile_z;
        const int lo = B.query_start_loc[tile_z];
        const int hi = B.query_start_loc[tile_z + 1];
        const int sa = B.seq_lens_after[tile_z];
        const int cb = B.context_lens_before != nullptr ? B.context_lens_before[tile_z] : 0;
        const int rm = B.valid_req_mask != nullptr ? (int)B.valid_req_mask[tile_z] : 1;
        t.rq_start = __builtin_amdgcn_readfirstlane(lo);
        t.rq_end = __builtin_amdgcn_readfirstlane(hi);
        t.seq_after = __builtin_amdgcn_readfirstlane(sa);
        t.ctx_before = B.context_lens_before != nullptr ? __builtin_amdgcn_readfirstlane(cb)
                                                        : t.seq_after - (t.rq_end - t.rq_start);
        t.hit = __builtin_amdgcn_readfirstlane(rm) != 0 && t.rq_end > t.rq_start;
        return t;
    }
    int tiles_before = 0;
    for (int base = 0; base < B.num_reqs; base += 64) {
        const int r = base + lane;
        const bool inb = r < B.num_reqs;
        const int lo = inb ? B.query_start_loc[r] : 0;
        const int hi = inb ? B.query_start_loc[r + 1] : 0;
        const int sa = inb ? B.seq_lens_after[r] : 0;
        const int cb = (inb && B.context_lens_before != nullptr) ? B.context_lens_before[r] : 0;
        const int rm = (inb && B.valid_req_mask != nullptr) ? (int)B.valid_req_mask[r] : 1;
        const int cnt = hi > lo ? fast_div(hi - lo + P.tok_tile - 1, P.tok_tile) : 0;
        int incl = cnt;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(incl, off, 64);
            if (lane >= off) incl += up;
        }
        const int first = tiles_before + incl - cnt;
        const unsigned long long hits = __ballot(cnt > 0 && tile_z >= first && tile_z < first + cnt);
        if (hits != 0ull) {
            const int src = __builtin_ctzll(hits);
            t.req = base + src;
            t.rq_start = __builtin_amdgcn_readlane(lo, src);
            t.rq_end = __builtin_amdgcn_readlane(hi, src);
            t.seq_after = __builtin_amdgcn_readlane(sa, src);
            t.ctx_before = B.context_lens_before != nullptr ? __builtin_amdgcn_readlane(cb, src)
                                                            : t.seq_after - (t.rq_end - t.rq_start);
            t.tile_in_req = tile_z - __builtin_amdgcn_readlane(first, src);
            t.hit = __builtin_amdgcn_readlane(rm, src) != 0;
            return t;
        }
        tiles_before += __builtin_amdgcn_readlane(incl, 63);
    }
    return t;
}

// LDS-direct loads (gfx950): each active lane's 16 bytes go from global memory straight to LDS at
// m0 + OFFSET + lane * 16, without passing through registers; the immediate OFFSET is added to
// the global address as well.  Written as assembly so that
// the compiler does not know the instruction writes LDS: it would otherwise make every later
// table read (absolute addresses it cannot tell apart from the staging area) wait for the load
// unit.  The waits are placed by hand (wait_vm): loads return in order, so "all but the N most
// recent" is a safe condition whatever other loads the compiler has in flight.
// STREAM: the load carries the non-temporal hint (decode batches: every key is read by exactly one
// workgroup; a plain streaming read of HBM gains 8 to 13 % from the hint, the 32-sequence batch 2 %).
// One 16-row run (2112 bytes = 132 pieces of 16 bytes) is moved by three such instructions of 44
// lanes each, with M0 written once.
template <bool STREAM>
__device__ __forceinline__ void lds_load_run(uint32_t voffset, const uint8_t* sbase, uint32_t lds_addr) {
    if constexpr (STREAM) {
        asm volatile(
            "s_mov_b32 m0, %2\n\ts_nop 0\n\t"
            "global_load_lds_dwordx4 %0, %1 offset:0 nt\n\t"
            "global_load_lds_dwordx4 %0, %1 offset:704 nt\n\t"
            "global_load_lds_dwordx4 %0, %1 offset:1408 nt"
            :
            : "v"(voffset), "s"(sbase), "s"(lds_addr)
            : "memory");
    } else {
        asm volatile(
            "s_mov_b32 m0, %2\n\ts_nop 0\n\t"
            "global_load_lds_dwordx4 %0, %1 offset:0\n\t"
            "global_load_lds_dwordx4 %0, %1 offset:704\n\t"
            "global_load_lds_dwordx4 %0, %1 offset:1408"
            :
            : "v"(voffset), "s"(sbase), "s"(lds_addr)
            : "memory");
    }
}
// lane L of every row of 16 lanes, in all lanes of that row (one VALU move)
// value of the lane eight places on inside the row of 16 lanes (DPP row_ror:8)
__device__ __forceinline__ float row_ror8(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, true));
}
template <int L>
__device__ __forceinline__ uint32_t row_bcast(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x150 + L, 0xF, 0xF, true);  // row_newbcast:L
}
template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __forceinline__ void wait_lds_reads() { asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory"); }

// The work of one workgroup on one tile.  BAL = false: the tile and the chunk come from
// blockIdx (grid = chunks x (kv head, q subgroup) x tiles).  BAL = true: they come from `item`
// (balanced decode: every workgroup owns an equal share of the batch's units).
//
// LDS: [pair table 64 KB][kTq4Waves staging areas of 8448 B][query operand table 9216 B][(m, l) tables].
// A staging area holds one 32-token unit as it lies in the pages, written by LDS-direct loads:
// K rows 0-31, then V rows 0-31, 132 bytes each (four runs of 16 rows = 2112 bytes).
// SP: the keys below *P.key_floor belong to a shared-prefix pass (see AttnParams); a separate
// instantiation, so that the plain form carries no trace of it.
template <typename TQ, bool BAL, bool SP = false, bool STREAM = BAL>
__device__ __forceinline__ void tq4_tile(const AttnParams& P, uint8_t* smem, const BalItem& item, bool build_table) {
    static_assert(!(SP && BAL), "shared-prefix pass: split-K form only");
    constexpr int kWaves = kTq4Waves;
    uint8_t* stage_all = smem + kLutBytes;

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;  // MFMA column = query row of this lane; also A-operand row
    const int b = lane >> 4;  // MFMA k-block / output row group
    const warp34_kv_layer_layout& L = P.L;
    const warp34_attention_batch& B = P.B;

    // ---- tile identification ---------------------------------------------------------------------
    // blockIdx.z counts TILES (groups of tok_tile consecutive query tokens of one request), so
    // every workgroup that is launched has work.  When no request can have more than one tile
    // (max_q_len <= tok_tile, e.g. decode) tile z is request z; otherwise the tile is located
    // with a prefix sum over the requests' tile counts.
    const int tile_z = BAL ? item.req : (int)blockIdx.z;
    const int kv_sub = (int)blockIdx.y;
    const int kv_head = fast_div(kv_sub, P.q_subgroups);
    const int q_head_base = kv_head * P.gqa + (kv_sub - kv_head * P.q_subgroups) * P.q_group;
    const int chunk = BAL ? 0 : (int)blockIdx.x;

    // The request lookup goes first: its loads head the longest dependency chain of the prologue
    // (lengths -> chunk geometry -> page ids -> the first K / V loads).
    bool req_hit = false;
    int req = -1, rq_start = 0, rq_end = 0, seq_after = 0, ctx_before = 0, tile_in_req = 0;
    int spec_slot_base = -1, spec_vec = -1;
    int a_lo = 0, a_hi = 0, a_sa = 0, a_cb = 0, a_rm = 0;
    if constexpr (BAL) {
        req = item.req;
        rq_start = item.rq_start;
        rq_end = item.rq_end;
        seq_after = item.seq_after;
        ctx_before = item.ctx_before;
        req_hit = true;
        // the piece's first unit is known: its block-table slice is requested together with the
        // query rows
        spec_slot_base = div_block(item.u_begin * kUnit, P);
        const int slot = spec_slot_base + lane;
        if (slot < B.max_blocks_per_req) spec_vec = B.block_tables[(size_t)req * B.max_blocks_per_req + slot];
    } else if (P.tiles_by_request) {
        req = tile_z;  // < num_reqs by the launch geometry
        // Speculative block-table load, in flight together with the request's lengths: it
        // assumes that the request's length is the host's bound max_seq_len.  When the guess is
        // wrong the ids are fetched again below, so it changes the latency only, never the result.
        if (B.sliding_window <= 0 && B.max_seq_len > 0) {
            spec_slot_base = div_block(chunk * P.spec_upc * kUnit, P);
            const int slot = spec_slot_base + lane;
            if (slot < B.max_blocks_per_req)
                spec_vec = B.block_tables[(size_t)req * B.max_blocks_per_req + slot];
        }
        // one vector load per array (all lanes the same address), no scalar-cache round trip;
        // the values are made scalar after the table has been built, so that the build overlaps
        // the round trip
        a_lo = B.query_start_loc[req];
        a_hi = B.query_start_loc[req + 1];
        a_sa = B.seq_lens_after[req];
        a_cb = B.context_lens_before != nullptr ? B.context_lens_before[req] : 0;
        a_rm = B.valid_req_mask != nullptr ? (int)B.valid_req_mask[req] : 1;
    } else {
        const TileInfo ti = locate_tile(P, tile_z, lane);
        req = ti.req;
        rq_start = ti.rq_start;
        rq_end = ti.rq_end;
        seq_after = ti.seq_after;
        ctx_before = ti.ctx_before;
        tile_in_req = ti.tile_in_req;
        req_hit = ti.hit;
    }
    // While the request's lengths are on their way: the raw query rows of this wave's columns and
    // the table.  The first token of the tile is guessed (exact when every request has a whole
    // number of tiles); a wrong guess is corrected after the lookup.
    const int tok_guess = BAL ? item.rq_start
                              : min(P.tiles_by_request ? tile_z : tile_z * P.tok_tile, B.total_tokens - 1);
    constexpr int kColsPerWave = (16 + kWaves - 1) / kWaves;
    uint2 q_raw[kColsPerWave];
    auto load_q = [&](int tokbase) {
#pragma unroll
        for (int c = 0; c < kColsPerWave; ++c) {
            const int col = wave + c * kWaves;
            const int t = fast_div(col, P.q_group);
            const int a = col - t * P.q_group;
            q_raw[c] = uint2{0u, 0u};
            if (col < 16 && tokbase + t < B.total_tokens) {
                const uint16_t* qrow =
                    P.q + ((size_t)(tokbase + t) * P.num_q_heads + (size_t)(q_head_base + a)) * kHeadDim;
                q_raw[c] = *reinterpret_cast<const uint2*>(qrow + 4 * lane);
            }
        }
    };
    load_q(tok_guess);
    // validity of the token of this lane's column
    bool tok_ok;
    auto load_tok_ok_col = [&](int tokbase, int column) {
        const int tok = tokbase + fast_div(column, P.q_group);
        tok_ok = tok < B.total_tokens &&
                 (B.valid_token_mask == nullptr || B.valid_token_mask[min(tok, B.total_tokens - 1)] != 0);
    };
    auto load_tok_ok = [&](int tokbase) { load_tok_ok_col(tokbase, n); };
    load_tok_ok(tok_guess);

    if (build_table) {
        // entry e = (gain*centroid[e & 15], gain*centroid[e >> 4]) as packed fp16, 64 copies of 4 bytes.
        // Thread t writes the 16-byte slots t + 512 i (conflict-free), i.e. entries (t >> 4) + 32 i:
        // their low code (t >> 4) & 15 is the thread's own, their high code (t >> 8) + 2 i is the
        // same in the whole wave.  Lane j < 16 computes centroid j once; everything else is lane
        // traffic, so the build costs a few dozen instructions per wave.
        static_assert(kWaves == 8, "table build: 512 threads");
        const uint32_t c_bits = (uint32_t)F16::from_f32(kLutGain * centroid_of_code(lane & 15));
        const uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute(((tid >> 4) & 15) << 2, (int)c_bits);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)c_bits, (wave >> 2) + 2 * i);
            const uint32_t v = lo | (hi << 16);
            *reinterpret_cast<u4*>(smem + (tid + 512 * i) * 16) = u4{v, v, v, v};
        }
    }

    if (!BAL && P.tiles_by_request) {
        rq_start = __builtin_amdgcn_readfirstlane(a_lo);
        rq_end = __builtin_amdgcn_readfirstlane(a_hi);
        seq_after = __builtin_amdgcn_readfirstlane(a_sa);
        ctx_before = B.context_lens_before != nullptr ? __builtin_amdgcn_readfirstlane(a_cb)
                                                      : seq_after - (rq_end - rq_start);
        req_hit = __builtin_amdgcn_readfirstlane(a_rm) != 0 && rq_end > rq_start;
    }
    if (!req_hit) return;  // no such tile, empty or masked request: outputs untouched
    const int tok0 = rq_start + tile_in_req * P.tok_tile;
    if (tok0 != tok_guess) {  // wave-uniform, rare
        load_q(tok0);
        load_tok_ok(tok0);
    }

    int tile_tokens = rq_end - tok0;
    if (tile_tokens > P.tok_tile) tile_tokens = P.tok_tile;

    // A tile with at most eight columns (a decode step of up to eight query heads per kv head) runs
    // "packed": columns 8-15 repeat columns 0-7 -- same query, same scores, same probabilities -- and
    // carry the LOW-order fp16 part of the value weights where columns 0-7 carry the high-order
    // part, so one MFMA per value tile does the work of two.  The two halves are added up before
    // the waves merge.
    const bool pack = tile_tokens * P.q_group <= 8;  // wave-uniform
    const int ncol = pack ? (n & 7) : n;             // the query column this lane works for
    if (pack && ncol != n) load_tok_ok_col(tok0, ncol);

    // Column info: per lane (= per query column) the visible key range, and for the tile the union
    // and the intersection of the ranges.  Without a token mask and a window -- the common case --
    // the tile-wide values follow from scalars (every token of the tile is live, the ranges start
    // at 0 and their ends grow with the token: the union is the last token's range, the
    // intersection the first one's), and the per-lane part waits until the first loads are out.
    int col_lo = 0, col_hi = -1;
    bool col_ok = false;
    int u_lo = 0x7fffffff, u_hi = -1;  // union of the visible ranges
    int i_lo = 0, i_hi = 0x7fffffff;   // intersection of the visible ranges
    uint32_t ok_mask = 0u;             // bit c: column c is live (wave-uniform)
    const bool simple = B.valid_token_mask == nullptr && B.sliding_window <= 0;
    // keys below the floor were handled by the shared-prefix pass (a multiple of the unit size)
    int key_floor = 0;
    if constexpr (SP) key_floor = __builtin_amdgcn_readfirstlane(*P.key_floor);
    auto column_info = [&](bool accumulate) {
        const int t = fast_div(ncol, P.q_group);
        const int tok = tok0 + t;
        const bool ok = t < tile_tokens && tok_ok;
        const int q_off = tok - rq_start;
        int mx = (B.mask_mode == WARP34_ATTN_MASK_NONCAUSAL_WINDOW) ? seq_after - 1 : ctx_before + q_off;
        if (mx >= seq_after) mx = seq_after - 1;
        int mn = key_floor;
        if (B.sliding_window > 0) mn = max(key_floor, ctx_before + q_off - B.sliding_window + 1);
        col_ok = ok;
        col_lo = ok ? mn : 0;
        col_hi = ok ? mx : -1;
        if (accumulate && ok) {
            i_lo = max(i_lo, mn);
            i_hi = min(i_hi, mx);
            if (mn <= mx) {
                u_lo = min(u_lo, mn);
                u_hi = max(u_hi, mx);
            }
        }
        ok_mask = (uint32_t)(__ballot(ok) & (pack ? 0xFFull : 0xFFFFull));  // mirror columns produce no output
    };
    if (simple) {
        if (tok0 >= B.total_tokens) return;  // no live column
        const int q_off0 = tok0 - rq_start;
        const bool window = B.mask_mode == WARP34_ATTN_MASK_NONCAUSAL_WINDOW;
        int hi_first = window ? seq_after - 1 : ctx_before + q_off0;
        int hi_last = window ? seq_after - 1 : ctx_before + q_off0 + tile_tokens - 1;
        if (hi_first >= seq_after) hi_first = seq_after - 1;
        if (hi_last >= seq_after) hi_last = seq_after - 1;
        u_lo = key_floor;
        u_hi = hi_last >= key_floor ? hi_last : -1;
        i_lo = key_floor;
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
        if (ok_mask == 0u) return;  // whole tile masked: outputs untouched
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

    // ---- staging machinery ----------------------------------------------------------------------
    const uint8_t* k_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.k_base) +
                            (size_t)kv_head * L.k_head_stride_bytes;
    const uint8_t* v_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.v_base) +
                            (size_t)kv_head * L.v_head_stride_bytes;
    const uint32_t stage_addr = (uint32_t)(kLutBytes + wave * kStageTq4);  // LDS byte address (the block starts at 0)
    uint8_t* stage = stage_all + wave * kStageTq4;

    // The physical page ids come from ONE vector load per 64 block-table slots: lane l holds
    // the id of slot slot_base + l, a unit picks its two ids with readlane.  No scalar memory
    // loads remain in the loop (they share the LDS wait counter and would serialise it).
    const int32_t* req_blocks = B.block_tables + (size_t)req * B.max_blocks_per_req;
    int slot_base = div_block(cu_first * kUnit, P);
    int page_vec;
    // (Loaded and waited for in one assembly statement: were the load the compiler's, it would place
    // a vmcnt(0) in front of every readlane of page_vec -- once per unit -- and that wait, which
    // cannot tell the compiler's loads from the LDS-direct ones, would make every unit wait for all
    // the K / V data in flight.  The reload happens once per 64 block-table slots.)
    auto load_page_vec = [&]() {
        const int slot = slot_base + lane;
        int32_t ids = -1;
        if (slot < B.max_blocks_per_req) {
            const int32_t* src = req_blocks + slot;
            asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=v"(ids) : "v"(src) : "memory");
        }
        page_vec = ids;
    };
    // Runs that do not overlap the visible key range, or whose block-table entry is missing,
    // are read from page 0 of the slab instead: every row they deliver is masked, and any
    // TQ4 bytes dequantise to finite values.
    const uint8_t* nk[2];  // run bases of the unit that is loaded next (wave-uniform)
    const uint8_t* nv[2];
    auto locate_unit = [&](int unit) {
        if (P.unit_in_page) {  // uniform for the launch
            const int pos = unit * kUnit;
            const int page_slot = div_block(pos, P);
            const int in_page = pos - page_slot * L.block_size;
            int rel = page_slot - slot_base;
            if (rel >= 64) {  // wave-uniform, at most once per 64 slots
                slot_base = page_slot;
                load_page_vec();
                rel = 0;
            }
            const int32_t pg = __builtin_amdgcn_readlane(page_vec, rel);
            // (the unit overlaps the visible key range, so its page holds a visible key and its
            // block-table entry is a real page; rows of the unit outside the range are masked)
            const bool live = pg >= 0;
            const uint64_t tok_off = (uint64_t)((uint32_t)in_page * (uint32_t)kTq4RowBytes);
            const uint64_t koff = live ? (uint64_t)(uint32_t)pg * (uint32_t)L.k_page_stride_bytes + tok_off : 0;
            const uint64_t voff = live ? (uint64_t)(uint32_t)pg * (uint32_t)L.v_page_stride_bytes + tok_off : 0;
            nk[0] = k_base + koff;
            nk[1] = nk[0] + kRunBytes;
            nv[0] = v_base + voff;
            nv[1] = nv[0] + kRunBytes;
            return;
        }
#pragma unroll
        for (int gidx = 0; gidx < 2; ++gidx) {
            const int pos = unit * kUnit + 16 * gidx;
            const int page_slot = div_block(pos, P);
            const int in_page = pos - page_slot * L.block_size;
            int rel = page_slot - slot_base;
            if (rel >= 64) {  // wave-uniform, at most once per 64 slots
                slot_base = page_slot;
                load_page_vec();
                rel = 0;
            }
            const int32_t pg = __builtin_amdgcn_readlane(page_vec, rel);
            const bool live = pos <= u_hi && pos + 15 >= u_lo && pg >= 0;
            const size_t koff = live ? (size_t)pg * L.k_page_stride_bytes + (size_t)in_page * L.k_token_stride_bytes : 0;
            const size_t voff = live ? (size_t)pg * L.v_page_stride_bytes + (size_t)in_page * L.v_token_stride_bytes : 0;
            nk[gidx] = k_base + koff;
            nv[gidx] = v_base + voff;
        }
    };
    // six load instructions per half unit: a 16-row run is 2112 bytes = 132 pieces of 16 bytes, moved
    // by three instructions of 44 lanes each (the instruction's immediate offset moves the global
    // AND the LDS address, so the rows arrive contiguous, as they lie in the page)
    const uint32_t lane16 = (uint32_t)lane * 16u;
    auto issue_k = [&]() {
        if (lane < 44) {
#pragma unroll
            for (int r = 0; r < 2; ++r) lds_load_run<STREAM>(lane16, nk[r], stage_addr + r * kRunBytes);
        }
    };
    auto issue_v = [&]() {
        if (lane < 44) {
#pragma unroll
            for (int r = 0; r < 2; ++r) lds_load_run<STREAM>(lane16, nv[r], stage_addr + (2 + r) * kRunBytes);
        }
    };
    constexpr int kLoadsPerHalf = 6;

    // Units are dealt to the waves by a fixed rule, never handed out dynamically: which wave
    // sums which keys decides the floating-point result, and the output has to be the same bits
    // on every run and under every page permutation.  The rule deals the units to the four
    // SIMDs in turn and, inside a SIMD, to its waves in turn (wave w runs on SIMD w mod 4): with
    // a wave count that is not a multiple of four the SIMDs still get equal shares.
    const int simd = wave & 3, wslot = wave >> 2;
    const int simd_waves = (kWaves - simd + 3) / 4;
    auto nth_unit = [&](int j) -> int { return cu_first + 4 * (wslot + simd_waves * j) + simd; };

    // first unit's K half goes in flight before the rest of the prologue
    int unit = nth_unit(0);
    if (slot_base == spec_slot_base) {
        page_vec = spec_vec;
    } else {
        load_page_vec();
    }
    // The raw query rows are consumed after the first K / V loads have gone out.  Loads return in
    // order, so a wait for them placed behind those loads would wait for the K / V data as well:
    // the (empty) statement makes the compiler finish its own loads here, where they have long landed.
#pragma unroll
    for (int c = 0; c < kColsPerWave; ++c) asm volatile("" ::"v"(q_raw[c].x), "v"(q_raw[c].y));
    if (unit < cu_end) {
        locate_unit(unit);
        issue_k();  // (its V half follows below, behind the query operands)
    }
    if (simple) column_info(false);

    // ---- prologue: the query operand table ---------------------------------------------------------
    // B operands of the QK MFMAs, nine per lane (five for the first half-row, four for the second),
    // in the order the loop reads them: slot (n, b) holds 9 x 16 bytes.  Operand (h, m) of k-block
    // b pairs with row dword D = tq4_qk_dword(h, m, b); its eight elements (tq4_dword_elem) are
    // contiguous in the query row: dword D < 16 covers elements 8 D - 4 .. 8 D + 3 (the first four
    // are scale nibbles for D = 0 and stay zero), dword 16 elements 124 .. 127 and zeros, dword
    // 17 + k elements 128 + 8 k .. 128 + 8 k + 7.  A lane of the rotating wave holds elements
    // 4 lane .. 4 lane + 3 of its column, i.e. one half of one operand, and writes it there.
    // All the constant factors of the scores (softmax scale, log2 e, 1 / table gain) go into Q'.
    uint8_t* qop = stage_all + kWaves * kStageTq4;
    const float q_scale = B.sm_scale * kLog2e * kLutInvGain;
    // where this lane's four elements go: operand (k-block, mf) and which half of it
    int q_kb, q_mf, q_half;
    {
        int D, half;
        if (lane < 32) {
            D = (lane + 1) >> 1;
            half = (lane & 1) ? 0 : 1;
        } else {
            D = 17 + ((lane - 32) >> 1);
            half = lane & 1;
        }
        const int Dh = D < 17 ? D : D - 17;  // dword inside its half-row
        const int grp = (Dh >> 2) & 3;       // 4-dword group -> k-block (groups 1 and 2 swapped)
        q_kb = D == 16 ? 0 : (grp == 1 ? 2 : grp == 2 ? 1 : grp);
        q_mf = D == 16 ? 4 : (D < 16 ? (Dh & 3) : 5 + (Dh & 3));
        q_half = half;
    }
    static_assert(kColsPerWave == 2 && kWaves == 8, "a packed tile's mirror column col + 8 belongs to the wave of col");
    uint2 packed_prev = {0u, 0u};
#pragma unroll
    for (int c = 0; c < kColsPerWave; ++c) {
        const int col = wave + c * kWaves;
        if (col < 16) {  // wave-uniform
            float q_rot[4];
            q_rot[0] = TQ::to_f32((uint16_t)(q_raw[c].x & 0xFFFFu));
            q_rot[1] = TQ::to_f32((uint16_t)(q_raw[c].x >> 16));
            q_rot[2] = TQ::to_f32((uint16_t)(q_raw[c].y & 0xFFFFu));
            q_rot[3] = TQ::to_f32((uint16_t)(q_raw[c].y >> 16));
            const bool okc = (ok_mask >> col) & 1u;
            uint2 packed = {0u, 0u};
            if (pack && c == 1) {  // mirror column: the operands of column col - 8
                packed = packed_prev;
            } else if (okc) {  // dead columns stay zero: no need to rotate them
                if (P.rot_q) {  // keys stored rotated (uniform for the launch)
#pragma unroll
                    for (int k = 0; k < 4; ++k) q_rot[k] = apply_sign(q_rot[k], 4 * lane + k);
                    wht256_wave(q_rot, lane);
                }
                packed.x = pack_h2(q_rot[0] * q_scale, q_rot[1] * q_scale);
                packed.y = pack_h2(q_rot[2] * q_scale, q_rot[3] * q_scale);
            }
            packed_prev = packed;
            uint8_t* slot0 = qop + (size_t)(col * 4) * 144;
            *reinterpret_cast<uint2*>(slot0 + q_kb * 144 + q_mf * 16 + q_half * 8) = packed;
            // the parts no element maps to: the scale nibbles of dword 0 (k-block 0, operand 0,
            // first half), the second half of operand 4 in k-block 0, operand 4 of k-blocks 1-3
            if (lane < 8) {
                int zkb, zoff;
                if (lane == 0) {
                    zkb = 0; zoff = 0;
                } else if (lane == 1) {
                    zkb = 0; zoff = 4 * 16 + 8;
                } else {
                    zkb = 1 + (lane - 2) / 2; zoff = 4 * 16 + 8 * ((lane - 2) & 1);
                }
                *reinterpret_cast<uint2*>(slot0 + zkb * 144 + zoff) = uint2{0u, 0u};
            }
        }
    }
    // The V half of the first unit is requested only now, about 1 us after its K half.  At one
    // sequence all 2048 waves of the chip start together: asked for at once, the first K and V
    // halves are 17 MB that arrive over 3 us in no useful order; with the V halves held back the
    // K halves are there after half of that, the first scores are computed while the V halves
    // travel, and the call is 0.3 to 0.7 us shorter (three boxes, three rounds each).  The order
    // of the requests -- K then V -- is what the waits in the loop count on, and stays.
    if (unit < cu_end) issue_v();
    __syncthreads();  // the pair table and the query operands are complete

    // ---- per-wave state -----------------------------------------------------------------------
    const uint32_t lut_lane = (uint32_t)lane << 2;  // byte 0 of every table address
    const uint8_t* my_qop = qop + (size_t)(n * 4 + b) * 144;
    h8 bq[9];  // the query operands of this lane stay in registers
#pragma unroll
    for (int mf = 0; mf < 9; ++mf) bq[mf] = *reinterpret_cast<const h8*>(my_qop + 16 * mf);

    f4 o_acc[2][8];
    float m_run = kNegBig, l_run = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) o_acc[h][j] = f4{0.f, 0.f, 0.f, 0.f};

    // rows of the staging area: K rows 0-31, then V rows 0-31, 132 bytes each
    const uint8_t* ka_lo = stage + unit_token(0, n >> 2, n & 3) * kTq4RowBytes;  // A row of sub-tile 0; sub-tile 1: + 8 rows
    const uint8_t* kt_lo = stage + unit_token(0, b, 0) * kTq4RowBytes;           // token of output row 4b; + 8 s + i rows
    const uint8_t* vt_lo = kt_lo + 2 * kRunBytes;
    const uint32_t vt_lo_addr = stage_addr + (uint32_t)(2 * kRunBytes + unit_token(0, b, 0) * kTq4RowBytes);  // its LDS address
    const uint8_t* kt_n = kt_lo + (n & 3) * kTq4RowBytes;  // the token whose K scales this lane fetches (+ 8 s rows)
    const uint8_t* vt_n = vt_lo + (8 * ((n >> 2) & 1) + (n & 3)) * kTq4RowBytes;  // ... and V scales: token n & 7

    // one 32-token unit.  MASKED = false (wave-uniform) is the interior case: every token of the
    // unit is visible to every live column, so the compares / selects are branched over.
    // HAS_NEXT: the wave has another unit, whose two halves are requested as soon as the raw rows of
    // this unit's halves have been read out of the staging area.
    auto process_unit = [&](int t0, const bool MASKED, const bool HAS_NEXT) {
        // ---- raw K dwords and K scales -------------------------------------------------------------
        wait_vm<kLoadsPerHalf>();  // this unit's K half has landed (its V half may still be in flight)
        uint32_t kw[2][9], ksc[2][4];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const uint32_t* row32 = reinterpret_cast<const uint32_t*>(ka_lo + s * 8 * kTq4RowBytes);
#pragma unroll
            for (int mf = 0; mf < 9; ++mf) kw[s][mf] = row32[tq4_qk_dword(mf < 5 ? 0 : 1, mf < 5 ? mf : mf - 5, b)];
            // The two scales of token unit_token(s, b, i) in one register, d0 | d1 << 16.  The 16
            // lanes of a row need the same four tokens: lane n reads token n & 3 and the values
            // are handed round inside the row.
            const uint32_t* r32 = reinterpret_cast<const uint32_t*>(kt_n + 8 * s * kTq4RowBytes);
            const uint32_t mine = __builtin_amdgcn_perm(r32[16], r32[0], 0x07060100u);
            ksc[s][0] = row_bcast<0>(mine);
            ksc[s][1] = row_bcast<1>(mine);
            ksc[s][2] = row_bcast<2>(mine);
            ksc[s][3] = row_bcast<3>(mine);
        }
        wait_lds_reads();
        if (HAS_NEXT) issue_k();  // nk was located by the caller

        // ---- S^T = K Q'^T for the two 16-key sub-tiles ------------------------------------------
        // Six batches of three operands (twelve table reads, three MFMAs), software-pipelined: the
        // table reads of batch k + 1 are requested before the MFMAs of batch k are issued, so the
        // wave does not sit out the LDS latency of every batch.
        constexpr int kQkOrder[9] = {0, 5, 1, 6, 2, 7, 3, 8, 4};
        f4 s_acc[2][2];
#pragma unroll
        for (int s = 0; s < 2; ++s) s_acc[s][0] = s_acc[s][1] = f4{0.f, 0.f, 0.f, 0.f};
        u4 qa[2][3];
        auto qk_reads = [&](int bt, u4 (&a)[3]) {
            const int s = bt / 3;
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                const uint32_t w = kw[s][kQkOrder[3 * (bt % 3) + k]];
                a[k][0] = lut_read(w, lut_lane, 0x0c0c0400u);
                a[k][1] = lut_read(w, lut_lane, 0x0c0c0500u);
                a[k][2] = lut_read(w, lut_lane, 0x0c0c0600u);
                a[k][3] = lut_read(w, lut_lane, 0x0c0c0700u);
            }
        };
        qk_reads(0, qa[0]);
#pragma unroll
        for (int bt = 0; bt < 6; ++bt) {
            if (bt + 1 < 6) qk_reads(bt + 1, qa[(bt + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            const int s = bt / 3;
#pragma unroll
            for (int k = 0; k < 3; ++k) {
                const int mf = kQkOrder[3 * (bt % 3) + k];
                const int h = mf < 5 ? 0 : 1;
                s_acc[s][h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, qa[bt & 1][k]), bq[mf],
                                                                    s_acc[s][h], 0, 0, 0);
            }
        }
        // rows 4b+i of the result are tokens unit_token(s, b, i); apply the K scales
        float sc[8];
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                sc[4 * s + i] = __builtin_fmaf(s_acc[s][1][i], half_hi_to_f32(ksc[s][i]), mul_by_half_lo(s_acc[s][0][i], ksc[s][i]));
        if (MASKED) {
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int pos = t0 + unit_token(t >> 2, b, t & 3);
                const bool vis = col_ok && pos >= col_lo && pos <= col_hi;
                sc[t] = vis ? sc[t] : kNegBig;
            }
        }

        // ---- raw V dwords of this lane's 8 tokens ------------------------------------------
        if (HAS_NEXT) {
            wait_vm<kLoadsPerHalf>();  // the V half has landed; the next K half may be in flight
        } else {
            wait_vm<0>();
        }
        // per token: the two scales (d0 | d1 << 16), the dword of the first half-row that holds this
        // lane's codes (dword n; for n = 0 codes 0-3 and 124-127 are put together from dwords 0 and
        // 16) and the dword of the second half-row
        uint32_t vsc[8], vw[2][8];
        {
            // lane n reads dwords 0 and 16 of token n & 7 (of the eight this row of lanes works on)
            // and hands the scale pair and the n = 0 column round inside the row
            const uint32_t* r32 = reinterpret_cast<const uint32_t*>(vt_n);
            const uint32_t d0 = r32[0], d16 = r32[16];
            const uint32_t mine_sc = __builtin_amdgcn_perm(d16, d0, 0x07060100u);
            const uint32_t mine_c0 = __builtin_amdgcn_alignbit(d16, d0, 16);
            uint32_t c0[8];
            vsc[0] = row_bcast<0>(mine_sc); c0[0] = row_bcast<0>(mine_c0);
            vsc[1] = row_bcast<1>(mine_sc); c0[1] = row_bcast<1>(mine_c0);
            vsc[2] = row_bcast<2>(mine_sc); c0[2] = row_bcast<2>(mine_c0);
            vsc[3] = row_bcast<3>(mine_sc); c0[3] = row_bcast<3>(mine_c0);
            vsc[4] = row_bcast<4>(mine_sc); c0[4] = row_bcast<4>(mine_c0);
            vsc[5] = row_bcast<5>(mine_sc); c0[5] = row_bcast<5>(mine_c0);
            vsc[6] = row_bcast<6>(mine_sc); c0[6] = row_bcast<6>(mine_c0);
            vsc[7] = row_bcast<7>(mine_sc); c0[7] = row_bcast<7>(mine_c0);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const uint32_t* row32 = reinterpret_cast<const uint32_t*>(vt_lo + (8 * (t >> 2) + (t & 3)) * kTq4RowBytes);
                // (lane n = 0 reads dword 0 and drops it; the read is volatile so that it stays one
                // unconditional instruction instead of a branch around the lanes with n = 0, and goes
                // through an LDS-typed address: a volatile read through a generic pointer would be a
                // FLAT load, which completes out of order with the LDS-direct loads and would break
                // the hand-placed vmcnt waits)
                typedef __attribute__((address_space(3))) const volatile uint32_t lds_vol_u32;
                const uint32_t first_half = *reinterpret_cast<lds_vol_u32*>(
                    (uintptr_t)(vt_lo_addr + (uint32_t)((8 * (t >> 2) + (t & 3)) * kTq4RowBytes + 4 * n)));
                vw[0][t] = n == 0 ? c0[t] : first_half;
                vw[1][t] = row32[17 + n];
            }
        }
        wait_lds_reads();
        if (HAS_NEXT) issue_v();

        // ---- online softmax (log2 domain), per lane = per query column --------------------
        float p[8];
        {
            float mx = fmaxf(max3(sc[0], sc[1], sc[2]), max3(sc[3], sc[4], max3(sc[5], sc[6], sc[7])));
            mx = max_over_rows(mx);
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            float psum = 0.f;
            // (the MASKED tests sit outside the unrolled loops: one wave-uniform branch per block
            // instead of one per element, and the eight exponentials can overlap)
#pragma unroll
            for (int t = 0; t < 8; ++t) p[t] = __builtin_amdgcn_exp2f(sc[t] - m_new);
            if (MASKED) {
#pragma unroll
                for (int t = 0; t < 8; ++t) p[t] = sc[t] > 0.5f * kNegBig ? p[t] : 0.f;
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
        }

        // ---- O^T += V^T P^T ------------------------------------------------------------------
        // weights of each half: probability times the half-row scale of the value row, as a high
        // and a low fp16 operand (split_h2)
        if (MASKED) {
            // masked tokens have p == 0; their scale pair is zeroed so that a garbage scale (rows
            // beyond the sequence end) cannot inject NaN into the weights
#pragma unroll
            for (int t = 0; t < 8; ++t) vsc[t] = p[t] > 0.f ? vsc[t] : 0u;
        }
        u4 ph[2], pl[2];
        uint32_t lo[2][4], hi[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float w[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) w[t] = h == 0 ? mul_by_half_lo(p[t], vsc[t]) : mul_by_half_hi(p[t], vsc[t]);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                uint32_t whi, wlo;
                split_h2(w[2 * k], w[2 * k + 1], whi, wlo);
                ph[h][k] = (pack && (n & 8)) ? wlo : whi;  // packed: the mirror columns take the low-order part
                pl[h][k] = wlo;
                const uint32_t wa = vw[h][2 * k], wb = vw[h][2 * k + 1];
                // byte q of lo / hi = (nibble 2q / 2q+1 of token a) | (same nibble of token b) << 4
                lo[h][k] = (wa & 0x0F0F0F0Fu) | ((wb << 4) & 0xF0F0F0F0u);
                hi[h][k] = ((wa >> 4) & 0x0F0F0F0Fu) | (wb & 0xF0F0F0F0u);
            }
        }
        // four batches of four value tiles (16 table reads, eight MFMAs), pipelined like the QK batches
        u4 va[2][4];
        auto pv_reads = [&](int bt, u4 (&a)[4]) {
            const int h = bt >> 1;
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const int j = 4 * (bt & 1) + jj;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t src = (j & 1) ? hi[h][k] : lo[h][k];
                    const uint32_t sel = 0x0c0c0400u + ((uint32_t)(j >> 1) << 8);
                    a[jj][k] = lut_read(src, lut_lane, sel);
                }
            }
        };
        pv_reads(0, va[0]);
#pragma unroll
        for (int bt = 0; bt < 4; ++bt) {
            if (bt + 1 < 4) pv_reads(bt + 1, va[(bt + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            const int h = bt >> 1;
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const int j = 4 * (bt & 1) + jj;
                const h8 av = __builtin_bit_cast(h8, va[bt & 1][jj]);
                o_acc[h][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, __builtin_bit_cast(h8, ph[h]), o_acc[h][j], 0, 0, 0);
            }
            if (!pack) {
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    const int j = 4 * (bt & 1) + jj;
                    const h8 av = __builtin_bit_cast(h8, va[bt & 1][jj]);
                    o_acc[h][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, __builtin_bit_cast(h8, pl[h]), o_acc[h][j], 0, 0, 0);
                }
            }
        }
    };

    for (int j = 0; unit < cu_end; ++j) {
        const int next_unit = nth_unit(j + 1);
        const bool has_next = next_unit < cu_end;
        if (has_next) locate_unit(next_unit);
        const int t0 = unit * kUnit;
        const bool masked = !(t0 >= i_lo && t0 + kUnit - 1 <= i_hi);
        // The two waves of a SIMD take turns at the higher issue priority, unit by unit: left alone,
        // the arbiter favours the older wave every time and the younger one finishes its units late.
        if ((j + wslot) & 1) {
            __builtin_amdgcn_s_setprio(1);
        } else {
            __builtin_amdgcn_s_setprio(0);
        }
        process_unit(t0, masked, has_next);
        unit = next_unit;
    }
    __builtin_amdgcn_s_setprio(0);
    wait_vm<0>();  // nothing of this wave may still be on its way into LDS when the areas are reused

    // ---- packed tile: column n += its mirror column n + 8 (the low-order share of the weights) ----
    // Both lanes of a pair end up with sums, and both take part in the stores below: lane n < 8 keeps
    // the value tiles with even j in the even slots, its mirror lane those with odd j.
    if (pack) {
        const bool upper = (n & 8) != 0;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float even = o_acc[h][2 * i][k], odd = o_acc[h][2 * i + 1][k];
                    const float keep = upper ? odd : even;   // this lane's tile of the pair
                    const float give = upper ? even : odd;   // what the mirror lane keeps
                    o_acc[h][2 * i][k] = keep + row_ror8(give);
                }
    }

    // ---- combine the per-lane partial sums of l over the four k-block lanes of a column ------
    l_run = sum_over_rows(l_run);

    // ---- merge the waves' states through LDS ---------------------------------------------------
    // Every wave publishes (m, l) and its O, as it stands, in its own region -- its own staging area,
    // which nobody else touches, so the stores need not wait for the other waves -- and after ONE
    // barrier wave c adds up column c of the eight regions, each weighted by 2^(m_w - m_tot), in wave
    // order.  A region holds eight columns: a tile with live columns in both halves (more than
    // eight columns, never a decode step) takes a second pass.
    // Region layout: column stride kMergeColStride dwords; inside a column the four values a lane
    // holds for one MFMA result (rows 4b..4b+3 of (h, j)) are contiguous at ((h*8 + j)*4 + b)*4,
    // so a lane stores them with one 128-bit write and the adding wave reads one 128-bit piece per
    // lane and region.  The sums reach the element order of the head dimension (lane l: elements
    // 4 l .. 4 l + 3) through a 1 KB transposition buffer per wave in the idle query operand table.
    constexpr int kColStride = kMergeColStride;
    constexpr int kRegion = 8 * kColStride;
    static_assert(kRegion * 4 == kStageTq4, "a wave's merge region is its own staging area");
    static_assert(kWaves * 1024 <= kQopBytes, "transposition buffers");
    float* xbuf = reinterpret_cast<float*>(stage_all);
    float* tbuf = reinterpret_cast<float*>(qop) + wave * 256;
    // [kWaves][16][2]: in an area of its own, a wave publishes its state while others are still in their loops
    float* mlbuf = reinterpret_cast<float*>(smem + ml_offset_for(1));
    static_assert(kWaves * kRegion == merge_floats_for(1), "merge layout");
    if (b == 0) {
        mlbuf[(wave * 16 + n) * 2 + 0] = m_run;
        mlbuf[(wave * 16 + n) * 2 + 1] = l_run;
    }
    auto store_region = [&](int half) {
        float* c = xbuf + wave * kRegion + (n & 7) * kColStride;
        if (pack) {  // (half 0) all 64 lanes store: eight tiles each, see above
            if (col_ok) {
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        *reinterpret_cast<f4*>(c + ((h * 8 + 2 * i + (n >> 3)) * 4 + b) * 4) = o_acc[h][2 * i];
            }
        } else if ((n >> 3) == half && col_ok) {  // dead columns are never read back
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < 8; ++j) *reinterpret_cast<f4*>(c + ((h * 8 + j) * 4 + b) * 4) = o_acc[h][j];
        }
    };
    const bool live0 = (ok_mask & 0xFFu) != 0u, live1 = (ok_mask >> 8) != 0u;  // the same in every wave
    store_region(live0 ? 0 : 1);

    int merge_slot[4];  // region slot of element 4*lane + k (inverse of tq4_pv_elem)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int e = 4 * lane + k;
        int h, j, r;
        if (e >= 128) {
            h = 1; r = (e - 128) >> 3; j = e & 7;
        } else if (e < 4) {
            h = 0; r = 0; j = e;
        } else if (e >= 124) {
            h = 0; r = 0; j = e - 120;
        } else {
            h = 0; r = (e + 4) >> 3; j = (e + 4) & 7;
        }
        merge_slot[k] = ((h * 8 + j) * 4 + (r >> 2)) * 4 + (r & 3);
    }
    __syncthreads();  // every wave is done with the table, and the regions of the first pass are there
#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
        if (!(half ? live1 : live0)) continue;
        if (half == 1 && live0) {
            __syncthreads();  // the first pass has read the regions
            store_region(1);
            __syncthreads();
        }
        const int col = 8 * half + wave;
        if (wave < 8 && ((ok_mask >> col) & 1u)) {
            // state of the column in the eight waves (the same addresses in every lane)
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
                tot += *reinterpret_cast<const f4*>(xbuf + w * kRegion + wave * kColStride + 4 * lane) * wgt;
            }
            *reinterpret_cast<f4*>(tbuf + 4 * lane) = tot;
            // element e = 4*lane + k is value (h, j, row r) with e = tq4_pv_elem(h, j, r); the reads
            // follow the write of the same wave in LDS order
            float v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = tbuf[merge_slot[k]];
            const int t = fast_div(col, P.q_group);
            const int a = col - t * P.q_group;
            const size_t row = (size_t)(tok0 + t) * P.num_q_heads + (size_t)(q_head_base + a);
            if (BAL ? item.n_chunks > 1 : P.max_chunks > 1) {
                // un-normalised, rotated, still carrying the table gain; the merge kernel finishes
                const size_t prow = BAL ? bal_partial_row(item.slot, (int)gridDim.y, kv_sub, col)
                                        : row * (SP ? P.part_stride : P.max_chunks) + chunk;
                float* dst = P.part_acc + prow * kHeadDim;
                *reinterpret_cast<f4*>(dst + 4 * lane) = f4{v[0], v[1], v[2], v[3]};
                if (lane == 0) {
                    // (m, l, number of chunks of this row, -): one record per chunk, every record
                    // carries the count so the merge needs no dependent load
                    *reinterpret_cast<f4*>(P.part_ml + prow * 4) = f4{m_col, l_col, (float)g.n_chunks, 0.f};
                }
            } else {
                const float inv = l_col > 0.f ? kLutInvGain / l_col : 0.f;
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] *= inv;
                if (P.rot_out) {  // values stored rotated
                    wht256_wave(v, lane);
#pragma unroll
                    for (int k = 0; k < 4; ++k) v[k] = apply_sign(v[k], 4 * lane + k);
                }
                store_out_row<TQ>(P, row, lane, v);
            }
        }
    }
}

template <typename TQ, int NT, bool SP = false>
__global__ __launch_bounds__(kTq4Waves * 64, 1) void paged_attn_tq4_kernel(const AttnParams P) {
    static_assert(NT == 1, "one 16-column tile per workgroup");
    extern __shared__ __align__(16) uint8_t smem[];
    // lut_read() addresses the table absolutely: the dynamic block starts at LDS address 0 because
    // the kernel has no static LDS (checked on the host before the first launch)
    // decode steps (no request has more than one tile): every key is read by one workgroup only,
    // the loads carry the streaming hint; one body per kind of load
    if (!SP && P.tiles_by_request != 0 && P.q_subgroups == 1) {  // uniform for the grid
        tq4_tile<TQ, false, SP, true>(P, smem, BalItem{}, true);
    } else {
        tq4_tile<TQ, false, SP, false>(P, smem, BalItem{}, true);
    }
}

// Balanced decode: grid = (groups, kv head x q subgroup).  Every wave computes the plan (the
// loads are the same addresses in every wave of the chip and stay in cache) and calls
// tile(piece) for the pieces of its workgroup's share, in order.
template <typename TileFn>
__device__ __forceinline__ void bal_for_each_piece(const AttnParams& P, TileFn&& tile) {
    const int lane = (int)threadIdx.x & 63;
    const int num_reqs = P.B.num_reqs;
    // the first 64 requests are loaded once: their lane values serve the total and the search for
    // the first piece (most workgroups have exactly one piece, most batches at most 64 requests)
    const BalReq q0 = bal_load_req(P, lane);
    const int incl0 = wave_incl_scan(q0.cost, lane);
    int total = __builtin_amdgcn_readlane(incl0, 63);
    // wave 0 of workgroup (0, 0) records the requests no workgroup will work on
    const bool recorder = blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x < 64;
    auto record_idle = [&](const BalReq& q, int r) {
        if (!recorder || r >= num_reqs) return;
        if (q.units == 0) {
            for (int t = q.lo; t < q.hi && t < P.B.total_tokens; ++t)
                *reinterpret_cast<int4*>(P.bal_table + 4 * (size_t)t) = int4{0, q.live ? 0 : -1, t - q.lo, 0};
        }
        if (r == num_reqs - 1) {
            for (int t = max(q.hi, 0); t < P.B.total_tokens; ++t)
                *reinterpret_cast<int4*>(P.bal_table + 4 * (size_t)t) = int4{0, -1, 0, 0};
        }
    };
    record_idle(q0, lane);
    for (int base = 64; base < num_reqs; base += 64) {
        const BalReq q = bal_load_req(P, base + lane);
        record_idle(q, base + lane);
        total += __builtin_amdgcn_readlane(wave_incl_scan(q.cost, lane), 63);
    }
    const int share = bal_share(total, (int)gridDim.x, P.min_upc + kBalPieceCost);
    const int my_begin = (int)blockIdx.x * share;
    int my_end = my_begin + share;
    if (my_end > total) my_end = total;
    if (my_begin >= total) return;

    // The pieces of this share, in order.  Nothing but a few scalars stays live across a tile:
    // the 64-request group that holds the next piece is loaded and scanned again after each one.
    int base = 0, before = 0, taken = 0;  // group, units before it, pieces of it already done
    BalItem it{};
    int piece_end = 0;
    // next piece inside the group whose lane values are (q, incl); false: the group has none left
    auto scan_group = [&](const BalReq& q, int incl) -> bool {
        const int start = before + incl - q.units;  // of the real units, behind the charge
        unsigned long long hits = __ballot(q.units > 0 && start < my_end && start + q.units > my_begin);
        for (int skip = 0; skip < taken && hits != 0ull; ++skip) hits &= hits - 1ull;
        if (hits == 0ull) {
            before += __builtin_amdgcn_readlane(incl, 63);
            base += 64;
            taken = 0;
            return false;
        }
        const int src = __builtin_ctzll(hits);
        const int r_start = __builtin_amdgcn_readlane(start, src);
        const int r_units = __builtin_amdgcn_readlane(q.units, src);
        it.req = base + src;
        it.rq_start = __builtin_amdgcn_readlane(q.lo, src);
        it.rq_end = __builtin_amdgcn_readlane(q.hi, src);
        it.seq_after = __builtin_amdgcn_readlane(q.sa, src);
        it.ctx_before = __builtin_amdgcn_readlane(q.cb, src);
        it.u_begin = max(my_begin, r_start) - r_start;
        it.u_end = min(my_end, r_start + r_units) - r_start;
        it.n_chunks = (r_start + r_units - 1) / share - r_start / share + 1;
        it.slot = (int)blockIdx.x + it.req;
        piece_end = r_start + it.u_end;
        if (it.u_begin == 0 && blockIdx.y == 0 && (int)threadIdx.x < it.rq_end - it.rq_start &&
            it.rq_start + (int)threadIdx.x < P.B.total_tokens) {  // first piece: one entry per query token
            *reinterpret_cast<int4*>(P.bal_table + 4 * (size_t)(it.rq_start + (int)threadIdx.x)) =
                int4{it.slot, it.n_chunks, (int)threadIdx.x, 0};
        }
        ++taken;
        return true;
    };
    auto find_next = [&]() -> bool {
        while (base < num_reqs && before < my_end) {
            const BalReq q = bal_load_req(P, base + lane);
            if (scan_group(q, wave_incl_scan(q.cost, lane))) return true;
        }
        return false;
    };
    bool have = scan_group(q0, incl0);
    if (!have) have = find_next();
    while (have) {
        tile(it);
        if (piece_end >= my_end) break;  // the share ends with this piece
        __syncthreads();  // the tile's merge regions alias what the next piece sets up
        have = find_next();
    }
}

template <typename TQ>
__global__ __launch_bounds__(kTq4Waves * 64, 1) void paged_attn_tq4_balanced_kernel(const AttnParams P) {
    extern __shared__ __align__(16) uint8_t smem[];
    // the pair table survives a piece (the merge regions lie in the staging areas): built once
    bool first = true;
    bal_for_each_piece(P, [&](const BalItem& it) {
        tq4_tile<TQ, true>(P, smem, it, first);
        first = false;
    });
}

// Merge for the balanced decode kernel: one workgroup of 1024 threads per (token, q head) row.
// The token's table entry says where its partials are; rows whose request was not cut (one
// piece) were finished by the attention kernel, rows of live requests without visible keys are
// zero, rows of masked requests stay untouched.
template <typename TQ>
__global__ __launch_bounds__(1024) void balanced_merge_kernel(const AttnParams P, int kv_subs, float out_scale,
                                                              int rotate) {
    __shared__ f4 s_acc[kMergeGroups][64];
    __shared__ f4 s_rec[256];
    __shared__ float s_red[kMergeGroups];
    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int grp = tid >> 6;
    const long long row = (long long)blockIdx.x;
    const int tok = (int)(row / P.num_q_heads);
    const int head = (int)(row - (long long)tok * P.num_q_heads);
    const int4 entry = *reinterpret_cast<const int4*>(P.bal_table + 4 * (size_t)tok);  // same address in every lane
    const int n_chunks = entry.y;
    if (n_chunks < 0 || n_chunks == 1) return;  // masked, or finished by the attention kernel
    if (n_chunks == 0) {                        // no visible key: zeros
        const float zero[4] = {0.f, 0.f, 0.f, 0.f};
        if (grp == 0) store_out_row<TQ>(P, (size_t)row, lane, zero);
        return;
    }
    const int col = entry.z * P.q_group + head % P.q_group;
    const int kv_sub = head / P.q_group;  // = kv_head * q_subgroups + subgroup
    const size_t prow0 = bal_partial_row(entry.x, kv_subs, kv_sub, col);
    const size_t pstride = (size_t)kv_subs * 16;  // partial rows between consecutive slots
    if (tid < n_chunks && tid < 256) s_rec[tid] = *reinterpret_cast<const f4*>(P.part_ml + (prow0 + tid * pstride) * 4);
    f4 a[kMergeMaxPerGroup];
#pragma unroll
    for (int k = 0; k < kMergeMaxPerGroup; ++k) {
        const int s = grp + k * kMergeGroups;
        a[k] = f4{0.f, 0.f, 0.f, 0.f};
        if (s < n_chunks) a[k] = *reinterpret_cast<const f4*>(P.part_acc + (prow0 + s * pstride) * kHeadDim + 4 * lane);
    }
    __syncthreads();
    float m_tot = kNegBig;
    for (int s = lane; s < n_chunks; s += 64) {
        const f4 r = s_rec[s];
        if (r[1] > 0.f) m_tot = fmaxf(m_tot, r[0]);
    }
    m_tot = fmaxf(m_tot, lane_xor<1>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<2>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<4>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<8>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<16>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<32>(m_tot, lane));
    f4 v = {0.f, 0.f, 0.f, 0.f};
    float l_part = 0.f;
#pragma unroll
    for (int k = 0; k < kMergeMaxPerGroup; ++k) {
        const int s = grp + k * kMergeGroups;
        if (s < n_chunks) {
            const f4 r = s_rec[s];
            if (r[1] > 0.f) {
                const float w = __builtin_amdgcn_exp2f(r[0] - m_tot);
                l_part += r[1] * w;
                v += a[k] * w;
            }
        }
    }
    s_acc[grp][lane] = v;
    if (lane == 0) s_red[grp] = l_part;
    __syncthreads();
    if (grp != 0) return;
    float l_tot = 0.f;
    f4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < kMergeGroups; ++k) {
        tot += s_acc[k][lane];
        l_tot += s_red[k];
    }
    const float inv = l_tot > 0.f ? out_scale / l_tot : 0.f;
    float o[4] = {tot[0] * inv, tot[1] * inv, tot[2] * inv, tot[3] * inv};
    if (rotate) {
        wht256_wave(o, lane);
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = apply_sign(o[k], 4 * lane + k);
    }
    store_out_row<TQ>(P, (size_t)row, lane, o);
}

// Merge of the split-K partials (op_paged_attn.cu:1132-1218): m_tot = max m_s,
// w_s = 2^(m_s - m_tot), out = sum acc_s w_s / sum l_s w_s, then one inverse rotation.
// One workgroup of 1024 threads per (token, q head) row: 16 groups of 64 threads stride the
// chunks, each thread owns 4 of the 256 columns; the groups are summed through LDS.
// Everything the row needs (validity, chunk records, accumulators) is requested in ONE memory
// round trip: records and accumulators of all max_chunks slots are loaded speculatively and
// the slots beyond the row's chunk count are discarded with selects.
template <typename TQ, bool SP = false, int HD = kHeadDim>
__global__ __launch_bounds__(1024) void split_merge_kernel(const float* part_acc_in, const float* part_ml_in,
                                                           int max_chunks_in, const AttnParams P,
                                                           float out_scale, int rotate) {
    __shared__ f4 s_acc[kMergeGroups][64];
    __shared__ f4 s_rec[256];
    __shared__ float s_red[kMergeGroups];
    __shared__ int s_valid;
    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int grp = tid >> 6;
    const long long row = (long long)blockIdx.x;
    const int tok = (int)(row / P.num_q_heads);
    const warp34_attention_batch& B = P.B;
    // the leading arguments repeat P.part_acc / P.part_ml / P.max_chunks: they are preloaded into
    // scalar registers at wave launch, so the speculative loads below do not wait for the
    // kernel-argument fetch
    const float* ml = part_ml_in + (size_t)row * max_chunks_in * 4;
    const float* acc = part_acc_in + (size_t)row * max_chunks_in * kHeadDim;

    // speculative loads: chunk records (one per thread) and this thread's accumulator slices
    f4 rec = {kNegBig, 0.f, 0.f, 0.f};
    if (tid < max_chunks_in) rec = *reinterpret_cast<const f4*>(ml + 4 * tid);
    f4 a[kMergeMaxPerGroup];
#pragma unroll
    for (int k = 0; k < kMergeMaxPerGroup; ++k) {
        const int s = grp + k * kMergeGroups;
        a[k] = f4{0.f, 0.f, 0.f, 0.f};
        // (records keep a 256-float stride at every head dimension; lanes beyond the row load nothing)
        if (s < max_chunks_in && (HD == 256 || 4 * lane < HD))
            a[k] = *reinterpret_cast<const f4*>(acc + (size_t)s * kHeadDim + 4 * lane);
    }
    // row validity (wave 0): token mask and owning request, first match wins
    if (grp == 0) {
        bool ok = B.valid_token_mask == nullptr || B.valid_token_mask[tok] != 0;
        bool found = false;
        for (int base = 0; base < B.num_reqs && !found; base += 64) {
            const int r = base + lane;
            const bool inb = r < B.num_reqs;
            const int lo = inb ? B.query_start_loc[r] : 0x7fffffff;
            const int hi = inb ? B.query_start_loc[r + 1] : -0x7fffffff;
            const int rm = (inb && B.valid_req_mask != nullptr) ? (int)B.valid_req_mask[r] : 1;
            const unsigned long long hits = __ballot(inb && tok >= lo && tok < hi);
            if (hits != 0ull) {
                found = true;
                ok = ok && __builtin_amdgcn_readlane(rm, __builtin_ctzll(hits)) != 0;
            }
        }
        if (lane == 0) s_valid = (ok && found) ? 1 : 0;
    }
    if (tid < 256) s_rec[tid] = rec;
    __syncthreads();
    if (!s_valid) return;  // masked row: output untouched (uniform for the block)
    int n_chunks = (int)s_rec[0][2];
    if (n_chunks > P.max_chunks) n_chunks = P.max_chunks;
    // slots of the row: its split-K chunks, then (SP, behind a gap) those of the shared-prefix pass
    auto live_slot = [&](int s) {
        if constexpr (SP) return s < n_chunks || (s >= P.pf_slot_base && s < P.pf_slot_base + P.pf_split);
        return s < n_chunks;
    };
    const int n_slots = SP ? max_chunks_in : n_chunks;

    // global maximum of m over chunks with l > 0 (every thread scans the LDS copy)
    float m_tot = kNegBig;
    for (int s = lane; s < n_slots; s += 64) {
        if (!live_slot(s)) continue;
        const f4 r = s_rec[s];
        if (r[1] > 0.f) m_tot = fmaxf(m_tot, r[0]);
    }
    m_tot = fmaxf(m_tot, lane_xor<1>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<2>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<4>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<8>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<16>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<32>(m_tot, lane));

    f4 v = {0.f, 0.f, 0.f, 0.f};
    float l_part = 0.f;
#pragma unroll
    for (int k = 0; k < kMergeMaxPerGroup; ++k) {
        const int s = grp + k * kMergeGroups;
        if (s < n_slots && live_slot(s)) {
            const f4 r = s_rec[s];
            if (r[1] > 0.f) {
                const float w = __builtin_amdgcn_exp2f(r[0] - m_tot);
                l_part += r[1] * w;
                v += a[k] * w;
            }
        }
    }
    s_acc[grp][lane] = v;
    if (lane == 0) s_red[grp] = l_part;
    __syncthreads();
    if (grp != 0) return;
    float l_tot = 0.f;
    f4 tot = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < kMergeGroups; ++k) {
        tot += s_acc[k][lane];
        l_tot += s_red[k];
    }
    const float inv = l_tot > 0.f ? out_scale / l_tot : 0.f;
    float o[4] = {tot[0] * inv, tot[1] * inv, tot[2] * inv, tot[3] * inv};
    if (rotate) {
        wht256_wave(o, lane);
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = apply_sign(o[k], 4 * lane + k);
    }
    store_out_row<TQ, HD>(P, (size_t)row, lane, o);
}

}  // namespace w34

#include "paged_attn_rows.h"
#include "paged_prefill_tq4.h"
#include "qsa_sparse_tq4.h"
#include "qsa_sparse_rows.h"

namespace w34 {

// ---- host side ---------------------------------------------------------------------------------
constexpr int kMaxChunksCap = 256;
// 256 tokens, one unit per wave: 7 to 12 % faster than 16 at 16K-32K keys, same as 4
constexpr int kMinUnitsPerChunk = 8;
// Split geometry is sized for the layout the path is built for, two kv heads per device: 128
// chunks (or shares) per kv head.  The counts below depend on the batch and on gqa only, never
// on local_kv_heads: a rank that holds one kv head of a sharded model computes every row with
// the same chunks, in the same order, as a rank that holds all of them (bit-identical outputs
// under head sharding, op_paged_attn.cu:1301-1304), at the price of half-filled compute units
// on such a rank.
constexpr int kTargetWorkgroupsPerHead = 128;

static size_t partial_bytes(long long rows, int max_chunks) {
    return (size_t)rows * (size_t)max_chunks * (kHeadDim + 4) * sizeof(float);
}

// Cap on chunks per tile: a function of total_tokens (tiles), gqa (q subgroups per kv head) and
// the scratch size only.
static int choose_max_chunks(const warp34_exec* ex, int total_tokens, int num_q_heads, int tok_tile,
                             int q_subgroups) {
    if (ex->scratch_ptr == 0 || (ex->scratch_ptr & 15u) != 0u) return 1;
    const int tiles = (total_tokens + tok_tile - 1) / tok_tile;
    const long long per_chunk = (long long)(tiles > 0 ? tiles : 1) * (q_subgroups > 0 ? q_subgroups : 1);
    int want = (int)(kTargetWorkgroupsPerHead / per_chunk);
    if (want > kMaxChunksCap) want = kMaxChunksCap;
    if (want < 2) return 1;
    const long long rows = (long long)total_tokens * num_q_heads;
    while (want > 1 && partial_bytes(rows, want) > ex->scratch_size) want >>= 1;
    return want < 2 ? 1 : want;
}

// One attribute call per kernel instantiation and device.  The record is process-wide and
// lock-free: slot i belongs to the first kernel that claims it, bit d of its mask says that
// device d is configured.  Kernels that address their dequantisation table absolutely
// (lds_base_zero) also have their static LDS size checked here: it must be zero, so that the
// dynamic block starts at LDS address 0.
constexpr int kLdsRecordSlots = 96;
static std::atomic<const void*> g_lds_fn[kLdsRecordSlots];
static std::atomic<unsigned long long> g_lds_devs[kLdsRecordSlots];

template <typename KernelT>
static int ensure_dynamic_lds(KernelT kernel, int bytes, bool lds_base_zero = false) {
    int dev = 0;
    hipError_t rc = hipGetDevice(&dev);
    if (rc != hipSuccess) return (int)rc;
    const void* fn = (const void*)kernel;
    int slot = -1;
    for (int i = 0; i < kLdsRecordSlots; ++i) {
        const void* cur = g_lds_fn[i].load(std::memory_order_acquire);
        if (cur == nullptr) {
            const void* expect = nullptr;
            if (g_lds_fn[i].compare_exchange_strong(expect, fn, std::memory_order_acq_rel)) cur = fn;
            else cur = expect;
        }
        if (cur == fn) {
            slot = i;
            break;
        }
    }
    const bool tracked = slot >= 0 && dev >= 0 && dev < 64;
    if (tracked && ((g_lds_devs[slot].load(std::memory_order_acquire) >> dev) & 1ull)) return 0;
    if (lds_base_zero) {
        hipFuncAttributes attr;
        rc = hipFuncGetAttributes(&attr, fn);
        if (rc != hipSuccess) return (int)rc;
        if (attr.sharedSizeBytes != 0) return (int)hipErrorInvalidConfiguration;
    }
    rc = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (rc != hipSuccess) return (int)rc;
    if (tracked) g_lds_devs[slot].fetch_or(1ull << dev, std::memory_order_release);
    return 0;
}

// Decode batches of several requests take the balanced path: no request has more than one
// tile, no window, no token mask (the plan counts units of [0, last key]), usable scratch.
static bool balanced_decode_applicable(const warp34_exec* ex, const warp34_attention_batch* batch,
                                       int tiles_by_request, int force_single) {
    return tiles_by_request && batch->num_reqs >= 2 && !force_single && batch->sliding_window <= 0 &&
           batch->valid_token_mask == nullptr && ex->scratch_ptr != 0 && (ex->scratch_ptr & 15u) == 0u;
}
// shares of a balanced decode batch per (kv head, q subgroup): a function of gqa only
static int balanced_groups(int q_subgroups) {
    int groups = kTargetWorkgroupsPerHead / (q_subgroups > 0 ? q_subgroups : 1);
    if (groups > kMergeGroups * kMergeMaxPerGroup - 1) groups = kMergeGroups * kMergeMaxPerGroup - 1;
    return groups < 1 ? 1 : groups;
}

// P.spec_* = chunk_geom(0, max_seq_len - 1, P.max_chunks, P.min_upc), worked out on the host
static void fill_spec_geometry(AttnParams& P, int max_seq_len) {
    if (max_seq_len <= 0) return;
    P.spec_units = ((max_seq_len - 1) >> 5) + 1;
    int nc = (P.spec_units + P.min_upc - 1) / P.min_upc;
    if (nc > P.max_chunks) nc = P.max_chunks;
    if (nc < 1) nc = 1;
    P.spec_upc = (P.spec_units + nc - 1) / nc;
    if (P.spec_upc < 1) P.spec_upc = 1;
    P.spec_chunks = (P.spec_units + P.spec_upc - 1) / P.spec_upc;
    if (P.spec_chunks < 1) P.spec_chunks = 1;
}

// ---- shared-prefix pass (verify batches whose requests share their leading pages) ----
// The host cannot see the block tables, so a one-workgroup kernel finds the common leading run:
// the pages that every request's block table holds at the same index and that lie below every
// request's first query position (every query of the batch sees all of their keys).  It leaves
// the length in tokens (a multiple of the unit; 0 below kSpMinTokens) and the descriptor of one
// pseudo request -- all query tokens of the batch over exactly those keys -- in the header.
struct SpHeader {
    int32_t floor;   // keys [0, floor) are the shared prefix
    int32_t qsl[2];  // query_start_loc of the pseudo request: {0, total_tokens}
    int32_t seq;     // its seq_lens_after (= floor)
    int32_t ctx;     // its context_lens_before (= floor: every key visible to every token)
    int32_t pad[3];
};
constexpr int kSpMinTokens = 4096;

__global__ __launch_bounds__(1024) void shared_prefix_probe_kernel(const warp34_attention_batch B, int block_size,
                                                                   SpHeader* hdr) {
    __shared__ int s_first_diff, s_min_ctx;
    const int tid = (int)threadIdx.x;
    if (tid == 0) {
        s_first_diff = B.max_blocks_per_req;
        s_min_ctx = 0x7fffffff;
    }
    __syncthreads();
    for (int r = tid; r < B.num_reqs; r += 1024) {
        const int q_len = B.query_start_loc[r + 1] - B.query_start_loc[r];
        const int ctx = B.context_lens_before != nullptr ? B.context_lens_before[r] : B.seq_lens_after[r] - q_len;
        atomicMin(&s_min_ctx, ctx < 0 ? 0 : ctx);
    }
    __syncthreads();
    int max_pages = s_min_ctx / block_size;  // pages that lie entirely below every first query position
    if (max_pages > B.max_blocks_per_req) max_pages = B.max_blocks_per_req;
    // one request per wave (r = 1 + wave, + 16, ...), sixteen pages per lane and round trip: the
    // loads of a batch are independent of each other
    const int wave = tid >> 6, lane = tid & 63;
    int first_diff = 0x7fffffff;
    for (int r = 1 + wave; r < B.num_reqs; r += 16) {
        const int32_t* row = B.block_tables + (size_t)r * B.max_blocks_per_req;
        for (int base = lane; base < max_pages; base += 16 * 64) {
            int32_t mine[16], ref[16];
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                const int p = base + 64 * k;
                const int pc = p < max_pages ? p : 0;
                mine[k] = row[pc];
                ref[k] = B.block_tables[pc];
            }
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                const int p = base + 64 * k;
                if (p < max_pages && mine[k] != ref[k] && p < first_diff) first_diff = p;
            }
        }
    }
    if (first_diff != 0x7fffffff) atomicMin(&s_first_diff, first_diff);
    __syncthreads();
    if (tid == 0) {
        const int pages = s_first_diff < max_pages ? s_first_diff : max_pages;
        int floor = (pages * block_size) & ~(kUnit - 1);
        if (floor < kSpMinTokens) floor = 0;
        hdr->floor = floor;
        hdr->qsl[0] = 0;
        hdr->qsl[1] = B.total_tokens;
        hdr->seq = floor;
        hdr->ctx = floor;
    }
}

// Batches that may take the pass: several requests, a few query tokens each (a verify step),
// long contexts, plain causal masking.  (Decode batches keep the balanced shares; the pass costs
// two small launches and wide partial records when nothing is shared.)
static bool shared_prefix_applicable(const warp34_attention_batch* b, int q_group, int force_single) {
    return !force_single && b->num_reqs >= 4 && b->max_q_len >= 2 && b->max_q_len <= kPfRows / q_group &&
           b->total_tokens >= 16 && b->max_seq_len >= 8 * kSpMinTokens && b->sliding_window <= 0 &&
           b->mask_mode == WARP34_ATTN_MASK_CAUSAL && b->valid_token_mask == nullptr && b->valid_req_mask == nullptr &&
           b->context_lens_before != nullptr && (q_group & (q_group - 1)) == 0;
}
// parts of the prefix per tile: a function of the batch and of gqa only, never of the number of
// local kv heads (a rank with one kv head must produce the bits of a rank with two)
static int shared_prefix_parts(int total_tokens, int q_group, int q_subgroups) {
    const int tiles = (total_tokens + kPfRows / q_group - 1) / (kPfRows / q_group) * q_subgroups;
    int parts = (kTargetWorkgroupsPerHead + tiles - 1) / tiles;  // about one workgroup per CU at two kv heads
    return parts < 1 ? 1 : (parts > 32 ? 32 : parts);
}

template <typename TQ>
static int launch_tq4(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                      const warp34_attention_batch* batch, const void* q, void* out, int num_q_heads,
                      int force_single, const void* gate) {
    AttnParams P{};
    P.L = *layout;
    P.B = *batch;
    P.block_magic = block_magic_for(layout->block_size);
    P.q = (const uint16_t*)q;
    P.out = (uint16_t*)out;
    P.gate = (const uint16_t*)gate;
    P.rot_q = layout->k_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 ? 1 : 0;
    P.rot_out = layout->v_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 ? 1 : 0;
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
    // One N tile (16 query columns) per workgroup, also for verify batches: the two-tile variant
    // (4 waves, 32 columns) halves the key reads but runs at half the occupancy and measured
    // slower (2.04 ms against 1.64 ms on 16 requests x 4 query tokens at 262 144 keys).
    const int nt = 1;
    P.tok_tile = (16 * nt) / q_group;
    if (P.tok_tile < 1) P.tok_tile = 1;
    P.min_upc = kMinUnitsPerChunk;
    P.unit_in_page = (layout->block_size % kUnit == 0 && layout->k_page_stride_bytes <= 0xFFFFFFFFull &&
                      layout->v_page_stride_bytes <= 0xFFFFFFFFull)
                         ? 1
                         : 0;
    P.max_chunks = force_single ? 1 : choose_max_chunks(ex, batch->total_tokens, num_q_heads, P.tok_tile,
                                                        P.q_subgroups);
    P.part_acc = nullptr;
    P.part_ml = nullptr;
    const long long rows = (long long)batch->total_tokens * num_q_heads;
    // grid.x: chunks that can exist given the host's upper bound on the sequence length
    int grid_x = P.max_chunks;
    if (batch->max_seq_len > 0) {
        const int units = (batch->max_seq_len + kUnit - 1) / kUnit + 1;
        const int bound = (units + P.min_upc - 1) / P.min_upc;
        if (bound < grid_x) grid_x = bound < 1 ? 1 : bound;
    }
    // No tile has more chunks than that: the cap is lowered to it, which changes no chunk (a
    // tile's count is limited by its own units first) and keeps the partial records, and what
    // the merge kernel loads ahead of knowing the count, as small as the bound allows.
    P.max_chunks = grid_x;
    P.part_stride = grid_x;
    fill_spec_geometry(P, batch->max_seq_len);
    if (P.max_chunks > 1) {
        uint8_t* ws = reinterpret_cast<uint8_t*>((uintptr_t)ex->scratch_ptr);
        P.part_acc = reinterpret_cast<float*>(ws);
        P.part_ml = P.part_acc + (size_t)rows * P.max_chunks * kHeadDim;
    }
    // grid.z: tiles.  One per request when no request can have two; otherwise the upper bound
    // sum_r ceil(q_r / tok_tile) <= total_tokens / tok_tile + num_reqs
    P.tiles_by_request = (batch->max_q_len > 0 && batch->max_q_len <= P.tok_tile) ? 1 : 0;
    const int grid_z = P.tiles_by_request ? batch->num_reqs : batch->total_tokens / P.tok_tile + batch->num_reqs;
    const int kv_subs = layout->local_kv_heads * P.q_subgroups;
    const dim3 grid((unsigned)grid_x, (unsigned)kv_subs, (unsigned)grid_z);
    hipStream_t stream = (hipStream_t)ex->stream;
    int rc;
    // Verify batches: the keys every request has in common go through the tile kernel once, for
    // all query rows of the batch (its dequantisation is shared by 128 rows instead of 16); the
    // decode kernel takes the private rest, the merge kernel both sets of partial records.
    if (P.max_chunks > 1 && shared_prefix_applicable(batch, q_group, force_single)) {
        const int parts = shared_prefix_parts(batch->total_tokens, q_group, P.q_subgroups);
        const int stride = P.max_chunks + parts;
        const size_t need = partial_bytes(rows, stride) + sizeof(SpHeader);
        if (stride <= kMergeGroups * kMergeMaxPerGroup && need <= ex->scratch_size) {
            P.part_stride = stride;
            P.pf_split = parts;
            P.pf_slot_base = P.max_chunks;
            P.part_ml = P.part_acc + (size_t)rows * stride * kHeadDim;
            SpHeader* hdr = reinterpret_cast<SpHeader*>(P.part_ml + (size_t)rows * stride * 4);
            P.key_floor = &hdr->floor;
            hipLaunchKernelGGL(shared_prefix_probe_kernel, dim3(1), dim3(1024), 0, stream, *batch, layout->block_size, hdr);
            rc = (int)hipGetLastError();
            if (rc) return rc;
            AttnParams T = P;  // the pseudo request of the header, 128-row tiles
            T.B.num_reqs = 1;
            T.B.query_start_loc = hdr->qsl;
            T.B.seq_lens_after = &hdr->seq;
            T.B.context_lens_before = &hdr->ctx;
            T.B.max_q_len = batch->total_tokens;
            T.tok_tile = kPfRows / q_group;
            T.key_floor = nullptr;
            const int pf_tiles = (batch->total_tokens + T.tok_tile - 1) / T.tok_tile;
            using PfL = PfLds<WARP34_KV_FORMAT_TQ4>;
            rc = ensure_dynamic_lds(paged_prefill_tq4_kernel<TQ, WARP34_KV_FORMAT_TQ4, false, true, true>, PfL::kSmem, true);
            if (rc) return rc;
            hipLaunchKernelGGL((paged_prefill_tq4_kernel<TQ, WARP34_KV_FORMAT_TQ4, false, true, true>),
                               dim3((unsigned)(pf_tiles * parts), (unsigned)kv_subs, 1u), dim3(12 * 64), PfL::kSmem,
                               stream, T);
            rc = (int)hipGetLastError();
            if (rc) return rc;
            rc = ensure_dynamic_lds(paged_attn_tq4_kernel<TQ, 1, true>, smem_bytes_for(1), true);
            if (rc) return rc;
            hipLaunchKernelGGL((paged_attn_tq4_kernel<TQ, 1, true>), grid, dim3(waves_for(1) * 64), smem_bytes_for(1),
                               stream, P);
            rc = (int)hipGetLastError();
            if (rc) return rc;
            hipLaunchKernelGGL((split_merge_kernel<TQ, true>), dim3((unsigned)rows), dim3(1024), 0, stream,
                               (const float*)P.part_acc, (const float*)P.part_ml, stride, P, kLutInvGain, P.rot_out);
            return (int)hipGetLastError();
        }
    }
    // Decode batches of several requests: equal shares of the batch's units per workgroup
    // instead of per-request chunks (the requests' lengths are unknown to the host and differ).
    if (balanced_decode_applicable(ex, batch, P.tiles_by_request, force_single)) {
        const int groups = balanced_groups(P.q_subgroups);
        const size_t prows = bal_partial_row(groups + batch->num_reqs, kv_subs, 0, 0);
        if (partial_bytes((long long)prows, 1) + (size_t)batch->total_tokens * 16 <= ex->scratch_size) {
            P.part_acc = reinterpret_cast<float*>((uintptr_t)ex->scratch_ptr);
            P.part_ml = P.part_acc + prows * kHeadDim;
            P.bal_table = reinterpret_cast<int32_t*>(P.part_ml + prows * 4);
            P.max_chunks = groups + 1;
            rc = ensure_dynamic_lds(paged_attn_tq4_balanced_kernel<TQ>, smem_bytes_for(1), true);
            if (rc) return rc;
            hipLaunchKernelGGL((paged_attn_tq4_balanced_kernel<TQ>), dim3((unsigned)groups, (unsigned)kv_subs),
                               dim3(waves_for(1) * 64), smem_bytes_for(1), stream, P);
            rc = (int)hipGetLastError();
            if (rc) return rc;
            hipLaunchKernelGGL((balanced_merge_kernel<TQ>),
                               dim3((unsigned)rows), dim3(1024), 0, stream, P,
                               kv_subs, kLutInvGain, P.rot_out);
            return (int)hipGetLastError();
        }
    }
    rc = ensure_dynamic_lds(paged_attn_tq4_kernel<TQ, 1>, smem_bytes_for(1), true);
    if (rc) return rc;
    hipLaunchKernelGGL((paged_attn_tq4_kernel<TQ, 1>), grid, dim3(waves_for(1) * 64), smem_bytes_for(1), stream, P);
    rc = (int)hipGetLastError();
    if (rc) return rc;
    if (P.max_chunks > 1) {
        hipLaunchKernelGGL((split_merge_kernel<TQ>), dim3((unsigned)rows), dim3(1024), 0, stream,
                           (const float*)P.part_acc, (const float*)P.part_ml, P.max_chunks, P, kLutInvGain, P.rot_out);
        rc = (int)hipGetLastError();
    }
    return rc;
}

// VRES: value rows stored rotated in an 8-bit format (residual operand, see rows_tile)
template <typename TQ, int KVF, bool VRES = false, int HD = kHeadDim>
static int launch_rows(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                       const warp34_attention_batch* batch, const void* q, void* out, int num_q_heads,
                       int force_single, const void* gate) {
    AttnParams P{};
    P.L = *layout;
    P.B = *batch;
    P.block_magic = block_magic_for(layout->block_size);
    P.q = (const uint16_t*)q;
    P.out = (uint16_t*)out;
    P.gate = (const uint16_t*)gate;
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
    P.tok_tile = 16 / q_group;  // one N tile
    if (P.tok_tile < 1) P.tok_tile = 1;
    P.min_upc = kMinUnitsPerChunk;
    P.max_chunks = force_single ? 1 : choose_max_chunks(ex, batch->total_tokens, num_q_heads, P.tok_tile,
                                                        P.q_subgroups);
    P.part_acc = nullptr;
    P.part_ml = nullptr;
    const long long rows = (long long)batch->total_tokens * num_q_heads;
    int grid_x = P.max_chunks;
    if (batch->max_seq_len > 0) {
        const int units = (batch->max_seq_len + kUnit - 1) / kUnit + 1;
        const int bound = (units + P.min_upc - 1) / P.min_upc;
        if (bound < grid_x) grid_x = bound < 1 ? 1 : bound;
    }
    // No tile has more chunks than that: the cap is lowered to it, which changes no chunk (a
    // tile's count is limited by its own units first) and keeps the partial records, and what
    // the merge kernel loads ahead of knowing the count, as small as the bound allows.
    P.max_chunks = grid_x;
    P.part_stride = grid_x;
    fill_spec_geometry(P, batch->max_seq_len);
    if (P.max_chunks > 1) {
        uint8_t* ws = reinterpret_cast<uint8_t*>((uintptr_t)ex->scratch_ptr);
        P.part_acc = reinterpret_cast<float*>(ws);
        P.part_ml = P.part_acc + (size_t)rows * P.max_chunks * kHeadDim;
    }
    P.tiles_by_request = (batch->max_q_len > 0 && batch->max_q_len <= P.tok_tile) ? 1 : 0;
    P.rot_q = layout->k_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 ? 1 : 0;
    P.rot_out = layout->v_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 ? 1 : 0;
    const int grid_z = P.tiles_by_request ? batch->num_reqs : batch->total_tokens / P.tok_tile + batch->num_reqs;
    const int kv_subs = layout->local_kv_heads * P.q_subgroups;
    const dim3 grid((unsigned)grid_x, (unsigned)kv_subs, (unsigned)grid_z);
    hipStream_t stream = (hipStream_t)ex->stream;
    int rc;
    if (HD == kHeadDim && balanced_decode_applicable(ex, batch, P.tiles_by_request, force_single)) {
        const int groups = balanced_groups(P.q_subgroups);
        const size_t prows = bal_partial_row(groups + batch->num_reqs, kv_subs, 0, 0);
        if (partial_bytes((long long)prows, 1) + (size_t)batch->total_tokens * 16 <= ex->scratch_size) {
            P.part_acc = reinterpret_cast<float*>((uintptr_t)ex->scratch_ptr);
            P.part_ml = P.part_acc + prows * kHeadDim;
            P.bal_table = reinterpret_cast<int32_t*>(P.part_ml + prows * 4);
            P.max_chunks = groups + 1;
            rc = ensure_dynamic_lds(paged_attn_rows_balanced_kernel<TQ, KVF, VRES>, kv16_smem_bytes(1));
            if (rc) return rc;
            hipLaunchKernelGGL((paged_attn_rows_balanced_kernel<TQ, KVF, VRES>), dim3((unsigned)groups, (unsigned)kv_subs),
                               dim3(kKv16Waves * 64), kv16_smem_bytes(1), stream, P);
            rc = (int)hipGetLastError();
            if (rc) return rc;
            hipLaunchKernelGGL((balanced_merge_kernel<TQ>),
                               dim3((unsigned)rows), dim3(1024), 0, stream, P,
                               kv_subs, 1.0f, P.rot_out);
            return (int)hipGetLastError();
        }
    }
    rc = ensure_dynamic_lds(paged_attn_rows_kernel<TQ, 1, KVF, VRES, HD>, kv16_smem_bytes(1));
    if (rc) return rc;
    hipLaunchKernelGGL((paged_attn_rows_kernel<TQ, 1, KVF, VRES, HD>), grid, dim3(kKv16Waves * 64), kv16_smem_bytes(1), stream, P);
    rc = (int)hipGetLastError();
    if (rc) return rc;
    if (P.max_chunks > 1) {
        hipLaunchKernelGGL((split_merge_kernel<TQ, false, HD>), dim3((unsigned)rows), dim3(1024), 0, stream,
                           (const float*)P.part_acc, (const float*)P.part_ml, P.max_chunks, P, 1.0f, P.rot_out);
        rc = (int)hipGetLastError();
    }
    return rc;
}

// Chunked prefill over TQ4 pages: one workgroup per (128-row query tile, kv head x q subgroup,
// request); no split (a prefill batch has thousands of tiles).
static bool prefill_tq4_applicable(const warp34_kv_layer_layout* layout, const warp34_attention_batch* batch,
                                   int num_q_heads) {
    const int gqa = num_q_heads / layout->local_kv_heads;
    int q_group = gqa;
    if (q_group > 16) {
        for (int d = 16; d >= 1; --d)
            if (gqa % d == 0) {
                q_group = d;
                break;
            }
    }
    return q_group > 0 && (q_group & (q_group - 1)) == 0 && batch->max_q_len > 0;
}

template <typename TQ, int KVF>
static int launch_prefill_tq4(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                              const warp34_attention_batch* batch, const void* q, void* out, int num_q_heads,
                              const void* gate) {
    AttnParams P{};
    P.L = *layout;
    P.B = *batch;
    P.block_magic = block_magic_for(layout->block_size);
    P.q = (const uint16_t*)q;
    P.out = (uint16_t*)out;
    P.gate = (const uint16_t*)gate;
    P.part_acc = nullptr;
    P.part_ml = nullptr;
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
    P.tok_tile = kPfRows / q_group;
    P.max_chunks = 1;
    P.min_upc = kMinUnitsPerChunk;
    const int tiles = (batch->max_q_len + P.tok_tile - 1) / P.tok_tile;
    const dim3 grid((unsigned)tiles, (unsigned)(layout->local_kv_heads * P.q_subgroups), (unsigned)batch->num_reqs);
    P.rot_q = layout->k_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 ? 1 : 0;
    P.rot_out = layout->v_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 ? 1 : 0;
    constexpr bool k8bit = KVF == WARP34_KV_FORMAT_FP8_E4M3 || KVF == WARP34_KV_FORMAT_Q8_0;
    int rc;
    if constexpr (k8bit) {
        if (P.rot_out) {  // rotated 8-bit value rows: codes in the value tile, block scales in the weights
            rc = ensure_dynamic_lds(paged_prefill_tq4_kernel<TQ, KVF, true>, PfLds<KVF>::kSmem, true);
            if (rc) return rc;
            hipLaunchKernelGGL((paged_prefill_tq4_kernel<TQ, KVF, true>), grid, dim3(kPfWaves * 64), PfLds<KVF>::kSmem,
                               (hipStream_t)ex->stream, P);
            return (int)hipGetLastError();
        }
    }
    if constexpr (KVF == WARP34_KV_FORMAT_TQ4) {  // twelve waves: eight multiply, four dequantise
        rc = ensure_dynamic_lds(paged_prefill_tq4_kernel<TQ, KVF, false, true>, PfLds<KVF>::kSmem, true);
        if (rc) return rc;
        hipLaunchKernelGGL((paged_prefill_tq4_kernel<TQ, KVF, false, true>), grid, dim3(12 * 64), PfLds<KVF>::kSmem,
                           (hipStream_t)ex->stream, P);
        return (int)hipGetLastError();
    } else {
        rc = ensure_dynamic_lds(paged_prefill_tq4_kernel<TQ, KVF, false>, PfLds<KVF>::kSmem, true);
        if (rc) return rc;
        hipLaunchKernelGGL((paged_prefill_tq4_kernel<TQ, KVF, false>), grid, dim3(kPfWaves * 64), PfLds<KVF>::kSmem,
                           (hipStream_t)ex->stream, P);
        return (int)hipGetLastError();
    }
}

static bool is_kv16(const warp34_kv_layer_layout* l, int format) {
    return (l->head_dim == 256 || l->head_dim == 128) && l->k_format == format && l->v_format == format &&
           l->k_transform == WARP34_KV_TRANSFORM_IDENTITY && l->v_transform == WARP34_KV_TRANSFORM_IDENTITY;
}

static bool kv16_geometry_ok(const warp34_kv_layer_layout* l, const void* q, const void* out) {
    const unsigned row_bytes = 2u * (unsigned)l->head_dim;
    return l->block_size > 0 && (l->block_size % 16) == 0 && l->k_token_stride_bytes == row_bytes &&
           l->v_token_stride_bytes == row_bytes && (l->k_base & 15u) == 0 && (l->v_base & 15u) == 0 &&
           (l->k_page_stride_bytes & 15u) == 0 && (l->k_head_stride_bytes & 15u) == 0 &&
           (l->v_page_stride_bytes & 15u) == 0 && (l->v_head_stride_bytes & 15u) == 0 &&
           (((uintptr_t)q) & 15u) == 0 && (((uintptr_t)out) & 7u) == 0;
}

// 8-bit rows: both slabs in the same format, each stored plain or rotated
static bool is_kv8(const warp34_kv_layer_layout* l, int format) {
    const auto xf_ok = [](int t) {
        return t == WARP34_KV_TRANSFORM_IDENTITY || t == WARP34_KV_TRANSFORM_RADEMACHER_WHT256;
    };
    return l->head_dim == 256 && l->k_format == format && l->v_format == format && xf_ok(l->k_transform) &&
           xf_ok(l->v_transform);
}

// 16-token runs must be contiguous and 16-byte aligned for the staging copy
static bool kv8_geometry_ok(const warp34_kv_layer_layout* l, const void* q, const void* out, unsigned row_bytes) {
    return l->block_size > 0 && (l->block_size % 16) == 0 && l->k_token_stride_bytes == row_bytes &&
           l->v_token_stride_bytes == row_bytes && (l->k_base & 15u) == 0 && (l->v_base & 15u) == 0 &&
           (l->k_page_stride_bytes & 15u) == 0 && (l->k_head_stride_bytes & 15u) == 0 &&
           (l->v_page_stride_bytes & 15u) == 0 && (l->v_head_stride_bytes & 15u) == 0 &&
           (((uintptr_t)q) & 15u) == 0 && (((uintptr_t)out) & 7u) == 0;
}

static bool is_tq4_wht(const warp34_kv_layer_layout* l) {
    return l->head_dim == 256 && l->k_format == WARP34_KV_FORMAT_TQ4 && l->v_format == WARP34_KV_FORMAT_TQ4 &&
           l->k_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 &&
           l->v_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256;
}

// TQ4 pages at head dimension 256, each slab stored rotated or plain (op_paged_attn.cu:347,570:
// the query is rotated for rotated keys, the output rotated back for rotated values)
static bool is_tq4(const warp34_kv_layer_layout* l) {
    const auto xf_ok = [](int t) {
        return t == WARP34_KV_TRANSFORM_IDENTITY || t == WARP34_KV_TRANSFORM_RADEMACHER_WHT256;
    };
    return l->head_dim == 256 && l->k_format == WARP34_KV_FORMAT_TQ4 && l->v_format == WARP34_KV_FORMAT_TQ4 &&
           xf_ok(l->k_transform) && xf_ok(l->v_transform);
}

static bool tq4_geometry_ok(const warp34_kv_layer_layout* l, const void* q) {
    // 16-token runs must be contiguous and 16-byte aligned for the staging copy
    return l->block_size > 0 && (l->block_size % 16) == 0 && l->k_token_stride_bytes == kTq4RowBytes &&
           l->v_token_stride_bytes == kTq4RowBytes && (l->k_base & 15u) == 0 && (l->v_base & 15u) == 0 &&
           (l->k_page_stride_bytes & 15u) == 0 && (l->k_head_stride_bytes & 15u) == 0 &&
           (l->v_page_stride_bytes & 15u) == 0 && (l->v_head_stride_bytes & 15u) == 0 &&
           (((uintptr_t)q) & 7u) == 0;
}

static int common_checks(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                         const warp34_attention_batch* batch, const void* q, void* out, int num_q_heads) {
    if (!ex || !layout || !batch || !q || !out) return (int)hipErrorInvalidValue;
    return 0;
}

template <typename TQ>
static int attention_entry(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                           const warp34_attention_batch* batch, const void* q, void* out, int num_q_heads,
                           int force, const void* gate = nullptr) {
    // force (the test selector): 0 = the dispatch below, 1 = the decode / verify kernel as a single
    // pass, 2 = the 128-row tile kernel (where the batch shape admits it, else as 1)
    const int force_single = force != 0 ? 1 : 0;
    const bool force_tile = force == 2;
    if (layout->local_kv_heads <= 0 || num_q_heads % layout->local_kv_heads != 0 || batch->num_reqs <= 0 ||
        !batch->query_start_loc || !batch->seq_lens_after || !batch->block_tables ||
        batch->max_blocks_per_req <= 0 || batch->sliding_window < 0 ||
        (batch->mask_mode != WARP34_ATTN_MASK_CAUSAL && batch->mask_mode != WARP34_ATTN_MASK_NONCAUSAL_WINDOW)) {
        return (int)hipErrorInvalidValue;
    }
    if (is_tq4(layout)) {
        if (!tq4_geometry_ok(layout, q) || (((uintptr_t)out) & 7u) != 0) return (int)hipErrorNotSupported;
        // Many query rows per request and enough tiles to fill the chip: the tile kernel shares
        // every dequantised key block between 128 query rows.
        const bool many_rows = batch->max_q_len >= 32 &&
                               (long long)batch->total_tokens * num_q_heads >= 128ll * kPfRows;
        if ((force_tile || (!force && many_rows)) && prefill_tq4_applicable(layout, batch, num_q_heads))
            return launch_prefill_tq4<TQ, WARP34_KV_FORMAT_TQ4>(ex, layout, batch, q, out, num_q_heads, gate);
        return launch_tq4<TQ>(ex, layout, batch, q, out, num_q_heads, force_single, gate);
    }
    // 16-bit pages: the storage type must be the query type (FP16 pages with the f16 entry
    // point, BF16 pages with the bf16 one, as in the reference)
    if (is_kv16(layout, TQ::kStorageFormat)) {
        if (!kv16_geometry_ok(layout, q, out)) return (int)hipErrorNotSupported;
        // many query rows per request: the tile kernel (rows copied as stored)
        const bool many_rows = batch->max_q_len >= 32 &&
                               (long long)batch->total_tokens * num_q_heads >= 128ll * kPfRows;
        // head dimension 128 (op_kv_cache.cu:1227): the decode / verify kernel serves every batch shape
        if (layout->head_dim == 128)
            return launch_rows<TQ, TQ::kStorageFormat, false, 128>(ex, layout, batch, q, out, num_q_heads, force_single, gate);
        if ((force_tile || (!force && many_rows)) && prefill_tq4_applicable(layout, batch, num_q_heads))
            return launch_prefill_tq4<TQ, TQ::kStorageFormat>(ex, layout, batch, q, out, num_q_heads, gate);
        return launch_rows<TQ, TQ::kStorageFormat>(ex, layout, batch, q, out, num_q_heads, force_single, gate);
    }
    // 8-bit pages (the tail layers of the default TQ4 policy, cache.rs:87-109)
    if (is_kv8(layout, WARP34_KV_FORMAT_FP8_E4M3)) {
        if (!kv8_geometry_ok(layout, q, out, 264)) return (int)hipErrorNotSupported;
        // many query rows per request: the tile kernel (FP8 rows have the shape of TQ4 rows)
        const bool many_rows = batch->max_q_len >= 32 &&
                               (long long)batch->total_tokens * num_q_heads >= 128ll * kPfRows;
        if ((force_tile || (!force && many_rows)) && prefill_tq4_applicable(layout, batch, num_q_heads))
            return launch_prefill_tq4<TQ, WARP34_KV_FORMAT_FP8_E4M3>(ex, layout, batch, q, out, num_q_heads, gate);
        if (layout->v_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256)
            return launch_rows<TQ, WARP34_KV_FORMAT_FP8_E4M3, true>(ex, layout, batch, q, out, num_q_heads, force_single, gate);
        return launch_rows<TQ, WARP34_KV_FORMAT_FP8_E4M3>(ex, layout, batch, q, out, num_q_heads, force_single, gate);
    }
    if (is_kv8(layout, WARP34_KV_FORMAT_Q8_0)) {
        if (!kv8_geometry_ok(layout, q, out, 272)) return (int)hipErrorNotSupported;
        const bool many_rows = batch->max_q_len >= 32 &&
                               (long long)batch->total_tokens * num_q_heads >= 128ll * kPfRows;
        if ((force_tile || (!force && many_rows)) && prefill_tq4_applicable(layout, batch, num_q_heads))
            return launch_prefill_tq4<TQ, WARP34_KV_FORMAT_Q8_0>(ex, layout, batch, q, out, num_q_heads, gate);
        if (layout->v_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256)
            return launch_rows<TQ, WARP34_KV_FORMAT_Q8_0, true>(ex, layout, batch, q, out, num_q_heads, force_single, gate);
        return launch_rows<TQ, WARP34_KV_FORMAT_Q8_0>(ex, layout, batch, q, out, num_q_heads, force_single, gate);
    }
    return (int)hipErrorNotSupported;
}

// QSA sparse paged attention (op_qsa.cu:1446-1571).  Argument checks and error codes follow the
// reference's launcher; the split count is this kernel's own (enough workgroups to fill the chip,
// at least one unit per wave and split, scratch permitting).
static int launch_qsa_sparse(const warp34_exec* ex, const void* q, const void* gate,
                             const warp34_kv_layer_layout* layout, const int32_t* selected_phys_blocks,
                             const int32_t* selected_logical_blocks, const int32_t* num_selected_blocks,
                             const int32_t* token_seq_pos, const uint8_t* valid_token_mask, void* out,
                             int num_tokens, int local_q_heads, int select_k_blocks, float sm_scale, int had64) {
    if (!ex || !q || !layout || !selected_phys_blocks || !selected_logical_blocks || !num_selected_blocks ||
        !token_seq_pos || !out || num_tokens < 0 || local_q_heads <= 0 || layout->local_kv_heads <= 0 ||
        (local_q_heads % layout->local_kv_heads) != 0 || layout->head_dim != 256 || select_k_blocks < 0) {
        return (int)hipErrorInvalidValue;
    }
    if (num_tokens == 0) return 0;
    // page formats: rotated TQ4, FP16, FP8-E4M3 and Q8_0 (plain or rotated); anything else
    // (mixed K / V formats, BF16 pages) is reported as unsupported, never computed some other way
    constexpr int kFormTq4 = 1000;  // not a WARP34_KV_FORMAT_* value (FP16 is 0)
    int form = -1;  // kFormTq4, else the row format
    if (is_tq4_wht(layout)) {
        if (!tq4_geometry_ok(layout, q) || (((uintptr_t)out) & 7u) != 0) return (int)hipErrorNotSupported;
        form = kFormTq4;
    } else if (is_kv16(layout, WARP34_KV_FORMAT_FP16)) {
        if (!kv16_geometry_ok(layout, q, out)) return (int)hipErrorNotSupported;
        form = WARP34_KV_FORMAT_FP16;
    } else if (is_kv8(layout, WARP34_KV_FORMAT_FP8_E4M3)) {
        if (!kv8_geometry_ok(layout, q, out, 264)) return (int)hipErrorNotSupported;
        form = WARP34_KV_FORMAT_FP8_E4M3;
    } else if (is_kv8(layout, WARP34_KV_FORMAT_Q8_0)) {
        if (!kv8_geometry_ok(layout, q, out, 272)) return (int)hipErrorNotSupported;
        form = WARP34_KV_FORMAT_Q8_0;
    } else {
        return (int)hipErrorNotSupported;
    }
    if (gate != nullptr && (((uintptr_t)gate) & 7u) != 0) return (int)hipErrorNotSupported;
    QsaParams P{};
    P.L = *layout;
    P.q = (const uint16_t*)q;
    P.gate = (const uint16_t*)gate;
    P.out = (uint16_t*)out;
    P.sel_phys = selected_phys_blocks;
    P.sel_log = selected_logical_blocks;
    P.num_sel = num_selected_blocks;
    P.seq_pos = token_seq_pos;
    P.valid_token_mask = valid_token_mask;
    P.num_tokens = num_tokens;
    P.num_q_heads = local_q_heads;
    P.gqa = local_q_heads / layout->local_kv_heads;
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
    P.select_k = select_k_blocks;
    P.groups_per_page = layout->block_size / 4;
    P.gpp_shift = -1;
    for (int k = 0; k < 30; ++k)
        if ((1 << k) == P.groups_per_page) P.gpp_shift = k;
    P.sm_scale = sm_scale;
    P.had64 = had64;
    P.out_scale = form == kFormTq4 ? kLutInvGain : 1.0f;
    P.rot_q = layout->k_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 ? 1 : 0;
    P.rot_out = layout->v_transform == WARP34_KV_TRANSFORM_RADEMACHER_WHT256 ? 1 : 0;
    const int kv_subs = layout->local_kv_heads * P.q_subgroups;
    // work items of a token: 32-key units (TQ4) or 16-key halves (row formats), one per wave and turn
    const int max_units = form == kFormTq4 ? (select_k_blocks + 7) / 8 : (select_k_blocks + 3) / 4;
    long long want = 256ll / ((long long)num_tokens * kv_subs);
    if (want > kQsaMaxSplits) want = kQsaMaxSplits;
    const int by_units = (max_units + kQsaWaves - 1) / kQsaWaves;
    if (want > by_units) want = by_units;
    if (want < 1) want = 1;
    const size_t rows = (size_t)num_tokens * local_q_heads;
    const size_t need = rows * (size_t)want * (kHeadDim + 4) * sizeof(float);
    P.n_splits = (want > 1 && ex->scratch_ptr != 0 && (ex->scratch_ptr & 15u) == 0u && ex->scratch_size >= need)
                     ? (int)want
                     : 1;
    if (P.n_splits > 1) {
        P.part_acc = reinterpret_cast<float*>((uintptr_t)ex->scratch_ptr);
        P.part_ml = P.part_acc + rows * P.n_splits * kHeadDim;
    }
    hipStream_t stream = (hipStream_t)ex->stream;
    const dim3 grid((unsigned)num_tokens, (unsigned)kv_subs, (unsigned)P.n_splits);
    int rc;
    auto launch_rows_form = [&](auto kernel) {
        const int smem = kv16_smem_bytes(1);
        int r = ensure_dynamic_lds(kernel, smem);
        if (r) return r;
        hipLaunchKernelGGL(kernel, grid, dim3(kKv16Waves * 64), smem, stream, P);
        return (int)hipGetLastError();
    };
    if (form == kFormTq4) {
        rc = ensure_dynamic_lds(qsa_sparse_tq4_kernel, kQsaSmem, true);
        if (rc) return rc;
        hipLaunchKernelGGL(qsa_sparse_tq4_kernel, grid, dim3(kQsaWaves * 64), kQsaSmem, stream, P);
        rc = (int)hipGetLastError();
    } else if (form == WARP34_KV_FORMAT_FP16) {
        rc = launch_rows_form(qsa_sparse_rows_kernel<WARP34_KV_FORMAT_FP16>);
    } else if (form == WARP34_KV_FORMAT_FP8_E4M3) {
        rc = P.rot_out ? launch_rows_form(qsa_sparse_rows_kernel<WARP34_KV_FORMAT_FP8_E4M3, true>)
                       : launch_rows_form(qsa_sparse_rows_kernel<WARP34_KV_FORMAT_FP8_E4M3, false>);
    } else {
        rc = P.rot_out ? launch_rows_form(qsa_sparse_rows_kernel<WARP34_KV_FORMAT_Q8_0, true>)
                       : launch_rows_form(qsa_sparse_rows_kernel<WARP34_KV_FORMAT_Q8_0, false>);
    }
    if (rc) return rc;
    if (P.n_splits > 1) {
        hipLaunchKernelGGL(qsa_sparse_merge_kernel, dim3((unsigned)rows), dim3(64), 0, stream, P);
        rc = (int)hipGetLastError();
    }
    return rc;
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
        // the reference also asks the device generation here (op_paged_attn.cu:1259); gfx950 has FP8
        if (layout->head_dim != 256) return (int)hipErrorInvalidValue;
    }
    if (batch->total_tokens <= 0 || num_q_heads <= 0) return 0;
    return attention_entry<F16>(ex, layout, batch, q_in, attn_out, num_q_heads, 0);
}

// warp34_paged_attention_f16 with the output gate of the gated full-attention layers applied as
// the rows leave the kernels (no counterpart in the reference, which calls
// warp34_apply_attn_output_gate_f16 afterwards, model/forward.rs:1192-1211): attn_out receives the
// bits of that sequence, the ungated output never goes to memory.  gate: fp16
// [total_tokens, num_q_heads, 256], 8-byte aligned; rows the attention leaves untouched (masked
// tokens and requests) stay untouched.
extern "C" int warp34_paged_attention_gated_f16(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                                const warp34_attention_batch* batch, const void* q_in,
                                                const void* gate, void* attn_out, int num_q_heads) {
    const int rc = common_checks(ex, layout, batch, q_in, attn_out, num_q_heads);
    if (rc) return rc;
    if (gate == nullptr) return (int)hipErrorInvalidValue;
    if (layout->k_format == WARP34_KV_FORMAT_FP8_E4M3 || layout->v_format == WARP34_KV_FORMAT_FP8_E4M3) {
        if (layout->head_dim != 256) return (int)hipErrorInvalidValue;
    }
    if (batch->total_tokens <= 0 || num_q_heads <= 0) return 0;
    if ((((uintptr_t)gate) & 7u) != 0) return (int)hipErrorNotSupported;
    return attention_entry<F16>(ex, layout, batch, q_in, attn_out, num_q_heads, 0, gate);
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
    // the reference's selector picks the 16-row kernel (0) or one of its 64 / 128-row prefill kernels;
    // here: the decode / verify kernel as a single pass, or the 128-row tile kernel
    return attention_entry<F16>(ex, layout, batch, q_in, attn_out, num_q_heads, use_64q == 0 ? 1 : 2);
}

// Scratch that lets a batch split fully, computed the way the launchers compute it.
// q_group / q_subgroups as in launch_tq4 / launch_rows; local_kv_heads <= 0: not known, take the
// largest need over all layouts with this many q heads.
static size_t scratch_bytes_for(int local_kv_heads, int total_tokens, int num_reqs, int num_q_heads,
                                int max_seq_len, int max_q_len = 0) {
    if (total_tokens <= 0 || num_q_heads <= 0) return 0;
    int q_group = 1, q_subgroups = 1, kv_subs = num_q_heads;  // the bound when the layout is unknown
    int tok_tile = 16;
    if (local_kv_heads > 0 && num_q_heads % local_kv_heads == 0) {
        const int gqa = num_q_heads / local_kv_heads;
        q_group = gqa;
        if (q_group > 16) {
            for (int d = 16; d >= 1; --d)
                if (gqa % d == 0) {
                    q_group = d;
                    break;
                }
        }
        q_subgroups = gqa / q_group;
        kv_subs = local_kv_heads * q_subgroups;
        tok_tile = 16 / q_group < 1 ? 1 : 16 / q_group;
    }
    const int tiles = (total_tokens + tok_tile - 1) / tok_tile;
    long long want = kTargetWorkgroupsPerHead / ((long long)tiles * q_subgroups);
    if (want > kMaxChunksCap) want = kMaxChunksCap;
    if (max_seq_len > 0) {
        const int units = (max_seq_len + kUnit - 1) / kUnit + 1;
        const int bound = (units + kMinUnitsPerChunk - 1) / kMinUnitsPerChunk;
        if (bound < want) want = bound;
    }
    size_t bytes = want >= 2 ? partial_bytes((long long)total_tokens * num_q_heads, (int)want) : 0;
    // verify batches over long contexts may take the shared-prefix pass: its partial slots sit
    // behind the split-K ones, and a header behind the records
    if (want >= 2 && total_tokens >= 16 && (num_reqs < 0 || num_reqs >= 4) && max_seq_len >= 8 * kSpMinTokens &&
        (max_q_len <= 0 || (max_q_len >= 2 && max_q_len <= kPfRows / q_group)) && (q_group & (q_group - 1)) == 0) {
        const int parts = shared_prefix_parts(total_tokens, q_group, q_subgroups);
        if ((int)want + parts <= kMergeGroups * kMergeMaxPerGroup)
            bytes = partial_bytes((long long)total_tokens * num_q_heads, (int)want + parts) + sizeof(SpHeader);
    }
    // balanced decode: (shares + requests) partial slots of 16 columns per (kv head, q subgroup)
    // and the per-token table
    // (only batches in which no request has more than one tile take it; max_q_len <= 0: not known)
    if (num_reqs < 0 || num_reqs > total_tokens) num_reqs = total_tokens;
    if (num_reqs >= 2 && max_q_len <= tok_tile) {
        const size_t prows = bal_partial_row(balanced_groups(q_subgroups) + num_reqs, kv_subs, 0, 0);
        const size_t bal = partial_bytes((long long)prows, 1) + (size_t)total_tokens * 16;
        if (bal > bytes) bytes = bal;
    }
    return bytes;
}

extern "C" size_t warp34_paged_attention_scratch_bytes(int total_tokens, int num_q_heads, int max_seq_len) {
    return scratch_bytes_for(0, total_tokens, -1, num_q_heads, max_seq_len);
}

extern "C" size_t warp34_paged_attention_scratch_bytes_for_layout(const warp34_kv_layer_layout* layout,
                                                                  int total_tokens, int num_reqs, int num_q_heads,
                                                                  int max_seq_len) {
    if (!layout) return 0;
    return scratch_bytes_for(layout->local_kv_heads, total_tokens, num_reqs, num_q_heads, max_seq_len);
}

// op_qsa.cu:1711-1730
extern "C" int warp34_qsa_sparse_paged_attn_f16(const warp34_exec* ex, const void* q, const void* gate,
                                                const warp34_kv_layer_layout* kv_layout,
                                                const int32_t* selected_phys_blocks,
                                                const int32_t* selected_logical_blocks,
                                                const int32_t* num_selected_blocks, const int32_t* token_seq_pos,
                                                const uint8_t* valid_token_mask, void* out, int num_tokens,
                                                int local_q_heads, int select_k_blocks, float sm_scale) {
    return launch_qsa_sparse(ex, q, gate, kv_layout, selected_phys_blocks, selected_logical_blocks,
                             num_selected_blocks, token_seq_pos, valid_token_mask, out, num_tokens, local_q_heads,
                             select_k_blocks, sm_scale, 0);
}

// op_qsa.cu:1732-1751
extern "C" int warp34_qsa_sparse_paged_attn_hadamard_f16(
    const warp34_exec* ex, const void* q, const void* gate, const warp34_kv_layer_layout* kv_layout,
    const int32_t* selected_phys_blocks, const int32_t* selected_logical_blocks,
    const int32_t* num_selected_blocks, const int32_t* token_seq_pos, const uint8_t* valid_token_mask, void* out,
    int num_tokens, int local_q_heads, int select_k_blocks, float sm_scale) {
    return launch_qsa_sparse(ex, q, gate, kv_layout, selected_phys_blocks, selected_logical_blocks,
                             num_selected_blocks, token_seq_pos, valid_token_mask, out, num_tokens, local_q_heads,
                             select_k_blocks, sm_scale, 1);
}

// ---- an entry point that allocates nothing -----------------------------------------------------
// warp34_paged_attention_bf16 with the split-K scratch in a file-scope device array instead of
// ex->scratch_ptr, for callers that cannot provide (or allocate) a workspace.  Every device the
// library runs on holds its own copy of the array at its own address; the address is looked up
// once per device, with that device current, and kept.  The array's NAME is a host-side stand-in
// and is never passed to a kernel or a runtime call: only the looked-up address is.
namespace w34 {
constexpr size_t kStaticScratchBytes = WARP34_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];
constexpr int kStaticScratchDevices = 64;
static std::atomic<uintptr_t> g_static_scratch_addr[kStaticScratchDevices];

static int static_scratch_address(uintptr_t* out) {
    int dev = 0;
    hipError_t rc = hipGetDevice(&dev);
    if (rc != hipSuccess) return (int)rc;
    if (dev < 0 || dev >= kStaticScratchDevices) return (int)hipErrorInvalidDevice;
    uintptr_t addr = g_static_scratch_addr[dev].load(std::memory_order_acquire);
    if (addr == 0) {
        void* sym = nullptr;
        rc = hipGetSymbolAddress(&sym, HIP_SYMBOL(g_static_scratch));
        if (rc != hipSuccess) return (int)rc;
        if (sym == nullptr || ((uintptr_t)sym & 15u) != 0u) return (int)hipErrorInvalidSymbol;
        addr = (uintptr_t)sym;
        g_static_scratch_addr[dev].store(addr, std::memory_order_release);
    }
    *out = addr;
    return 0;
}
}  // namespace w34

extern "C" int warp34_paged_attention_bf16_static_scratch(const warp34_exec* ex, const warp34_kv_layer_layout* layout,
                                                          const warp34_attention_batch* batch, const void* q_in,
                                                          void* attn_out, int num_q_heads) {
    const int rc = common_checks(ex, layout, batch, q_in, attn_out, num_q_heads);
    if (rc) return rc;
    if (num_q_heads <= 0 || batch->total_tokens < 0) return (int)hipErrorInvalidValue;
    if (!batch->total_tokens) return 0;
    // The array serves every batch the way an 8 MiB ex->scratch would: the launchers take fewer
    // chunks, or leave a pass out, when the records of the full split do not fit.  Refused are only
    // batches too large for the array to be of any use: not even two records per query row fit.
    const long long rows = (long long)batch->total_tokens * num_q_heads;
    if (partial_bytes(rows, 2) > kStaticScratchBytes) return (int)hipErrorOutOfMemory;
    uintptr_t addr = 0;
    const int arc = static_scratch_address(&addr);
    if (arc) return arc;
    warp34_exec own = *ex;
    own.scratch_ptr = addr;
    own.scratch_size = kStaticScratchBytes;
    return attention_entry<BF16>(&own, layout, batch, q_in, attn_out, num_q_heads, 0);
}
