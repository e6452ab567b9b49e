// QSA sparse paged attention over TQ4 pages for gfx950: every query token attends over its own
// list of selected 4-token groups (ops/op_qsa.cu:716-1158, 1446-1571 of the reference).
//
// The streaming core is the one of the dense TQ4 decode kernel (pair table in LDS, S^T = K Q'^T
// and O^T += V^T P^T on v_mfma_f32_16x16x32_f16, one query column per lane); what differs is where
// the keys come from.  A 32-token unit is eight selected groups; a group is four consecutive rows
// of one page, 528 bytes = 33 16-byte pieces, so a unit is still 4 x 132 pieces per K and V and
// lands in LDS in the layout the core expects.  Only the piece addresses change: they are
// per-lane (group id -> page, row) instead of a wave-uniform run base.
//
//   grid  = (query tokens, kv heads x q subgroups, splits), block = 8 waves
//   split = an equal share of the token's units; every split writes an (m, l) record (l = 0
//           without work), the merge kernel adds them up.  One split finishes in the kernel.
//   tail  = rotate back, sigmoid gate, fp16 rounding, optional H64 / 8 over every 64-element
//           block of the rounded row (ops/hadamard_inline.cuh:11-50)
//
// Included by paged_attn.hip after the dense kernels (shares their device helpers).
#pragma once

namespace w34 {

constexpr int kQsaWaves = 8;
constexpr int kQsaLoopBytes = kLutBytes + kQsaWaves * kStageTq4;
constexpr int kQsaColStride = 260;
constexpr int kQsaRegion = 16 * kQsaColStride;  // floats per wave
constexpr int kQsaMergeBytes = kQsaWaves * kQsaRegion * 4;
constexpr int kQsaMlBytes = (kQsaWaves + 1) * 16 * 2 * 4;
constexpr int kQsaSmem = (kQsaLoopBytes > kQsaMergeBytes ? kQsaLoopBytes : kQsaMergeBytes) + kQsaMlBytes;
constexpr int kQsaMaxSplits = 16;

struct QsaParams {
    warp34_kv_layer_layout L;
    const uint16_t* q;
    const uint16_t* gate;  // may be null
    uint16_t* out;
    const int32_t* sel_phys;
    const int32_t* sel_log;
    const int32_t* num_sel;
    const int32_t* seq_pos;
    const uint8_t* valid_token_mask;  // may be null
    float* part_acc;  // [rows][n_splits][256]
    float* part_ml;   // [rows][n_splits][4]: m, l, -, -
    int num_tokens, num_q_heads, gqa, q_group, q_subgroups, select_k, n_splits, had64;
    int groups_per_page;
    int gpp_shift;  // log2(groups_per_page), or -1 when it is not a power of two
    float sm_scale;
    float out_scale;  // factor of the un-normalised sums (the table gain of the TQ4 form, else 1)
    int rot_q;        // row-format form: K rows are stored rotated, rotate the query rows
    int rot_out;      // V rows are stored rotated: rotate the finished row back
};

// The end of a row: v = element 4 lane + k of the normalised sum in the rotated domain.
__device__ __forceinline__ uint2 qsa_load_gate(const uint16_t* gate, size_t row, int lane) {
    return gate != nullptr ? *reinterpret_cast<const uint2*>(gate + row * kHeadDim + 4 * lane) : uint2{0u, 0u};
}
// g: the row's gate values (qsa_load_gate, requested by the caller ahead of the sums)
__device__ __forceinline__ void qsa_finish_row(float (&v)[4], int lane, size_t row, bool rotate,
                                               bool has_gate, uint2 g, bool had64, uint16_t* out) {
    if (rotate) {
        wht256_wave(v, lane);
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = apply_sign(v[k], 4 * lane + k);
    }
    if (has_gate) {
        const float gv[4] = {F16::to_f32((uint16_t)(g.x & 0xFFFFu)), F16::to_f32((uint16_t)(g.x >> 16)),
                             F16::to_f32((uint16_t)(g.y & 0xFFFFu)), F16::to_f32((uint16_t)(g.y >> 16))};
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] *= 1.0f / (1.0f + expf(-gv[k]));
    }
    uint16_t h[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) h[k] = F16::from_f32(v[k]);
    if (had64) {
        // H64 / 8 over the 16 lanes that hold one 64-element block, on the rounded values, sums in
        // fp32 in the reference's order
        float x[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) x[k] = F16::to_f32(h[k]);
        const float a0 = x[0] + x[1], a1 = x[0] - x[1], a2 = x[2] + x[3], a3 = x[2] - x[3];
        x[0] = a0 + a2;
        x[1] = a1 + a3;
        x[2] = a0 - a2;
        x[3] = a1 - a3;
        wht_stage<1>(x, lane);
        wht_stage<2>(x, lane);
        wht_stage<4>(x, lane);
        wht_stage<8>(x, lane);
#pragma unroll
        for (int k = 0; k < 4; ++k) h[k] = F16::from_f32(x[k] * 0.125f);
    }
    uint2 o;
    o.x = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
    o.y = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
    *reinterpret_cast<uint2*>(out + row * kHeadDim + 4 * lane) = o;
}

__global__ __launch_bounds__(kQsaWaves * 64, 1) void qsa_sparse_tq4_kernel(const QsaParams P) {
    extern __shared__ __align__(16) uint8_t smem[];
    // lut_read() addresses the table absolutely: the dynamic block starts at LDS address 0 because
    // the kernel has no static LDS (checked on the host before the first launch)
    uint8_t* stage_all = smem + kLutBytes;

    const int tid = (int)threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int b = lane >> 4;
    const warp34_kv_layer_layout& L = P.L;

    const int tok = (int)blockIdx.x;
    const int kv_sub = (int)blockIdx.y;
    const int split = (int)blockIdx.z;
    const int kv_head = fast_div(kv_sub, P.q_subgroups);
    const int q_head_base = kv_head * P.gqa + (kv_sub - kv_head * P.q_subgroups) * P.q_group;

    // ---- this token's list ------------------------------------------------------------------------
    // The counts and the list entries of this wave's first unit are requested together: the first
    // unit is guessed from the list's capacity (exact when the list is full, the common case) and
    // fetched again when the guess is wrong, so the guess changes the latency only.
    const int32_t* tok_phys = P.sel_phys + (size_t)tok * P.select_k;
    const int32_t* tok_log = P.sel_log + (size_t)tok * P.select_k;
    const int upc_guess = fast_div(((P.select_k + 7) >> 3) + P.n_splits - 1, P.n_splits);
    const int unit_guess = split * upc_guess + wave;
    int spec_id = -1, spec_lg = 0;
    {
        const int gi = unit_guess * 8 + (lane & 7);
        if (gi < P.select_k) {
            spec_id = tok_phys[gi];
            spec_lg = tok_log[gi];
        }
    }
    int a_live = 1, a_sel = P.num_sel[tok], a_pos = P.seq_pos[tok];  // one vector load each, no scalar-cache trip
    if (P.valid_token_mask != nullptr) a_live = (int)P.valid_token_mask[tok];

    // ---- query rows of this wave's columns (column c = q head q_head_base + c, c < q_group) ----------
    constexpr int kColsPerWave = 16 / kQsaWaves;
    uint2 q_raw[kColsPerWave];
#pragma unroll
    for (int c = 0; c < kColsPerWave; ++c) {
        const int col = wave + c * kQsaWaves;
        q_raw[c] = uint2{0u, 0u};
        if (col < P.q_group) {
            const uint16_t* qrow = P.q + ((size_t)tok * P.num_q_heads + (size_t)(q_head_base + col)) * kHeadDim;
            q_raw[c] = *reinterpret_cast<const uint2*>(qrow + 4 * lane);
        }
    }
    {
        // entry e = (gain * centroid[e & 15], gain * centroid[e >> 4]) as packed fp16, 64 copies
        const int e = tid >> 1;
        const uint32_t v = pack_h2(kLutGain * centroid_of_code(e & 15), kLutGain * centroid_of_code(e >> 4));
        u4 vv = {v, v, v, v};
        u4* dst = reinterpret_cast<u4*>(smem + e * 256 + (tid & 1) * 128);
#pragma unroll
        for (int k = 0; k < 8; ++k) dst[k] = vv;
    }

    int n_sel = __builtin_amdgcn_readfirstlane(a_live) != 0 ? __builtin_amdgcn_readfirstlane(a_sel) : 0;
    if (n_sel > P.select_k) n_sel = P.select_k;
    if (n_sel < 0) n_sel = 0;
    const int seq_pos = __builtin_amdgcn_readfirstlane(a_pos);
    const int n_units = (n_sel + 7) >> 3;
    const int upc = fast_div(n_units + P.n_splits - 1, P.n_splits);
    const int cu_first = split * upc;
    int cu_end = cu_first + upc;
    if (cu_end > n_units) cu_end = n_units;

    // ---- staging machinery ------------------------------------------------------------------------
    const uint8_t* k_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.k_base) + (size_t)kv_head * L.k_head_stride_bytes;
    const uint8_t* v_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.v_base) + (size_t)kv_head * L.v_head_stride_bytes;
    uint8_t* stage = stage_all + wave * kStageTq4;
    // Piece p of a 16-row run belongs to group p / 33 of the run's four groups.  Lane l carries
    // pieces l and 64 + l of every run; lanes 0-15 also carry the tail pieces 128 + (l & 3) of run
    // l >> 2.
    const int pa_g = lane / 33, pa_o = lane - 33 * pa_g;
    const int pb_g = (64 + lane) / 33, pb_o = 64 + lane - 33 * pb_g;
    const int pt_o = 29 + (lane & 3);  // pieces 128-131 are pieces 29-32 of group 3
    u4 pf[9];
    // lane l holds group (l & 7) of a unit: physical id (or -1) and first key position (or a
    // position that is never visible)
    auto load_groups = [&](int unit, int& id_vec, int& pos_vec) {
        const int gi = unit * 8 + (lane & 7);
        int id = -1, lg = 0;
        if (gi < n_sel) {
            id = tok_phys[gi];
            lg = tok_log[gi];
        }
        id_vec = id;
        pos_vec = id >= 0 ? 4 * lg : 0x3fffffff;
    };
    // Base of a group's four rows in the K and the V slab.  The ids come out of readlane, so this
    // is scalar arithmetic; a skipped group reads group 0 of page 0: any TQ4 bytes dequantise to
    // finite values, and every key of such a group is masked.
    auto group_base = [&](int id, const uint8_t*& kp, const uint8_t*& vp) {
        const int gid = id >= 0 ? id : 0;
        // pages of 2^k tokens (the usual case): shift and mask
        const int pg = P.gpp_shift >= 0 ? gid >> P.gpp_shift : gid / P.groups_per_page;
        const int row = (gid - pg * P.groups_per_page) * 4;
        kp = k_base + (size_t)pg * L.k_page_stride_bytes + (size_t)row * L.k_token_stride_bytes;
        vp = v_base + (size_t)pg * L.v_page_stride_bytes + (size_t)row * L.v_token_stride_bytes;
    };
    auto issue_loads = [&](int id_vec) {
        const uint8_t *kt[2], *vt[2];
#pragma unroll
        for (int hr = 0; hr < 2; ++hr) {  // rows 0-15 / 16-31 of the unit = groups 0-3 / 4-7
            const uint8_t *kg[4], *vg[4];
#pragma unroll
            for (int gi = 0; gi < 4; ++gi) group_base(__builtin_amdgcn_readlane(id_vec, 4 * hr + gi), kg[gi], vg[gi]);
            // piece lane: group 0 or 1; piece 64 + lane: group 1, 2 or 3
            const uint8_t* ka = (pa_g == 0 ? kg[0] : kg[1]) + 16 * pa_o;
            const uint8_t* va = (pa_g == 0 ? vg[0] : vg[1]) + 16 * pa_o;
            const uint8_t* kb = (pb_g == 1 ? kg[1] : pb_g == 2 ? kg[2] : kg[3]) + 16 * pb_o;
            const uint8_t* vb = (pb_g == 1 ? vg[1] : pb_g == 2 ? vg[2] : vg[3]) + 16 * pb_o;
            pf[2 * hr] = *(global_cu4*)ka;
            pf[2 * hr + 1] = *(global_cu4*)kb;
            pf[4 + 2 * hr] = *(global_cu4*)va;
            pf[4 + 2 * hr + 1] = *(global_cu4*)vb;
            kt[hr] = kg[3];
            vt[hr] = vg[3];
        }
        {
            const int r = (lane >> 2) & 3;  // run: K rows 0-15, K rows 16-31, V rows 0-15, V rows 16-31
            const uint8_t* base = r == 0 ? kt[0] : r == 1 ? kt[1] : r == 2 ? vt[0] : vt[1];
            pf[8] = *(global_cu4*)(base + 16 * pt_o);
        }
    };
    auto commit_loads = [&]() {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            *reinterpret_cast<u4*>(stage + r * kRunBytes + 16 * lane) = pf[2 * r];
            *reinterpret_cast<u4*>(stage + r * kRunBytes + 1024 + 16 * lane) = pf[2 * r + 1];
        }
        if (lane < 16) *reinterpret_cast<u4*>(stage + (lane >> 2) * kRunBytes + 2048 + 16 * (lane & 3)) = pf[8];
    };

    int unit = cu_first + wave;
    int id_vec = -1, pos_vec = 0x3fffffff;
    if (unit < cu_end) {
        if (unit == unit_guess) {  // wave-uniform
            const bool in_list = unit * 8 + (lane & 7) < n_sel;
            id_vec = in_list ? spec_id : -1;
            pos_vec = id_vec >= 0 ? 4 * spec_lg : 0x3fffffff;
        } else {
            load_groups(unit, id_vec, pos_vec);
        }
    }
    issue_loads(id_vec);  // harmless for a wave without work

    // ---- rotated, scaled fp16 queries to LDS, then the B operands of the QK MFMAs -----------------
    constexpr int kQStride = 264;
    _Float16* qlds = reinterpret_cast<_Float16*>(stage_all);
    const float q_scale = P.sm_scale * kLog2e * kLutInvGain;
#pragma unroll
    for (int c = 0; c < kColsPerWave; ++c) {
        const int col = wave + c * kQsaWaves;
        float qv[4] = {F16::to_f32((uint16_t)(q_raw[c].x & 0xFFFFu)), F16::to_f32((uint16_t)(q_raw[c].x >> 16)),
                       F16::to_f32((uint16_t)(q_raw[c].y & 0xFFFFu)), F16::to_f32((uint16_t)(q_raw[c].y >> 16))};
        if (col < P.q_group) {  // wave-uniform; dead columns stay zero
#pragma unroll
            for (int k = 0; k < 4; ++k) qv[k] = apply_sign(qv[k], 4 * lane + k);
            wht256_wave(qv, lane);
        }
        uint2 packed;
        packed.x = pack_h2(qv[0] * q_scale, qv[1] * q_scale);
        packed.y = pack_h2(qv[2] * q_scale, qv[3] * q_scale);
        *reinterpret_cast<uint2*>(qlds + col * kQStride + 4 * lane) = packed;
    }
    __syncthreads();
    h8 bq[9];
    {
        const int kb = 8 * (b & 1) + 4 * (b >> 1);
        const uint8_t* qrow = reinterpret_cast<const uint8_t*>(qlds + n * kQStride);
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            const int D = kb + m;
            u2v lo = *reinterpret_cast<const u2v*>(qrow + (D > 0 ? 16 * D - 8 : 0));
            if (D == 0) lo = u2v{0u, 0u};
            const u2v hi = *reinterpret_cast<const u2v*>(qrow + 16 * D);
            bq[m] = __builtin_bit_cast(h8, u4{lo[0], lo[1], hi[0], hi[1]});
        }
        {
            u2v lo = *reinterpret_cast<const u2v*>(qrow + 248);
            if (b != 0) lo = u2v{0u, 0u};
            bq[4] = __builtin_bit_cast(h8, u4{lo[0], lo[1], 0u, 0u});
        }
#pragma unroll
        for (int m = 0; m < 4; ++m) bq[5 + m] = *reinterpret_cast<const h8*>(qrow + 256 + 16 * (kb + m));
    }
    __syncthreads();  // qlds is dead, the staging area may be overwritten; the table is complete

    const uint32_t lut_lane = (uint32_t)lane << 2;
    const bool col_ok = n < P.q_group;
    f4 o_acc[2][8];
    float m_run = kNegBig, l_run = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) o_acc[h][j] = f4{0.f, 0.f, 0.f, 0.f};

    // One 32-token unit.  gp0 / gp1: first key position of the groups that hold this lane's key
    // slots 0-3 / 4-7 (group 4 (b & 1) + (b >> 1), and that group + 2).
    auto process_unit = [&](int gp0, int gp1, const bool MASKED) {
        const uint8_t* k_rows = stage;
        const uint8_t* v_rows = stage + 2 * kRunBytes;
        float sc[8];
        uint32_t kw[2][9], ks0[2][4], ks16[2][4];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int arow = unit_token(s, n >> 2, n & 3);
            const uint32_t* row32 = reinterpret_cast<const uint32_t*>(k_rows + arow * kTq4RowBytes);
#pragma unroll
            for (int mf = 0; mf < 9; ++mf) kw[s][mf] = row32[tq4_qk_dword(mf < 5 ? 0 : 1, mf < 5 ? mf : mf - 5, b)];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t* r32 = reinterpret_cast<const uint32_t*>(k_rows + unit_token(s, b, i) * kTq4RowBytes);
                ks0[s][i] = r32[0];
                ks16[s][i] = r32[16];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            u4 a[9];
#pragma unroll
            for (int mf = 0; mf < 9; ++mf) {
                const uint32_t w = kw[s][mf];
                a[mf][0] = lut_read(w, lut_lane, 0x0c0c0400u);
                a[mf][1] = lut_read(w, lut_lane, 0x0c0c0500u);
                a[mf][2] = lut_read(w, lut_lane, 0x0c0c0600u);
                a[mf][3] = lut_read(w, lut_lane, 0x0c0c0700u);
            }
            __builtin_amdgcn_sched_barrier(0);
            f4 s_acc[2] = {f4{0.f, 0.f, 0.f, 0.f}, f4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
            for (int m = 0; m < 5; ++m) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    if (h == 1 && m == 4) continue;
                    const int mf = h == 0 ? m : 5 + m;
                    s_acc[h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a[mf]), bq[mf], s_acc[h], 0, 0, 0);
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
                sc[4 * s + i] = half_lo_to_f32(ks0[s][i]) * s_acc[0][i] + half_hi_to_f32(ks16[s][i]) * s_acc[1][i];
        }
        if (MASKED) {
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int pos = (t < 4 ? gp0 : gp1) + (t & 3);
                sc[t] = (col_ok && pos <= seq_pos) ? sc[t] : kNegBig;
            }
        }
        uint32_t vd0[8], vd16[8], vwr[8], vw1[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const int trow = unit_token(t >> 2, b, t & 3);
            const uint32_t* row32 = reinterpret_cast<const uint32_t*>(v_rows + trow * kTq4RowBytes);
            vd0[t] = row32[0];
            vd16[t] = row32[16];
            vwr[t] = row32[n];
            vw1[t] = row32[17 + n];
        }
        float p[8];
        {
            float mx = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
            mx = max_over_rows(mx);
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
            m_run = m_new;
            float psum = 0.f;
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
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            // probability times the half-row scale of the value row, as a high and a low fp16
            // operand (split_h2): one rounding would be shared by the whole scale block
            uint32_t pb_hi[4], pb_lo[4];
            {
                float w[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) w[t] = p[t] * (h == 0 ? half_lo_to_f32(vd0[t]) : half_hi_to_f32(vd16[t]));
                if (MASKED) {
#pragma unroll
                    for (int t = 0; t < 8; ++t) w[t] = p[t] > 0.f ? w[t] : 0.f;
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) split_h2(w[2 * k], w[2 * k + 1], pb_hi[k], pb_lo[k]);
            }
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
                lo[k] = (wa & 0x0F0F0F0Fu) | ((wb << 4) & 0xF0F0F0F0u);
                hi[k] = ((wa >> 4) & 0x0F0F0F0Fu) | (wb & 0xF0F0F0F0u);
            }
            u4 a[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const uint32_t src = (j & 1) ? hi[k] : lo[k];
                    const uint32_t sel = 0x0c0c0400u + ((uint32_t)(j >> 1) << 8);
                    a[j][k] = lut_read(src, lut_lane, sel);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            const u4 ph = {pb_hi[0], pb_hi[1], pb_hi[2], pb_hi[3]};
            const u4 pl = {pb_lo[0], pb_lo[1], pb_lo[2], pb_lo[3]};
#pragma unroll
            for (int j = 0; j < 8; ++j)
                o_acc[h][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a[j]),
                                                                    __builtin_bit_cast(h8, ph), o_acc[h][j], 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 8; ++j)  // (a pass of its own: a tile's two MFMAs are not back to back)
                o_acc[h][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a[j]),
                                                                    __builtin_bit_cast(h8, pl), o_acc[h][j], 0, 0, 0);
        }
    };

    while (unit < cu_end) {
        commit_loads();
        const int cur_pos_vec = pos_vec;
        const int next_unit = unit + kQsaWaves;
        if (next_unit < cu_end) {
            load_groups(next_unit, id_vec, pos_vec);
            issue_loads(id_vec);
        }
        const int ga = 4 * (b & 1) + (b >> 1);
        const int gp0 = __shfl(cur_pos_vec, ga, 64);
        const int gp1 = __shfl(cur_pos_vec, ga + 2, 64);
        // interior unit: all eight groups present and wholly in front of the token's position
        const bool interior = __ballot(lane < 8 && cur_pos_vec + 3 > seq_pos) == 0ull;
        process_unit(gp0, gp1, !interior);
        unit = next_unit;
    }

    // ---- merge the waves' states through LDS (layout as in the dense kernel) -------------------------
    l_run = sum_over_rows(l_run);
    float* xbuf = reinterpret_cast<float*>(smem);
    float* mlbuf = reinterpret_cast<float*>(smem + (kQsaSmem - kQsaMlBytes));
    if (b == 0) {
        mlbuf[(wave * 16 + n) * 2 + 0] = m_run;
        mlbuf[(wave * 16 + n) * 2 + 1] = l_run;
    }
    __syncthreads();  // every wave is done with the table and with its staging area
    {
        float mt = kNegBig;
#pragma unroll
        for (int w = 0; w < kQsaWaves; ++w) mt = fmaxf(mt, mlbuf[(w * 16 + n) * 2]);
        float lt = 0.f;
#pragma unroll
        for (int w = 0; w < kQsaWaves; ++w)
            lt += mlbuf[(w * 16 + n) * 2 + 1] * __builtin_amdgcn_exp2f(mlbuf[(w * 16 + n) * 2] - mt);
        const float wgt = __builtin_amdgcn_exp2f(m_run - mt);
        float* c = xbuf + wave * kQsaRegion + n * kQsaColStride;
        if (col_ok) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < 8; ++j) *reinterpret_cast<f4*>(c + ((h * 8 + j) * 4 + b) * 4) = o_acc[h][j] * wgt;
        }
        float* mltot = mlbuf + kQsaWaves * 16 * 2;
        if (wave == 0 && b == 0) {
            mltot[n * 2 + 0] = mt;
            mltot[n * 2 + 1] = lt;
        }
    }
    __syncthreads();
    const float* mltot = mlbuf + kQsaWaves * 16 * 2;

    int merge_slot[4];  // region slot of element 4 lane + k (inverse of tq4_pv_elem)
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
    for (int col = wave; col < P.q_group; col += kQsaWaves) {
        const size_t row = (size_t)tok * P.num_q_heads + (size_t)(q_head_base + col);
        uint2 g = {0u, 0u};
        if (P.n_splits == 1) g = qsa_load_gate(P.gate, row, lane);
        float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < kQsaWaves; ++w) {
            const float* c = xbuf + w * kQsaRegion + col * kQsaColStride;
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] += c[merge_slot[k]];
        }
        const float m_col = mltot[col * 2 + 0];
        const float l_col = mltot[col * 2 + 1];
        if (P.n_splits > 1) {
            const size_t prow = row * P.n_splits + split;
            *reinterpret_cast<f4*>(P.part_acc + prow * kHeadDim + 4 * lane) = f4{v[0], v[1], v[2], v[3]};
            if (lane == 0) *reinterpret_cast<f4*>(P.part_ml + prow * 4) = f4{m_col, l_col, 0.f, 0.f};
        } else {
            if (!(l_col > 0.f)) {  // masked token or no visible key: a row of (positive) zeros
                *reinterpret_cast<uint2*>(P.out + row * kHeadDim + 4 * lane) = uint2{0u, 0u};
                continue;
            }
            const float inv = kLutInvGain / l_col;
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] *= inv;
            qsa_finish_row(v, lane, row, true, P.gate != nullptr, g, P.had64 != 0, P.out);
        }
    }
}

// One wave per (token, q head) row: lane s holds the record of split s (n_splits <= 16).
__global__ __launch_bounds__(64) void qsa_sparse_merge_kernel(const QsaParams P) {
    const int lane = (int)threadIdx.x;
    const size_t row = (size_t)blockIdx.x;
    const float* ml = P.part_ml + row * P.n_splits * 4;
    const float* acc = P.part_acc + row * P.n_splits * kHeadDim;
    f4 rec = {kNegBig, 0.f, 0.f, 0.f};
    if (lane < P.n_splits) rec = *reinterpret_cast<const f4*>(ml + 4 * lane);
    const uint2 g = qsa_load_gate(P.gate, row, lane);
    f4 a[kQsaMaxSplits];
#pragma unroll
    for (int s = 0; s < kQsaMaxSplits; ++s) {
        a[s] = f4{0.f, 0.f, 0.f, 0.f};
        if (s < P.n_splits) a[s] = *reinterpret_cast<const f4*>(acc + (size_t)s * kHeadDim + 4 * lane);
    }
    float m_tot = rec[1] > 0.f ? rec[0] : kNegBig;
    m_tot = fmaxf(m_tot, lane_xor<1>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<2>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<4>(m_tot, lane));
    m_tot = fmaxf(m_tot, lane_xor<8>(m_tot, lane));
    const float w_my = rec[1] > 0.f ? __builtin_amdgcn_exp2f(rec[0] - m_tot) : 0.f;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    float l_tot = 0.f;
#pragma unroll
    for (int s = 0; s < kQsaMaxSplits; ++s) {
        const float ws = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w_my), s));
        const float ls = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(rec[1]), s));
        if (s < P.n_splits && ws > 0.f) {  // wave-uniform
            l_tot += ls * ws;
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] += a[s][k] * ws;
        }
    }
    if (!(l_tot > 0.f)) {  // masked token or no visible key: a row of (positive) zeros
        *reinterpret_cast<uint2*>(P.out + row * kHeadDim + 4 * lane) = uint2{0u, 0u};
        return;
    }
    const float inv = P.out_scale / l_tot;
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] *= inv;
    qsa_finish_row(v, lane, row, P.rot_out != 0, P.gate != nullptr, g, P.had64 != 0, P.out);
}

}  // namespace w34
