// QSA sparse paged attention over pages whose rows are read as stored (FP16, FP8-E4M3-256,
// Q8_0-64; the 8-bit formats plain or rotated) for gfx950: the FP16, Q8_0 and FP8 branches of
// ops/op_qsa.cu:716-1073 of the reference.  Same decomposition as the TQ4 form in
// qsa_sparse_tq4.h (grid = tokens x (kv head, q subgroup) x splits, 8 waves, split records,
// qsa_sparse_merge_kernel), with the per-half body of the row-format decode kernel
// (paged_attn_rows.h): a 16-token half is four selected groups; a group is four consecutive rows
// of one page, so a half is gathered as four runs of 4 x row bytes and staged in LDS exactly as
// the dense kernel stages a contiguous run.
#pragma once

namespace w34 {

// VRES (8-bit value rows stored rotated): a second operand with the rounding residuals of
// fp16(d * code) and a second MFMA per P V tile, as in rows_tile.
template <int KVF, bool VRES = false>
__global__ __launch_bounds__(kKv16Waves * 64, 1) void qsa_sparse_rows_kernel(const QsaParams P) {
    static_assert(!VRES || KVF == WARP34_KV_FORMAT_FP8_E4M3 || KVF == WARP34_KV_FORMAT_Q8_0, "residual operand: 8-bit rows");
    constexpr bool K8 = KVF == WARP34_KV_FORMAT_FP8_E4M3 || KVF == WARP34_KV_FORMAT_Q8_0;
    constexpr bool FP8 = KVF == WARP34_KV_FORMAT_FP8_E4M3;
    constexpr int kWaves = kKv16Waves;
    constexpr int kRowStride = K8 ? kKv8RowStride : kKv16RowStride;  // LDS row stride
    constexpr int kRowBytes = K8 ? (FP8 ? 264 : 272) : 512;          // row in memory
    extern __shared__ __align__(16) uint8_t smem[];

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
    const bool col_ok = n < P.q_group;

    // ---- this token's list: counts and the entries of this wave's first half together (the first
    // half is guessed from the list's capacity and fetched again when the guess is wrong) ----
    const int32_t* tok_phys = P.sel_phys + (size_t)tok * P.select_k;
    const int32_t* tok_log = P.sel_log + (size_t)tok * P.select_k;
    const int hpc_guess = fast_div(((P.select_k + 3) >> 2) + P.n_splits - 1, P.n_splits);
    const int half_guess = split * hpc_guess + wave;
    int spec_id = -1, spec_lg = 0;
    {
        const int gi = half_guess * 4 + (lane & 3);
        if (gi < P.select_k) {
            spec_id = tok_phys[gi];
            spec_lg = tok_log[gi];
        }
    }
    int a_live = 1, a_sel = P.num_sel[tok], a_pos = P.seq_pos[tok];
    if (P.valid_token_mask != nullptr) a_live = (int)P.valid_token_mask[tok];

    // ---- query rows in MFMA B layout: lane (n, b) holds Q[column n][32 m + 8 b .. + 7] ----
    u4 bq[8];
    const bool rot_q = K8 && P.rot_q != 0;  // workgroup-uniform
    if (!rot_q) {
        const uint16_t* qrow = P.q + ((size_t)tok * P.num_q_heads + (size_t)(q_head_base + min(n, P.q_group - 1))) * kHeadDim;
#pragma unroll
        for (int m = 0; m < 8; ++m) bq[m] = *reinterpret_cast<const u4*>(qrow + 32 * m + 8 * b);
    } else {
        // rotated K rows: sign + WHT256 on the query rows (one row per wave at a time), staged as
        // fp16 in the still unused staging area and read back in MFMA layout
        constexpr int kQStride = 264;  // halves
        _Float16* qlds = reinterpret_cast<_Float16*>(smem);
        for (int col = wave; col < 16; col += kWaves) {
            const uint16_t* qrow = P.q + ((size_t)tok * P.num_q_heads + (size_t)(q_head_base + min(col, P.q_group - 1))) * kHeadDim;
            const uint2 raw = *reinterpret_cast<const uint2*>(qrow + 4 * lane);
            float v[4] = {F16::to_f32((uint16_t)(raw.x & 0xFFFFu)), F16::to_f32((uint16_t)(raw.x >> 16)),
                          F16::to_f32((uint16_t)(raw.y & 0xFFFFu)), F16::to_f32((uint16_t)(raw.y >> 16))};
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
        for (int m = 0; m < 8; ++m) bq[m] = *reinterpret_cast<const u4*>(qlds + n * kQStride + 32 * m + 8 * b);
        __syncthreads();  // the staging area is reused by the K/V rows
    }
    if (!col_ok) {
#pragma unroll
        for (int m = 0; m < 8; ++m) bq[m] = u4{0u, 0u, 0u, 0u};
    }

    int n_sel = __builtin_amdgcn_readfirstlane(a_live) != 0 ? __builtin_amdgcn_readfirstlane(a_sel) : 0;
    if (n_sel > P.select_k) n_sel = P.select_k;
    if (n_sel < 0) n_sel = 0;
    const int seq_pos = __builtin_amdgcn_readfirstlane(a_pos);
    const int n_halves = (n_sel + 3) >> 2;
    const int hpc = fast_div(n_halves + P.n_splits - 1, P.n_splits);
    const int ch_first = split * hpc;
    int ch_end = ch_first + hpc;
    if (ch_end > n_halves) ch_end = n_halves;

    const uint8_t* k_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.k_base) + (size_t)kv_head * L.k_head_stride_bytes;
    const uint8_t* v_base = reinterpret_cast<const uint8_t*>((uintptr_t)L.v_base) + (size_t)kv_head * L.v_head_stride_bytes;
    uint8_t* stage = smem + wave * kKv16Stage;  // [K rows 0..15][V rows 0..15], kRowStride each

    // lane l holds group (l & 3) of a half: physical id (or -1) and first key position (or a
    // position that is never visible)
    auto load_groups = [&](int half, int& id_vec, int& pos_vec) {
        const int gi = half * 4 + (lane & 3);
        int id = -1, lg = 0;
        if (gi < n_sel) {
            id = tok_phys[gi];
            lg = tok_log[gi];
        }
        id_vec = id;
        pos_vec = id >= 0 ? 4 * lg : 0x3fffffff;
    };
    // A half is fetched as 16-byte pieces c = lane + 64 i; piece c belongs to group c / kPpg
    // (kPpg pieces per group of four rows).  The four group bases are scalar (readlane).
    constexpr int kPieces = kRowBytes;            // 16 rows x row bytes / 16
    constexpr int kPpg = kRowBytes / 4;           // 128, 66 or 68
    constexpr int kLoads = (kPieces + 63) / 64;   // 8 or 5
    u4 pf[2 * kLoads];
    auto issue_half = [&](int id_vec) {
        const uint8_t *kg[4], *vg[4];
#pragma unroll
        for (int gi = 0; gi < 4; ++gi) {
            const int id = __builtin_amdgcn_readlane(id_vec, gi);
            const int gid = id >= 0 ? id : 0;  // skipped group: group 0 of page 0, its rows are stored as zeros
            const int pg = P.gpp_shift >= 0 ? gid >> P.gpp_shift : gid / P.groups_per_page;
            const int row = (gid - pg * P.groups_per_page) * 4;
            kg[gi] = k_base + (size_t)pg * L.k_page_stride_bytes + (size_t)row * L.k_token_stride_bytes;
            vg[gi] = v_base + (size_t)pg * L.v_page_stride_bytes + (size_t)row * L.v_token_stride_bytes;
        }
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            // pieces beyond the run (last, partial round of the 8-bit formats) re-read piece 0
            const int c = (kPieces % 64 == 0 || lane + 64 * i < kPieces) ? lane + 64 * i : 0;
            const int g_lo = (64 * i) / kPpg;  // group of lane 0's piece; lanes further up may be in the next one
            const int g = c / kPpg;
            const int o = c - g * kPpg;
            const uint8_t* kp = kg[g_lo];
            const uint8_t* vp = vg[g_lo];
            if (g_lo < 3 && (64 * i + 63) / kPpg > g_lo) {
                kp = g > g_lo ? kg[g_lo + 1] : kp;
                vp = g > g_lo ? vg[g_lo + 1] : vp;
            }
            if (g < g_lo) {  // the wrapped-around piece 0
                kp = kg[0];
                vp = vg[0];
            }
            pf[i] = *(global_cu4*)(kp + 16 * o);
            pf[kLoads + i] = *(global_cu4*)(vp + 16 * o);
        }
    };
    // rows that are not visible are stored as zeros: unwritten pool memory may hold NaN patterns,
    // and 0 * NaN would poison the P V product
    auto commit_half = [&](int pos_vec, bool edge) {
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
                    if (edge) {
                        const int pos = __shfl(pos_vec, (int)(row >> 2), 64) + (int)(row & 3u);
                        if (pos > seq_pos) {
                            k8 = u2v{0u, 0u};
                            v8 = u2v{0u, 0u};
                        }
                    }
                    *reinterpret_cast<u2v*>(k_rows + row * kRowStride + 8 * col) = k8;
                    *reinterpret_cast<u2v*>(v_rows + row * kRowStride + 8 * col) = v8;
                }
            } else {
                constexpr int kPiecesPerRow = kRowBytes / 16;  // 32 or 17
                const int row = (int)((unsigned)c / (unsigned)kPiecesPerRow);
                const int col = c - row * kPiecesPerRow;
                if (edge) {
                    const int pos = __shfl(pos_vec, row >> 2, 64) + (row & 3);
                    if (pos > seq_pos) {
                        kv = u4{0u, 0u, 0u, 0u};
                        vv = u4{0u, 0u, 0u, 0u};
                    }
                }
                *reinterpret_cast<u4*>(k_rows + row * kRowStride + 16 * col) = kv;
                *reinterpret_cast<u4*>(v_rows + row * kRowStride + 16 * col) = vv;
            }
        }
    };

    f4 o_acc[2][8];
    float m_run = kNegBig, l_run = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int j = 0; j < 8; ++j) o_acc[h][j] = f4{0.f, 0.f, 0.f, 0.f};
    const float score_scale = P.sm_scale * kLog2e;

    // gp: first key position of group b, the group of this lane's four tokens (rows 4b..4b+3)
    auto process_half = [&](int gp, const bool MASKED) {
        const uint8_t* k_rows = stage;
        const uint8_t* v_rows = stage + 16 * kRowStride;
        f4 s_acc = f4{0.f, 0.f, 0.f, 0.f};
        u2v a_v[2][8];
        u2v a_vr[VRES ? 2 : 1][VRES ? 8 : 1];  // residuals of a_v
        if constexpr (K8) {
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
                    dk[i][kb] = *reinterpret_cast<const float*>(k_rows + (4 * b + i) * kRowStride + (FP8 ? 256 + 4 * kb : 68 * kb));
#pragma unroll
            for (int kb = 0; kb < kBlocks; ++kb) {
                f4 part = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int mm = 0; mm < kMPerBlock; ++mm)
                    part = mfma_x32<false>(ka[kb * kMPerBlock + mm], bq[kb * kMPerBlock + mm], part);
#pragma unroll
                for (int i = 0; i < 4; ++i) s_acc[i] += dk[i][kb] * part[i];
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float vf[4][8];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint8_t* vrow = v_rows + (4 * b + i) * kRowStride;
                    const int blk = 2 * h + (n >> 3);
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
            u4 ka[8];
#pragma unroll
            for (int m = 0; m < 8; ++m) ka[m] = *reinterpret_cast<const u4*>(k_rows + n * kRowStride + 64 * m + 16 * b);
#pragma unroll
            for (int m = 0; m < 8; ++m) s_acc = mfma_x32<false>(ka[m], bq[m], s_acc);
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                u4 vr[4];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    vr[i] = *reinterpret_cast<const u4*>(v_rows + (4 * b + i) * kRowStride + 256 * h + 16 * n);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
                    a_v[h][j] = u2v{__builtin_amdgcn_perm(vr[1][j >> 1], vr[0][j >> 1], sel),
                                    __builtin_amdgcn_perm(vr[3][j >> 1], vr[2][j >> 1], sel)};
                }
            }
        }
        float sc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) sc[i] = s_acc[i] * score_scale;
        if (MASKED) {
#pragma unroll
            for (int i = 0; i < 4; ++i) sc[i] = (col_ok && gp + i <= seq_pos) ? sc[i] : kNegBig;
        }
        float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        mx = max_over_rows(mx);
        const float m_new = fmaxf(m_run, mx);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
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
        l_run = l_run * alpha + psum;
        if (__ballot(alpha != 1.0f) != 0ull) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < 8; ++j) o_acc[h][j] *= alpha;
        }
        const u2v pb = u2v{pack_h2(p[0], p[1]), pack_h2(p[2], p[3])};
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int j = 0; j < 8; ++j) o_acc[h][j] = mfma_x16<false>(a_v[h][j], pb, o_acc[h][j]);
        if constexpr (VRES) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < 8; ++j) o_acc[h][j] = mfma_x16<false>(a_vr[h][j], pb, o_acc[h][j]);
        }
    };

    int half = ch_first + wave;
    int id_vec = -1, pos_vec = 0x3fffffff;
    if (half < ch_end) {
        if (half == half_guess) {  // wave-uniform
            const bool in_list = half * 4 + (lane & 3) < n_sel;
            id_vec = in_list ? spec_id : -1;
            pos_vec = id_vec >= 0 ? 4 * spec_lg : 0x3fffffff;
        } else {
            load_groups(half, id_vec, pos_vec);
        }
    }
    issue_half(id_vec);  // harmless for a wave without work
    while (half < ch_end) {
        const int cur_pos_vec = pos_vec;
        // interior half: all four groups present and wholly in front of the token's position
        const bool edge = __ballot(lane < 4 && cur_pos_vec + 3 > seq_pos) != 0ull;
        commit_half(cur_pos_vec, edge);
        const int next_half = half + kWaves;
        if (next_half < ch_end) {
            load_groups(next_half, id_vec, pos_vec);
            issue_half(id_vec);
        }
        process_half(__shfl(cur_pos_vec, b, 64), edge);
        half = next_half;
    }

    // ---- merge of the waves' states (scheme and region layout of the dense kernels) ----
    l_run = sum_over_rows(l_run);
    constexpr int kColStride = kKv16ColStride;
    constexpr int kRegion = 16 * kColStride;
    float* xbuf = reinterpret_cast<float*>(smem);
    float* mlbuf = reinterpret_cast<float*>(smem + kv16_ml_offset(1));
    if (b == 0) {
        mlbuf[(wave * 16 + n) * 2 + 0] = m_run;
        mlbuf[(wave * 16 + n) * 2 + 1] = l_run;
    }
    __syncthreads();
    {
        float mt = kNegBig;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) mt = fmaxf(mt, mlbuf[(w * 16 + n) * 2]);
        float lt = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) lt += mlbuf[(w * 16 + n) * 2 + 1] * __builtin_amdgcn_exp2f(mlbuf[(w * 16 + n) * 2] - mt);
        const float wgt = __builtin_amdgcn_exp2f(m_run - mt);
        float* c = xbuf + wave * kRegion + n * kColStride;
        if (col_ok) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < 8; ++j) *reinterpret_cast<f4*>(c + ((h * 8 + j) * 4 + b) * 4) = o_acc[h][j] * wgt;
        }
        float* mltot = mlbuf + kWaves * 16 * 2;
        if (wave == 0 && b == 0) {
            mltot[n * 2 + 0] = mt;
            mltot[n * 2 + 1] = lt;
        }
    }
    __syncthreads();
    const float* mltot = mlbuf + kWaves * 16 * 2;
    // element e = 128 h + 8 r + j sits in slot ((h*8 + j)*4 + (r >> 2))*4 + (r & 3)
    int merge_slot[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int e = 4 * lane + k;
        const int h = e >> 7, r = (e >> 3) & 15, j = e & 7;
        merge_slot[k] = ((h * 8 + j) * 4 + (r >> 2)) * 4 + (r & 3);
    }
    for (int col = wave; col < P.q_group; col += kWaves) {
        const size_t row = (size_t)tok * P.num_q_heads + (size_t)(q_head_base + col);
        uint2 g = {0u, 0u};
        if (P.n_splits == 1) g = qsa_load_gate(P.gate, row, lane);
        float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float* c = xbuf + w * kRegion + col * kColStride;
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
            const float inv = 1.0f / l_col;
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] *= inv;
            qsa_finish_row(v, lane, row, P.rot_out != 0, P.gate != nullptr, g, P.had64 != 0, P.out);
        }
    }
}

}  // namespace w34
