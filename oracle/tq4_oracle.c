/*
 * tq4_oracle.c -- CPU restatement of the reference's TQ4 quantize-on-append, paged
 * layout addressing and paged GQA attention.  TEST INFRASTRUCTURE ONLY (see tq4_oracle.h
 * for the declared numerics and for what pins each function).
 *
 * Build: gcc -O2 -std=c99 -ffp-contract=off -fno-fast-math -fPIC -shared -pthread
 */
#define _GNU_SOURCE
#include "tq4_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

/* ---- tables: csrc/tq/tq4_codebook.cuh:46-101 (numeric literals are the contract) ---- */
static const float kCentroids[16] = {
    -1.694104124e-1f, -1.285881878e-1f, -1.006979993e-1f, -7.824930800e-2f,
    -5.873210384e-2f, -4.094919437e-2f, -2.420087619e-2f, -8.008373692e-3f,
    8.008373692e-3f,  2.420087619e-2f,  4.094919437e-2f,  5.873210384e-2f,
    7.824930800e-2f,  1.006979993e-1f,  1.285881878e-1f,  1.694104124e-1f,
};
static const float kBoundaries[15] = {
    -1.489993001e-1f, -1.146430936e-1f, -8.947365365e-2f, -6.849070592e-2f,
    -4.984064910e-2f, -3.257503528e-2f, -1.610462494e-2f, 0.000000000e0f,
    1.610462494e-2f,  3.257503528e-2f,  4.984064910e-2f,  6.849070592e-2f,
    8.947365365e-2f,  1.146430936e-1f,  1.489993001e-1f,
};
/* Seed-42 Rademacher diagonal, bit i set <=> sign[i] = -1 (little-endian 64-bit words). */
static const uint64_t kSignMask[4] = {
    0x4897475229e1d357ull, 0xf1297e2aeebc0de4ull, 0xe2eb25d0ba639274ull, 0x36b5bda1fde0ee14ull,
};
static float g_signs[256];
static pthread_once_t g_once = PTHREAD_ONCE_INIT;
static void init_tables(void) {
    for (int i = 0; i < 256; ++i)
        g_signs[i] = ((kSignMask[i >> 6] >> (i & 63)) & 1ull) ? -1.0f : 1.0f;
}
const float* tq4o_centroids256(void) { return kCentroids; }
const float* tq4o_boundaries256(void) { return kBoundaries; }
const float* tq4o_signs256(void) {
    pthread_once(&g_once, init_tables);
    return g_signs;
}

/* ---- 16-bit float conversions, round to nearest even ---- */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float tq4o_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-8f;
        return sign ? -v : v;
    }
    if (exp == 31) return u2f(sign | 0x7F800000u | (man << 13));
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t tq4o_f32_to_f16(float f) {
    uint32_t x = f2u(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((ax > 0x7F800000u) ? 0x200u : 0u));
    if (ax >= 0x477FF000u) /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    if (ax < 0x38800000u) { /* below the smallest normal half: subnormal or zero */
        if (ax < 0x33000000u) return sign; /* < 2^-25 rounds to zero (2^-25 itself ties to even = 0) */
        uint32_t e = ax >> 23;                       /* biased fp32 exponent, 102..112 */
        uint32_t m = (ax & 0x7FFFFFu) | 0x800000u;   /* 24-bit significand */
        uint32_t shift = 126u - e;                   /* 14..24: result = m >> shift in units of 2^-24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t e = (ax >> 23) - 112u;
    uint32_t m = ax & 0x7FFFFFu;
    uint32_t q = (e << 10) | (m >> 13);
    uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

float tq4o_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

uint16_t tq4o_f32_to_bf16(float f) {
    uint32_t x = f2u(f);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7FFFu + lsb;
    return (uint16_t)(x >> 16);
}

static inline float load16(const uint16_t* p, int dtype) {
    return dtype == TQ4O_DT_BF16 ? tq4o_bf16_to_f32(*p) : tq4o_f16_to_f32(*p);
}

/* ---- WHT-256: csrc/tq/tq4_kv_common.cuh:75-107.
 * Butterfly stages over index bits 0..7 in that order; the element with the bit clear
 * becomes a+b, the one with the bit set a-b (a = bit-clear element); the last stage
 * multiplies both results by 1/16. ---- */
void tq4o_wht256(float* x) {
    for (int h = 1; h < 256; h <<= 1) {
        for (int i = 0; i < 256; ++i) {
            if (i & h) continue;
            float a = x[i], b = x[i | h];
            if (h == 128) {
                x[i] = (a + b) * 0.0625f;
                x[i | h] = (a - b) * 0.0625f;
            } else {
                x[i] = a + b;
                x[i | h] = a - b;
            }
        }
    }
}

/* 32-lane xor-butterfly sum, csrc/tq/tq4_kv_common.cuh:54-60 */
static float warp_sum32(const float* lane_vals) {
    float cur[32], nxt[32];
    memcpy(cur, lane_vals, sizeof(cur));
    for (int off = 16; off > 0; off >>= 1) {
        for (int l = 0; l < 32; ++l) nxt[l] = cur[l] + cur[l ^ off];
        memcpy(cur, nxt, sizeof(cur));
    }
    return cur[0];
}

/* ---- TQ4 encode: op_kv_cache.cu:152-218.  Element i lives in lane i%32, register i/32. ---- */
void tq4o_encode_row(const float* x, uint8_t* dst) {
    const float* sg = tq4o_signs256();
    float y[256];
    for (int i = 0; i < 256; ++i) y[i] = x[i] * sg[i]; /* :163-167 */
    tq4o_wht256(y);                                    /* :168 */

    float tmp[32];
    float s_sq[2] = {0.0f, 0.0f};
    for (int j = 0; j < 4; ++j) { /* :170-175 */
        for (int l = 0; l < 32; ++l) tmp[l] = y[l + 32 * j] * y[l + 32 * j];
        s_sq[0] += warp_sum32(tmp);
        for (int l = 0; l < 32; ++l) tmp[l] = y[l + 32 * (j + 4)] * y[l + 32 * (j + 4)];
        s_sq[1] += warp_sum32(tmp);
    }
    float inv_norm[2];
    for (int h = 0; h < 2; ++h) { /* :176-179 */
        float rs = (float)(1.0 / sqrt((double)s_sq[h]));
        inv_norm[h] = (s_sq[h] > 1e-20f) ? (0.7071067811865475f * rs) : 0.0f;
    }

    uint8_t code[256];
    float vc_dot[2] = {0.0f, 0.0f}, c_sq[2] = {0.0f, 0.0f};
    for (int j = 0; j < 8; ++j) { /* :184-209 */
        float vc[32], cc[32];
        for (int l = 0; l < 32; ++l) {
            const int i = l + 32 * j;
            const float rv = y[i] * inv_norm[j >> 2];
            int q = 0;
            for (int t = 0; t < 15; ++t) q += (rv > kBoundaries[t]) ? 1 : 0;
            code[i] = (uint8_t)q;
            const float c = kCentroids[q];
            vc[l] = y[i] * c;
            cc[l] = c * c;
        }
        vc_dot[j >> 2] += warp_sum32(vc);
        c_sq[j >> 2] += warp_sum32(cc);
    }
    for (int h = 0; h < 2; ++h) { /* :193-198 pack, :210-215 scale */
        uint8_t* blk = dst + 66 * h;
        const float d = (c_sq[h] > 1e-10f) ? (vc_dot[h] / c_sq[h]) : 0.0f;
        const uint16_t dh = tq4o_f32_to_f16(d);
        blk[0] = (uint8_t)(dh & 0xFF);
        blk[1] = (uint8_t)(dh >> 8);
        for (int m = 0; m < 64; ++m)
            blk[2 + m] = (uint8_t)(code[128 * h + 2 * m] | (code[128 * h + 2 * m + 1] << 4));
    }
}

/* ---- TQ4 without the rotation (any transform but WHT-256 at head_dim 256): op_kv_cache.cu:219-264.
 * One 66-byte block per 128 elements; thread t of 128 holds element t.  Sums go through
 * block_reduce_sum_128 (tq/tq4_kv_common.cuh:109-124): a 32-lane butterfly per warp, then the same
 * butterfly over the four warp sums in lanes 0-3 of warp 0 (the other lanes hold 0). ---- */
static float block_sum128(const float* v) {
    float w[32];
    memset(w, 0, sizeof(w));
    for (int k = 0; k < 4; ++k) w[k] = warp_sum32(v + 32 * k);
    return warp_sum32(w);
}

void tq4o_encode_row_plain(const float* x, int head_dim, uint8_t* dst) {
    for (int sb = 0; sb < head_dim / 128; ++sb) {
        const float* xs = x + 128 * sb;
        uint8_t* blk = dst + 66 * sb;
        float t[128];
        for (int i = 0; i < 128; ++i) t[i] = xs[i] * xs[i];
        const float norm_x = sqrtf(block_sum128(t)); /* :231 */
        const float inv_norm = (norm_x > 1e-12f) ? (0.7071067811865475f / norm_x) : 0.0f;
        uint8_t code[128];
        float xc[128], cc[128];
        for (int i = 0; i < 128; ++i) { /* :235-245 */
            const float u = xs[i] * inv_norm;
            int q = 0;
            for (int b = 0; b < 15; ++b)
                if (u > kBoundaries[b]) q = b + 1;
            code[i] = (uint8_t)q;
            const float c = kCentroids[q];
            xc[i] = xs[i] * c;
            cc[i] = c * c;
        }
        const float xc_dot = block_sum128(xc); /* :246-248 */
        const float c_sq = block_sum128(cc);
        const float d = (c_sq > 1e-12f) ? (xc_dot / c_sq) : 0.0f;
        const uint16_t dh = tq4o_f32_to_f16(d);
        blk[0] = (uint8_t)(dh & 0xFF);
        blk[1] = (uint8_t)(dh >> 8);
        for (int m = 0; m < 64; ++m) /* :253-261: element 2m low nibble, 2m + 1 high */
            blk[2 + m] = (uint8_t)((code[2 * m] & 0x0F) | ((code[2 * m + 1] & 0x0F) << 4));
    }
}

/* ---- TQ4 dequant: op_kv_cache.cu:298-306 ---- */
void tq4o_dequant_row(const uint8_t* src, float* y) {
    for (int col = 0; col < 256; ++col) {
        const int sb = col >> 7, idx = col & 127;
        const uint8_t* blk = src + 66 * sb;
        const float d = tq4o_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        const uint8_t packed = blk[2 + (idx >> 1)];
        const uint8_t nib = (idx & 1) ? (uint8_t)(packed >> 4) : (uint8_t)(packed & 0x0F);
        y[col] = d * kCentroids[nib];
    }
}

/* ---- OCP FP8 E4M3: sign, 4 exponent bits (bias 7), 3 mantissa bits; no infinities, 0x7f/0xff
 * are NaN, largest finite 448 (0x7e) ---- */
float tq4o_e4m3_to_f32(uint8_t c) {
    const int e = (c >> 3) & 15, m = c & 7;
    float v;
    if (e == 15 && m == 7) return u2f(0x7fc00000u);
    if (e == 0) v = (float)m * 0.001953125f;                    /* m * 2^-9 */
    else v = u2f((uint32_t)(e - 7 + 127) << 23 | (uint32_t)m << 20);
    return (c & 0x80) ? -v : v;
}

uint8_t tq4o_f32_to_e4m3(float f) {
    const uint32_t u = f2u(f);
    const uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    const uint32_t ax = u & 0x7fffffffu;
    if (ax > 0x7f800000u) return (uint8_t)(sign | 0x7f);        /* NaN */
    const float a = u2f(ax);
    if (a >= 448.0f) return (uint8_t)(sign | 0x7e);             /* saturate (also +-inf) */
    if (a < 0.015625f) {                                        /* below 2^-6: multiples of 2^-9 */
        const float q = rintf(a * 512.0f);                      /* exact product, ties to even */
        return (uint8_t)(sign | (uint8_t)q);                    /* 8 == 0x08 == 2^-6 */
    }
    /* normal: keep 3 mantissa bits, round the other 20 to nearest even */
    uint32_t r = ax + 0x7ffffu + ((ax >> 20) & 1u);
    r >>= 20;                                                   /* exponent (8 bits) and 3 mantissa bits */
    const int code = (int)r - ((127 - 7) << 3);
    return (uint8_t)(sign | (uint8_t)(code > 0x7e ? 0x7e : code));
}

void tq4o_encode_row_fp8(const float* x, uint8_t* dst) {
    for (int h = 0; h < 2; ++h) {
        float amax = 0.0f;
        for (int c = 0; c < 128; ++c) amax = fmaxf(amax, fabsf(x[128 * h + c]));
        const float d = amax * (1.0f / 448.0f);
        const float inv_d = (d > 1e-30f) ? (1.0f / d) : 0.0f;
        memcpy(dst + 256 + 4 * h, &d, 4);
        for (int c = 0; c < 128; ++c) dst[128 * h + c] = tq4o_f32_to_e4m3(x[128 * h + c] * inv_d);
    }
}

void tq4o_dequant_row_fp8(const uint8_t* src, float* y) {
    for (int h = 0; h < 2; ++h) {
        float d;
        memcpy(&d, src + 256 + 4 * h, 4);
        for (int c = 0; c < 128; ++c) y[128 * h + c] = d * tq4o_e4m3_to_f32(src[128 * h + c]);
    }
}

void tq4o_encode_row_q8(const float* x, uint8_t* dst) {
    for (int sb = 0; sb < 4; ++sb) {
        float amax = 0.0f;
        for (int c = 0; c < 64; ++c) amax = fmaxf(amax, fabsf(x[64 * sb + c]));
        const float d = amax / 127.0f;
        const float inv_d = (d > 1e-12f) ? (1.0f / d) : 0.0f;
        memcpy(dst + 68 * sb, &d, 4);
        for (int c = 0; c < 64; ++c) {
            float q = roundf(x[64 * sb + c] * inv_d);           /* half away from zero */
            q = fminf(127.0f, fmaxf(-127.0f, q));
            dst[68 * sb + 4 + c] = (uint8_t)(int8_t)q;
        }
    }
}

void tq4o_dequant_row_q8(const uint8_t* src, float* y) {
    for (int sb = 0; sb < 4; ++sb) {
        float d;
        memcpy(&d, src + 68 * sb, 4);
        for (int c = 0; c < 64; ++c) y[64 * sb + c] = d * (float)(int8_t)src[68 * sb + 4 + c];
    }
}

void tq4o_unrotate_row(const float* y, float* x) {
    const float* sg = tq4o_signs256();
    float t[256];
    memcpy(t, y, sizeof(t));
    tq4o_wht256(t);
    for (int i = 0; i < 256; ++i) x[i] = t[i] * sg[i];
}

/* ---- request lookup shared by write and attention: op_kv_cache.cu:385-398 ---- */
static int find_req(const tq4o_batch* B, int tok, int* q_start, int* q_end) {
    for (int r = 0; r < B->num_reqs; ++r) {
        const int lo = B->query_start_loc[r], hi = B->query_start_loc[r + 1];
        if (tok >= lo && tok < hi) {
            *q_start = lo;
            *q_end = hi;
            return r;
        }
    }
    return -1;
}

static int write_row(uint8_t* dst, int format, int transform, const uint16_t* src, int head_dim,
                     int in_dtype) {
    if (format == TQ4O_FMT_FP16 || format == TQ4O_FMT_BF16) { /* op_kv_cache.cu:18-31 */
        uint16_t* d16 = (uint16_t*)dst;
        for (int c = 0; c < head_dim; ++c) {
            const int same = (format == TQ4O_FMT_FP16 && in_dtype == TQ4O_DT_F16) ||
                             (format == TQ4O_FMT_BF16 && in_dtype == TQ4O_DT_BF16);
            if (same) {
                d16[c] = src[c];
            } else {
                const float f = load16(src + c, in_dtype);
                d16[c] = format == TQ4O_FMT_BF16 ? tq4o_f32_to_bf16(f) : tq4o_f32_to_f16(f);
            }
        }
        return 0;
    }
    if (format == TQ4O_FMT_TQ4 && transform == TQ4O_XF_WHT256 && head_dim == 256) {
        float x[256];
        for (int c = 0; c < 256; ++c) x[c] = load16(src + c, in_dtype);
        tq4o_encode_row(x, dst);
        return 0;
    }
    if (format == TQ4O_FMT_TQ4 && head_dim > 0 && head_dim <= 256 && (head_dim % 128) == 0) { /* op_kv_cache.cu:219 */
        float x[256];
        for (int c = 0; c < head_dim; ++c) x[c] = load16(src + c, in_dtype);
        tq4o_encode_row_plain(x, head_dim, dst);
        return 0;
    }
    if ((format == TQ4O_FMT_Q8_0 || format == TQ4O_FMT_FP8) && head_dim == 256) {
        float x[256];
        for (int c = 0; c < 256; ++c) x[c] = load16(src + c, in_dtype);
        if (transform == TQ4O_XF_WHT256) { /* op_kv_cache.cu:39-45,68-74: sign diagonal, then WHT */
            const float* sg = tq4o_signs256();
            for (int c = 0; c < 256; ++c) x[c] *= sg[c];
            tq4o_wht256(x);
        }
        if (format == TQ4O_FMT_FP8) tq4o_encode_row_fp8(x, dst);
        else tq4o_encode_row_q8(x, dst);
        return 0;
    }
    return -1;
}

/* ---- QK RMSNorm + RoPE over packed bf16 rows, optionally with the K/V rows written into the
 * paged cache: qk_norm_rope_bf16_warp, ops/op_dflash2.cu:338-418 ----
 * Declared numerics: fp32 in source order without contraction; the sum of squares in the order
 * of reduce_sum256_exact_warp (op_dflash2.cu:30-39: per lane ((v0+v128)+(v64+v192)) +
 * ((v32+v160)+(v96+v224)), then the 32-lane xor butterfly 16,8,4,2,1); rsqrt(x) :=
 * fl32(1/sqrt(x) in fp64); bf16 round-to-nearest-even. */
static float sum256_warp_order(const float* sq) { /* sq[c], c = lane + 32 k */
    float lane_sum[32];
    for (int lane = 0; lane < 32; ++lane) {
        const float v0 = sq[lane], v32 = sq[lane + 32], v64 = sq[lane + 64], v96 = sq[lane + 96];
        const float v128 = sq[lane + 128], v160 = sq[lane + 160], v192 = sq[lane + 192], v224 = sq[lane + 224];
        lane_sum[lane] = ((v0 + v128) + (v64 + v192)) + ((v32 + v160) + (v96 + v224));
    }
    for (int mask = 16; mask >= 1; mask >>= 1) {
        float next[32];
        for (int lane = 0; lane < 32; ++lane) next[lane] = lane_sum[lane] + lane_sum[lane ^ mask];
        memcpy(lane_sum, next, sizeof(next));
    }
    return lane_sum[0];
}

int tq4o_qk_norm_rope_bf16(uint16_t* qkv, uint16_t* q_out, const int32_t* positions, const uint16_t* qw,
                           const uint16_t* kw, const void* table, int table_is_f32, int rows, int q_heads,
                           int kv_heads, int dim, int table_rows, float eps, const tq4o_layout* L,
                           const int32_t* write_slot_mapping) {
    if (!qkv || !positions || !qw || !kw || !table || rows < 0 || q_heads < 0 || kv_heads <= 0 || dim <= 0 ||
        dim > 256 || (dim & 1) || table_rows <= 0 || !(eps > 0.0f)) {
        return -1;
    }
    const int half = dim / 2;
    const size_t row_elems = (size_t)(q_heads + 2 * kv_heads) * dim;
    for (int row = 0; row < rows; ++row) {
        const int pos = positions[row];
        if (pos < 0 || pos >= table_rows) continue; /* :356 */
        for (int head = 0; head < q_heads + kv_heads; ++head) {
            uint16_t* src = qkv + (size_t)row * row_elems + (size_t)head * dim;
            const uint16_t* w = head < q_heads ? qw : kw;
            float sq[256];
            for (int c = 0; c < 256; ++c) {
                const float x = c < dim ? tq4o_bf16_to_f32(src[c]) : 0.0f;
                sq[c] = x * x;
            }
            const float sum_sq = sum256_warp_order(sq);
            const float mean = sum_sq / (float)dim + eps;
            const float inv = (float)(1.0 / sqrt((double)mean));
            uint16_t out[256];
            for (int c = 0; c < half; ++c) {
                const float a = tq4o_bf16_to_f32(tq4o_f32_to_bf16(tq4o_bf16_to_f32(src[c]) * inv * tq4o_bf16_to_f32(w[c])));
                const float b = tq4o_bf16_to_f32(
                    tq4o_f32_to_bf16(tq4o_bf16_to_f32(src[half + c]) * inv * tq4o_bf16_to_f32(w[half + c])));
                float cosine, sine;
                if (table_is_f32) {
                    const float* t = (const float*)table + (size_t)pos * dim;
                    cosine = t[c];
                    sine = t[half + c];
                } else {
                    const uint16_t* t = (const uint16_t*)table + (size_t)pos * dim;
                    cosine = tq4o_bf16_to_f32(t[c]);
                    sine = tq4o_bf16_to_f32(t[half + c]);
                }
                const float ac = a * cosine, bs = b * sine, bc = b * cosine, as = a * sine;
                out[c] = tq4o_f32_to_bf16(ac - bs);
                out[half + c] = tq4o_f32_to_bf16(bc + as);
            }
            uint16_t* dst = (q_out != NULL && head < q_heads) ? q_out + ((size_t)row * q_heads + head) * dim : src;
            if (write_slot_mapping != NULL && L != NULL && head >= q_heads && write_slot_mapping[row] >= 0) {
                /* rotated K and the untouched V go to the cache, the packed row keeps its K (:387-403) */
                const int slot = write_slot_mapping[row];
                const int kv_head = head - q_heads;
                const int page = slot / L->block_size, off = slot % L->block_size;
                uint8_t* k_dst = L->k_base + (size_t)page * L->k_page_stride + (size_t)kv_head * L->k_head_stride +
                                 (size_t)off * L->k_token_stride;
                uint8_t* v_dst = L->v_base + (size_t)page * L->v_page_stride + (size_t)kv_head * L->v_head_stride +
                                 (size_t)off * L->v_token_stride;
                const uint16_t* v_src = src + (size_t)kv_heads * dim;
                if (write_row(k_dst, L->k_format, L->k_transform, out, dim, TQ4O_DT_BF16) != 0) return -2;
                if (write_row(v_dst, L->v_format, L->v_transform, v_src, dim, TQ4O_DT_BF16) != 0) return -2;
            } else {
                memcpy(dst, out, (size_t)dim * sizeof(uint16_t));
            }
        }
    }
    return 0;
}

/* ---- output gate: apply_attn_output_gate_f16_kernel, ops/op_norms_rope_act.cu:742-759 ----
 * out = fp16(a * (1 / (1 + expf(-g)))) in fp32, source order. */
int tq4o_apply_attn_output_gate_f16(const uint16_t* attn_out, const uint16_t* gate, uint16_t* out,
                                    const uint8_t* valid_token_mask, int num_tokens, int total_dim) {
    if (!attn_out || !gate || !out) return -1;
    for (int tok = 0; tok < num_tokens; ++tok) {
        if (valid_token_mask != NULL && valid_token_mask[tok] == 0) continue;
        for (int col = 0; col < total_dim; ++col) {
            const size_t idx = (size_t)tok * total_dim + col;
            const float a = tq4o_f16_to_f32(attn_out[idx]);
            const float g = tq4o_f16_to_f32(gate[idx]);
            const float sig = 1.0f / (1.0f + expf(-g));
            out[idx] = tq4o_f32_to_f16(a * sig);
        }
    }
    return 0;
}

/* ---- paged append: op_kv_cache.cu:325-368 ---- */
int tq4o_kv_cache_write(const tq4o_layout* L, const tq4o_batch* B, const uint16_t* k_in,
                        const uint16_t* v_in, int k_row_stride, int v_row_stride, int in_dtype) {
    for (int tok = 0; tok < B->total_tokens; ++tok) {
        if (B->valid_token_mask && B->valid_token_mask[tok] == 0) continue;
        if (B->valid_req_mask && B->query_start_loc && B->num_reqs > 0) {
            int a, b;
            const int r = find_req(B, tok, &a, &b);
            if (r < 0 || B->valid_req_mask[r] == 0) continue;
        }
        const int32_t slot = B->write_slot_mapping[tok];
        if (slot < 0) continue;
        const int page = slot / L->block_size, off = slot % L->block_size;
        for (int h = 0; h < L->local_kv_heads; ++h) {
            uint8_t* kd = L->k_base + (size_t)page * L->k_page_stride + (size_t)h * L->k_head_stride +
                          (size_t)off * L->k_token_stride;
            uint8_t* vd = L->v_base + (size_t)page * L->v_page_stride + (size_t)h * L->v_head_stride +
                          (size_t)off * L->v_token_stride;
            const uint16_t* ks = k_in + (size_t)tok * k_row_stride + (size_t)h * L->head_dim;
            const uint16_t* vs = v_in + (size_t)tok * v_row_stride + (size_t)h * L->head_dim;
            if (write_row(kd, L->k_format, L->k_transform, ks, L->head_dim, in_dtype)) return -1;
            if (write_row(vd, L->v_format, L->v_transform, vs, L->head_dim, in_dtype)) return -1;
        }
    }
    return 0;
}

/* read one stored row as fp32 (op_kv_cache.cu:288-306) */
static void read_row(const uint8_t* row, int format, int head_dim, float* y) {
    if (format == TQ4O_FMT_TQ4) {
        tq4o_dequant_row(row, y);
        return;
    }
    if (format == TQ4O_FMT_FP8) { /* op_paged_attn.cu:73-103 */
        tq4o_dequant_row_fp8(row, y);
        return;
    }
    if (format == TQ4O_FMT_Q8_0) { /* op_paged_attn.cu:59-71 */
        tq4o_dequant_row_q8(row, y);
        return;
    }
    const uint16_t* p = (const uint16_t*)row;
    for (int c = 0; c < head_dim; ++c)
        y[c] = format == TQ4O_FMT_BF16 ? tq4o_bf16_to_f32(p[c]) : tq4o_f16_to_f32(p[c]);
}

/* Visible key range of one query token: op_kv_cache.cu:406-424.  Returns 0 when the row
 * is skipped (masked / no owning request). */
static int row_range(const tq4o_batch* B, int tok, int* req, int* min_kv, int* max_kv) {
    if (B->valid_token_mask && B->valid_token_mask[tok] == 0) return 0;
    int q_start = 0, q_end = 0;
    const int r = find_req(B, tok, &q_start, &q_end);
    if (r < 0) return 0;
    if (B->valid_req_mask && B->valid_req_mask[r] == 0) return 0;
    const int q_off = tok - q_start;
    const int ctx_before = B->context_lens_before ? B->context_lens_before[r]
                                                  : (B->seq_lens_after[r] - (q_end - q_start));
    const int seq_after = B->seq_lens_after[r];
    int mx = (B->mask_mode == 1) ? (seq_after - 1) : (ctx_before + q_off);
    if (mx >= seq_after) mx = seq_after - 1;
    int mn = 0;
    if (B->sliding_window > 0) {
        const int ws = ctx_before + q_off - B->sliding_window + 1;
        if (ws > mn) mn = ws;
    }
    *req = r;
    *min_kv = mn;
    *max_kv = mx;
    return 1;
}

static inline const uint8_t* kv_row_ptr(const uint8_t* base, uint64_t ps, uint64_t hs, uint64_t ts,
                                        const tq4o_batch* B, int req, int kv_head, int pos, int bs) {
    const int32_t page = B->block_tables[(size_t)req * B->max_blocks_per_req + pos / bs];
    return base + (size_t)page * ps + (size_t)kv_head * hs + (size_t)(pos % bs) * ts;
}

/* Partial softmax state of `g` query heads of one kv head over keys [lo, hi]:
 * acc[g][head_dim] un-normalised, m[g] running max, l[g] sum of exp(score - m).
 * fp64 throughout (declared oracle numerics). */
static void attend_range(const tq4o_layout* L, const tq4o_batch* B, int req, int kv_head,
                         const float* qrows /* [g][hd], already rotated */, int g, int lo, int hi,
                         double* acc, double* m, double* l) {
    const int hd = L->head_dim;
    const int n = hi - lo + 1;
    float kv[256];
    double* sc = (double*)malloc((size_t)g * (size_t)(n > 0 ? n : 1) * sizeof(double));
    for (int a = 0; a < g; ++a) {
        m[a] = -INFINITY;
        l[a] = 0.0;
        for (int c = 0; c < hd; ++c) acc[(size_t)a * hd + c] = 0.0;
    }
    for (int pos = lo; pos <= hi; ++pos) {
        read_row(kv_row_ptr(L->k_base, L->k_page_stride, L->k_head_stride, L->k_token_stride, B, req,
                            kv_head, pos, L->block_size),
                 L->k_format, hd, kv);
        for (int a = 0; a < g; ++a) {
            const float* q = qrows + (size_t)a * hd;
            double dot = 0.0;
            for (int c = 0; c < hd; ++c) dot += (double)q[c] * (double)kv[c];
            const double s = dot * (double)B->sm_scale;
            sc[(size_t)a * n + (pos - lo)] = s;
            if (s > m[a]) m[a] = s;
        }
    }
    for (int a = 0; a < g; ++a)
        for (int i = 0; i < n; ++i) {
            const double p = exp(sc[(size_t)a * n + i] - m[a]);
            sc[(size_t)a * n + i] = p;
            l[a] += p;
        }
    for (int pos = lo; pos <= hi; ++pos) {
        read_row(kv_row_ptr(L->v_base, L->v_page_stride, L->v_head_stride, L->v_token_stride, B, req,
                            kv_head, pos, L->block_size),
                 L->v_format, hd, kv);
        for (int a = 0; a < g; ++a) {
            const double p = sc[(size_t)a * n + (pos - lo)];
            double* ac = acc + (size_t)a * hd;
            for (int c = 0; c < hd; ++c) ac[c] += p * (double)kv[c];
        }
    }
    free(sc);
}

/* load + optionally rotate the query rows of one (token, kv head): op_kv_cache.cu:435-451 */
static void load_q(const tq4o_layout* L, const uint16_t* q, int q_dtype, int tok, int num_q_heads,
                   int q_head0, int g, float* qrows) {
    const int hd = L->head_dim;
    const float* sg = tq4o_signs256();
    for (int a = 0; a < g; ++a) {
        const uint16_t* src = q + ((size_t)tok * num_q_heads + q_head0 + a) * hd;
        float* dst = qrows + (size_t)a * hd;
        for (int c = 0; c < hd; ++c) dst[c] = load16(src + c, q_dtype);
        if (hd == 256 && L->k_transform == TQ4O_XF_WHT256) {
            for (int c = 0; c < 256; ++c) dst[c] *= sg[c];
            tq4o_wht256(dst);
        }
    }
}

/* finalise one row: normalise, un-rotate (op_kv_cache.cu:762-790) */
static void store_out(const tq4o_layout* L, const double* acc, double l, float* out_row) {
    const int hd = L->head_dim;
    float t[256];
    const double inv = l > 0.0 ? 1.0 / l : 0.0;
    for (int c = 0; c < hd; ++c) t[c] = (float)(acc[c] * inv);
    if (hd == 256 && L->v_transform == TQ4O_XF_WHT256)
        tq4o_unrotate_row(t, out_row);
    else
        memcpy(out_row, t, (size_t)hd * sizeof(float));
}

/* merge chunk states in chunk order (fp64) */
static void merge_state(double* acc, double* m, double* l, const double* acc2, double m2, double l2,
                        int hd) {
    if (l2 <= 0.0) return;
    if (*l <= 0.0) {
        memcpy(acc, acc2, (size_t)hd * sizeof(double));
        *m = m2;
        *l = l2;
        return;
    }
    const double mt = *m > m2 ? *m : m2;
    const double w1 = exp(*m - mt), w2 = exp(m2 - mt);
    for (int c = 0; c < hd; ++c) acc[c] = acc[c] * w1 + acc2[c] * w2;
    *l = *l * w1 + l2 * w2;
    *m = mt;
}

#define ORACLE_CHUNK 2048 /* keys per work item; fixed so results do not depend on threads */

typedef struct {
    const tq4o_layout* L;
    const tq4o_batch* B;
    const uint16_t* q;
    int q_dtype, num_q_heads, g;
    /* work items */
    int n_items;
    int* it_tok;
    int* it_kvh;
    int* it_req;
    int* it_lo;
    int* it_hi;
    double* it_acc; /* [n_items][g][hd] */
    double* it_m;   /* [n_items][g] */
    double* it_l;
    int next;
    pthread_mutex_t mu;
} attn_job;

static void* attn_worker(void* arg) {
    attn_job* J = (attn_job*)arg;
    const int hd = J->L->head_dim;
    float* qrows = (float*)malloc((size_t)J->g * hd * sizeof(float));
    for (;;) {
        pthread_mutex_lock(&J->mu);
        const int it = J->next++;
        pthread_mutex_unlock(&J->mu);
        if (it >= J->n_items) break;
        load_q(J->L, J->q, J->q_dtype, J->it_tok[it], J->num_q_heads, J->it_kvh[it] * J->g, J->g, qrows);
        attend_range(J->L, J->B, J->it_req[it], J->it_kvh[it], qrows, J->g, J->it_lo[it], J->it_hi[it],
                     J->it_acc + (size_t)it * J->g * hd, J->it_m + (size_t)it * J->g,
                     J->it_l + (size_t)it * J->g);
    }
    free(qrows);
    return NULL;
}

int tq4o_paged_attention(const tq4o_layout* L, const tq4o_batch* B, const uint16_t* q, int q_dtype,
                         float* out, int num_q_heads, int n_threads) {
    if (L->local_kv_heads <= 0 || num_q_heads % L->local_kv_heads) return -1;
    if (L->head_dim > 256) return -1;
    const int hd = L->head_dim, g = num_q_heads / L->local_kv_heads;
    attn_job J;
    memset(&J, 0, sizeof(J));
    J.L = L; J.B = B; J.q = q; J.q_dtype = q_dtype; J.num_q_heads = num_q_heads; J.g = g;
    pthread_mutex_init(&J.mu, NULL);
    /* enumerate items */
    size_t cap = 0;
    for (int pass = 0; pass < 2; ++pass) {
        int n = 0;
        for (int tok = 0; tok < B->total_tokens; ++tok) {
            int req, lo, hi;
            if (!row_range(B, tok, &req, &lo, &hi)) continue;
            for (int h = 0; h < L->local_kv_heads; ++h) {
                int c0 = lo;
                do {
                    int c1 = c0 + ORACLE_CHUNK - 1;
                    if (c1 > hi) c1 = hi;
                    if (pass) {
                        J.it_tok[n] = tok; J.it_kvh[n] = h; J.it_req[n] = req;
                        J.it_lo[n] = c0; J.it_hi[n] = c1;
                    }
                    ++n;
                    c0 = c1 + 1;
                } while (c0 <= hi);
            }
        }
        if (!pass) {
            cap = (size_t)(n > 0 ? n : 1);
            J.n_items = n;
            J.it_tok = (int*)malloc(cap * sizeof(int));
            J.it_kvh = (int*)malloc(cap * sizeof(int));
            J.it_req = (int*)malloc(cap * sizeof(int));
            J.it_lo = (int*)malloc(cap * sizeof(int));
            J.it_hi = (int*)malloc(cap * sizeof(int));
            J.it_acc = (double*)malloc(cap * g * hd * sizeof(double));
            J.it_m = (double*)malloc(cap * g * sizeof(double));
            J.it_l = (double*)malloc(cap * g * sizeof(double));
        }
    }
    if (n_threads < 1) n_threads = 1;
    if (n_threads > 256) n_threads = 256;
    if (n_threads == 1) {
        attn_worker(&J);
    } else {
        pthread_t th[256];
        for (int t = 0; t < n_threads; ++t) pthread_create(&th[t], NULL, attn_worker, &J);
        for (int t = 0; t < n_threads; ++t) pthread_join(th[t], NULL);
    }
    /* merge the chunk states of every (token, kv head) in chunk order and store */
    double* acc = (double*)malloc((size_t)hd * sizeof(double));
    int it = 0;
    while (it < J.n_items) {
        const int tok = J.it_tok[it], h = J.it_kvh[it];
        int end = it;
        while (end < J.n_items && J.it_tok[end] == tok && J.it_kvh[end] == h) ++end;
        for (int a = 0; a < g; ++a) {
            double m = -INFINITY, l = 0.0;
            for (int c = 0; c < hd; ++c) acc[c] = 0.0;
            for (int k = it; k < end; ++k)
                merge_state(acc, &m, &l, J.it_acc + ((size_t)k * g + a) * hd, J.it_m[(size_t)k * g + a],
                            J.it_l[(size_t)k * g + a], hd);
            store_out(L, acc, l, out + ((size_t)tok * num_q_heads + (size_t)h * g + a) * hd);
        }
        it = end;
    }
    free(acc);
    free(J.it_tok); free(J.it_kvh); free(J.it_req); free(J.it_lo); free(J.it_hi);
    free(J.it_acc); free(J.it_m); free(J.it_l);
    pthread_mutex_destroy(&J.mu);
    return 0;
}

/* ---- split-KV: op_paged_attn.cu:323-341 (page partition), :544-558 (fp32 partials),
 * :1132-1218 (merge in fp32: m_tot, w = exp(m_s - m_tot), sum acc*w / sum l*w) ---- */
int tq4o_paged_attention_split(const tq4o_layout* L, const tq4o_batch* B, const uint16_t* q,
                               int q_dtype, float* out, int num_q_heads, int n_splits) {
    if (L->local_kv_heads <= 0 || num_q_heads % L->local_kv_heads) return -1;
    if (n_splits < 1) n_splits = 1;
    const int hd = L->head_dim, g = num_q_heads / L->local_kv_heads, bs = L->block_size;
    float* qrows = (float*)malloc((size_t)g * hd * sizeof(float));
    double* acc = (double*)malloc((size_t)g * hd * sizeof(double));
    double* m = (double*)malloc((size_t)g * sizeof(double));
    double* l = (double*)malloc((size_t)g * sizeof(double));
    float* p_acc = (float*)malloc((size_t)n_splits * g * hd * sizeof(float));
    float* p_m = (float*)malloc((size_t)n_splits * g * sizeof(float));
    float* p_l = (float*)malloc((size_t)n_splits * g * sizeof(float));
    for (int tok = 0; tok < B->total_tokens; ++tok) {
        int req, lo, hi;
        if (!row_range(B, tok, &req, &lo, &hi)) continue;
        const int first_page = lo / bs;
        const int total_pages = hi >= lo ? hi / bs - first_page + 1 : 0;
        const int pps = (total_pages + n_splits - 1) / n_splits > 0 ? (total_pages + n_splits - 1) / n_splits : 1;
        for (int h = 0; h < L->local_kv_heads; ++h) {
            load_q(L, q, q_dtype, tok, num_q_heads, h * g, g, qrows);
            int active = 0;
            for (int s = 0; s < n_splits; ++s) {
                const int p0 = first_page + s * pps, p1 = p0 + pps;
                int klo = p0 * bs, khi = p1 * bs - 1;
                if (klo < lo) klo = lo;
                if (khi > hi) khi = hi;
                if (klo > khi) break;
                attend_range(L, B, req, h, qrows, g, klo, khi, acc, m, l);
                for (int a = 0; a < g; ++a) {
                    for (int c = 0; c < hd; ++c)
                        p_acc[((size_t)s * g + a) * hd + c] = (float)acc[(size_t)a * hd + c];
                    p_m[(size_t)s * g + a] = (float)m[a];
                    p_l[(size_t)s * g + a] = (float)l[a];
                }
                ++active;
            }
            for (int a = 0; a < g; ++a) {
                float m_tot = -INFINITY;
                for (int s = 0; s < active; ++s)
                    if (p_l[(size_t)s * g + a] > 0.0f && p_m[(size_t)s * g + a] > m_tot)
                        m_tot = p_m[(size_t)s * g + a];
                float l_tot = 0.0f;
                float o[256];
                for (int c = 0; c < hd; ++c) o[c] = 0.0f;
                for (int s = 0; s < active; ++s) {
                    const float ls = p_l[(size_t)s * g + a];
                    if (!(ls > 0.0f)) continue;
                    const float w = expf(p_m[(size_t)s * g + a] - m_tot);
                    l_tot += ls * w;
                    for (int c = 0; c < hd; ++c) o[c] += p_acc[((size_t)s * g + a) * hd + c] * w;
                }
                const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
                for (int c = 0; c < hd; ++c) o[c] *= inv;
                float* dst = out + ((size_t)tok * num_q_heads + (size_t)h * g + a) * hd;
                if (hd == 256 && L->v_transform == TQ4O_XF_WHT256)
                    tq4o_unrotate_row(o, dst);
                else
                    memcpy(dst, o, (size_t)hd * sizeof(float));
            }
        }
    }
    free(qrows); free(acc); free(m); free(l); free(p_acc); free(p_m); free(p_l);
    return 0;
}

/* ---- ops/op_norms_rope_act.cu:524-689,1201-1246: fused_qk_rmsnorm_rope_gate_f16_kernel, the
 * producer of the target model's full-attention layers.  Per (token, head): Gemma RMSNorm
 * (x * rsqrt(mean x^2 + eps) * (1 + w), rounded to fp16), rotation of the pairs (i, i + rotary/2)
 * of the first `rotary_dim` elements by the angle pos_plane(i) * theta^(-2i/rotary_dim) with
 * fp16-rounded sine and cosine (:649-657), the other elements copied; the gate half of every Q
 * head is copied to gate_out (:562-585).  Position planes (:639-645): pair i takes plane 1 if
 * i % 3 == 1 and i < 3 s1, plane 2 if i % 3 == 2 and i < 3 s2, else plane 0.
 * Declared numerics: fp32 in source order, no contraction; the sum of squares as the kernel's
 * 128-thread block forms it for head sizes that are multiples of 8 (thread t adds the eight
 * squares of elements 8t .. 8t+7 in order, 32-lane xor butterflies, the warps' sums added by a
 * butterfly over warp 0: :586-604, :28-46); rsqrt, powf, sinf, cosf := the double-precision
 * result rounded once to fp32. ---- */
int tq4o_fused_qk_rmsnorm_rope_gate_f16(const uint16_t* q_gate_in, const uint16_t* k_in, const uint16_t* q_norm_w,
                                        const uint16_t* k_norm_w, const int32_t* positions,
                                        const uint8_t* valid_token_mask, uint16_t* q_out, uint16_t* k_out,
                                        uint16_t* gate_out, int num_tokens, int pos_plane_stride, int num_q_heads,
                                        int num_kv_heads, int head_dim, int rotary_dim, int mrope_s0, int mrope_s1,
                                        int mrope_s2, int q_gate_row_stride, int k_row_stride, float rope_theta,
                                        float rms_eps) {
    (void)mrope_s0;
    if (!q_gate_in || !k_in || !q_norm_w || !k_norm_w || !positions || !q_out || !k_out || !gate_out) return -1;
    if (num_tokens <= 0) return 0;
    if (q_gate_row_stride < num_q_heads * 2 * head_dim || k_row_stride < num_kv_heads * head_dim) return -1;
    if (head_dim <= 0 || (head_dim & 7) || head_dim > 1024 || rotary_dim < 0 || (rotary_dim & 1) ||
        rotary_dim > head_dim)
        return -2; /* the restated summation order is the vectorised one */
    const int half_rot = rotary_dim / 2;
    float* normed = (float*)malloc((size_t)head_dim * sizeof(float));
    for (int tok = 0; tok < num_tokens; ++tok) {
        if (valid_token_mask && valid_token_mask[tok] == 0) continue;
        for (int head_idx = 0; head_idx < num_q_heads + num_kv_heads; ++head_idx) {
            const int is_q = head_idx < num_q_heads;
            const int local = is_q ? head_idx : head_idx - num_q_heads;
            const uint16_t* src;
            const uint16_t* w;
            uint16_t* dst;
            if (is_q) {
                const uint16_t* base = q_gate_in + (size_t)tok * q_gate_row_stride + (size_t)local * 2 * head_dim;
                src = base;
                memcpy(gate_out + ((size_t)tok * num_q_heads + local) * head_dim, base + head_dim,
                       (size_t)head_dim * sizeof(uint16_t));
                w = q_norm_w;
                dst = q_out + ((size_t)tok * num_q_heads + local) * head_dim;
            } else {
                src = k_in + (size_t)tok * k_row_stride + (size_t)local * head_dim;
                w = k_norm_w;
                dst = k_out + ((size_t)tok * num_kv_heads + local) * head_dim;
            }
            /* sum of squares: 128 threads, thread t owns vector t (8 elements) when t < head_dim / 8 */
            float part[128];
            for (int t = 0; t < 128; ++t) {
                float acc = 0.0f;
                if (8 * t < head_dim) {
                    for (int j = 0; j < 8; ++j) {
                        const float v = tq4o_f16_to_f32(src[8 * t + j]);
                        const float sq = v * v;
                        acc = acc + sq;
                    }
                }
                part[t] = acc;
            }
            float warp_sums[32];
            for (int k = 0; k < 32; ++k) warp_sums[k] = 0.0f;
            for (int wv = 0; wv < 4; ++wv) warp_sums[wv] = warp_sum32(part + 32 * wv);
            const float sum_sq = warp_sum32(warp_sums);
            const float mean = sum_sq / (float)head_dim + rms_eps;
            const float inv_rms = (float)(1.0 / sqrt((double)mean));
            for (int i = 0; i < head_dim; ++i) {
                const float v = tq4o_f16_to_f32(src[i]) * inv_rms;
                const float wt = 1.0f + tq4o_f16_to_f32(w[i]);
                normed[i] = tq4o_f16_to_f32(tq4o_f32_to_f16(v * wt));
            }
            for (int i = 0; i < half_rot; ++i) {
                int plane = 0;
                if ((i % 3) == 1 && i < mrope_s1 * 3) plane = 1;
                else if ((i % 3) == 2 && i < mrope_s2 * 3) plane = 2;
                const float pos = (float)positions[(size_t)plane * pos_plane_stride + tok];
                const float expo = (float)(2 * i) / (float)rotary_dim;
                const float pw = (float)pow((double)rope_theta, (double)expo);
                const float inv_freq = 1.0f / pw;
                const float angle = pos * inv_freq;
                const float sin_a = tq4o_f16_to_f32(tq4o_f32_to_f16((float)sin((double)angle)));
                const float cos_a = tq4o_f16_to_f32(tq4o_f32_to_f16((float)cos((double)angle)));
                const float x1 = normed[i], x2 = normed[i + half_rot];
                const float a = x1 * cos_a, b = x2 * sin_a, c = x2 * cos_a, d = x1 * sin_a;
                dst[i] = tq4o_f32_to_f16(a - b);
                dst[i + half_rot] = tq4o_f32_to_f16(c + d);
            }
            for (int i = rotary_dim; i < head_dim; ++i) dst[i] = tq4o_f32_to_f16(normed[i]);
        }
    }
    free(normed);
    return 0;
}

/* ---- deterministic synthetic inputs ---- */
uint64_t tq4o_splitmix64(uint64_t* s) {
    uint64_t z = (*s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static void normal_pair(uint64_t* s, double* z0, double* z1) {
    const double u1 = ((double)(tq4o_splitmix64(s) >> 11) + 1.0) * 0x1.0p-53; /* (0,1] */
    const double u2 = (double)(tq4o_splitmix64(s) >> 11) * 0x1.0p-53;         /* [0,1) */
    const double r = sqrt(-2.0 * log(u1));
    const double a = 6.283185307179586476925 * u2;
    *z0 = r * cos(a);
    *z1 = r * sin(a);
}

static inline uint16_t store16(float f, int dtype) {
    return dtype == TQ4O_DT_BF16 ? tq4o_f32_to_bf16(f) : tq4o_f32_to_f16(f);
}

void tq4o_fill_normal(uint16_t* dst, size_t n, uint64_t seed, int dtype) {
    uint64_t s = seed;
    for (size_t i = 0; i < n; i += 2) {
        double a, b;
        normal_pair(&s, &a, &b);
        dst[i] = store16((float)a, dtype);
        if (i + 1 < n) dst[i + 1] = store16((float)b, dtype);
    }
}

void tq4o_permutation(int32_t* dst, int n, uint64_t seed) {
    uint64_t s = seed ^ 0xA5A5A5A5DEADBEEFull;
    for (int i = 0; i < n; ++i) dst[i] = i;
    for (int i = n - 1; i > 0; --i) { /* Fisher-Yates */
        const int j = (int)(tq4o_splitmix64(&s) % (uint64_t)(i + 1));
        const int32_t t = dst[i];
        dst[i] = dst[j];
        dst[j] = t;
    }
}

void tq4o_fill_kv_rows(uint16_t* dst, size_t rows, int kv_heads, int head_dim, uint64_t seed,
                       int dtype, int n_outliers) {
    /* outlier channels per kv head: first n_outliers of a seeded permutation of 0..head_dim-1 */
    float* gain = (float*)malloc((size_t)kv_heads * head_dim * sizeof(float));
    int32_t* perm = (int32_t*)malloc((size_t)head_dim * sizeof(int32_t));
    for (int h = 0; h < kv_heads; ++h) {
        for (int c = 0; c < head_dim; ++c) gain[(size_t)h * head_dim + c] = 1.0f;
        tq4o_permutation(perm, head_dim, seed * 1315423911ull + (uint64_t)h + 17u);
        for (int k = 0; k < n_outliers && k < head_dim; ++k) gain[(size_t)h * head_dim + perm[k]] = 20.0f;
    }
    uint64_t s = seed;
    const size_t per_row = (size_t)kv_heads * head_dim;
    const size_t n = rows * per_row;
    for (size_t i = 0; i < n; i += 2) {
        double a, b;
        normal_pair(&s, &a, &b);
        dst[i] = store16((float)a * gain[i % per_row], dtype);
        if (i + 1 < n) dst[i + 1] = store16((float)b * gain[(i + 1) % per_row], dtype);
    }
    free(gain);
    free(perm);
}

/* ---- QSA sparse paged attention: op_qsa.cu:716-1073 (grouped kernel), :1075-1158 (split merge),
 * :1161-1445 (generic kernel), hadamard_inline.cuh:11-50 (per-64 output transform) ----
 * Every query token attends over its own list of selected 4-token groups.  Group j of token t is
 * rows (phys % gpp) * 4 .. + 3 of physical page phys / gpp with gpp = block_size / 4
 * (phys = selected_phys_blocks[t * select_k + j]); its keys sit at sequence positions
 * 4 * selected_logical_blocks[..] + 0..3.  A group with phys < 0 and a key behind token_seq_pos[t]
 * are skipped.  The normalised sum is rotated back, multiplied by sigmoid(gate) and rounded to
 * fp16; the hadamard form then transforms every 64-element block of the rounded row.  Masked
 * tokens and tokens without a visible key give zero rows.  Scores and sums in fp64 (declared
 * oracle numerics); the per-64 transform in fp32 in the reference's order of additions. */
static void hadamard64_rows_f16(uint16_t* row, int n) {
    for (int blk = 0; blk + 64 <= n; blk += 64) {
        float v[16][4];
        for (int l = 0; l < 16; ++l) {
            const float x0 = tq4o_f16_to_f32(row[blk + 4 * l]), x1 = tq4o_f16_to_f32(row[blk + 4 * l + 1]);
            const float x2 = tq4o_f16_to_f32(row[blk + 4 * l + 2]), x3 = tq4o_f16_to_f32(row[blk + 4 * l + 3]);
            const float a0 = x0 + x1, a1 = x0 - x1, a2 = x2 + x3, a3 = x2 - x3;
            v[l][0] = a0 + a2; v[l][1] = a1 + a3; v[l][2] = a0 - a2; v[l][3] = a1 - a3;
        }
        for (int h = 1; h < 16; h <<= 1) {
            float w[16][4];
            for (int l = 0; l < 16; ++l)
                for (int k = 0; k < 4; ++k) {
                    const float o = v[l ^ h][k];
                    w[l][k] = (l & h) ? (o - v[l][k]) : (v[l][k] + o);
                }
            memcpy(v, w, sizeof(v));
        }
        for (int l = 0; l < 16; ++l)
            for (int k = 0; k < 4; ++k) row[blk + 4 * l + k] = tq4o_f32_to_f16(v[l][k] * 0.125f);
    }
}

int tq4o_qsa_sparse_paged_attn_f16(const tq4o_layout* L, const uint16_t* q, const uint16_t* gate,
                                   const int32_t* selected_phys_blocks, const int32_t* selected_logical_blocks,
                                   const int32_t* num_selected_blocks, const int32_t* token_seq_pos,
                                   const uint8_t* valid_token_mask, uint16_t* out, int num_tokens,
                                   int local_q_heads, int select_k_blocks, float sm_scale, int hadamard64) {
    if (!L || !q || !selected_phys_blocks || !selected_logical_blocks || !num_selected_blocks || !token_seq_pos ||
        !out || num_tokens < 0 || local_q_heads <= 0 || L->local_kv_heads <= 0 ||
        local_q_heads % L->local_kv_heads || L->head_dim != 256 || select_k_blocks < 0)
        return -1;
    const int hd = 256, g = local_q_heads / L->local_kv_heads, gpp = L->block_size >> 2;
    if (gpp <= 0 || g > 64) return -1;
    float* qrows = (float*)malloc((size_t)g * hd * sizeof(float));
    double* acc = (double*)malloc((size_t)g * hd * sizeof(double));
    double* sc = (double*)malloc((size_t)(select_k_blocks > 0 ? select_k_blocks : 1) * 4 * g * sizeof(double));
    const uint8_t** vrows = (const uint8_t**)malloc((size_t)(select_k_blocks > 0 ? select_k_blocks : 1) * 4 * sizeof(void*));
    float kv[256], res[256];
    for (int tok = 0; tok < num_tokens; ++tok) {
        if (valid_token_mask && !valid_token_mask[tok]) {
            memset(out + (size_t)tok * local_q_heads * hd, 0, (size_t)local_q_heads * hd * 2);
            continue;
        }
        int n_sel = num_selected_blocks[tok];
        if (n_sel > select_k_blocks) n_sel = select_k_blocks;
        const int seq_pos = token_seq_pos[tok];
        for (int h = 0; h < L->local_kv_heads; ++h) {
            load_q(L, q, TQ4O_DT_F16, tok, local_q_heads, h * g, g, qrows);
            int n = 0;
            double m[64];
            for (int a = 0; a < g; ++a) m[a] = -INFINITY;
            for (int j = 0; j < n_sel; ++j) {
                const int32_t phys = selected_phys_blocks[(size_t)tok * select_k_blocks + j];
                const int32_t lg = selected_logical_blocks[(size_t)tok * select_k_blocks + j];
                for (int off = 0; off < 4; ++off) {
                    if (phys < 0 || lg * 4 + off > seq_pos) continue;
                    const size_t page = (size_t)(phys / gpp), row = (size_t)(phys % gpp) * 4 + off;
                    read_row(L->k_base + page * L->k_page_stride + (size_t)h * L->k_head_stride + row * L->k_token_stride,
                             L->k_format, hd, kv);
                    vrows[n] = L->v_base + page * L->v_page_stride + (size_t)h * L->v_head_stride + row * L->v_token_stride;
                    for (int a = 0; a < g; ++a) {
                        double dot = 0.0;
                        for (int c = 0; c < hd; ++c) dot += (double)qrows[(size_t)a * hd + c] * (double)kv[c];
                        const double s = dot * (double)sm_scale;
                        sc[(size_t)n * g + a] = s;
                        if (s > m[a]) m[a] = s;
                    }
                    ++n;
                }
            }
            double l[64];
            for (int a = 0; a < g; ++a) l[a] = 0.0;
            for (size_t i = 0; i < (size_t)g * hd; ++i) acc[i] = 0.0;
            for (int i = 0; i < n; ++i) {
                read_row(vrows[i], L->v_format, hd, kv);
                for (int a = 0; a < g; ++a) {
                    const double p = exp(sc[(size_t)i * g + a] - m[a]);
                    l[a] += p;
                    for (int c = 0; c < hd; ++c) acc[(size_t)a * hd + c] += p * (double)kv[c];
                }
            }
            for (int a = 0; a < g; ++a) {
                const size_t rowi = (size_t)tok * local_q_heads + (size_t)h * g + a;
                store_out(L, acc + (size_t)a * hd, l[a], res);
                uint16_t* dst = out + rowi * hd;
                for (int c = 0; c < hd; ++c) {
                    double val = (double)res[c];
                    if (gate) val *= 1.0 / (1.0 + exp(-(double)tq4o_f16_to_f32(gate[rowi * hd + c])));
                    dst[c] = tq4o_f32_to_f16((float)val);
                }
                if (hadamard64) hadamard64_rows_f16(dst, hd);
            }
        }
    }
    free(qrows); free(acc); free(sc); free(vrows);
    return 0;
}

int tq4o_hw_threads(void) {
    long n = sysconf(_SC_NPROCESSORS_ONLN);
    return n > 0 ? (int)n : 1;
}
