/*
 * CPU ORACLE -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the CPU reference path of allpaka's fused per-layer
 * ops.  Nothing the product ships may link, load or call this file: only the
 * test-suite, the smoke check and the benchmark's cpu_baseline leg use it, and
 * only as the checker / the timed CPU baseline.  Each function names the
 * reference lines it follows.  Build: see oracle/Makefile
 * (gcc -O2 -ffp-contract=off -fno-fast-math; glibc libm, the same symbols the
 * reference's Rust std lowers f32::exp / sin / cos / powf to on linux-gnu).
 *
 * Pinning status (what checks each function besides this file itself):
 *   f16<->f32                : reference specials + round-trip list + exhaustive
 *                              65536-code comparison against numpy float16.
 *   scale_min_k4, Q8_0, Q4_K : the reference's own known-answer vectors, plus a
 *                              second independent numpy decoder on random bytes.
 *   Q2_K/Q3_K/Q5_K/Q6_K      : the reference's own bit-layout vectors.
 *   Q5_0                     : the reference holds no vector for it; pinned by a
 *                              hand-worked block (high bits at elements 0, 15,
 *                              16, 31, one-bit and one-nibble walks) and by a
 *                              second numpy decoder written from ggml's published
 *                              dequantize_row_q5_0 on random bytes.
 *   F16/BF16/F32 rows        : hand-worked bit patterns; bf16 over all 65536 codes.
 *   sum_sq/rmsnorm*          : reference vectors + numpy float64 closed form.
 *   rope_*                   : reference vectors (identity at pos 0, one-hot
 *                              pairing, cached==naive bit-identical, partial
 *                              rotary) + numpy closed form.
 *   silu/swiglu/softmax      : reference vectors + numpy closed form.
 *   route_gated/route        : reference vectors.  Equal selection values
 *                              (bit-equal logits, or distinct logits whose
 *                              scores round to one f32) are parity unpinned
 *                              wherever they occur, unless k == n: the
 *                              reference first runs select_nth_unstable_by
 *                              (moe.rs:579), which leaves order[..k] in an
 *                              unspecified order, and the stable sort that
 *                              follows (moe.rs:581) keeps equal values in THAT
 *                              order, not in index order.  Which of two equal
 *                              values across the k boundary is kept, the order
 *                              of equal picks inside the top k, and (with a
 *                              selection bias, where equal selection values
 *                              need not have equal scores) the summation order
 *                              of `total` are therefore implementation-defined
 *                              in the reference.  The oracle resolves all of
 *                              them as "lower index first".  Without a bias
 *                              equal picks have equal scores, so ids as a set
 *                              inside the top k and every weight are still the
 *                              reference's; only the order of the equal ids is
 *                              the oracle's choice.
 *   moe_group                : brute force + invariants on small inputs.
 *   *_f16 activations        : the reference has no fp16 activations; these are
 *                              defined here as widen -> f32 reference op -> one
 *                              RNE rounding.  Parity unpinned (no reference
 *                              counterpart exists); the f32 core they wrap is
 *                              pinned as above.
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORA_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ dtype */

/* crates/allpaka-dtype/src/lib.rs:129-146 */
ORA_API float ora_f16_to_f32(uint16_t h) {
    uint32_t sign = (h >> 15) & 1u, exp = (h >> 10) & 0x1fu, frac = h & 0x3ffu, bits;
    if (exp == 0 && frac == 0) {
        bits = sign << 31;
    } else if (exp == 0) {
        uint32_t p = 31u - (uint32_t)__builtin_clz(frac);
        uint32_t e = 127u - 24u + p;
        uint32_t f = (frac << (23u - p)) & 0x7fffffu;
        bits = (sign << 31) | (e << 23) | f;
    } else if (exp == 0x1f && frac == 0) {
        bits = (sign << 31) | 0x7f800000u;
    } else if (exp == 0x1f) {
        bits = (sign << 31) | 0x7f800000u | (frac << 13);
    } else {
        bits = (sign << 31) | ((exp + 127u - 15u) << 23) | (frac << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* crates/allpaka-dtype/src/lib.rs:151-184 (round-to-nearest-even) */
ORA_API uint16_t ora_f32_to_f16(float x) {
    uint32_t bits;
    memcpy(&bits, &x, 4);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    uint32_t mag = bits & 0x7fffffffu;
    if (mag >= 0x7f800000u) {
        uint16_t man = mag > 0x7f800000u ? 0x200 : 0;
        return (uint16_t)(sign | 0x7c00 | man);
    }
    int32_t exp = (int32_t)(mag >> 23) - 127;
    if (exp >= 16) return (uint16_t)(sign | 0x7c00);
    if (exp >= -14) {
        uint32_t man = mag & 0x7fffffu;
        uint16_t h = (uint16_t)((((uint32_t)(exp + 15)) << 10) | (man >> 13));
        uint32_t rest = man & 0x1fffu;
        if (rest > 0x1000u || (rest == 0x1000u && (h & 1))) h++;
        return (uint16_t)(sign | h);
    }
    if (exp < -25) return sign;
    uint32_t man = (mag & 0x7fffffu) | 0x800000u;
    uint32_t shift = (uint32_t)(-exp - 14);
    uint16_t h = (uint16_t)(man >> (13 + shift));
    uint32_t rest = man & ((1u << (13 + shift)) - 1u);
    uint32_t halfway = 1u << (12 + shift);
    if (rest > halfway || (rest == halfway && (h & 1))) h++;
    return (uint16_t)(sign | h);
}

/* crates/allpaka-dtype/src/lib.rs:188-190 */
ORA_API float ora_bf16_to_f32(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

ORA_API void ora_f16_to_f32_slice(const uint16_t *h, float *out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = ora_f16_to_f32(h[i]);
}
ORA_API void ora_f32_to_f16_slice(const float *x, uint16_t *out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = ora_f32_to_f16(x[i]);
}

/* crates/allpaka-dtype/src/lib.rs:382-390 */
ORA_API void ora_scale_min_k4(int j, const uint8_t *p, float *sc, float *mn) {
    if (j < 4) {
        *sc = (float)(p[j] & 63);
        *mn = (float)(p[j + 4] & 63);
    } else {
        uint8_t s = (uint8_t)((p[j + 4] & 0xf) | ((p[j - 4] >> 6) << 4));
        uint8_t m = (uint8_t)((p[j + 4] >> 4) | ((p[j] >> 6) << 4));
        *sc = (float)s;
        *mn = (float)m;
    }
}

/* crates/allpaka-dtype/src/lib.rs:395-422, written per scale (the reference's
 * own test :461-476 states the same per-element rule). */
static void unpack_q3_k_scales_raw(const uint8_t *p, int8_t out[16]) {
    for (int i = 0; i < 16; i++) {
        uint8_t lo = i < 8 ? (uint8_t)(p[i] & 0xf) : (uint8_t)(p[i - 8] >> 4);
        uint8_t hi = (uint8_t)((p[8 + i % 4] >> (2 * (i / 4))) & 3);
        out[i] = (int8_t)(lo | (hi << 4));
    }
}

/* Unified dequant format codes, crates/allpaka-backend/src/gpu/common.rs:47-61 */
enum { FMT_Q4K = 0, FMT_Q5K, FMT_Q6K, FMT_Q8_0, FMT_Q2K, FMT_Q3K, FMT_Q5_0, FMT_F16, FMT_F32, FMT_BF16 };

/* block geometry, crates/allpaka-dtype/src/lib.rs:79-108 */
ORA_API int ora_block_elements(int fmt) {
    switch (fmt) {
    case FMT_F32: case FMT_F16: case FMT_BF16: return 1;
    case FMT_Q5_0: case FMT_Q8_0: return 32;
    case FMT_Q2K: case FMT_Q3K: case FMT_Q4K: case FMT_Q5K: case FMT_Q6K: return 256;
    default: return 0;
    }
}
ORA_API int ora_block_bytes(int fmt) {
    switch (fmt) {
    case FMT_F32: return 4;
    case FMT_F16: case FMT_BF16: return 2;
    case FMT_Q8_0: return 34;
    case FMT_Q5_0: return 22;
    case FMT_Q2K: return 84;
    case FMT_Q3K: return 110;
    case FMT_Q4K: return 144;
    case FMT_Q5K: return 176;
    case FMT_Q6K: return 210;
    default: return 0;
    }
}
/* crates/allpaka-dtype/src/lib.rs:112-124; -1 = unsupported type, -2 = ragged. */
ORA_API int64_t ora_expected_bytes(int fmt, size_t elements) {
    int be = ora_block_elements(fmt), bb = ora_block_bytes(fmt);
    if (!be || !bb) return -1;
    if (elements % (size_t)be) return -2;
    return (int64_t)(elements / (size_t)be * (size_t)bb);
}
/* crates/allpaka-backend/src/gpu/common.rs:77-88 */
ORA_API uint32_t ora_embed_row_groups(uint32_t fmt, size_t n_in) {
    size_t g = fmt <= 5 ? (n_in + 255) / 256 : (n_in + 31) / 32;
    return g == 0 ? 1u : (uint32_t)g;
}

/* ---------------------------------------------------------------- dequant */

static inline float rd_f16(const uint8_t *b) { return ora_f16_to_f32((uint16_t)(b[0] | (b[1] << 8))); }

/* crates/allpaka-gguf/src/dequant.rs:94-126 (non-aarch64 arm :122-125) */
static void dq_q8_0(const uint8_t *b, float *out) {
    float d = rd_f16(b);
    for (int i = 0; i < 32; i++) out[i] = d * (float)(int8_t)b[2 + i];
}
/* dequant.rs:131-141 */
static void dq_q5_0(const uint8_t *b, float *out) {
    float d = rd_f16(b);
    uint32_t qh = (uint32_t)b[2] | ((uint32_t)b[3] << 8) | ((uint32_t)b[4] << 16) | ((uint32_t)b[5] << 24);
    const uint8_t *qs = b + 6;
    for (int j = 0; j < 16; j++) {
        int32_t x0 = (int32_t)((uint32_t)(qs[j] & 0x0f) | (((qh >> j) & 1u) << 4)) - 16;
        int32_t x1 = (int32_t)((uint32_t)(qs[j] >> 4) | (((qh >> (j + 16)) & 1u) << 4)) - 16;
        out[j] = d * (float)x0;
        out[j + 16] = d * (float)x1;
    }
}
/* dequant.rs:150-174 */
static void dq_q2_k(const uint8_t *b, float *out) {
    const uint8_t *scales = b, *qs = b + 16;
    float d = rd_f16(b + 80), dmin = rd_f16(b + 82);
    int is = 0, pos = 0;
    for (int half = 0; half < 2; half++) {
        const uint8_t *q = qs + half * 32;
        for (int shift = 0; shift < 8; shift += 2)
            for (int group = 0; group < 2; group++) {
                uint8_t sc = scales[is];
                float dl = d * (float)(sc & 0xf);
                float ml = dmin * (float)(sc >> 4);
                for (int l = 0; l < 16; l++) {
                    uint8_t quant = (uint8_t)((q[group * 16 + l] >> shift) & 3);
                    out[pos + l] = dl * (float)quant - ml;
                }
                pos += 16;
                is++;
            }
    }
}
/* dequant.rs:176-204 */
static void dq_q3_k(const uint8_t *b, float *out) {
    const uint8_t *hmask = b, *qs = b + 32, *packed = b + 96;
    float d_all = rd_f16(b + 108);
    int8_t sr[16];
    unpack_q3_k_scales_raw(packed, sr);
    int is = 0, pos = 0;
    uint8_t m = 1;
    for (int half = 0; half < 2; half++) {
        const uint8_t *q = qs + half * 32;
        for (int shift = 0; shift < 8; shift += 2) {
            for (int group = 0; group < 2; group++) {
                float dl = d_all * (float)((int32_t)sr[is] - 32);
                for (int l = 0; l < 16; l++) {
                    int idx = group * 16 + l;
                    int32_t quant = (int32_t)((q[idx] >> shift) & 3) - ((hmask[idx] & m) ? 0 : 4);
                    out[pos + l] = dl * (float)quant;
                }
                pos += 16;
                is++;
            }
            m = (uint8_t)(m << 1);
        }
    }
}
/* dequant.rs:211-231: d*sc, dmin*mn, (d*sc)*q and the subtraction are four
 * separately rounded f32 operations (this file is built with -ffp-contract=off). */
static void dq_q4_k(const uint8_t *b, float *out) {
    float d = rd_f16(b), dmin = rd_f16(b + 2);
    const uint8_t *packed = b + 4, *qs = b + 16;
    for (int pair = 0; pair < 4; pair++) {
        const uint8_t *q = qs + pair * 32;
        float sc1, mn1, sc2, mn2;
        ora_scale_min_k4(pair * 2, packed, &sc1, &mn1);
        ora_scale_min_k4(pair * 2 + 1, packed, &sc2, &mn2);
        float d_sc1 = d * sc1, dm1 = dmin * mn1, d_sc2 = d * sc2, dm2 = dmin * mn2;
        int base = pair * 64;
        for (int l = 0; l < 32; l++) {
            out[base + l] = d_sc1 * (float)(q[l] & 0xf) - dm1;
            out[base + 32 + l] = d_sc2 * (float)(q[l] >> 4) - dm2;
        }
    }
}
/* dequant.rs:238-263 */
static void dq_q5_k(const uint8_t *b, float *out) {
    float d = rd_f16(b), dmin = rd_f16(b + 2);
    const uint8_t *packed = b + 4, *qh = b + 16, *qs = b + 48;
    for (int pair = 0; pair < 4; pair++) {
        const uint8_t *q = qs + pair * 32;
        float sc1, mn1, sc2, mn2;
        ora_scale_min_k4(pair * 2, packed, &sc1, &mn1);
        ora_scale_min_k4(pair * 2 + 1, packed, &sc2, &mn2);
        float d_sc1 = d * sc1, dm1 = dmin * mn1, d_sc2 = d * sc2, dm2 = dmin * mn2;
        uint8_t bit1 = (uint8_t)(1u << (pair * 2)), bit2 = (uint8_t)(1u << (pair * 2 + 1));
        int base = pair * 64;
        for (int l = 0; l < 32; l++) {
            uint8_t hi1 = (qh[l] & bit1) ? 16 : 0, hi2 = (qh[l] & bit2) ? 16 : 0;
            out[base + l] = d_sc1 * (float)(uint8_t)((q[l] & 0xf) + hi1) - dm1;
            out[base + 32 + l] = d_sc2 * (float)(uint8_t)((q[l] >> 4) + hi2) - dm2;
        }
    }
}
/* dequant.rs:271-295: d * scale * q is evaluated left to right, (d*scale)*q. */
static void dq_q6_k(const uint8_t *b, float *out) {
    const uint8_t *ql0 = b, *qh0 = b + 128, *scales = b + 192;
    float d = rd_f16(b + 208);
    for (int half = 0; half < 2; half++) {
        const uint8_t *ql = ql0 + half * 64, *qh = qh0 + half * 32, *sc = scales + half * 8;
        float *o = out + half * 128;
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            int32_t q1 = (int32_t)(int8_t)((ql[l] & 0xf) | ((qh[l] & 3) << 4)) - 32;
            int32_t q2 = (int32_t)(int8_t)((ql[l + 32] & 0xf) | (((qh[l] >> 2) & 3) << 4)) - 32;
            int32_t q3 = (int32_t)(int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
            int32_t q4 = (int32_t)(int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
            o[l] = d * (float)(int8_t)sc[is] * (float)q1;
            o[32 + l] = d * (float)(int8_t)sc[is + 2] * (float)q2;
            o[64 + l] = d * (float)(int8_t)sc[is + 4] * (float)q3;
            o[96 + l] = d * (float)(int8_t)sc[is + 6] * (float)q4;
        }
    }
}

/* crates/allpaka-gguf/src/dequant.rs:26-91.  Returns 0 ok, 1 = the reference's
 * GgufError::Dequant (wrong byte count, ragged element count, unknown type). */
ORA_API int ora_dequant_into(int fmt, const uint8_t *data, size_t nbytes, float *dst, size_t elements) {
    int64_t expected = ora_expected_bytes(fmt, elements);
    if (expected < 0 || (size_t)expected != nbytes) return 1;
    size_t i;
    switch (fmt) {
    case FMT_F32: memcpy(dst, data, nbytes); break;
    case FMT_F16: for (i = 0; i < elements; i++) dst[i] = rd_f16(data + 2 * i); break;
    case FMT_BF16: for (i = 0; i < elements; i++) dst[i] = ora_bf16_to_f32((uint16_t)(data[2 * i] | (data[2 * i + 1] << 8))); break;
    case FMT_Q5_0: for (i = 0; i < elements / 32; i++) dq_q5_0(data + 22 * i, dst + 32 * i); break;
    case FMT_Q8_0: for (i = 0; i < elements / 32; i++) dq_q8_0(data + 34 * i, dst + 32 * i); break;
    case FMT_Q2K: for (i = 0; i < elements / 256; i++) dq_q2_k(data + 84 * i, dst + 256 * i); break;
    case FMT_Q3K: for (i = 0; i < elements / 256; i++) dq_q3_k(data + 110 * i, dst + 256 * i); break;
    case FMT_Q4K: for (i = 0; i < elements / 256; i++) dq_q4_k(data + 144 * i, dst + 256 * i); break;
    case FMT_Q5K: for (i = 0; i < elements / 256; i++) dq_q5_k(data + 176 * i, dst + 256 * i); break;
    case FMT_Q6K: for (i = 0; i < elements / 256; i++) dq_q6_k(data + 210 * i, dst + 256 * i); break;
    default: return 1;
    }
    return 0;
}

/* QuantMat::new + row_into, crates/allpaka-backend/src/quantmat/mod.rs:39-89.
 * 0 ok; 2 = new() would bail (unsupported type / ragged row / wrong byte count);
 * 3 = row out of range; 4 = destination length mismatch. */
ORA_API int ora_quantmat_row_into(const uint8_t *data, size_t data_len, int fmt, size_t n_out, size_t n_in,
                                  size_t j, float *dst, size_t dst_len) {
    int be = ora_block_elements(fmt), bb = ora_block_bytes(fmt);
    if (!be || !bb) return 2;
    if (n_in % (size_t)be) return 2;
    size_t row_bytes = n_in / (size_t)be * (size_t)bb;
    if (row_bytes * n_out != data_len) return 2;
    if (j >= n_out) return 3;
    if (dst_len != n_in) return 4;
    return ora_dequant_into(fmt, data + j * row_bytes, row_bytes, dst, n_in);
}

/* The embedding gather as its callers run it: a serial loop of row_into over the
 * token ids (crates/allpaka-model/src/model/prefill.rs:92-106, decode.rs:422-431);
 * an id >= vocab is rejected before anything is written (returns 3). */
ORA_API int ora_embed_rows(const uint8_t *data, size_t data_len, int fmt, size_t vocab, size_t n_in,
                           const uint32_t *ids, size_t t, float *out) {
    for (size_t i = 0; i < t; i++)
        if (ids[i] >= vocab) return 3;
    for (size_t i = 0; i < t; i++) {
        int rc = ora_quantmat_row_into(data, data_len, fmt, vocab, n_in, ids[i], out + i * n_in, n_in);
        if (rc) return rc;
    }
    return 0;
}

/* ------------------------------------------------------------------- norm */

/* crates/allpaka-backend/src/ops/norm.rs:42-78, the x86_64 avx2+fma arm, written
 * lane by lane: two 4-lane f64 accumulators over 8-element steps, combined as
 * (acc0+acc1) lane-wise, then lo+hi halves, then the two remaining lanes, then a
 * scalar tail.  A square of an f32 is exact in f64, so fma(d,d,acc) == d*d+acc. */
ORA_API double ora_sum_sq_f64(const float *x, size_t n) {
    double acc0[4] = {0, 0, 0, 0}, acc1[4] = {0, 0, 0, 0};
    size_t i = 0;
    while (i + 8 <= n) {
        for (int l = 0; l < 4; l++) {
            double d0 = (double)x[i + l], d1 = (double)x[i + 4 + l];
            acc0[l] = d0 * d0 + acc0[l];
            acc1[l] = d1 * d1 + acc1[l];
        }
        i += 8;
    }
    double sum[4];
    for (int l = 0; l < 4; l++) sum[l] = acc0[l] + acc1[l];
    double pair0 = sum[0] + sum[2], pair1 = sum[1] + sum[3];
    double total = pair0 + pair1;
    while (i < n) {
        double v = (double)x[i];
        total += v * v;
        i++;
    }
    return total;
}

/* norm.rs:115-187 */
ORA_API void ora_rmsnorm(float *x, const float *w, size_t n, float eps) {
    double mean_sq = ora_sum_sq_f64(x, n) / (double)n;
    double scale = 1.0 / sqrt(mean_sq + (double)eps);
    for (size_t i = 0; i < n; i++) x[i] = (float)((double)x[i] * scale) * w[i];
}
/* norm.rs:193-269 */
ORA_API void ora_rmsnorm_into(float *dst, const float *src, const float *w, size_t n, float eps) {
    double mean_sq = ora_sum_sq_f64(src, n) / (double)n;
    double scale = 1.0 / sqrt(mean_sq + (double)eps);
    for (size_t i = 0; i < n; i++) dst[i] = (float)((double)src[i] * scale) * w[i];
}

/* --- the reference's worker-pool partition rule ---------------------------
 * crates/allpaka-backend/src/thread_pool.rs:210-231 par_for_chunks: up to
 * n_workers contiguous chunks of ceil(total/nt) items; worker 0 is the caller. */
typedef void (*chunk_fn)(size_t start, size_t end, void *ctx);
typedef struct { chunk_fn f; void *ctx; size_t start, end; } chunk_job;
static void *chunk_tramp(void *p) {
    chunk_job *j = (chunk_job *)p;
    j->f(j->start, j->end, j->ctx);
    return NULL;
}
static void par_for_chunks(size_t total, size_t n_workers, chunk_fn f, void *ctx) {
    if (total == 0 || n_workers == 0) return;
    size_t nt = n_workers < total ? n_workers : total;
    if (nt <= 1) { f(0, total, ctx); return; }
    size_t per = (total + nt - 1) / nt, chunks = (total + per - 1) / per;
    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * chunks);
    chunk_job *jobs = (chunk_job *)malloc(sizeof(chunk_job) * chunks);
    for (size_t c = 0; c < chunks; c++) {
        jobs[c].f = f; jobs[c].ctx = ctx;
        jobs[c].start = c * per;
        jobs[c].end = jobs[c].start + per < total ? jobs[c].start + per : total;
    }
    for (size_t c = 1; c < chunks; c++) pthread_create(&th[c], NULL, chunk_tramp, &jobs[c]);
    chunk_tramp(&jobs[0]);
    for (size_t c = 1; c < chunks; c++) pthread_join(th[c], NULL);
    free(th); free(jobs);
}

typedef struct { float *dst; const float *src, *w; size_t n; float eps; } rows_ctx;
static void rows_chunk(size_t s, size_t e, void *p) {
    rows_ctx *c = (rows_ctx *)p;
    for (size_t r = s; r < e; r++) ora_rmsnorm_into(c->dst + r * c->n, c->src + r * c->n, c->w, c->n, c->eps);
}
/* norm.rs:275-304.  Returns 1 where the reference panics with "dst holds fewer
 * rows than src"; `threads` stands for thread_pool::cpu_threads(). */
ORA_API int ora_rmsnorm_rows_into(float *dst, size_t dst_len, const float *src, size_t src_len, const float *w,
                                  size_t n, float eps, size_t threads) {
    size_t rows = src_len / n;
    if (dst_len < rows * n) return 1;
    size_t t = threads < (rows ? rows : 1) ? threads : (rows ? rows : 1);
    rows_ctx c = {dst, src, w, n, eps};
    if (t <= 1 || rows < 4 || src_len < 16384) { rows_chunk(0, rows, &c); return 0; }
    par_for_chunks(rows, t, rows_chunk, &c);
    return 0;
}

/* crates/allpaka-backend/src/ops/blas.rs:105-178; returns 1 where the reference
 * asserts equal lengths. */
ORA_API int ora_add_assign_slice(float *a, size_t a_len, const float *b, size_t b_len) {
    if (a_len != b_len) return 1;
    for (size_t i = 0; i < a_len; i++) a[i] += b[i];
    return 0;
}
typedef struct { float *a; const float *b; size_t per, total; } add_ctx;
static void add_chunk(size_t cs, size_t ce, void *p) {
    add_ctx *c = (add_ctx *)p;
    size_t s = cs * c->per, e = ce * c->per < c->total ? ce * c->per : c->total;
    for (size_t i = s; i < e; i++) c->a[i] += c->b[i];
}
/* blas.rs:182-213 */
ORA_API int ora_add_assign_par(float *a, size_t a_len, const float *b, size_t b_len, size_t threads) {
    if (a_len != b_len) return 1;
    size_t per = (a_len + threads - 1) / (threads ? threads : 1);
    if (per < ((size_t)1 << 16)) per = (size_t)1 << 16;
    if (a_len <= per || threads <= 1) return ora_add_assign_slice(a, a_len, b, b_len);
    add_ctx c = {a, b, per, a_len};
    par_for_chunks((a_len + per - 1) / per, threads, add_chunk, &c);
    return 0;
}
/* blas.rs:25-102, x86 avx2+fma arm: dst = fma(src, scale, dst) (one rounding). */
ORA_API int ora_add_scaled_slice(float *dst, size_t dst_len, const float *src, size_t src_len, float scale) {
    if (dst_len != src_len) return 1;
    for (size_t i = 0; i < dst_len; i++) dst[i] = fmaf(src[i], scale, dst[i]);
    return 0;
}

/* ------------------------------------------------------------------- rope */

/* crates/allpaka-backend/src/ops/rope.rs:8-12 */
ORA_API void ora_rope_inv_freq(size_t head_dim, float base, float *out) {
    for (size_t i = 0; i < head_dim / 2; i++) out[i] = powf(base, -2.0f * (float)i / (float)head_dim);
}
/* rope.rs:18-22; out is [half][2] = [sin, cos] (the array form the callers
 * keep, crates/allpaka-model/src/model/session.rs:34-50). */
ORA_API void ora_rope_sin_cos(uint32_t pos, const float *inv, size_t half, float *out) {
    for (size_t i = 0; i < half; i++) {
        float a = (float)pos * inv[i];
        out[2 * i] = sinf(a);
        out[2 * i + 1] = cosf(a);
    }
}
/* rope.rs:70-81; returns 1 where the reference asserts x.len() >= 2*half. */
ORA_API int ora_rope_neox_cached_from_array(float *x, size_t x_len, const float *table, size_t half) {
    if (x_len < 2 * half) return 1;
    for (size_t i = 0; i < half; i++) {
        float s = table[2 * i], c = table[2 * i + 1];
        float a = x[i], b = x[i + half];
        x[i] = a * c - b * s;
        x[i + half] = a * s + b * c;
    }
    return 0;
}
/* rope.rs:52-64 (NORM pairing, kept for the pairing known-answer test) */
ORA_API int ora_rope_norm_cached_from_array(float *x, size_t x_len, const float *table, size_t half) {
    if (x_len < 2 * half) return 1;
    for (size_t i = 0; i < half; i++) {
        float s = table[2 * i], c = table[2 * i + 1];
        float a = x[2 * i], b = x[2 * i + 1];
        x[2 * i] = a * c - b * s;
        x[2 * i + 1] = a * s + b * c;
    }
    return 0;
}
/* rope.rs:105-117, the naive form */
ORA_API void ora_rope_neox(float *x, size_t d, uint32_t pos, float base) {
    size_t half = d / 2;
    for (size_t i = 0; i < half; i++) {
        float theta = (float)pos * powf(base, -2.0f * (float)i / (float)d);
        float s = sinf(theta), c = cosf(theta);
        float a = x[i], b = x[i + half];
        x[i] = a * c - b * s;
        x[i + half] = a * s + b * c;
    }
}
/* rope.rs:90-101 */
ORA_API void ora_rope_norm(float *x, size_t d, uint32_t pos, float base) {
    for (size_t i = 0; i < d / 2; i++) {
        float theta = (float)pos * powf(base, -2.0f * (float)i / (float)d);
        float s = sinf(theta), c = cosf(theta);
        float a = x[2 * i], b = x[2 * i + 1];
        x[2 * i] = a * c - b * s;
        x[2 * i + 1] = a * s + b * c;
    }
}

/* The only caller loop of per-head QK-norm + RoPE,
 * crates/allpaka-model/src/model/attention.rs:131-165: for row i, every head of
 * q then of k gets rmsnorm(head, w, eps) (when a weight is given) followed by
 * the NeoX rotation with that row's table rope_flat[i*half .. (i+1)*half]. */
/* style 0: RopeStyle::Neox, 1: RopeStyle::Norm (rope_from_arrays, attention.rs:62-67) */
ORA_API void ora_qknorm_rope_rows_style(float *q, float *k, size_t rows, size_t n_q, size_t n_kv, size_t head_dim,
                                        const float *qw, const float *kw, const float *rope_flat, size_t half, float eps,
                                        int style) {
    for (size_t i = 0; i < rows; i++) {
        const float *rope = rope_flat + i * half * 2;
        for (size_t h = 0; h < n_q; h++) {
            float *head = q + (i * n_q + h) * head_dim;
            if (qw) ora_rmsnorm(head, qw, head_dim, eps);
            if (style) ora_rope_norm_cached_from_array(head, head_dim, rope, half);
            else ora_rope_neox_cached_from_array(head, head_dim, rope, half);
        }
    }
    for (size_t i = 0; i < rows; i++) {
        const float *rope = rope_flat + i * half * 2;
        for (size_t h = 0; h < n_kv; h++) {
            float *head = k + (i * n_kv + h) * head_dim;
            if (kw) ora_rmsnorm(head, kw, head_dim, eps);
            if (style) ora_rope_norm_cached_from_array(head, head_dim, rope, half);
            else ora_rope_neox_cached_from_array(head, head_dim, rope, half);
        }
    }
}
ORA_API void ora_qknorm_rope_rows(float *q, float *k, size_t rows, size_t n_q, size_t n_kv, size_t head_dim,
                                  const float *qw, const float *kw, const float *rope_flat, size_t half, float eps) {
    ora_qknorm_rope_rows_style(q, k, rows, n_q, n_kv, head_dim, qw, kw, rope_flat, half, eps, 0);
}

/* add_bias_rows, crates/allpaka-model/src/model/loader.rs:519-523: every row of bias_len elements gets
 * ops::add_assign_slice(row, bias); a trailing partial row is left alone (chunks_exact_mut). */
ORA_API void ora_add_bias_rows(float *rows, size_t len, const float *bias, size_t bias_len) {
    for (size_t r = 0; r + bias_len <= len && bias_len; r += bias_len)
        for (size_t i = 0; i < bias_len; i++) rows[r + i] += bias[i];
}

/* ------------------------------------------------------------- activation */

/* crates/allpaka-backend/src/ops/activation.rs:19-22 */
ORA_API float ora_silu(float x) { return x / (1.0f + expf(-x)); }
/* activation.rs:57-58,116-119 (the non-aarch64 arm); 1 = length assert. */
ORA_API int ora_swiglu(float *gate, size_t g_len, const float *up, size_t u_len) {
    if (g_len != u_len) return 1;
    for (size_t i = 0; i < g_len; i++) gate[i] = ora_silu(gate[i]) * up[i];
    return 0;
}
/* activation.rs:44-51: GeGLU with the tanh GELU (Gemma's FFN), the same formula as ggml_gelu; every product
 * in the reference's left-to-right order, tanhf from libm as Rust's f32::tanh.  1 = length assert. */
ORA_API float ora_gelu_tanh_mul(float x, float u) {
    const float SQRT_2_OVER_PI = 0.7978846f;
    return 0.5f * x * (1.0f + tanhf(SQRT_2_OVER_PI * x * (1.0f + 0.044715f * x * x))) * u;
}
ORA_API int ora_geglu_tanh(float *gate, size_t g_len, const float *up, size_t u_len) {
    if (g_len != u_len) return 1;
    for (size_t i = 0; i < g_len; i++) gate[i] = ora_gelu_tanh_mul(gate[i], up[i]);
    return 0;
}
/* activation.rs:5-16 (f32::max fold: a NaN operand is ignored) */
ORA_API void ora_softmax(float *x, size_t n) {
    float mx = -INFINITY;
    for (size_t i = 0; i < n; i++) mx = fmaxf(mx, x[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) {
        x[i] = expf(x[i] - mx);
        sum += x[i];
    }
    float inv = 1.0f / sum;
    for (size_t i = 0; i < n; i++) x[i] *= inv;
}
/* activation.rs:36-40 */
ORA_API void ora_sigmoid(float *x, size_t n) {
    for (size_t i = 0; i < n; i++) x[i] = 1.0f / (1.0f + expf(-x[i]));
}

/* ----------------------------------------------------------------- router */

/* f32::total_cmp key (Rust core: bits ^ (((bits as i32) >> 31) as u32 >> 1)) */
static inline int32_t total_key(float f) {
    int32_t b;
    memcpy(&b, &f, 4);
    return b ^ (int32_t)(((uint32_t)(b >> 31)) >> 1);
}

/* Descending by total_cmp, ties -> lower index first.  Inside the top-k this is
 * exactly the reference's stable sort_by (crates/allpaka-model/src/model/moe.rs:582);
 * at the k boundary the reference's select_nth_unstable_by (:579) leaves exact
 * ties implementation-defined and this oracle takes the lower index, the rule
 * the reference's accelerator kernels state. */
static void topk_desc(const float *sel, size_t n, size_t k, size_t *out) {
    uint8_t *taken = (uint8_t *)calloc(n, 1);
    for (size_t r = 0; r < k; r++) {
        size_t best = n;
        for (size_t e = 0; e < n; e++) {
            if (taken[e]) continue;
            if (best == n || total_key(sel[e]) > total_key(sel[best])) best = e;
        }
        taken[best] = 1;
        out[r] = best;
    }
    free(taken);
}

/* crates/allpaka-model/src/model/moe.rs:524-594.  gating: 0 softmax, 1 sigmoid.
 * Returns the number of picks written (min(k, n)). */
ORA_API size_t ora_route_gated(const float *logits, size_t n, size_t k, int gating, int norm, float scale,
                               const float *bias, uint32_t *ids, float *w) {
    if (k > n) k = n;
    if (k == 0) return 0;
    float *scores = (float *)malloc(sizeof(float) * n);
    float *sel = (float *)malloc(sizeof(float) * n);
    size_t *order = (size_t *)malloc(sizeof(size_t) * k);
    memcpy(scores, logits, sizeof(float) * n);
    if (gating == 0) ora_softmax(scores, n); else ora_sigmoid(scores, n);
    for (size_t i = 0; i < n; i++) sel[i] = bias ? scores[i] + bias[i] : scores[i];
    topk_desc(sel, n, k, order);
    float total = 0.0f;
    for (size_t r = 0; r < k; r++) total += scores[order[r]];
    for (size_t r = 0; r < k; r++) {
        size_t e = order[r];
        float wt = (norm && total > 0.0f) ? scores[e] / total : (norm ? 1.0f / (float)k : scores[e]);
        ids[r] = (uint32_t)e;
        w[r] = wt * scale;
    }
    free(scores); free(sel); free(order);
    return k;
}

/* The selection order taken on the RAW logits instead of the gated scores
 * (what an accelerator that never materialises probabilities does; monotone-
 * equivalent for softmax without bias unless two distinct logits round to one
 * probability).  Tests assert both orders agree on the seeded inputs. */
ORA_API size_t ora_topk_by_logits(const float *logits, size_t n, size_t k, uint32_t *ids) {
    if (k > n) k = n;
    if (k == 0) return 0;
    size_t *order = (size_t *)malloc(sizeof(size_t) * k);
    topk_desc(logits, n, k, order);
    for (size_t r = 0; r < k; r++) ids[r] = (uint32_t)order[r];
    free(order);
    return k;
}

/* moe.rs:623-658, the legacy contract on already-softmaxed probabilities. */
ORA_API size_t ora_route(const float *probs, size_t n, size_t k, uint32_t *ids, float *w) {
    if (k > n) k = n;
    if (k == 0) return 0;
    size_t *order = (size_t *)malloc(sizeof(size_t) * k);
    topk_desc(probs, n, k, order);
    float total = 0.0f;
    for (size_t r = 0; r < k; r++) total += probs[order[r]];
    for (size_t r = 0; r < k; r++) {
        ids[r] = (uint32_t)order[r];
        w[r] = total > 0.0f ? probs[order[r]] / total : 1.0f / (float)k;
    }
    free(order);
    return k;
}

typedef struct { const float *logits; size_t n, k; int gating, norm; float scale; const float *bias; uint32_t *ids; float *w; } route_ctx;
static void route_chunk(size_t s, size_t e, void *p) {
    route_ctx *c = (route_ctx *)p;
    for (size_t t = s; t < e; t++)
        ora_route_gated(c->logits + t * c->n, c->n, c->k, c->gating, c->norm, c->scale, c->bias, c->ids + t * c->k, c->w + t * c->k);
}
/* Per-token routing spread over the pool, moe.rs:204-227. */
ORA_API void ora_route_rows(const float *logits, size_t rows, size_t n, size_t k, int gating, int norm, float scale,
                            const float *bias, uint32_t *ids, float *w, size_t threads) {
    if (k > n) k = n;
    if (k == 0 || rows == 0) return;
    route_ctx c = {logits, n, k, gating, norm, scale, bias, ids, w};
    par_for_chunks(rows, threads < rows ? threads : rows, route_chunk, &c);
}

/* Token -> expert grouping ("permute"):
 *   groups[e].push((token, w)) scanning tokens ascending and picks best-first
 *   (moe.rs:229-236); `used` = non-empty experts ascending (:247); table rows
 *   [expert, row0, rows] for used experts only and tok[] = token per flat row,
 *   expert-major, token-ascending within an expert (:260-271); per-token hit
 *   lists in ascending expert order, flattened into CSR tok_off/hit_row/hit_w
 *   (crates/allpaka-model/src/model/prefill.rs:624-675, no shared expert).
 * Returns n_used; table holds 3*n_used values; tok/hit_row/hit_w hold rows*k;
 * tok_off holds rows+1. */
ORA_API size_t ora_moe_group(const uint32_t *ids, const float *w, size_t rows, size_t k, size_t n_expert,
                             uint32_t *table, uint32_t *tok, uint32_t *tok_off, uint32_t *hit_row, float *hit_w) {
    uint32_t *count = (uint32_t *)calloc(n_expert, sizeof(uint32_t));
    uint32_t *row0 = (uint32_t *)calloc(n_expert, sizeof(uint32_t));
    uint32_t *fill = (uint32_t *)calloc(n_expert, sizeof(uint32_t));
    uint32_t *nhits = (uint32_t *)calloc(rows ? rows : 1, sizeof(uint32_t));
    for (size_t i = 0; i < rows * k; i++) count[ids[i]]++;
    size_t n_used = 0;
    uint32_t r0 = 0;
    for (size_t e = 0; e < n_expert; e++) {
        row0[e] = r0;
        if (count[e]) {
            table[3 * n_used] = (uint32_t)e;
            table[3 * n_used + 1] = r0;
            table[3 * n_used + 2] = count[e];
            n_used++;
        }
        r0 += count[e];
    }
    /* groups in push order: token ascending, picks best-first */
    for (size_t t = 0; t < rows; t++)
        for (size_t j = 0; j < k; j++) {
            uint32_t e = ids[t * k + j];
            tok[row0[e] + fill[e]++] = (uint32_t)t;
        }
    /* hits per token in ascending expert order */
    memset(fill, 0, n_expert * sizeof(uint32_t));
    for (size_t t = 0; t <= rows; t++) tok_off[t] = (uint32_t)(t * k);
    /* walk experts ascending; within an expert rows are token-ascending, and a
     * token may (pathologically) appear twice -- keep push order as the reference does */
    uint32_t *gtok = (uint32_t *)malloc(sizeof(uint32_t) * (rows * k + 1));
    float *gw = (float *)malloc(sizeof(float) * (rows * k + 1));
    for (size_t t = 0; t < rows; t++)
        for (size_t j = 0; j < k; j++) {
            uint32_t e = ids[t * k + j];
            uint32_t r = row0[e] + fill[e]++;
            gtok[r] = (uint32_t)t;
            gw[r] = w[t * k + j];
        }
    for (size_t e = 0; e < n_expert; e++)
        for (uint32_t ri = 0; ri < count[e]; ri++) {
            uint32_t r = row0[e] + ri, t = gtok[r];
            hit_row[t * k + nhits[t]] = r;
            hit_w[t * k + nhits[t]] = gw[r];
            nhits[t]++;
        }
    free(count); free(row0); free(fill); free(nhits); free(gtok); free(gw);
    return n_used;
}

/* The shared expert's hit, crates/allpaka-model/src/model/prefill.rs:621-635: after the routed hits of token i,
 * h.push((total_rows + i, 1.0)); then the flattening of :658-675 (hits in list order, tok_off = running length). */
ORA_API void ora_moe_shared_hits(const uint32_t *tok_off, const uint32_t *hit_row, const float *hit_w, size_t rows,
                                 size_t total_rows, uint32_t *tok_off_out, uint32_t *hit_row_out, float *hit_w_out) {
    size_t n = 0;
    tok_off_out[0] = 0;
    for (size_t i = 0; i < rows; i++) {
        for (uint32_t h = tok_off[i]; h < tok_off[i + 1]; h++) {
            hit_row_out[n] = hit_row[h];
            hit_w_out[n] = hit_w[h];
            n++;
        }
        hit_row_out[n] = (uint32_t)(total_rows + i);
        hit_w_out[n] = 1.0f;
        n++;
        tok_off_out[i + 1] = (uint32_t)n;
    }
}

/* Gathered activations in tok order, moe.rs:348-352: dst[r,:] = src[tok[r],:]. */
ORA_API void ora_gather_rows(const float *src, const uint32_t *tok, size_t total_rows, size_t cols, float *dst) {
    for (size_t r = 0; r < total_rows; r++) memcpy(dst + r * cols, src + (size_t)tok[r] * cols, cols * sizeof(float));
}

/* ------------------------------------------------ fused contracts (f32) */

/* OP-B: x += delta (blas.rs:105-178) then h = rmsnorm_into(x) (norm.rs:193-269),
 * the order the decode loop runs them (crates/allpaka-model/src/model/decode.rs:584,764).
 * delta may be NULL (norm only). */
ORA_API void ora_add_rmsnorm_rows(float *x, const float *delta, float *h, const float *gamma, size_t n, size_t rows, float eps) {
    for (size_t r = 0; r < rows; r++) {
        float *xr = x + r * n;
        if (delta)
            for (size_t i = 0; i < n; i++) xr[i] += delta[r * n + i];
        ora_rmsnorm_into(h + r * n, xr, gamma, n, eps);
    }
}

/* ----------------------------------- fp16-activation variants (build-defined)
 * The reference keeps every activation in f32.  These variants define the fp16
 * storage forms: widen to f32, run the f32 reference arithmetic, round ONCE to
 * fp16 (RNE, ora_f32_to_f16).  For the fused add+norm the sum v = f32(x)+f32(d)
 * is stored as f16(v) but the norm uses the unrounded v. */
ORA_API void ora_add_rmsnorm_rows_f16(uint16_t *x, const uint16_t *delta, uint16_t *h, const float *gamma, size_t n, size_t rows, float eps) {
    float *v = (float *)malloc(sizeof(float) * n);
    float *o = (float *)malloc(sizeof(float) * n);
    for (size_t r = 0; r < rows; r++) {
        for (size_t i = 0; i < n; i++) {
            float a = ora_f16_to_f32(x[r * n + i]);
            if (delta) a += ora_f16_to_f32(delta[r * n + i]);
            v[i] = a;
        }
        if (delta)
            for (size_t i = 0; i < n; i++) x[r * n + i] = ora_f32_to_f16(v[i]);
        ora_rmsnorm_into(o, v, gamma, n, eps);
        for (size_t i = 0; i < n; i++) h[r * n + i] = ora_f32_to_f16(o[i]);
    }
    free(v); free(o);
}
ORA_API void ora_qknorm_rope_rows_style_f16(uint16_t *q, uint16_t *k, size_t rows, size_t n_q, size_t n_kv, size_t head_dim,
                                            const float *qw, const float *kw, const float *rope_flat, size_t half, float eps,
                                            int style) {
    size_t nq = rows * n_q * head_dim, nk = rows * n_kv * head_dim;
    float *qf = (float *)malloc(sizeof(float) * (nq ? nq : 1)), *kf = (float *)malloc(sizeof(float) * (nk ? nk : 1));
    ora_f16_to_f32_slice(q, qf, nq);
    ora_f16_to_f32_slice(k, kf, nk);
    ora_qknorm_rope_rows_style(qf, kf, rows, n_q, n_kv, head_dim, qw, kw, rope_flat, half, eps, style);
    ora_f32_to_f16_slice(qf, q, nq);
    ora_f32_to_f16_slice(kf, k, nk);
    free(qf); free(kf);
}
ORA_API void ora_qknorm_rope_rows_f16(uint16_t *q, uint16_t *k, size_t rows, size_t n_q, size_t n_kv, size_t head_dim,
                                      const float *qw, const float *kw, const float *rope_flat, size_t half, float eps) {
    ora_qknorm_rope_rows_style_f16(q, k, rows, n_q, n_kv, head_dim, qw, kw, rope_flat, half, eps, 0);
}
ORA_API void ora_swiglu_f16(uint16_t *gate, const uint16_t *up, size_t n) {
    for (size_t i = 0; i < n; i++)
        gate[i] = ora_f32_to_f16(ora_silu(ora_f16_to_f32(gate[i])) * ora_f16_to_f32(up[i]));
}
ORA_API void ora_geglu_tanh_f16(uint16_t *gate, const uint16_t *up, size_t n) {
    for (size_t i = 0; i < n; i++)
        gate[i] = ora_f32_to_f16(ora_gelu_tanh_mul(ora_f16_to_f32(gate[i]), ora_f16_to_f32(up[i])));
}
ORA_API int ora_embed_rows_f16(const uint8_t *data, size_t data_len, int fmt, size_t vocab, size_t n_in,
                               const uint32_t *ids, size_t t, uint16_t *out) {
    float *row = (float *)malloc(sizeof(float) * (n_in ? n_in : 1));
    int rc = 0;
    for (size_t i = 0; i < t && !rc; i++)
        if (ids[i] >= vocab) rc = 3;
    for (size_t i = 0; i < t && !rc; i++) {
        rc = ora_quantmat_row_into(data, data_len, fmt, vocab, n_in, ids[i], row, n_in);
        if (!rc) ora_f32_to_f16_slice(row, out + i * n_in, n_in);
    }
    free(row);
    return rc;
}
ORA_API void ora_gather_rows_f16(const uint16_t *src, const uint32_t *tok, size_t total_rows, size_t cols, uint16_t *dst) {
    for (size_t r = 0; r < total_rows; r++) memcpy(dst + r * cols, src + (size_t)tok[r] * cols, cols * sizeof(uint16_t));
}

/* ----------------------------------------------------------- KV cache store
 * KvCache::store_at (crates/allpaka-model/src/kv.rs:682-697): row i's k and v (kv_dim
 * floats each) narrowed to f16 with ops::f16::from_f32 (= f32_to_f16, RNE) at cache row
 * pos[i] of the layer's K and V planes.  Returns 1 where the reference asserts
 * "position past capacity" (nothing is written for that row). */
ORA_API int ora_kv_store_rows(const float *k, const float *v, size_t rows, size_t kv_dim, const uint32_t *pos,
                              size_t capacity, uint16_t *k_cache, uint16_t *v_cache) {
    int bad = 0;
    for (size_t i = 0; i < rows; i++) {
        if (pos[i] >= capacity) { bad = 1; continue; }
        ora_f32_to_f16_slice(k + i * kv_dim, k_cache + (size_t)pos[i] * kv_dim, kv_dim);
        ora_f32_to_f16_slice(v + i * kv_dim, v_cache + (size_t)pos[i] * kv_dim, kv_dim);
    }
    return bad;
}
/* fp16 activations: the rows are already halves; the store is a copy. */
ORA_API int ora_kv_store_rows_f16(const uint16_t *k, const uint16_t *v, size_t rows, size_t kv_dim, const uint32_t *pos,
                                  size_t capacity, uint16_t *k_cache, uint16_t *v_cache) {
    int bad = 0;
    for (size_t i = 0; i < rows; i++) {
        if (pos[i] >= capacity) { bad = 1; continue; }
        memcpy(k_cache + (size_t)pos[i] * kv_dim, k + i * kv_dim, kv_dim * 2);
        memcpy(v_cache + (size_t)pos[i] * kv_dim, v + i * kv_dim, kv_dim * 2);
    }
    return bad;
}

/* ------------------------------------------------- MoE combine + residual + norm
 * Ffn::moe_batch combine (crates/allpaka-model/src/model/moe.rs:298-333): per token, out row
 * starts at zero and gains every hit with ops::add_scaled_slice (fma(src, w, dst), blas.rs:25-102)
 * in CSR order; the caller then does ops::add_assign_slice(x, out) (decode.rs:775) and the next
 * ops::rmsnorm_into (prefill.rs:155/314).  h may be NULL (no norm). */
ORA_API void ora_moe_combine_add_rmsnorm(float *x, const float *flat, const uint32_t *tok_off, const uint32_t *hit_row,
                                         const float *hit_w, float *h, const float *gamma, size_t n, size_t rows, float eps) {
    float *out = (float *)malloc(sizeof(float) * n);
    for (size_t t = 0; t < rows; t++) {
        for (size_t i = 0; i < n; i++) out[i] = 0.0f;
        for (uint32_t k = tok_off[t]; k < tok_off[t + 1]; k++)
            ora_add_scaled_slice(out, n, flat + (size_t)hit_row[k] * n, n, hit_w[k]);
        ora_add_assign_slice(x + t * n, n, out, n);
        if (h) ora_rmsnorm_into(h + t * n, x + t * n, gamma, n, eps);
    }
    free(out);
}
/* fp16 activations (build-defined): widen, the f32 arithmetic above, one RNE rounding of x and of h;
 * the norm uses the unrounded sum, as ora_add_rmsnorm_rows_f16. */
ORA_API void ora_moe_combine_add_rmsnorm_f16(uint16_t *x, const uint16_t *flat, const uint32_t *tok_off, const uint32_t *hit_row,
                                             const float *hit_w, uint16_t *h, const float *gamma, size_t n, size_t rows, float eps) {
    float *out = (float *)malloc(sizeof(float) * n), *v = (float *)malloc(sizeof(float) * n), *o = (float *)malloc(sizeof(float) * n);
    for (size_t t = 0; t < rows; t++) {
        for (size_t i = 0; i < n; i++) out[i] = 0.0f;
        for (uint32_t k = tok_off[t]; k < tok_off[t + 1]; k++)
            for (size_t i = 0; i < n; i++) out[i] = fmaf(ora_f16_to_f32(flat[(size_t)hit_row[k] * n + i]), hit_w[k], out[i]);
        for (size_t i = 0; i < n; i++) {
            v[i] = ora_f16_to_f32(x[t * n + i]) + out[i];
            x[t * n + i] = ora_f32_to_f16(v[i]);
        }
        if (h) {
            ora_rmsnorm_into(o, v, gamma, n, eps);
            for (size_t i = 0; i < n; i++) h[t * n + i] = ora_f32_to_f16(o[i]);
        }
    }
    free(out); free(v); free(o);
}

/* Model::forward_greedy's pick (crates/allpaka-model/src/model/decode.rs:628-630):
 * (0..n).max_by(|a, b| logits[a].total_cmp(&logits[b])) -- Iterator::max_by keeps the LAST
 * maximum, so ties go to the higher index; empty -> 0. */
ORA_API uint32_t ora_argmax_last(const float *logits, size_t n) {
    if (n == 0) return 0;
    size_t best = 0;
    for (size_t i = 1; i < n; i++)
        if (total_key(logits[i]) >= total_key(logits[best])) best = i;
    return (uint32_t)best;
}
