/*
 * CPU oracle for the sparse MoE block (router -> top-k -> dispatch -> SwiGLU experts ->
 * weighted combine).
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It restates, in plain C, the CPU algorithms of the
 * reference (physics515/Mummu) for this one path so that the HIP kernels can be checked
 * against them.  Nothing in the shipped library links, calls or falls back to it; only
 * tests, the smoke check and the benchmark's cpu_baseline leg load it.
 *
 * Every function names the reference file:line it follows (paths relative to the
 * reference checkout, crates/mummu/src/...).
 *
 * Arithmetic the reference takes from third-party crates that are not in its tree
 * (burn-flex / gemm: the router Linear's summation order, softmax, top-k tie order, RmsNorm)
 * or from the platform libm (Rust f32::exp) is NOT pinned by the reference at the last
 * ulp.  For each of those this oracle fixes one deterministic definition:
 *
 *   orc_expf           - a fully specified single-precision exp (fma Horner form).  Pinned
 *                        against libm to <= 2 ulp over a dense sweep (tests).
 *   orc_router_dot     - the router logit summation order (512 strided partial sums, a
 *                        fixed tree).  Pinned against an f64 dot product (tests).  PARITY
 *                        UNPINNED versus the reference at ulp level: burn's Linear order
 *                        is third-party; the reference's own test holds it to 1e-5 only
 *                        (nn/moe.rs:2177-2202).
 *   orc_route_olmoe    - softmax/top-k/renorm as the reference's scalar restatement of its
 *                        tensor path does it (nn/moe.rs:2138-2152).  Tie order and last-ulp
 *                        softmax rounding of burn itself are PARITY UNPINNED.
 *   orc_rmsnorm        - x * rsqrt(mean(x^2) + eps) * gamma, sum of squares in the router's
 *                        512-partial order.
 *                        PARITY UNPINNED (burn RmsNorm is third-party).
 *   orc_gate_energy    - sum over the intermediate width of silu(x . gate_i)^2, squares added in row
 *                        order in f32.  PARITY UNPINNED at ulp level (the reference takes matmul,
 *                        silu, powf and sum_dim from burn, nn/moe.rs:508-521); pinned by the tests
 *                        against an f64 evaluation on the dequantized gate rows.
 *
 * Everything else (GGUF dequantizers, f16 conversion, the 8-lane dot, silu, the
 * qwen4exp router, expert FFN, ascending-expert two-rounding combine) is fully specified
 * in the reference tree and restated bit for bit.
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (see oracle/Makefile).  The
 * -ffp-contract=off flag is load-bearing: the reference rounds multiply and add
 * separately wherever it says "two roundings".
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* ggml type ids (gguf.rs:298-324). */
enum {
    ORC_F32 = 0,
    ORC_F16 = 1,
    ORC_Q4_0 = 2,
    ORC_Q4_1 = 3,
    ORC_Q5_0 = 6,
    ORC_Q5_1 = 7,
    ORC_Q8_0 = 8,
    ORC_Q4_K = 12,
    ORC_Q5_K = 13,
    ORC_Q6_K = 14,
    ORC_BF16 = 30
};

/* Status codes shared with the tests. */
enum {
    ORC_OK = 0,
    ORC_ERR_TYPE = 1,      /* dtype without a dequantizer here */
    ORC_ERR_BLOCKS = 2,    /* byte count is not whole blocks / row not whole blocks */
    ORC_ERR_TOPK = 3,      /* k outside 1..=E */
    ORC_ERR_NONFINITE = 4, /* a router logit is inf/NaN */
    ORC_ERR_RANGE = 5,     /* expert id / layer out of range */
    ORC_ERR_SHAPE = 6
};

/* ------------------------------------------------------------------------------------
 * Block geometry: gguf.rs:331-382 (block_size, bytes_per_block).
 * ---------------------------------------------------------------------------------- */
ORC_API int orc_block_size(int type) {
    switch (type) {
    case ORC_F32: case ORC_F16: case ORC_BF16: return 1;
    case ORC_Q4_0: case ORC_Q4_1: case ORC_Q5_0: case ORC_Q5_1: case ORC_Q8_0: return 32;
    case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: return 256;
    default: return 0;
    }
}

ORC_API int orc_block_bytes(int type) {
    switch (type) {
    case ORC_F32: return 4;
    case ORC_F16: case ORC_BF16: return 2;
    case ORC_Q4_0: return 18;
    case ORC_Q4_1: return 20;
    case ORC_Q5_0: return 22;
    case ORC_Q5_1: return 24;
    case ORC_Q8_0: return 34;
    case ORC_Q4_K: return 144;
    case ORC_Q5_K: return 176;
    case ORC_Q6_K: return 210;
    default: return 0;
    }
}

/* ------------------------------------------------------------------------------------
 * IEEE half -> single, exact, subnormals included: gguf.rs:1466-1468 (half::f16 -> f32).
 * Written with integer arithmetic only so it cannot depend on the host's F16C support.
 * ---------------------------------------------------------------------------------- */
static inline float bits_to_f32(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}

static inline uint32_t f32_to_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

ORC_API float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0x1Fu) { /* inf / NaN: payload moves up 13 bits */
        return bits_to_f32(sign | 0x7F800000u | (man << 13));
    }
    if (exp == 0) {
        if (man == 0) return bits_to_f32(sign);
        /* subnormal half = man * 2^-24: normalise */
        int shift = 0;
        while ((man & 0x400u) == 0) {
            man <<= 1;
            shift++;
        }
        man &= 0x3FFu;
        uint32_t e32 = (uint32_t)(127 - 15 - shift + 1);
        return bits_to_f32(sign | (e32 << 23) | (man << 13));
    }
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

static inline uint16_t rd_u16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* ------------------------------------------------------------------------------------
 * Dequantizers.  Each follows the reference function named beside it; the grouping of
 * the multiplies ((d*sc)*q, then minus the hoisted dmin*m) is the reference's.
 * ---------------------------------------------------------------------------------- */

/* gguf.rs:1535-1543 */
static void dequant_q8_0(const uint8_t *b, float *out) {
    float d = orc_f16_to_f32(rd_u16(b));
    for (int i = 0; i < 32; i++) out[i] = d * (float)(int8_t)b[2 + i];
}

/* gguf.rs:1547-1553 (Q4_0: low nibbles are elements 0..16, high 16..32, x = d*(q-8)) */
static void dequant_q4_0(const uint8_t *b, float *out) {
    float d = orc_f16_to_f32(rd_u16(b));
    for (int i = 0; i < 16; i++) {
        out[i] = d * (float)((int)(b[2 + i] & 0x0F) - 8);
        out[i + 16] = d * (float)((int)(b[2 + i] >> 4) - 8);
    }
}

/* gguf.rs:1556-1572 (Q4_1: x = d*q + m) */
static void dequant_q4_1(const uint8_t *b, float *out) {
    float d = orc_f16_to_f32(rd_u16(b));
    float m = orc_f16_to_f32(rd_u16(b + 2));
    for (int i = 0; i < 16; i++) {
        float lo = d * (float)(b[4 + i] & 0x0F);
        float hi = d * (float)(b[4 + i] >> 4);
        out[i] = lo + m;
        out[i + 16] = hi + m;
    }
}

/* gguf.rs:1575-1588 (Q5_0: fifth bits in a u32, x = d*(q-16)) */
static void dequant_q5_0(const uint8_t *b, float *out) {
    float d = orc_f16_to_f32(rd_u16(b));
    uint32_t qh = (uint32_t)b[2] | ((uint32_t)b[3] << 8) | ((uint32_t)b[4] << 16) | ((uint32_t)b[5] << 24);
    for (int i = 0; i < 16; i++) {
        int lo = (b[6 + i] & 0x0F) | (int)(((qh >> i) & 1u) << 4);
        int hi = (b[6 + i] >> 4) | (int)(((qh >> (i + 16)) & 1u) << 4);
        out[i] = d * (float)(lo - 16);
        out[i + 16] = d * (float)(hi - 16);
    }
}

/* gguf.rs:1591-1610 (Q5_1: x = d*q + m) */
static void dequant_q5_1(const uint8_t *b, float *out) {
    float d = orc_f16_to_f32(rd_u16(b));
    float m = orc_f16_to_f32(rd_u16(b + 2));
    uint32_t qh = (uint32_t)b[4] | ((uint32_t)b[5] << 8) | ((uint32_t)b[6] << 16) | ((uint32_t)b[7] << 24);
    for (int i = 0; i < 16; i++) {
        int lo = (b[8 + i] & 0x0F) | (int)(((qh >> i) & 1u) << 4);
        int hi = (b[8 + i] >> 4) | (int)(((qh >> (i + 16)) & 1u) << 4);
        float plo = d * (float)lo;
        float phi = d * (float)hi;
        out[i] = plo + m;
        out[i + 16] = phi + m;
    }
}

/* gguf.rs:1685-1697 (get_scale_min_k4) */
static void scale_min_k4(const uint8_t *s, int j, float *sc, float *m) {
    uint8_t a, b;
    if (j < 4) {
        a = s[j] & 63;
        b = s[j + 4] & 63;
    } else {
        a = (uint8_t)((s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4));
        b = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
    *sc = (float)a;
    *m = (float)b;
}

/* gguf.rs:1701-1726 */
static void dequant_q4_k(const uint8_t *b, float *out) {
    float d = orc_f16_to_f32(rd_u16(b));
    float dmin = orc_f16_to_f32(rd_u16(b + 2));
    const uint8_t *scales = b + 4;
    const uint8_t *qs = b + 16;
    for (int chunk = 0; chunk < 4; chunk++) {
        float sc1, m1, sc2, m2;
        scale_min_k4(scales, chunk * 2, &sc1, &m1);
        scale_min_k4(scales, chunk * 2 + 1, &sc2, &m2);
        const uint8_t *q = qs + chunk * 32;
        float min1 = dmin * m1;
        float min2 = dmin * m2;
        float ds1 = d * sc1;
        float ds2 = d * sc2;
        float *o = out + chunk * 64;
        for (int i = 0; i < 32; i++) {
            float p = ds1 * (float)(q[i] & 0x0F);
            o[i] = p - min1;
        }
        for (int i = 0; i < 32; i++) {
            float p = ds2 * (float)(q[i] >> 4);
            o[32 + i] = p - min2;
        }
    }
}

/* gguf.rs:1731-1765 (Q5_K: Q4_K plus 32 B of fifth bits, two qh bits per byte per chunk) */
static void dequant_q5_k(const uint8_t *b, float *out) {
    float d = orc_f16_to_f32(rd_u16(b));
    float dmin = orc_f16_to_f32(rd_u16(b + 2));
    const uint8_t *scales = b + 4;
    const uint8_t *qh = b + 16;
    const uint8_t *qs = b + 48;
    for (int chunk = 0; chunk < 4; chunk++) {
        float sc1, m1, sc2, m2;
        scale_min_k4(scales, chunk * 2, &sc1, &m1);
        scale_min_k4(scales, chunk * 2 + 1, &sc2, &m2);
        const uint8_t *q = qs + chunk * 32;
        uint8_t u1 = (uint8_t)(1u << (2 * chunk));
        uint8_t u2 = (uint8_t)(2u << (2 * chunk));
        float min1 = dmin * m1;
        float min2 = dmin * m2;
        float ds1 = d * sc1;
        float ds2 = d * sc2;
        float *o = out + chunk * 64;
        for (int i = 0; i < 32; i++) {
            int v = (q[i] & 0x0F) + ((qh[i] & u1) ? 16 : 0);
            float p = ds1 * (float)v;
            o[i] = p - min1;
        }
        for (int i = 0; i < 32; i++) {
            int v = (q[i] >> 4) + ((qh[i] & u2) ? 16 : 0);
            float p = ds2 * (float)v;
            o[32 + i] = p - min2;
        }
    }
}

/* gguf.rs:1769-1797 (Q6_K: 128 B ql + 64 B qh + 16 i8 scales + f16 d; x = d*sc*(q-32)) */
static void dequant_q6_k(const uint8_t *b, float *out) {
    const uint8_t *ql = b;
    const uint8_t *qh = b + 128;
    const int8_t *sc = (const int8_t *)(b + 192);
    float d = orc_f16_to_f32(rd_u16(b + 208));
    for (int half = 0; half < 2; half++) {
        const uint8_t *l = ql + half * 64;
        const uint8_t *h = qh + half * 32;
        const int8_t *s = sc + half * 8;
        float *o = out + half * 128;
        for (int i = 0; i < 32; i++) {
            int is = i / 16;
            int q1 = (int)((l[i] & 0x0F) | (((h[i] >> 0) & 3) << 4)) - 32;
            int q2 = (int)((l[i + 32] & 0x0F) | (((h[i] >> 2) & 3) << 4)) - 32;
            int q3 = (int)((l[i] >> 4) | (((h[i] >> 4) & 3) << 4)) - 32;
            int q4 = (int)((l[i + 32] >> 4) | (((h[i] >> 6) & 3) << 4)) - 32;
            o[i] = d * (float)s[is] * (float)q1;
            o[i + 32] = d * (float)s[is + 2] * (float)q2;
            o[i + 64] = d * (float)s[is + 4] * (float)q3;
            o[i + 96] = d * (float)s[is + 6] * (float)q4;
        }
    }
}

/* gguf.rs:1403-1463: whole blocks only, empty input refused. */
ORC_API int orc_dequantize(int type, const uint8_t *bytes, size_t nbytes, float *out) {
    int bpb = orc_block_bytes(type);
    int bs = orc_block_size(type);
    if (bpb == 0) return ORC_ERR_TYPE;
    if (nbytes == 0 || nbytes % (size_t)bpb != 0) return ORC_ERR_BLOCKS;
    size_t blocks = nbytes / (size_t)bpb;
    for (size_t i = 0; i < blocks; i++) {
        const uint8_t *b = bytes + i * (size_t)bpb;
        float *o = out + i * (size_t)bs;
        switch (type) {
        case ORC_F32: *o = bits_to_f32((uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) | ((uint32_t)b[3] << 24)); break;
        case ORC_F16: *o = orc_f16_to_f32(rd_u16(b)); break;
        case ORC_BF16: *o = bits_to_f32((uint32_t)rd_u16(b) << 16); break;
        case ORC_Q4_0: dequant_q4_0(b, o); break;
        case ORC_Q4_1: dequant_q4_1(b, o); break;
        case ORC_Q5_0: dequant_q5_0(b, o); break;
        case ORC_Q5_1: dequant_q5_1(b, o); break;
        case ORC_Q8_0: dequant_q8_0(b, o); break;
        case ORC_Q4_K: dequant_q4_k(b, o); break;
        case ORC_Q5_K: dequant_q5_k(b, o); break;
        case ORC_Q6_K: dequant_q6_k(b, o); break;
        default: return ORC_ERR_TYPE;
        }
    }
    return ORC_OK;
}

/* ------------------------------------------------------------------------------------
 * experts.rs:463-478 - inner product with eight independent lane accumulators over
 * chunks of 8, combined ((a0+a4)+(a1+a5))+((a2+a6)+(a3+a7)), then a scalar tail.
 * Multiply and add round separately (Rust does not contract).
 * ---------------------------------------------------------------------------------- */
ORC_API float orc_dot(const float *a, const float *b, size_t n) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    size_t chunks = n / 8;
    for (size_t c = 0; c < chunks; c++) {
        for (int l = 0; l < 8; l++) {
            float p = a[c * 8 + l] * b[c * 8 + l];
            acc[l] = acc[l] + p;
        }
    }
    float s = ((acc[0] + acc[4]) + (acc[1] + acc[5])) + ((acc[2] + acc[6]) + (acc[3] + acc[7]));
    for (size_t i = chunks * 8; i < n; i++) {
        float p = a[i] * b[i];
        s = s + p;
    }
    return s;
}

/* ------------------------------------------------------------------------------------
 * Deterministic expf.  The reference calls Rust's f32::exp (platform libm), which is not
 * the same function on every host; this one is specified operation by operation so the
 * CPU oracle and the GPU kernels can agree bit for bit:
 *   n  = round-to-nearest-even(x * log2(e))          (magic-constant add/sub)
 *   r  = fma(-n, ln2_lo, fma(-n, ln2_hi, x))          (Cody-Waite)
 *   p  = 1 + r + r^2 * P5(r)                           (Horner, every step one fmaf)
 *   result = p * 2^n, the scale applied in two exact power-of-two factors so that
 *            subnormal results round once.
 * x >= 88.7228394 -> +inf, x < -103.9720840 -> +0, NaN -> NaN.
 * ---------------------------------------------------------------------------------- */
ORC_API float orc_expf(float x) {
    if (x != x) return x;
    if (x >= 88.7228394f) return INFINITY;
    if (x < -103.9720840f) return 0.0f;
    const float LOG2E = 1.44269502f;
    const float LN2_HI = 0.693359375f;
    const float LN2_LO = -2.12194440e-4f;
    const float MAGIC = 12582912.0f; /* 1.5 * 2^23 */
    float t = fmaf(x, LOG2E, MAGIC);
    float n = t - MAGIC;
    float r = fmaf(-n, LN2_HI, x);
    r = fmaf(-n, LN2_LO, r);
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    float r2 = r * r;
    float y = fmaf(p, r2, r);
    y = y + 1.0f;
    int ni = (int)n;
    /* split 2^n = 2^a * 2^b with both factors normal */
    int a = ni / 2;
    int b = ni - a;
    float sa = bits_to_f32((uint32_t)(a + 127) << 23);
    float sb = bits_to_f32((uint32_t)(b + 127) << 23);
    y = y * sa;
    y = y * sb;
    return y;
}

/* experts.rs:485-487 and nn/moe.rs:2095-2097: x / (1 + e^-x). */
ORC_API float orc_silu(float x) {
    float e = orc_expf(-x);
    float den = 1.0f + e;
    return x / den;
}

/* ------------------------------------------------------------------------------------
 * Router, qwen4exp flavour: experts.rs:502-582.
 *   softmax_row: shift by max, f64 normaliser, multiply by the f32 reciprocal (:502-515)
 *   top-k: insertion into a <=k list, strictly-greater wins, so a lower id keeps a tie and
 *          equal slots ascend by id (:557-573)
 *   renormalize: f64 sum narrowed to f32, clamped below at 2^-14, divide (:520-526)
 * Non-finite logits and k outside 1..=E are refused (:542-553); *bad_index receives the
 * flat index of the first non-finite logit.
 * ---------------------------------------------------------------------------------- */
#define ORC_WEIGHT_SUM_FLOOR (1.0f / 16384.0f) /* experts.rs:74 */

static void topk_insert(const float *probs, int n_experts, int k, uint32_t *ids, float *w) {
    int len = 0;
    for (int id = 0; id < n_experts; id++) {
        float p = probs[id];
        if (len == k && p <= w[k - 1]) continue;
        /* partition_point(|q| q >= p): first position whose prob is < p */
        int pos = 0;
        while (pos < len && w[pos] >= p) pos++;
        int last = (len < k) ? len : k - 1;
        for (int j = last; j > pos; j--) {
            w[j] = w[j - 1];
            ids[j] = ids[j - 1];
        }
        w[pos] = p;
        ids[pos] = (uint32_t)id;
        if (len < k) len++;
    }
}

/* experts.rs:520-526: divide by the f64-accumulated sum, clamped below at 2^-14. */
ORC_API void orc_renormalize_ggml(float *top, int k) {
    double wsum = 0.0;
    for (int s = 0; s < k; s++) wsum += (double)top[s];
    float fs = (float)wsum;
    if (!(fs > ORC_WEIGHT_SUM_FLOOR)) fs = ORC_WEIGHT_SUM_FLOOR; /* f32::max(sum, floor) */
    for (int s = 0; s < k; s++) top[s] = top[s] / fs;
}

ORC_API int orc_route_ggml(const float *logits, size_t n, int n_experts, int k, uint32_t *ids,
                           float *weights, int64_t *bad_index) {
    if (n_experts <= 0 || k <= 0 || k > n_experts) return ORC_ERR_TOPK;
    for (size_t i = 0; i < n * (size_t)n_experts; i++) {
        if (!isfinite(logits[i])) {
            if (bad_index) *bad_index = (int64_t)i;
            return ORC_ERR_NONFINITE;
        }
    }
    float *probs = (float *)malloc(sizeof(float) * (size_t)n_experts);
    for (size_t t = 0; t < n; t++) {
        const float *row = logits + t * (size_t)n_experts;
        float max = -INFINITY;
        for (int e = 0; e < n_experts; e++) max = (row[e] > max) ? row[e] : max;
        double sum = 0.0;
        for (int e = 0; e < n_experts; e++) {
            float v = orc_expf(row[e] - max);
            sum += (double)v;
            probs[e] = v;
        }
        float scale = (float)(1.0 / sum);
        for (int e = 0; e < n_experts; e++) probs[e] = probs[e] * scale;
        uint32_t *tid = ids + t * (size_t)k;
        float *tw = weights + t * (size_t)k;
        topk_insert(probs, n_experts, k, tid, tw);
        orc_renormalize_ggml(tw, k);
    }
    free(probs);
    return ORC_OK;
}

/* ------------------------------------------------------------------------------------
 * Router, SparseMoe flavour: nn/moe.rs:144-150 as spelled out by the reference's own
 * scalar restatement, nn/moe.rs:2138-2152:
 *   max-shifted exp, f32 sequential total, probs = exp/total; stable descending order
 *   (so the lower id is first among equals); weights = probs (divided by their f32
 *   sequential sum over the picked slots iff norm_topk_prob).
 * Non-finite logits are refused here too (the reference's sort would panic on NaN).
 * ---------------------------------------------------------------------------------- */
ORC_API int orc_route_olmoe(const float *logits, size_t n, int n_experts, int k, int norm_topk_prob,
                            uint32_t *ids, float *weights, int64_t *bad_index) {
    if (n_experts <= 0 || k <= 0 || k > n_experts) return ORC_ERR_TOPK;
    for (size_t i = 0; i < n * (size_t)n_experts; i++) {
        if (!isfinite(logits[i])) {
            if (bad_index) *bad_index = (int64_t)i;
            return ORC_ERR_NONFINITE;
        }
    }
    float *probs = (float *)malloc(sizeof(float) * (size_t)n_experts);
    for (size_t t = 0; t < n; t++) {
        const float *row = logits + t * (size_t)n_experts;
        float max = -INFINITY;
        for (int e = 0; e < n_experts; e++) max = (row[e] > max) ? row[e] : max;
        float total = 0.0f;
        for (int e = 0; e < n_experts; e++) {
            probs[e] = orc_expf(row[e] - max);
            total = total + probs[e];
        }
        for (int e = 0; e < n_experts; e++) probs[e] = probs[e] / total;
        uint32_t *tid = ids + t * (size_t)k;
        float *tw = weights + t * (size_t)k;
        topk_insert(probs, n_experts, k, tid, tw);
        if (norm_topk_prob) {
            float denom = 0.0f;
            for (int s = 0; s < k; s++) denom = denom + tw[s];
            for (int s = 0; s < k; s++) tw[s] = tw[s] / denom;
        }
    }
    free(probs);
    return ORC_OK;
}

/* ------------------------------------------------------------------------------------
 * Router logits.  Reference: a bias-free Linear, logits[t,e] = sum_i x[t,i] * W[e,i]
 * (nn/moe.rs:139; weight in GGUF order ffn_gate_inp ne=[H,E], i.e. row-major [E,H],
 * models/olmoe.rs:338-339).  The reference's summation order lives in the third-party
 * gemm crate; this build's fixed order (mirrored exactly by the HIP router kernel) is:
 *
 *   512 partial sums; element i goes to partial (i mod 512), partials accumulate with one
 *   fma per element in ascending i.  View the partials as 64 groups of 8 consecutive
 *   ones: each group folds as ((a0+a4)+(a1+a5))+((a2+a6)+(a3+a7)) - the reference dot's
 *   own final fold, experts.rs:473 - and the 64 group sums fold pairwise over adjacent
 *   groups: s[l] += s[l+1] for even l, then s[l] += s[l+2] for l % 4 == 0, ... up to +32.
 *
 * The weight is converted to f32 exactly (F32/F16/BF16) before the fma.
 * ---------------------------------------------------------------------------------- */
static float load_as_f32(const void *w, int type, size_t i) {
    switch (type) {
    case ORC_F32: return ((const float *)w)[i];
    case ORC_F16: return orc_f16_to_f32(((const uint16_t *)w)[i]);
    default: return bits_to_f32((uint32_t)((const uint16_t *)w)[i] << 16);
    }
}

ORC_API float orc_router_dot(const float *x, const void *w, int wtype, size_t row_offset, size_t n) {
    float acc[512];
    for (int i = 0; i < 512; i++) acc[i] = 0.0f;
    for (size_t i = 0; i < n; i++) {
        float wv = load_as_f32(w, wtype, row_offset + i);
        acc[i & 511] = fmaf(x[i], wv, acc[i & 511]);
    }
    float s[64];
    for (int l = 0; l < 64; l++) {
        const float *a = acc + l * 8;
        s[l] = ((a[0] + a[4]) + (a[1] + a[5])) + ((a[2] + a[6]) + (a[3] + a[7]));
    }
    for (int off = 1; off < 64; off <<= 1) /* pairwise tree over adjacent lane sums */
        for (int l = 0; l < 64; l += 2 * off) s[l] = s[l] + s[l + off];
    return s[0];
}

ORC_API int orc_router_logits(const float *x, const void *w, int wtype, size_t n, size_t hidden,
                              int n_experts, float *logits) {
    if (wtype != ORC_F32 && wtype != ORC_F16 && wtype != ORC_BF16) return ORC_ERR_TYPE;
#pragma omp parallel for schedule(static)
    for (long t = 0; t < (long)n; t++)
        for (int e = 0; e < n_experts; e++)
            logits[(size_t)t * (size_t)n_experts + (size_t)e] =
                orc_router_dot(x + (size_t)t * hidden, w, wtype, (size_t)e * hidden, hidden);
    return ORC_OK;
}

/* ------------------------------------------------------------------------------------
 * experts.rs:329-348, 401-457: W_e . x for n rows.  out[t*out_dim + r] = dot(row r, x_t)
 * with rows dequantized chunk by chunk (the chunking does not change a bit, :1316-1353,
 * so rows are dequantized one at a time here).  bytes points at ONE expert's rows.
 * ---------------------------------------------------------------------------------- */
ORC_API int orc_matvec(int type, const uint8_t *bytes, size_t in_dim, size_t out_dim, const float *xs,
                       size_t n, float *out) {
    int bs = orc_block_size(type), bpb = orc_block_bytes(type);
    if (bs == 0) return ORC_ERR_TYPE;
    if (in_dim == 0 || in_dim % (size_t)bs != 0) return ORC_ERR_BLOCKS; /* experts.rs:150-154 */
    size_t row_bytes = in_dim / (size_t)bs * (size_t)bpb;
    int rc = ORC_OK;
#pragma omp parallel
    {
        float *row = (float *)malloc(sizeof(float) * in_dim);
#pragma omp for schedule(static)
        for (long r = 0; r < (long)out_dim; r++) {
            int e = orc_dequantize(type, bytes + (size_t)r * row_bytes, row_bytes, row);
            if (e != ORC_OK) {
#pragma omp atomic write
                rc = e;
                continue;
            }
            for (size_t t = 0; t < n; t++) out[t * out_dim + (size_t)r] = orc_dot(row, xs + t * in_dim, in_dim);
        }
        free(row);
    }
    return rc;
}

/* One layer's expert banks in GGUF order (expert-major, row-major, whole blocks per row):
 * gate/up ne=[H, I, E], down ne=[I, H, E] (experts.rs:122-136, nn/moe.rs:22-30). */
typedef struct {
    int hidden, inter, n_experts;
    int gate_type, up_type, down_type;
    const uint8_t *gate, *up, *down;
} orc_banks;

static size_t bank_row_bytes(int type, size_t in_dim) {
    return in_dim / (size_t)orc_block_size(type) * (size_t)orc_block_bytes(type);
}

static int banks_check(const orc_banks *b) {
    int types[3] = {b->gate_type, b->up_type, b->down_type};
    size_t ins[3] = {(size_t)b->hidden, (size_t)b->hidden, (size_t)b->inter};
    if (b->hidden < 1 || b->inter < 1 || b->n_experts < 1) return ORC_ERR_SHAPE;
    for (int i = 0; i < 3; i++) {
        int bs = orc_block_size(types[i]);
        if (bs == 0) return ORC_ERR_TYPE;
        if (ins[i] % (size_t)bs != 0) return ORC_ERR_BLOCKS;
    }
    return ORC_OK;
}

/* experts.rs:781-845 (ffn) with the diagnostic activation emulation off (its default):
 * down(silu(gate.x) * (up.x)) over n rows; xs [n x H] -> out [n x H]. */
ORC_API int orc_expert_ffn(const orc_banks *b, int expert, const float *xs, size_t n, float *out) {
    int rc = banks_check(b);
    if (rc != ORC_OK) return rc;
    if (expert < 0 || expert >= b->n_experts) return ORC_ERR_RANGE;
    if (n == 0) return ORC_OK;
    size_t H = (size_t)b->hidden, I = (size_t)b->inter;
    const uint8_t *g = b->gate + (size_t)expert * I * bank_row_bytes(b->gate_type, H);
    const uint8_t *u = b->up + (size_t)expert * I * bank_row_bytes(b->up_type, H);
    const uint8_t *d = b->down + (size_t)expert * H * bank_row_bytes(b->down_type, I);
    float *hid = (float *)malloc(sizeof(float) * n * I);
    float *upv = (float *)malloc(sizeof(float) * n * I);
    rc = orc_matvec(b->gate_type, g, H, I, xs, n, hid);
    if (rc == ORC_OK) rc = orc_matvec(b->up_type, u, H, I, xs, n, upv);
    if (rc == ORC_OK) {
        for (size_t i = 0; i < n * I; i++) hid[i] = orc_silu(hid[i]) * upv[i];
        rc = orc_matvec(b->down_type, d, I, H, hid, n, out);
    }
    free(hid);
    free(upv);
    return rc;
}

/* nn/packed_gemv.rs:370-451 (packed_gemv_kernel at split 1) == the dequantize-then-matmul form it is
 * tested against (:1593-1624): y[r][n] = sum over k, in order, of float(q(k, n)) * (x[r][k] * scale(k, n/32)),
 * the inner product rounded, the outer product rounded, then added.  Layout pack.rs:940-985: values two's
 * complement in `bits` (4 or 8) bits, element j of a u32 word at bits j*bits, words along N; one f32 scale
 * per (k, 32 consecutive n).  xs [m x K] -> out [m x N]. */
ORC_API int orc_q4s_gemv(const uint32_t *words, const float *scales, int k_len, int n, int bits, const float *xs,
                         size_t m, float *out) {
    if (bits != 4 && bits != 8) return ORC_ERR_TYPE;
    if (k_len < 1 || n < 1 || n % 32 != 0) return ORC_ERR_BLOCKS;
    int per = 32 / bits;
    size_t n_words = (size_t)n / (size_t)per, n_blocks = (size_t)n / 32;
    for (size_t r = 0; r < m; r++) {
        for (int c = 0; c < n; c++) {
            float acc = 0.0f;
            for (int k = 0; k < k_len; k++) {
                uint32_t word = words[(size_t)k * n_words + (size_t)(c / per)];
                uint32_t raw = (word >> ((uint32_t)(c % per) * (uint32_t)bits)) & ((1u << bits) - 1u);
                int q = (int)raw;
                if (raw >= (1u << (bits - 1))) q -= (1 << bits);
                float x_scaled = xs[r * (size_t)k_len + (size_t)k] * scales[(size_t)k * n_blocks + (size_t)(c / 32)];
                float prod = (float)q * x_scaled;
                acc = acc + prod;
            }
            out[r * (size_t)n + (size_t)c] = acc;
        }
    }
    return ORC_OK;
}

/* nn/moe.rs:508-521 (DeviceExpert::gate_energy): per row, the sum over the intermediate width of
 * silu(x . gate_i)^2 - the gate product only, on the dequantized gate rows; the squares are added in
 * row order i = 0, 1, ... in f32.  xs [n x H] -> out [n]. */
ORC_API int orc_gate_energy(const orc_banks *b, int expert, const float *xs, size_t n, float *out) {
    int rc = banks_check(b);
    if (rc != ORC_OK) return rc;
    if (expert < 0 || expert >= b->n_experts) return ORC_ERR_RANGE;
    if (n == 0) return ORC_OK;
    size_t H = (size_t)b->hidden, I = (size_t)b->inter;
    const uint8_t *g = b->gate + (size_t)expert * I * bank_row_bytes(b->gate_type, H);
    float *hid = (float *)malloc(sizeof(float) * n * I);
    rc = orc_matvec(b->gate_type, g, H, I, xs, n, hid);
    if (rc == ORC_OK) {
        for (size_t t = 0; t < n; t++) {
            float e = 0.0f;
            for (size_t i = 0; i < I; i++) {
                float s = orc_silu(hid[t * I + i]);
                float sq = s * s;
                e = e + sq;
            }
            out[t] = e;
        }
    }
    free(hid);
    return rc;
}

/* ------------------------------------------------------------------------------------
 * experts.rs:1092-1150 (apply_routing) == nn/moe.rs:296-328 (run_local) ==
 * nn/moe.rs:1545-1607 (run_layer): bucket (token, weight) by expert in token-major,
 * slot-minor order; every hit expert runs once on exactly its rows; results are
 * scatter-added in ASCENDING EXPERT ID with two roundings (weighted = w*v; o += weighted).
 * hits (optional, [E]) accumulates rows served per expert (nn/moe.rs:1562-1564).
 * ---------------------------------------------------------------------------------- */
ORC_API int orc_apply_routing(const orc_banks *b, const uint32_t *ids, const float *weights, size_t n, int k,
                              const float *xs, float *out, uint64_t *hits) {
    int rc = banks_check(b);
    if (rc != ORC_OK) return rc;
    size_t H = (size_t)b->hidden;
    int E = b->n_experts;
    for (size_t i = 0; i < n * (size_t)k; i++)
        if (ids[i] >= (uint32_t)E) return ORC_ERR_RANGE;
    memset(out, 0, sizeof(float) * n * H);
    size_t *count = (size_t *)calloc((size_t)E, sizeof(size_t));
    for (size_t i = 0; i < n * (size_t)k; i++) count[ids[i]]++;
    for (int e = 0; e < E; e++) {
        size_t m = count[e];
        if (m == 0) continue;
        if (hits) hits[e] += (uint64_t)m;
        size_t *rows = (size_t *)malloc(sizeof(size_t) * m);
        float *w = (float *)malloc(sizeof(float) * m);
        float *gathered = (float *)malloc(sizeof(float) * m * H);
        float *y = (float *)malloc(sizeof(float) * m * H);
        size_t j = 0;
        for (size_t t = 0; t < n; t++)
            for (int s = 0; s < k; s++)
                if (ids[t * (size_t)k + (size_t)s] == (uint32_t)e) {
                    rows[j] = t;
                    w[j] = weights[t * (size_t)k + (size_t)s];
                    memcpy(gathered + j * H, xs + t * H, sizeof(float) * H);
                    j++;
                }
        rc = orc_expert_ffn(b, e, gathered, m, y);
        if (rc == ORC_OK) {
            for (size_t i = 0; i < m; i++) {
                float *dst = out + rows[i] * H;
                for (size_t c = 0; c < H; c++) {
                    float weighted = w[i] * y[i * H + c];
                    dst[c] = dst[c] + weighted;
                }
            }
        }
        free(rows);
        free(w);
        free(gathered);
        free(y);
        if (rc != ORC_OK) break;
    }
    free(count);
    return rc;
}

/* ------------------------------------------------------------------------------------
 * The whole block.  flavour 0 = SparseMoe / SparseMoePerExpert (nn/moe.rs:116-177,
 * 214-328): router Linear -> orc_route_olmoe -> routed experts.  flavour 1 = qwen4exp
 * routed_moe on these logits (experts.rs:1066-1076), which always renormalises.
 * router_w is row-major [E, H] in router_type (F32/F16/BF16).
 * ids_out/w_out ([n*k], optional) receive the routing; logits_out ([n*E], optional).
 * ---------------------------------------------------------------------------------- */
ORC_API int orc_moe_forward(const orc_banks *b, const void *router_w, int router_type, int flavour, int k,
                            int norm_topk_prob, const float *xs, size_t n, float *out, uint32_t *ids_out,
                            float *w_out, float *logits_out, uint64_t *hits) {
    int rc = banks_check(b);
    if (rc != ORC_OK) return rc;
    int E = b->n_experts;
    if (k < 1 || k > E) return ORC_ERR_TOPK;
    float *logits = (float *)malloc(sizeof(float) * n * (size_t)E);
    uint32_t *ids = (uint32_t *)malloc(sizeof(uint32_t) * n * (size_t)k);
    float *w = (float *)malloc(sizeof(float) * n * (size_t)k);
    int64_t bad = -1;
    rc = orc_router_logits(xs, router_w, router_type, n, (size_t)b->hidden, E, logits);
    if (rc == ORC_OK)
        rc = flavour == 1 ? orc_route_ggml(logits, n, E, k, ids, w, &bad)
                          : orc_route_olmoe(logits, n, E, k, norm_topk_prob, ids, w, &bad);
    if (rc == ORC_OK) rc = orc_apply_routing(b, ids, w, n, k, xs, out, hits);
    if (rc == ORC_OK) {
        if (ids_out) memcpy(ids_out, ids, sizeof(uint32_t) * n * (size_t)k);
        if (w_out) memcpy(w_out, w, sizeof(float) * n * (size_t)k);
        if (logits_out) memcpy(logits_out, logits, sizeof(float) * n * (size_t)E);
    }
    free(logits);
    free(ids);
    free(w);
    return rc;
}

/* ------------------------------------------------------------------------------------
 * nn/moe.rs:151-176, the dense-mask formulation: EVERY expert runs on EVERY token and
 * the per-token weight row (probability on the top-k, exact zero elsewhere) scales the
 * results away; experts are summed in ascending id.  Same mathematics as the routed
 * path, E/k times the work - this is the algorithm behind the reference's published
 * 0.76 s/token and is what the CPU baseline times for the f32 configuration.
 * ---------------------------------------------------------------------------------- */
ORC_API int orc_moe_forward_dense_mask(const orc_banks *b, const void *router_w, int router_type, int k,
                                       int norm_topk_prob, const float *xs, size_t n, float *out) {
    int rc = banks_check(b);
    if (rc != ORC_OK) return rc;
    int E = b->n_experts;
    size_t H = (size_t)b->hidden;
    if (k < 1 || k > E) return ORC_ERR_TOPK;
    float *logits = (float *)malloc(sizeof(float) * n * (size_t)E);
    uint32_t *ids = (uint32_t *)malloc(sizeof(uint32_t) * n * (size_t)k);
    float *w = (float *)malloc(sizeof(float) * n * (size_t)k);
    float *dense_w = (float *)calloc(n * (size_t)E, sizeof(float));
    float *y = (float *)malloc(sizeof(float) * n * H);
    rc = orc_router_logits(xs, router_w, router_type, n, H, E, logits);
    if (rc == ORC_OK) rc = orc_route_olmoe(logits, n, E, k, norm_topk_prob, ids, w, NULL);
    if (rc == ORC_OK) {
        for (size_t t = 0; t < n; t++)
            for (int s = 0; s < k; s++) dense_w[t * (size_t)E + ids[t * (size_t)k + (size_t)s]] = w[t * (size_t)k + (size_t)s];
        memset(out, 0, sizeof(float) * n * H);
        for (int e = 0; e < E && rc == ORC_OK; e++) {
            rc = orc_expert_ffn(b, e, xs, n, y);
            if (rc != ORC_OK) break;
            for (size_t t = 0; t < n; t++) {
                float we = dense_w[t * (size_t)E + (size_t)e];
                for (size_t c = 0; c < H; c++) {
                    float scaled = y[t * H + c] * we;
                    out[t * H + c] = out[t * H + c] + scaled;
                }
            }
        }
    }
    free(logits);
    free(ids);
    free(w);
    free(dense_w);
    free(y);
    return rc;
}

/* ------------------------------------------------------------------------------------
 * Layer wrapper, models/olmoe.rs:566-572 and 1742-1755: h2 = RmsNorm(x; gamma, eps),
 * x = x + MoE(h2).  burn's RmsNorm is x * rsqrt(mean(x^2) + eps) * gamma; its rounding is
 * third-party (PARITY UNPINNED).  Fixed here: the sum of squares in the same 512-partial
 * fma order as the router logits (orc_router_dot of the row with itself), mean = sum / H,
 * r = 1/sqrt(mean + eps) (correctly rounded sqrt and divide), y = (x * r) * gamma.
 * ---------------------------------------------------------------------------------- */
ORC_API void orc_rmsnorm(const float *x, const float *gamma, float eps, size_t n, size_t hidden, float *out) {
    for (size_t t = 0; t < n; t++) {
        const float *row = x + t * hidden;
        float ss = orc_router_dot(row, row, ORC_F32, 0, hidden);
        float mean = ss / (float)hidden;
        float r = 1.0f / sqrtf(mean + eps);
        for (size_t i = 0; i < hidden; i++) {
            float v = row[i] * r;
            out[t * hidden + i] = v * gamma[i];
        }
    }
}

/* x <- x + MoE(RmsNorm(x)) for n_layers layers (in place on x, [n x H]).  banks, routers,
 * gammas are arrays of n_layers entries; all routers share router_type. */
ORC_API int orc_layer_stack(const orc_banks *banks, const void *const *routers, int router_type,
                            const float *const *gammas, float eps, int n_layers, int flavour, int k,
                            int norm_topk_prob, float *x, size_t n, uint32_t *ids_out) {
    size_t H = (size_t)banks[0].hidden;
    float *h2 = (float *)malloc(sizeof(float) * n * H);
    float *moe = (float *)malloc(sizeof(float) * n * H);
    int rc = ORC_OK;
    for (int l = 0; l < n_layers && rc == ORC_OK; l++) {
        orc_rmsnorm(x, gammas[l], eps, n, H, h2);
        rc = orc_moe_forward(&banks[l], routers[l], router_type, flavour, k, norm_topk_prob, h2, n, moe,
                             ids_out ? ids_out + (size_t)l * n * (size_t)k : NULL, NULL, NULL, NULL);
        if (rc == ORC_OK)
            for (size_t i = 0; i < n * H; i++) x[i] = x[i] + moe[i];
    }
    free(h2);
    free(moe);
    return rc;
}

/* ------------------------------------------------------------------------------------
 * Tolerance reference, following the reference's own test oracle
 * (experts.rs:1244-1271, 1466-1532): the block in f64 over the whole dequantized
 * matrices for a GIVEN routing, plus `mag`, the root-sum-square magnitude of the terms of
 * each output (weighted like the output), against which relative closeness is measured.
 * The hidden activation is computed in f64 and narrowed to f32 as that test does (:1510).
 * ---------------------------------------------------------------------------------- */
ORC_API int orc_moe_ref_f64(const orc_banks *b, const uint32_t *ids, const float *weights, size_t n, int k,
                            const float *xs, double *want, double *mag) {
    int rc = banks_check(b);
    if (rc != ORC_OK) return rc;
    size_t H = (size_t)b->hidden, I = (size_t)b->inter;
    int E = b->n_experts;
    for (size_t i = 0; i < n * (size_t)k; i++)
        if (ids[i] >= (uint32_t)E) return ORC_ERR_RANGE;
    memset(want, 0, sizeof(double) * n * H);
    memset(mag, 0, sizeof(double) * n * H);
    size_t gr = bank_row_bytes(b->gate_type, H), ur = bank_row_bytes(b->up_type, H), dr = bank_row_bytes(b->down_type, I);
    float *wg = (float *)malloc(sizeof(float) * I * H);
    float *wu = (float *)malloc(sizeof(float) * I * H);
    float *wd = (float *)malloc(sizeof(float) * H * I);
    float *hid = (float *)malloc(sizeof(float) * I);
    for (int e = 0; e < E && rc == ORC_OK; e++) {
        int used = 0;
        for (size_t i = 0; i < n * (size_t)k && !used; i++) used = ids[i] == (uint32_t)e;
        if (!used) continue;
        rc = orc_dequantize(b->gate_type, b->gate + (size_t)e * I * gr, I * gr, wg);
        if (rc == ORC_OK) rc = orc_dequantize(b->up_type, b->up + (size_t)e * I * ur, I * ur, wu);
        if (rc == ORC_OK) rc = orc_dequantize(b->down_type, b->down + (size_t)e * H * dr, H * dr, wd);
        if (rc != ORC_OK) break;
        for (size_t t = 0; t < n; t++)
            for (int s = 0; s < k; s++) {
                if (ids[t * (size_t)k + (size_t)s] != (uint32_t)e) continue;
                double weight = (double)weights[t * (size_t)k + (size_t)s];
                const float *x = xs + t * H;
#pragma omp parallel for schedule(static)
                for (long j = 0; j < (long)I; j++) {
                    double g = 0.0, u = 0.0;
                    for (size_t i = 0; i < H; i++) {
                        g += (double)wg[(size_t)j * H + i] * (double)x[i];
                        u += (double)wu[(size_t)j * H + i] * (double)x[i];
                    }
                    hid[j] = (float)(g / (1.0 + exp(-g)) * u);
                }
#pragma omp parallel for schedule(static)
                for (long c = 0; c < (long)H; c++) {
                    double o = 0.0, m2 = 0.0;
                    for (size_t j = 0; j < I; j++) {
                        double term = (double)wd[(size_t)c * I + j] * (double)hid[j];
                        o += term;
                        m2 += term * term;
                    }
                    double scaled = weight * o;
                    want[t * H + (size_t)c] += scaled;
                    double scaled_mag = weight * sqrt(m2);
                    mag[t * H + (size_t)c] += scaled_mag;
                }
            }
    }
    free(wg);
    free(wu);
    free(wd);
    free(hid);
    return rc;
}
