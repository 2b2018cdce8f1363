/* CPU oracle (TEST INFRASTRUCTURE) - see p1a_oracle.h for scope and for what pins each function. */
#include "p1a_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- f16 <-> f32, IEEE round-to-nearest-even, subnormals kept (the device uses v_cvt_f16_f32 in RNE mode;
 * the reference uses __float2half, src/fast/kv_q8.cuh:25,48) ---- */
uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t a = x & 0x7fffffffu;
    if (a >= 0x7f800000u) return (uint16_t) (sign | 0x7c00u | (a > 0x7f800000u ? 0x200u | ((a >> 13) & 0x3ffu) : 0u));
    if (a >= 0x477ff000u) return (uint16_t) (sign | 0x7c00u);           /* rounds to >= 65520 -> inf */
    if (a >= 0x38800000u) {                                           /* normal half */
        const uint32_t m = a - 0x38000000u;                           /* rebias exponent 127 -> 15 */
        const uint32_t r = m + 0xfffu + ((m >> 13) & 1u);             /* RNE on the 13 dropped bits */
        return (uint16_t) (sign | (r >> 13));
    }
    if (a < 0x33000000u) return (uint16_t) sign;                      /* < 2^-25 -> 0 (ties at 2^-25 go to even = 0) */
    {                                                                 /* subnormal half */
        const int e = (int) (a >> 23);                                /* 102..112 */
        const uint32_t m = (a & 0x7fffffu) | 0x800000u;               /* 24-bit significand */
        const int sh = 126 - e;                                       /* 14..24 bits dropped */
        const uint32_t q = m >> sh, rem = m & ((1u << sh) - 1u), half = 1u << (sh - 1);
        uint32_t r = q;
        if (rem > half || (rem == half && (q & 1u))) ++r;
        return (uint16_t) (sign | r);
    }
}

float orc_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t) (h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    uint32_t x;
    if (e == 0x1f) x = sign | 0x7f800000u | (m << 13);
    else if (e) x = sign | ((e + 112u) << 23) | (m << 13);
    else if (!m) x = sign;
    else {
        int s = 0;
        uint32_t mm = m;
        while (!(mm & 0x400u)) { mm <<= 1; ++s; }
        x = sign | ((uint32_t) (113 - s) << 23) | ((mm & 0x3ffu) << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* src/fast/attn.cu:501-503 */
size_t orc_kv_row_bytes(uint32_t type, int Hkv, int D) {
    if (type == ORC_KV_F16) return (size_t) Hkv * D * 2;
    if (type == ORC_KV_Q8_0) return (size_t) Hkv * (D / 32) * 34;
    return (size_t) Hkv * (D / 32) * 18;
}

/* src/fast/kv_page.cuh:21-31, src/fast/attn.cuh:23-27 */
size_t orc_kv_off(const orc_kv *c, int t, int p) {
    const size_t rowb = orc_kv_row_bytes(c->type, c->Hkv, c->D);
    if (!c->pt) return (size_t) p * rowb;
    const int32_t *tab = c->rtab ? c->pt + c->rtab[t] : c->pt;
    return (size_t) tab[p >> c->psh] * c->pstride + (size_t) (p & ((1 << c->psh) - 1)) * rowb;
}

/* src/fast/kv_q8.cuh:20-26 (= ggml quantize_row_q8_0_ref, ggml-quants.c:276-299):
 * d = amax / 127 (f32), id = d ? 1/d : 0, q = roundf(x * id) (half away from zero), scale stored as RNE f16 of d. */
void orc_quant_q8_0_block(const float *x, uint16_t *d_bits, int8_t *q) {
    float amax = 0.0f;
    for (int j = 0; j < 32; ++j) {
        const float a = fabsf(x[j]);
        if (a > amax) amax = a;
    }
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    *d_bits = orc_f32_to_f16(d);
    for (int j = 0; j < 32; ++j) {
        volatile float p = x[j] * id; /* product rounded to f32 before roundf */
        q[j] = (int8_t) (int) roundf(p);
    }
}

/* src/fast/kv_q8.cuh:32-49 (= ggml quantize_row_q4_0_ref, ggml-quants.c:113-147): max = the signed value of largest
 * magnitude (first one on ties; 0 when every |x| is 0), d = max / -8, q = min(15, (int)(x * id + 8.5f)) with the
 * product and the sum rounded separately; byte j = q[j] | q[j + 16] << 4. */
void orc_quant_q4_0_block(const float *x, uint8_t *blk18) {
    float amax = 0.0f, mx = 0.0f;
    for (int j = 0; j < 32; ++j) {
        const float a = fabsf(x[j]);
        if (amax < a) { amax = a; mx = x[j]; }
    }
    const float d = mx / -8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const uint16_t db = orc_f32_to_f16(d);
    blk18[0] = (uint8_t) (db & 0xff);
    blk18[1] = (uint8_t) (db >> 8);
    for (int j = 0; j < 16; ++j) {
        volatile float p0 = x[j] * id, p1 = x[j + 16] * id;
        volatile float s0 = p0 + 8.5f, s1 = p1 + 8.5f;
        int q0 = (int) s0, q1 = (int) s1;
        if (q0 > 15) q0 = 15;
        if (q1 > 15) q1 = 15;
        blk18[2 + j] = (uint8_t) (q0 | (q1 << 4));
    }
}

/* row layouts: src/fast/attn.cuh:1-7 and src/fast/kv_q8.cuh:1-5 (q8_0: per head D/32 f16 scales then D int8;
 * q4_0: D/32 ggml blocks of 18 B; f16: plain halves); appends: src/fast/attn.cu:245-283 */
static void append_head(uint32_t type, int D, const float *x, uint8_t *dst) {
    if (type == ORC_KV_F16) {
        for (int i = 0; i < D; ++i) {
            const uint16_t h = orc_f32_to_f16(x[i]);
            dst[2 * i] = (uint8_t) (h & 0xff);
            dst[2 * i + 1] = (uint8_t) (h >> 8);
        }
    } else if (type == ORC_KV_Q8_0) {
        const int nb = D / 32;
        for (int b = 0; b < nb; ++b) {
            uint16_t d;
            orc_quant_q8_0_block(x + 32 * b, &d, (int8_t *) dst + 2 * nb + 32 * b);
            dst[2 * b] = (uint8_t) (d & 0xff);
            dst[2 * b + 1] = (uint8_t) (d >> 8);
        }
    } else {
        for (int b = 0; b < D / 32; ++b) orc_quant_q4_0_block(x + 32 * b, dst + 18 * b);
    }
}

static size_t head_bytes(uint32_t type, int D) { return orc_kv_row_bytes(type, 1, D); }

void orc_kv_append_rows(const orc_kv *c, const float *k, const float *v, const int32_t *pos, int T) {
    const size_t hb = head_bytes(c->type, c->D);
    for (int t = 0; t < T; ++t) {
        const size_t o = orc_kv_off(c, t, pos[t]);
        for (int h = 0; h < c->Hkv; ++h) {
            const size_t src = ((size_t) t * c->Hkv + h) * c->D;
            append_head(c->type, c->D, k + src, (uint8_t *) c->k + o + h * hb);
            append_head(c->type, c->D, v + src, (uint8_t *) c->v + o + h * hb);
        }
    }
}

/* element reader: tests/fast_attn_test.cu:34-44 (value = code * f32(f16 scale); q4_0 value = (nibble - 8) * scale) */
void orc_kv_read_head(const orc_kv *c, int which, int t, int p, int hk, float *dst) {
    const uint8_t *row = (const uint8_t *) (which ? c->v : c->k) + orc_kv_off(c, t, p) + hk * head_bytes(c->type, c->D);
    const int D = c->D;
    if (c->type == ORC_KV_F16) {
        for (int i = 0; i < D; ++i) dst[i] = orc_f16_to_f32((uint16_t) (row[2 * i] | (row[2 * i + 1] << 8)));
    } else if (c->type == ORC_KV_Q8_0) {
        const int nb = D / 32;
        const int8_t *qs = (const int8_t *) row + 2 * nb;
        for (int b = 0; b < nb; ++b) {
            const float d = orc_f16_to_f32((uint16_t) (row[2 * b] | (row[2 * b + 1] << 8)));
            for (int i = 0; i < 32; ++i) dst[32 * b + i] = d * (float) qs[32 * b + i];
        }
    } else {
        for (int b = 0; b < D / 32; ++b) {
            const uint8_t *blk = row + 18 * b;
            const float d = orc_f16_to_f32((uint16_t) (blk[0] | (blk[1] << 8)));
            for (int i = 0; i < 16; ++i) {
                dst[32 * b + i] = (float) ((int) (blk[2 + i] & 15) - 8) * d;
                dst[32 * b + 16 + i] = (float) ((int) (blk[2 + i] >> 4) - 8) * d;
            }
        }
    }
}

/* src/kernels.cu:85-88 */
void orc_gate(float *x, const float *g, size_t n) {
    for (size_t i = 0; i < n; ++i) x[i] *= 1.0f / (1.0f + expf(-g[i]));
}

/* src/kernels.cu:34-42 with w == NULL */
void orc_rmsnorm_heads(float *x, size_t nheads, int D, float eps) {
    for (size_t r = 0; r < nheads; ++r) {
        float *xr = x + r * D;
        float ss = 0.0f;
        for (int i = 0; i < D; ++i) ss += xr[i] * xr[i];
        const float sc = 1.0f / sqrtf(ss / (float) D + eps);
        for (int i = 0; i < D; ++i) xr[i] = xr[i] * sc;
    }
}

/*
 * Attention-layer input prep, the front half of the engine's attn_prep (src/fast/fused.cuh:101-113, kernel
 * src/fast/fused.cu:512-573): per token t and head,
 *   q heads : gate[t][h] = second half of the head's (q | gate) slice of qg (src/kernels.cu:95-106), then
 *             q[t][h] = rope(rmsnorm(first half) * q_norm);
 *   k heads : rope(rmsnorm(k) * k_norm) -> quantized K row of the cache; v heads: raw v -> V row (kv_q8.cuh:20-49);
 * cache row of token t = pos[t] when p0 < 0, else p0 + t; the ROTARY position is pos[t] in both cases (fused.cu:548).
 * RMS norm: src/kernels.cu:34-42 / fused.cu:540-550 (x * rsqrt(mean(x^2) + eps) * w); NEOX rope on the first n_rot
 * dims: pairs (j, j + n_rot/2), theta = pos * freq_base^(-2j/n_rot) (fused.cu:553-562).
 * The order of the floating-point operations is FIXED here (and the GPU kernel keeps the same order, so that the K
 * codes can be compared bit for bit): the sum of squares is formed per group of 4 consecutive dims, left to right,
 * and the groups are added in a balanced binary tree over 64 slots (empty slots are 0); the scale is 1 / sqrtf(...)
 * with IEEE division and square root (the reference uses the approximate rsqrtf, a difference of an ulp); the
 * rotation angle is pos * (float) base^(-2j/n_rot) in fp32 and its cosine / sine are rounded to fp32 (the reference
 * calls CUDA's powf / cosf / sinf, fused.cu:551-553, whose last bits no other machine reproduces); products and sums
 * are rounded separately (no fused multiply-add).
 * Power, cosine and sine are spelled out below in IEEE double operations in a fixed order - NOT taken from libm - so
 * that the result bits do not depend on the math library: ln by the atanh series on the frexp mantissa, e^x by
 * Cody-Waite reduction with a degree-13 Taylor polynomial, sin / cos by reduction against pi/2 held in four 24-bit
 * pieces and the fdlibm kernel polynomials. tests/test_oracle_prep.py pins them against numpy's float64 functions.
 */
static double prep_log(double x) {
    const double LN2_HI = 6.93147180369123816490e-01, LN2_LO = 1.90821492927058770002e-10;
    int e = 0;
    double m = frexp(x, &e);
    if (m < 7.07106781186547524401e-01) { m = m * 2.0; e -= 1; }
    const double s = (m - 1.0) / (m + 1.0), z = s * s;
    double p = 1.0 / 25.0;
    for (int k = 23; k >= 1; k -= 2) p = p * z + 1.0 / (double) k;
    const double lm = (2.0 * s) * p;
    return (double) e * LN2_HI + ((double) e * LN2_LO + lm);
}
static double prep_exp(double x) {
    const double LOG2E = 1.44269504088896338700e+00, LN2_HI = 6.93147180369123816490e-01, LN2_LO = 1.90821492927058770002e-10;
    static const double inv_fact[14] = {1.0, 1.0, 0.5, 1.0 / 6.0, 1.0 / 24.0, 1.0 / 120.0, 1.0 / 720.0, 1.0 / 5040.0, 1.0 / 40320.0,
                                        1.0 / 362880.0, 1.0 / 3628800.0, 1.0 / 39916800.0, 1.0 / 479001600.0, 1.0 / 6227020800.0};
    const double k = rint(x * LOG2E);
    const double r = (x - k * LN2_HI) - k * LN2_LO;
    double p = inv_fact[13];
    for (int i = 12; i >= 0; --i) p = p * r + inv_fact[i];
    return ldexp(p, (int) k);
}
static void prep_sincos(double t, float *c, float *s) {
    static const double pio2[4] = {1.57079625129699707031e+00, 7.54978941586159635335e-08, 5.39030252995776476554e-15, 3.28200341580791294123e-22};
    static const double S[6] = {-1.66666666666666324348e-01, 8.33333333332248946124e-03, -1.98412698298579493134e-04,
                                2.75573137070700676789e-06, -2.50507602534068634195e-08, 1.58969099521155010221e-10};
    static const double C[6] = {4.16666666666666019037e-02, -1.38888888888741095749e-03, 2.48015872894767294178e-05,
                                -2.75573143513906633035e-07, 2.08757232129817482790e-09, -1.13596475577881948265e-11};
    const double n = rint(t * 6.36619772367581382433e-01);
    double r = t;
    for (int i = 0; i < 4; ++i) r = r - n * pio2[i];
    const double z = r * r;
    double ps = S[4] + z * S[5], pc = C[4] + z * C[5];
    for (int i = 3; i >= 0; --i) { ps = S[i] + z * ps; pc = C[i] + z * pc; }
    const double sn = r + (z * r) * ps;
    const double cs = 1.0 - (0.5 * z - (z * z) * pc);
    switch ((int) ((long long) n & 3)) {
        case 0: *c = (float) cs; *s = (float) sn; break;
        case 1: *c = (float) -sn; *s = (float) cs; break;
        case 2: *c = (float) -cs; *s = (float) -sn; break;
        default: *c = (float) sn; *s = (float) -cs; break;
    }
}
/* exported for the tests that pin the three recipes */
double orc_prep_inv_freq(float freq_base, int j, int n_rot) { return prep_exp(((-2.0 * (double) j) / (double) n_rot) * prep_log((double) freq_base)); }
void orc_prep_sincos(float theta, float *c, float *s) { prep_sincos((double) theta, c, s); }

/* interleaved M-RoPE (src/fast/mrope.cuh:1-8, 25-33): rotary pair j takes the position of one of three streams by its
 * sector = j % sect: sector % 3 == 1 and < 3 s1 -> h; sector % 3 == 2 and < 3 s2 -> w; sector % 3 == 0 and < 3 s0 -> t;
 * anything else -> the 4th stream, which is 0. mr == NULL: every pair takes pos. */
static int mrope_pick(const orc_mrope *mr, int t, int j, int pos) {
    if (!mr || !mr->p) return pos;
    const int sector = j % mr->sect;
    int s;
    if (sector % 3 == 1 && sector < 3 * mr->s1) s = 1;
    else if (sector % 3 == 2 && sector < 3 * mr->s2) s = 2;
    else if (sector % 3 == 0 && sector < 3 * mr->s0) s = 0;
    else return 0;
    return mr->p[(size_t) s * mr->stride + t];
}

static void prep_norm_rope(const float *src, const float *w, int D, int n_rot, float freq_base, float eps, int pos, const orc_mrope *mr, int t, float *dst) {
    float part[64];
    for (int i = 0; i < 64; ++i) {
        part[i] = 0.0f;
        if (4 * i < D) {
            const float *a = src + 4 * i;
            float s = a[0] * a[0];
            s = s + a[1] * a[1];
            s = s + a[2] * a[2];
            s = s + a[3] * a[3];
            part[i] = s;
        }
    }
    for (int m = 1; m < 64; m <<= 1)
        for (int i = 0; i < 64; i += 2 * m) part[i] = part[i] + part[i + m];
    const float sc = 1.0f / sqrtf(part[0] / (float) D + eps);
    for (int i = 0; i < D; ++i) {
        float o = src[i] * sc;
        if (w) o = o * w[i];
        dst[i] = o;
    }
    const int half = n_rot / 2;
    const double ln_base = prep_log((double) freq_base);
    for (int j = 0; j < half; ++j) {
        const float inv = (float) prep_exp(((-2.0 * (double) j) / (double) n_rot) * ln_base);
        const float theta = (float) mrope_pick(mr, t, j, pos) * inv;
        float c, sn;
        prep_sincos((double) theta, &c, &sn);
        const float x0 = dst[j], x1 = dst[j + half];
        const float a0 = x0 * c, a1 = x1 * sn, b0 = x0 * sn, b1 = x1 * c;
        dst[j] = a0 - a1;
        dst[j + half] = b0 + b1;
    }
}

int orc_attn_prep(const float *qg, const float *k, const float *v, const float *q_norm, const float *k_norm,
                  const int32_t *pos, float *q, float *gate, const orc_kv *c, int p0, int T, int Hq, int Hkv, int D,
                  int n_rot, float freq_base, float eps, int ldq, int ldk, int ldv) {
    return orc_attn_prep_mrope(qg, k, v, q_norm, k_norm, pos, q, gate, c, p0, T, Hq, Hkv, D, n_rot, freq_base, eps, ldq, ldk, ldv, NULL);
}

int orc_attn_prep_mrope(const float *qg, const float *k, const float *v, const float *q_norm, const float *k_norm,
                        const int32_t *pos, float *q, float *gate, const orc_kv *c, int p0, int T, int Hq, int Hkv, int D,
                        int n_rot, float freq_base, float eps, int ldq, int ldk, int ldv, const orc_mrope *mr) {
    if (mr && mr->p && mr->sect <= 0) return -1;
    if (!pos || D % 32 || D > 256 || n_rot % 8 || n_rot > D || c->D != D || c->Hkv != Hkv) return -1;
    if (!ldq) ldq = Hq * 2 * D;
    if (!ldk) ldk = Hkv * D;
    if (!ldv) ldv = Hkv * D;
    float *kr = (float *) malloc(sizeof(float) * (size_t) Hkv * D);
    float *vr = (float *) malloc(sizeof(float) * (size_t) Hkv * D);
    orc_kv one = *c;
    for (int t = 0; t < T; ++t) {
        for (int h = 0; h < Hq; ++h) {
            const float *src = qg + (size_t) t * ldq + (size_t) h * 2 * D;
            memcpy(gate + ((size_t) t * Hq + h) * D, src + D, sizeof(float) * D);
            prep_norm_rope(src, q_norm, D, n_rot, freq_base, eps, pos[t], mr, t, q + ((size_t) t * Hq + h) * D);
        }
        for (int h = 0; h < Hkv; ++h) {
            prep_norm_rope(k + (size_t) t * ldk + (size_t) h * D, k_norm, D, n_rot, freq_base, eps, pos[t], mr, t, kr + (size_t) h * D);
            memcpy(vr + (size_t) h * D, v + (size_t) t * ldv + (size_t) h * D, sizeof(float) * D);
        }
        /* row t of the batch: its own page table (rtab[t]) and its own position */
        const int32_t row = p0 < 0 ? pos[t] : p0 + t;
        one.rtab = c->rtab ? c->rtab + t : NULL;
        orc_kv_append_rows(&one, kr, vr, &row, 1);
    }
    free(kr);
    free(vr);
    return 0;
}

/*
 * Benchmark fill (src/fast/attn.cu:538-557 fill_random_k, :559-581 kv_fill_random). The cache is taken as 16-bit words;
 * word w (index inside the contiguous cache, or inside the page for a paged one) gets
 *   h = (uint32) w * 2654435761 ^ seed;  h ^= h >> 16;  h *= 0x7feb352d;  h ^= h >> 15;  h *= 0x846ca68b;  h ^= h >> 16
 *   f16:  K = f16((h & 0xffff) / 32768 - 1), V = f16((h >> 16) / 32768 - 1)
 *   scale words (q8_0: the first D/32 words of a head row; q4_0: every 9th word): f16(1/127) resp. f16(0.125), K and V
 *   other words: K = low half of h, V = high half.
 * Paged: logical page g of the sequence is filled as a contiguous cache at its page base with seed + g * 0x632be5ab.
 */
static void fill_words(uint16_t *k, uint16_t *v, size_t w0, size_t nw, uint32_t type, int D, int head_words, uint32_t seed) {
    for (size_t i = 0; i < nw; ++i) {
        const size_t w = w0 + i;
        uint32_t h = (uint32_t) w * 2654435761u ^ seed;
        h ^= h >> 16; h *= 0x7feb352du; h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 16;
        const int hw = (int) (w % (size_t) head_words);
        uint16_t a, b;
        if (type == ORC_KV_F16) {
            a = orc_f32_to_f16((float) (h & 0xffffu) / 32768.0f - 1.0f);
            b = orc_f32_to_f16((float) (h >> 16) / 32768.0f - 1.0f);
        } else if ((type == ORC_KV_Q8_0 && hw < D / 32) || (type == ORC_KV_Q4_0 && hw % 9 == 0)) {
            a = b = orc_f32_to_f16(type == ORC_KV_Q8_0 ? 1.0f / 127.0f : 0.125f);
        } else {
            a = (uint16_t) h;
            b = (uint16_t) (h >> 16);
        }
        k[w] = a;
        v[w] = b;
    }
}

void orc_kv_fill_random(const orc_kv *c, int p0, int p1, uint32_t seed) {
    if (!c->k || p1 <= p0) return;
    const size_t rowb = orc_kv_row_bytes(c->type, c->Hkv, c->D);
    const int head_words = (int) (rowb / c->Hkv / 2);
    if (!c->pt) {
        fill_words((uint16_t *) c->k, (uint16_t *) c->v, (size_t) p0 * rowb / 2, (size_t) (p1 - p0) * rowb / 2, c->type, c->D, head_words, seed);
        return;
    }
    const int32_t *pt = c->pt + (c->rtab ? c->rtab[0] : 0);
    const int ps = 1 << c->psh;
    for (int a = p0; a < p1;) {
        const int pg = a >> c->psh, b = p1 < (pg + 1) * ps ? p1 : (pg + 1) * ps;
        uint16_t *kp = (uint16_t *) ((uint8_t *) c->k + (size_t) pt[pg] * c->pstride);
        uint16_t *vp = (uint16_t *) ((uint8_t *) c->v + (size_t) pt[pg] * c->pstride);
        fill_words(kp, vp, (size_t) (a - pg * ps) * rowb / 2, (size_t) (b - a) * rowb / 2, c->type, c->D, head_words,
                   seed + (uint32_t) pg * 0x632be5abu);
        a = b;
    }
}

/*
 * a16 activation quantize of the engine's quantized matvec (src/fast/matvec_a16.cu:29-100 quantize_a16, restated for
 * fused producers in src/fast/a16q.cuh:21-45): per token row t of n values, per group g of 32 values
 *   amax = max |v| (clamped to 65504 when it would round to an infinite f16), id = amax > 0 ? 1 / amax : 0,
 *   w = v * id (rounded), sum = sum of w: the 4 values of a lane (lane l holds values 4l..4l+3) added in order from +0,
 *   then the 8 lane sums in an xor butterfly with strides 4, 2, 1;
 *   qbuf as half2 words: word (t * ng + g) * 16 + slot holds two scaled values, slot order of matvec_a16.cu:89-99;
 *   word T * ng * 16 + t * ng + g holds (f16(amax), f16(sum)).
 */
void orc_a16_quant(const float *y, int T, int n, uint16_t *qbuf) {
    const int ng = n / 32;
    uint16_t *ads = qbuf + (size_t) T * ng * 16 * 2;
    for (int t = 0; t < T; ++t)
        for (int g = 0; g < ng; ++g) {
            const float *v = y + (size_t) t * n + (size_t) g * 32;
            float amax = 0.0f;
            for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(v[i]));
            amax = amax < 65520.0f ? amax : 65504.0f;
            const float id = amax > 0.0f ? 1.0f / amax : 0.0f;
            float w[32], ls[8];
            for (int l = 0; l < 8; ++l) {
                float sum = 0.0f;
                for (int i = 0; i < 4; ++i) {
                    w[4 * l + i] = v[4 * l + i] * id;
                    sum = sum + w[4 * l + i];
                }
                ls[l] = sum;
            }
            for (int st = 4; st > 0; st >>= 1) {
                float nx[8];
                for (int l = 0; l < 8; ++l) nx[l] = ls[l] + ls[l ^ st];
                memcpy(ls, nx, sizeof ls);
            }
            uint16_t *qs = qbuf + ((size_t) t * ng + g) * 16 * 2;
            for (int l = 0; l < 8; ++l) {
                const int off = l >= 4 ? 1 : 0, k = l - 4 * off;
                qs[(4 * k + 0 + off) * 2 + 0] = orc_f32_to_f16(w[4 * l + 0]);
                qs[(4 * k + 0 + off) * 2 + 1] = orc_f32_to_f16(w[4 * l + 2]);
                qs[(4 * k + 2 + off) * 2 + 0] = orc_f32_to_f16(w[4 * l + 1]);
                qs[(4 * k + 2 + off) * 2 + 1] = orc_f32_to_f16(w[4 * l + 3]);
            }
            ads[((size_t) t * ng + g) * 2 + 0] = orc_f32_to_f16(amax);
            ads[((size_t) t * ng + g) * 2 + 1] = orc_f32_to_f16(ls[0]);
        }
}

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/*
 * Attention of src/kernels.cu:143-166 (attention_k): for query row t and head h, kv head hk = h / (Hq / Hkv),
 * n_kv = pos[t] + 1 visible keys, score_j = (q . k_j) * scale, mx = max score, den = sum exp(score - mx),
 * out = sum exp(score_j - mx) v_j / den, all fp32; then the gate of src/kernels.cu:85-88 when given.
 * Keys are walked in fixed chunks of ORC_CHUNK so that the partial sums (and hence the bits) do not depend on the
 * thread count; the reference kernel sums sequentially, the difference is a few fp32 ulps.
 * The cache is read through the page table (src/fast/kv_page.cuh:21-31) and dequantized as tests/fast_attn_test.cu:34-44.
 */
#define ORC_CHUNK 256

int orc_attn_rows(const orc_kv *c, const float *q, float *out, const float *gate, int T, const int32_t *pos, int Hq,
                  float scale, int f64) {
    const int D = c->D, Hkv = c->Hkv;
    if (Hkv <= 0 || Hq % Hkv || D <= 0 || T < 0) return -1;
    const int G = Hq / Hkv;
    for (int t = 0; t < T; ++t) {
        for (int hk = 0; hk < Hkv; ++hk) {
            const int n = pos[t] + 1;
            const int nch = (n + ORC_CHUNK - 1) / ORC_CHUNK;
            float *sc = (float *) malloc((size_t) G * n * sizeof(float));
            double *scd = f64 ? (double *) malloc((size_t) G * n * sizeof(double)) : NULL;
            double *part = (double *) calloc((size_t) nch * G * D, sizeof(double));
            if (!sc || !part || (f64 && !scd)) { free(sc); free(scd); free(part); return -2; }
            /* pass 1: scores */
#pragma omp parallel
            {
                float *row = (float *) malloc((size_t) D * sizeof(float));
#pragma omp for schedule(static)
                for (int j = 0; j < n; ++j) {
                    orc_kv_read_head(c, 0, t, j, hk, row);
                    for (int g = 0; g < G; ++g) {
                        const float *qr = q + ((size_t) t * Hq + hk * G + g) * D;
                        if (f64) {
                            double d = 0.0;
                            for (int i = 0; i < D; ++i) d += (double) qr[i] * (double) row[i];
                            scd[(size_t) g * n + j] = d * (double) scale;
                        } else {
                            float d8[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                            for (int i = 0; i < D; i += 8)
                                for (int u = 0; u < 8; ++u) d8[u] += qr[i + u] * row[i + u];
                            const float d = ((d8[0] + d8[4]) + (d8[2] + d8[6])) + ((d8[1] + d8[5]) + (d8[3] + d8[7]));
                            sc[(size_t) g * n + j] = d * scale;
                        }
                    }
                }
                free(row);
            }
            /* max and denominator per head */
            double mxd[64], dend[64];
            float mxf[64], denf[64];
            if (G > 64) { free(sc); free(scd); free(part); return -1; }
            for (int g = 0; g < G; ++g) {
                if (f64) {
                    double mx = -INFINITY, den = 0.0;
                    for (int j = 0; j < n; ++j) mx = scd[(size_t) g * n + j] > mx ? scd[(size_t) g * n + j] : mx;
                    for (int j = 0; j < n; ++j) den += exp(scd[(size_t) g * n + j] - mx);
                    mxd[g] = mx; dend[g] = den;
                } else {
                    float mx = -INFINITY, den = 0.0f;
                    for (int j = 0; j < n; ++j) mx = fmaxf(mx, sc[(size_t) g * n + j]);
                    for (int j = 0; j < n; ++j) den += expf(sc[(size_t) g * n + j] - mx);
                    mxf[g] = mx; denf[g] = den;
                }
            }
            /* pass 2: weighted V, per fixed chunk */
#pragma omp parallel
            {
                float *row = (float *) malloc((size_t) D * sizeof(float));
                float *accf = (float *) malloc((size_t) G * D * sizeof(float));
#pragma omp for schedule(static)
                for (int ch = 0; ch < nch; ++ch) {
                    const int j0 = ch * ORC_CHUNK, j1 = j0 + ORC_CHUNK < n ? j0 + ORC_CHUNK : n;
                    double *pa = part + (size_t) ch * G * D;
                    memset(accf, 0, (size_t) G * D * sizeof(float));
                    for (int j = j0; j < j1; ++j) {
                        orc_kv_read_head(c, 1, t, j, hk, row);
                        for (int g = 0; g < G; ++g) {
                            if (f64) {
                                const double p = exp(scd[(size_t) g * n + j] - mxd[g]);
                                for (int i = 0; i < D; ++i) pa[(size_t) g * D + i] += p * (double) row[i];
                            } else {
                                const float p = expf(sc[(size_t) g * n + j] - mxf[g]);
                                float *a = accf + (size_t) g * D;
                                for (int i = 0; i < D; ++i) a[i] += p * row[i];
                            }
                        }
                    }
                    if (!f64) for (int i = 0; i < G * D; ++i) pa[i] = (double) accf[i];
                }
                free(row);
                free(accf);
            }
            for (int g = 0; g < G; ++g) {
                float *o = out + ((size_t) t * Hq + hk * G + g) * D;
                for (int i = 0; i < D; ++i) {
                    if (f64) {
                        double a = 0.0;
                        for (int ch = 0; ch < nch; ++ch) a += part[((size_t) ch * G + g) * D + i];
                        o[i] = (float) (a / dend[g]);
                    } else {
                        float a = 0.0f;
                        for (int ch = 0; ch < nch; ++ch) a += (float) part[((size_t) ch * G + g) * D + i];
                        o[i] = a / denf[g];
                    }
                }
            }
            free(sc); free(scd); free(part);
        }
    }
    if (gate) {
        if (f64) {
            for (size_t i = 0; i < (size_t) T * Hq * D; ++i) out[i] = (float) ((double) out[i] / (1.0 + exp(-(double) gate[i])));
        } else {
            orc_gate(out, gate, (size_t) T * Hq * D);
        }
    }
    return 0;
}
