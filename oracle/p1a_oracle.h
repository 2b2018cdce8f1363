/*
 * CPU oracle for the paged-KV attention path (TEST INFRASTRUCTURE, not product code).
 *
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may link or call this. It is a plain-C
 * restatement of the arithmetic of the reference engine's attention path; every function cites the reference
 * file:line it follows (paths relative to the reference tree).
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   orc_quant_q8_0_block / orc_quant_q4_0_block : golden vectors produced by the reference's vendored ggml C
 *       quantizers (tests/golden/quant_golden.npz) + closed forms (zero block, +-amax codes, ties, half-way cases).
 *   orc_f32_to_f16 / orc_f16_to_f32           : exhaustive against numpy float16 (all 65536 halves; 2^20 floats).
 *   orc_kv_off / orc_kv_row_bytes / row layout : byte formulas of src/fast/attn.cuh:1-32 and the independent
 *       element reader of tests/fast_attn_test.cu:34-44, restated in numpy; paged(perm) == contiguous invariant.
 *   orc_attn_rows                              : numpy float64 softmax(QK^T)V on the dequantized cache, n = 1,
 *       equal-V, dominant-logit, causality and shift-invariance closed forms.
 *   orc_gate                                   : g = 0 -> x0.5, sigma(g) + sigma(-g) = 1.
 *   orc_attn_prep                              : numpy float64 restatement of norm * weight and the NEOX rotation (to a few
 *       fp32 ulps); closed forms (position 0 rotates nothing, the rotation keeps pair norms, q . k after rope depends on
 *       the position difference only, a constant head norms to w); KV rows == orc_kv_append_rows of the normed, roped k.
 *       Its power / cosine / sine recipes (IEEE double operations in a fixed order, no libm: orc_prep_inv_freq,
 *       orc_prep_sincos) against numpy's float64 pow / cos / sin rounded to fp32: equal but for rare last-bit roundings
 *       (the double result sits within 2^-50 of a rounding boundary), over all rotary pairs and angles up to 2^29.
 *   orc_attn_prep_mrope                        : t = h = w = p is bitwise plain NEOX at p (src/fast/mrope.cuh:6-7); the
 *       stream of every rotary pair from a table written out by hand from the rule's words for sections [11, 11, 10, 0]
 *       and [2, 1, 1, 0]; moving one stream changes exactly the pairs of that stream.
 *   orc_a16_quant                              : an independent numpy float32 restatement (element -> slot map written out
 *       from the engine's comment, not from its index arithmetic), closed forms (zero group, unit group, clamp at 65520).
 *   orc_kv_fill_random                         : the reference holds no vectors for its benchmark fill; pinned by the two
 *       fixed points of its word hash (word 0 / seed 0 and word 1 / seed = the multiplier both hash to 0, hence f16 -1.0
 *       or code 0), a big-integer restatement of the hash written out step by step, the places and bits of the scale
 *       words, the value range, additivity over position ranges and paged == page-by-page contiguous with the page seeds.
 * No function of this file is "parity unpinned".
 */
#ifndef P1A_ORACLE_H
#define P1A_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_KV_F16 = 1, ORC_KV_Q4_0 = 2, ORC_KV_Q8_0 = 8 }; /* src/fast/attn.cuh:14-16 */

/* host-memory twin of the engine's kv_cache descriptor (src/fast/attn.cuh:18-32) */
typedef struct orc_kv {
    uint32_t type;
    int32_t n_ctx, Hkv, D;
    void *k, *v;
    const int32_t *pt;   /* page table(s); NULL = contiguous */
    const int32_t *rtab; /* per-row element offsets into pt; NULL = 0 */
    int32_t psh;
    size_t pstride;
} orc_kv;

uint16_t orc_f32_to_f16(float f);
float orc_f16_to_f32(uint16_t h);

size_t orc_kv_row_bytes(uint32_t type, int Hkv, int D);
/* byte offset of position p of query row t inside the K (or V) region */
size_t orc_kv_off(const orc_kv *c, int t, int p);

/* one 32-value block: scale bits (f16) + 32 int8 codes */
void orc_quant_q8_0_block(const float *x, uint16_t *d_bits, int8_t *q);
/* one 32-value block -> the 18-byte ggml block_q4_0 */
void orc_quant_q4_0_block(const float *x, uint8_t *blk18);

/* k, v: [T][Hkv][D] f32 -> cache rows at pos[t] (t-th row uses rtab[t] when present) */
void orc_kv_append_rows(const orc_kv *c, const float *k, const float *v, const int32_t *pos, int T);
/* dequantize one (position, kv head) row of K (which = 0) or V (which = 1) into dst[D] */
void orc_kv_read_head(const orc_kv *c, int which, int t, int p, int hk, float *dst);

/* q, out: [T][Hq][D] f32. Row t sees positions 0..pos[t] of its own sequence. gate ([T][Hq*D], may be NULL)
 * multiplies the normalised output by sigmoid(gate). f64 != 0: all arithmetic in double (error budgeting). */
int orc_attn_rows(const orc_kv *c, const float *q, float *out, const float *gate, int T, const int32_t *pos, int Hq,
                  float scale, int f64);
void orc_gate(float *x, const float *g, size_t n);
/* per-head RMS norm with unit weight, in place: x * rsqrt(mean(x^2) + eps) */
void orc_rmsnorm_heads(float *x, size_t nheads, int D, float eps);
/* attention-layer input prep (q | gate split, RMS norm * weight, NEOX rope, quantize-append): src/fast/fused.cuh:101-113.
 * qg [T][ldq] (Hq heads of q | gate), k, v [T][ld] f32; q [T][Hq][D], gate [T][Hq*D] out; K / V rows written to c.
 * ld* = 0: dense. q_norm / k_norm [D] may be NULL. Returns 0, or -1 for an unsupported shape. */
int orc_attn_prep(const float *qg, const float *k, const float *v, const float *q_norm, const float *k_norm,
                  const int32_t *pos, float *q, float *gate, const orc_kv *c, int p0, int T, int Hq, int Hkv, int D,
                  int n_rot, float freq_base, float eps, int ldq, int ldk, int ldv);
/* the same with interleaved M-RoPE positions (src/fast/mrope.cuh:14-33, src/fast/fused.cuh:108-113): rotary pair j of
 * row t rotates by the position of the stream its sector selects; cache rows still come from pos / p0. mr == NULL or
 * mr->p == NULL: plain NEOX. */
typedef struct orc_mrope {
    const int32_t *p;   /* [3][stride]: t, h, w positions of the rows */
    int stride;
    int s0, s1, s2;     /* sections, in rotary pairs */
    int sect;           /* sum of all four sections */
} orc_mrope;
int orc_attn_prep_mrope(const float *qg, const float *k, const float *v, const float *q_norm, const float *k_norm,
                        const int32_t *pos, float *q, float *gate, const orc_kv *c, int p0, int T, int Hq, int Hkv, int D,
                        int n_rot, float freq_base, float eps, int ldq, int ldk, int ldv, const orc_mrope *mr);
/* the rotary recipes of orc_attn_prep, exported for the tests that pin them: base^(-2j/n_rot) in double, and the fp32
 * cosine / sine of an fp32 angle */
double orc_prep_inv_freq(float freq_base, int j, int n_rot);
void orc_prep_sincos(float theta, float *c, float *s);
/* a16 activation quantize (src/fast/a16q.cuh:21-45 = src/fast/matvec_a16.cu:29-100): y [T][n] f32, n % 32 == 0 ->
 * qbuf: T * n/32 * 16 half2 of scaled values (slot order of the engine), then T * n/32 half2 (amax, sum). */
void orc_a16_quant(const float *y, int T, int n, uint16_t *qbuf);
/* benchmark fill of positions p0 .. p1 - 1 of ONE sequence (page table pt + (rtab ? rtab[0] : 0)) with hashed 16-bit
 * words: src/fast/attn.cu:538-581 (kv_fill_random; the engine's bench_fill_kv, src/tp_model.cu:3195-3209, calls it). */
void orc_kv_fill_random(const orc_kv *c, int p0, int p1, uint32_t seed);
int orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
