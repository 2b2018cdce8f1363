/*
 * p1a_attn.h - C ABI of the MI355X (gfx950) paged-KV attention library: quantize-on-append KV write, split-K
 * decode / MTP multi-token verify, chunked causal prefill and the fused sigmoid output gate.
 *
 * Each entry point replaces one function of the reference engine's C++ attention surface (namespace p100e::fast);
 * the reference file:line is given with every declaration (paths relative to the reference tree). The C++ mirror of
 * that surface, with the reference's names and argument order, is include/p100e_fast_attn.hpp; it only calls the
 * functions below.
 *
 * Conventions shared by all entry points
 *   - All tensor pointers are DEVICE pointers; `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *   - Return value: 0 = work enqueued; negative (P1A_E_*) = refused, NOTHING was launched and the outputs are
 *     untouched; a diagnostic goes to stderr and to p1a_last_error(). No exceptions, no host synchronisation.
 *   - Positions (`p0_dev`, `pos_rows`) and page tables (`pt`, `rtab`) are read ON THE DEVICE when the kernels run,
 *     so a captured hipGraph replays correctly at any depth.
 *   - Split-K scratch is owned by the library per (device, stream). It is allocated on the first decode call (or by
 *     p1a_warmup) at the footprint of P1A_MAX_ROWS rows of that call's head shape and is never freed or moved while the
 *     library is loaded (p1a_release() frees everything), so a captured hipGraph stays valid whatever is called later
 *     on its stream. Nothing is allocated during stream capture: warm up (or make one eager call) first.
 */
#ifndef P1A_ATTN_H
#define P1A_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* KV storage modes; values equal the reference's (= the ggml type ids). src/fast/attn.cuh:14-16 */
#define P1A_KV_F16  1u
#define P1A_KV_Q4_0 2u
#define P1A_KV_Q8_0 8u

#define P1A_OK            0
#define P1A_E_SHAPE      (-1) /* unsupported shape / type / alignment */
#define P1A_E_ARG        (-2) /* null or inconsistent argument */
#define P1A_E_SCRATCH    (-3) /* scratch allocation failed or caller scratch too small */
#define P1A_E_LAUNCH     (-4) /* the HIP runtime reported a launch error */
#define P1A_E_STATE      (-5) /* pool / sequence manager: the pool or the sequence is not in a state that allows it */
#define P1A_E_IO         (-6) /* session file: cannot open, short read / write, or not a loadable file */

#define P1A_MAX_ROWS 32 /* query rows per p1a_attn_decode call (the reference allows 8: src/fast/attn.cuh:66) */

/*
 * POD copy of the reference's `struct kv_cache` (src/fast/attn.cuh:18-32); same fields, same meaning.
 * Position p of query row t lives at
 *     base + pt[(rtab ? rtab[t] : 0) + (p >> psh)] * pstride + (p & (2^psh - 1)) * row_bytes      (pt != NULL)
 *     base + p * row_bytes                                                                        (pt == NULL)
 * with base = k or v. Row layouts (per position: Hkv heads back to back):
 *     f16  : D halves per head
 *     q8_0 : per head D/32 f16 scales, then D int8 codes (272 B at D = 256)            src/fast/kv_q8.cuh:1-5
 *     q4_0 : per head D/32 ggml block_q4_0 (f16 d, 16 B: byte i = v[i] | v[i+16] << 4)   src/fast/attn.cuh:4-5
 * The layer is selected by the k / v base pointers, the slot by pt (or rtab[t]), the storage mode by type.
 */
typedef struct p1a_kv {
    uint32_t type;
    int32_t n_ctx, Hkv, D;
    void *k;
    void *v;
    const int32_t *pt;
    const int32_t *rtab;
    int32_t psh;
    size_t pstride;
} p1a_kv;

/* bytes of one position (all kv heads) of K or V. Replaces kv_row_bytes, src/fast/attn.cu:501-503. */
size_t p1a_kv_row_bytes(uint32_t type, int Hkv, int D);

/*
 * Quantize-on-append KV write: k, v [T][Hkv][D] f32 -> cache rows. Row t goes to position
 *     pos_rows[t]            when pos_rows != NULL (each row in its own sequence, table pt + rtab[t])
 *     *p0_dev + t            else when p0_dev != NULL
 *     p0 + t                 otherwise.
 * Codes and scales are bit-identical to ggml's quantize_row_q8_0_ref / quantize_row_q4_0_ref.
 * Replaces kv_append (src/fast/attn.cuh:37-38, attn.cu:583-585), kv_append_dev (attn.cuh:58, attn.cu:587-589) and
 * the cache-write half of attn_prep in its device-position mode (src/fast/fused.cuh:101-113, fused.cu:512-526,563-572).
 * k, v must be 16-byte aligned; D % 32 == 0 for the quantized types.
 */
int p1a_kv_append(const p1a_kv *c, const float *k, const float *v, int p0, const int32_t *p0_dev,
                  const int32_t *pos_rows, int T, void *stream);

/*
 * Benchmark fill: positions p0 .. p1 - 1 of ONE sequence (page table pt + (rtab ? rtab[0] : 0), or contiguous) get hashed
 * 16-bit words - f16 values in [-1, 1], or random codes under constant block scales (q8_0 1/127, q4_0 0.125) - the same
 * bytes the reference writes for the same seed. The page table is read on the device (the reference copies it back).
 * Replaces kv_fill_random (src/fast/attn.cuh:70, attn.cu:538-581), which the engine's bench_fill_kv calls
 * (src/tp_model.cu:3195-3209).
 */
int p1a_kv_fill_random(const p1a_kv *c, int p0, int p1, uint32_t seed, void *stream);

/*
 * Attention-layer input prep in one launch: per token t
 *     qg [T][ldq] (Hq heads, each D floats of q followed by D floats of gate) -> gate [T][Hq*D] (copy) and
 *                                                                                q [T][Hq][D] = rope(rmsnorm(q) * q_norm)
 *     k  [T][ldk] (Hkv heads of D) -> rope(rmsnorm(k) * k_norm) -> K cache row;   v [T][ldv] -> V cache row
 * with rmsnorm(x) = x / sqrt(mean(x^2) + eps) per head, the NEOX rotation of dims (j, j + n_rot/2), j < n_rot/2, by
 * pos[t] * freq_base^(-2j/n_rot), and the quantizing write of p1a_kv_append. The cache row of token t is p0 + t, or
 * pos[t] (read on the device, own page table pt + rtab[t]) when p0 < 0; the rotary position is pos[t] in both cases.
 * ld* = 0 means dense rows; q_norm / k_norm ([D]) may be NULL. D <= 256, n_rot % 8 == 0.
 * Replaces the front half of attn_prep (src/fast/fused.cuh:101-113, kernel src/fast/fused.cu:512-573) = k::split_q_gate
 * + fast::rmsnorm + k::rope_neox + kv_append of the unfused path (src/tp_model.cu:1717-1734).
 */
int p1a_attn_prep(const float *qg, const float *k, const float *v, const float *q_norm, const float *k_norm,
                  const int32_t *pos, float *q, float *gate, const p1a_kv *c, int p0, int T, int Hq, int n_rot,
                  float freq_base, float eps, int ldq, int ldk, int ldv, void *stream);
/*
 * The same with interleaved M-RoPE positions (images in the context): mr_pos [3][mr_stride] holds the t / h / w positions
 * of the rows; rotary pair j takes the stream its sector = j % sect selects (sector % 3 == 1 and < 3 s1 -> h,
 * % 3 == 2 and < 3 s2 -> w, % 3 == 0 and < 3 s0 -> t, otherwise position 0); s0, s1, s2 are the sections in rotary
 * pairs, sect the sum of all four. Cache rows still come from pos / p0. mr_pos == NULL is p1a_attn_prep.
 * Replaces attn_prep with mr.p != nullptr (src/fast/fused.cuh:108-113, src/fast/mrope.cuh:14-33).
 */
int p1a_attn_prep_mrope(const float *qg, const float *k, const float *v, const float *q_norm, const float *k_norm,
                        const int32_t *pos, float *q, float *gate, const p1a_kv *c, int p0, int T, int Hq, int n_rot,
                        float freq_base, float eps, int ldq, int ldk, int ldv, const int32_t *mr_pos, int mr_stride,
                        int s0, int s1, int s2, int sect, void *stream);

/*
 * Decode / MTP-verify attention: q, out [T][Hq][D] f32;
 *     out[t][h] = softmax_{j <= pos(t)} (scale * q[t][h] . K[j][h / (Hq/Hkv)]) . V[j][h / (Hq/Hkv)]
 * and, when gate != NULL (gate [T][Hq*D] f32), out *= 1 / (1 + exp(-gate)) fused into the final merge.
 * pos(t) = pos_rows[t] | *p0_dev + t | p0 + t as for p1a_kv_append. With pos_rows, `rows_per_seq` consecutive rows
 * share one sequence (the page table of the first row of each group): 1 = every row on its own (the reference's
 * attn_decode_rows), n > 1 = n-token verify blocks of several sequences in one call, each block reading its KV once.
 * Without pos_rows all T rows belong to one sequence and share the KV read in groups of up to 4 rows.
 * The key partition does not depend on T, p0 or the batch composition: row t of any call is bitwise the T = 1 call
 * at pos(t) on that sequence, and a paged cache gives the bits of the contiguous one.
 * Shapes: any D % 32 == 0 up to 512 and any Hq % Hkv == 0; the matrix-pipe kernels take D = 64 / 128 / 256 with Hq / Hkv <= 16
 * and pages of >= 16 positions (f16 and the quantized types at D = 256 with 16-byte aligned bases and page strides, the
 * quantized types at D = 64 / 128 with 4-byte aligned ones), everything else a slow generic kernel.
 * Replaces attn_decode (src/fast/attn.cuh:44, attn.cu:638-648), attn_decode_dev (attn.cuh:59-60, attn.cu:656-666),
 * attn_decode_rows (attn.cuh:64-65, attn.cu:650-654) and attn_decode2 (src/fast/attn_dec2.cuh:17-18); the gate
 * replaces the separate sigmoid_mul launch (src/kernels.cu:85-93).
 */
int p1a_attn_decode(const float *q, const p1a_kv *c, float *out, const float *gate, int T, int p0,
                    const int32_t *p0_dev, const int32_t *pos_rows, int rows_per_seq, int Hq, float scale,
                    void *stream);

/*
 * The same call that also emits the a16 activation buffer of the (gated) output rows, the input format of the engine's
 * quantized output-projection matvec: qbuf holds p1a_a16_bytes(T, Hq*D) bytes - per row and 32-value group 16 half2 of
 * value / amax (the engine's slot order), then per row and group one half2 (amax, sum of the scaled values). qbuf ==
 * NULL is p1a_attn_decode. Replaces attn_decode* followed by ew_quant(EW_SIGMOID_MUL, ...) at the fused decode call
 * site (src/tp_model.cu:1388-1397; layout src/fast/a16q.cuh:1-10, arithmetic :21-45 = src/fast/matvec_a16.cu:29-100).
 */
int p1a_attn_decode_a16(const float *q, const p1a_kv *c, float *out, const float *gate, void *qbuf, int T, int p0,
                        const int32_t *p0_dev, const int32_t *pos_rows, int rows_per_seq, int Hq, float scale,
                        void *stream);
/*
 * p1a_attn_decode_a16 for callers that cannot allocate (code under hipGraph capture on a stream the library has not seen,
 * tight serving loops, harnesses that forbid hipMalloc): NO COUNTERPART IN THE REFERENCE. Same arguments, same kernels,
 * same result bits, but the split partials live in a fixed array in device memory (P1A_NOALLOC_SCRATCH_BYTES, one copy per
 * GPU, held until the process ends) instead of the library's per-stream buffers, and the call never allocates or frees
 * anything. A call whose partials do not fit (T * Hq * splits * (D + 2) * 4 bytes; 8 rows of the 24 / 4 / 256 shape fit for
 * every KV type: CUs / Hkv = 64 split streams on a 256-CU part) is refused with P1A_E_SCRATCH. Every call on one GPU shares that GPU's array: calls that overlap on one GPU
 * (two streams, two threads) race - serialise them. The array's address is looked up on the first call per device (or by
 * p1a_warmup).
 */
#define P1A_NOALLOC_SCRATCH_BYTES (32u << 20)
int p1a_attn_decode_noalloc(const float *q, const p1a_kv *c, float *out, const float *gate, void *qbuf, int T, int p0,
                            const int32_t *p0_dev, const int32_t *pos_rows, int rows_per_seq, int Hq, float scale,
                            void *stream);
/* bytes of the a16 buffer of T rows of n values (n % 32 == 0): T * n/32 * (16 + 1) half2 */
size_t p1a_a16_bytes(int T, int n);
/*
 * Elementwise gate + a16 quantize over [T][n]: op 0: y = silu(a) * b, op 1: y = a * sigmoid(b); qbuf = a16(y).
 * lda / ldb (0 = n) are the row strides of a and b; y is dense and may alias a when lda == n. n % 32 == 0.
 * Replaces ew_quant (src/fast/fused.cuh:92-98, kernel src/fast/fused.cu:478-496).
 */
int p1a_ew_quant(int op, const float *a, const float *b, float *y, void *qbuf, int T, int n, int lda, int ldb, void *stream);

/*
 * Chunked causal prefill: q, out [T][Hq][D] f32, query t at position p0 + t sees cache positions 0..p0+t of ONE
 * sequence (page table pt + (rtab ? rtab[0] : 0)); the cache must already hold positions 0..p0+T-1 (append first).
 * fp16 MFMA products with fp32 accumulation; gate as in p1a_attn_decode. `scratch` is optional caller-supplied device
 * memory (256-byte aligned): with at least p1a_attn_prefill_scratch_bytes(...) bytes a q8_0 / q4_0 cache is converted to
 * f16 once per call instead of once per workgroup (same result bits, about 10-35 % less time). With less, or NULL - the
 * reference's attn_prefill brings none - the library uses a staging copy of its own, kept per (device, stream) like its
 * split scratch (allocated and grown outside stream capture only, never freed before p1a_release, at most
 * p1a_set_prefill_staging_limit bytes, 1 GiB unless set); where it has none the kernel converts on the fly. Results do not
 * depend on which of the three happened. Rows of the cache past position p0 + T - 1 may be fetched (never past the end of a
 * page, or of a contiguous cache) but are never weighted, whatever they hold.
 * Replaces attn_prefill (src/fast/attn.cuh:46-50) and attn_fold (src/fast/attn_fold.cuh:19-26).
 */
int p1a_attn_prefill(const float *q, const p1a_kv *c, float *out, const float *gate, int T, int p0, int Hq,
                     float scale, void *scratch, size_t scratch_bytes, void *stream);
/* bytes of scratch that enable the convert-once variant and hold the partials of a key-split call:
 * roundup(2 * roundup(p0 + T, 16) * Hkv * D * 2, 256) + (key splits > 1 ? roundup(T * Hq * splits * 8, 256) + T * Hq * splits * D * 4 : 0).
 * Replaces attn_fold_scratch_bytes (src/fast/attn_fold.cuh:19). */
size_t p1a_attn_prefill_scratch_bytes(int T, int p0, int Hq, int Hkv, int D);
/* Key splits a prefill call of this shape takes on the current device (1 = none). A chunk of few token blocks over a long
 * context (the last chunk of a prompt, a short turn of a long chat) would occupy T/128 * Hq workgroups, each walking every
 * key; its keys are then dealt to several workgroups per (token block, q head) and the partials merged (the nsplit of
 * attn_fold, src/fast/attn_fold.cuh:19-26, chosen by the library). The count depends on (T, p0, Hq) and the device's CU
 * count only, never on the scratch passed or on the state of the stream; partials that do not fit the caller's scratch
 * live in buffers the library keeps per (device, stream) for this purpose (never freed before p1a_release). They cannot
 * be allocated during stream capture: such a call is refused with P1A_E_SCRATCH unless p1a_warmup_prefill (or an eager
 * call of the shape) came first. */
int p1a_attn_prefill_key_splits(int T, int p0, int Hq);
/* Largest f16 staging copy the library keeps per (device, stream) for p1a_attn_prefill calls without caller scratch
 * (bytes; 0 = never: such calls convert inside the kernel). No counterpart in the reference. */
void p1a_set_prefill_staging_limit(size_t bytes);
/* Allocate the library's key-split partial buffers of (current device, stream) for a prefill call of this shape (a no-op
 * for shapes that take one split) and its f16 staging copy (when within the limit), so that the call can be captured. No counterpart in the reference, whose attn_fold
 * takes all scratch from the caller (src/fast/attn_fold.cuh:25-26). */
int p1a_warmup_prefill(int T, int p0, int Hq, int Hkv, int D, void *stream);

/* Standalone sigmoid gate x[i] *= 1 / (1 + exp(-g[i])). Replaces k::sigmoid_mul, src/kernels.cu:85-93. */
int p1a_sigmoid_mul(float *x, const float *g, size_t n, void *stream);

/*
 * Allocate the split-K scratch of (current device, stream) for Hq heads of size D (always at the P1A_MAX_ROWS footprint:
 * `rows` is only checked), so that later decode calls of that head shape on that stream never allocate (graph
 * capture). Mirrors the warm-up call the reference asks for (src/fast/attn.cuh:40-42; the reference allocates at its
 * ATTN_MAX_ROWS footprint on first use, src/fast/attn_dec2.cu:452-464,503-517).
 */
int p1a_warmup(int rows, int Hq, int Hkv, int D, void *stream);
/* split-stream count used for Hkv kv heads on the current device / override it (0 = default). Mirror
 * attn_dec2_nsplit / attn_dec2_set_nsplit, src/fast/attn_dec2.cuh:19-20. Never change it between graph captures. */
int p1a_get_nsplit(int Hkv);
void p1a_set_nsplit(int n);
/* Bytes of split scratch one decode call of these arguments needs (accumulators rounded up to 256 bytes, then the (m, l)
 * pairs), and the bytes the library keeps per (device, stream) for a head shape - the larger of the two is what a first call
 * allocates. A cache the MFMA kernel cannot take (misaligned base or page stride, pages of fewer than 16 positions, head
 * sizes other than 64 / 128 / 256) takes the generic kernel, which leaves more partials per row; both are covered. No GPU call is made
 * (without a device the plan of a 256-CU part is returned). No counterpart in the reference, whose scratch size is a
 * compile-time constant (src/fast/attn_dec2.cu:452-464). rows_per_seq as for p1a_attn_decode (T for a call without
 * pos_rows). */
size_t p1a_decode_scratch_bytes(const p1a_kv *c, int Hq, int T, int rows_per_seq);
size_t p1a_decode_footprint_bytes(int Hq, int Hkv, int D);
/* An identity of everything in this library that can change output BITS for a head shape on the current device: library
 * version and numerics revision, CU count, split-stream count (P1A_DEC_SPLIT / p1a_set_nsplit included). Two processes with
 * equal ids produce bit-identical attention outputs for equal inputs; the engine folds such switches into the numerics
 * hash of its session files (src/tp_model.cu:3697-3735). The prefill key-split plan is a function of (T, p0, Hq) and the
 * CU count, so it is covered. */
#define P1A_NUMERICS_REV 4
uint64_t p1a_numerics_id(int Hq, int Hkv);
/* Re-read the environment switch that is baked into captured graphs (P1A_DEC_SPLIT, the split-stream count); returns 1
 * when it differs from what was last read - the very first read included, as in the reference - (the caller must then drop
 * its captured graphs), else 0.
 * Replaces attn_dec2_reload_env, src/fast/attn_dec2.cuh:21 (called from src/tp_model.cu:3229). */
int p1a_reload_env(void);
/* Benchmarks only (no counterpart in the reference, whose benches time both kernels together): p1a_attn_decode without
 * its merge kernel - the split-K kernel runs and leaves its partials in the library's scratch, `out` is untouched - so
 * that kernel can be event-timed alone. The flag is an argument of this call: no process-wide state. */
int p1a_bench_decode_split_only(const float *q, const p1a_kv *c, float *out, int T, int p0, const int32_t *p0_dev,
                                const int32_t *pos_rows, int rows_per_seq, int Hq, float scale, void *stream);
/* Benchmarks only (no counterpart in the reference): a plain read of `bytes` bytes of device memory (16 bytes per lane,
 * one contiguous span per workgroup, four workgroups per compute unit, nothing computed) - the time the memory system needs for a launch of that size,
 * to set a decode launch of the same number of KV bytes against. bytes is rounded down to a multiple of 16. */
int p1a_bench_stream_read(const void *src, size_t bytes, void *stream);
/* free every scratch buffer of the current process (after synchronising the devices that own them); graphs captured
 * before this call must not be replayed after it */
void p1a_release(void);

const char *p1a_last_error(void);
const char *p1a_version(void);

#ifdef __cplusplus
}
#endif
#endif /* P1A_ATTN_H */
