// C++ mirror of the reference engine's attention call surface (namespace p100e::fast) for MI355X.
//
// Same names, argument order, defaults and error behaviour as the reference headers (paths relative to the reference
// tree): src/fast/attn.cuh:12-70, src/fast/attn_dec2.cuh:17-21, src/fast/attn_fold.cuh:18-26. cudaStream_t becomes
// hipStream_t; src/fast/fused.cuh:101-113 (attn_prep) is mirrored too; everything is a thin inline call into the C ABI of include/p1a_attn.h (libp1a_attn.so), so a caller
// that links the reference's static library p100e_fast_attn can link this instead without touching its call sites.
// Additions, all optional: a trailing `gate` argument (fused sigmoid output gate; nullptr = the reference's
// behaviour) and `rows_per_seq` on attn_decode_rows (verify blocks that share one KV read).
#pragma once
#include <cstddef>
#include <cstdint>
#include <hip/hip_runtime_api.h>

#include "p1a_attn.h"

namespace p100e::fast {

constexpr uint32_t KV_F16 = P1A_KV_F16;     // == GGML_TYPE_F16    (src/fast/attn.cuh:14)
constexpr uint32_t KV_Q4_0 = P1A_KV_Q4_0;   // == GGML_TYPE_Q4_0   (src/fast/attn.cuh:15)
constexpr uint32_t KV_Q8_0 = P1A_KV_Q8_0;   // == GGML_TYPE_Q8_0   (src/fast/attn.cuh:16)

// src/fast/attn.cuh:18-32, field for field
struct kv_cache {
    uint32_t type = KV_F16;
    int n_ctx = 0, Hkv = 0, D = 0;
    void * k = nullptr;
    void * v = nullptr;
    const int32_t * pt = nullptr;
    const int32_t * rtab = nullptr;
    int psh = 0;
    size_t pstride = 0;
};

namespace detail {
inline p1a_kv pod(const kv_cache & c) {
    p1a_kv r;
    r.type = c.type; r.n_ctx = c.n_ctx; r.Hkv = c.Hkv; r.D = c.D;
    r.k = c.k; r.v = c.v; r.pt = c.pt; r.rtab = c.rtab; r.psh = c.psh; r.pstride = c.pstride;
    return r;
}
}   // namespace detail

// src/fast/attn.cuh:34
inline size_t kv_row_bytes(uint32_t type, int Hkv, int D) { return p1a_kv_row_bytes(type, Hkv, D); }

// src/fast/attn.cuh:35-36: contiguous test / bench caches; k == nullptr on failure. Zero-filled.
inline void kv_free(kv_cache & c) {
    if (c.k) (void) hipFree(c.k);
    if (c.v) (void) hipFree(c.v);
    c.k = c.v = nullptr;
}
inline kv_cache kv_alloc(uint32_t type, int n_ctx, int Hkv, int D) {
    kv_cache c;
    c.type = type; c.n_ctx = n_ctx; c.Hkv = Hkv; c.D = D;
    if (type != KV_F16 && type != KV_Q4_0 && type != KV_Q8_0) return c;
    if (type != KV_F16 && D % 32) return c;
    const size_t bytes = kv_row_bytes(type, Hkv, D) * (size_t) n_ctx;
    if (hipMalloc(&c.k, bytes) != hipSuccess || hipMalloc(&c.v, bytes) != hipSuccess ||
        hipMemset(c.k, 0, bytes) != hipSuccess || hipMemset(c.v, 0, bytes) != hipSuccess) {
        (void) hipGetLastError();
        kv_free(c);
    }
    return c;
}

// src/fast/attn.cuh:70 (attn.cu:559-581): benchmark fill of positions p0 .. p1 - 1, the same bytes for the same seed
inline void kv_fill_random(kv_cache & c, int p0, int p1, uint32_t seed, hipStream_t s) {
    if (!c.k || p1 <= p0) return;
    const p1a_kv p = detail::pod(c);
    (void) p1a_kv_fill_random(&p, p0, p1, seed, s);
}

// src/fast/attn.cuh:37-38
inline void kv_append(kv_cache & c, const float * k, const float * v, int p0, int T, hipStream_t s) {
    const p1a_kv p = detail::pod(c);
    (void) p1a_kv_append(&p, k, v, p0, nullptr, nullptr, T, s);
}
// src/fast/attn.cuh:58
inline void kv_append_dev(kv_cache & c, const float * k, const float * v, const int32_t * p0_dev, int T, hipStream_t s) {
    const p1a_kv p = detail::pod(c);
    (void) p1a_kv_append(&p, k, v, 0, p0_dev, nullptr, T, s);
}
// The cache-write half of attn_prep in its device-position mode (src/fast/fused.cuh:101-113 with p0 < 0): row t goes
// to position pos[t] of its own sequence (c.rtab). k is expected normed and roped already.
inline bool kv_append_rows(kv_cache & c, const float * k, const float * v, const int32_t * pos, int T, hipStream_t s) {
    const p1a_kv p = detail::pod(c);
    return p1a_kv_append(&p, k, v, -1, nullptr, pos, T, s) == P1A_OK;
}

// src/fast/mrope.cuh:14-19, field for field
struct mrope_pos {
    const int32_t * p = nullptr;   // device [3][stride] positions (t, h, w) of the rows; nullptr = plain NEOX
    int stride = 0;                // row stride between the three streams
    int s0 = 0, s1 = 0, s2 = 0;    // sections (in rotary pairs)
    int sect = 0;                  // sum of all sections
};

// src/fast/fused.cuh:101-113 (Hkv and D must be the cache's)
inline bool attn_prep(const float * qg, const float * k, const float * v, const float * q_norm, const float * k_norm,
                      const int32_t * pos, float * q, float * gate, kv_cache & c, int p0, int T, int Hq, int Hkv, int D,
                      int n_rot, float freq_base, float eps, hipStream_t s, int ldq = 0, int ldk = 0, int ldv = 0,
                      const mrope_pos & mr = mrope_pos{}) {
    if (Hkv != c.Hkv || D != c.D) return false;
    const p1a_kv p = detail::pod(c);
    return p1a_attn_prep_mrope(qg, k, v, q_norm, k_norm, pos, q, gate, &p, p0, T, Hq, n_rot, freq_base, eps, ldq, ldk, ldv,
                               mr.p, mr.stride, mr.s0, mr.s1, mr.s2, mr.sect, s) == P1A_OK;
}

// src/fast/fused.cuh:91-98
enum ew_op : int { EW_SILU_MUL = 0, EW_SIGMOID_MUL = 1 };
inline bool ew_quant(ew_op op, const float * a, const float * b, float * y, void * qbuf, int T, int n, hipStream_t s,
                     int lda = 0, int ldb = 0) {
    return p1a_ew_quant((int) op, a, b, y, qbuf, T, n, lda, ldb, s) == P1A_OK;
}

// src/fast/attn.cuh:39-44. false = nothing launched, out untouched.
inline bool attn_decode(const float * q, const kv_cache & c, float * out, int T, int p0, int Hq, float scale,
                        hipStream_t s, const float * gate = nullptr) {
    const p1a_kv p = detail::pod(c);
    return p1a_attn_decode(q, &p, out, gate, T, p0, nullptr, nullptr, 0, Hq, scale, s) == P1A_OK;
}
// src/fast/attn.cuh:59-60 (max_n is accepted for source compatibility: the grid never depends on the depth)
// (qbuf: also emit the a16 activation buffer of the gated rows, i.e. the ew_quant(EW_SIGMOID_MUL) that follows in the engine)
inline bool attn_decode_dev(const float * q, const kv_cache & c, float * out, int T, const int32_t * p0_dev, int max_n,
                            int Hq, float scale, hipStream_t s, const float * gate = nullptr, void * qbuf = nullptr) {
    (void) max_n;
    const p1a_kv p = detail::pod(c);
    return p1a_attn_decode_a16(q, &p, out, gate, qbuf, T, 0, p0_dev, nullptr, 0, Hq, scale, s) == P1A_OK;
}
// src/fast/attn.cuh:61-66
constexpr int ATTN_MAX_ROWS = P1A_MAX_ROWS;
inline bool attn_decode_rows(const float * q, const kv_cache & c, float * out, int T, const int32_t * pos, int Hq,
                             float scale, hipStream_t s, const float * gate = nullptr, int rows_per_seq = 1,
                             void * qbuf = nullptr) {
    if (!pos) return false;
    const p1a_kv p = detail::pod(c);
    return p1a_attn_decode_a16(q, &p, out, gate, qbuf, T, 0, nullptr, pos, rows_per_seq, Hq, scale, s) == P1A_OK;
}
// src/fast/attn_dec2.cuh:17-20
inline bool attn_decode2(const float * q, const kv_cache & c, float * out, int T, int p0, const int32_t * p0_dev, int Hq,
                         float scale, hipStream_t s, const int32_t * pos_rows = nullptr) {
    const p1a_kv p = detail::pod(c);
    return p1a_attn_decode(q, &p, out, nullptr, T, p0, p0_dev, pos_rows, 1, Hq, scale, s) == P1A_OK;
}
inline int attn_dec2_nsplit(int Hkv) { return p1a_get_nsplit(Hkv); }
inline void attn_dec2_set_nsplit(int n) { p1a_set_nsplit(n); }
// src/fast/attn_dec2.cuh:21: re-read the environment switch baked into captured graphs (here P1A_DEC_SPLIT); true if it
// changed, i.e. the caller's graphs must be dropped (src/tp_model.cu:3229)
inline bool attn_dec2_reload_env() { return p1a_reload_env() != 0; }

// src/fast/attn.cuh:46-53
inline bool attn_prefill(const float * q, const kv_cache & c, float * out, int T, int p0, int Hq, float scale,
                         hipStream_t s, const float * gate = nullptr) {
    const p1a_kv p = detail::pod(c);
    return p1a_attn_prefill(q, &p, out, gate, T, p0, Hq, scale, nullptr, 0, s) == P1A_OK;
}
inline bool attn_prefill_variant(const float * q, const kv_cache & c, float * out, int T, int p0, int Hq, float scale,
                                 hipStream_t s, int /*variant: one kernel here*/) {
    return attn_prefill(q, c, out, T, p0, Hq, scale, s);
}
// src/fast/attn_fold.cuh:19-26 (chunk / nsplit are accepted and ignored: P never leaves the chip, and the library picks
// the key splits of a short chunk over a long context itself, p1a_attn_prefill_key_splits). The scratch is optional
// here: a buffer of attn_fold_scratch_bytes(T, Hkv, ..., p0) bytes lets a quantized cache be converted to f16 once per
// call and holds the split partials; the reference's own size (which knows nothing of p0) is accepted too: what does
// not fit takes the on-the-fly kernel / the library's own buffers, with the same result bits.
inline size_t attn_fold_scratch_bytes(int T, int Hkv, int /*chunk*/, int /*nsplit*/, int p0 = 0) {
    return p1a_attn_prefill_scratch_bytes(T, p0, 6 * Hkv, Hkv, 256);
}
inline bool attn_fold(const float * q, const kv_cache & c, float * out, int T, int p0, int Hq, float scale, void * scratch,
                      size_t scratch_bytes, hipStream_t s, int /*chunk*/ = 0, int /*nsplit*/ = 0, const float * gate = nullptr) {
    const p1a_kv p = detail::pod(c);
    return p1a_attn_prefill(q, &p, out, gate, T, p0, Hq, scale, scratch, scratch_bytes, s) == P1A_OK;
}

// src/kernels.cuh sigmoid_mul (src/kernels.cu:85-93): x *= sigmoid(g)
inline void sigmoid_mul(float * x, const float * g, int64_t n, hipStream_t s) { (void) p1a_sigmoid_mul(x, g, (size_t) n, s); }

}   // namespace p100e::fast
