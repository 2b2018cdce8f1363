// extern "C" layer of the paged-KV attention library: argument validation (refusals launch nothing), split-K
// scratch ownership per (device, stream), split-count bookkeeping. All device work lives in the other .hip files.
#include "p1a_common.hpp"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace p1a {

static thread_local char g_err[256] = "";

void set_error(const char * fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    fprintf(stderr, "p1a_attn: %s\n", g_err);
}

namespace {

// Split partials per (device, stream): calls on different streams of one device may overlap; a stream keeps its
// buffer (captured graphs hold the pointer), which only ever grows, and only outside capture.
struct scratch { int dev = -1; hipStream_t s = nullptr; float * o = nullptr; float * ml = nullptr; size_t cap_o = 0, cap_ml = 0; };
constexpr int MAX_SCR = 64;
scratch g_scr[MAX_SCR];
int g_nscr = 0;
std::mutex g_mu;
int g_nsplit_override = 0;
bool g_skip_merge = false;
int g_cus[16] = {0};

}   // namespace

int cu_count() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    int & n = g_cus[dev & 15];
    if (!n && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 256;
    return n;
}

namespace {

scratch * scratch_for(hipStream_t s, size_t need_o, size_t need_ml, bool quiet = false) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lk(g_mu);
    scratch * e = nullptr;
    for (int i = 0; i < g_nscr; ++i) if (g_scr[i].dev == dev && g_scr[i].s == s) e = &g_scr[i];
    if (!e) {
        if (g_nscr == MAX_SCR) { if (!quiet) set_error("too many (device, stream) pairs"); return nullptr; }
        e = &g_scr[g_nscr++];
        e->dev = dev; e->s = s;
    }
    if (need_o > e->cap_o || need_ml > e->cap_ml) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (s && hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone) {
            if (!quiet) set_error("split scratch would have to grow during stream capture: call p1a_warmup first");
            return nullptr;
        }
        float * no = nullptr, * nm = nullptr;
        if (hipMalloc(&no, need_o) != hipSuccess || hipMalloc(&nm, need_ml) != hipSuccess) {
            (void) hipGetLastError();
            if (no) (void) hipFree(no);
            if (!quiet) set_error("split scratch allocation failed (%zu bytes)", need_o + need_ml);
            return nullptr;
        }
        if (e->o) { (void) hipStreamSynchronize(s); (void) hipFree(e->o); (void) hipFree(e->ml); }
        e->o = no; e->ml = nm; e->cap_o = need_o; e->cap_ml = need_ml;
    }
    return e;
}

bool kv_ok(const p1a_kv * c, const char * who) {
    if (!c || !c->k || !c->v) { set_error("%s: null cache", who); return false; }
    if (c->type != P1A_KV_F16 && c->type != P1A_KV_Q8_0 && c->type != P1A_KV_Q4_0) { set_error("%s: unknown KV type %u", who, c->type); return false; }
    if (c->Hkv < 1 || c->D < 32 || c->D % 32 || c->D > 512) { set_error("%s: unsupported shape (Hkv=%d D=%d)", who, c->Hkv, c->D); return false; }
    if (c->pt && (c->psh < 0 || c->psh > 24 || c->pstride == 0)) { set_error("%s: bad page geometry (psh=%d pstride=%zu)", who, c->psh, c->pstride); return false; }
    return true;
}

// requested split-stream count: the setter, then the environment, else 0 = the plan's default for the device
int nsplit_req() {
    static const int env = getenv("P1A_DEC_SPLIT") ? atoi(getenv("P1A_DEC_SPLIT")) : 0;
    return g_nsplit_override > 0 ? g_nsplit_override : (env > 0 ? env : 0);
}

}   // namespace

bool split_scratch(hipStream_t s, size_t bytes_o, size_t bytes_ml, float *& o, float *& ml) {
    scratch * e = scratch_for(s, bytes_o, bytes_ml, true);
    if (!e) return false;
    o = e->o; ml = e->ml;
    return true;
}

}   // namespace p1a

using namespace p1a;

extern "C" {

size_t p1a_kv_row_bytes(uint32_t type, int Hkv, int D) {
    return type == P1A_KV_F16 ? (size_t) Hkv * D * 2 : type == P1A_KV_Q8_0 ? (size_t) Hkv * (D / 32) * 34 : (size_t) Hkv * (D / 32) * 18;
}

int p1a_kv_append(const p1a_kv * c, const float * k, const float * v, int p0, const int32_t * p0_dev,
                  const int32_t * pos_rows, int T, void * stream) {
    if (!kv_ok(c, "p1a_kv_append")) return P1A_E_ARG;
    if (!k || !v || T < 0) { set_error("p1a_kv_append: null input or negative T"); return P1A_E_ARG; }
    if (T == 0) return P1A_OK;
    if ((((uintptr_t) k | (uintptr_t) v) & 15) || (c->Hkv * c->D) % 32) { set_error("p1a_kv_append: k/v must be 16-byte aligned, Hkv*D %% 32 == 0"); return P1A_E_SHAPE; }
    if (T > 65535) { set_error("p1a_kv_append: T=%d exceeds 65535 rows per call", T); return P1A_E_SHAPE; }
    if (!pos_rows && !p0_dev && p0 < 0) { set_error("p1a_kv_append: negative p0"); return P1A_E_ARG; }
    return launch_append(*c, k, v, p0, p0_dev, pos_rows, T, (hipStream_t) stream);
}

int p1a_kv_fill_random(const p1a_kv * c, int p0, int p1, uint32_t seed, void * stream) {
    if (!kv_ok(c, "p1a_kv_fill_random")) return P1A_E_ARG;
    if (p0 < 0) { set_error("p1a_kv_fill_random: negative p0"); return P1A_E_ARG; }
    if (p1 <= p0) return P1A_OK;
    if (c->type != P1A_KV_F16 && c->D % 32) { set_error("p1a_kv_fill_random: D %% 32 != 0"); return P1A_E_SHAPE; }
    if (!c->pt && p1 > c->n_ctx) { set_error("p1a_kv_fill_random: positions up to %d in a cache of %d", p1, c->n_ctx); return P1A_E_ARG; }
    return launch_fill_random(*c, p0, p1, seed, (hipStream_t) stream);
}

int p1a_attn_prep(const float * qg, const float * k, const float * v, const float * q_norm, const float * k_norm,
                  const int32_t * pos, float * q, float * gate, const p1a_kv * c, int p0, int T, int Hq, int n_rot,
                  float freq_base, float eps, int ldq, int ldk, int ldv, void * stream) {
    return p1a_attn_prep_mrope(qg, k, v, q_norm, k_norm, pos, q, gate, c, p0, T, Hq, n_rot, freq_base, eps, ldq, ldk, ldv,
                               nullptr, 0, 0, 0, 0, 0, stream);
}

int p1a_attn_prep_mrope(const float * qg, const float * k, const float * v, const float * q_norm, const float * k_norm,
                        const int32_t * pos, float * q, float * gate, const p1a_kv * c, int p0, int T, int Hq, int n_rot,
                        float freq_base, float eps, int ldq, int ldk, int ldv, const int32_t * mr_pos, int mr_stride,
                        int s0, int s1, int s2, int sect, void * stream) {
    if (!kv_ok(c, "p1a_attn_prep")) return P1A_E_ARG;
    if (mr_pos && (sect <= 0 || mr_stride < T || s0 < 0 || s1 < 0 || s2 < 0)) {
        set_error("p1a_attn_prep: M-RoPE needs sect > 0, sections >= 0 and a stream stride of at least T (sect=%d stride=%d)", sect, mr_stride);
        return P1A_E_ARG;
    }
    if (!qg || !k || !v || !pos || !q || !gate || T < 0 || Hq < 1) { set_error("p1a_attn_prep: null argument or bad T / Hq"); return P1A_E_ARG; }
    if (T == 0) return P1A_OK;
    const int D = c->D, Hkv = c->Hkv;
    if (D > 256 || n_rot < 0 || n_rot % 8 || n_rot > D || T > 65535) {
        set_error("p1a_attn_prep: unsupported shape (D=%d n_rot=%d T=%d): D <= 256, n_rot %% 8 == 0, n_rot <= D", D, n_rot, T);
        return P1A_E_SHAPE;
    }
    if (!ldq) ldq = Hq * 2 * D;
    if (!ldk) ldk = Hkv * D;
    if (!ldv) ldv = Hkv * D;
    const uintptr_t al = (uintptr_t) qg | (uintptr_t) k | (uintptr_t) v | (uintptr_t) q | (uintptr_t) gate | (uintptr_t) q_norm | (uintptr_t) k_norm;
    if ((al & 15) || ((ldq | ldk | ldv) & 3) || ldq < Hq * 2 * D || ldk < Hkv * D || ldv < Hkv * D) {
        set_error("p1a_attn_prep: pointers must be 16-byte aligned, row strides multiples of 4 floats and at least one row");
        return P1A_E_SHAPE;
    }
    const mrope_view mr{mr_pos, mr_stride, s0, s1, s2, sect};
    return launch_prep(*c, qg, k, v, q_norm, k_norm, pos, q, gate, p0, T, Hq, n_rot, freq_base, eps, ldq, ldk, ldv, mr, (hipStream_t) stream);
}

size_t p1a_a16_bytes(int T, int n) { return T < 0 || n < 0 ? 0 : (size_t) T * (size_t) (n / 32) * 17 * 4; }

int p1a_ew_quant(int op, const float * a, const float * b, float * y, void * qbuf, int T, int n, int lda, int ldb, void * stream) {
    if (!a || !b || !y || !qbuf || T < 0 || (op != 0 && op != 1)) { set_error("p1a_ew_quant: null argument, negative T or unknown op"); return P1A_E_ARG; }
    if (T == 0) return P1A_OK;
    if (!lda) lda = n;
    if (!ldb) ldb = n;
    const uintptr_t al = (uintptr_t) a | (uintptr_t) b | (uintptr_t) y | (uintptr_t) qbuf;
    if (n < 32 || n % 32 || (al & 15) || ((lda | ldb) & 3) || lda < n || ldb < n || T > 65535 || (y == a && lda != n)) {
        set_error("p1a_ew_quant: n %% 32 == 0, 16-byte aligned pointers, row strides multiples of 4 and >= n (y may alias a only when dense)");
        return P1A_E_SHAPE;
    }
    return launch_ew_quant(op, a, b, y, qbuf, T, n, lda, ldb, (hipStream_t) stream);
}

int p1a_attn_decode(const float * q, const p1a_kv * c, float * out, const float * gate, int T, int p0,
                    const int32_t * p0_dev, const int32_t * pos_rows, int rows_per_seq, int Hq, float scale,
                    void * stream) {
    return p1a_attn_decode_a16(q, c, out, gate, nullptr, T, p0, p0_dev, pos_rows, rows_per_seq, Hq, scale, stream);
}

int p1a_attn_decode_a16(const float * q, const p1a_kv * c, float * out, const float * gate, void * qbuf, int T, int p0,
                        const int32_t * p0_dev, const int32_t * pos_rows, int rows_per_seq, int Hq, float scale,
                        void * stream) {
    if (!kv_ok(c, "p1a_attn_decode")) return P1A_E_ARG;
    if (qbuf && (((uintptr_t) qbuf & 15) || (Hq * c->D) % 32)) { set_error("p1a_attn_decode: qbuf must be 16-byte aligned and Hq*D %% 32 == 0"); return P1A_E_SHAPE; }
    if (!q || !out) { set_error("p1a_attn_decode: null q/out"); return P1A_E_ARG; }
    if (T < 1 || T > P1A_MAX_ROWS || Hq < c->Hkv || Hq % c->Hkv) {
        set_error("p1a_attn_decode: unsupported shape (D=%d Hq=%d Hkv=%d T=%d)", c->D, Hq, c->Hkv, T);
        return P1A_E_SHAPE;
    }
    if ((((uintptr_t) q | (uintptr_t) out | (uintptr_t) gate) & 15)) { set_error("p1a_attn_decode: q/out/gate must be 16-byte aligned"); return P1A_E_SHAPE; }
    if (!pos_rows && !p0_dev && p0 < 0) { set_error("p1a_attn_decode: negative p0"); return P1A_E_ARG; }
    hipStream_t s = (hipStream_t) stream;
    decode_args a;
    a.q = q; a.out = out; a.gate = gate; a.T = T; a.p0 = p0; a.p0_dev = p0_dev; a.pos_rows = pos_rows;
    a.Hq = Hq; a.scale = scale;
    a.rows_per_group = decode_rows_per_group(*c, Hq, pos_rows ? (rows_per_seq < 1 ? 1 : rows_per_seq) : T);
    // a sequence's rows must split into whole groups, or a group would mix two sequences
    while (pos_rows && rows_per_seq > 1 && rows_per_seq % a.rows_per_group) --a.rows_per_group;
    a.nsplit = nsplit_req();
    a.cus = cu_count();
    a.skip_merge = g_skip_merge;
    a.qbuf = qbuf;
    size_t need_o, need_ml;
    decode_scratch_need(*c, Hq, T < 8 ? 8 : T, a.rows_per_group, a.nsplit, a.cus, need_o, need_ml);
    scratch * sc = scratch_for(s, need_o, need_ml);
    if (!sc) return P1A_E_SCRATCH;
    a.part_o = sc->o; a.part_ml = sc->ml;
    return launch_decode(*c, a, s);
}

int p1a_warmup(int rows, int Hq, int Hkv, int D, void * stream) {
    if (rows < 1 || rows > P1A_MAX_ROWS || Hq < 1 || Hkv < 1 || Hq % Hkv || D < 32) { set_error("p1a_warmup: bad shape"); return P1A_E_ARG; }
    // the largest footprint over the kernels and row groupings a (Hq, Hkv, D) cache can take
    p1a_kv c;
    memset(&c, 0, sizeof c);
    c.Hkv = Hkv; c.D = D; c.k = c.v = (void *) 16;
    size_t need_o = 0, need_ml = 0;
    const uint32_t types[3] = {P1A_KV_F16, P1A_KV_Q8_0, P1A_KV_Q4_0};
    for (uint32_t ty : types)
        for (int rg = 1; rg <= 4; ++rg) {
            size_t o, m;
            c.type = ty;
            decode_scratch_need(c, Hq, rows < 8 ? 8 : rows, rg, nsplit_req(), cu_count(), o, m);
            if (o > need_o) need_o = o;
            if (m > need_ml) need_ml = m;
        }
    return scratch_for((hipStream_t) stream, need_o, need_ml) ? P1A_OK : P1A_E_SCRATCH;
}

int p1a_attn_prefill(const float * q, const p1a_kv * c, float * out, const float * gate, int T, int p0, int Hq,
                     float scale, void * scratch, size_t scratch_bytes, void * stream) {
    if (!kv_ok(c, "p1a_attn_prefill")) return P1A_E_ARG;
    if (!q || !out || T < 1 || p0 < 0) { set_error("p1a_attn_prefill: bad argument"); return P1A_E_ARG; }
    if (Hq < c->Hkv || Hq % c->Hkv) { set_error("p1a_attn_prefill: unsupported shape (Hq=%d Hkv=%d)", Hq, c->Hkv); return P1A_E_SHAPE; }
    if ((((uintptr_t) q | (uintptr_t) out | (uintptr_t) gate) & 15)) { set_error("p1a_attn_prefill: q/out/gate must be 16-byte aligned"); return P1A_E_SHAPE; }
    return launch_prefill(*c, q, out, gate, T, p0, Hq, scale, scratch, scratch_bytes, (hipStream_t) stream);
}

int p1a_sigmoid_mul(float * x, const float * g, size_t n, void * stream) {
    if (!x || !g) { set_error("p1a_sigmoid_mul: null argument"); return P1A_E_ARG; }
    if (!n) return P1A_OK;
    return launch_sigmoid_mul(x, g, n, (hipStream_t) stream);
}

int p1a_get_nsplit(int Hkv) {
    p1a_kv c;
    memset(&c, 0, sizeof c);
    c.type = P1A_KV_Q8_0; c.Hkv = Hkv < 1 ? 1 : Hkv; c.D = 256; c.k = c.v = (void *) 16;
    return decode_nsplit(c, 6 * c.Hkv, nsplit_req(), cu_count());
}

void p1a_set_nsplit(int n) { g_nsplit_override = n > 0 ? n : 0; }

void p1a_bench_skip_merge(int on) { g_skip_merge = on != 0; }

int p1a_bench_stream_read(const void * src, size_t bytes, void * stream) {
    if (!src || bytes < 16 || ((uintptr_t) src & 15)) { set_error("p1a_bench_stream_read: null, short or misaligned source"); return P1A_E_ARG; }
    return launch_stream_read(src, bytes, (hipStream_t) stream);
}

void p1a_release(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    int cur = 0;
    (void) hipGetDevice(&cur);
    for (int i = 0; i < g_nscr; ++i) {
        if (!g_scr[i].o) continue;
        (void) hipSetDevice(g_scr[i].dev);
        (void) hipDeviceSynchronize();
        (void) hipFree(g_scr[i].o);
        (void) hipFree(g_scr[i].ml);
        g_scr[i] = scratch{};
    }
    g_nscr = 0;
    (void) hipSetDevice(cur);
}

const char * p1a_last_error(void) { return g_err; }
const char * p1a_version(void) { return "p1a_attn 0.1 (gfx950)"; }

}   // extern "C"
