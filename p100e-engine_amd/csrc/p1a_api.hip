// extern "C" layer of the paged-KV attention library: argument validation (refusals launch nothing), split-K
// scratch ownership per (device, stream), split-count bookkeeping. All device work lives in the other .hip files.
#include "p1a_common.hpp"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

// Split scratch of the allocation-free decode entry point (p1a_attn_decode_noalloc): a fixed array in device memory,
// one copy per GPU, held until the process ends. In host code the array's NAME is only a handle: its device address is
// asked for once per device with hipGetSymbolAddress and only that address is ever handed to kernels.
static __device__ __align__(256) unsigned char scratch[P1A_NOALLOC_SCRATCH_BYTES];

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

// Split partials per (device, stream): calls on different streams of one device may overlap. A captured graph holds the
// pointers it was recorded with, so a buffer is NEVER freed while the library lives: the decode buffers are allocated on
// the first call at the footprint of P1A_MAX_ROWS rows of that call's head shape (every KV type and row grouping), and
// in the rare case that a later call needs more (another head shape, a larger split count) the new buffer replaces the
// old one only for later calls - the old one stays allocated (g_retired) until p1a_release(). Nothing is allocated
// while the stream is being captured. The partials of a key-split prefill have a pair of their own.
struct bufpair { float * o = nullptr; float * ml = nullptr; size_t cap_o = 0, cap_ml = 0; };
struct stream_bufs { int dev = -1; hipStream_t s = nullptr; bufpair dec, pf; void * stage = nullptr; size_t cap_stage = 0; bool stage_captured = false; };
constexpr int MAX_SCR = 64;
constexpr int MAX_RETIRED = 1024;
stream_bufs g_scr[MAX_SCR];
int g_nscr = 0;
struct retired { int dev; void * p; };
retired g_retired[MAX_RETIRED];
int g_nretired = 0;
std::mutex g_mu;
int g_nsplit_override = 0;
int g_env_split = -1;   // P1A_DEC_SPLIT as last read (-1 = not read yet)
size_t g_stage_limit = (size_t) 1 << 30;   // largest f16 staging copy the library keeps per (device, stream); 0 = none
int g_cus[16] = {0};
constexpr int MAX_DEV = 64;
void * g_static_scratch[MAX_DEV] = {nullptr};   // device address of `scratch` on each device (nullptr = not asked for yet)

}   // namespace

// the device address of the static split scratch on the CURRENT device (resolved on the first call per device), or
// nullptr with the error set
void * static_scratch() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) { set_error("p1a_attn_decode_noalloc: no current device"); return nullptr; }
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_static_scratch[dev]) {
        void * ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(::scratch));
        if (e != hipSuccess || !ptr) {
            (void) hipGetLastError();
            set_error("p1a_attn_decode_noalloc: hipGetSymbolAddress failed (%s)", hipGetErrorString(e));
            return nullptr;
        }
        g_static_scratch[dev] = ptr;
    }
    return g_static_scratch[dev];
}

int cu_count() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    int & n = g_cus[dev & 15];
    if (!n && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 256;
    return n;
}

namespace {

enum which_buf { BUF_DECODE, BUF_PREFILL };

// the buffer pair `w` of (current device, s) with at least these capacities, or nullptr (error set unless quiet)
bufpair * scratch_for(hipStream_t s, which_buf w, size_t need_o, size_t need_ml, bool quiet = false) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lk(g_mu);
    stream_bufs * e = nullptr;
    for (int i = 0; i < g_nscr; ++i) if (g_scr[i].dev == dev && g_scr[i].s == s) e = &g_scr[i];
    if (!e) {
        if (g_nscr == MAX_SCR) { if (!quiet) set_error("too many (device, stream) pairs"); return nullptr; }
        e = &g_scr[g_nscr++];
        e->dev = dev; e->s = s;
    }
    bufpair & b = w == BUF_DECODE ? e->dec : e->pf;
    if (need_o > b.cap_o || need_ml > b.cap_ml) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (s && hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone) {
            if (!quiet) set_error("split scratch would have to be allocated during stream capture: call p1a_warmup%s first", w == BUF_PREFILL ? "_prefill" : "");
            return nullptr;
        }
        if (b.o && g_nretired + 2 > MAX_RETIRED) { if (!quiet) set_error("split scratch replaced too often"); return nullptr; }
        if (need_o < b.cap_o) need_o = b.cap_o;
        if (need_ml < b.cap_ml) need_ml = b.cap_ml;
        float * no = nullptr, * nm = nullptr;
        if (hipMalloc(&no, need_o) != hipSuccess || hipMalloc(&nm, need_ml) != hipSuccess) {
            (void) hipGetLastError();
            if (no) (void) hipFree(no);
            if (!quiet) set_error("split scratch allocation failed (%zu bytes)", need_o + need_ml);
            return nullptr;
        }
        // the replaced buffers stay allocated: a graph captured earlier on this stream may still write and read them
        if (b.o) { g_retired[g_nretired++] = retired{dev, b.o}; g_retired[g_nretired++] = retired{dev, b.ml}; }
        b.o = no; b.ml = nm; b.cap_o = need_o; b.cap_ml = need_ml;
    }
    return &b;
}

bool kv_ok(const p1a_kv * c, const char * who) {
    if (!c || !c->k || !c->v) { set_error("%s: null cache", who); return false; }
    if (c->type != P1A_KV_F16 && c->type != P1A_KV_Q8_0 && c->type != P1A_KV_Q4_0) { set_error("%s: unknown KV type %u", who, c->type); return false; }
    if (c->Hkv < 1 || c->D < 32 || c->D % 32 || c->D > 512) { set_error("%s: unsupported shape (Hkv=%d D=%d)", who, c->Hkv, c->D); return false; }
    if (c->pt && (c->psh < 0 || c->psh > 24 || c->pstride == 0)) { set_error("%s: bad page geometry (psh=%d pstride=%zu)", who, c->psh, c->pstride); return false; }
    return true;
}

// requested split-stream count: the setter, then the environment, else 0 = the plan's default for the device
int read_env_split() {
    const char * e = getenv("P1A_DEC_SPLIT");
    const int v = e && *e ? atoi(e) : 0;
    return v > 0 ? v : 0;
}
int nsplit_req() {
    if (g_env_split < 0) g_env_split = read_env_split();
    return g_nsplit_override > 0 ? g_nsplit_override : g_env_split;
}

// the decode split buffers of a head shape: P1A_MAX_ROWS rows, the largest need over the KV types and row groupings
void decode_footprint(int Hq, int Hkv, int D, size_t & need_o, size_t & need_ml) {
    p1a_kv c;
    memset(&c, 0, sizeof c);
    c.Hkv = Hkv; c.D = D;
    need_o = need_ml = 0;
    const uint32_t types[3] = {P1A_KV_F16, P1A_KV_Q8_0, P1A_KV_Q4_0};
    // (a cache the MFMA kernel cannot take - a misaligned base, short pages - goes to the generic kernel, which leaves more
    // partials per row: both plans count, so that a warm-up also covers such caches)
    for (uintptr_t base : {(uintptr_t) 16, (uintptr_t) 2})
        for (uint32_t ty : types)
            for (int rg = 1; rg <= 4; ++rg) {
                size_t o, m;
                c.type = ty;
                c.k = c.v = (void *) base;
                decode_scratch_need(c, Hq, P1A_MAX_ROWS, rg, nsplit_req(), cu_count(), o, m);
                if (o > need_o) need_o = o;
                if (m > need_ml) need_ml = m;
            }
}

// ext / ext_bytes: split scratch brought by the caller of this function (the allocation-free entry point); nullptr = the
// library's own per-stream buffers
int decode_call(const float * q, const p1a_kv * c, float * out, const float * gate, void * qbuf, int T, int p0,
                const int32_t * p0_dev, const int32_t * pos_rows, int rows_per_seq, int Hq, float scale, bool split_only,
                hipStream_t s, void * ext = nullptr, size_t ext_bytes = 0) {
    if (!kv_ok(c, "p1a_attn_decode")) return P1A_E_ARG;
    if (qbuf && (((uintptr_t) qbuf & 15) || (Hq * c->D) % 32)) { set_error("p1a_attn_decode: qbuf must be 16-byte aligned and Hq*D %% 32 == 0"); return P1A_E_SHAPE; }
    if (!q || !out) { set_error("p1a_attn_decode: null q/out"); return P1A_E_ARG; }
    if (T < 1 || T > P1A_MAX_ROWS || Hq < c->Hkv || Hq % c->Hkv) {
        set_error("p1a_attn_decode: unsupported shape (D=%d Hq=%d Hkv=%d T=%d)", c->D, Hq, c->Hkv, T);
        return P1A_E_SHAPE;
    }
    if ((((uintptr_t) q | (uintptr_t) out | (uintptr_t) gate) & 15)) { set_error("p1a_attn_decode: q/out/gate must be 16-byte aligned"); return P1A_E_SHAPE; }
    if (!pos_rows && !p0_dev && p0 < 0) { set_error("p1a_attn_decode: negative p0"); return P1A_E_ARG; }
    decode_args a;
    a.q = q; a.out = out; a.gate = gate; a.T = T; a.p0 = p0; a.p0_dev = p0_dev; a.pos_rows = pos_rows;
    a.Hq = Hq; a.scale = scale;
    a.rows_per_group = decode_rows_per_group(*c, Hq, pos_rows ? (rows_per_seq < 1 ? 1 : rows_per_seq) : T);
    // a sequence's rows must split into whole groups, or a group would mix two sequences
    while (pos_rows && rows_per_seq > 1 && rows_per_seq % a.rows_per_group) --a.rows_per_group;
    a.nsplit = nsplit_req();
    a.cus = cu_count();
    a.skip_merge = split_only;
    a.qbuf = qbuf;
    size_t need_o, need_ml;
    if (ext) {
        decode_scratch_need(*c, Hq, T, a.rows_per_group, a.nsplit, a.cus, need_o, need_ml);
        need_o = (need_o + 255) & ~(size_t) 255;
        if (need_o + need_ml > ext_bytes) {
            set_error("p1a_attn_decode_noalloc: this call needs %zu bytes of split scratch, the static buffer holds %zu", need_o + need_ml, ext_bytes);
            return P1A_E_SCRATCH;
        }
        a.part_o = reinterpret_cast<float *>(ext);
        a.part_ml = reinterpret_cast<float *>(reinterpret_cast<char *>(ext) + need_o);
        a.cap_o = need_o; a.cap_ml = ext_bytes - need_o;
        return launch_decode(*c, a, s);
    }
    // the footprint of the head shape (so that the pointer never changes again), and never less than THIS call needs
    size_t real_o, real_ml;
    decode_scratch_need(*c, Hq, T, a.rows_per_group, a.nsplit, a.cus, real_o, real_ml);
    decode_footprint(Hq, c->Hkv, c->D, need_o, need_ml);
    if (real_o > need_o) need_o = real_o;
    if (real_ml > need_ml) need_ml = real_ml;
    bufpair * sc = scratch_for(s, BUF_DECODE, need_o, need_ml);
    if (!sc) return P1A_E_SCRATCH;
    a.part_o = sc->o; a.part_ml = sc->ml;
    a.cap_o = sc->cap_o; a.cap_ml = sc->cap_ml;
    return launch_decode(*c, a, s);
}

}   // namespace

bool split_scratch(hipStream_t s, size_t bytes_o, size_t bytes_ml, float *& o, float *& ml) {
    bufpair * e = scratch_for(s, BUF_PREFILL, bytes_o, bytes_ml);
    if (!e) return false;
    o = e->o; ml = e->ml;
    return true;
}

// The library's own f16 staging copy for a prefill over a quantized cache without caller scratch: a buffer of at least
// `bytes` bytes of (current device, s), or nullptr when there is none to be had now - over the limit, allocation failed, or
// the stream is being captured and the buffer would have to be allocated or grown. Never an error: the caller then
// converts inside the kernel, with the same result bits. Grown in steps (64 MiB granules, at least half as much again).
// A replaced buffer is freed on the spot (hipFree waits for the work that still reads it) unless a call under stream
// capture has been handed it - a captured graph holds its address - in which case it stays allocated until
// p1a_release(): what the library keeps per (device, stream) is at most the limit, plus what graphs pin.
void * stage_scratch(hipStream_t s, size_t bytes) {
    int dev = 0;
    if (!bytes || bytes > g_stage_limit || hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lk(g_mu);
    stream_bufs * e = nullptr;
    for (int i = 0; i < g_nscr; ++i) if (g_scr[i].dev == dev && g_scr[i].s == s) e = &g_scr[i];
    if (!e) {
        if (g_nscr == MAX_SCR) return nullptr;
        e = &g_scr[g_nscr++];
        e->dev = dev; e->s = s;
    }
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    const bool capturing = s && hipStreamIsCapturing(s, &st) == hipSuccess && st != hipStreamCaptureStatusNone;
    if (bytes <= e->cap_stage) { if (capturing) e->stage_captured = true; return e->stage; }
    if (capturing) return nullptr;
    if (e->stage && e->stage_captured && g_nretired + 1 > MAX_RETIRED) return nullptr;
    const size_t gran = (size_t) 64 << 20;
    size_t want = (bytes + gran - 1) / gran * gran;
    if (want < e->cap_stage + e->cap_stage / 2) want = e->cap_stage + e->cap_stage / 2;
    if (want > g_stage_limit) want = g_stage_limit;
    if (want < bytes) want = bytes;
    void * p = nullptr;
    if (hipMalloc(&p, want) != hipSuccess) { (void) hipGetLastError(); return nullptr; }
    if (e->stage) {
        if (e->stage_captured) g_retired[g_nretired++] = retired{dev, e->stage};
        else (void) hipFree(e->stage);
    }
    e->stage = p; e->cap_stage = want; e->stage_captured = false;
    return p;
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
    if (!(freq_base > 0.0f) || !(freq_base < 3.0e38f)) { set_error("p1a_attn_prep: freq_base must be a positive finite number"); return P1A_E_ARG; }
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
    return decode_call(q, c, out, gate, qbuf, T, p0, p0_dev, pos_rows, rows_per_seq, Hq, scale, false, (hipStream_t) stream);
}

int p1a_attn_decode_noalloc(const float * q, const p1a_kv * c, float * out, const float * gate, void * qbuf, int T, int p0,
                            const int32_t * p0_dev, const int32_t * pos_rows, int rows_per_seq, int Hq, float scale,
                            void * stream) {
    void * ptr = static_scratch();
    if (!ptr) return P1A_E_SCRATCH;
    return decode_call(q, c, out, gate, qbuf, T, p0, p0_dev, pos_rows, rows_per_seq, Hq, scale, false, (hipStream_t) stream,
                       ptr, P1A_NOALLOC_SCRATCH_BYTES);
}

int p1a_bench_decode_split_only(const float * q, const p1a_kv * c, float * out, int T, int p0, const int32_t * p0_dev,
                                const int32_t * pos_rows, int rows_per_seq, int Hq, float scale, void * stream) {
    return decode_call(q, c, out, nullptr, nullptr, T, p0, p0_dev, pos_rows, rows_per_seq, Hq, scale, true, (hipStream_t) stream);
}

int p1a_warmup(int rows, int Hq, int Hkv, int D, void * stream) {
    if (rows < 1 || rows > P1A_MAX_ROWS || Hq < 1 || Hkv < 1 || Hq % Hkv || D < 32) { set_error("p1a_warmup: bad shape"); return P1A_E_ARG; }
    size_t need_o, need_ml;
    decode_footprint(Hq, Hkv, D, need_o, need_ml);
    (void) static_scratch();   // set-up time: the allocation-free entry point then has nothing left to resolve on this device
    return scratch_for((hipStream_t) stream, BUF_DECODE, need_o, need_ml) ? P1A_OK : P1A_E_SCRATCH;
}

int p1a_warmup_prefill(int T, int p0, int Hq, int Hkv, int D, void * stream) {
    if (T < 1 || p0 < 0 || Hq < 1 || Hkv < 1 || Hq % Hkv || D < 32) { set_error("p1a_warmup_prefill: bad shape"); return P1A_E_ARG; }
    size_t bo, bm;
    prefill_part_need(T, p0, Hq, D, bo, bm);
    // (the f16 staging copy of a quantized cache, when it is within the limit: optional, a call without it converts in the kernel)
    (void) stage_scratch((hipStream_t) stream, prefill_stage_bytes(p0 + T, Hkv, D));
    if (!bo) return P1A_OK;
    return scratch_for((hipStream_t) stream, BUF_PREFILL, bo, bm) ? P1A_OK : P1A_E_SCRATCH;
}

void p1a_set_prefill_staging_limit(size_t bytes) { g_stage_limit = bytes; }

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

size_t p1a_decode_scratch_bytes(const p1a_kv * c, int Hq, int T, int rows_per_seq) {
    if (!c || c->Hkv < 1 || Hq < c->Hkv || Hq % c->Hkv || T < 1) return 0;
    int rg = decode_rows_per_group(*c, Hq, rows_per_seq < 1 ? 1 : rows_per_seq);
    while (rows_per_seq > 1 && rows_per_seq % rg) --rg;
    size_t o, m;
    decode_scratch_need(*c, Hq, T, rg, nsplit_req(), cu_count(), o, m);
    return ((o + 255) & ~(size_t) 255) + m;
}

size_t p1a_decode_footprint_bytes(int Hq, int Hkv, int D) {
    if (Hkv < 1 || Hq < Hkv || Hq % Hkv || D < 32) return 0;
    size_t o, m;
    decode_footprint(Hq, Hkv, D, o, m);
    return ((o + 255) & ~(size_t) 255) + m;
}

uint64_t p1a_numerics_id(int Hq, int Hkv) {
    // FNV-1a over what fixes the summation order of the results on this device
    uint64_t h = 1469598103934665603ull;
    auto mix = [&](uint64_t v) { for (int i = 0; i < 8; ++i) { h ^= (v >> (8 * i)) & 0xff; h *= 1099511628211ull; } };
    for (const char * p = p1a_version(); *p; ++p) { h ^= (unsigned char) *p; h *= 1099511628211ull; }
    mix((uint64_t) P1A_NUMERICS_REV);
    mix((uint64_t) cu_count());
    mix((uint64_t) p1a_get_nsplit(Hkv < 1 ? 1 : Hkv));
    mix((uint64_t) (Hq > 0 ? Hq : 0));
    mix((uint64_t) (Hkv > 0 ? Hkv : 0));
    return h;
}

int p1a_reload_env(void) {
    const int v = read_env_split();
    // (the first read counts as a change, as in the reference, whose switch starts out unread: src/fast/attn_dec2.cu reload)
    const bool changed = v != g_env_split;
    g_env_split = v;
    return changed ? 1 : 0;
}

int p1a_bench_stream_read(const void * src, size_t bytes, void * stream) {
    if (!src || bytes < 16 || ((uintptr_t) src & 15)) { set_error("p1a_bench_stream_read: null, short or misaligned source"); return P1A_E_ARG; }
    return launch_stream_read(src, bytes, (hipStream_t) stream);
}

void p1a_release(void) {
    std::lock_guard<std::mutex> lk(g_mu);
    int cur = 0;
    (void) hipGetDevice(&cur);
    for (int i = 0; i < g_nscr; ++i) {
        (void) hipSetDevice(g_scr[i].dev);
        (void) hipDeviceSynchronize();
        for (bufpair * b : {&g_scr[i].dec, &g_scr[i].pf})
            if (b->o) { (void) hipFree(b->o); (void) hipFree(b->ml); }
        if (g_scr[i].stage) (void) hipFree(g_scr[i].stage);
        g_scr[i] = stream_bufs{};
    }
    g_nscr = 0;
    for (int i = 0; i < g_nretired; ++i) {
        (void) hipSetDevice(g_retired[i].dev);
        (void) hipFree(g_retired[i].p);
    }
    g_nretired = 0;
    (void) hipSetDevice(cur);
}

const char * p1a_last_error(void) { return g_err; }
const char * p1a_version(void) { return "p1a_attn 0.1 (gfx950)"; }

}   // extern "C"
