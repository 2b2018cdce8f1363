// Paged KV pool, sequence manager and P100ESQ2 session files for one GPU (one tensor-parallel rank). Host code: page
// and slot free lists, per-sequence page tables (pinned host copy + stream-ordered upload of new entries), 2-D copies
// between the pool ([K | V][kv layer][page]) and the offload image ([page][K | V][kv layer]) of a sequence.
// A pool created with host_memory = 1 keeps everything in host memory and makes no GPU call (session-file tools, tests).
#include "p1a_common.hpp"
#include "p1a_pool.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace {

using p1a::set_error;

// One sequence of the pool. While it is resident it owns a row of the page table (its slot) and the pages listed here,
// in position order; once offloaded it owns neither, only the host image of its pages and state.
struct seq_t {
    bool used = false;                // this entry of the sequence table is taken
    int slot = -1;                    // resident: which page-table row and state block are its own; -1 while offloaded
    int n_past = 0;                   // positions that hold KV (the next token goes to position n_past)
    std::vector<int32_t> toks;        // the token ids behind those positions, one per position
    std::vector<int32_t> pages;       // resident: pool page of every 2^psh positions, ascending by position
    char * host = nullptr;            // offloaded: the image - page after page, each page_bytes, then the state block
    int host_pages = 0;               // pages in that image
    size_t host_bytes = 0;            // bytes of that image (counted against the pool's host budget)
};

}   // namespace

struct p1a_pool {
    p1a_pool_cfg cfg;
    hipStream_t s = nullptr;
    bool hostmem = false;
    size_t rowb = 0, pblk = 0, page_bytes = 0;
    int n_pages = 0, max_pages = 0;
    char * kv_pool = nullptr;
    char * state_pool = nullptr;
    int32_t * ptab_h = nullptr, * ptab_d = nullptr;      // [max_slots][max_pages]
    int32_t * rtab_h = nullptr, * rtab_d = nullptr;      // [RT_CAP]
    std::vector<int> free_pages, free_slots;
    std::vector<seq_t> seqs;
    uint64_t fp[15] = {0};
    size_t host_bytes = 0;
    static constexpr int RT_CAP = 1024;

    // ---- memory operations: the GPU's, or plain host memory ----
    bool ok(hipError_t e, const char * what) const {
        if (e == hipSuccess) return true;
        (void) hipGetLastError();
        set_error("%s: %s", what, hipGetErrorString(e));
        return false;
    }
    char * dev_alloc(size_t n) const {
        if (hostmem) return (char *) malloc(n ? n : 1);
        void * q = nullptr;
        return hipMalloc(&q, n ? n : 1) == hipSuccess ? (char *) q : ((void) hipGetLastError(), nullptr);
    }
    void dev_free(void * q) const { if (!q) return; if (hostmem) free(q); else (void) hipFree(q); }
    char * pin_alloc(size_t n) const {
        if (hostmem) return (char *) malloc(n ? n : 1);
        void * q = nullptr;   // allocated pinned (registering existing memory is not relied on)
        return hipHostMalloc(&q, n ? n : 1, hipHostMallocPortable) == hipSuccess ? (char *) q : ((void) hipGetLastError(), nullptr);
    }
    void pin_free(void * q) const { if (!q) return; if (hostmem) free(q); else (void) hipHostFree(q); }
    bool zero(void * q, size_t n) const {
        if (!n) return true;
        if (hostmem) { memset(q, 0, n); return true; }
        return ok(hipMemsetAsync(q, 0, n, s), "fill");
    }
    bool copy(void * d, const void * sp, size_t n, hipMemcpyKind k) const {
        if (!n) return true;
        if (hostmem) { memcpy(d, sp, n); return true; }
        return ok(hipMemcpyAsync(d, sp, n, k, s), "copy");
    }
    bool copy2d(void * d, size_t dp, const void * sp, size_t spitch, size_t w, size_t h, hipMemcpyKind k) const {
        if (!w || !h) return true;
        if (hostmem) {
            for (size_t i = 0; i < h; ++i) memcpy((char *) d + i * dp, (const char *) sp + i * spitch, w);
            return true;
        }
        return ok(hipMemcpy2DAsync(d, dp, sp, spitch, w, h, k, s), "2-D copy");
    }
    bool sync() const { return hostmem || ok(hipStreamSynchronize(s), "stream synchronize"); }

    int ps() const { return 1 << cfg.psh; }
    size_t region() const { return (size_t) n_pages * pblk; }     // one layer's K (or V) pages
    int pages_for(int n) const { return (n + ps() - 1) >> cfg.psh; }
    seq_t * get(int id) { return id >= 0 && id < (int) seqs.size() ? &seqs[id] : nullptr; }
    const seq_t * get(int id) const { return id >= 0 && id < (int) seqs.size() ? &seqs[id] : nullptr; }
    char * state_of(int slot) const { return cfg.state_bytes && slot >= 0 ? state_pool + (size_t) slot * cfg.state_bytes : nullptr; }
    size_t host_used() const { return host_bytes; }
    bool over_budget(size_t more) const { return cfg.host_budget && host_used() + more > cfg.host_budget; }
};

namespace {

// page i of a resident sequence <-> its place in an offload image (two 2-D blocks per page: K layers, V layers)
bool page_to_image(const p1a_pool * p, int page, char * img, hipMemcpyKind k) {
    for (int kv = 0; kv < 2; ++kv)
        if (!p->copy2d(img + (size_t) kv * p->cfg.n_kv_layers * p->pblk, p->pblk,
                       p->kv_pool + (size_t) kv * p->cfg.n_kv_layers * p->region() + (size_t) page * p->pblk, p->region(),
                       p->pblk, (size_t) p->cfg.n_kv_layers, k)) return false;
    return true;
}
bool image_to_page(const p1a_pool * p, const char * img, int page, hipMemcpyKind k) {
    for (int kv = 0; kv < 2; ++kv)
        if (!p->copy2d(p->kv_pool + (size_t) kv * p->cfg.n_kv_layers * p->region() + (size_t) page * p->pblk, p->region(),
                       img + (size_t) kv * p->cfg.n_kv_layers * p->pblk, p->pblk, p->pblk, (size_t) p->cfg.n_kv_layers, k)) return false;
    return true;
}

int new_id(p1a_pool * p) {
    for (int i = 0; i < (int) p->seqs.size(); ++i) if (!p->seqs[i].used) return i;
    p->seqs.emplace_back();
    return (int) p->seqs.size() - 1;
}

// offloaded -> resident with the first np saved pages; state: also the state block (the host copy's, i.e. of n_past)
int restore_impl(p1a_pool * p, int id, int np, bool state) {
    seq_t * q = p->get(id);
    if (!q || !q->used || q->slot >= 0) { set_error("seq_restore: sequence not offloaded"); return P1A_E_STATE; }
    if (np < 0 || np > q->host_pages) { set_error("seq_restore: page count out of range"); return P1A_E_ARG; }
    if (p->free_slots.empty()) { set_error("seq_restore: no free sequence slot"); return P1A_E_STATE; }
    if ((int) p->free_pages.size() < np) { set_error("seq_restore: KV pool full"); return P1A_E_STATE; }
    if (!p->sync()) return P1A_E_LAUNCH;
    q->slot = p->free_slots.back();
    p->free_slots.pop_back();
    q->pages.clear();
    // a failure below leaves the sequence as it was: offloaded, its host copy intact, pages and slot given back
    auto undo = [&](int rc) {
        (void) p->sync();
        for (auto it = q->pages.rbegin(); it != q->pages.rend(); ++it) p->free_pages.push_back(*it);
        q->pages.clear();
        p->free_slots.push_back(q->slot);
        q->slot = -1;
        return rc;
    };
    if (np > 0) {
        const int rc = p1a_seq_ensure_pages(p, id, std::min(np << p->cfg.psh, p->cfg.n_ctx));
        if (rc < 0) return undo(rc);
    }
    for (int i = 0; i < np; ++i)
        if (!image_to_page(p, q->host + (size_t) i * p->page_bytes, q->pages[i], hipMemcpyHostToDevice)) return undo(P1A_E_LAUNCH);
    const char * st = q->host + (size_t) q->host_pages * p->page_bytes;
    if (p->cfg.state_bytes) {
        if (state) { if (!p->copy(p->state_of(q->slot), st, p->cfg.state_bytes, hipMemcpyHostToDevice)) return undo(P1A_E_LAUNCH); }
        else if (!p->zero(p->state_of(q->slot), p->cfg.state_bytes)) return undo(P1A_E_LAUNCH);
    }
    if (!p->sync()) return undo(P1A_E_LAUNCH);
    p->pin_free(q->host);
    q->host = nullptr;
    p->host_bytes -= q->host_bytes;
    q->host_bytes = 0;
    q->host_pages = 0;
    return P1A_OK;
}

const char kSeqMagic[8] = {'P', '1', '0', '0', 'E', 'S', 'Q', '2'};
const char * kFpNames[15] = {"model file size", "tensor count", "embedding", "layers", "vocab", "KV type", "page shift",
                             "GPU count / tensor-parallel split", "page bytes", "state bytes", "KV layers", "MTP block",
                             "GGUF metadata hash", "tensor table hash", "tensor content sample hash"};

}   // namespace

extern "C" {

p1a_pool * p1a_pool_create(const p1a_pool_cfg * cfg, void * stream) {
    if (!cfg) { set_error("p1a_pool_create: null configuration"); return nullptr; }
    if (cfg->kv_type != P1A_KV_F16 && cfg->kv_type != P1A_KV_Q8_0 && cfg->kv_type != P1A_KV_Q4_0) { set_error("p1a_pool_create: unknown KV type %u", cfg->kv_type); return nullptr; }
    if (cfg->n_kv_layers < 1 || cfg->Hkv < 1 || cfg->D < 32 || cfg->D % 32 || cfg->psh < 0 || cfg->psh > 24 || cfg->n_ctx < 1 || cfg->max_slots < 1) {
        set_error("p1a_pool_create: bad geometry (layers %d, Hkv %d, D %d, psh %d, n_ctx %d, slots %d)", cfg->n_kv_layers, cfg->Hkv, cfg->D, cfg->psh, cfg->n_ctx, cfg->max_slots);
        return nullptr;
    }
    p1a_pool * p = new p1a_pool;
    p->cfg = *cfg;
    p->s = (hipStream_t) stream;
    p->hostmem = cfg->host_memory != 0;
    p->rowb = p1a_kv_row_bytes(cfg->kv_type, cfg->Hkv, cfg->D);
    p->pblk = (size_t) p->ps() * p->rowb;                          // one page of one layer's K (or V)
    p->page_bytes = (size_t) cfg->n_kv_layers * 2 * p->pblk;
    p->max_pages = p->pages_for(cfg->n_ctx);
    int64_t np;
    if (cfg->tokens >= 0) {
        np = (cfg->tokens + p->ps() - 1) >> cfg->psh;
    } else {
        size_t fr = 0, tot = 0;
        if (p->hostmem) { set_error("alloc_pool: a host-memory pool needs an explicit size"); delete p; return nullptr; }
        if (!p->ok(hipMemGetInfo(&fr, &tot), "alloc_pool")) { delete p; return nullptr; }
        const size_t keep = cfg->reserve_mb << 20;
        np = fr > keep ? (int64_t) ((fr - keep) / p->page_bytes) : 0;
        np = std::min<int64_t>(np, (int64_t) cfg->max_slots * p->max_pages);   // more than every slot at n_ctx is useless
    }
    if (np < 1) { set_error("alloc_pool: no room for a single KV page"); delete p; return nullptr; }
    if (np > INT32_MAX / 2) { set_error("alloc_pool: too many pages"); delete p; return nullptr; }
    p->n_pages = (int) np;
    const size_t tab = (size_t) cfg->max_slots * p->max_pages * 4;
    p->kv_pool = p->dev_alloc((size_t) np * p->page_bytes);
    p->state_pool = cfg->state_bytes ? p->dev_alloc((size_t) cfg->max_slots * cfg->state_bytes) : nullptr;
    p->ptab_h = (int32_t *) p->pin_alloc(tab);
    p->rtab_h = (int32_t *) p->pin_alloc(p1a_pool::RT_CAP * 4);
    p->ptab_d = p->hostmem ? p->ptab_h : (int32_t *) p->dev_alloc(tab);
    p->rtab_d = p->hostmem ? p->rtab_h : (int32_t *) p->dev_alloc(p1a_pool::RT_CAP * 4);
    if (!p->kv_pool || (cfg->state_bytes && !p->state_pool) || !p->ptab_h || !p->rtab_h || !p->ptab_d || !p->rtab_d) {
        set_error("alloc_pool: allocation of %zu MiB failed", ((size_t) np * p->page_bytes) >> 20);
        p1a_pool_destroy(p);
        return nullptr;
    }
    memset(p->ptab_h, 0, tab);
    memset(p->rtab_h, 0, p1a_pool::RT_CAP * 4);
    // finite contents: rows past a sequence's end inside a page may be read (and weighted by zero) by a consumer
    bool fine = p->zero(p->kv_pool, (size_t) np * p->page_bytes);
    if (!p->hostmem) fine = fine && p->zero(p->ptab_d, tab) && p->zero(p->rtab_d, p1a_pool::RT_CAP * 4);
    if (!fine || !p->sync()) { p1a_pool_destroy(p); return nullptr; }
    for (int i = p->n_pages - 1; i >= 0; --i) p->free_pages.push_back(i);      // handed out in ascending order
    for (int i = cfg->max_slots - 1; i >= 0; --i) p->free_slots.push_back(i);
    p->fp[5] = cfg->kv_type; p->fp[6] = (uint64_t) cfg->psh; p->fp[7] = 1; p->fp[8] = p->page_bytes;
    p->fp[9] = cfg->state_bytes; p->fp[10] = (uint64_t) cfg->n_kv_layers;
    return p;
}

void p1a_pool_destroy(p1a_pool * p) {
    if (!p) return;
    (void) p->sync();
    for (seq_t & q : p->seqs) if (q.host) p->pin_free(q.host);
    p->dev_free(p->kv_pool);
    p->dev_free(p->state_pool);
    if (!p->hostmem) { p->dev_free(p->ptab_d); p->dev_free(p->rtab_d); }
    p->pin_free(p->ptab_h);
    p->pin_free(p->rtab_h);
    delete p;
}

int p1a_pool_n_pages(const p1a_pool * p) { return p ? p->n_pages : P1A_E_ARG; }
int p1a_pool_free_pages(const p1a_pool * p) { return p ? (int) p->free_pages.size() : P1A_E_ARG; }
int p1a_pool_max_pages(const p1a_pool * p) { return p ? p->max_pages : P1A_E_ARG; }
size_t p1a_pool_page_bytes(const p1a_pool * p) { return p ? p->page_bytes : 0; }
size_t p1a_pool_host_used(const p1a_pool * p) { return p ? p->host_used() : 0; }

static int kv_of(const p1a_pool * p, int layer, p1a_kv * out) {
    if (!p || !out) { set_error("p1a_pool_kv: null argument"); return P1A_E_ARG; }
    if (layer < 0 || layer >= p->cfg.n_kv_layers) { set_error("p1a_pool_kv: layer %d of %d", layer, p->cfg.n_kv_layers); return P1A_E_ARG; }
    out->type = p->cfg.kv_type; out->n_ctx = p->cfg.n_ctx; out->Hkv = p->cfg.Hkv; out->D = p->cfg.D;
    out->k = p->kv_pool + (size_t) layer * p->region();
    out->v = p->kv_pool + (size_t) (p->cfg.n_kv_layers + layer) * p->region();
    out->pt = p->ptab_d; out->rtab = nullptr; out->psh = p->cfg.psh; out->pstride = p->pblk;
    return P1A_OK;
}

int p1a_pool_kv_seq(const p1a_pool * p, int layer, int id, p1a_kv * out) {
    const int rc = kv_of(p, layer, out);
    if (rc < 0) return rc;
    const seq_t * q = p->get(id);
    if (!q || !q->used || q->slot < 0) { set_error("kv_seq: sequence %d is not resident", id); return P1A_E_STATE; }
    out->pt = p->ptab_d + (size_t) q->slot * p->max_pages;
    return P1A_OK;
}

int p1a_pool_kv_rows(const p1a_pool * p, int layer, p1a_kv * out) {
    const int rc = kv_of(p, layer, out);
    if (rc < 0) return rc;
    out->rtab = p->rtab_d;
    return P1A_OK;
}

int p1a_pool_set_rows(p1a_pool * p, const int * ids, int nrows) {
    if (!p || !ids || nrows < 1 || nrows > p1a_pool::RT_CAP) { set_error("p1a_pool_set_rows: bad arguments (rows %d)", nrows); return P1A_E_ARG; }
    for (int t = 0; t < nrows; ++t) {
        const seq_t * q = p->get(ids[t]);
        if (!q || !q->used || q->slot < 0) { set_error("p1a_pool_set_rows: sequence %d is not resident", ids[t]); return P1A_E_STATE; }
    }
    // (the pinned source is rewritten by the next call: the previous upload must have left it)
    if (!p->sync()) return P1A_E_LAUNCH;
    for (int t = 0; t < nrows; ++t) p->rtab_h[t] = p->get(ids[t])->slot * p->max_pages;
    if (!p->hostmem && !p->copy(p->rtab_d, p->rtab_h, (size_t) nrows * 4, hipMemcpyHostToDevice)) return P1A_E_LAUNCH;
    return P1A_OK;
}

void * p1a_pool_state(const p1a_pool * p, int id) {
    const seq_t * q = p ? p->get(id) : nullptr;
    return q && q->used ? p->state_of(q->slot) : nullptr;
}

int p1a_seq_create(p1a_pool * p) {
    if (!p) return P1A_E_ARG;
    if (p->free_slots.empty()) { set_error("no free sequence slot (max_seqs %d)", p->cfg.max_slots); return P1A_E_STATE; }
    if (!p->sync()) return P1A_E_LAUNCH;
    const int id = new_id(p);
    seq_t & q = p->seqs[id];
    q = seq_t{};
    q.used = true;
    q.slot = p->free_slots.back();
    p->free_slots.pop_back();
    if (!p->zero(p->state_of(q.slot), p->cfg.state_bytes)) {
        p->free_slots.push_back(q.slot);
        q = seq_t{};
        return P1A_E_LAUNCH;
    }
    return id;
}

int p1a_seq_free(p1a_pool * p, int id) {
    seq_t * q = p ? p->get(id) : nullptr;
    if (!q) { set_error("seq_free: no such sequence"); return P1A_E_ARG; }
    if (!q->used) return P1A_OK;
    if (!p->sync()) return P1A_E_LAUNCH;
    for (auto it = q->pages.rbegin(); it != q->pages.rend(); ++it) p->free_pages.push_back(*it);
    if (q->slot >= 0) p->free_slots.push_back(q->slot);
    if (q->host) p->pin_free(q->host);
    p->host_bytes -= q->host_bytes;
    *q = seq_t{};
    return P1A_OK;
}

int p1a_seq_ensure_pages(p1a_pool * p, int id, int n) {
    seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used || q->slot < 0) { set_error("sequence %d is not resident", id); return P1A_E_STATE; }
    if (n > p->cfg.n_ctx) { set_error("context full"); return P1A_E_STATE; }
    const int need = p->pages_for(std::max(n, 0));
    const int have = (int) q->pages.size();
    if (need <= have) return P1A_OK;
    if (need - have > (int) p->free_pages.size()) {
        set_error("KV pool full (%zu free pages, need %d)", p->free_pages.size(), need - have);
        return P1A_E_STATE;
    }
    int32_t * row = p->ptab_h + (size_t) q->slot * p->max_pages;
    for (int i = have; i < need; ++i) {
        const int pg = p->free_pages.back();
        p->free_pages.pop_back();
        q->pages.push_back(pg);
        row[i] = pg;
    }
    // stream-ordered upload of the new entries (pinned source: entries [have, need) are not written again while it is
    // in flight - later growth writes later entries, slot reuse goes through a synchronize)
    if (!p->hostmem && !p->copy(p->ptab_d + (size_t) q->slot * p->max_pages + have, row + have, (size_t) (need - have) * 4, hipMemcpyHostToDevice))
        return P1A_E_LAUNCH;
    return P1A_OK;
}

int p1a_seq_len(const p1a_pool * p, int id) { const seq_t * q = p ? p->get(id) : nullptr; return q && q->used ? q->n_past : P1A_E_ARG; }
int p1a_seq_resident(const p1a_pool * p, int id) { const seq_t * q = p ? p->get(id) : nullptr; return q && q->used && q->slot >= 0; }
int p1a_seq_pages(const p1a_pool * p, int id) {
    const seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used) return P1A_E_ARG;
    return q->slot >= 0 ? (int) q->pages.size() : q->host_pages;
}
size_t p1a_seq_host_bytes(const p1a_pool * p, int id) { const seq_t * q = p ? p->get(id) : nullptr; return q ? q->host_bytes : 0; }

int p1a_seq_advance(p1a_pool * p, int id, const int32_t * toks, int T) {
    seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used || q->slot < 0) { set_error("seq_advance: sequence not resident"); return P1A_E_STATE; }
    if (T < 0) { set_error("seq_advance: negative row count"); return P1A_E_ARG; }
    const int rc = p1a_seq_ensure_pages(p, id, q->n_past + T);
    if (rc < 0) return rc;
    for (int t = 0; t < T; ++t) q->toks.push_back(toks ? toks[t] : -1);
    q->n_past += T;
    return q->n_past;
}

int p1a_seq_rollback(p1a_pool * p, int id, int T, int n_keep) {
    seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used || q->slot < 0) { set_error("rollback: sequence not resident"); return P1A_E_STATE; }
    if (n_keep < 1 || n_keep > T || T > q->n_past) { set_error("rollback out of range"); return P1A_E_ARG; }
    q->n_past -= T - n_keep;          // attention KV: later positions are simply overwritten
    q->toks.resize(q->n_past);
    return q->n_past;
}

int p1a_seq_truncate(p1a_pool * p, int id, int n) {
    seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used || q->slot < 0) { set_error("seq_truncate: sequence not resident"); return P1A_E_STATE; }
    if (n < 0 || n > q->n_past) { set_error("seq_truncate: position out of range"); return P1A_E_ARG; }
    if (n == q->n_past) return P1A_OK;
    // nothing in flight may still read the pages given back, or the page-table entries rewritten later
    if (!p->sync()) return P1A_E_LAUNCH;
    const int keep = p->pages_for(n);
    for (int i = (int) q->pages.size() - 1; i >= keep; --i) p->free_pages.push_back(q->pages[i]);
    if ((int) q->pages.size() > keep) q->pages.resize(keep);
    q->n_past = n;
    q->toks.resize(n);
    return P1A_OK;
}

int p1a_seq_fork(p1a_pool * p, int src, int n) {
    if (!p) return P1A_E_ARG;
    {
        const seq_t * q = p->get(src);
        if (!q || !q->used || q->slot < 0) { set_error("seq_fork: source not resident"); return P1A_E_STATE; }
        if (n < 0 || n > q->n_past) { set_error("seq_fork: position out of range"); return P1A_E_ARG; }
        if (p->free_slots.empty()) { set_error("seq_fork: no free sequence slot"); return P1A_E_STATE; }
        if ((int) p->free_pages.size() < p->pages_for(n)) { set_error("seq_fork: KV pool full"); return P1A_E_STATE; }
    }
    const int id = p1a_seq_create(p);   // may grow the sequence table: pointers taken after
    if (id < 0) return id;
    const int np = p->pages_for(n);
    auto drop = [&](int rc) { (void) p1a_seq_free(p, id); return rc; };   // a failed fork leaves no half-made copy behind
    if (np > 0) {
        const int rc = p1a_seq_ensure_pages(p, id, std::min(np << p->cfg.psh, p->cfg.n_ctx));
        if (rc < 0) return drop(rc);
    }
    const seq_t & q = p->seqs[src];
    seq_t & d = p->seqs[id];
    for (int i = 0; i < np; ++i)   // every KV layer's K and V of page i: one 2-D copy (rows = 2 x layers, pitch = a region)
        if (!p->copy2d(p->kv_pool + (size_t) d.pages[i] * p->pblk, p->region(), p->kv_pool + (size_t) q.pages[i] * p->pblk,
                       p->region(), p->pblk, (size_t) 2 * p->cfg.n_kv_layers, hipMemcpyDeviceToDevice)) return drop(P1A_E_LAUNCH);
    if (!p->sync()) return drop(P1A_E_LAUNCH);
    d.n_past = n;
    d.toks.assign(q.toks.begin(), q.toks.begin() + n);
    return id;
}

int p1a_seq_offload(p1a_pool * p, int id) {
    seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used || q->slot < 0) { set_error("seq_offload: sequence not resident"); return P1A_E_STATE; }
    const size_t bytes = q->pages.size() * p->page_bytes + p->cfg.state_bytes;
    if (p->over_budget(bytes)) {
        set_error("seq_offload: host budget exceeded (%zu MiB > %zu MiB)", (p->host_used() + bytes) >> 20, p->cfg.host_budget >> 20);
        return P1A_E_STATE;
    }
    if (!p->sync()) return P1A_E_LAUNCH;
    q->host = p->pin_alloc(bytes);
    if (!q->host) { set_error("seq_offload: pinned host allocation of %zu MiB failed", bytes >> 20); return P1A_E_SCRATCH; }
    auto undo = [&](int rc) { (void) p->sync(); p->pin_free(q->host); q->host = nullptr; return rc; };   // still resident
    for (size_t i = 0; i < q->pages.size(); ++i)
        if (!page_to_image(p, q->pages[i], q->host + i * p->page_bytes, hipMemcpyDeviceToHost)) return undo(P1A_E_LAUNCH);
    if (!p->copy(q->host + q->pages.size() * p->page_bytes, p->state_of(q->slot), p->cfg.state_bytes, hipMemcpyDeviceToHost)) return undo(P1A_E_LAUNCH);
    if (!p->sync()) return undo(P1A_E_LAUNCH);
    q->host_pages = (int) q->pages.size();
    q->host_bytes = bytes;
    p->host_bytes += bytes;
    for (auto it = q->pages.rbegin(); it != q->pages.rend(); ++it) p->free_pages.push_back(*it);
    q->pages.clear();
    p->free_slots.push_back(q->slot);
    q->slot = -1;
    return P1A_OK;
}

int p1a_seq_restore(p1a_pool * p, int id) {
    const seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used || q->slot >= 0) { set_error("seq_restore: sequence not offloaded"); return P1A_E_STATE; }
    return restore_impl(p, id, q->host_pages, true);
}

int p1a_seq_restore_prefix(p1a_pool * p, int id, int n) {
    seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used || q->slot >= 0) { set_error("seq_restore_prefix: sequence not offloaded"); return P1A_E_STATE; }
    if (n < 0 || n > q->n_past) { set_error("seq_restore_prefix: position out of range"); return P1A_E_ARG; }
    const int rc = restore_impl(p, id, std::min(q->host_pages, p->pages_for(n)), n == q->n_past);
    if (rc < 0) return rc;
    q = p->get(id);
    q->n_past = n;
    q->toks.resize(n);
    return P1A_OK;
}

int p1a_seq_pages_out(p1a_pool * p, int id, int p0, int n, char * dst) {
    const seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used || q->slot < 0 || !dst) { set_error("pages_out: sequence not resident"); return P1A_E_STATE; }
    if (p0 < 0 || n < 0 || p0 + n > (int) q->pages.size()) { set_error("pages_out: page range out of the sequence"); return P1A_E_ARG; }
    for (int i = 0; i < n; ++i)
        if (!page_to_image(p, q->pages[p0 + i], dst + (size_t) i * p->page_bytes, hipMemcpyDeviceToHost)) return P1A_E_LAUNCH;
    return P1A_OK;
}

int p1a_seq_tokens(const p1a_pool * p, int id, int32_t * dst, int cap) {
    const seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used) { set_error("seq_tokens: no such sequence"); return P1A_E_ARG; }
    const int n = std::min(cap, (int) q->toks.size());
    if (dst && n > 0) memcpy(dst, q->toks.data(), (size_t) n * 4);
    return (int) q->toks.size();
}

int p1a_pool_set_fingerprint(p1a_pool * p, const uint64_t fp[15]) {
    if (!p || !fp) return P1A_E_ARG;
    for (int i = 0; i < 15; ++i) if (i < 5 || i > 10) p->fp[i] = fp[i];
    return P1A_OK;
}

int p1a_pool_fingerprint(const p1a_pool * p, uint64_t fp[15]) {
    if (!p || !fp) return P1A_E_ARG;
    memcpy(fp, p->fp, sizeof p->fp);
    return P1A_OK;
}

int p1a_seq_write(p1a_pool * p, int id, const char * path) {
    seq_t * q = p ? p->get(id) : nullptr;
    if (!q || !q->used || !path) { set_error("seq_write: no such sequence"); return P1A_E_ARG; }
    FILE * f = fopen(path, "wb");
    if (!f) { set_error("seq_write: cannot open %s", path); return P1A_E_IO; }
    bool good = true;
    auto wr = [&](const void * src, size_t n) { if (good && n && fwrite(src, 1, n, f) != n) good = false; };
    const bool res = q->slot >= 0;
    const int np = res ? (int) q->pages.size() : q->host_pages;
    const int32_t hdr[3] = {q->n_past, (int32_t) q->toks.size(), np};
    wr(kSeqMagic, 8);
    wr(p->fp, sizeof p->fp);
    wr(hdr, sizeof hdr);
    wr(q->toks.data(), q->toks.size() * 4);
    int rc = P1A_OK;
    if (!res) {
        wr(q->host, (size_t) np * p->page_bytes + p->cfg.state_bytes);
    } else {
        // resident: through a pinned staging buffer, up to 32 pages at a time
        if (!p->sync()) rc = P1A_E_LAUNCH;
        const int chunk = std::max(1, std::min(np, 32));
        char * st = rc == P1A_OK ? p->pin_alloc(std::max((size_t) chunk * p->page_bytes, p->cfg.state_bytes)) : nullptr;
        if (rc == P1A_OK && !st) { set_error("seq_write: pinned staging allocation failed"); rc = P1A_E_SCRATCH; }
        for (int p0 = 0; rc == P1A_OK && p0 < np; p0 += chunk) {
            const int n = std::min(chunk, np - p0);
            rc = p1a_seq_pages_out(p, id, p0, n, st);
            if (rc == P1A_OK && !p->sync()) rc = P1A_E_LAUNCH;
            if (rc == P1A_OK) wr(st, (size_t) n * p->page_bytes);
        }
        if (rc == P1A_OK && p->cfg.state_bytes) {
            if (!p->copy(st, p->state_of(q->slot), p->cfg.state_bytes, hipMemcpyDeviceToHost) || !p->sync()) rc = P1A_E_LAUNCH;
            else wr(st, p->cfg.state_bytes);
        }
        p->pin_free(st);
    }
    if (fclose(f) != 0) good = false;
    if (rc == P1A_OK && !good) { set_error("seq_write: write failed (disk full?)"); rc = P1A_E_IO; }
    return rc;
}

int p1a_seq_read(p1a_pool * p, const char * path) {
    if (!p || !path) return P1A_E_ARG;
    FILE * f = fopen(path, "rb");
    if (!f) { set_error("seq_read: cannot open %s", path); return P1A_E_IO; }
    bool good = true;
    auto rd = [&](void * dst, size_t n) { if (good && n && fread(dst, 1, n, f) != n) good = false; };
    auto fail = [&](int code) { fclose(f); return code; };
    char mg[8];
    rd(mg, 8);
    if (!good) { set_error("seq_read: short file"); return fail(P1A_E_IO); }
    if (!memcmp(mg, "P100ESQ1", 8)) { set_error("seq_read: a version 1 sequence file (no content / numerics fingerprint): not loadable"); return fail(P1A_E_IO); }
    if (memcmp(mg, kSeqMagic, 8)) { set_error("seq_read: not a p100e sequence file"); return fail(P1A_E_IO); }
    uint64_t fp[15];
    rd(fp, sizeof fp);
    if (!good) { set_error("seq_read: short file"); return fail(P1A_E_IO); }
    for (int i = 0; i < 15; ++i)
        if (fp[i] != p->fp[i]) {
            set_error("seq_read: saved with another model / KV layout (%s %llu vs %llu)", kFpNames[i], (unsigned long long) fp[i], (unsigned long long) p->fp[i]);
            return fail(P1A_E_IO);
        }
    int32_t hdr[3];
    rd(hdr, sizeof hdr);
    if (!good) { set_error("seq_read: short file"); return fail(P1A_E_IO); }
    const int n_past = hdr[0], ntok = hdr[1], np = hdr[2];
    if (n_past < 0 || n_past > p->cfg.n_ctx || ntok != n_past || np < 0 || np > p->max_pages || ((int64_t) np << p->cfg.psh) < n_past) {
        set_error("seq_read: bad header (or the sequence exceeds this engine's context)");
        return fail(P1A_E_IO);
    }
    std::vector<int32_t> toks((size_t) ntok);
    rd(toks.data(), (size_t) ntok * 4);
    if (!good) { set_error("seq_read: short file"); return fail(P1A_E_IO); }
    const int64_t vocab = (int64_t) p->fp[4];
    for (int32_t t : toks)
        if (t < -1 || (vocab > 0 && t >= vocab)) { set_error("seq_read: token id %d out of range", t); return fail(P1A_E_IO); }
    const size_t bytes = (size_t) np * p->page_bytes + p->cfg.state_bytes;
    if (p->over_budget(bytes)) {
        set_error("seq_read: host budget exceeded (%zu MiB > %zu MiB)", (p->host_used() + bytes) >> 20, p->cfg.host_budget >> 20);
        return fail(P1A_E_STATE);
    }
    char * host = p->pin_alloc(bytes);
    if (!host) { set_error("seq_read: pinned host allocation of %zu MiB failed", bytes >> 20); return fail(P1A_E_SCRATCH); }
    rd(host, bytes);
    if (!good) { p->pin_free(host); set_error("seq_read: short file"); return fail(P1A_E_IO); }
    fclose(f);
    const int id = new_id(p);
    seq_t & q = p->seqs[id];
    q = seq_t{};
    q.used = true;
    q.slot = -1;
    q.n_past = n_past;
    q.toks = std::move(toks);
    q.host = host;
    q.host_pages = np;
    q.host_bytes = bytes;
    p->host_bytes += bytes;
    return id;
}

int p1a_verify_accept(const int32_t * tokens, const int32_t * greedy, int T, int budget, int * n_accept, int32_t * next) {
    if (!tokens || !greedy || T < 1 || budget < 1) { set_error("p1a_verify_accept: bad arguments (T %d, budget %d)", T, budget); return P1A_E_ARG; }
    int a = 0;
    while (a < T - 1 && greedy[a] == tokens[1 + a]) ++a;
    if (n_accept) *n_accept = a;
    if (next) *next = greedy[a];
    return std::min(a + 1, budget);
}

}   // extern "C"
