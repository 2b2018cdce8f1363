// C++ face of include/p1a_pool.h with the reference's member names and error behaviour: the pool / sequence members of
// `class tp_model` (src/tp_model.h:371-475, src/tp_model.cu:3303-3966) for one GPU, as a class of its own. Every refusal
// throws std::runtime_error with the reference's message, as the members it replaces do.
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "p100e_fast_attn.hpp"
#include "p1a_pool.h"

namespace p100e {

class kv_pool {
public:
    // geometry of this rank: KV type, KV layers in a page, its kv heads, head size, page shift, per-sequence cap, slots
    kv_pool(uint32_t kv_type, int n_kv_layers, int Hkv, int D, int psh, int n_ctx, int max_slots, hipStream_t s,
            size_t state_bytes = 0, size_t host_budget = 0)
        : cfg_{kv_type, n_kv_layers, Hkv, D, psh, n_ctx, max_slots, 0, 0, state_bytes, host_budget, 0}, s_(s) {}
    kv_pool(const kv_pool &) = delete;
    kv_pool & operator=(const kv_pool &) = delete;
    ~kv_pool() { p1a_pool_destroy(p_); }

    // tp_model::alloc_pool (tp_model.cu:3880): tokens < 0 = by the free memory of the device minus reserve_mb
    void alloc_pool(int64_t tokens, size_t reserve_mb = 1024) {
        if (p_) throw std::runtime_error("alloc_pool: the pool exists already");
        cfg_.tokens = tokens;
        cfg_.reserve_mb = reserve_mb;
        p_ = p1a_pool_create(&cfg_, (void *) s_);
        if (!p_) throw std::runtime_error(p1a_last_error());
    }
    int64_t pool_tokens() const { return (int64_t) p1a_pool_n_pages(need()) << cfg_.psh; }
    int free_pages() const { return p1a_pool_free_pages(need()); }
    size_t host_used() const { return p1a_pool_host_used(need()); }

    // tp_model::kv_seq / kv_rows (tp_model.cu:3327-3337)
    fast::kv_cache kv_seq(int il, int id) const { p1a_kv c; ck(p1a_pool_kv_seq(need(), il, id, &c)); return cache_of(c); }
    fast::kv_cache kv_rows(int il) const { p1a_kv c; ck(p1a_pool_kv_rows(need(), il, &c)); return cache_of(c); }
    void set_rows(const std::vector<int> & ids) { ck(p1a_pool_set_rows(need(), ids.data(), (int) ids.size())); }
    void * state(int id) const { return p1a_pool_state(need(), id); }

    void ensure_pages(int id, int n) { ck(p1a_seq_ensure_pages(need(), id, n)); }
    int seq_create() { return ck(p1a_seq_create(need())); }
    void seq_free(int id) { ck(p1a_seq_free(need(), id)); }
    int seq_len(int id) const { return ck(p1a_seq_len(need(), id)); }
    bool seq_resident(int id) const { return p1a_seq_resident(need(), id) > 0; }
    int seq_pages(int id) const { return ck(p1a_seq_pages(need(), id)); }
    size_t seq_host_bytes(int id) const { return p1a_seq_host_bytes(need(), id); }
    void seq_offload(int id) { ck(p1a_seq_offload(need(), id)); }
    void seq_restore(int id) { ck(p1a_seq_restore(need(), id)); }
    void seq_restore_prefix(int id, int n) { ck(p1a_seq_restore_prefix(need(), id, n)); }
    void seq_truncate(int id, int n) { ck(p1a_seq_truncate(need(), id, n)); }
    int seq_fork(int src, int n) { return ck(p1a_seq_fork(need(), src, n)); }
    void pages_out(int id, int p0, int n, char * dst) { ck(p1a_seq_pages_out(need(), id, p0, n, dst)); }
    // what a forward step / tp_model::rollback (tp_model.cu:3159-3170) do to a sequence's bookkeeping
    int advance(int id, const std::vector<int32_t> & toks) { return ck(p1a_seq_advance(need(), id, toks.data(), (int) toks.size())); }
    int rollback(int id, int T, int n_keep) { return ck(p1a_seq_rollback(need(), id, T, n_keep)); }

    void set_fingerprint(const std::vector<uint64_t> & fp) {
        if (fp.size() != 15) throw std::runtime_error("fingerprint: 15 fields");
        ck(p1a_pool_set_fingerprint(need(), fp.data()));
    }
    std::vector<uint64_t> fingerprint() const { std::vector<uint64_t> fp(15); ck(p1a_pool_fingerprint(need(), fp.data())); return fp; }
    // tp_model::seq_write / seq_read (tp_model.cu:3739-3863), by path
    void seq_write(int id, const std::string & path) { ck(p1a_seq_write(need(), id, path.c_str())); }
    int seq_read(const std::string & path) { return ck(p1a_seq_read(need(), path.c_str())); }

private:
    p1a_pool * need() const {
        if (!p_) throw std::runtime_error("KV pool not allocated (alloc_pool)");
        return p_;
    }
    static fast::kv_cache cache_of(const p1a_kv & r) {
        fast::kv_cache c;
        c.type = r.type; c.n_ctx = r.n_ctx; c.Hkv = r.Hkv; c.D = r.D;
        c.k = r.k; c.v = r.v; c.pt = r.pt; c.rtab = r.rtab; c.psh = r.psh; c.pstride = r.pstride;
        return c;
    }
    static int ck(int rc) {
        if (rc < 0) throw std::runtime_error(p1a_last_error());
        return rc;
    }
    p1a_pool_cfg cfg_;
    hipStream_t s_;
    p1a_pool * p_ = nullptr;
};

}   // namespace p100e
