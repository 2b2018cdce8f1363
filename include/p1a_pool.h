/* Paged KV pool + sequence manager + P100ESQ2 session files, one GPU (one tensor-parallel rank).
 *
 * The consumer of the KV byte layout on either side of the attention path: it owns the pool the p1a_kv descriptors point
 * into, hands pages to sequences, and moves sequences between the GPU, pinned host memory and session files in the
 * engine's own formats, so that pages written here are interchangeable with the engine's. Each entry cites the
 * reference member (src/tp_model.cu) it replaces. Host code; the only device work is copies and fills.
 *
 * Pool layout (tp_model.cu:3874-3879, 3934-3942): one allocation [K | V][kv layer][page][2^psh positions][row bytes]:
 * layer li's K pages start at li * n_pages * pblk, its V pages at (n_kv_layers + li) * n_pages * pblk, pblk = 2^psh * row
 * bytes = the page stride of every descriptor. The pool is zero-filled once (tp_model.cu:3932-3933).
 * Page tables: int32 [max_slots][max_pages], max_pages = ceil(n_ctx / 2^psh); a sequence's row is its slot's
 * (tp_model.cu:3329); the batched row table is rtab[row] = slot * max_pages (tp_model.cu:3335, 4009).
 * Offload / file image of a sequence (tp_model.cu:3432-3434, 3688-3691): [page][K | V][kv layer][pblk] then the state
 * block - independent of the pool size.
 *
 * Return values: >= 0 success (ids, counts), < 0 a P1A_E_* code; p1a_last_error() holds the message, which repeats the
 * reference's exception text. Not thread-safe: one host thread drives a pool (src/tp_model.h:371).
 */
#ifndef P1A_POOL_H
#define P1A_POOL_H

#include <stddef.h>
#include <stdint.h>
#include "p1a_attn.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct p1a_pool p1a_pool;

typedef struct p1a_pool_cfg {
    uint32_t kv_type;     /* P1A_KV_F16 / P1A_KV_Q4_0 / P1A_KV_Q8_0 */
    int n_kv_layers;      /* KV layers in a page (attention layers + the MTP block), tp_model.h:472 */
    int Hkv, D;           /* this rank's kv heads, head size */
    int psh;              /* page shift (2^psh positions per page), tp_model.h:470 */
    int n_ctx;            /* per-sequence cap */
    int max_slots;        /* resident sequences */
    int64_t tokens;       /* pool size in tokens, rounded up to pages; < 0: what the device's free memory holds after
                             reserve_mb (tp_model.cu:3896-3915) */
    size_t reserve_mb;
    size_t state_bytes;   /* opaque per-sequence state that travels with a sequence (the engine's [conv | ssm] block of the
                             delta-net layers, tp_model.cu:3476-3478); zeroed at seq_create; 0 = none */
    size_t host_budget;   /* pinned host bytes offloaded sequences may hold (tp_model.cu:3446-3448); 0 = no limit */
    int host_memory;      /* 1: pool and tables live in host memory and no GPU call is made - for tools that read or
                             write session files on a machine without a GPU, and for tests of this host logic.
                             Descriptors of such a pool must not be handed to the attention entry points. */
} p1a_pool_cfg;

/* alloc_pool (tp_model.cu:3880-3966) + the slot / table set-up of the constructor. stream: the hipStream_t the copies,
 * fills and table uploads are ordered on (the model's stream S.s). NULL on failure. */
p1a_pool * p1a_pool_create(const p1a_pool_cfg * cfg, void * stream);
void p1a_pool_destroy(p1a_pool * p);

int p1a_pool_n_pages(const p1a_pool * p);
int p1a_pool_free_pages(const p1a_pool * p);
int p1a_pool_max_pages(const p1a_pool * p);        /* page-table entries per sequence */
size_t p1a_pool_page_bytes(const p1a_pool * p);    /* one page across all layers, K and V (tp_model.cu:3890) */
size_t p1a_pool_host_used(const p1a_pool * p);

/* kv_seq (tp_model.cu:3327-3331): layer's descriptor with pt = the sequence's table row, rtab = NULL */
int p1a_pool_kv_seq(const p1a_pool * p, int layer, int id, p1a_kv * out);
/* kv_rows (tp_model.cu:3333-3337): pt = the whole table, rtab = the device row table last written by p1a_pool_set_rows */
int p1a_pool_kv_rows(const p1a_pool * p, int layer, p1a_kv * out);
/* the row table of a batched step: row t belongs to sequence ids[t] (tp_model.cu:4005-4010); stream-ordered upload */
int p1a_pool_set_rows(p1a_pool * p, const int * ids, int nrows);
/* the sequence's state block in the pool's memory (NULL when state_bytes == 0 or not resident) */
void * p1a_pool_state(const p1a_pool * p, int id);

int p1a_seq_create(p1a_pool * p);                              /* tp_model.cu:3384-3403 -> id */
int p1a_seq_free(p1a_pool * p, int id);                        /* :3405-3416 */
int p1a_seq_ensure_pages(p1a_pool * p, int id, int n);         /* :3358-3382: pages for positions 0..n-1 */
int p1a_seq_len(const p1a_pool * p, int id);                   /* :3425 */
int p1a_seq_resident(const p1a_pool * p, int id);              /* :3426 */
int p1a_seq_pages(const p1a_pool * p, int id);                 /* :3427 */
size_t p1a_seq_host_bytes(const p1a_pool * p, int id);         /* :3428 */
/* bookkeeping of a forward step: T rows were appended at n_past (tokens toks[0..T-1], NULL = -1 as bench_fill_kv does,
 * tp_model.h:452); pages are ensured first */
int p1a_seq_advance(p1a_pool * p, int id, const int32_t * toks, int T);
/* rollback (tp_model.cu:3159-3170): of the last step's T rows keep the first n_keep; later KV rows are simply overwritten */
int p1a_seq_rollback(p1a_pool * p, int id, int T, int n_keep);
int p1a_seq_truncate(p1a_pool * p, int id, int n);             /* :3544-3559 */
int p1a_seq_fork(p1a_pool * p, int src, int n);                /* :3572-3603 -> id of the copy holding positions 0..n-1 */
int p1a_seq_offload(p1a_pool * p, int id);                     /* :3435-3490 */
int p1a_seq_restore(p1a_pool * p, int id);                     /* :3492-3496 */
int p1a_seq_restore_prefix(p1a_pool * p, int id, int n);       /* :3561-3570 */
/* pages_out (:3673-3684): resident pages p0..p0+n-1 -> dst in the offload layout; stream-ordered */
int p1a_seq_pages_out(p1a_pool * p, int id, int p0, int n, char * dst);
/* the sequence's tokens (n_past of them) */
int p1a_seq_tokens(const p1a_pool * p, int id, int32_t * dst, int cap);

/* The 15 x u64 fingerprint of session files (tp_model.cu:3693-3695, 3713-3716). The pool fills the KV-layout fields
 * itself - [5] KV type, [6] page shift, [7] GPU count (1), [8] page bytes, [9] state bytes, [10] KV layers - and takes
 * the model-identity fields ([0-4], [11-14]) from fp. */
int p1a_pool_set_fingerprint(p1a_pool * p, const uint64_t fp[15]);
int p1a_pool_fingerprint(const p1a_pool * p, uint64_t fp[15]);
/* seq_write / seq_read (tp_model.cu:3739-3863): "P100ESQ2" | fingerprint | n_past, n_tok, pages (i32) | tokens | pages x
 * page_bytes in the offload layout | state. seq_read returns the id of a new OFFLOADED sequence (restore it to use it). */
int p1a_seq_write(p1a_pool * p, int id, const char * path);
int p1a_seq_read(p1a_pool * p, const char * path);

/* MTP verify bookkeeping (src/sched.cpp:1053-1087, src/tp_mtp.cu:796-823): row r of a verify step carries the token
 * tokens[r] (tokens[0] = the last accepted token, then the drafts); greedy[r] is the model's token after row r.
 * Accepts drafts while greedy[r] == tokens[r + 1]; *n_accept = how many, *next = greedy[n_accept]; returns the rows to
 * keep q = min(n_accept + 1, budget) (budget = tokens still wanted, >= 1) - the caller emits q tokens and rolls back
 * (T, q). Pure host logic. */
int p1a_verify_accept(const int32_t * tokens, const int32_t * greedy, int T, int budget, int * n_accept, int32_t * next);

#ifdef __cplusplus
}
#endif
#endif
