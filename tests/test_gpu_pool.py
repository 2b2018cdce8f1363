"""The device pool / sequence manager (include/p1a_pool.h) under the attention entry points: KV written through the
pool's descriptors decodes like the oracle on the same rows, the session file holds exactly the oracle's KV bytes
(so pages are interchangeable with the engine's: src/tp_model.cu:3688-3691), and a sequence survives offload / restore
and a file round trip bit for bit."""
import importlib
import struct

import numpy as np
import pytest
import torch

import _inputs as I
import _oracle as O
from _gpu import dev

p1a = importlib.import_module("p100e-engine_amd")
pytestmark = pytest.mark.gpu


class Desc:
    """a p1a_kv struct handed out by the pool, in the shape the binding's entry points take"""

    def __init__(self, st):
        self._st = st

    def struct(self):
        return self._st


@pytest.mark.parametrize("kv_type", [p1a.KV_Q8_0, p1a.KV_Q4_0, p1a.KV_F16])
def test_pool_sequences_decode_like_the_oracle_and_survive_moves(kv_type, tmp_path):
    L, Hq, Hkv, D, psh, il = 2, 24, 4, 256, 5, 1
    pool = p1a.Pool(kv_type, L, Hkv, D, psh, n_ctx=1024, max_slots=3, tokens=32 * 40, state_bytes=128)
    ident = [9, 8, 7, 6, 151936, 0, 0, 0, 0, 0, 0, 1, 3, 4, 5]
    pool.set_fingerprint(ident)
    a, b = pool.seq_create(), pool.seq_create()
    lens = {a: 0, b: 0}
    rows = {a: ([], []), b: ([], [])}
    for step, T in enumerate([70, 1, 33, 100, 4]):           # grown in turns: the two sequences' pages interleave
        for s in (a, b):
            _, k, v, _ = I.qkv(1000 + step * 7 + s, T, 1, Hq, Hkv, D)
            pool.seq_advance(s, toks=[step] * T)
            for l in range(L):                                # the other layer gets other rows
                kk, vv = (k, v) if l == il else (v, k)
                p1a.kv_append(Desc(pool.kv_seq(l, s)), dev(kk), dev(vv), lens[s], T)
            rows[s][0].append(k)
            rows[s][1].append(v)
            lens[s] += T
    torch.cuda.synchronize()
    scale = 1.0 / 16
    host = {}
    for s in (a, b):                                          # the oracle's cache of the same rows, contiguous
        h = O.HostKV.contiguous(kv_type, lens[s], Hkv, D)
        O.kv_append_rows(h.view(), np.concatenate(rows[s][0]), np.concatenate(rows[s][1]), np.arange(lens[s]))
        host[s] = h

    def decode(desc, s, T=4):
        q = I.qkv(77 + s, 1, T, Hq, Hkv, D)[0]
        out = torch.empty((T, Hq, D), device="cuda")
        p1a.attn_decode(dev(q), Desc(desc), out, T, lens[s] - T, Hq, scale)
        torch.cuda.synchronize()
        want = O.attn_rows(host[s].view(), q, np.arange(lens[s] - T, lens[s]), Hq, scale)
        got = out.cpu().numpy()
        assert np.abs(got - want).max() <= 2e-3 and np.linalg.norm(got - want) <= 1e-3 * np.linalg.norm(want)
        return got

    ref = {s: decode(pool.kv_seq(il, s), s) for s in (a, b)}
    # the file holds the oracle's bytes: [page][K|V][layer][page rows]
    path = str(tmp_path / "a.p100esq")
    pool.seq_write(a, path)
    raw = open(path, "rb").read()
    rb = O.row_bytes(kv_type, Hkv, D)
    pblk = 32 * rb
    n_past, n_tok, npg = struct.unpack("<3i", raw[128:140])
    assert raw[:8] == b"P100ESQ2" and n_past == lens[a] == n_tok and npg == (lens[a] + 31) // 32
    body = np.frombuffer(raw, np.uint8, offset=140 + 4 * n_tok)
    pages = body[:npg * L * 2 * pblk].reshape(npg, 2, L, pblk)
    hk, hv = host[a].k.reshape(lens[a], rb), host[a].v.reshape(lens[a], rb)
    for p in range(lens[a]):
        assert np.array_equal(pages[p >> 5, 0, il, (p & 31) * rb:(p & 31) * rb + rb], hk[p]), p
        assert np.array_equal(pages[p >> 5, 1, il, (p & 31) * rb:(p & 31) * rb + rb], hv[p]), p
    # fork, offload + restore onto other pages, file -> another pool: the same bits every time
    f = pool.seq_fork(a, lens[a])
    lens[f], host[f] = lens[a], host[a]
    q4 = I.qkv(77 + a, 1, 4, Hq, Hkv, D)[0]

    def bits(desc, n):
        out = torch.empty((4, Hq, D), device="cuda")
        p1a.attn_decode(dev(q4), Desc(desc), out, 4, n - 4, Hq, scale)
        torch.cuda.synchronize()
        return out.cpu().numpy()

    assert np.array_equal(bits(pool.kv_seq(il, f), lens[a]), ref[a])
    pool.seq_free(f)
    pool.seq_offload(a)
    filler = pool.seq_create()
    pool.ensure_pages(filler, 32 * 3)
    pool.seq_restore(a)
    assert np.array_equal(bits(pool.kv_seq(il, a), lens[a]), ref[a])
    pool2 = p1a.Pool(kv_type, L, Hkv, D, psh, n_ctx=2048, max_slots=2, tokens=32 * 64, state_bytes=128)
    pool2.set_fingerprint(ident)
    x = pool2.seq_create()
    pool2.ensure_pages(x, 100)
    r = pool2.seq_read(path)
    pool2.seq_restore(r)
    assert pool2.seq_len(r) == lens[a] and np.array_equal(bits(pool2.kv_seq(il, r), lens[a]), ref[a])
    # batched rows of both sequences through the pool's row table
    pool.set_rows([b, a])
    q2 = np.concatenate([I.qkv(77 + b, 1, 4, Hq, Hkv, D)[0][3:4], q4[3:4]])
    out = torch.empty((2, Hq, D), device="cuda")
    p1a.attn_decode_rows(dev(q2), Desc(pool.kv_rows(il)), out, 2, dev(np.array([lens[b] - 1, lens[a] - 1], np.int32)), Hq, scale)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.array_equal(got[0], ref[b][3]) and np.array_equal(got[1], ref[a][3])
    pool2.close()
    pool.close()


def test_verify_steps_with_rollback_keep_the_cache_consistent():
    """An MTP verify loop (src/tp_mtp.cu:779-823): each step appends 1 + 3 rows, a prefix is accepted, the rest rolled
    back and overwritten by the next step. The cache must end up as if only the kept rows had ever been written."""
    kv_type, L, Hq, Hkv, D, psh = p1a.KV_Q8_0, 1, 24, 4, 256, 4
    pool = p1a.Pool(kv_type, L, Hkv, D, psh, n_ctx=512, max_slots=1, tokens=512)
    s = pool.seq_create()
    rng = np.random.default_rng(5)
    kept_k, kept_v, n = [], [], 0
    _, k0, v0, _ = I.qkv(1, 37, 1, Hq, Hkv, D)
    pool.seq_advance(s, toks=list(range(37)))
    p1a.kv_append(Desc(pool.kv_seq(0, s)), dev(k0), dev(v0), 0, 37)
    kept_k.append(k0); kept_v.append(v0); n = 37
    for step in range(12):
        T = 4
        _, k, v, _ = I.qkv(100 + step, T, 1, Hq, Hkv, D)
        tokens = [int(x) for x in rng.integers(0, 50, T)]
        greedy = list(tokens[1:]) + [int(rng.integers(0, 50))]
        cut = int(rng.integers(0, T))                         # the first wrong draft
        if cut < T - 1:
            greedy[cut] = tokens[cut + 1] + 1
        pool.seq_advance(s, toks=tokens)
        p1a.kv_append(Desc(pool.kv_seq(0, s)), dev(k), dev(v), n, T)
        keep, n_acc, _ = p1a.verify_accept(tokens, greedy, budget=100)
        assert keep == min(cut, T - 1) + 1 == n_acc + 1
        assert pool.rollback(s, T, keep) == n + keep
        kept_k.append(k[:keep]); kept_v.append(v[:keep]); n += keep
    torch.cuda.synchronize()
    assert pool.seq_len(s) == n
    h = O.HostKV.contiguous(kv_type, n, Hkv, D)
    O.kv_append_rows(h.view(), np.concatenate(kept_k), np.concatenate(kept_v), np.arange(n))
    q, _, _, _ = I.qkv(9, 1, 1, Hq, Hkv, D)
    out = torch.empty((1, Hq, D), device="cuda")
    p1a.attn_decode(dev(q), Desc(pool.kv_seq(0, s)), out, 1, n - 1, Hq, 1 / 16)
    torch.cuda.synchronize()
    want = O.attn_rows(h.view(), q, np.array([n - 1]), Hq, 1 / 16)
    got = out.cpu().numpy()
    assert np.abs(got - want).max() <= 2e-3 and np.linalg.norm(got - want) <= 1e-3 * np.linalg.norm(want)
    pool.close()
