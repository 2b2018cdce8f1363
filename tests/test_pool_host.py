"""Host logic of the paged KV pool / sequence manager / P100ESQ2 session files (include/p1a_pool.h), on a pool kept in
host memory (no GPU call). Checked against the reference's rules restated here by hand from src/tp_model.cu: pool layout
:3874-3879 and :3934-3942, ensure_pages :3358-3382, truncate :3544-3559, fork :3572-3603, offload image :3432-3434,
session file :3688-3691, verify bookkeeping src/sched.cpp:1053-1087."""
import ctypes
import importlib
import os
import struct

import numpy as np
import pytest

p1a = importlib.import_module("p100e-engine_amd")
KV_F16, KV_Q4_0, KV_Q8_0 = p1a.KV_F16, p1a.KV_Q4_0, p1a.KV_Q8_0


def rowb(t, Hkv, D):   # src/fast/attn.cu:501-503
    return {KV_F16: Hkv * D * 2, KV_Q8_0: Hkv * (D // 32) * 34, KV_Q4_0: Hkv * (D // 32) * 18}[t]


def mk(t=KV_Q8_0, L=3, Hkv=2, D=64, psh=4, n_ctx=200, slots=3, tokens=640, **kw):
    return p1a.Pool(t, L, Hkv, D, psh, n_ctx, slots, tokens, host_memory=True, **kw)


def table_row(c, n):
    return list((ctypes.c_int32 * n).from_address(c.pt)) if n else []


def pos_bytes(pool, mem, layer, seq, p, which):
    """the row of position p of a sequence, through the descriptor's addressing rule (src/fast/attn.cuh:23-27)"""
    c = pool.kv_seq(layer, seq)
    base0 = pool.kv_rows(0).k
    rb = rowb(c.type, c.Hkv, c.D)
    pt = table_row(c, (p >> c.psh) + 1)
    off = (c.k if which == 0 else c.v) - base0 + pt[p >> c.psh] * c.pstride + (p & ((1 << c.psh) - 1)) * rb
    return mem[off:off + rb]


def fill_seq(pool, mem, seq, n, L, seed):
    """write recognisable rows at positions 0..n-1 of every layer, K and V; returns them [layer][K|V][p]"""
    rng = np.random.default_rng(seed)
    pool.seq_advance(seq, toks=[int(x) for x in rng.integers(0, 1000, n)])
    want = {}
    for li in range(L):
        for w in range(2):
            for p in range(n):
                row = pos_bytes(pool, mem, li, seq, p, w)
                row[:] = rng.integers(0, 256, row.size, dtype=np.uint8)
                want[(li, w, p)] = row.copy()
    return want


def check_seq(pool, mem, seq, want, L, n):
    for li in range(L):
        for w in range(2):
            for p in range(n):
                assert np.array_equal(pos_bytes(pool, mem, li, seq, p, w), want[(li, w, p)]), (li, w, p)


@pytest.mark.parametrize("t", [KV_F16, KV_Q8_0, KV_Q4_0])
def test_pool_geometry_and_descriptors(t):
    L, Hkv, D, psh = 3, 2, 64, 4
    pool = mk(t, L, Hkv, D, psh, n_ctx=200, slots=3, tokens=630)
    rb = rowb(t, Hkv, D)
    pblk = (1 << psh) * rb
    assert pool.n_pages == (630 + 15) // 16 and pool.free_pages == pool.n_pages
    assert pool.max_pages == (200 + 15) // 16
    assert pool.page_bytes == L * 2 * pblk
    base = pool.kv_rows(0).k
    for li in range(L):
        c = pool.kv_rows(li)
        assert (c.type, c.Hkv, c.D, c.psh, c.pstride, c.n_ctx) == (t, Hkv, D, psh, pblk, 200)
        assert c.k - base == li * pool.n_pages * pblk and c.v - base == (L + li) * pool.n_pages * pblk
        assert c.rtab is not None
    assert not pool.memory().any()                       # zero-filled (tp_model.cu:3932-3933)
    fp = pool.fingerprint()
    assert fp[5:11] == [t, psh, 1, pool.page_bytes, 0, L]
    with pytest.raises(p1a.P1AError, match="layer"):
        pool.kv_rows(L)


def test_pages_are_handed_out_in_order_and_come_back():
    pool = mk(tokens=16 * 10, n_ctx=160, slots=3)          # 10 pages
    a, b = pool.seq_create(), pool.seq_create()
    pool.ensure_pages(a, 17)                               # 2 pages
    pool.ensure_pages(b, 1)
    pool.ensure_pages(a, 40)                               # a third page for a
    assert table_row(pool.kv_seq(0, a), 3) == [0, 1, 3] and table_row(pool.kv_seq(0, b), 1) == [2]
    assert pool.seq_pages(a) == 3 and pool.free_pages == 6
    pool.ensure_pages(a, 40)                               # nothing new
    assert pool.free_pages == 6
    # the two sequences' table rows are max_pages apart in one table (tp_model.cu:3329)
    assert pool.kv_seq(0, a).pt != pool.kv_seq(0, b).pt and abs(pool.kv_seq(0, a).pt - pool.kv_seq(0, b).pt) == 4 * pool.max_pages
    with pytest.raises(p1a.P1AError, match="context full"):
        pool.ensure_pages(a, 161)
    with pytest.raises(p1a.P1AError, match=r"KV pool full \(6 free pages, need 7\)"):
        c = pool.seq_create()
        pool.ensure_pages(c, 16 * 7)
    # truncate gives back the pages past the cut, last first; they are the next ones handed out
    pool.seq_advance(a, T=40)
    pool.seq_truncate(a, 16)
    assert pool.seq_pages(a) == 1 and pool.seq_len(a) == 16 and pool.free_pages == 8
    pool.ensure_pages(b, 48)
    assert table_row(pool.kv_seq(0, b), 3) == [2, 1, 3]
    with pytest.raises(p1a.P1AError, match="position out of range"):
        pool.seq_truncate(a, 17)
    pool.seq_free(b)
    assert pool.free_pages == 9 and not pool.seq_resident(b)
    with pytest.raises(p1a.P1AError, match="not resident"):
        pool.ensure_pages(b, 1)


def test_slots_run_out_and_are_reused():
    pool = mk(slots=2)
    a, b = pool.seq_create(), pool.seq_create()
    with pytest.raises(p1a.P1AError, match=r"no free sequence slot \(max_seqs 2\)"):
        pool.seq_create()
    pool.seq_free(a)
    assert pool.seq_create() == a                          # the first unused id is taken again


def test_row_table_of_a_batched_step():
    pool = mk(slots=3)
    ids = [pool.seq_create() for _ in range(3)]
    pool.set_rows([ids[2], ids[0], ids[0], ids[1]])
    c = pool.kv_rows(1)
    rt = list((ctypes.c_int32 * 4).from_address(c.rtab))
    slots = [(pool.kv_seq(0, i).pt - c.pt) // 4 for i in ids]   # each sequence's slot * max_pages (tp_model.cu:4009)
    assert rt == [slots[2], slots[0], slots[0], slots[1]] and sorted(s // pool.max_pages for s in slots) == [0, 1, 2]


def test_advance_and_rollback_bookkeeping():
    pool = mk()
    a = pool.seq_create()
    assert pool.seq_advance(a, toks=[5, 6, 7]) == 3
    assert pool.seq_advance(a, toks=[8, 9, 10, 11]) == 7      # a verify step of 4 rows
    assert pool.rollback(a, 4, 2) == 5 and pool.seq_tokens(a) == [5, 6, 7, 8, 9]
    assert pool.rollback(a, 4, 4) == 5                         # nothing to drop
    with pytest.raises(p1a.P1AError, match="rollback out of range"):
        pool.rollback(a, 4, 0)
    with pytest.raises(p1a.P1AError, match="rollback out of range"):
        pool.rollback(a, 6, 1)
    assert pool.seq_advance(a, T=2) == 7 and pool.seq_tokens(a)[-2:] == [-1, -1]   # rows without tokens (tp_model.h:452)
    assert pool.seq_pages(a) == 1


def test_fork_copies_every_layer_and_is_independent():
    L = 3
    pool = mk(L=L, tokens=16 * 12)
    mem = pool.memory()
    a = pool.seq_create()
    want = fill_seq(pool, mem, a, 37, L, seed=1)
    b = pool.seq_fork(a, 20)                                   # 2 pages
    assert pool.seq_len(b) == 20 and pool.seq_pages(b) == 2 and pool.seq_tokens(b) == pool.seq_tokens(a)[:20]
    assert set(table_row(pool.kv_seq(0, a), 3)).isdisjoint(table_row(pool.kv_seq(0, b), 2))
    check_seq(pool, mem, b, want, L, 20)
    # whole pages are copied: the rest of the second page too
    check_seq(pool, mem, b, want, L, 32)
    pos_bytes(pool, mem, 1, b, 3, 0)[:] = 0xEE
    check_seq(pool, mem, a, want, L, 37)                       # the source does not see the copy's writes
    with pytest.raises(p1a.P1AError, match="position out of range"):
        pool.seq_fork(a, 38)


def test_offload_restore_round_trip_and_prefix():
    L = 2
    pool = mk(L=L, tokens=16 * 8, slots=2, state_bytes=24)
    mem = pool.memory()
    a = pool.seq_create()
    want = fill_seq(pool, mem, a, 50, L, seed=2)               # 4 pages
    st = (ctypes.c_uint8 * 24).from_address(pool.state(a))
    st[:] = bytes(range(100, 124))
    pool.seq_offload(a)
    assert not pool.seq_resident(a) and pool.free_pages == 8 and pool.seq_pages(a) == 4
    assert pool.seq_host_bytes(a) == 4 * pool.page_bytes + 24 == pool.host_used
    # somebody else takes the first pages meanwhile
    b = pool.seq_create()
    pool.ensure_pages(b, 33)
    mem[:] = 0x55
    pool.seq_restore(a)
    assert pool.seq_resident(a) and pool.host_used == 0 and table_row(pool.kv_seq(0, a), 4) == [3, 4, 5, 6]
    check_seq(pool, mem, a, want, L, 50)
    assert bytes((ctypes.c_uint8 * 24).from_address(pool.state(a))) == bytes(range(100, 124))
    # prefix: only the pages of the first n positions come back, the state block starts from zero (tp_model.cu:3561-3570)
    pool.seq_offload(a)
    pool.seq_restore_prefix(a, 20)
    assert pool.seq_len(a) == 20 and pool.seq_pages(a) == 2 and len(pool.seq_tokens(a)) == 20
    check_seq(pool, mem, a, want, L, 20)
    assert bytes((ctypes.c_uint8 * 24).from_address(pool.state(a))) == bytes(24)
    with pytest.raises(p1a.P1AError, match="not offloaded"):
        pool.seq_restore(a)


def test_host_budget_is_enforced():
    pool = mk(L=1, tokens=16 * 8, host_budget=3 * 1024)
    a = pool.seq_create()
    pool.seq_advance(a, T=40)                                   # 3 pages of 16 * 272 * 2 bytes: over 3 KiB
    with pytest.raises(p1a.P1AError, match="host budget exceeded"):
        pool.seq_offload(a)
    assert pool.seq_resident(a)


def parse_session(path, L, pblk, state_bytes):
    """independent reader of the file format (tp_model.cu:3688-3691)"""
    raw = open(path, "rb").read()
    assert raw[:8] == b"P100ESQ2"
    fp = list(struct.unpack("<15Q", raw[8:128]))
    n_past, n_tok, np_ = struct.unpack("<3i", raw[128:140])
    toks = list(struct.unpack(f"<{n_tok}i", raw[140:140 + 4 * n_tok]))
    body = np.frombuffer(raw, dtype=np.uint8, offset=140 + 4 * n_tok)
    assert body.size == np_ * L * 2 * pblk + state_bytes
    pages = body[:np_ * L * 2 * pblk].reshape(np_, 2, L, pblk)      # [page][K|V][kv layer][page rows]
    return fp, n_past, toks, pages, bytes(body[np_ * L * 2 * pblk:])


@pytest.mark.parametrize("resident", [True, False])
def test_session_file_layout_and_reload_into_another_pool(tmp_path, resident):
    L, Hkv, D, psh, t = 2, 2, 64, 4, KV_Q8_0
    pool = mk(t, L, Hkv, D, psh, n_ctx=200, slots=2, tokens=16 * 9, state_bytes=16)
    ident = [11, 22, 33, 44, 1000, 0, 0, 0, 0, 0, 0, 1, 77, 88, 99]
    pool.set_fingerprint(ident)
    mem = pool.memory()
    other = pool.seq_create()
    pool.ensure_pages(other, 20)                                # so the saved sequence does not sit on pages 0..
    a = pool.seq_create()
    want = fill_seq(pool, mem, a, 41, L, seed=3)                # 3 pages
    (ctypes.c_uint8 * 16).from_address(pool.state(a))[:] = bytes(range(16))
    if not resident:
        pool.seq_offload(a)
    path = str(tmp_path / "s.p100esq")
    pool.seq_write(a, path)
    rb = rowb(t, Hkv, D)
    pblk = 16 * rb
    fp, n_past, toks, pages, state = parse_session(path, L, pblk, 16)
    assert fp == ident[:5] + [t, psh, 1, L * 2 * pblk, 16, L] + ident[11:]
    assert n_past == 41 and toks == pool.seq_tokens(a) and state == bytes(range(16))
    for li in range(L):
        for w in range(2):
            for p in range(41):
                assert np.array_equal(pages[p >> psh, w, li, (p & 15) * rb:(p & 15) * rb + rb], want[(li, w, p)])
    # a pool of another size (the image does not depend on it), pages taken in between
    pool2 = mk(t, L, Hkv, D, psh, n_ctx=300, slots=3, tokens=16 * 20, state_bytes=16)
    pool2.set_fingerprint(ident)
    x = pool2.seq_create()
    pool2.ensure_pages(x, 70)
    b = pool2.seq_read(path)
    assert not pool2.seq_resident(b) and pool2.seq_len(b) == 41 and pool2.seq_pages(b) == 3
    pool2.seq_restore(b)
    check_seq(pool2, pool2.memory(), b, want, L, 41)
    assert bytes((ctypes.c_uint8 * 16).from_address(pool2.state(b))) == bytes(range(16))
    assert pool2.seq_tokens(b) == toks


def test_session_file_refusals(tmp_path):
    pool = mk(L=1, tokens=16 * 4)
    ident = [1, 2, 3, 4, 50, 0, 0, 0, 0, 0, 0, 0, 5, 6, 7]
    pool.set_fingerprint(ident)
    a = pool.seq_create()
    pool.seq_advance(a, toks=[1, 2, 49])
    good = str(tmp_path / "g")
    pool.seq_write(a, good)
    raw = open(good, "rb").read()

    def attempt(data, match, p=pool):
        f = str(tmp_path / "x")
        open(f, "wb").write(data)
        free, used = p.free_pages, p.host_used
        with pytest.raises(p1a.P1AError, match=match):
            p.seq_read(f)
        assert (p.free_pages, p.host_used) == (free, used)       # a refused file leaves nothing behind

    attempt(b"P100ESQ1" + raw[8:], "version 1 sequence file")
    attempt(b"GGUFGGUF" + raw[8:], "not a p100e sequence file")
    attempt(raw[:-1], "short file")
    attempt(raw[:100], "short file")
    bad_tok = bytearray(raw)
    bad_tok[140 + 8:140 + 12] = struct.pack("<i", 50)
    attempt(bytes(bad_tok), "token id 50 out of range")
    bad_hdr = bytearray(raw)
    bad_hdr[136:140] = struct.pack("<i", 0)                      # 0 pages cannot hold 3 positions
    attempt(bytes(bad_hdr), "bad header")
    other = mk(L=1, tokens=16 * 4, psh=5)
    other.set_fingerprint(ident)
    attempt(raw, r"another model / KV layout \(page shift 4 vs 5\)", other)
    other2 = mk(L=1, tokens=16 * 4)
    other2.set_fingerprint(ident[:12] + [9, 6, 7])
    attempt(raw, r"GGUF metadata hash 5 vs 9", other2)
    with pytest.raises(p1a.P1AError, match="cannot open"):
        pool.seq_read(str(tmp_path / "missing"))


def test_verify_accept_follows_the_scheduler():
    va = p1a.verify_accept
    # tokens = [last, d1, d2, d3]; greedy[r] = the model's token after row r (src/sched.cpp:1066-1069)
    assert va([7, 1, 2, 3], [1, 2, 3, 4], 10) == (4, 3, 4)          # all drafts accepted + the bonus token
    assert va([7, 1, 2, 3], [9, 2, 3, 4], 10) == (1, 0, 9)          # first draft wrong: only the corrected token
    assert va([7, 1, 2, 3], [1, 2, 8, 4], 10) == (3, 2, 8)
    assert va([7], [5], 10) == (1, 0, 5)                             # plain decode row
    assert va([7, 1, 2, 3], [1, 2, 3, 4], 2) == (2, 3, 4)           # only two tokens still wanted (sched.cpp:1079)
    with pytest.raises(p1a.P1AError):
        va([7, 1], [1, 2], 0)
