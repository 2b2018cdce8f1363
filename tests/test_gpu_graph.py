"""The decode step as the engine runs it: captured once into a graph (after p1a_warmup, so that the library's split
buffers exist), replayed at other depths with the positions read on the device (src/tp_model.cu:1379-1397); the split
count knobs (attn_dec2_nsplit / attn_dec2_set_nsplit, src/fast/attn_dec2.cuh:19-20); p1a_release."""
import numpy as np
import pytest
import torch

import _inputs as I
import _oracle as O
from _gpu import Pool, check, dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kv_type", [O.KV_Q8_0, O.KV_Q4_0])
def test_captured_step_replays_at_any_depth(p1a, kv_type):
    """one verify step (attn_prep with device positions: q | gate split, norm, rope, quantizing KV write; then the decode
    over device positions with the fused gate) captured at one depth and replayed at others, with new inputs copied into
    the captured buffers: the same bits as the eager calls, and the oracle's attention"""
    Hq, Hkv, D, psh, T, n_rot = 12, 2, 256, 5, 4, 64
    lens = [40]
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [3000], seed=111, fill="none")
    twin = Pool(p1a, kv_type, Hq, Hkv, D, psh, [3000], seed=111, fill="none")    # the eager side writes its own cache
    g = I.rng(112)
    hist_k, hist_v = I.normal(g, (2990, Hkv, D)), I.normal(g, (2990, Hkv, D))
    for p in (pool, twin):
        p1a.kv_append(p.dev_seq(0), dev(hist_k), dev(hist_v), 0, 2990)
    O.kv_append_rows(pool.host_seq(0), hist_k, hist_v, np.arange(2990))
    qn, kn = dev((1.0 + 0.1 * I.normal(g, (D,))).astype(np.float32)), dev((1.0 + 0.1 * I.normal(g, (D,))).astype(np.float32))
    s = torch.cuda.Stream()
    qg, k, v = (torch.zeros((T, Hq, 2 * D), device="cuda"), torch.zeros((T, Hkv, D), device="cuda"), torch.zeros((T, Hkv, D), device="cuda"))
    pos = torch.zeros(T, dtype=torch.int32, device="cuda")
    q, gate, out = torch.zeros((T, Hq, D), device="cuda"), torch.zeros((T, Hq * D), device="cuda"), torch.zeros((T, Hq, D), device="cuda")
    c = pool.dev_seq(0)

    def step(cache, out_):
        p1a.attn_prep(qg, k, v, qn, kn, pos, q, gate, cache.with_rows(rt), -1, T, Hq, n_rot, 1e7, 1e-6)
        p1a.attn_decode_dev(q, cache, out_, T, pos, 0, Hq, 1 / 16, gate=gate)

    rt = torch.zeros(T, dtype=torch.int32, device="cuda")        # every row in the sequence's own table (offset 0)
    with torch.cuda.stream(s):
        p1a.warmup(T, Hq, Hkv, D)
        s.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            step(c, out)
    for depth in (100, 2990 - T, 31, 1024, 2047):
        hq, hk, hv = I.normal(g, (T, Hq, 2 * D)), I.normal(g, (T, Hkv, D)), I.normal(g, (T, Hkv, D))
        hp = (depth + np.arange(T)).astype(np.int32)
        with torch.cuda.stream(s):
            qg.copy_(dev(hq)); k.copy_(dev(hk)); v.copy_(dev(hv)); pos.copy_(dev(hp))
            graph.replay()
            s.synchronize()
            got = out.cpu().numpy().copy()
            eager = torch.zeros((T, Hq, D), device="cuda")
            step(twin.dev_seq(0), eager)
            s.synchronize()
        assert np.array_equal(got, eager.cpu().numpy()), depth
        assert np.array_equal(pool.dpool.cpu().numpy(), twin.dpool.cpu().numpy()), depth
        # (the oracle on the same cache bytes: the rows below `depth` are the history, then whatever earlier steps wrote)
        host = O.HostKV.paged(kv_type, Hkv, D, psh, pool.np_pages, pool.tabs, pool.maxp, n_layers=2, layer=1, pool=pool.dpool.cpu().numpy().copy())
        ref = O.attn_rows(host.view(pt=pool.tabs), q.cpu().numpy(), hp, Hq, 1 / 16, gate=gate.cpu().numpy())
        check(got, ref, f"captured step at depth {depth}, type {kv_type}")


def test_growth_during_capture_is_refused_and_knobs(p1a):
    Hq, Hkv, D, n = 12, 2, 256, 2000
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, 6, [n], seed=113)
    q, _, _, gate = I.qkv(114, 1, 2, Hq, Hkv, D)
    dq, dg = dev(q), dev(gate)
    ref = O.attn_rows(pool.host_seq(0), q, np.array([n - 2, n - 1], np.int32), Hq, 1 / 16, gate=gate)
    c = pool.dev_seq(0)
    out = torch.zeros((2, Hq, D), device="cuda")
    # a stream the library has never seen: its split buffers would have to be allocated inside the capture
    s = torch.cuda.Stream()
    refused = False
    with torch.cuda.stream(s):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            try:
                p1a.attn_decode(dq, c, out, 2, n - 2, Hq, 1 / 16, gate=dg)
            except p1a.P1AError:
                refused = True
    assert refused
    # the split count: the default, a smaller one (other partials, the same attention), back
    n0 = p1a.get_nsplit(Hkv)
    assert n0 >= 8
    p1a.attn_decode(dq, c, out, 2, n - 2, Hq, 1 / 16, gate=dg)
    torch.cuda.synchronize()
    base = out.cpu().numpy().copy()
    check(base, ref, "default split count")
    p1a.set_nsplit(16)
    try:
        assert p1a.get_nsplit(Hkv) == 16
        p1a.attn_decode(dq, c, out, 2, n - 2, Hq, 1 / 16, gate=dg)
        torch.cuda.synchronize()
        check(out.cpu().numpy(), ref, "16 split streams")
    finally:
        p1a.set_nsplit(0)
    assert p1a.get_nsplit(Hkv) == n0
    # release: every buffer of the library goes; the next call brings its own back and gives the same bits
    p1a.lib().p1a_release()
    p1a.attn_decode(dq, c, out, 2, n - 2, Hq, 1 / 16, gate=dg)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), base)


def test_two_streams_and_two_host_threads(p1a):
    """calls on different streams of one device may overlap (the split buffers belong to a (device, stream) pair, the table of
    pairs is mutex-protected): two host threads, each on its own stream, run decode and key-split prefill calls over their
    own sequences at the same time, many times; every result equals the one computed alone"""
    import threading
    Hq, Hkv, D, psh = 12, 2, 256, 6
    lens = [6000, 4500]
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, psh, lens, seed=115)
    work = []
    for sq, n in enumerate(lens):
        q, _, _, gate = I.qkv(116 + sq, 1, 4, Hq, Hkv, D)
        qp, _, _, gp = I.qkv(118 + sq, 1, 100, Hq, Hkv, D, f16_inputs=True)
        work.append(dict(c=pool.dev_seq(sq), n=n, q=dev(q), g=dev(gate), qp=dev(qp), gp=dev(gp)))
    assert p1a.prefill_key_splits(100, lens[0] - 100, Hq) > 1
    def once(w, out, outp):
        p1a.attn_decode(w["q"], w["c"], out, 4, w["n"] - 4, Hq, 1 / 16, gate=w["g"])
        p1a.attn_prefill(w["qp"], w["c"], outp, 100, w["n"] - 100, Hq, 1 / 16, gate=w["gp"])
    alone = []
    for w in work:
        out, outp = torch.zeros((4, Hq, D), device="cuda"), torch.zeros((100, Hq, D), device="cuda")
        once(w, out, outp)
        torch.cuda.synchronize()
        alone.append((out.clone(), outp.clone()))
    bad = []
    def run(i):
        s = torch.cuda.Stream()
        w = work[i]
        with torch.cuda.stream(s):
            for rep in range(40):
                out, outp = torch.zeros((4, Hq, D), device="cuda"), torch.zeros((100, Hq, D), device="cuda")
                once(w, out, outp)
                if rep % 8 == 7:
                    s.synchronize()
                    if not (torch.equal(out, alone[i][0]) and torch.equal(outp, alone[i][1])):
                        bad.append((i, rep))
            s.synchronize()
    th = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    for t in th: t.start()
    for t in th: t.join()
    assert not bad, bad


def test_captured_graph_survives_larger_calls_on_its_stream(p1a):
    """the engine's normal flow: a decode graph captured after the warm-up, then eager work on the same stream that needs
    the library's buffers at other sizes - a 32-row decode, a key-split prefill without caller scratch, a decode of another
    head shape (more scratch than the first footprint) - and then the graph again: the buffers it holds are still there,
    so it gives the bits of the eager call"""
    Hq, Hkv, D, psh, n = 12, 2, 256, 6, 5000
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, psh, [n], seed=121)
    c = pool.dev_seq(0)
    q, _, _, gate = I.qkv(122, 1, 4, Hq, Hkv, D)
    dq, dg = dev(q), dev(gate)
    pos = dev(np.array([n - 4], np.int32))
    s = torch.cuda.Stream()
    out = torch.zeros((4, Hq, D), device="cuda")
    big = Pool(p1a, O.KV_F16, 32, 2, 256, 6, [600], seed=123)           # GQA 16: another head shape, a larger footprint
    qb, _, _, _ = I.qkv(124, 1, 2, 32, 2, 256)
    q32, _, _, g32 = I.qkv(125, 1, 32, Hq, Hkv, D)
    qp, _, _, gp = I.qkv(126, 1, 100, Hq, Hkv, D, f16_inputs=True)
    assert p1a.prefill_key_splits(100, n - 100, Hq) > 1
    with torch.cuda.stream(s):
        p1a.warmup(8, Hq, Hkv, D)
        eager = torch.zeros((4, Hq, D), device="cuda")
        p1a.attn_decode_dev(dq, c, eager, 4, pos, 0, Hq, 1 / 16, gate=dg)
        s.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            p1a.attn_decode_dev(dq, c, out, 4, pos, 0, Hq, 1 / 16, gate=dg)
        graph.replay()
        s.synchronize()
        assert torch.equal(out, eager)
        # eager calls that need other buffers
        o32 = torch.zeros((32, Hq, D), device="cuda")
        p1a.attn_decode(dev(q32), c, o32, 32, n - 32, Hq, 1 / 16, gate=dev(g32))
        op = torch.zeros((100, Hq, D), device="cuda")
        p1a.attn_prefill(dev(qp), c, op, 100, n - 100, Hq, 1 / 16, gate=dev(gp))
        ob = torch.zeros((2, 32, 256), device="cuda")
        p1a.attn_decode(dev(qb), big.dev_seq(0), ob, 2, 598, 32, 1 / 16)
        s.synchronize()
        check(o32.cpu().numpy(), O.attn_rows(pool.host_seq(0), q32, (n - 32 + np.arange(32)).astype(np.int32), Hq, 1 / 16, gate=g32), "32 rows")
        for rep in range(3):
            out.zero_()
            graph.replay()
            # (the program's own eager work between replays)
            p1a.attn_decode(dev(qb), big.dev_seq(0), ob, 2, 598, 32, 1 / 16)
            s.synchronize()
            assert torch.equal(out, eager), rep


def test_captured_key_split_prefill_is_refused_or_exact(p1a):
    """the key-split count fixes the result bits, so it never depends on whether the stream is being captured: without the
    library's partial buffers the captured call is refused; after p1a_warmup_prefill it gives the eager bits"""
    Hq, Hkv, D, psh, n, T = 12, 2, 256, 6, 6000, 100
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, psh, [n], seed=127)
    c = pool.dev_seq(0)
    qp, _, _, gp = I.qkv(128, 1, T, Hq, Hkv, D, f16_inputs=True)
    dq, dg = dev(qp), dev(gp)
    assert p1a.prefill_key_splits(T, n - T, Hq) > 1
    eager = torch.zeros((T, Hq, D), device="cuda")
    p1a.attn_prefill(dq, c, eager, T, n - T, Hq, 1 / 16, gate=dg)
    torch.cuda.synchronize()
    s = torch.cuda.Stream()                                            # a stream the library has never seen
    out = torch.zeros((T, Hq, D), device="cuda")
    refused = False
    with torch.cuda.stream(s):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            try:
                p1a.attn_prefill(dq, c, out, T, n - T, Hq, 1 / 16, gate=dg)
            except p1a.P1AError:
                refused = True
    assert refused
    s2 = torch.cuda.Stream()
    with torch.cuda.stream(s2):
        p1a.warmup_prefill(T, n - T, Hq, Hkv, D)
        s2.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s2):
            p1a.attn_prefill(dq, c, out, T, n - T, Hq, 1 / 16, gate=dg)
        for rep in range(2):
            out.zero_()
            graph.replay()
            s2.synchronize()
            assert torch.equal(out, eager), rep



def test_batched_rows_in_a_graph(p1a):
    """A batched call (8 rows of 4 sequences at their own positions - the two-workgroups-per-CU build of the kernel) captured
    once and replayed while the sequences grow: every replay equals the eager call and, row by row, the call of that row alone"""
    Hq, Hkv, D, psh = 24, 4, 256, 6
    lens = [900, 450, 1300, 70]
    pool = Pool(p1a, O.KV_Q4_0, Hq, Hkv, D, psh, lens, seed=52)
    rows = [(s, 0) for s in range(4) for _ in range(2)]
    q = dev(I.normal(I.rng(53), (8, Hq, D)))
    gate = dev(I.normal(I.rng(54), (8, Hq * D)))
    rt = dev(np.array([s * pool.maxp for s, _ in rows], np.int32))
    cr = pool.devkv.with_rows(rt)
    pos = dev(np.zeros(8, np.int32))
    out_g = torch.empty((8, Hq, D), device="cuda")
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        p1a.warmup(8, Hq, Hkv, D)
        pos.copy_(torch.tensor([10, 11] * 4, dtype=torch.int32))
        s.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            p1a.attn_decode_rows(q, cr, out_g, 8, pos, Hq, 1 / 16, gate=gate, rows_per_seq=2)
        for back in (40, 20, 0):
            ph = np.array([lens[sq] - 2 - back + t for sq in range(4) for t in range(2)], np.int32)
            pos.copy_(torch.from_numpy(ph))
            g.replay()
            s.synchronize()
            eager = torch.empty_like(out_g)
            p1a.attn_decode_rows(q, cr, eager, 8, pos, Hq, 1 / 16, gate=gate, rows_per_seq=2)
            s.synchronize()
            assert torch.equal(out_g, eager), back
            for t in range(8):
                one = torch.empty((1, Hq, D), device="cuda")
                p1a.attn_decode_rows(q[t:t + 1], pool.devkv.with_rows(rt[t:t + 1]), one, 1, pos[t:t + 1], Hq, 1 / 16, gate=gate[t:t + 1])
                s.synchronize()
                assert torch.equal(one[0], out_g[t]), (back, t)


def test_demoted_cache_on_a_fresh_stream_gets_the_scratch_it_needs(p1a):
    """a cache the MFMA kernel cannot take (pages of 4 positions) goes to the generic kernel, which leaves four times the
    partials per split stream; on a stream the library has not seen, after a release, the buffers it allocates must hold
    them (they are sized from the call's own need as well as from the head shape's footprint), and a negative row
    position reads no stream at all"""
    Hq, Hkv, D, psh, T = 4, 4, 256, 2, 9
    n = 300
    p1a.lib().p1a_release()
    pool = Pool(p1a, O.KV_Q4_0, Hq, Hkv, D, psh, [n], seed=131)
    c = pool.dev_seq(0)
    need = p1a.decode_scratch_bytes(c.struct(), Hq, T, 1)
    assert need <= p1a.decode_footprint_bytes(Hq, Hkv, D)
    q, _, _, gate = I.qkv(132, 1, T, Hq, Hkv, D)
    ref = O.attn_rows(pool.host_seq(0), q, (n - T + np.arange(T)).astype(np.int32), Hq, 1 / 16, gate=gate)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        out = torch.zeros((T, Hq, D), device="cuda")
        guard = torch.full((1 << 22,), 7.0, device="cuda")          # allocated right behind: must stay as it is
        p1a.attn_decode(dev(q), c, out, T, n - T, Hq, 1 / 16, gate=dev(gate))
        s.synchronize()
    check(out.cpu().numpy(), ref, "generic kernel on a fresh stream")
    assert bool((guard == 7.0).all())
