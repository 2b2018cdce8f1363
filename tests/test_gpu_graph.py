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
