"""Seeded sweeps over the shapes the C ABI accepts, each case against the CPU oracle (tolerance of the path: max-abs
2e-3 - times max|ref| where a context of a few keys makes that exceed 1 - and rel-L2 1e-3): KV type, head counts, head dimension, page size, number of sequences, rows per sequence, lengths,
gate on / off. The fixed-shape tests cover the engine's configurations; these look for a combination nobody thought of
(ragged last pages, sequences shorter than a tile, a single key, page sizes below the MFMA kernels' minimum)."""
import numpy as np
import pytest
import torch

import _inputs as I
import _oracle as O
from _gpu import Pool, check, dev

pytestmark = pytest.mark.gpu
TYPES = [O.KV_F16, O.KV_Q8_0, O.KV_Q4_0]


def draw_shape(g):
    kv_type = TYPES[int(g.integers(3))]
    D = int(g.choice([64, 128, 256], p=[0.2, 0.2, 0.6]))
    Hkv = int(g.choice([1, 2, 3, 4]))
    gqa = int(g.choice([1, 2, 4, 6, 8]))
    psh = int(g.choice([2, 4, 5, 6, 8]))
    return kv_type, D, Hkv, gqa, psh


@pytest.mark.parametrize("case", range(40))
def test_decode_random_case(p1a, case):
    g = I.rng(9000 + case)
    kv_type, D, Hkv, gqa, psh = draw_shape(g)
    Hq = Hkv * gqa
    nseq = int(g.integers(1, 5))
    rps = int(g.integers(1, 5))
    # lengths from one key up; every few cases a sequence that ends exactly on a page or tile boundary
    lens = [max(rps, int(np.exp(g.uniform(0, np.log(2500))))) for _ in range(nseq)]
    if case % 3 == 0:
        lens[0] = max(rps, (lens[0] >> psh) << psh)
    if case % 5 == 0:
        lens[-1] = max(rps, (lens[-1] // 16) * 16 + 1)
    use_gate = bool(g.integers(2))
    scale = float(g.choice([1 / 16, 0.1, 0.125]))
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, lens, seed=9100 + case)
    T = nseq * rps
    q, _, _, gate = I.qkv(9200 + case, 1, T, Hq, Hkv, D)
    pos = np.array([lens[s] - rps + t for s in range(nseq) for t in range(rps)], np.int32)
    scattered = case % 2 == 1
    if scattered:   # the rows of a group at any positions of their sequence, in any order (they still share one KV read)
        pos = np.array([int(g.integers(0, lens[s])) for s in range(nseq) for _ in range(rps)], np.int32)
    rtab = np.array([s * pool.maxp for s in range(nseq) for _ in range(rps)], np.int32)
    ref = O.attn_rows(pool.host.view(rtab=rtab), q, pos, Hq, scale, gate=gate if use_gate else None)
    out = torch.full((T, Hq, D), float("nan"), device="cuda")
    what = f"decode case {case}: type {kv_type} {Hq}/{Hkv}/{D} psh {psh} lens {lens} rows/seq {rps} gate {use_gate} pos {pos.tolist()}"
    print(what, flush=True)
    p1a.attn_decode_rows(dev(q), pool.devkv.with_rows(dev(rtab)), out, T, dev(pos), Hq, scale,
                         gate=dev(gate) if use_gate else None, rows_per_seq=rps)
    torch.cuda.synchronize()
    check(out.cpu().numpy(), ref, what)
    if case % 4 == 0:   # the same call with the a16 activation buffer of its (gated) rows: same output bits, the oracle's buffer
        out2 = torch.full((T, Hq, D), float("nan"), device="cuda")
        qb = torch.zeros(p1a.a16_bytes(T, Hq * D) // 2, dtype=torch.int16, device="cuda")
        p1a.attn_decode_rows(dev(q), pool.devkv.with_rows(dev(rtab)), out2, T, dev(pos), Hq, scale,
                             gate=dev(gate) if use_gate else None, rows_per_seq=rps, qbuf=qb)
        torch.cuda.synchronize()
        assert torch.equal(out, out2), what
        assert np.array_equal(qb.cpu().numpy().view(np.uint16), O.a16_quant(out2.cpu().numpy().reshape(T, Hq * D))), what
    if scattered:   # every row alone at its position: the same bits as in the batch
        for t in range(min(T, 6)):
            one = torch.full((1, Hq, D), float("nan"), device="cuda")
            p1a.attn_decode(dev(q[t:t + 1]), pool.dev_seq(t // rps), one, 1, int(pos[t]), Hq, scale, gate=dev(gate[t:t + 1]) if use_gate else None)
            torch.cuda.synchronize()
            assert torch.equal(one[0], out[t]), (what, t)
        return
    # the first sequence alone, through the one-sequence entry (host position): the same bits as its rows in the batch
    one = torch.full((rps, Hq, D), float("nan"), device="cuda")
    p1a.attn_decode(dev(q[:rps]), pool.dev_seq(0), one, rps, lens[0] - rps, Hq, scale, gate=dev(gate[:rps]) if use_gate else None)
    torch.cuda.synchronize()
    assert torch.equal(one, out[:rps]), what


@pytest.mark.parametrize("case", range(24))
def test_prefill_random_case(p1a, case):
    g = I.rng(9500 + case)
    kv_type, D, Hkv, gqa, psh = draw_shape(g)
    Hq = Hkv * gqa
    p0 = int(g.choice([0, int(g.integers(1, 1500))]))
    T = int(np.exp(g.uniform(0, np.log(700)))) if case % 3 else int(g.integers(100, 600))
    if case % 4 == 0:
        T = max(1, (T // 128) * 128)                          # whole token blocks
    use_gate = bool(g.integers(2))
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [p0 + T, 40], seed=9600 + case)
    q, _, _, gate = I.qkv(9700 + case, 1, T, Hq, Hkv, D, f16_inputs=True)
    pos = p0 + np.arange(T, dtype=np.int32)
    ref = O.attn_rows(pool.host_seq(0), q, pos, Hq, 0.1, gate=gate if use_gate else None)
    what = f"prefill case {case}: type {kv_type} {Hq}/{Hkv}/{D} psh {psh} p0 {p0} T {T} gate {use_gate}"
    print(what, flush=True)
    c = pool.dev_seq(0)
    out = torch.full((T, Hq, D), float("nan"), device="cuda")
    p1a.attn_prefill(dev(q), c, out, T, p0, Hq, 0.1, gate=dev(gate) if use_gate else None)
    torch.cuda.synchronize()
    check(out.cpu().numpy(), ref, what)
    # with caller scratch (a quantized cache converted once per call): the same bits
    nb = p1a.prefill_scratch_bytes(T, p0, Hq, Hkv, D)
    if nb:
        scr = torch.empty(nb, dtype=torch.uint8, device="cuda")
        out2 = torch.full((T, Hq, D), float("nan"), device="cuda")
        p1a.attn_prefill(dev(q), c, out2, T, p0, Hq, 0.1, gate=dev(gate) if use_gate else None, scratch=scr)
        torch.cuda.synchronize()
        assert torch.equal(out, out2), what


@pytest.mark.parametrize("case", range(16))
def test_append_random_case(p1a, case):
    """quantize-on-append into a paged pool in chunks of random size through the three position forms (host p0, device
    p0, one position per row): every byte of the pool as the oracle writes it. Magnitudes from 1e-7 (scales that are f16
    subnormals or underflow to zero) to 3e4 (close to the largest f16 scale), zero blocks and rows sprinkled in."""
    g = I.rng(9800 + case)
    kv_type = TYPES[int(g.integers(3))]
    Hkv = int(g.choice([1, 2, 3, 4]))
    D = int(g.choice([32, 64, 96, 128, 256]))
    psh = int(g.choice([0, 2, 4, 5, 8]))
    lens = [int(np.exp(g.uniform(0, np.log(900)))) if i else int(g.integers(100, 700)) for i in range(int(g.integers(1, 4)))]
    pool = Pool(p1a, kv_type, Hkv, Hkv, D, psh, lens, seed=9900 + case, n_layers=int(g.integers(1, 4)), layer=0, fill="none")
    what = f"append case {case}: type {kv_type} Hkv {Hkv} D {D} psh {psh} lens {lens}"
    print(what, flush=True)
    p0d = dev(np.array([0], np.int32))
    for s, n in enumerate(lens):
        mag = np.exp(g.uniform(np.log(1e-7), np.log(3e4), size=(n, Hkv, D // 32, 1))).astype(np.float32)
        k = (I.normal(g, (n, Hkv, D // 32, 32)) * mag).reshape(n, Hkv, D)
        v = (I.normal(g, (n, Hkv, D // 32, 32)) * mag[::-1]).reshape(n, Hkv, D)
        k[g.integers(n)] = 0.0
        v[g.integers(n), g.integers(Hkv), :32] = 0.0
        O.kv_append_rows(pool.host.view(rtab=np.full(n, s * pool.maxp, np.int32)), k, v, np.arange(n))
        dk, dv, c = dev(k), dev(v), pool.dev_seq(s)
        a = 0
        while a < n:
            m = min(n - a, int(g.integers(1, 200)))
            form = int(g.integers(3))
            if form == 0:
                p1a.kv_append(c, dk[a:], dv[a:], a, m)
            elif form == 1:
                p0d.fill_(a)
                p1a.kv_append_dev(c, dk[a:], dv[a:], p0d, m)
            else:   # rows in a shuffled order, through the row table
                order = g.permutation(m)
                cr = pool.devkv.with_rows(dev(np.full(m, s * pool.maxp, np.int32)))
                idx = torch.from_numpy(a + order).cuda()
                p1a.kv_append_rows(cr, dk[idx].contiguous(), dv[idx].contiguous(), dev((a + order).astype(np.int32)), m)
            a += m
    torch.cuda.synchronize()
    assert np.array_equal(pool.dpool.cpu().numpy(), pool.host.pool), what


@pytest.mark.parametrize("case", range(16))
def test_prep_random_case(p1a, case):
    """attn_prep (q | gate split, per-head RMS norm * weight, NEOX rotation of the first n_rot dims, quantizing KV write)
    over random shapes, rotary widths, row strides, positions up to a million, host-position and device-position mode, with
    and without interleaved M-RoPE: gate, q, V bytes and K bytes all bit for bit the oracle's"""
    g = I.rng(9300 + case)
    kv_type = TYPES[int(g.integers(3))]
    D = int(g.choice([64, 128, 256]))
    Hkv = int(g.choice([1, 2, 4]))
    Hq = Hkv * int(g.choice([1, 2, 6]))
    n_rot = int(g.choice([0, 8, 32, 64, D]))
    T = int(g.integers(1, 24))
    base = float(g.choice([1e4, 1e6, 1e7]))
    dev_pos = bool(g.integers(2))
    far = int(g.choice([0, 1000, 250000, 1000000]))            # rotary positions far from the cache rows (M-RoPE style offsets aside)
    n_ctx = 64
    rows = g.permutation(n_ctx)[:T].astype(np.int32) if dev_pos else (int(g.integers(0, n_ctx - T)) + np.arange(T)).astype(np.int32)
    qg = I.normal(g, (T, Hq, 2 * D)); k = I.normal(g, (T, Hkv, D)) * 1.3; v = I.normal(g, (T, Hkv, D))
    qn = (1.0 + 0.1 * I.normal(g, (D,))).astype(np.float32); kn = (1.0 + 0.1 * I.normal(g, (D,))).astype(np.float32)
    use_mr = bool(g.integers(2)) and n_rot >= 8
    mr_host = mr_dev = None
    if use_mr:
        npairs = n_rot // 2
        s0 = int(g.integers(0, npairs + 1)); s1 = int(g.integers(0, npairs - s0 + 1)); s2 = int(g.integers(0, npairs - s0 - s1 + 1))
        sect = npairs if g.integers(2) else s0 + s1 + s2 + int(g.integers(0, 3))
        sect = max(sect, 1)
        stride = T + int(g.integers(0, 4))
        mp = np.zeros((3, stride), np.int32)
        mp[:, :T] = far + g.integers(0, 5000, size=(3, T))
        mr_host, mr_dev = (mp, (s0, s1, s2), sect), (dev(mp), stride, (s0, s1, s2), sect)
    pos = rows if (dev_pos or not far) and not use_mr else rows          # cache rows = rotary positions unless M-RoPE gives its own
    ldq, ldk, ldv = Hq * 2 * D + 4 * int(g.integers(0, 3)), Hkv * D + 4 * int(g.integers(0, 3)), Hkv * D + 4 * int(g.integers(0, 3))
    def strided(a, ld):
        buf = np.full((T, ld), 3.0, np.float32)
        buf[:, : a[0].size] = a.reshape(T, -1)
        return buf
    what = f"prep case {case}: type {kv_type} {Hq}/{Hkv}/{D} n_rot {n_rot} T {T} base {base:g} dev_pos {dev_pos} mrope {mr_host[1:] if use_mr else None}"
    print(what, flush=True)
    host = O.HostKV.contiguous(kv_type, n_ctx, Hkv, D)
    p0 = -1 if dev_pos else int(rows[0])
    q_ref, gate_ref = O.attn_prep(host, qg, k, v, qn, kn, pos, p0, Hq, n_rot, base, 1e-6, mrope=mr_host)
    c = p1a.KVCache.contiguous(kv_type, n_ctx, Hkv, D)
    q = torch.zeros((T, Hq, D), device="cuda"); gate = torch.zeros((T, Hq * D), device="cuda")
    p1a.attn_prep(dev(strided(qg, ldq)), dev(strided(k, ldk)), dev(strided(v, ldv)), dev(qn), dev(kn), dev(pos), q, gate, c, p0, T, Hq,
                  n_rot, base, 1e-6, ldq=ldq, ldk=ldk, ldv=ldv, mrope=mr_dev)
    torch.cuda.synchronize()
    assert np.array_equal(gate.cpu().numpy(), gate_ref), what
    assert np.array_equal(q.cpu().numpy().view(np.int32), q_ref.view(np.int32)), what
    assert np.array_equal(c._keep[1].cpu().numpy(), host.v), what
    assert np.array_equal(c._keep[0].cpu().numpy(), host.k), what
