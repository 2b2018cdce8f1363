"""attn_prep on the GPU (through the C ABI) vs the oracle: gate, q and the KV bytes (K codes included) must match bit for
bit - both sides keep one operation order and spell out power, cosine and sine in IEEE double operations instead of
calling a math library; then the prepared cache and q drive a decode."""
import numpy as np
import pytest
import torch

import _inputs as I
import _oracle as O
from _gpu import check, dev

pytestmark = pytest.mark.gpu
TYPES = [O.KV_F16, O.KV_Q8_0, O.KV_Q4_0]


def make(seed, T, Hq, Hkv, D):
    g = I.rng(seed)
    qg = I.normal(g, (T, Hq, 2 * D))
    k = I.normal(g, (T, Hkv, D)) * 1.3
    v = I.normal(g, (T, Hkv, D))
    qn = (1.0 + 0.1 * I.normal(g, (D,))).astype(np.float32)
    kn = (1.0 + 0.1 * I.normal(g, (D,))).astype(np.float32)
    return qg, k, v, qn, kn


def ulp_diff(a, b):
    ia = a.view(np.int32).astype(np.int64)
    ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7fffffff), ia)
    ib = np.where(ib < 0, -(ib & 0x7fffffff), ib)
    return np.abs(ia - ib)


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("Hq,Hkv,D,n_rot", [(24, 4, 256, 64), (4, 1, 64, 64), (8, 2, 128, 32)])
def test_host_position_contiguous(p1a, kv_type, Hq, Hkv, D, n_rot):
    T, p0, n_ctx, base, eps = 7, 9, 32, 1e7, 1e-6
    qg, k, v, qn, kn = make(D + n_rot, T, Hq, Hkv, D)
    pos = (p0 + np.arange(T)).astype(np.int32)
    host = O.HostKV.contiguous(kv_type, n_ctx, Hkv, D)
    q_ref, gate_ref = O.attn_prep(host, qg, k, v, qn, kn, pos, p0, Hq, n_rot, base, eps)
    c = p1a.KVCache.contiguous(kv_type, n_ctx, Hkv, D)
    q = torch.zeros((T, Hq, D), device="cuda")
    gate = torch.zeros((T, Hq * D), device="cuda")
    p1a.attn_prep(dev(qg), dev(k), dev(v), dev(qn), dev(kn), dev(pos), q, gate, c, p0, T, Hq, n_rot, base, eps)
    torch.cuda.synchronize()
    assert np.array_equal(gate.cpu().numpy(), gate_ref)
    assert np.array_equal(q.cpu().numpy().view(np.int32), q_ref.view(np.int32))
    assert np.array_equal(c._keep[1].cpu().numpy(), host.v)
    assert np.array_equal(c._keep[0].cpu().numpy(), host.k)


@pytest.mark.parametrize("kv_type", TYPES)
def test_device_positions_paged_rows_then_decode(p1a, kv_type):
    """rows of four sequences, each at its own position through its own page table (p0 < 0), strided inputs; then the
    prepared q / gate / cache drive attn_decode_rows and must give the oracle's attention"""
    Hq, Hkv, D, n_rot, base, eps, psh = 12, 2, 256, 64, 1e7, 1e-6, 4
    lens = [40, 17, 63, 5]
    T = len(lens)
    max_pages, n_pages = 5, 24
    g = I.rng(77)
    table = g.permutation(n_pages)[: T * max_pages].astype(np.int32)
    rtab = (np.arange(T) * max_pages).astype(np.int32)
    hostp = O.HostKV.paged(kv_type, Hkv, D, psh, n_pages, table, max_pages)
    host = hostp.view(rtab=rtab)
    dtab, drt = dev(table), dev(rtab)
    dc = p1a.KVCache.paged(kv_type, Hkv, D, psh, n_pages, dtab, max_pages).with_rows(drt)
    # history: every sequence gets lens[s] - 1 earlier rows through the plain append (same bytes on both sides)
    for s, n in enumerate(lens):
        if n > 1:
            _, kh, vh, _ = I.qkv(900 + s, n - 1, 1, Hq, Hkv, D)
            O.kv_append_rows(host.view(rtab=np.full(n - 1, s * max_pages, np.int32)), kh, vh, np.arange(n - 1))
            p1a.kv_append(dc.slot(s, max_pages), dev(kh), dev(vh), 0, n - 1)
    qg, k, v, qn, kn = make(5, T, Hq, Hkv, D)
    pos = np.array([n - 1 for n in lens], np.int32)
    # strided inputs: rows carry padding, as slices of a concatenated projection output do
    ldq, ldk, ldv = Hq * 2 * D + 8, Hkv * D + 4, Hkv * D + 12
    def strided(a, ld):
        buf = np.full((T, ld), 7.0, np.float32)
        buf[:, : a[0].size] = a.reshape(T, -1)
        return buf
    q_ref, gate_ref = O.attn_prep(host, qg, k, v, qn, kn, pos, -1, Hq, n_rot, base, eps)
    q = torch.zeros((T, Hq, D), device="cuda")
    gate = torch.zeros((T, Hq * D), device="cuda")
    dpos = dev(pos)
    p1a.attn_prep(dev(strided(qg, ldq)), dev(strided(k, ldk)), dev(strided(v, ldv)), dev(qn), dev(kn), dpos, q, gate, dc, -1, T, Hq,
                  n_rot, base, eps, ldq=ldq, ldk=ldk, ldv=ldv)
    torch.cuda.synchronize()
    assert np.array_equal(gate.cpu().numpy(), gate_ref)
    assert np.array_equal(q.cpu().numpy().view(np.int32), q_ref.view(np.int32))
    assert np.array_equal(dc._keep[0].cpu().numpy(), hostp.pool)          # every byte of the pool: history rows and the prepared ones
    out = torch.zeros((T, Hq, D), device="cuda")
    p1a.attn_decode_rows(q, dc, out, T, dpos, Hq, 1 / 16, gate=gate)
    torch.cuda.synchronize()
    ref = O.attn_rows(host, q_ref, pos, Hq, 1 / 16, gate=gate_ref)
    check(out.cpu().numpy(), ref, f"prep -> decode_rows type {kv_type}")


def test_refusals(p1a):
    c = p1a.KVCache.contiguous(O.KV_Q8_0, 8, 2, 256)
    z = torch.zeros(4 * 2 * 256 * 2, device="cuda")
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    with pytest.raises(p1a.P1AError):       # n_rot not a multiple of 8
        p1a.attn_prep(z, z, z, None, None, pos, z, z, c, 0, 1, 4, 12, 1e7, 1e-6)
    with pytest.raises(p1a.P1AError):       # no positions
        p1a.attn_prep(z, z, z, None, None, None, z, z, c, 0, 1, 4, 64, 1e7, 1e-6)
    with pytest.raises(p1a.P1AError):       # row stride shorter than a row
        p1a.attn_prep(z, z, z, None, None, pos, z, z, c, 0, 1, 4, 64, 1e7, 1e-6, ldq=64)
    torch.cuda.synchronize()


def test_ew_quant_sigmoid_and_silu(p1a):
    """gate + a16 emit (src/fast/fused.cu:478-496): y within fp32 rounding of the oracle, the a16 bytes exactly the oracle's
    quantization of the y the GPU wrote; strided a / b; y aliasing a"""
    T, n = 3, 6144
    g = I.rng(41)
    a = I.normal(g, (T, n)) * 2.0
    b = I.normal(g, (T, n))
    a[1, 64:96] = 0.0                                           # an all-zero group
    lda, ldb = n + 8, n + 32
    ap = np.zeros((T, lda), np.float32); ap[:, :n] = a
    bp = np.zeros((T, ldb), np.float32); bp[:, :n] = b
    for op in (1, 0):
        y = torch.zeros((T, n), device="cuda")
        qb = torch.zeros(p1a.a16_bytes(T, n) // 2, dtype=torch.int16, device="cuda")
        p1a.ew_quant(op, dev(ap), dev(bp), y, qb, T, n, lda=lda, ldb=ldb)
        torch.cuda.synchronize()
        yh = y.cpu().numpy()
        if op == 1:
            ref = a.astype(np.float64) / (1.0 + np.exp(-b.astype(np.float64)))
        else:
            ref = a.astype(np.float64) / (1.0 + np.exp(-a.astype(np.float64))) * b.astype(np.float64)
        assert np.max(np.abs(yh - ref)) <= 4e-7 * max(1.0, np.abs(ref).max())
        assert np.array_equal(qb.cpu().numpy().view(np.uint16), O.a16_quant(yh)), op
    # in place: y aliases a (dense rows)
    ya = dev(a)
    qb = torch.zeros(p1a.a16_bytes(T, n) // 2, dtype=torch.int16, device="cuda")
    p1a.ew_quant(1, ya, dev(b), ya, qb, T, n)
    torch.cuda.synchronize()
    assert np.array_equal(qb.cpu().numpy().view(np.uint16), O.a16_quant(ya.cpu().numpy()))
    with pytest.raises(p1a.P1AError):
        p1a.ew_quant(1, ya, dev(b), ya, qb, T, n - 4)          # n % 32 != 0
    torch.cuda.synchronize()


@pytest.mark.parametrize("kv_type", [O.KV_Q8_0, O.KV_F16])
def test_decode_emits_a16(p1a, kv_type):
    """the decode call with a qbuf: same output bits as without, and qbuf = a16(gated output)"""
    from _gpu import Pool
    Hq, Hkv, D, psh = 24, 4, 256, 6
    lens = [300, 77]
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, lens, seed=13)
    T = 3
    q, _, _, gate = I.qkv(61, 1, T, Hq, Hkv, D)
    pos = np.array([299, 76, 150], np.int32)
    rt = np.array([0, pool.maxp, 0], np.int32)
    c = pool.devkv.with_rows(dev(rt))
    o1 = torch.zeros((T, Hq, D), device="cuda"); o2 = torch.zeros((T, Hq, D), device="cuda")
    qb = torch.zeros(p1a.a16_bytes(T, Hq * D) // 2, dtype=torch.int16, device="cuda")
    dq, dg, dp = dev(q), dev(gate), dev(pos)
    p1a.attn_decode_rows(dq, c, o1, T, dp, Hq, 1 / 16, gate=dg)
    p1a.attn_decode_rows(dq, c, o2, T, dp, Hq, 1 / 16, gate=dg, qbuf=qb)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2)
    assert np.array_equal(qb.cpu().numpy().view(np.uint16), O.a16_quant(o2.cpu().numpy().reshape(T, Hq * D)))


@pytest.mark.parametrize("kv_type", TYPES)
def test_mrope_positions(p1a, kv_type):
    """interleaved M-RoPE (src/fast/mrope.cuh): image rows with their own t / h / w, the same bars as the plain rotation;
    and text rows (t = h = w = p) give the plain call's bits."""
    Hq, Hkv, D, n_rot, T, n_ctx, base, eps = 24, 4, 256, 64, 9, 64, 1e7, 1e-6
    qg, k, v, qn, kn = make(77, T, Hq, Hkv, D)
    pos = (20 + np.arange(T)).astype(np.int32)                            # cache rows
    P = 1000                                                               # a 3 x 3 image placed at P: t = P, h = P + i / 3, w = P + i % 3
    mp = np.zeros((3, T + 3), np.int32)                                   # (a stride larger than T)
    mp[0, :T], mp[1, :T], mp[2, :T] = P, P + np.arange(T) // 3, P + np.arange(T) % 3
    host = O.HostKV.contiguous(kv_type, n_ctx, Hkv, D)
    q_ref, gate_ref = O.attn_prep(host, qg, k, v, qn, kn, pos, -1, Hq, n_rot, base, eps, mrope=(mp, (11, 11, 10), 32))
    c = p1a.KVCache.contiguous(kv_type, n_ctx, Hkv, D)
    q = torch.zeros((T, Hq, D), device="cuda")
    gate = torch.zeros((T, Hq * D), device="cuda")
    p1a.attn_prep(dev(qg), dev(k), dev(v), dev(qn), dev(kn), dev(pos), q, gate, c, -1, T, Hq, n_rot, base, eps,
                  mrope=(dev(mp), T + 3, (11, 11, 10), 32))
    torch.cuda.synchronize()
    assert np.array_equal(gate.cpu().numpy(), gate_ref)
    assert np.array_equal(q.cpu().numpy().view(np.int32), q_ref.view(np.int32))
    assert np.array_equal(c._keep[1].cpu().numpy(), host.v)
    assert np.array_equal(c._keep[0].cpu().numpy(), host.k)
    # text rows
    c1, c2 = p1a.KVCache.contiguous(kv_type, n_ctx, Hkv, D), p1a.KVCache.contiguous(kv_type, n_ctx, Hkv, D)
    q1, q2 = torch.zeros_like(q), torch.zeros_like(q)
    p1a.attn_prep(dev(qg), dev(k), dev(v), dev(qn), dev(kn), dev(pos), q1, gate, c1, -1, T, Hq, n_rot, base, eps)
    p1a.attn_prep(dev(qg), dev(k), dev(v), dev(qn), dev(kn), dev(pos), q2, gate, c2, -1, T, Hq, n_rot, base, eps,
                  mrope=(dev(np.stack([pos, pos, pos])), T, (11, 11, 10), 32))
    torch.cuda.synchronize()
    assert torch.equal(q1, q2) and torch.equal(c1._keep[0], c2._keep[0]) and torch.equal(c1._keep[1], c2._keep[1])
    with pytest.raises(p1a.P1AError, match="M-RoPE"):
        p1a.attn_prep(dev(qg), dev(k), dev(v), dev(qn), dev(kn), dev(pos), q2, gate, c2, -1, T, Hq, n_rot, base, eps,
                      mrope=(dev(mp), T + 3, (11, 11, 10), 0))
