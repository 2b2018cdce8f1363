"""Pins the oracle's attention (a restatement of src/kernels.cu:143-166 of the reference) against textbook
softmax(QK^T)V in numpy float64 on the dequantized cache, and against closed forms."""
import numpy as np
import pytest

import _oracle as O
import _inputs as I

TYPES = [O.KV_F16, O.KV_Q8_0, O.KV_Q4_0]


def dequant_all(c, n, t=0):
    K = np.stack([np.stack([O.kv_read_head(c, 0, t, p, h) for h in range(c.Hkv)]) for p in range(n)])
    V = np.stack([np.stack([O.kv_read_head(c, 1, t, p, h) for h in range(c.Hkv)]) for p in range(n)])
    return K.astype(np.float64), V.astype(np.float64)


def np_attn(q, K, V, pos, Hq, scale):
    T, _, D = q.shape
    Hkv = K.shape[1]
    out = np.zeros((T, Hq, D))
    for t in range(T):
        n = pos[t] + 1
        for h in range(Hq):
            hk = h // (Hq // Hkv)
            s = (K[:n, hk] @ q[t, h].astype(np.float64)) * scale
            p = np.exp(s - s.max())
            out[t, h] = (p[:, None] * V[:n, hk]).sum(0) / p.sum()
    return out


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("Hq,Hkv,D,n", [(24, 4, 256, 300), (4, 1, 64, 512), (8, 2, 128, 77)])
def test_against_numpy_float64(kv_type, Hq, Hkv, D, n):
    T = 3
    q, k, v, gate = I.qkv(5, n, T, Hq, Hkv, D)
    c = O.HostKV.contiguous(kv_type, n, Hkv, D)
    O.kv_append_rows(c, k, v, np.arange(n))
    pos = np.array([n - 3, n - 2, n - 1], np.int32)
    scale = 1.0 / np.sqrt(D)
    K, V = dequant_all(c, n)
    ref = np_attn(q, K, V, pos, Hq, scale)
    got32 = O.attn_rows(c, q, pos, Hq, scale)
    got64 = O.attn_rows(c, q, pos, Hq, scale, f64=True)
    assert np.max(np.abs(got64 - ref)) < 2e-7 * max(1.0, np.abs(ref).max())
    ma, rl = I.errors(got32, ref)
    assert ma < 5e-6 and rl < 5e-6
    # gate: sigmoid in float64
    gg = O.attn_rows(c, q, pos, Hq, scale, gate=gate)
    refg = ref / (1.0 + np.exp(-gate.reshape(T, Hq, D).astype(np.float64)))
    assert I.errors(gg, refg)[1] < 5e-6


def test_closed_forms():
    Hq, Hkv, D = 6, 1, 256
    g = I.rng(9)
    q = I.normal(g, (1, Hq, D))
    k = I.normal(g, (40, Hkv, D))
    v = I.normal(g, (40, Hkv, D))
    for kv_type in TYPES:
        c = O.HostKV.contiguous(kv_type, 40, Hkv, D)
        O.kv_append_rows(c, k, v, np.arange(40))
        # n = 1: the output is the dequantized V row exactly
        out = O.attn_rows(c, q, np.array([0]), Hq, 0.0625)
        for h in range(Hq):
            assert np.array_equal(out[0, h], O.kv_read_head(c, 1, 0, 0, 0))
        # causality: bytes past pos do not matter
        a = O.attn_rows(c, q, np.array([17]), Hq, 0.0625)
        rb = O.row_bytes(kv_type, Hkv, D)
        c.k[18 * rb:] = 0xA5
        c.v[18 * rb:] = 0x5A
        b = O.attn_rows(c, q, np.array([17]), Hq, 0.0625)
        assert np.array_equal(a, b)
    # all V rows equal -> that row (to rounding); softmax shift invariance: adding a constant key offset along q
    c = O.HostKV.contiguous(O.KV_F16, 40, Hkv, D)
    v1 = np.repeat(v[:1], 40, 0)
    O.kv_append_rows(c, k, v1, np.arange(40))
    out = O.attn_rows(c, q, np.array([39]), Hq, 0.0625)
    assert np.max(np.abs(out[0, 0] - O.kv_read_head(c, 1, 0, 0, 0))) < 1e-6
    # one dominant logit: k_j = 50 * q / |q| for j = 7 -> out ~ V[7]
    k2 = k.copy() * 0.01
    k2[7, 0] = 50.0 * q[0, 0] / np.linalg.norm(q[0, 0])
    c = O.HostKV.contiguous(O.KV_F16, 40, Hkv, D)
    O.kv_append_rows(c, k2, v, np.arange(40))
    out = O.attn_rows(c, q, np.array([39]), Hq, 1.0)
    assert np.max(np.abs(out[0, 0] - O.kv_read_head(c, 1, 0, 7, 0))) < 1e-5


def test_gqa_head_map_and_gate():
    Hq, Hkv, D, n = 8, 2, 64, 20
    g = I.rng(4)
    q = I.normal(g, (1, Hq, D))
    k = I.normal(g, (n, Hkv, D))
    v = np.zeros((n, Hkv, D), np.float32)
    v[:, 0], v[:, 1] = 1.0, -2.0                      # head h must read kv head h // 4
    c = O.HostKV.contiguous(O.KV_F16, n, Hkv, D)
    O.kv_append_rows(c, k, v, np.arange(n))
    out = O.attn_rows(c, q, np.array([n - 1]), Hq, 0.125)
    assert np.allclose(out[0, :4], 1.0, atol=1e-6) and np.allclose(out[0, 4:], -2.0, atol=1e-6)
    z = np.zeros((1, Hq * D), np.float32)
    gated = O.attn_rows(c, q, np.array([n - 1]), Hq, 0.125, gate=z)
    assert np.array_equal(gated, out * np.float32(0.5))  # sigmoid(0) = 0.5 exactly
    x = np.ones(64, np.float32)
    gp, gm = x.copy(), x.copy()
    gv = I.normal(g, (64,))
    O.lib().orc_gate(gp.ctypes.data, gv.ctypes.data, 64)
    O.lib().orc_gate(gm.ctypes.data, (-gv).ctypes.data, 64)
    assert np.max(np.abs(gp + gm - 1.0)) < 2e-7        # sigma(g) + sigma(-g) = 1


def test_rows_equal_single_and_paged():
    kv_type, Hq, Hkv, D, psh, MAXP = O.KV_Q8_0, 12, 2, 256, 4, 8
    ps = 1 << psh
    g = I.rng(21)
    lens = [100, 40]
    NP = 20
    perm = g.permutation(NP).astype(np.int32)
    tabs = np.zeros(2 * MAXP, np.int32)
    tabs[:7] = perm[:7]
    tabs[MAXP:MAXP + 3] = perm[7:10]
    paged = O.HostKV.paged(kv_type, Hkv, D, psh, NP, tabs, MAXP)
    conts = []
    for s, n in enumerate(lens):
        k = I.normal(g, (n, Hkv, D))
        v = I.normal(g, (n, Hkv, D))
        cont = O.HostKV.contiguous(kv_type, n, Hkv, D)
        O.kv_append_rows(cont, k, v, np.arange(n))
        O.kv_append_rows(paged.view(rtab=np.full(n, s * MAXP, np.int32)), k, v, np.arange(n))
        conts.append(cont)
    q = I.normal(g, (3, Hq, D))
    rows = [(0, 99), (1, 39), (0, 15)]
    pos = np.array([p for _, p in rows], np.int32)
    rtab = np.array([s * MAXP for s, _ in rows], np.int32)
    multi = O.attn_rows(paged.view(rtab=rtab), q, pos, Hq, 0.0625)
    for t, (s, p) in enumerate(rows):
        single = O.attn_rows(conts[s], q[t:t + 1], np.array([p]), Hq, 0.0625)
        assert np.array_equal(multi[t], single[0])
