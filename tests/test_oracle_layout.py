"""Pins the oracle's cache layout and paged addressing against an independent numpy restatement of the byte
formulas in the reference (src/fast/attn.cuh:1-32, src/fast/kv_q8.cuh:1-5) and its element reader
(tests/fast_attn_test.cu:34-44)."""
import ctypes

import numpy as np
import pytest

import _oracle as O
import _inputs as I

TYPES = [O.KV_F16, O.KV_Q8_0, O.KV_Q4_0]


def np_row(kv_type, x):
    """x [Hkv][D] f32 -> bytes of one cache row, assembled by hand from block quantizer outputs."""
    Hkv, D = x.shape
    out = []
    for h in range(Hkv):
        if kv_type == O.KV_F16:
            out.append(x[h].astype(np.float16).view(np.uint8))
        elif kv_type == O.KV_Q8_0:
            d, q = O.quant_q8_0(x[h].reshape(-1, 32))
            out.append(d.view(np.uint8))            # D/32 scales first
            out.append(q.reshape(-1).view(np.uint8))  # then D codes
        else:
            out.append(O.quant_q4_0(x[h].reshape(-1, 32)).reshape(-1))
    return np.concatenate(out)


def np_read(kv_type, row, Hkv, D, hk, d):
    """one element, the way the reference's test reads it"""
    if kv_type == O.KV_F16:
        return np.float32(row.view(np.float16)[hk * D + d])
    if kv_type == O.KV_Q8_0:
        hb = D // 32 * 34
        h = row[hk * hb:(hk + 1) * hb]
        return np.float32(h[:D // 32 * 2].view(np.float16)[d >> 5]) * np.float32(h[D // 32 * 2:].view(np.int8)[d])
    b = row[hk * (D // 32 * 18) + (d >> 5) * 18:][:18]
    sc = np.float32(b[:2].view(np.float16)[0])
    i = d & 31
    by = int(b[2 + (i & 15)])
    return np.float32((by & 15 if i < 16 else by >> 4) - 8) * sc


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("Hkv,D", [(4, 256), (1, 64), (2, 128)])
def test_row_bytes_and_layout(kv_type, Hkv, D):
    want = {O.KV_F16: Hkv * D * 2, O.KV_Q8_0: Hkv * (D // 32) * 34, O.KV_Q4_0: Hkv * (D // 32) * 18}[kv_type]
    assert O.row_bytes(kv_type, Hkv, D) == want
    g = I.rng(3)
    k = I.normal(g, (5, Hkv, D))
    v = I.normal(g, (5, Hkv, D))
    c = O.HostKV.contiguous(kv_type, 8, Hkv, D)
    O.kv_append_rows(c, k, v, np.array([2, 3, 4, 5, 6]))
    rb = want
    assert not c.k[:2 * rb].any() and not c.k[7 * rb:].any()
    for t in range(5):
        assert np.array_equal(c.k[(2 + t) * rb:(3 + t) * rb], np_row(kv_type, k[t]))
        assert np.array_equal(c.v[(2 + t) * rb:(3 + t) * rb], np_row(kv_type, v[t]))
    for hk, d in [(0, 0), (Hkv - 1, D - 1), (0, 17), (Hkv - 1, 33 % D)]:
        got = O.kv_read_head(c, 1, 0, 4, hk)[d]
        assert got == np_read(kv_type, c.v[4 * rb:5 * rb], Hkv, D, hk, d)


@pytest.mark.parametrize("kv_type", TYPES)
def test_paged_equals_contiguous(kv_type):
    Hkv, D, psh, NP, MAXP, NLAY = 2, 64, 4, 24, 10, 3
    ps = 1 << psh
    rb = O.row_bytes(kv_type, Hkv, D)
    g = I.rng(11)
    lens = [37, 150, 16]
    perm = g.permutation(NP).astype(np.int32)
    tabs = np.full(3 * MAXP, -1, np.int32)
    used = 0
    for s, n in enumerate(lens):
        for p in range((n + ps - 1) // ps):
            tabs[s * MAXP + p] = perm[used]
            used += 1
    paged = O.HostKV.paged(kv_type, Hkv, D, psh, NP, tabs, MAXP, n_layers=NLAY, layer=1)
    assert paged.pstride == NLAY * 2 * ps * rb
    for s, n in enumerate(lens):
        k = I.normal(g, (n, Hkv, D))
        v = I.normal(g, (n, Hkv, D))
        cont = O.HostKV.contiguous(kv_type, n, Hkv, D)
        O.kv_append_rows(cont, k, v, np.arange(n))
        pv = paged.view(rtab=np.full(n, s * MAXP, np.int32))
        O.kv_append_rows(pv, k, v, np.arange(n))
        st = pv.struct()
        for p in range(n):
            # the formula of src/fast/attn.cuh:23-27 by hand
            o = int(tabs[s * MAXP + (p >> psh)]) * paged.pstride + (p & (ps - 1)) * rb
            assert O.lib().orc_kv_off(ctypes.byref(st), 0, p) == o
            ko = 1 * 2 * ps * rb + o
            assert np.array_equal(paged.pool[ko:ko + rb], cont.k[p * rb:(p + 1) * rb])
            assert np.array_equal(paged.pool[ko + ps * rb:ko + ps * rb + rb], cont.v[p * rb:(p + 1) * rb])
    # other layers of the pool untouched
    view = paged.pool.reshape(NP, NLAY, 2 * ps * rb)
    assert not view[:, 0].any() and not view[:, 2].any()
