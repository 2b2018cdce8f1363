"""Pins the oracle's attn_prep (a restatement of src/fast/fused.cu:512-573 of the reference: q | gate split, per-head
RMS norm * weight, NEOX rope on the first n_rot dims, quantize-append) against numpy float64 and closed forms."""
import numpy as np
import pytest

import _oracle as O
import _inputs as I

TYPES = [O.KV_F16, O.KV_Q8_0, O.KV_Q4_0]


def np_norm_rope(x, w, n_rot, base, eps, pos):
    """float64 textbook: x * rsqrt(mean(x^2) + eps) * w, then rotate pairs (j, j + n_rot/2) by pos * base^(-2j/n_rot)"""
    x = x.astype(np.float64)
    y = x / np.sqrt((x * x).mean() + eps)
    if w is not None:
        y = y * w.astype(np.float64)
    half = n_rot // 2
    j = np.arange(half)
    th = pos * base ** (-2.0 * j / n_rot)
    c, s = np.cos(th), np.sin(th)
    x0, x1 = y[:half].copy(), y[half:n_rot].copy()
    y[:half] = x0 * c - x1 * s
    y[half:n_rot] = x0 * s + x1 * c
    return y


def make(seed, T, Hq, Hkv, D):
    g = I.rng(seed)
    qg = I.normal(g, (T, Hq, 2 * D))
    k = I.normal(g, (T, Hkv, D))
    v = I.normal(g, (T, Hkv, D))
    qn = (1.0 + 0.1 * I.normal(g, (D,))).astype(np.float32)
    kn = (1.0 + 0.1 * I.normal(g, (D,))).astype(np.float32)
    return qg, k, v, qn, kn


@pytest.mark.parametrize("Hq,Hkv,D,n_rot", [(24, 4, 256, 64), (4, 1, 64, 64), (8, 2, 128, 32)])
def test_against_numpy_float64(Hq, Hkv, D, n_rot):
    T, base, eps = 5, 1e7, 1e-6
    qg, k, v, qn, kn = make(3, T, Hq, Hkv, D)
    pos = np.array([0, 1, 17, 4000, 65535], np.int32)
    c = O.HostKV.contiguous(O.KV_F16, 70000, Hkv, D)
    q, gate = O.attn_prep(c, qg, k, v, qn, kn, pos, -1, Hq, n_rot, base, eps)
    assert np.array_equal(gate.reshape(T, Hq, D), qg[:, :, D:])                 # the gate is a plain copy
    for t in range(T):
        for h in range(Hq):
            ref = np_norm_rope(qg[t, h, :D], qn, n_rot, base, eps, float(pos[t]))
            # fp32 angle: pos * inv_freq carries up to pos * 2^-24 of absolute angle error at the largest positions
            tol = 4e-6 + 2.0 * pos[t] * 2.0 ** -24
            assert np.max(np.abs(q[t, h] - ref)) < tol * max(1.0, np.abs(ref).max()), (t, h)
        for h in range(Hkv):
            ref = np_norm_rope(k[t, h], kn, n_rot, base, eps, float(pos[t]))
            got = O.kv_read_head(c, 0, 0, int(pos[t]), h)                       # f16 cache: half precision of the roped k
            assert np.max(np.abs(got - ref)) < 2e-3 * max(1.0, np.abs(ref).max())
            assert np.array_equal(O.kv_read_head(c, 1, 0, int(pos[t]), h), v[t, h].astype(np.float16).astype(np.float32))


def test_closed_forms():
    Hq, Hkv, D, n_rot, base = 2, 1, 64, 64, 1e4
    qg, k, v, qn, kn = make(8, 3, Hq, Hkv, D)
    c = O.HostKV.contiguous(O.KV_F16, 64, Hkv, D)
    # position 0 rotates nothing: q is the plain norm
    q0, _ = O.attn_prep(c, qg, k, v, None, None, np.zeros(3, np.int32), 0, Hq, n_rot, base)
    ref = O.rmsnorm_heads(qg[:, :, :D].copy(), D)
    assert np.max(np.abs(q0 - ref)) < 2e-6
    # a constant head norms to +-1 * w (eps aside)
    qc = np.full((1, Hq, 2 * D), -3.0, np.float32)
    q1, _ = O.attn_prep(c, qc, k[:1], v[:1], qn, None, np.zeros(1, np.int32), 0, Hq, n_rot, base, eps=0.0)
    assert np.allclose(q1[0, 0], -qn, rtol=0, atol=2e-7)
    # the rotation keeps the norm of every pair, and q . k after rope depends on the position difference only
    pa = np.array([5, 105, 1005], np.int32)
    kk = np.repeat(k[:1], 3, 0)
    qq = np.repeat(qg[:1], 3, 0)
    ca = O.HostKV.contiguous(O.KV_F16, 2048, Hkv, D)
    qa, _ = O.attn_prep(ca, qq, kk, v, None, None, pa, -1, Hq, n_rot, base)
    qb, _ = O.attn_prep(ca, qq, kk, v, None, None, pa + 7, -1, Hq, n_rot, base)
    half = n_rot // 2
    n0 = qa[:, :, :half] ** 2 + qa[:, :, half:n_rot] ** 2
    n1 = q0[:1, :, :half] ** 2 + q0[:1, :, half:n_rot] ** 2
    assert np.allclose(n0, np.repeat(n1, 3, 0), rtol=2e-5, atol=1e-6)
    # <rope(x, p + 7), rope(y, p)> is the same for every p: use q head 0 as x, q head 1 as y
    dots = [(qb[i, 0].astype(np.float64) * qa[i, 1].astype(np.float64)).sum() for i in range(3)]
    assert max(dots) - min(dots) < 2e-3 * max(1.0, abs(dots[0]))


@pytest.mark.parametrize("kv_type", TYPES)
def test_kv_rows_are_the_append_of_the_roped_k(kv_type):
    """device-position mode, per-row page tables: the K / V bytes equal a plain append of the normed, roped k"""
    Hq, Hkv, D, n_rot, base, psh = 8, 2, 128, 64, 1e7, 4
    T = 4
    qg, k, v, qn, kn = make(11, T, Hq, Hkv, D)
    max_pages, n_pages = 8, 40
    g = I.rng(5)
    table = g.permutation(n_pages)[: T * max_pages].astype(np.int32)
    rtab = (np.arange(T) * max_pages).astype(np.int32)
    pos = np.array([0, 33, 100, 127], np.int32)
    c1 = O.HostKV.paged(kv_type, Hkv, D, psh, n_pages, table, max_pages).view(rtab=rtab)
    c1.pool = None
    O.attn_prep(c1, qg, k, v, qn, kn, pos, -1, Hq, n_rot, base)
    # reference chain: norm + rope through the q path of the same function (heads of k fed as "q | gate" slices)
    kq = np.concatenate([k, np.zeros_like(k)], axis=2)
    cf = O.HostKV.contiguous(O.KV_F16, 128, Hkv, D)
    kr, _ = O.attn_prep(cf, kq, k, v, kn, None, pos, -1, Hkv, n_rot, base)
    c2 = O.HostKV.paged(kv_type, Hkv, D, psh, n_pages, table, max_pages).view(rtab=rtab)
    O.kv_append_rows(c2, kr, v, pos)
    assert np.array_equal(c1.k, c2.k) and np.array_equal(c1.v, c2.v)
    # host-position mode writes rows p0 + t of ONE table while the angle still follows pos[t]
    c3 = O.HostKV.contiguous(kv_type, 16, Hkv, D)
    c4 = O.HostKV.contiguous(kv_type, 16, Hkv, D)
    O.attn_prep(c3, qg, k, v, qn, kn, pos, 3, Hq, n_rot, base)
    O.kv_append_rows(c4, kr, v, 3 + np.arange(T))
    assert np.array_equal(c3.k, c4.k) and np.array_equal(c3.v, c4.v)


def np_a16(y):
    """independent float32 restatement of the a16 activation quantize (src/fast/matvec_a16.cu:29-100): the slot of each
    element is written out from the engine's comment 'lanes holding elements 0..15 write outputs 4k+0 / 4k+2; those
    holding 16..31 write 4k+1 / 4k+3', lane = 4 consecutive elements, pairs (v0, v2) and (v1, v3)"""
    T, n = y.shape
    ng = n // 32
    out = np.zeros((T, ng, 16, 2), np.float16)
    ads = np.zeros((T, ng, 2), np.float16)
    for t in range(T):
        for g in range(ng):
            v = y[t, 32 * g:32 * g + 32].astype(np.float32)
            amax = np.float32(np.abs(v).max())
            if not amax < np.float32(65520.0):
                amax = np.float32(65504.0)
            idv = np.float32(1.0) / amax if amax > 0 else np.float32(0.0)
            w = (v * idv).astype(np.float32)
            for x in range(32):
                hi, xx = x // 16, x % 16
                k, i = xx // 4, xx % 4
                out[t, g, 4 * k + 2 * (i & 1) + hi, i >> 1] = np.float16(w[x])
            lane = [np.float32(0.0)] * 8
            for l in range(8):
                s_ = np.float32(0.0)
                for i in range(4):
                    s_ = np.float32(s_ + w[4 * l + i])
                lane[l] = s_
            for st in (4, 2, 1):
                lane = [np.float32(lane[l] + lane[l ^ st]) for l in range(8)]
            ads[t, g] = (np.float16(amax), np.float16(lane[0]))
    return np.concatenate([out.reshape(-1).view(np.uint16), ads.reshape(-1).view(np.uint16)])


def test_a16_quant_against_numpy_and_closed_forms():
    g = I.rng(31)
    y = (I.normal(g, (3, 256)) * np.array([[1.0], [300.0], [1e-3]], np.float32)).astype(np.float32)
    y[0, 32:64] = 0.0                     # an all-zero group: amax 0, scale 0, every value 0
    y[1, 64:96] = 1.0                     # a unit group: every value 1, sum 32
    y[2, 0] = 7.0e4                       # above the f16 range: the stored scale clamps to 65504, values scale by 1 / 65504
    got = O.a16_quant(y)
    assert np.array_equal(got, np_a16(y))
    ng = 8
    vals = got[: 3 * ng * 32].view(np.float16).reshape(3, ng, 32)
    ads = got[3 * ng * 32:].view(np.float16).reshape(3, ng, 2)
    assert np.all(vals[0, 1] == 0) and ads[0, 1, 0] == 0 and ads[0, 1, 1] == 0
    assert np.all(vals[1, 2] == 1) and ads[1, 2, 0] == 1 and ads[1, 2, 1] == 32
    assert ads[2, 0, 0] == np.float16(65504.0) and np.isfinite(vals[2, 0].astype(np.float32)).all()
    assert np.float32(vals[2, 0].astype(np.float32).max()) > 1.0      # |v| / 65504 passes 1 for the clamped group
    # every scaled value is v / amax: the largest magnitude of an ordinary group is exactly 1
    assert np.abs(vals[0, 0].astype(np.float32)).max() == 1.0


# ---- interleaved M-RoPE (src/fast/mrope.cuh) ----
# Which stream each rotary pair of the first 32 uses with the model's sections [11, 11, 10, 0] (sect 32), written out by
# hand from the rule's words: streams interleave t, h, w, t, h, w, ... while their sections last (t and h 11 pairs each =
# sectors below 33, w 10 pairs = sectors below 30), so sector 29 (29 % 3 == 2, but 29 < 30) is still w and nothing falls
# to the fourth stream.
STREAMS_11_11_10 = "thw" * 10 + "th"
# sections [2, 1, 1, 0] (sect 4): sector 0 -> t; 1 -> h (1 < 3); 2 -> w (2 < 3); 3 -> 3 % 3 == 0 and 3 < 6 -> t
STREAMS_2_1_1 = "thwt"


def stream_table(sections, n):
    s0, s1, s2, s3 = sections
    sect = s0 + s1 + s2 + s3
    tab = {(11, 11, 10, 0): STREAMS_11_11_10, (2, 1, 1, 0): STREAMS_2_1_1}[tuple(sections)]
    return [tab[j % sect] for j in range(n)], sect


def test_mrope_text_rows_are_plain_neox_bitwise():
    """t = h = w = p: every pair rotates by p (src/fast/mrope.cuh:6-7)"""
    Hq, Hkv, D, n_rot, T = 4, 1, 256, 64, 6
    qg, k, v, qn, kn = make(11, T, Hq, Hkv, D)
    pos = np.array([0, 3, 500, 501, 9000, 65000], np.int32)
    for kt in TYPES:
        c1, c2 = O.HostKV.contiguous(kt, 66000, Hkv, D), O.HostKV.contiguous(kt, 66000, Hkv, D)
        q1, g1 = O.attn_prep(c1, qg, k, v, qn, kn, pos, -1, Hq, n_rot, 1e7)
        q2, g2 = O.attn_prep(c2, qg, k, v, qn, kn, pos, -1, Hq, n_rot, 1e7, mrope=(np.stack([pos, pos, pos]), (11, 11, 10), 32))
        assert np.array_equal(q1, q2) and np.array_equal(g1, g2)
        assert np.array_equal(c1.k, c2.k) and np.array_equal(c1.v, c2.v)


@pytest.mark.parametrize("sections,n_rot", [((11, 11, 10, 0), 64), ((2, 1, 1, 0), 32), ((11, 11, 10, 0), 128)])
def test_mrope_each_pair_rotates_by_its_stream(sections, n_rot):
    """against float64 with the stream of every pair taken from the hand-written tables"""
    Hq, Hkv, D, T, base, eps = 2, 1, 128, 3, 1e6, 1e-6
    qg, k, v, qn, kn = make(12, T, Hq, Hkv, D)
    streams, sect = stream_table(sections, n_rot // 2)
    mp = np.array([[7, 100, 2000], [9, 140, 2077], [30, 101, 1950]], np.int32)      # t, h, w of the 3 rows
    pos = np.array([5, 6, 7], np.int32)                                              # cache rows: unrelated to the rotation
    c = O.HostKV.contiguous(O.KV_F16, 16, Hkv, D)
    q, _ = O.attn_prep(c, qg, k, v, qn, kn, pos, -1, Hq, n_rot, base, eps, mrope=(mp, sections[:3], sect))
    half = n_rot // 2
    for t in range(T):
        x = qg[t, 0, :D].astype(np.float64)
        y = x / np.sqrt((x * x).mean() + eps) * qn.astype(np.float64)
        p = np.array([mp["thw".index(s), t] for s in streams], np.float64)
        th = p * base ** (-2.0 * np.arange(half) / n_rot)
        ref = y.copy()
        ref[:half] = y[:half] * np.cos(th) - y[half:n_rot] * np.sin(th)
        ref[half:n_rot] = y[:half] * np.sin(th) + y[half:n_rot] * np.cos(th)
        assert np.max(np.abs(q[t, 0] - ref)) < (4e-6 + 2.0 * p.max() * 2.0 ** -24) * max(1.0, np.abs(ref).max())
        # the K row landed at pos[t], rotated the same way
        got = O.kv_read_head(c, 0, 0, int(pos[t]), 0)
        xk = k[t, 0].astype(np.float64)
        yk = xk / np.sqrt((xk * xk).mean() + eps) * kn.astype(np.float64)
        refk = yk.copy()
        refk[:half] = yk[:half] * np.cos(th) - yk[half:n_rot] * np.sin(th)
        refk[half:n_rot] = yk[:half] * np.sin(th) + yk[half:n_rot] * np.cos(th)
        assert np.max(np.abs(got - refk)) < 2e-3 * max(1.0, np.abs(refk).max())


def test_mrope_moving_one_stream_moves_only_its_pairs():
    Hq, Hkv, D, n_rot = 1, 1, 64, 64
    qg, k, v, qn, kn = make(13, 1, Hq, Hkv, D)
    streams, sect = stream_table((11, 11, 10, 0), 32)
    base_p = np.array([[50], [50], [50]], np.int32)
    c = O.HostKV.contiguous(O.KV_F16, 4, Hkv, D)
    q0, _ = O.attn_prep(c, qg, k, v, qn, kn, np.array([0], np.int32), -1, Hq, n_rot, 1e4, mrope=(base_p, (11, 11, 10), sect))
    for si, name in enumerate("thw"):
        mp = base_p.copy()
        mp[si, 0] = 61
        q1, _ = O.attn_prep(c, qg, k, v, qn, kn, np.array([0], np.int32), -1, Hq, n_rot, 1e4, mrope=(mp, (11, 11, 10), sect))
        changed = {j for j in range(32) if q1[0, 0, j] != q0[0, 0, j] or q1[0, 0, j + 32] != q0[0, 0, j + 32]}
        assert changed == {j for j in range(32) if streams[j] == name}


def test_rotary_recipes_against_numpy_float64():
    """the oracle's power / cosine / sine are IEEE double recipes in a fixed order (no math library, so the GPU kernel can
    reproduce every bit); here they are held against numpy's float64 functions: base^(-2j/n) to 32 ulps of double (e^(x ln b)
    carries |x| roundings of x; the value is used rounded to fp32, 2^29 times coarser), the
    fp32 cosine and sine of an fp32 angle equal to the rounded float64 value except for rare last-bit roundings"""
    import ctypes
    L = O.lib()
    for base in (1e7, 1e4, 5e5, 1e6, 2.0, 123456.789):
        for n_rot in (8, 32, 64, 128, 256):
            for j in range(n_rot // 2):
                got = L.orc_prep_inv_freq(base, j, n_rot)
                want = float(np.float64(np.float32(base)) ** (-2.0 * j / n_rot))
                assert abs(got - want) <= 32 * np.spacing(want), (base, n_rot, j, got, want)
    g = np.random.default_rng(5)
    angles = np.concatenate([
        g.uniform(0, 7, 20000), g.uniform(0, 3e5, 20000), g.uniform(0, 2.0 ** 29, 5000), np.arange(0, 64) * (np.pi / 4),
        np.arange(1, 4000) * (np.pi / 2), [0.0, 1e-30, 1e-8, 262143.0, 1e6],
    ]).astype(np.float32)
    c, s = ctypes.c_float(), ctypes.c_float()
    off = 0
    for th in angles:
        L.orc_prep_sincos(float(th), ctypes.byref(c), ctypes.byref(s))
        wc, ws = np.float32(np.cos(np.float64(th))), np.float32(np.sin(np.float64(th)))
        for got, want in ((np.float32(c.value), wc), (np.float32(s.value), ws)):
            if got != want:
                off += 1
                assert abs(np.float64(got) - np.float64(want)) <= np.spacing(np.abs(want)) , (th, got, want)
    assert off <= 4, off          # (a float64 result within a few 2^-53 of an fp32 rounding boundary may round the other way)
    L.orc_prep_sincos(0.0, ctypes.byref(c), ctypes.byref(s))
    assert c.value == 1.0 and s.value == 0.0
