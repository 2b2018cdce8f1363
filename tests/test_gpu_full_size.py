"""The benchmark configurations at their FULL sizes (the other test files run them scaled down): KV written by the GPU
append must equal the oracle's bytes, attention must match the oracle within the path's tolerance (every row of every
configuration, the 4096 prefill rows included), and the size-independent identities must hold:
batched rows == solo rows and verify rows == single-row calls bit for bit, prefill with and without scratch bit for
bit, prefill rows == decode rows at their positions."""
import numpy as np
import pytest
import torch

import _inputs as I
import _oracle as O
from _gpu import Pool, check, dev

pytestmark = pytest.mark.gpu
Hq, Hkv, D, PSH = 24, 4, 256, 8


def gpu_fill(p1a, pool):
    """write every sequence through the library's own quantizing append; the device pool must then equal the oracle's"""
    for s, n in enumerate(pool.lens):
        c = pool.dev_seq(s)
        for a in range(0, n, 8192):
            b = min(n, a + 8192)
            p1a.kv_append(c, dev(pool.k[s][a:b]), dev(pool.v[s][a:b]), a, b - a)
    torch.cuda.synchronize()
    assert np.array_equal(pool.dpool.cpu().numpy(), pool.host.pool)


def test_config2_decode_32k_q8_0(p1a):
    n = 32768
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, PSH, [n], seed=2)
    pool.dpool.zero_()
    gpu_fill(p1a, pool)
    q, _, _, gate = I.qkv(20, 1, 1, Hq, Hkv, D)
    ref = O.attn_rows(pool.host_seq(0), q, np.array([n - 1], np.int32), Hq, 1 / 16, gate=gate)
    out = torch.empty((1, Hq, D), device="cuda")
    p1a.attn_decode(dev(q), pool.dev_seq(0), out, 1, n - 1, Hq, 1 / 16, gate=dev(gate))
    check(out.cpu().numpy(), ref, "config 2", flat=True)
    # device-resident position: same bits
    out2 = torch.empty_like(out)
    p1a.attn_decode_dev(dev(q), pool.dev_seq(0), out2, 1, dev(np.array([n - 1], np.int32)), n, Hq, 1 / 16, gate=dev(gate))
    assert torch.equal(out, out2)


def test_config3_batched_8_slots(p1a):
    g = I.rng(3)
    lens = [int(np.exp(g.uniform(np.log(1024), np.log(32768)))) for _ in range(8)]
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, PSH, lens, seed=3)
    q, _, _, gate = I.qkv(30, 1, 8, Hq, Hkv, D)
    pos = np.array([n - 1 for n in lens], np.int32)
    rtab = np.array([s * pool.maxp for s in range(8)], np.int32)
    ref = O.attn_rows(pool.host.view(rtab=rtab), q, pos, Hq, 1 / 16, gate=gate)
    out = torch.empty((8, Hq, D), device="cuda")
    p1a.attn_decode_rows(dev(q), pool.devkv.with_rows(dev(rtab)), out, 8, dev(pos), Hq, 1 / 16, gate=dev(gate))
    check(out.cpu().numpy(), ref, "config 3", flat=True)
    for t in range(8):
        one = torch.empty((1, Hq, D), device="cuda")
        p1a.attn_decode(dev(q[t:t + 1]), pool.dev_seq(t), one, 1, int(pos[t]), Hq, 1 / 16, gate=dev(gate[t:t + 1]))
        assert torch.equal(one[0], out[t]), t


def test_config4_verify_4x4_q4_0_64k(p1a):
    n, R = 65536, 4
    pool = Pool(p1a, O.KV_Q4_0, Hq, Hkv, D, PSH, [n] * 4, seed=4, f16_inputs=True)
    q, _, _, _ = I.qkv(40, 1, 4 * R, Hq, Hkv, D, f16_inputs=True)
    pos = np.array([n - R + t for _ in range(4) for t in range(R)], np.int32)
    rtab = np.array([s * pool.maxp for s in range(4) for _ in range(R)], np.int32)
    ref = O.attn_rows(pool.host.view(rtab=rtab), q, pos, Hq, 1 / 16)
    out = torch.empty((4 * R, Hq, D), device="cuda")
    p1a.attn_decode_rows(dev(q), pool.devkv.with_rows(dev(rtab)), out, 4 * R, dev(pos), Hq, 1 / 16, rows_per_seq=R)
    check(out.cpu().numpy(), ref, "config 4", flat=True)
    for t in (0, 3, 6, 9, 15):                                  # verify rows == single-row calls
        one = torch.empty((1, Hq, D), device="cuda")
        p1a.attn_decode(dev(q[t:t + 1]), pool.dev_seq(t // R), one, 1, int(pos[t]), Hq, 1 / 16)
        assert torch.equal(one[0], out[t]), t


def test_config5_append_4096_then_prefill_over_32768(p1a):
    p0, T = 28672, 4096
    n = p0 + T
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, PSH, [n], seed=5)
    pool.dpool.zero_()
    c = pool.dev_seq(0)
    k, v = pool.k[0], pool.v[0]
    for a in range(0, p0, 4096):
        p1a.kv_append(c, dev(k[a:a + 4096]), dev(v[a:a + 4096]), a, 4096)
    p1a.kv_append(c, dev(k[p0:]), dev(v[p0:]), p0, T)           # the chunk's own K/V: codes bit-exact
    torch.cuda.synchronize()
    assert np.array_equal(pool.dpool.cpu().numpy(), pool.host.pool)
    q, _, _, gate = I.qkv(50, 1, T, Hq, Hkv, D, f16_inputs=True)
    dq, dg = dev(q), dev(gate)
    out = torch.full((T, Hq, D), float("nan"), device="cuda")
    p1a.attn_prefill(dq, c, out, T, p0, Hq, 1 / 16, gate=dg)
    scr = torch.full((p1a.prefill_scratch_bytes(T, p0, Hq, Hkv, D),), 0xff, dtype=torch.uint8, device="cuda")
    out2 = torch.full((T, Hq, D), float("nan"), device="cuda")
    p1a.attn_prefill(dq, c, out2, T, p0, Hq, 1 / 16, gate=dg, scratch=scr)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and torch.equal(out, out2)
    # the oracle on ALL 4096 rows (about half a minute of host time), in blocks so that progress shows
    got = out.cpu().numpy()
    worst = (0.0, 0.0)
    for a in range(0, T, 512):
        rows = np.arange(a, a + 512)
        ref = O.attn_rows(pool.host_seq(0), q[rows], (p0 + rows).astype(np.int32), Hq, 1 / 16, gate=gate[rows])
        ma, rl = check(got[rows], ref, f"config 5 rows {a}..{a + 511}", flat=True)
        worst = (max(worst[0], ma), max(worst[1], rl))
        print(f"config 5: rows {a}..{a + 511} checked", flush=True)
    print(f"[parity] config 5, all {T} rows: worst block max_abs={worst[0]:.3e} rel_l2={worst[1]:.3e}")
    # every 97th prefill row against the decode kernel at its position (two independent kernels)
    pick = np.arange(0, T, 97)
    dec = torch.empty((len(pick), Hq, D), device="cuda")
    for i, t in enumerate(pick):
        p1a.attn_decode(dq[t:t + 1], c, dec[i:i + 1], 1, p0 + int(t), Hq, 1 / 16, gate=dg[t:t + 1])
    torch.cuda.synchronize()
    ma, rl = I.errors(out.cpu().numpy()[pick], dec.cpu().numpy())
    assert ma < 1e-3 and rl < 5e-4, (ma, rl)


@pytest.mark.parametrize("kv_type", [O.KV_Q8_0, O.KV_F16])
def test_pages_beyond_4_gib(p1a, kv_type):
    """page bases are 64-bit (the engine keeps one layer's K region under 4 GiB to index it with 32 bits,
    src/tp_model.cu:3917-3919; this library does not): a pool of > 5 GB whose sequence lives in pages on both sides of the
    4 GiB line - append, decode, prefill and the benchmark fill all address them, and what they write is, page by page,
    the oracle's bytes for a contiguous cache"""
    Hq, Hkv, D, psh, n = 24, 4, 256, 8, 2000
    ps = 1 << psh
    rowb = p1a.kv_row_bytes(kv_type, Hkv, D)
    pstride = 2 * ps * rowb
    n_pages = (5 << 30) // pstride + 1
    line = (4 << 30) // pstride                                  # first page that starts beyond 4 GiB
    pages = [n_pages - 1, line + 90, 3, line + 1, n_pages - 2, line - 1, line + 700, 17]
    assert len(pages) * ps >= n and pages[0] * pstride > (5 << 30) - pstride
    tab = dev(np.array(pages, np.int32))
    pool = torch.empty(n_pages * pstride, dtype=torch.uint8, device="cuda")
    c = p1a.KVCache.paged(kv_type, Hkv, D, psh, n_pages, tab, len(pages), pool=pool)
    q, k, v, gate = I.qkv(123, n, 4, Hq, Hkv, D)
    host = O.HostKV.contiguous(kv_type, len(pages) * ps, Hkv, D)
    O.kv_append_rows(host, k, v, np.arange(n))
    p1a.kv_append(c, dev(k), dev(v), 0, n)
    torch.cuda.synchronize()
    for g, pg in enumerate(pages):                               # the device pages hold the oracle's rows
        rows = min(ps, n - g * ps)
        if rows <= 0:
            break
        kd = pool[pg * pstride: pg * pstride + rows * rowb].cpu().numpy()
        vd = pool[pg * pstride + ps * rowb: pg * pstride + ps * rowb + rows * rowb].cpu().numpy()
        assert np.array_equal(kd, host.k[g * ps * rowb: (g * ps + rows) * rowb]), g
        assert np.array_equal(vd, host.v[g * ps * rowb: (g * ps + rows) * rowb]), g
    pos = np.arange(n - 4, n, dtype=np.int32)
    ref = O.attn_rows(host, q, pos, Hq, 1 / 16, gate=gate)
    out = torch.empty((4, Hq, D), device="cuda")
    p1a.attn_decode(dev(q), c, out, 4, n - 4, Hq, 1 / 16, gate=dev(gate))
    check(out.cpu().numpy(), ref, f"decode over pages beyond 4 GiB, type {kv_type}")
    T = 300
    qp, _, _, gp = I.qkv(124, 1, T, Hq, Hkv, D, f16_inputs=True)
    refp = O.attn_rows(host, qp, np.arange(n - T, n, dtype=np.int32), Hq, 1 / 16, gate=gp)
    outp = torch.empty((T, Hq, D), device="cuda")
    p1a.attn_prefill(dev(qp), c, outp, T, n - T, Hq, 1 / 16, gate=dev(gp))
    check(outp.cpu().numpy(), refp, f"prefill over pages beyond 4 GiB, type {kv_type}")
    O.kv_fill_random(host, 100, n, 77)                           # (paged fill = page by page with the page's seed:
    hp = O.HostKV.paged(kv_type, Hkv, D, psh, len(pages), np.arange(len(pages), dtype=np.int32), len(pages))   # a compact host twin)
    hp.pool[:] = 0
    O.kv_append_rows(hp, k, v, np.arange(n))
    O.kv_fill_random(hp, 100, n, 77)
    p1a.kv_fill_random(c, 100, n, 77)
    torch.cuda.synchronize()
    for g, pg in enumerate(pages):
        got = pool[pg * pstride: (pg + 1) * pstride].cpu().numpy()
        rows = max(0, min(ps, n - g * ps))
        want = hp.pool[g * pstride: (g + 1) * pstride]
        assert np.array_equal(got[: rows * rowb], want[: rows * rowb]), g
        assert np.array_equal(got[ps * rowb: ps * rowb + rows * rowb], want[ps * rowb: ps * rowb + rows * rowb]), g
