"""Quantize-on-append on the GPU (through the C ABI) vs the oracle: every byte must match."""
import os

import numpy as np
import pytest
import torch

import _inputs as I
import _oracle as O
from _gpu import Pool, dev

pytestmark = pytest.mark.gpu
TYPES = [O.KV_F16, O.KV_Q8_0, O.KV_Q4_0]
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "quant_golden.npz"))


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("Hkv,D", [(4, 256), (1, 64), (2, 128), (3, 96)])
def test_contiguous_bytes(p1a, kv_type, Hkv, D):
    T, p0, n_ctx = 37, 5, 48
    g = I.rng(100 + D)
    k = I.normal(g, (T, Hkv, D)) * 1.7
    v = I.normal(g, (T, Hkv, D)) * 0.3
    k[3] = 0.0                      # an all-zero row
    v[4, :, :32] = 0.0
    host = O.HostKV.contiguous(kv_type, n_ctx, Hkv, D)
    O.kv_append_rows(host, k, v, p0 + np.arange(T))
    c = p1a.KVCache.contiguous(kv_type, n_ctx, Hkv, D)
    p1a.kv_append(c, dev(k), dev(v), p0, T)
    torch.cuda.synchronize()
    assert np.array_equal(c._keep[0].cpu().numpy(), host.k)
    assert np.array_equal(c._keep[1].cpu().numpy(), host.v)


@pytest.mark.parametrize("kv_type", [O.KV_Q8_0, O.KV_Q4_0])
def test_golden_blocks_on_gpu(p1a, kv_type):
    """the reference's own quantizer outputs, reproduced by the HIP kernel (edge cases included)"""
    x = GOLD["x"]
    n = x.shape[0] // 8 * 8
    rows = x[:n].reshape(n // 8, 1, 256)
    c = p1a.KVCache.contiguous(kv_type, n // 8, 1, 256)
    p1a.kv_append(c, dev(rows), dev(rows), 0, n // 8)
    torch.cuda.synchronize()
    got = c._keep[0].cpu().numpy().reshape(n // 8, -1)
    if kv_type == O.KV_Q8_0:
        assert np.array_equal(got[:, :16].copy().view(np.uint16).reshape(-1), GOLD["q8_d"][:n])
        assert np.array_equal(got[:, 16:].copy().view(np.int8).reshape(n, 32), GOLD["q8_q"][:n])
    else:
        assert np.array_equal(got.reshape(n, 18), GOLD["q4_blk"][:n])


@pytest.mark.parametrize("kv_type", TYPES)
def test_paged_dev_and_rows(p1a, kv_type):
    Hq, Hkv, D, psh = 12, 2, 256, 5
    lens = [70, 200, 33]
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, lens, seed=3, n_layers=3, layer=1, fill="none")
    # host side: oracle appends; device side: chunks via host p0, device p0, and multi-sequence rows
    for s, n in enumerate(lens):
        O.kv_append_rows(pool.host.view(rtab=np.full(n, s * pool.maxp, np.int32)), pool.k[s], pool.v[s], np.arange(n))
    dk = [dev(k) for k in pool.k]
    dv = [dev(v) for v in pool.v]
    c0 = pool.dev_seq(0)
    p1a.kv_append(c0, dk[0], dv[0], 0, 64)
    p1a.kv_append(c0, dk[0][64:], dv[0][64:], 64, lens[0] - 64)
    c1 = pool.dev_seq(1)
    p0d = dev(np.array([0], np.int32))
    for a in range(0, lens[1], 50):
        p0d.fill_(a)
        p1a.kv_append_dev(c1, dk[1][a:], dv[1][a:], p0d, min(50, lens[1] - a))
    # rows of sequences 2, 0 (rewrite), 2 in one call
    n2 = lens[2]
    rows_s = [2] * n2 + [0, 0]
    rows_p = list(range(n2)) + [10, 69]
    kk = torch.cat([dk[2], dk[0][10:11], dk[0][69:70]])
    vv = torch.cat([dv[2], dv[0][10:11], dv[0][69:70]])
    cr = pool.devkv.with_rows(dev(np.array([s * pool.maxp for s in rows_s], np.int32)))
    p1a.kv_append_rows(cr, kk, vv, dev(np.array(rows_p, np.int32)), len(rows_p))
    torch.cuda.synchronize()
    assert np.array_equal(pool.dpool.cpu().numpy(), pool.host.pool)


@pytest.mark.parametrize("kv_type", TYPES)
def test_fill_random_bytes(p1a, kv_type):
    """the benchmark fill (the reference's kv_fill_random): contiguous and paged, whole and partial ranges, every byte as
    the oracle writes it and nothing else touched; a filled cache then decodes like the oracle"""
    Hq, Hkv, D, psh = 12, 2, 256, 5
    n = 300
    host = O.HostKV.contiguous(kv_type, n, Hkv, D)
    c = p1a.KVCache.contiguous(kv_type, n, Hkv, D)
    for a, b, seed in [(0, 100, 1), (100, 300, 1), (37, 41, 99), (50, 50, 5)]:
        O.kv_fill_random(host, a, b, seed)
        p1a.kv_fill_random(c, a, b, seed)
    torch.cuda.synchronize()
    assert np.array_equal(c._keep[0].cpu().numpy(), host.k) and np.array_equal(c._keep[1].cpu().numpy(), host.v)
    with pytest.raises(p1a.P1AError):
        p1a.kv_fill_random(c, 0, n + 1, 1)                       # past the end of a contiguous cache
    lens = [700, 90]
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, lens, seed=8, n_layers=3, layer=2, fill="none")
    pool.host.pool[:] = 0x33
    pool.dpool.fill_(0x33)
    for s, (a, b) in enumerate([(5, 700), (0, 90)]):
        O.kv_fill_random(pool.host_seq(s), a, b, 0x9e3779b9 * (s + 1))
        p1a.kv_fill_random(pool.dev_seq(s), a, b, 0x9e3779b9 * (s + 1))
    torch.cuda.synchronize()
    assert np.array_equal(pool.dpool.cpu().numpy(), pool.host.pool)
    from _gpu import check
    q, _, _, gate = I.qkv(9, 1, 2, Hq, Hkv, D)
    ref = O.attn_rows(pool.host_seq(0), q, np.array([698, 699], np.int32), Hq, 1 / 16, gate=gate)
    out = torch.empty((2, Hq, D), device="cuda")
    p1a.attn_decode(dev(q), pool.dev_seq(0), out, 2, 698, Hq, 1 / 16, gate=dev(gate))
    check(out.cpu().numpy(), ref, f"decode over a filled cache, type {kv_type}")


@pytest.mark.parametrize("kv_type", [O.KV_Q8_0, O.KV_Q4_0])
def test_half_way_points_and_golden_blocks_in_a_long_call(p1a, kv_type):
    """a call of a thousand rows: the reference quantizer's golden blocks - edge cases included - and blocks crafted so that
    x / d lands exactly on half-way points (x.5 must round away from zero), just inside them, on the clamp (q4_0: code
    16 -> 15) and on signed zeros, byte for byte the oracle's"""
    gold = GOLD["x"]
    n = gold.shape[0] // 8 * 8
    g = I.rng(4242)
    crafted = np.zeros((2048, 32), np.float32)
    for b in range(crafted.shape[0]):
        top = float(g.choice([127.0, 63.5, 254.0, 8.0, 1.0, 16.0, 0.5]))
        sign = -1.0 if b % 3 == 0 else 1.0
        crafted[b, 0] = sign * top                                  # the block maximum: d = top / 127 (q8_0), -+top / 8 (q4_0)
        ks = g.integers(-126, 127, 31).astype(np.float32)
        d8 = top / 127.0
        half = (ks + np.where(ks >= 0, 0.5, -0.5)) * d8             # exact half-way points of the q8_0 grid where representable
        near = np.nextafter(half.astype(np.float32), np.float32(0)) # ... and the float just inside them
        crafted[b, 1:] = np.where(g.integers(0, 3, 31) == 0, near, half).astype(np.float32)
        if b % 7 == 0:
            crafted[b, 5:9] = [0.0, -0.0, top / 16.0, -top / 16.0]
    x = np.concatenate([gold[:n], gold[:n], crafted.reshape(-1, 32)]).astype(np.float32)
    nb = x.shape[0] // 8 * 8
    rows = np.ascontiguousarray(x[:nb].reshape(nb // 8, 1, 256))
    host = O.HostKV.contiguous(kv_type, nb // 8, 1, 256)
    O.kv_append_rows(host, rows, rows[::-1].copy(), np.arange(nb // 8))
    c = p1a.KVCache.contiguous(kv_type, nb // 8, 1, 256)
    p1a.kv_append(c, dev(rows), dev(rows[::-1].copy()), 0, nb // 8)
    torch.cuda.synchronize()
    assert np.array_equal(c._keep[0].cpu().numpy(), host.k)
    assert np.array_equal(c._keep[1].cpu().numpy(), host.v)
    # and the golden bytes themselves
    got = c._keep[0].cpu().numpy().reshape(nb // 8, -1)[:n // 8]
    if kv_type == O.KV_Q8_0:
        assert np.array_equal(got[:, 16:].copy().view(np.int8).reshape(n, 32), GOLD["q8_q"][:n])
    else:
        assert np.array_equal(got.reshape(n, 18), GOLD["q4_blk"][:n])
