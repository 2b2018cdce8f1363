"""Decode / verify at the depths the engine's own test goes to (tests/fast_attn_test.cu:232-295 of the reference tree:
p0 up to 131072, T = 1 and 4 against an independent kernel, T-invariance at that depth) and at the engine's default
context limit of 262144 (src/engine.h:28); and prefill in the input regime of the engine's fold test
(tests/fast_attn_fold_test.cu:20-27,38-39: sum-of-three-uniforms values, every 37th dim of a row times 4, q scaled by 2 -
heavy-tailed logits carried by a few outlier dims, a peaked softmax) over 32 K keys.
The deep caches are written by the library's own quantizing append from values drawn on the device (its bytes are
checked against the oracle's elsewhere); the oracle then reads the very bytes the kernels read."""
import numpy as np
import pytest
import torch

import _inputs as I
import _oracle as O
from _gpu import check, dev

pytestmark = pytest.mark.gpu
Hq, Hkv, D, PSH = 24, 4, 256, 8


def deep_cache(p1a, kv_type, n, seed):
    ps = 1 << PSH
    maxp = (n + ps - 1) // ps + 1
    n_pages = maxp + 5
    table = I.rng(seed).permutation(n_pages)[:maxp].astype(np.int32)
    c = p1a.KVCache.paged(kv_type, Hkv, D, PSH, n_pages, dev(table), maxp)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    for a in range(0, n, 16384):
        m = min(16384, n - a)
        k = torch.randn((m, Hkv, D), generator=gen, device="cuda")
        k = k * torch.rsqrt((k * k).mean(dim=-1, keepdim=True) + 1e-6)
        v = torch.randn((m, Hkv, D), generator=gen, device="cuda")
        p1a.kv_append(c, k, v, a, m)
    torch.cuda.synchronize()
    host = O.HostKV.paged(kv_type, Hkv, D, PSH, n_pages, table, maxp, pool=c.pool.cpu().numpy())
    return c, host.view(pt=table)


@pytest.mark.parametrize("kv_type,p0", [(O.KV_Q8_0, 131072), (O.KV_Q4_0, 131072), (O.KV_F16, 131072), (O.KV_Q8_0, 262144), (O.KV_Q4_0, 262144)])
def test_decode_and_verify_at_depth(p1a, kv_type, p0):
    print(f"depth case: type {kv_type} p0 {p0}", flush=True)
    n = p0 + 4
    c, host = deep_cache(p1a, kv_type, n, 1000 + kv_type + p0 // 1024)
    q, _, _, gate = I.qkv(77 + kv_type, 1, 4, Hq, Hkv, D)
    dq, dg = dev(q), dev(gate)
    for T in (1, 4):
        pos = (p0 + np.arange(T)).astype(np.int32)
        ref = O.attn_rows(host, q[:T], pos, Hq, 1 / 16, gate=gate[:T])
        out = torch.zeros((T, Hq, D), device="cuda")
        p1a.attn_decode(dq[:T], c, out, T, p0, Hq, 1 / 16, gate=dg[:T])
        torch.cuda.synchronize()
        check(out.cpu().numpy(), ref, f"decode type {kv_type} p0 {p0} T {T}")
        out2 = torch.zeros_like(out)
        p1a.attn_decode_dev(dq[:T], c, out2, T, dev(pos[:1]), n, Hq, 1 / 16, gate=dg[:T])
        torch.cuda.synchronize()
        assert torch.equal(out, out2)                                   # device position == host position
        if T == 4:                                                       # T-invariance at this depth
            for t in range(4):
                one = torch.zeros((1, Hq, D), device="cuda")
                p1a.attn_decode(dq[t:t + 1], c, one, 1, p0 + t, Hq, 1 / 16, gate=dg[t:t + 1])
                torch.cuda.synchronize()
                assert torch.equal(one[0], out[t]), t


def hash32(x):
    x = x.astype(np.uint32)
    x ^= x >> np.uint32(16); x *= np.uint32(0x7feb352d); x ^= x >> np.uint32(15); x *= np.uint32(0x846ca68b); x ^= x >> np.uint32(16)
    return x


def fold_fill(n, seed, scale, Dh):
    """the fold test's generator (tests/fast_attn_fold_test.cu:20-27): value i = (three 16-bit uniforms summed / 65536 - 1.5)
    * scale, times 4 where (i % D) % 37 == 5"""
    with np.errstate(over="ignore"):
        i = np.arange(n, dtype=np.uint64)
        h1 = hash32((i * np.uint64(2654435761) + np.uint64(seed)) & np.uint64(0xffffffff))
        h2 = hash32(h1 + np.uint32(77))
        h3 = hash32(h2 + np.uint32(99))
    u = ((h1 & 0xffff).astype(np.float32) + (h2 & 0xffff).astype(np.float32) + (h3 & 0xffff).astype(np.float32)) / np.float32(65536.0) - np.float32(1.5)
    boost = np.where((i % Dh) % 37 == 5, np.float32(4.0), np.float32(1.0)).astype(np.float32)
    return (u * np.float32(scale) * boost).astype(np.float32)


@pytest.mark.parametrize("kv_type", [O.KV_F16, O.KV_Q8_0, O.KV_Q4_0])
def test_prefill_in_the_fold_tests_input_regime(p1a, kv_type):
    """peaked softmax (logits carried by seven outlier dims: standard deviation 1.5 to 2, a third of it from one dim) over
    32 K keys through the MFMA prefill and the decode kernel. The
    engine's own bar for f16 products in this regime is max|d| / max|ref| < 3e-2 and rms(d) / rms(ref) < 1e-2
    (tests/fast_attn_fold_test.cu:81-82); this path accumulates in fp32 and is held to its own bar here as well:
    max|d| <= 2e-3 max(1, max|ref|) and rel-L2 <= 1e-3."""
    hq, hkv, p0, T = 12, 2, 32768, 512
    n = p0 + T
    k = fold_fill(n * hkv * D, 1000, 1.0, D).reshape(n, hkv, D)
    v = fold_fill(n * hkv * D, 9000, 1.0, D).reshape(n, hkv, D)
    q = fold_fill(T * hq * D, 77 + p0, 2.0, D).reshape(T, hq, D)
    host = O.HostKV.contiguous(kv_type, n, hkv, D)
    O.kv_append_rows(host, k, v, np.arange(n))
    c = p1a.KVCache.contiguous(kv_type, n, hkv, D)
    for a in range(0, n, 8192):
        m = min(8192, n - a)
        p1a.kv_append(c, dev(k[a:a + m]), dev(v[a:a + m]), a, m)
    torch.cuda.synchronize()
    assert np.array_equal(c._keep[0].cpu().numpy(), host.k) and np.array_equal(c._keep[1].cpu().numpy(), host.v)
    pos = (p0 + np.arange(T)).astype(np.int32)
    ref = O.attn_rows(host, q, pos, hq, 1 / 16)
    logit_std = float(np.std((q[0, 0] @ k[:4096, 0].T) / 16))
    out = torch.zeros((T, hq, D), device="cuda")
    p1a.attn_prefill(dev(q), c, out, T, p0, hq, 1 / 16)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    ma, rl = I.errors(got, ref)
    mr = float(np.abs(ref).max())
    print(f"[parity] fold-regime prefill type {kv_type}: logit std {logit_std:.2f}, max|ref| {mr:.2f}, max_abs {ma:.2e}, rel_l2 {rl:.2e}")
    assert np.isfinite(got).all() and logit_std > 1.3
    assert ma <= 2e-3 * max(1.0, mr) and rl <= 1e-3, (ma, mr, rl)
    rows = np.arange(0, T, 61)
    dec = torch.zeros((len(rows), hq, D), device="cuda")
    for i, t in enumerate(rows):
        p1a.attn_decode(dev(q[t:t + 1]), c, dec[i:i + 1], 1, p0 + int(t), hq, 1 / 16)
    torch.cuda.synchronize()
    ma, rl = I.errors(dec.cpu().numpy(), ref[rows])
    print(f"[parity] fold-regime decode type {kv_type}: max_abs {ma:.2e}, rel_l2 {rl:.2e}")
    assert ma <= 2e-3 * max(1.0, mr) and rl <= 1e-3, (ma, mr, rl)
