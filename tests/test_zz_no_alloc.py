"""The allocation-free decode entry point (p1a_attn_decode_noalloc: split partials in a fixed array of device memory,
no hipMalloc / hipFree ever) against the entry point it is a variant of (p1a_attn_decode_a16), through the C ABI: the
same output and a16 bytes on two calls in a row, the second with a smaller input; oversized calls are refused."""
import ctypes

import numpy as np
import pytest
import torch

import _inputs as I
import _oracle as O
from _gpu import Pool, check, dev

pytestmark = pytest.mark.gpu


def ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def call(L, fn, q, c, out, gate, qbuf, T, p0, Hq, pos=None, rows_per_seq=0):
    return getattr(L, fn)(ptr(q), ctypes.byref(c.struct()), ptr(out), ptr(gate), ptr(qbuf), T, p0, None, ptr(pos), rows_per_seq, Hq,
                          ctypes.c_float(1 / 16), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))


@pytest.mark.parametrize("kv_type", [O.KV_Q8_0, O.KV_Q4_0, O.KV_F16])
def test_noalloc_equals_decode_on_two_calls_in_a_row(p1a, kv_type):
    L = p1a.lib()
    Hq, Hkv, D, psh = 24, 4, 256, 8
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [5000, 300], seed=500 + kv_type)
    # call 1: 8 rows (two 4-row verify blocks would need rows_per_seq; here one sequence) at depth 5000; call 2: one row at depth 300
    for T, sq, n in ((8, 0, 5000), (1, 1, 300)):
        q, _, _, gate = I.qkv(510 + T, 1, T, Hq, Hkv, D)
        dq, dg = dev(q), dev(gate)
        c = pool.dev_seq(sq)
        want, got = torch.zeros((T, Hq, D), device="cuda"), torch.full((T, Hq, D), float("nan"), device="cuda")
        qb1 = torch.zeros(p1a.a16_bytes(T, Hq * D) // 2, dtype=torch.int16, device="cuda")
        qb2 = torch.zeros_like(qb1)
        assert call(L, "p1a_attn_decode_a16", dq, c, want, dg, qb1, T, n - T, Hq) == 0
        assert call(L, "p1a_attn_decode_noalloc", dq, c, got, dg, qb2, T, n - T, Hq) == 0, L.p1a_last_error()
        torch.cuda.synchronize()
        assert torch.equal(want, got), (T, n)
        assert torch.equal(qb1, qb2), (T, n)
        ref = O.attn_rows(pool.host_seq(sq), q, (n - T + np.arange(T)).astype(np.int32), Hq, 1 / 16, gate=gate)
        check(got.cpu().numpy(), ref, f"noalloc decode type {kv_type} T {T} depth {n}")


def test_noalloc_rows_of_several_sequences_and_refusal(p1a):
    L = p1a.lib()
    Hq, Hkv, D, psh = 24, 4, 256, 8
    lens = [3000, 1200]
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, psh, lens, seed=520)
    R = 4
    q, _, _, gate = I.qkv(521, 1, 2 * R, Hq, Hkv, D)
    pos = dev(np.array([n - R + t for n in lens for t in range(R)], np.int32))
    rt = dev(np.array([s * pool.maxp for s in range(2) for _ in range(R)], np.int32))
    c = pool.devkv.with_rows(rt)
    dq, dg = dev(q), dev(gate)
    want, got = torch.zeros((2 * R, Hq, D), device="cuda"), torch.zeros((2 * R, Hq, D), device="cuda")
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        assert call(L, "p1a_attn_decode_a16", dq, c, want, dg, None, 2 * R, 0, Hq, pos=pos, rows_per_seq=R) == 0
        assert call(L, "p1a_attn_decode_noalloc", dq, c, got, dg, None, 2 * R, 0, Hq, pos=pos, rows_per_seq=R) == 0
        s.synchronize()
    assert torch.equal(want, got)
    # 32 rows of this shape need 50 MB of partials: more than the fixed array holds - refused, nothing launched
    q32 = torch.zeros((32, Hq, D), device="cuda")
    o32 = torch.full((32, Hq, D), 7.0, device="cuda")
    assert call(L, "p1a_attn_decode_noalloc", q32, pool.dev_seq(0), o32, None, None, 32, 100, Hq) == -3
    assert b"static buffer" in L.p1a_last_error()
    torch.cuda.synchronize()
    assert bool((o32 == 7.0).all())
