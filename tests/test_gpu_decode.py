"""Decode / MTP-verify attention on the GPU (through the C ABI) vs the CPU oracle, plus the bitwise invariances the
reference engine tests: paged == contiguous, row t of a T-row call == the T = 1 call, rows == single, device p0 ==
host p0. Tolerance of the path: max-abs 2e-3, rel-L2 1e-3 vs the fp32 oracle."""
import numpy as np
import pytest
import torch

import _inputs as I
import _oracle as O
from _gpu import Pool, check, dev

pytestmark = pytest.mark.gpu
TYPES = [O.KV_F16, O.KV_Q8_0, O.KV_Q4_0]


def run_decode(p1a, c, q, T, p0, Hq, scale, gate=None):
    out = torch.full((T, Hq, c.D), float("nan"), device="cuda")
    p1a.attn_decode(dev(q), c, out, T, p0, Hq, scale, gate=None if gate is None else dev(gate))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_config1_tiny_f16(p1a):
    """1 sequence, 4 q heads / 1 kv head, D 64, ctx 512, f16 KV in 16-token pages, identity table, scale 1/8, seed 0"""
    Hq, Hkv, D, n = 4, 1, 64, 512
    pool = Pool(p1a, O.KV_F16, Hq, Hkv, D, 4, [n], seed=0, n_layers=1, layer=0, f16_inputs=True, shuffle=False, spare_pages=0)
    assert np.array_equal(pool.tabs[:32], np.arange(32))
    q, _, _, _ = I.qkv(0, n, 1, Hq, Hkv, D, f16_inputs=True)
    ref = O.attn_rows(pool.host_seq(0), q, np.array([n - 1]), Hq, 0.125)
    out = run_decode(p1a, pool.dev_seq(0), q, 1, n - 1, Hq, 0.125)
    check(out, ref, "config 1", flat=True)


@pytest.mark.parametrize("kv_type", TYPES)
def test_decode_vs_oracle_paged(p1a, kv_type):
    Hq, Hkv, D, psh = 24, 4, 256, 8
    lens = [3000, 700]
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, lens, seed=17)
    scale = 1.0 / 16.0
    for s, p0, T in [(0, 2999, 1), (0, 2045, 4), (1, 0, 1), (1, 255, 2), (1, 256, 3), (0, 31, 1), (0, 32, 1), (1, 696, 4)]:
        q, _, _, gate = I.qkv(1000 + p0, 1, T, Hq, Hkv, D)
        pos = p0 + np.arange(T, dtype=np.int32)
        ref = O.attn_rows(pool.host_seq(s), q, pos, Hq, scale, gate=gate)
        out = run_decode(p1a, pool.dev_seq(s), q, T, p0, Hq, scale, gate=gate)
        check(out, ref, f"type {kv_type} seq {s} p0 {p0} T {T}")


@pytest.mark.parametrize("kv_type", TYPES)
def test_bitwise_invariances(p1a, kv_type):
    Hq, Hkv, D, psh = 12, 2, 256, 5
    lens = [700, 1500, 300]
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, lens, seed=5, n_layers=2, layer=1)
    scale = 1.0 / 16.0
    q = I.normal(I.rng(77), (8, Hq, D)) * 1.5
    dq = dev(q)
    conts = [pool.dev_contiguous(s) for s in range(3)]
    # paged == contiguous and T-invariance, host p0 and device p0
    p0d = dev(np.array([0], np.int32))
    for s in range(3):
        for T in (1, 2, 3, 4, 7):
            for p0 in (0, 1, 31, 32, 127, 128, 255, 256, 257, 511, 600, lens[s] - T):
                if p0 < 0 or p0 + T > lens[s]:
                    continue
                a = torch.empty((T, Hq, D), device="cuda")
                b = torch.empty((T, Hq, D), device="cuda")
                d = torch.empty((T, Hq, D), device="cuda")
                p1a.attn_decode(dq, conts[s], a, T, p0, Hq, scale)
                p1a.attn_decode(dq, pool.dev_seq(s), b, T, p0, Hq, scale)
                p0d.fill_(p0)
                p1a.attn_decode_dev(dq, pool.dev_seq(s), d, T, p0d, lens[s], Hq, scale)
                assert torch.equal(a, b), (s, T, p0)
                assert torch.equal(a, d), (s, T, p0)
                for t in range(T):
                    one = torch.empty((1, Hq, D), device="cuda")
                    p1a.attn_decode(dq[t:t + 1], conts[s], one, 1, p0 + t, Hq, scale)
                    assert torch.equal(one[0], a[t]), (s, T, p0, t)
    # multi-row: rows of 3 sequences in one call == T = 1 per row on the contiguous caches
    sets = [
        [(0, 699)],
        [(0, 699), (1, 1499), (2, 299)],
        [(1, 1099), (0, 600), (1, 900), (2, 250), (1, 430)],
        [(0, 650), (0, 651), (1, 1496), (1, 1497), (1, 1498), (2, 100), (2, 101), (2, 102)],
        [(2, 0), (0, 0), (1, 255), (1, 256), (0, 31), (0, 32)],
    ]
    for rows in sets:
        T = len(rows)
        pos = dev(np.array([p for _, p in rows], np.int32))
        rt = dev(np.array([s * pool.maxp for s, _ in rows], np.int32))
        out = torch.empty((T, Hq, D), device="cuda")
        p1a.attn_decode_rows(dq, pool.devkv.with_rows(rt), out, T, pos, Hq, scale)
        for t, (s, p) in enumerate(rows):
            one = torch.empty((1, Hq, D), device="cuda")
            p1a.attn_decode(dq[t:t + 1], conts[s], one, 1, p, Hq, scale)
            assert torch.equal(one[0], out[t]), (rows, t)
    # verify blocks of several sequences sharing their KV read: 3 sequences x 2 rows
    rows = [(0, 650), (0, 651), (1, 1496), (1, 1497), (2, 100), (2, 101)]
    pos = dev(np.array([p for _, p in rows], np.int32))
    rt = dev(np.array([s * pool.maxp for s, _ in rows], np.int32))
    out = torch.empty((6, Hq, D), device="cuda")
    p1a.attn_decode_rows(dq, pool.devkv.with_rows(rt), out, 6, pos, Hq, scale, rows_per_seq=2)
    for t, (s, p) in enumerate(rows):
        one = torch.empty((1, Hq, D), device="cuda")
        p1a.attn_decode(dq[t:t + 1], conts[s], one, 1, p, Hq, scale)
        assert torch.equal(one[0], out[t]), ("blocks", t)


@pytest.mark.parametrize("kv_type", [O.KV_F16, O.KV_Q8_0])
def test_t_invariance_sweep(p1a, kv_type):
    """Row t of a T-row call == the T = 1 call at p0 + t, bit for bit, at every depth 0..300 and every 37th up to 4096
    (the sweep of the reference's tests/fast_tinv_test.cu:41-60: Hq 12 / Hkv 2), and device p0 == host p0"""
    Hq, Hkv, D, psh, n = 12, 2, 256, 6, 4100
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [n], seed=15, fill="device")
    k = I.normal(I.rng(16), (n, Hkv, D))
    v = I.normal(I.rng(17), (n, Hkv, D))
    c = pool.dev_seq(0)
    p1a.kv_append(c, dev(k), dev(v), 0, n)
    dq = dev(I.normal(I.rng(18), (4, Hq, D)))
    depths = list(range(0, 301)) + list(range(300, 4096, 37))
    singles = {}
    one = torch.empty((1, Hq, D), device="cuda")
    p0d = dev(np.array([0], np.int32))
    for p0 in depths:
        for T in (2, 3, 4):
            a = torch.empty((T, Hq, D), device="cuda")
            p1a.attn_decode(dq, c, a, T, p0, Hq, 1 / 16)
            if T == 4:
                b = torch.empty((T, Hq, D), device="cuda")
                p0d.fill_(p0)
                p1a.attn_decode_dev(dq, c, b, T, p0d, n, Hq, 1 / 16)
                assert torch.equal(a, b), ("device p0", p0)
            for t in range(T):
                key = (t, p0 + t)
                if key not in singles:
                    p1a.attn_decode(dq[t:t + 1], c, one, 1, p0 + t, Hq, 1 / 16)
                    singles[key] = one[0].clone()
                assert torch.equal(singles[key], a[t]), (T, p0, t)


def test_config3_batched_slots(p1a):
    """8 slots sharing one paged q8_0 pool, lengths log-uniform in [1024, 32768] (scaled down 8x here; test_gpu_full_size.py runs the full size), page tables interleaved, one row per slot"""
    Hq, Hkv, D, psh = 24, 4, 256, 8
    g = I.rng(33)
    lens = [int(np.exp(g.uniform(np.log(128), np.log(4096)))) for _ in range(8)]
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, psh, lens, seed=33)
    q, _, _, gate = I.qkv(34, 1, 8, Hq, Hkv, D)
    pos = np.array([n - 1 for n in lens], np.int32)
    rtab = np.array([s * pool.maxp for s in range(8)], np.int32)
    ref = O.attn_rows(pool.host.view(rtab=rtab), q, pos, Hq, 1 / 16, gate=gate)
    out = torch.empty((8, Hq, D), device="cuda")
    p1a.attn_decode_rows(dev(q), pool.devkv.with_rows(dev(rtab)), out, 8, dev(pos), Hq, 1 / 16, gate=dev(gate))
    check(out.cpu().numpy(), ref, "config 3 (reduced)")
    # a call this wide lets a workgroup walk several split streams; every row must still be bit for bit the row of a call
    # of its own (one stream per workgroup)
    for t in range(8):
        one = torch.empty((1, Hq, D), device="cuda")
        p1a.attn_decode_rows(dev(q[t:t + 1]), pool.devkv.with_rows(dev(rtab[t:t + 1])), one, 1, dev(pos[t:t + 1]), Hq, 1 / 16,
                             gate=dev(gate[t:t + 1]))
        assert torch.equal(one[0], out[t]), t


def test_repeated_calls_give_the_same_bits(p1a):
    """The same call repeated: bit-identical outputs every time (a page-table entry used before it had arrived once made
    one call in a few differ), single row and 8 slots of unequal depth"""
    Hq, Hkv, D, psh = 24, 4, 256, 8
    lens = [8133, 19168, 27213, 2861, 6076, 9552, 23094, 1075]
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, psh, lens, seed=81, fill="device")
    g = I.rng(82)
    for s_, n in enumerate(lens):
        c = pool.dev_seq(s_)
        p1a.kv_append(c, dev(I.normal(g, (n, Hkv, D))), dev(I.normal(g, (n, Hkv, D))), 0, n)
    dq = dev(I.normal(g, (8, Hq, D)))
    pos = dev(np.array([n - 1 for n in lens], np.int32))
    rt = dev(np.array([s_ * pool.maxp for s_ in range(8)], np.int32))
    cr = pool.devkv.with_rows(rt)
    ref8 = torch.empty((8, Hq, D), device="cuda")
    p1a.attn_decode_rows(dq, cr, ref8, 8, pos, Hq, 1 / 16)
    ref1 = torch.empty((1, Hq, D), device="cuda")
    p1a.attn_decode(dq[2:3], pool.dev_seq(2), ref1, 1, lens[2] - 1, Hq, 1 / 16)
    assert torch.equal(ref1[0], ref8[2])
    for rep in range(150):
        out8 = torch.full((8, Hq, D), float("nan"), device="cuda")
        p1a.attn_decode_rows(dq, cr, out8, 8, pos, Hq, 1 / 16)
        out1 = torch.full((1, Hq, D), float("nan"), device="cuda")
        p1a.attn_decode(dq[2:3], pool.dev_seq(2), out1, 1, lens[2] - 1, Hq, 1 / 16)
        assert torch.equal(out8, ref8), rep
        assert torch.equal(out1, ref1), rep


@pytest.mark.parametrize("kv_type", [O.KV_Q4_0, O.KV_Q8_0])
def test_config4_verify_blocks(p1a, kv_type):
    """MTP verify: 4 sequences x 4 rows (1 accepted + 3 drafts), causal inside the block, f16-rounded inputs; context
    reduced to 4096 here"""
    Hq, Hkv, D, psh, n = 24, 4, 256, 8, 4096
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [n] * 4, seed=44, f16_inputs=True)
    q, _, _, _ = I.qkv(45, 1, 16, Hq, Hkv, D, f16_inputs=True)
    pos = np.array([n - 4 + t for _ in range(4) for t in range(4)], np.int32)
    rtab = np.array([s * pool.maxp for s in range(4) for _ in range(4)], np.int32)
    ref = O.attn_rows(pool.host.view(rtab=rtab), q, pos, Hq, 1 / 16)
    out = torch.empty((16, Hq, D), device="cuda")
    p1a.attn_decode_rows(dev(q), pool.devkv.with_rows(dev(rtab)), out, 16, dev(pos), Hq, 1 / 16, rows_per_seq=4)
    check(out.cpu().numpy(), ref, "config 4 (reduced)")


@pytest.mark.parametrize("kv_type,Hq,Hkv,D,rows", [(O.KV_Q8_0, 24, 4, 256, 1), (O.KV_Q8_0, 24, 4, 256, 2), (O.KV_Q4_0, 24, 4, 256, 1),
                                                   (O.KV_Q4_0, 24, 4, 256, 2), (O.KV_F16, 32, 8, 128, 1), (O.KV_F16, 32, 8, 128, 2),
                                                   (O.KV_F16, 16, 4, 64, 4), (O.KV_Q8_0, 32, 4, 256, 2), (O.KV_F16, 24, 4, 256, 1),
                                                   (O.KV_F16, 24, 4, 256, 2)])
def test_two_workgroups_per_cu_variant(p1a, kv_type, Hq, Hkv, D, rows):
    """A call of two or more workgroups per CU with one column tile per row group runs a kernel variant with half the tile
    slots (two workgroups share a CU): 5 sequences of unequal depth (one shorter than a unit, one a single key), 1 ... 4 rows
    each, 6 ... 16 live columns - every row vs the oracle and bit for bit the row of a call of its own, which is small
    enough to take the other variant."""
    psh = 7
    lens = [2300, 37, 1, 900, 4100][:5]
    lens = [max(n, rows) for n in lens]
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, lens, seed=71)
    T = len(lens) * rows
    q, _, _, gate = I.qkv(72, 1, T, Hq, Hkv, D)
    pos = np.array([n - rows + t for n in lens for t in range(rows)], np.int32)
    rtab = np.array([s * pool.maxp for s in range(len(lens)) for _ in range(rows)], np.int32)
    ref = O.attn_rows(pool.host.view(rtab=rtab), q, pos, Hq, 1 / 16, gate=gate)
    out = torch.full((T, Hq, D), float("nan"), device="cuda")
    p1a.attn_decode_rows(dev(q), pool.devkv.with_rows(dev(rtab)), out, T, dev(pos), Hq, 1 / 16, gate=dev(gate), rows_per_seq=rows)
    check(out.cpu().numpy(), ref, f"{len(lens)} sequences x {rows} rows, GQA {Hq // Hkv}, D {D}")
    for t in range(T):
        one = torch.empty((1, Hq, D), device="cuda")
        p1a.attn_decode_rows(dev(q[t:t + 1]), pool.devkv.with_rows(dev(rtab[t:t + 1])), one, 1, dev(pos[t:t + 1]), Hq, 1 / 16,
                             gate=dev(gate[t:t + 1]))
        assert torch.equal(one[0], out[t]), t


@pytest.mark.parametrize("kv_type,Hq,Hkv,rows", [(O.KV_Q8_0, 16, 2, 4), (O.KV_Q4_0, 32, 2, 2), (O.KV_F16, 16, 2, 4), (O.KV_Q8_0, 14, 2, 4)])
def test_widest_row_groups(p1a, kv_type, Hq, Hkv, rows):
    """Row groups that fill both 16-column tiles (GQA 8 x 4 rows, GQA 16 x 2 rows: 32 live columns, the most the
    workgroup's Q table holds) and one that leaves the second tile ragged (GQA 7 x 4 rows = 28): each row vs the oracle,
    and bit for bit the row of a call of its own"""
    D, psh, n = 256, 6, 1500
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [n, n], seed=61)
    T = 2 * rows
    q, _, _, gate = I.qkv(62, 1, T, Hq, Hkv, D)
    pos = np.array([n - rows + t for _ in range(2) for t in range(rows)], np.int32)
    rtab = np.array([s * pool.maxp for s in range(2) for _ in range(rows)], np.int32)
    ref = O.attn_rows(pool.host.view(rtab=rtab), q, pos, Hq, 1 / 16, gate=gate)
    out = torch.empty((T, Hq, D), device="cuda")
    p1a.attn_decode_rows(dev(q), pool.devkv.with_rows(dev(rtab)), out, T, dev(pos), Hq, 1 / 16, gate=dev(gate), rows_per_seq=rows)
    check(out.cpu().numpy(), ref, f"row groups of {rows} x GQA {Hq // Hkv}")
    for t in range(T):
        one = torch.empty((1, Hq, D), device="cuda")
        p1a.attn_decode_rows(dev(q[t:t + 1]), pool.devkv.with_rows(dev(rtab[t:t + 1])), one, 1, dev(pos[t:t + 1]), Hq, 1 / 16,
                             gate=dev(gate[t:t + 1]))
        assert torch.equal(one[0], out[t]), t


def test_descriptor_n_ctx_only_bounds(p1a):
    """n_ctx of the descriptor is the caller's word; the kernel uses it to bound an early page-table read, never to pick a
    page: an understated (or missing) n_ctx gives the same bits"""
    Hq, Hkv, D, psh, n = 24, 4, 256, 5, 3000
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, psh, [n], seed=71)
    dq = dev(I.normal(I.rng(72), (2, Hq, D)))
    c = pool.dev_seq(0)
    ref = torch.empty((2, Hq, D), device="cuda")
    p1a.attn_decode(dq, c, ref, 2, n - 2, Hq, 1 / 16)
    for n_ctx in (0, 1, 64, 1000):
        c.n_ctx = n_ctx
        out = torch.empty((2, Hq, D), device="cuda")
        p1a.attn_decode(dq, c, out, 2, n - 2, Hq, 1 / 16)
        assert torch.equal(out, ref), n_ctx


def test_other_shapes_and_refusals(p1a):
    # GQA 4 / D 128 f16, GQA 8 / D 64 f16 (MFMA path), q8_0 at D 128 (generic path)
    for kv_type, Hq, Hkv, D in [(O.KV_F16, 8, 2, 128), (O.KV_F16, 8, 1, 64), (O.KV_Q8_0, 8, 2, 128), (O.KV_Q4_0, 6, 3, 96)]:
        pool = Pool(p1a, kv_type, Hq, Hkv, D, 6, [333], seed=D)
        q, _, _, gate = I.qkv(D + 1, 1, 2, Hq, Hkv, D)
        ref = O.attn_rows(pool.host_seq(0), q, np.array([330, 331], np.int32), Hq, 0.1, gate=gate)
        out = run_decode(p1a, pool.dev_seq(0), q, 2, 330, Hq, 0.1, gate=gate)
        check(out, ref, f"shape {kv_type} {Hq}/{Hkv}/{D}")
    pool = Pool(p1a, O.KV_F16, 4, 2, 64, 4, [64], seed=1)
    out = torch.full((1, 5, 64), 7.0, device="cuda")
    with pytest.raises(p1a.P1AError):
        p1a.attn_decode(out, pool.dev_seq(0), out, 1, 5, 5, 0.125)      # Hq not a multiple of Hkv
    torch.cuda.synchronize()
    assert torch.all(out == 7.0)                                        # refused: out untouched


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("low_keys", [(0, 1, 2, 3), (4, 5, 6, 7), (32, 33, 34, 35), tuple(range(0, 16)), tuple(k for k in range(64) if not k & 4)])
def test_row_maximum_spans_all_lanes(p1a, kv_type, low_keys):
    """A lane holds four keys of a column and the row maximum is taken across lanes. Keys whose scores sit 2^30 below the
    rest, placed so that they fill whole lanes (and whole 16-lane rows), must not become the reference of the exponentials:
    with the maximum of only a part of the lanes P would overflow f16. (The cross-lane exchange once dropped half of
    its result; softmax does not care which reference it is given until the exponentials leave the f16 range, which
    RMS-normed random keys never make them do.)"""
    Hq, Hkv, D, psh, n = 12, 2, 256, 6, 200
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [n], seed=81, fill="none")
    q, k, v, gate = I.qkv(82, n, 2, Hq, Hkv, D)
    scale = 1.0 / 16.0
    for hk, h in ((0, 1), (1, 9)):   # one q head of each kv head gets the low keys: k = -c q / |q|^2 scores -c exactly
        qh = q[0, h]
        for key in low_keys:
            k[key, hk] = -(30.0 / (scale * 1.4426950408889634)) * qh / float(qh @ qh)
    O.kv_append_rows(pool.host_seq(0), k, v, np.arange(n))
    p1a.kv_append(pool.dev_seq(0), dev(k), dev(v), 0, n)
    pos = np.array([n - 2, n - 1], np.int32)
    ref = O.attn_rows(pool.host_seq(0), q, pos, Hq, scale, gate=gate)
    out = run_decode(p1a, pool.dev_seq(0), q, 2, n - 2, Hq, scale, gate=gate)
    check(out, ref, f"low keys {low_keys[:4]}.. type {kv_type}")


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("shape", ["stairs_up", "stairs_down", "spikes"])
def test_moving_maxima_and_uniform_rows(p1a, kv_type, shape):
    """scores whose level changes by 2^10 from one 16-key tile to the next (up: every tile moves the reference maximum
    and rescales the accumulators; down: the exponentials of later tiles underflow; spikes: single keys 2^25 above the
    rest, scattered over waves and split streams), on top of ordinary random scores; and a query of zeros, whose row
    must be the plain mean of the visible V rows (closed form)"""
    Hq, Hkv, D, psh, n = 12, 2, 256, 6, 20000
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [n], seed=83, fill="none")
    q, k, v, gate = I.qkv(84, n, 3, Hq, Hkv, D)
    scale, l2e = 1.0 / 16.0, 1.4426950408889634
    tile = np.arange(n) // 16
    level = {"stairs_up": 10.0 * (tile % 8), "stairs_down": -10.0 * (tile % 8),
             "spikes": np.where((np.arange(n) * 2654435761 % 4093) < 3, 25.0, 0.0)}[shape]
    for hk, h in ((0, 2), (1, 7)):
        qh = q[0, h]
        k[:, hk] += (level / (scale * l2e))[:, None] * (qh / float(qh @ qh))[None, :]
    q[2] = 0.0                                                       # the uniform row
    O.kv_append_rows(pool.host_seq(0), k, v, np.arange(n))
    p1a.kv_append(pool.dev_seq(0), dev(k), dev(v), 0, n)
    pos = np.array([n - 3, n - 2, n - 1], np.int32)
    ref = O.attn_rows(pool.host_seq(0), q, pos, Hq, scale)
    out = run_decode(p1a, pool.dev_seq(0), q, 3, n - 3, Hq, scale)
    # (scores of magnitude 2^5 .. 2^6: the f16 rounding of q and k, 2^-11 relative, moves a score by a few hundredths and
    # an exponential by a few percent - three times the bound that holds for RMS-normed keys)
    check(out, ref, f"{shape} type {kv_type}", rel_l2_tol=3e-3)
    vmean = np.stack([O.kv_read_head(pool.host_seq(0), 1, 0, p, hk) for p in range(n) for hk in range(Hkv)]).reshape(n, Hkv, D).astype(np.float64).mean(0)
    for h in range(Hq):
        assert np.abs(out[2, h] - vmean[h // (Hq // Hkv)]).max() < 2e-4, h


def test_standalone_gate_equals_the_fused_one(p1a):
    """sigmoid_mul (the engine's k::sigmoid_mul launch behind attention) on an ungated decode == the decode with the gate
    fused into its merge, bit for bit (one formula); and against the oracle's gate, with the closed form g = 0 -> x 0.5"""
    Hq, Hkv, D, n = 12, 2, 256, 900
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, 6, [n], seed=97)
    q, _, _, gate = I.qkv(98, 1, 3, Hq, Hkv, D)
    gate[0, :64] = 0.0
    gate[1, :8] = [-200.0, 200.0, -90.0, 90.0, -30.0, 30.0, -1e-8, 1e-8]      # saturation and the flat middle
    dq, dg = dev(q), dev(gate)
    plain = torch.empty((3, Hq, D), device="cuda")
    fused = torch.empty((3, Hq, D), device="cuda")
    p1a.attn_decode(dq, pool.dev_seq(0), plain, 3, n - 3, Hq, 1 / 16)
    p1a.attn_decode(dq, pool.dev_seq(0), fused, 3, n - 3, Hq, 1 / 16, gate=dg)
    ungated = plain.cpu().numpy().copy()
    p1a.sigmoid_mul(plain, dg)
    torch.cuda.synchronize()
    assert torch.equal(plain, fused)
    want = ungated.reshape(3, -1).copy()
    O.gate(want, gate)
    got = plain.cpu().numpy().reshape(3, -1)
    assert np.all(np.isfinite(got))
    assert np.abs(got - want).max() <= 1e-6 * max(1.0, np.abs(want).max())
    assert np.array_equal(got[0, :64], 0.5 * ungated.reshape(3, -1)[0, :64])
    assert np.all(got[1, [0]] == 0.0 * ungated.reshape(3, -1)[1, [0]])       # sigmoid(-200) = 0: expf overflows to inf, 1 / inf = 0


@pytest.mark.parametrize("kv_type,Hq,Hkv,D", [(O.KV_Q8_0, 24, 4, 128), (O.KV_Q4_0, 24, 4, 128), (O.KV_Q8_0, 16, 2, 64),
                                              (O.KV_Q4_0, 8, 2, 64), (O.KV_Q8_0, 32, 2, 128)])
def test_staged_tiles_for_small_heads(p1a, kv_type, Hq, Hkv, D):
    """q8_0 / q4_0 head rows at D = 64 or 128 are not whole 16-byte chunks; their raw tiles are fetched 4 bytes per lane,
    converted to f16 tiles by the wave that owns them and multiplied on the matrix pipe like an f16 cache (the reference
    refuses these shapes, src/fast/attn_dec2.cu:493). Every depth class against the oracle - one key, a ragged last tile,
    a tile boundary, several units - for 1 ... 4 rows (one and two column tiles); and the identities the D = 256 kernels keep:
    paged == contiguous, row t of a T-row call == the T = 1 call, batched rows == single, all bit for bit."""
    psh, n = 5, 2100
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [n, 700], seed=300 + D)
    cont = pool.dev_contiguous(0)
    scale = 1.0 / np.sqrt(D)
    for T, p0 in ((1, 0), (1, 14), (1, 15), (1, 16), (2, 255), (3, 511), (4, 1000), (1, n - 1), (4, n - 4)):
        q, _, _, gate = I.qkv(400 + T + p0, 1, T, Hq, Hkv, D)
        ref = O.attn_rows(pool.host_seq(0), q, (p0 + np.arange(T)).astype(np.int32), Hq, scale, gate=gate)
        out = run_decode(p1a, pool.dev_seq(0), q, T, p0, Hq, scale, gate=gate)
        check(out, ref, f"staged {kv_type} {Hq}/{Hkv}/{D} T {T} p0 {p0}")
        assert np.array_equal(out, run_decode(p1a, cont, q, T, p0, Hq, scale, gate=gate)), (T, p0)      # paged == contiguous
        for t in range(T):                                                                               # row t == the T = 1 call
            one = run_decode(p1a, pool.dev_seq(0), q[t:t + 1], 1, p0 + t, Hq, scale, gate=gate[t:t + 1])
            assert np.array_equal(one[0], out[t]), (T, p0, t)
    # rows of two sequences in one call == each on its own
    pos = np.array([n - 1, 699, 1234, 5], np.int32)
    rtab = np.array([0, pool.maxp, 0, pool.maxp], np.int32)
    q, _, _, gate = I.qkv(499, 1, 4, Hq, Hkv, D)
    ref = O.attn_rows(pool.host.view(rtab=rtab), q, pos, Hq, scale, gate=gate)
    out = torch.empty((4, Hq, D), device="cuda")
    p1a.attn_decode_rows(dev(q), pool.devkv.with_rows(dev(rtab)), out, 4, dev(pos), Hq, scale, gate=dev(gate))
    check(out.cpu().numpy(), ref, f"staged {kv_type} batched rows")
    for t in range(4):
        one = run_decode(p1a, pool.dev_seq(int(rtab[t] // pool.maxp)), q[t:t + 1], 1, int(pos[t]), Hq, scale, gate=gate[t:t + 1])
        assert np.array_equal(one[0], out[t].cpu().numpy()), t
