"""Chunked causal prefill on the GPU (through the C ABI) vs the CPU oracle: append the chunk (codes bit-exact), then
attention with the fused gate. Tolerance of the path: max-abs 2e-3, rel-L2 1e-3 vs the fp32 oracle."""
import numpy as np
import pytest
import torch

import _inputs as I
import _oracle as O
from _gpu import Pool, check, dev

pytestmark = pytest.mark.gpu
TYPES = [O.KV_F16, O.KV_Q8_0, O.KV_Q4_0]


def run_prefill(p1a, c, q, T, p0, Hq, scale, gate=None):
    out = torch.full((T, Hq, c.D), float("nan"), device="cuda")
    p1a.attn_prefill(dev(q), c, out, T, p0, Hq, scale, gate=None if gate is None else dev(gate))
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("p0,T", [(0, 1), (0, 200), (37, 100), (300, 129), (1000, 260)])
def test_prefill_vs_oracle(p1a, kv_type, p0, T):
    Hq, Hkv, D, psh = 12, 2, 256, 5
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [p0 + T, 50], seed=7 + p0, n_layers=2, layer=1)
    q, _, _, gate = I.qkv(500 + T, 1, T, Hq, Hkv, D, f16_inputs=True)
    pos = p0 + np.arange(T, dtype=np.int32)
    ref = O.attn_rows(pool.host_seq(0), q, pos, Hq, 1 / 16, gate=gate)
    out = run_prefill(p1a, pool.dev_seq(0), q, T, p0, Hq, 1 / 16, gate=gate)
    check(out, ref, f"prefill type {kv_type} p0 {p0} T {T}")


@pytest.mark.parametrize("kv_type,Hq,Hkv,D,psh", [(O.KV_F16, 4, 1, 64, 4), (O.KV_Q8_0, 8, 2, 128, 6), (O.KV_Q4_0, 4, 2, 64, 8), (O.KV_F16, 6, 1, 128, 7)])
def test_other_shapes(p1a, kv_type, Hq, Hkv, D, psh):
    p0, T = 100, 150
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [p0 + T], seed=D + psh)
    q, _, _, _ = I.qkv(D, 1, T, Hq, Hkv, D)
    pos = p0 + np.arange(T, dtype=np.int32)
    ref = O.attn_rows(pool.host_seq(0), q, pos, Hq, 0.1)
    out = run_prefill(p1a, pool.dev_seq(0), q, T, p0, Hq, 0.1)
    check(out, ref, f"prefill shape {kv_type} {Hq}/{Hkv}/{D} psh {psh}")
    # contiguous cache gives the same bits as the paged one
    out2 = run_prefill(p1a, pool.dev_contiguous(0), q, T, p0, Hq, 0.1)
    assert np.array_equal(out, out2)


def test_config5_append_then_prefill_reduced(p1a):
    """config 5 at 1/8 scale: 3584 tokens already in q8_0 pages, a 512-token chunk is quantized on append (codes
    bit-exact vs the oracle), then causal attention with the fused gate"""
    Hq, Hkv, D, psh, p0, T = 24, 4, 256, 8, 3584, 512
    pool = Pool(p1a, O.KV_Q8_0, Hq, Hkv, D, psh, [p0 + T], seed=55, f16_inputs=False, fill="none")
    k, v = pool.k[0], pool.v[0]
    O.kv_append_rows(pool.host_seq(0), k, v, np.arange(p0 + T))
    c = pool.dev_seq(0)
    p1a.kv_append(c, dev(k[:p0]), dev(v[:p0]), 0, p0)           # history
    p1a.kv_append(c, dev(k[p0:]), dev(v[p0:]), p0, T)           # the chunk's own K/V, before attention
    torch.cuda.synchronize()
    assert np.array_equal(pool.dpool.cpu().numpy(), pool.host.pool)
    q, _, _, gate = I.qkv(56, 1, T, Hq, Hkv, D, f16_inputs=True)
    rows = np.array([0, 1, 127, 128, 255, 300, 511])               # oracle on a sample of the rows
    ref = O.attn_rows(pool.host_seq(0), q[rows], (p0 + rows).astype(np.int32), Hq, 1 / 16, gate=gate[rows])
    out = run_prefill(p1a, c, q, T, p0, Hq, 1 / 16, gate=gate)
    assert np.all(np.isfinite(out))
    check(out[rows], ref, "config 5 (reduced)")


@pytest.mark.parametrize("kv_type", TYPES)
def test_prefill_rows_match_decode(p1a, kv_type):
    """mirror of the reference's prefill-vs-decode test: every prefill row is the decode result at its position
    (both paths round Q, K, V and P to f16 once, so they agree far inside the tolerance)"""
    Hq, Hkv, D, psh, p0, T = 12, 2, 256, 8, 700, 140
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [p0 + T], seed=91)
    q, _, _, _ = I.qkv(92, 1, T, Hq, Hkv, D)
    out = run_prefill(p1a, pool.dev_seq(0), q, T, p0, Hq, 1 / 16)
    dq = dev(q)
    dec = torch.empty((T, Hq, D), device="cuda")
    for t0 in range(0, T, 4):
        n = min(4, T - t0)
        p1a.attn_decode(dq[t0:t0 + n], pool.dev_seq(0), dec[t0:t0 + n], n, p0 + t0, Hq, 1 / 16)
    torch.cuda.synchronize()
    ma, rl = I.errors(out, dec.cpu().numpy())
    assert ma < 1e-3 and rl < 5e-4, (ma, rl)


@pytest.mark.parametrize("kv_type", [O.KV_Q8_0, O.KV_Q4_0])
@pytest.mark.parametrize("Hq,Hkv,D,psh", [(12, 2, 256, 5), (8, 2, 128, 4)])
def test_scratch_variant_gives_the_same_bits(p1a, kv_type, Hq, Hkv, D, psh):
    """with scratch - the caller's, or the library's own staging copy when the caller brings none - the quantized cache is
    converted to f16 once and the f16 kernel runs on the copy: same tiles, same products, same bits as the on-the-fly
    kernel (staging limit 0); a caller scratch that is too small silently takes the library's copy or the direct kernel"""
    p0, T = 777, 300
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [p0 + T, 40], seed=3 + psh, n_layers=2, layer=0)
    q, _, _, gate = I.qkv(70 + D, 1, T, Hq, Hkv, D, f16_inputs=True)
    p1a.set_prefill_staging_limit(0)                                   # no staging copy anywhere: dequantization in the kernel
    try:
        direct = run_prefill(p1a, pool.dev_seq(0), q, T, p0, Hq, 1 / 16, gate=gate)
    finally:
        p1a.set_prefill_staging_limit(1 << 30)
    a = run_prefill(p1a, pool.dev_seq(0), q, T, p0, Hq, 1 / 16, gate=gate)      # the library's own staging copy
    assert np.array_equal(a, direct)
    need = p1a.prefill_scratch_bytes(T, p0, Hq, Hkv, D)
    stage = 2 * ((p0 + T + 15) // 16 * 16) * Hkv * D * 2               # whole 16-key groups of f16 rows, K and V
    ks = p1a.prefill_key_splits(T, p0, Hq)                            # (this shape is split over the keys)
    r256 = lambda x: (x + 255) // 256 * 256
    assert need == r256(stage) + (r256(T * Hq * ks * 8) + T * Hq * ks * D * 4 if ks > 1 else 0)
    dq, dg = dev(q), dev(gate)
    for nbytes in (need, r256(stage), stage // 2):                    # everything fits / the copy only / nothing
        scr = torch.full((nbytes,), 0xff, dtype=torch.uint8, device="cuda")   # (what the copy does not write is NaN)
        out = torch.zeros((T, Hq, D), device="cuda")
        p1a.attn_prefill(dq, pool.dev_seq(0), out, T, p0, Hq, 1 / 16, gate=dg, scratch=scr)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), a), nbytes


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("p0,T", [(0, 37), (50, 130), (128, 1)])
def test_rows_past_the_last_position_are_never_weighted(p1a, kv_type, p0, T):
    """whatever lies in the cache past the last position - here NaN / Inf bit patterns - must not reach the output (the
    kernels may fetch such rows with a tile; they must not let them count)"""
    Hq, Hkv, D, psh = 12, 2, 256, 6
    n = p0 + T
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [n, 40], seed=41, n_layers=1, layer=0)
    q, _, _, gate = I.qkv(91, 1, T, Hq, Hkv, D, f16_inputs=True)
    want = O.attn_rows(pool.host_seq(0), q, np.arange(p0, p0 + T), Hq, 1 / 16, gate=gate)
    # poison every row of the sequence's last page past position n - 1, K and V
    c = pool.dev_seq(0)
    rb = O.row_bytes(kv_type, Hkv, D)
    ps = 1 << psh
    page = int(pool.tabs[(n - 1) >> psh])
    first = ((n - 1) & (ps - 1)) + 1
    if first < ps:
        for base in (0, ps * rb):                                  # K block, V block of the page (one layer)
            o = page * c.pstride + base + first * rb
            pool.dpool[o:o + (ps - first) * rb] = 0xff if kv_type != O.KV_F16 else 0x7e
    out = run_prefill(p1a, c, q, T, p0, Hq, 1 / 16, gate=gate)
    assert np.isfinite(out).all()
    ma, rl = I.errors(out, want)
    assert ma < 2e-3 and rl < 1e-3, (ma, rl)
    scr = torch.full((p1a.prefill_scratch_bytes(T, p0, Hq, Hkv, D),), 0xff, dtype=torch.uint8, device="cuda")
    out2 = torch.full((T, Hq, D), float("nan"), device="cuda")
    p1a.attn_prefill(dev(q), c, out2, T, p0, Hq, 1 / 16, gate=dev(gate), scratch=scr)
    torch.cuda.synchronize()
    assert np.array_equal(out2.cpu().numpy(), out)


def test_f16_contiguous_and_small_pages_take_the_same_bits(p1a):
    """f16, D = 256: a contiguous cache that ends right behind the last position (whole 16-key groups cannot be fetched:
    the register-staged kernel runs), one with room (tiles loaded straight into LDS) and 16-position pages must agree
    bit for bit, and with the oracle within the tolerance"""
    Hq, Hkv, D, p0, T = 12, 2, 256, 203, 170
    n = p0 + T                                                 # 373: not a multiple of 16
    q, k, v, gate = I.qkv(55, n, T, Hq, Hkv, D, f16_inputs=True)
    host = O.HostKV.contiguous(O.KV_F16, n, Hkv, D)
    O.kv_append_rows(host, k, v, np.arange(n))
    want = O.attn_rows(host.view(), q, np.arange(p0, n), Hq, 1 / 16, gate=gate)
    outs = []
    for n_ctx in (n, n + 40):
        c = p1a.KVCache.contiguous(O.KV_F16, n_ctx, Hkv, D)
        p1a.kv_append(c, dev(k), dev(v), 0, n)
        outs.append(run_prefill(p1a, c, q, T, p0, Hq, 1 / 16, gate=gate))
    pool = Pool(p1a, O.KV_F16, Hq, Hkv, D, 4, [n, 30], seed=55, n_layers=2, layer=1, fill="none")
    c = pool.dev_seq(0)
    p1a.kv_append(c, dev(k), dev(v), 0, n)
    outs.append(run_prefill(p1a, c, q, T, p0, Hq, 1 / 16, gate=gate))
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    ma, rl = I.errors(outs[0], want)
    assert ma < 2e-3 and rl < 1e-3, (ma, rl)


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("Hq,Hkv,D,p0,T", [(4, 1, 256, 6000, 100), (6, 2, 256, 9000, 260), (8, 2, 128, 5000, 70), (24, 4, 256, 12000, 33),
                                                 (2, 1, 256, 0, 2048)])   # (the first token blocks see fewer tiles than there are splits)
def test_key_split_chunks(p1a, kv_type, Hq, Hkv, D, p0, T):
    """a short chunk over a long context is split over the keys (several workgroups per token block and head, partials
    merged): against the oracle; every 7th row against the decode kernel at its position; and the same bits wherever the
    partials live (caller scratch, the library's buffers) and whatever else is in flight before"""
    ks = p1a.prefill_key_splits(T, p0, Hq)
    assert ks > 1, ks
    psh = 6
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [p0 + T], seed=p0 + T)
    q, _, _, gate = I.qkv(p0, 1, T, Hq, Hkv, D, f16_inputs=True)
    pos = p0 + np.arange(T, dtype=np.int32)
    ref = O.attn_rows(pool.host_seq(0), q, pos, Hq, 1 / 16, gate=gate)
    c = pool.dev_seq(0)
    out = run_prefill(p1a, c, q, T, p0, Hq, 1 / 16, gate=gate)
    check(out, ref, f"key-split prefill type {kv_type} {Hq}/{Hkv}/{D} p0 {p0} T {T} splits {ks}")
    dq, dg = dev(q), dev(gate)
    need = p1a.prefill_scratch_bytes(T, p0, Hq, Hkv, D)
    for nbytes in (need, need - 256, 4096):
        scr = torch.full((nbytes,), 0xff, dtype=torch.uint8, device="cuda")
        o2 = torch.zeros((T, Hq, D), device="cuda")
        p1a.attn_prefill(dq, c, o2, T, p0, Hq, 1 / 16, gate=dg, scratch=scr)
        torch.cuda.synchronize()
        assert np.array_equal(o2.cpu().numpy(), out), nbytes
    for t in range(0, T, 7 if T < 1000 else 97):
        one = torch.zeros((1, Hq, D), device="cuda")
        p1a.attn_decode(dq[t:t + 1], c, one, 1, p0 + t, Hq, 1 / 16, gate=dg[t:t + 1])
        ma, rl = I.errors(one.cpu().numpy()[0], out[t])
        assert ma < 2e-3 and rl < 1e-3, (t, ma, rl)


def test_key_split_plan():
    """the split count is a function of the shape and the device only: none for chunks that fill the device or contexts too
    short to share out, several for a short chunk over a long context; the scratch size says what it holds"""
    import importlib
    p1a = importlib.import_module("p100e-engine_amd")
    assert p1a.prefill_key_splits(4096, 28672, 24) == 1             # the benchmark chunk: 768 workgroups already
    assert p1a.prefill_key_splits(128, 0, 24) == 1                  # two tiles: nothing to share out
    assert p1a.prefill_key_splits(64, 511, 4) == 1                  # splits of fewer than 8 tiles are not worth their set-up
    assert p1a.prefill_key_splits(128, 32640, 24) >= 8
    assert p1a.prefill_key_splits(512, 32256, 24) >= 2
    for T, p0, Hq in [(128, 32640, 24), (33, 12000, 24), (300, 777, 12)]:
        ks = p1a.prefill_key_splits(T, p0, Hq)
        assert (p0 + T - 1) // 64 + 1 >= 8 * ks or ks == 1


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("which", ["lower_lane_everywhere", "lower_half", "upper_half", "first_32", "all_but_one"])
def test_row_maximum_spans_both_lane_halves(p1a, kv_type, which):
    """the two lanes of a query row each hold 16 keys of a 32-key half tile (keys with bit 2 clear / set) and the row
    maximum is taken across them: keys scoring 2^30 below the rest and filling one lane's share must not become the
    reference of the exponentials (P would leave the f16 range)"""
    Hq, Hkv, D, psh, p0, T = 4, 1, 256, 6, 130, 70
    n = p0 + T
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [n], seed=91, fill="none")
    q, k, v, gate = I.qkv(92, n, T, Hq, Hkv, D, f16_inputs=True)
    low = {"lower_lane_everywhere": [x for x in range(n) if not x & 4], "lower_half": [x for x in range(128) if not x & 4], "upper_half": [x for x in range(128) if x & 4],
           "first_32": list(range(32)), "all_but_one": [x for x in range(128) if x != 77]}[which]
    # the rows of head 2 share a direction (plus their own noise), and the low keys point against it: every row of that
    # head scores them about 30 (in powers of two) below zero, the other heads see them as ordinary keys
    qh = q[0, 2].copy()
    q[:, 2] = (qh[None, :] + 0.3 * q[:, 2]).astype(np.float16).astype(np.float32)
    for key in low:
        k[key, 0] = -(30.0 / (0.1 * 1.4426950408889634)) * qh / float(qh @ qh)
    O.kv_append_rows(pool.host_seq(0), k, v, np.arange(n))
    p1a.kv_append(pool.dev_seq(0), dev(k), dev(v), 0, n)
    pos = p0 + np.arange(T, dtype=np.int32)
    ref = O.attn_rows(pool.host_seq(0), q, pos, Hq, 0.1, gate=gate)
    out = run_prefill(p1a, pool.dev_seq(0), q, T, p0, Hq, 0.1, gate=gate)
    check(out, ref, f"prefill low keys {which} type {kv_type}")


@pytest.mark.parametrize("kv_type", TYPES)
@pytest.mark.parametrize("shape", ["stairs_up", "stairs_down", "spikes"])
def test_moving_maxima(p1a, kv_type, shape):
    """scores whose level changes by 2^10 from one 64-key tile to the next (up: every tile moves the reference maximum of
    every row and rescales both waves' accumulators; down: later exponentials underflow), or single keys 2^25 above the
    rest, on top of ordinary random scores; rows of one head share a direction so that the levels hold for all of them"""
    Hq, Hkv, D, psh, p0, T = 4, 1, 256, 6, 1500, 200
    n = p0 + T
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, [n], seed=93, fill="none")
    q, k, v, gate = I.qkv(94, n, T, Hq, Hkv, D, f16_inputs=True)
    qh = q[0, 1].copy()
    q[:, 1] = (qh[None, :] + 0.3 * q[:, 1]).astype(np.float16).astype(np.float32)
    tile = np.arange(n) // 64
    level = {"stairs_up": 10.0 * (tile % 6), "stairs_down": -10.0 * (tile % 6),
             "spikes": np.where((np.arange(n) * 2654435761 % 509) < 3, 25.0, 0.0)}[shape]
    k[:, 0] += (level / (0.1 * 1.4426950408889634))[:, None] * (qh / float(qh @ qh))[None, :]
    O.kv_append_rows(pool.host_seq(0), k, v, np.arange(n))
    p1a.kv_append(pool.dev_seq(0), dev(k), dev(v), 0, n)
    pos = p0 + np.arange(T, dtype=np.int32)
    ref = O.attn_rows(pool.host_seq(0), q, pos, Hq, 0.1, gate=gate)
    out = run_prefill(p1a, pool.dev_seq(0), q, T, p0, Hq, 0.1, gate=gate)
    # (scores of magnitude 2^5 .. 2^6: the f16 rounding of q and k, 2^-11 relative, moves a score by a few hundredths and
    # an exponential by a few percent - three times the bound that holds for RMS-normed keys)
    check(out, ref, f"prefill {shape} type {kv_type}", rel_l2_tol=3e-3)


@pytest.mark.parametrize("kv_type", TYPES)
def test_sequence_selected_through_the_row_table(p1a, kv_type):
    """one sequence per prefill call: its page table is pt + rtab[0] when the descriptor carries a row table (how a batched
    descriptor of the engine names a slot), the same bits as the descriptor whose pt already points at the slot's row; the
    benchmark fill follows the same rule"""
    Hq, Hkv, D, psh = 12, 2, 256, 5
    lens = [300, 700, 90]
    pool = Pool(p1a, kv_type, Hq, Hkv, D, psh, lens, seed=131)
    sq, T = 1, 180
    p0 = lens[sq] - T
    q, _, _, gate = I.qkv(132, 1, T, Hq, Hkv, D, f16_inputs=True)
    a = run_prefill(p1a, pool.dev_seq(sq), q, T, p0, Hq, 1 / 16, gate=gate)
    rt = dev(np.array([sq * pool.maxp, 0, 0], np.int32))
    b = run_prefill(p1a, pool.devkv.with_rows(rt), q, T, p0, Hq, 1 / 16, gate=gate)
    assert np.array_equal(a, b)
    ref = O.attn_rows(pool.host_seq(sq), q, p0 + np.arange(T, dtype=np.int32), Hq, 1 / 16, gate=gate)
    check(b, ref, f"prefill through the row table, type {kv_type}")
    O.kv_fill_random(pool.host.view(rtab=np.array([sq * pool.maxp], np.int32)), 10, 600, 5)
    p1a.kv_fill_random(pool.devkv.with_rows(rt), 10, 600, 5)
    torch.cuda.synchronize()
    assert np.array_equal(pool.dpool.cpu().numpy(), pool.host.pool)
