"""The oracle's benchmark cache fill (the reference's kv_fill_random, src/fast/attn.cu:538-581). The reference holds no
vectors for it, so the values are pinned by what can be worked out without it: the two fixed points of the word hash, a
big-integer restatement written out step by step, the places and bits of the scale words, the value range, additivity over
position ranges, and paged == page by page contiguous with the page seeds."""
import numpy as np
import pytest

import _inputs as I
import _oracle as O

TYPES = [O.KV_F16, O.KV_Q8_0, O.KV_Q4_0]
MUL = 2654435761


def mix(w, seed):
    """the word hash with Python integers, one step per line"""
    h = ((w & 0xffffffff) * MUL) & 0xffffffff
    h ^= seed & 0xffffffff
    h ^= h >> 16
    h = (h * 0x7feb352d) & 0xffffffff
    h ^= h >> 15
    h = (h * 0x846ca68b) & 0xffffffff
    h ^= h >> 16
    return h


def words(a):
    return a.view(np.uint16)


def test_fixed_points_of_the_hash():
    """word 0 with seed 0, and word 1 with seed = the multiplier, both start from h = 0, which every step keeps: f16 -1.0
    in K and V, code bytes 0 in a quantized cache"""
    assert mix(0, 0) == 0 and mix(1, MUL) == 0
    for seed, w in [(0, 0), (MUL, 1)]:
        c = O.HostKV.contiguous(O.KV_F16, 4, 1, 64)
        O.kv_fill_random(c, 0, 4, seed)
        assert words(c.k)[w] == 0xBC00 and words(c.v)[w] == 0xBC00
        c = O.HostKV.contiguous(O.KV_Q8_0, 4, 1, 64)          # words 0, 1 of a head are its two scales: look at word 2 + w
        O.kv_fill_random(c, 0, 4, seed)
        assert mix(2 + w, seed) != 0
    # a code word that hashes to 0: word 3 = (seed 3 * MUL)
    c = O.HostKV.contiguous(O.KV_Q8_0, 4, 1, 64)
    O.kv_fill_random(c, 0, 4, (3 * MUL) & 0xffffffff)
    assert words(c.k)[3] == 0 and words(c.v)[3] == 0


@pytest.mark.parametrize("kv_type", TYPES)
def test_words_against_the_integer_restatement(kv_type):
    Hkv, D, n, seed = 2, 64, 9, 0x9e3779b9
    c = O.HostKV.contiguous(kv_type, n, Hkv, D)
    O.kv_fill_random(c, 0, n, seed)
    kw, vw = words(c.k), words(c.v)
    head_words = O.row_bytes(kv_type, Hkv, D) // Hkv // 2
    sc8 = int(np.float16(np.float32(1.0) / np.float32(127.0)).view(np.uint16))
    for w in range(len(kw)):
        h = mix(w, seed)
        hw = w % head_words
        if kv_type == O.KV_F16:
            a = int(np.float16(np.float32(h & 0xffff) / np.float32(32768.0) - np.float32(1.0)).view(np.uint16))
            b = int(np.float16(np.float32(h >> 16) / np.float32(32768.0) - np.float32(1.0)).view(np.uint16))
        elif kv_type == O.KV_Q8_0 and hw < D // 32:
            a = b = sc8
        elif kv_type == O.KV_Q4_0 and hw % 9 == 0:
            a = b = 0x3000                                     # f16 0.125
        else:
            a, b = h & 0xffff, h >> 16
        assert (int(kw[w]), int(vw[w])) == (a, b), w


def test_scales_and_ranges():
    n, Hkv, D = 33, 3, 256
    c = O.HostKV.contiguous(O.KV_Q8_0, n, Hkv, D)
    O.kv_fill_random(c, 0, n, 7)
    rows = c.k.reshape(n, Hkv, 272)
    assert np.all(rows[:, :, :16].copy().view(np.float16) == np.float16(1 / 127))          # 8 scales lead every head row
    assert len(np.unique(rows[:, :, 16:])) == 256                                          # codes: every byte value occurs
    c = O.HostKV.contiguous(O.KV_Q4_0, n, Hkv, D)
    O.kv_fill_random(c, 0, n, 7)
    blk = c.v.reshape(n, Hkv, 8, 18)
    assert np.all(blk[..., :2].copy().view(np.float16) == np.float16(0.125))                # ggml block_q4_0: scale, 16 bytes
    c = O.HostKV.contiguous(O.KV_F16, n, Hkv, D)
    O.kv_fill_random(c, 0, n, 7)
    x = c.k.view(np.float16).astype(np.float32)
    assert x.min() >= -1.0 and x.max() <= 1.0 and abs(float(x.mean())) < 0.01     # (values just under 1 round up to it)
    # a decode over such a cache sees finite values of order one
    assert np.all(np.isfinite(O.kv_read_head(c, 0, 0, 5, 1)))


@pytest.mark.parametrize("kv_type", TYPES)
def test_ranges_add_up_and_leave_the_rest_alone(kv_type):
    n, Hkv, D, seed = 40, 2, 64, 123
    whole = O.HostKV.contiguous(kv_type, n, Hkv, D)
    O.kv_fill_random(whole, 0, n, seed)
    parts = O.HostKV.contiguous(kv_type, n, Hkv, D)
    for a, b in [(25, 40), (0, 10), (10, 25), (5, 5), (9, 3)]:
        O.kv_fill_random(parts, a, b, seed)
    assert np.array_equal(parts.k, whole.k) and np.array_equal(parts.v, whole.v)
    rb = O.row_bytes(kv_type, Hkv, D)
    some = O.HostKV.contiguous(kv_type, n, Hkv, D)
    some.k[:] = 0xA5
    some.v[:] = 0x5A
    O.kv_fill_random(some, 7, 19, seed)
    assert np.all(some.k[:7 * rb] == 0xA5) and np.all(some.k[19 * rb:] == 0xA5) and np.all(some.v[19 * rb:] == 0x5A)
    assert np.array_equal(some.k[7 * rb:19 * rb], whole.k[7 * rb:19 * rb])


@pytest.mark.parametrize("kv_type", TYPES)
def test_paged_is_page_by_page_contiguous(kv_type):
    """logical page g of the sequence = a contiguous cache of one page filled with seed + g * 0x632be5ab, at the page's base"""
    Hkv, D, psh, n_pages, max_pages, seed = 2, 64, 3, 11, 5, 0xdeadbeef
    ps = 1 << psh
    table = I.rng(5).permutation(n_pages)[: 2 * max_pages].astype(np.int32)
    c = O.HostKV.paged(kv_type, Hkv, D, psh, n_pages, table, max_pages, n_layers=2, layer=1)
    c.pool[:] = 0x77
    seq = c.view(rtab=np.array([max_pages], np.int32))            # the second sequence's row of the table
    p0, p1 = 3, 29
    O.kv_fill_random(seq, p0, p1, seed)
    rb = O.row_bytes(kv_type, Hkv, D)
    touched = np.zeros(c.pool.size, bool)
    for g in range((p1 - 1) // ps + 1):
        a, b = max(p0, g * ps), min(p1, (g + 1) * ps)
        if a >= b:
            continue
        one = O.HostKV.contiguous(kv_type, ps, Hkv, D)
        O.kv_fill_random(one, a - g * ps, b - g * ps, (seed + g * 0x632be5ab) & 0xffffffff)
        base = int(table[max_pages + g]) * c.pstride
        lo, hi = (a - g * ps) * rb, (b - g * ps) * rb
        assert np.array_equal(c.k[base + lo:base + hi], one.k[lo:hi]), g
        assert np.array_equal(c.v[base + lo:base + hi], one.v[lo:hi]), g
        koff = c.k.ctypes.data - c.pool.ctypes.data
        voff = c.v.ctypes.data - c.pool.ctypes.data
        touched[koff + base + lo:koff + base + hi] = True
        touched[voff + base + lo:voff + base + hi] = True
    assert np.all(c.pool[~touched] == 0x77)                        # other layers, pages and positions: untouched
