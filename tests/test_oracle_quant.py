"""Pins the oracle's quantizers and f16 conversions: golden vectors from the reference's own ggml C code,
closed forms, and exhaustive comparison with numpy's IEEE float16."""
import os

import numpy as np
import pytest

import _oracle as O

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "quant_golden.npz"))


def test_f16_to_f32_exhaustive():
    L = O.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([L.orc_f16_to_f32(int(b)) for b in bits], np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    assert np.all(np.isnan(got[np.isnan(ref)]))


def test_f32_to_f16_rne():
    L = O.lib()
    g = np.random.Generator(np.random.Philox(7))
    # random bit patterns (all exponents), every half and every midpoint between adjacent halves
    x = g.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    halves = np.arange(0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mids = ((halves[:-1].astype(np.float64) + halves[1:].astype(np.float64)) / 2).astype(np.float32)
    near = np.concatenate([np.nextafter(mids, np.float32(0)), mids, np.nextafter(mids, np.float32(1e9))])
    edge = np.array([65504, 65519.99, 65520, 65536, 1e9, np.inf, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26, 0.0], np.float32)
    x = np.concatenate([x, halves, near, -near, edge, -edge])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_f32_to_f16(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, ref)


def test_q8_0_matches_reference_ggml():
    d, q = O.quant_q8_0(GOLD["x"])
    assert np.array_equal(d, GOLD["q8_d"])
    assert np.array_equal(q, GOLD["q8_q"])


def test_q4_0_matches_reference_ggml():
    b = O.quant_q4_0(GOLD["x"])
    assert np.array_equal(b, GOLD["q4_blk"])


def test_closed_forms():
    z = np.zeros((1, 32), np.float32)
    d, q = O.quant_q8_0(z)
    assert d[0] == 0 and not q.any()
    b = O.quant_q4_0(z)
    # d = +0 / -8 = -0 (sign bit kept, as in the reference's C); every code (int)(0 + 8.5) = 8
    assert b[0, 0] == 0 and b[0, 1] == 0x80 and np.all(b[0, 2:] == 0x88)
    x = np.zeros((2, 32), np.float32)
    x[0, 7], x[1, 7] = 3.25, -3.25
    d, q = O.quant_q8_0(x)
    assert q[0, 7] == 127 and q[1, 7] == -127                                   # the amax element is +-127 exactly
    b = O.quant_q4_0(x)
    for r in range(2):                                                          # the max element maps to nibble 0
        assert (b[r, 2 + 7] & 15) == 0
    x = np.zeros((2, 32), np.float32)
    x[0, 3], x[0, 9] = 2.0, -2.0                                                # tie: the first wins -> d = 2 / -8
    x[1, 3], x[1, 9] = -2.0, 2.0
    b = O.quant_q4_0(x)
    d0 = b[0, :2].copy().view(np.float16)[0]
    d1 = b[1, :2].copy().view(np.float16)[0]
    assert d0 == np.float16(-0.25) and d1 == np.float16(0.25)
    assert (b[0, 2 + 3] & 15) == 0 and (b[0, 2 + 9] & 15) == 15                 # -max clamps from 16 to 15
    # round half away from zero: x / d = k + 0.5 exactly
    x = np.zeros((1, 32), np.float32)
    x[0, 0] = 127.0
    x[0, 1:5] = [0.5, 1.5, -0.5, -2.5]
    _, q = O.quant_q8_0(x)
    assert list(q[0, 1:5]) == [1, 2, -1, -3]


def test_codes_use_f32_scale_not_its_f16_rounding():
    # amax = 127 * (1 + 2^-12): d = 1 + 2^-12 is not a half; codes must come from the f32 d
    x = np.zeros((1, 32), np.float32)
    d32 = np.float32(1.0) + np.float32(2.0 ** -12)
    x[0, 0] = np.float32(127.0) * d32
    x[0, 1] = np.float32(100.5) * d32          # / f32 d -> 100.5 -> 101; / f16(d) = 1.0 -> 100.52 -> 101 as well
    x[0, 2] = np.float32(63.4999) * np.float32(1.0)
    d, q = O.quant_q8_0(x)
    assert d[0] == np.float16(1.0).view(np.uint16)
    assert q[0, 0] == 127


def test_dequant_reader_matches_reference_dequant():
    # orc_kv_read_head over a cache row built from the golden blocks == the reference's dequantize_row_*
    x = GOLD["x"][:8 * 16].reshape(16, 1, 256)
    for t, key in ((O.KV_Q8_0, "dq8"), (O.KV_Q4_0, "dq4")):
        c = O.HostKV.contiguous(t, 16, 1, 256)
        O.kv_append_rows(c, x, x, np.arange(16))
        for p in range(16):
            got = O.kv_read_head(c, 0, 0, p, 0)
            assert np.array_equal(got, GOLD[key][8 * p:8 * p + 8].reshape(256))
