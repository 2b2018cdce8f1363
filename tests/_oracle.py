"""ctypes access to the CPU oracle (oracle/libp1a_oracle.so) for the tests. The oracle is the checker only."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KV_F16, KV_Q4_0, KV_Q8_0 = 1, 2, 8


class orc_kv(ctypes.Structure):
    _fields_ = [
        ("type", ctypes.c_uint32), ("n_ctx", ctypes.c_int32), ("Hkv", ctypes.c_int32), ("D", ctypes.c_int32),
        ("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("pt", ctypes.c_void_p), ("rtab", ctypes.c_void_p),
        ("psh", ctypes.c_int32), ("pstride", ctypes.c_size_t),
    ]


class orc_mrope(ctypes.Structure):
    _fields_ = [("p", ctypes.c_void_p), ("stride", ctypes.c_int), ("s0", ctypes.c_int), ("s1", ctypes.c_int),
                ("s2", ctypes.c_int), ("sect", ctypes.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(ROOT, "oracle", "libp1a_oracle.so")
        if not os.path.exists(path):
            subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "libp1a_oracle.so"], check=True)
        L = ctypes.CDLL(path)
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_f32_to_f16.argtypes = [ctypes.c_float]
        L.orc_f16_to_f32.restype = ctypes.c_float
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_kv_row_bytes.restype = ctypes.c_size_t
        L.orc_kv_row_bytes.argtypes = [ctypes.c_uint32, ctypes.c_int, ctypes.c_int]
        L.orc_kv_off.restype = ctypes.c_size_t
        L.orc_kv_off.argtypes = [ctypes.POINTER(orc_kv), ctypes.c_int, ctypes.c_int]
        L.orc_quant_q8_0_block.argtypes = [ctypes.c_void_p] * 3
        L.orc_quant_q4_0_block.argtypes = [ctypes.c_void_p] * 2
        L.orc_kv_append_rows.argtypes = [ctypes.POINTER(orc_kv), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        L.orc_kv_read_head.argtypes = [ctypes.POINTER(orc_kv), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        L.orc_attn_rows.restype = ctypes.c_int
        L.orc_attn_rows.argtypes = [ctypes.POINTER(orc_kv), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                    ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_int]
        L.orc_gate.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
        L.orc_rmsnorm_heads.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_float]
        L.orc_attn_prep.argtypes = [ctypes.c_void_p] * 8 + [ctypes.POINTER(orc_kv)] + [ctypes.c_int] * 6 + [ctypes.c_float, ctypes.c_float] + [ctypes.c_int] * 3
        L.orc_attn_prep.restype = ctypes.c_int
        L.orc_attn_prep_mrope.argtypes = L.orc_attn_prep.argtypes + [ctypes.POINTER(orc_mrope)]
        L.orc_attn_prep_mrope.restype = ctypes.c_int
        L.orc_prep_inv_freq.argtypes = [ctypes.c_float, ctypes.c_int, ctypes.c_int]
        L.orc_prep_inv_freq.restype = ctypes.c_double
        L.orc_prep_sincos.argtypes = [ctypes.c_float, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]
        L.orc_prep_sincos.restype = None
        L.orc_a16_quant.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        L.orc_kv_fill_random.argtypes = [ctypes.POINTER(orc_kv), ctypes.c_int, ctypes.c_int, ctypes.c_uint32]
        L.orc_num_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def row_bytes(t, Hkv, D):
    return int(lib().orc_kv_row_bytes(t, Hkv, D))


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


class HostKV:
    """Host-memory KV cache with the engine's layout; `k`/`v` are uint8 numpy views into `pool` (or own arrays)."""

    def __init__(self, kv_type, n_ctx, Hkv, D, k, v, pt=None, rtab=None, psh=0, pstride=0):
        self.type, self.n_ctx, self.Hkv, self.D = kv_type, n_ctx, Hkv, D
        self.k, self.v, self.pt, self.rtab, self.psh, self.pstride = k, v, pt, rtab, psh, pstride

    @staticmethod
    def contiguous(kv_type, n_ctx, Hkv, D):
        rb = row_bytes(kv_type, Hkv, D)
        return HostKV(kv_type, n_ctx, Hkv, D, np.zeros(n_ctx * rb, np.uint8), np.zeros(n_ctx * rb, np.uint8))

    @staticmethod
    def paged(kv_type, Hkv, D, psh, n_pages, page_table, max_pages, n_layers=1, layer=0, pool=None):
        rb = row_bytes(kv_type, Hkv, D)
        ps = 1 << psh
        pstride = n_layers * 2 * ps * rb
        if pool is None:
            pool = np.zeros(n_pages * pstride, np.uint8)
        ko = layer * 2 * ps * rb
        c = HostKV(kv_type, max_pages * ps, Hkv, D, pool[ko:], pool[ko + ps * rb:], pt=page_table, psh=psh, pstride=pstride)
        c.pool = pool
        return c

    def view(self, pt=None, rtab=None):
        c = HostKV(self.type, self.n_ctx, self.Hkv, self.D, self.k, self.v, self.pt if pt is None else pt, rtab, self.psh, self.pstride)
        return c

    def struct(self):
        s = orc_kv()
        s.type, s.n_ctx, s.Hkv, s.D = self.type, self.n_ctx, self.Hkv, self.D
        s.k, s.v = self.k.ctypes.data, self.v.ctypes.data
        s.pt = None if self.pt is None else self.pt.ctypes.data
        s.rtab = None if self.rtab is None else self.rtab.ctypes.data
        s.psh, s.pstride = self.psh, self.pstride
        return s


def quant_q8_0(x):
    """x [n][32] f32 -> (d_bits [n] u16, q [n][32] i8)"""
    x = np.ascontiguousarray(x, np.float32)
    n = x.shape[0]
    d = np.zeros(n, np.uint16)
    q = np.zeros((n, 32), np.int8)
    L = lib()
    for i in range(n):
        L.orc_quant_q8_0_block(x[i].ctypes.data, d[i:].ctypes.data, q[i].ctypes.data)
    return d, q


def quant_q4_0(x):
    x = np.ascontiguousarray(x, np.float32)
    n = x.shape[0]
    b = np.zeros((n, 18), np.uint8)
    L = lib()
    for i in range(n):
        L.orc_quant_q4_0_block(x[i].ctypes.data, b[i].ctypes.data)
    return b


def kv_append_rows(c, k, v, pos):
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    pos = np.ascontiguousarray(pos, np.int32)
    lib().orc_kv_append_rows(ctypes.byref(c.struct()), _p(k), _p(v), _p(pos), len(pos))


def kv_read_head(c, which, t, p, hk):
    dst = np.zeros(c.D, np.float32)
    lib().orc_kv_read_head(ctypes.byref(c.struct()), which, t, p, hk, _p(dst))
    return dst


def attn_rows(c, q, pos, Hq, scale, gate=None, f64=False):
    q = np.ascontiguousarray(q, np.float32)
    pos = np.ascontiguousarray(pos, np.int32)
    out = np.zeros_like(q)
    g = None if gate is None else np.ascontiguousarray(gate, np.float32)
    rc = lib().orc_attn_rows(ctypes.byref(c.struct()), _p(q), _p(out), _p(g), len(pos), _p(pos), Hq, scale, 1 if f64 else 0)
    assert rc == 0, rc
    return out


def rmsnorm_heads(x, D, eps=1e-6):
    x = np.ascontiguousarray(x, np.float32).copy()
    lib().orc_rmsnorm_heads(_p(x), x.size // D, D, eps)
    return x


def attn_prep(c, qg, k, v, q_norm, k_norm, pos, p0, Hq, n_rot, freq_base, eps=1e-6, mrope=None):
    """q | gate split, norm, rope, quantize-append: returns (q, gate); K / V rows are written into c.
    mrope = (positions int32 [3][stride], (s0, s1, s2), sect): interleaved M-RoPE."""
    qg = np.ascontiguousarray(qg, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    pos = np.ascontiguousarray(pos, np.int32)
    T = len(pos)
    q = np.zeros((T, Hq, c.D), np.float32)
    gate = np.zeros((T, Hq * c.D), np.float32)
    qn = None if q_norm is None else np.ascontiguousarray(q_norm, np.float32)
    kn = None if k_norm is None else np.ascontiguousarray(k_norm, np.float32)
    if mrope is None:
        rc = lib().orc_attn_prep(_p(qg), _p(k), _p(v), _p(qn), _p(kn), _p(pos), _p(q), _p(gate), ctypes.byref(c.struct()), p0, T, Hq,
                                 c.Hkv, c.D, n_rot, freq_base, eps, 0, 0, 0)
    else:
        mp, (s0, s1, s2), sect = mrope
        mp = np.ascontiguousarray(mp, np.int32)
        mr = orc_mrope(mp.ctypes.data, mp.shape[1], s0, s1, s2, sect)
        rc = lib().orc_attn_prep_mrope(_p(qg), _p(k), _p(v), _p(qn), _p(kn), _p(pos), _p(q), _p(gate), ctypes.byref(c.struct()), p0, T,
                                       Hq, c.Hkv, c.D, n_rot, freq_base, eps, 0, 0, 0, ctypes.byref(mr))
    assert rc == 0, rc
    return q, gate


def a16_quant(y):
    """y [T][n] f32 -> the engine's a16 activation buffer as uint16 halves: [T*ng*16*2] values then [T*ng*2] (amax, sum)"""
    y = np.ascontiguousarray(y, np.float32)
    T, n = y.shape
    ng = n // 32
    q = np.zeros(T * ng * 34, np.uint16)
    lib().orc_a16_quant(_p(y), T, n, _p(q))
    return q


def kv_fill_random(c, p0, p1, seed):
    """benchmark fill of positions p0 .. p1 - 1 of one sequence (src/fast/attn.cu:559-581)"""
    st = c.struct()
    lib().orc_kv_fill_random(ctypes.byref(st), p0, p1, seed & 0xffffffff)


def gate(x, g):
    """in place: x *= 1 / (1 + exp(-g)) (src/kernels.cu:85-88); x, g float32 arrays of one size"""
    assert x.dtype == np.float32 and g.dtype == np.float32 and x.size == g.size and x.flags.c_contiguous and g.flags.c_contiguous
    lib().orc_gate(x.ctypes.data, g.ctypes.data, x.size)
