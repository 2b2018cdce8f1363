"""ctypes binding of include/p1a_attn.h. Function names follow the reference's C++ surface
(src/fast/attn.cuh:34-70 of the reference tree): kv_append, kv_append_dev, attn_decode, attn_decode_dev,
attn_decode_rows, attn_prefill; attn_prep is src/fast/fused.cuh:101-113."""
import ctypes
import os

KV_F16, KV_Q4_0, KV_Q8_0 = 1, 2, 8

EXPORTS = [
    "p1a_kv_row_bytes", "p1a_kv_append", "p1a_attn_prep", "p1a_attn_decode", "p1a_attn_decode_a16", "p1a_a16_bytes", "p1a_ew_quant", "p1a_attn_prefill", "p1a_attn_prefill_scratch_bytes",
    "p1a_sigmoid_mul", "p1a_warmup", "p1a_get_nsplit", "p1a_set_nsplit", "p1a_bench_skip_merge", "p1a_release", "p1a_last_error",
    "p1a_version",
]


class P1AError(RuntimeError):
    pass


class p1a_kv(ctypes.Structure):
    _fields_ = [
        ("type", ctypes.c_uint32), ("n_ctx", ctypes.c_int32), ("Hkv", ctypes.c_int32), ("D", ctypes.c_int32),
        ("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("pt", ctypes.c_void_p), ("rtab", ctypes.c_void_p),
        ("psh", ctypes.c_int32), ("pstride", ctypes.c_size_t),
    ]


def lib_path():
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "libp1a_attn.so")


_lib = None


def lib():
    """Load libp1a_attn.so (built by __graft_entry__.build() / csrc/Makefile). Raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise P1AError(f"{path} is missing: build it with `make -C p100e-engine_amd/csrc` (there is no fallback path)")
    L = ctypes.CDLL(path)
    vp, i32, f32, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
    kvp = ctypes.POINTER(p1a_kv)
    L.p1a_kv_row_bytes.restype = sz
    L.p1a_kv_row_bytes.argtypes = [ctypes.c_uint32, i32, i32]
    L.p1a_kv_append.restype = i32
    L.p1a_kv_append.argtypes = [kvp, vp, vp, i32, vp, vp, i32, vp]
    L.p1a_attn_prep.restype = i32
    L.p1a_attn_prep.argtypes = [vp] * 8 + [kvp, i32, i32, i32, i32, f32, f32, i32, i32, i32, vp]
    L.p1a_attn_decode_a16.restype = i32
    L.p1a_attn_decode_a16.argtypes = [vp, kvp, vp, vp, vp, i32, i32, vp, vp, i32, i32, f32, vp]
    L.p1a_a16_bytes.restype = sz
    L.p1a_a16_bytes.argtypes = [i32, i32]
    L.p1a_ew_quant.restype = i32
    L.p1a_ew_quant.argtypes = [i32, vp, vp, vp, vp, i32, i32, i32, i32, vp]
    L.p1a_attn_decode.restype = i32
    L.p1a_attn_decode.argtypes = [vp, kvp, vp, vp, i32, i32, vp, vp, i32, i32, f32, vp]
    L.p1a_attn_prefill.restype = i32
    L.p1a_attn_prefill.argtypes = [vp, kvp, vp, vp, i32, i32, i32, f32, vp, sz, vp]
    L.p1a_attn_prefill_scratch_bytes.restype = sz
    L.p1a_attn_prefill_scratch_bytes.argtypes = [i32, i32, i32, i32, i32]
    L.p1a_sigmoid_mul.restype = i32
    L.p1a_sigmoid_mul.argtypes = [vp, vp, sz, vp]
    L.p1a_warmup.restype = i32
    L.p1a_warmup.argtypes = [i32, i32, i32, i32, vp]
    L.p1a_get_nsplit.restype = i32
    L.p1a_get_nsplit.argtypes = [i32]
    L.p1a_set_nsplit.restype = None
    L.p1a_set_nsplit.argtypes = [i32]
    L.p1a_bench_skip_merge.restype = None
    L.p1a_bench_skip_merge.argtypes = [i32]
    L.p1a_release.restype = None
    L.p1a_last_error.restype = ctypes.c_char_p
    L.p1a_version.restype = ctypes.c_char_p
    _lib = L
    return L


def kv_row_bytes(kv_type, Hkv, D):
    return int(lib().p1a_kv_row_bytes(kv_type, Hkv, D))


def _check(rc, what):
    if rc != 0:
        raise P1AError(f"{what} refused (rc={rc}): {lib().p1a_last_error().decode()}")


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class KVCache:
    """Device KV cache of one layer, the twin of the reference's kv_cache (src/fast/attn.cuh:18-32).

    Contiguous: KVCache.contiguous(type, n_ctx, Hkv, D). Paged: KVCache.paged(...) lays a pool out as the engine does
    (src/tp_model.cu:3880-3942 of the reference): [page][layer][K|V][2^psh positions][row], one layer selected by the
    k / v base pointers, a slot by its page-table row.
    """

    def __init__(self, kv_type, n_ctx, Hkv, D, k, v, pt=None, rtab=None, psh=0, pstride=0, keep=()):
        self.type, self.n_ctx, self.Hkv, self.D = kv_type, n_ctx, Hkv, D
        self.k, self.v, self.pt, self.rtab, self.psh, self.pstride = k, v, pt, rtab, psh, pstride
        self._keep = keep   # tensors that own the memory

    @staticmethod
    def contiguous(kv_type, n_ctx, Hkv, D, device="cuda"):
        import torch
        rowb = kv_row_bytes(kv_type, Hkv, D)
        k = torch.zeros(n_ctx * rowb, dtype=torch.uint8, device=device)
        v = torch.zeros(n_ctx * rowb, dtype=torch.uint8, device=device)
        return KVCache(kv_type, n_ctx, Hkv, D, k.data_ptr(), v.data_ptr(), keep=(k, v))

    @staticmethod
    def paged(kv_type, Hkv, D, psh, n_pages, page_table, max_pages, n_layers=1, layer=0, device="cuda", pool=None):
        """page_table: int32 tensor [n_slots * max_pages] on the device (entries = page indices)."""
        import torch
        rowb = kv_row_bytes(kv_type, Hkv, D)
        ps = 1 << psh
        pstride = n_layers * 2 * ps * rowb
        if pool is None:
            pool = torch.zeros(n_pages * pstride, dtype=torch.uint8, device=device)
        base = pool.data_ptr()
        k = base + layer * 2 * ps * rowb
        v = k + ps * rowb
        c = KVCache(kv_type, max_pages * ps, Hkv, D, k, v, pt=page_table, psh=psh, pstride=pstride, keep=(pool, page_table))
        c.pool = pool
        return c

    def slot(self, s, max_pages):
        """The same cache seen through slot s's page-table row."""
        c = KVCache(self.type, self.n_ctx, self.Hkv, self.D, self.k, self.v, self.pt, None, self.psh, self.pstride, self._keep)
        c._pt_off = s * max_pages
        return c

    def with_rows(self, rtab):
        c = KVCache(self.type, self.n_ctx, self.Hkv, self.D, self.k, self.v, self.pt, rtab, self.psh, self.pstride,
                    self._keep + (rtab,))
        return c

    def struct(self):
        s = p1a_kv()
        s.type, s.n_ctx, s.Hkv, s.D = self.type, self.n_ctx, self.Hkv, self.D
        s.k, s.v = self.k, self.v
        off = getattr(self, "_pt_off", 0)
        s.pt = None if self.pt is None else self.pt.data_ptr() + 4 * off
        s.rtab = None if self.rtab is None else self.rtab.data_ptr()
        s.psh, s.pstride = self.psh, self.pstride
        return s


def kv_append(c, k, v, p0, T):
    """src/fast/attn.cuh:37-38 of the reference: k, v [T][Hkv][D] f32 -> cache positions p0..p0+T-1."""
    _check(lib().p1a_kv_append(ctypes.byref(c.struct()), _ptr(k), _ptr(v), p0, None, None, T, _stream()), "kv_append")


def kv_append_dev(c, k, v, p0_dev, T):
    """src/fast/attn.cuh:58: the first position is read from device memory."""
    _check(lib().p1a_kv_append(ctypes.byref(c.struct()), _ptr(k), _ptr(v), 0, _ptr(p0_dev), None, T, _stream()), "kv_append_dev")


def kv_append_rows(c, k, v, pos_rows, T):
    """Cache-write half of attn_prep in device-position mode (src/fast/fused.cuh:101-113): row t -> pos_rows[t] of
    its own sequence (c.rtab)."""
    _check(lib().p1a_kv_append(ctypes.byref(c.struct()), _ptr(k), _ptr(v), -1, None, _ptr(pos_rows), T, _stream()), "kv_append_rows")


def attn_prep(qg, k, v, q_norm, k_norm, pos, q, gate, c, p0, T, Hq, n_rot, freq_base, eps, ldq=0, ldk=0, ldv=0):
    """src/fast/fused.cuh:101-113: q | gate split, per-head RMS norm * weight, NEOX rope, quantizing KV write (p0 < 0:
    cache row of token t = pos[t], its own page table)."""
    _check(lib().p1a_attn_prep(_ptr(qg), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm), _ptr(pos), _ptr(q), _ptr(gate),
                               ctypes.byref(c.struct()), p0, T, Hq, n_rot, freq_base, eps, ldq, ldk, ldv, _stream()), "attn_prep")


def attn_decode(q, c, out, T, p0, Hq, scale, gate=None):
    """src/fast/attn.cuh:44."""
    _check(lib().p1a_attn_decode(_ptr(q), ctypes.byref(c.struct()), _ptr(out), _ptr(gate), T, p0, None, None, 0, Hq, scale, _stream()), "attn_decode")


def attn_decode_dev(q, c, out, T, p0_dev, max_n, Hq, scale, gate=None):
    """src/fast/attn.cuh:59-60 (max_n is accepted for signature parity; the grid never depends on the depth)."""
    _check(lib().p1a_attn_decode(_ptr(q), ctypes.byref(c.struct()), _ptr(out), _ptr(gate), T, 0, _ptr(p0_dev), None, 0, Hq, scale, _stream()), "attn_decode_dev")


def attn_decode_rows(q, c, out, T, pos, Hq, scale, gate=None, rows_per_seq=1, qbuf=None):
    """src/fast/attn.cuh:64-65; rows_per_seq > 1: consecutive rows form verify blocks that share one KV read; qbuf: also
    emit the a16 activation buffer of the gated rows (src/fast/fused.cu:478-496)."""
    _check(lib().p1a_attn_decode_a16(_ptr(q), ctypes.byref(c.struct()), _ptr(out), _ptr(gate), _ptr(qbuf), T, 0, None, _ptr(pos), rows_per_seq, Hq, scale, _stream()), "attn_decode_rows")


def a16_bytes(T, n):
    return int(lib().p1a_a16_bytes(T, n))


def ew_quant(op, a, b, y, qbuf, T, n, lda=0, ldb=0):
    """src/fast/fused.cuh:92-98: op 0 y = silu(a) * b, op 1 y = a * sigmoid(b); qbuf = a16(y)."""
    _check(lib().p1a_ew_quant(op, _ptr(a), _ptr(b), _ptr(y), _ptr(qbuf), T, n, lda, ldb, _stream()), "ew_quant")


def prefill_scratch_bytes(T, p0, Hq, Hkv, D):
    return int(lib().p1a_attn_prefill_scratch_bytes(T, p0, Hq, Hkv, D))


def attn_prefill(q, c, out, T, p0, Hq, scale, gate=None, scratch=None):
    """src/fast/attn.cuh:46-50 / src/fast/attn_fold.cuh:19-26."""
    nbytes = 0 if scratch is None else scratch.numel() * scratch.element_size()
    _check(lib().p1a_attn_prefill(_ptr(q), ctypes.byref(c.struct()), _ptr(out), _ptr(gate), T, p0, Hq, scale, _ptr(scratch), nbytes, _stream()), "attn_prefill")


def sigmoid_mul(x, g):
    _check(lib().p1a_sigmoid_mul(_ptr(x), _ptr(g), x.numel(), _stream()), "sigmoid_mul")


def warmup(rows, Hq, Hkv, D):
    _check(lib().p1a_warmup(rows, Hq, Hkv, D, _stream()), "warmup")


def get_nsplit(Hkv):
    return int(lib().p1a_get_nsplit(Hkv))


def set_nsplit(n):
    lib().p1a_set_nsplit(n)


def bench_skip_merge(on):
    lib().p1a_bench_skip_merge(1 if on else 0)
