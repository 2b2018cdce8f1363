"""ctypes binding of include/p1a_attn.h. Function names follow the reference's C++ surface
(src/fast/attn.cuh:34-70 of the reference tree): kv_append, kv_append_dev, attn_decode, attn_decode_dev,
attn_decode_rows, attn_prefill; attn_prep is src/fast/fused.cuh:101-113."""
import ctypes
import os

KV_F16, KV_Q4_0, KV_Q8_0 = 1, 2, 8

EXPORTS = [
    "p1a_kv_row_bytes", "p1a_kv_append", "p1a_kv_fill_random", "p1a_attn_prep", "p1a_attn_prep_mrope", "p1a_attn_decode", "p1a_attn_decode_a16", "p1a_attn_decode_noalloc", "p1a_a16_bytes", "p1a_ew_quant", "p1a_attn_prefill", "p1a_attn_prefill_scratch_bytes", "p1a_attn_prefill_key_splits",
    "p1a_sigmoid_mul", "p1a_warmup", "p1a_get_nsplit", "p1a_set_nsplit", "p1a_reload_env", "p1a_warmup_prefill", "p1a_set_prefill_staging_limit", "p1a_bench_decode_split_only", "p1a_bench_stream_read", "p1a_release", "p1a_last_error",
    "p1a_version", "p1a_decode_scratch_bytes", "p1a_decode_footprint_bytes", "p1a_numerics_id",
    # include/p1a_pool.h
    "p1a_pool_create", "p1a_pool_destroy", "p1a_pool_n_pages", "p1a_pool_free_pages", "p1a_pool_max_pages", "p1a_pool_page_bytes",
    "p1a_pool_host_used", "p1a_pool_kv_seq", "p1a_pool_kv_rows", "p1a_pool_set_rows", "p1a_pool_state", "p1a_seq_create", "p1a_seq_free",
    "p1a_seq_ensure_pages", "p1a_seq_len", "p1a_seq_resident", "p1a_seq_pages", "p1a_seq_host_bytes", "p1a_seq_advance",
    "p1a_seq_rollback", "p1a_seq_truncate", "p1a_seq_fork", "p1a_seq_offload", "p1a_seq_restore", "p1a_seq_restore_prefix",
    "p1a_seq_pages_out", "p1a_seq_tokens", "p1a_pool_set_fingerprint", "p1a_pool_fingerprint", "p1a_seq_write", "p1a_seq_read",
    "p1a_verify_accept",
]


class P1AError(RuntimeError):
    pass


class p1a_kv(ctypes.Structure):
    _fields_ = [
        ("type", ctypes.c_uint32), ("n_ctx", ctypes.c_int32), ("Hkv", ctypes.c_int32), ("D", ctypes.c_int32),
        ("k", ctypes.c_void_p), ("v", ctypes.c_void_p), ("pt", ctypes.c_void_p), ("rtab", ctypes.c_void_p),
        ("psh", ctypes.c_int32), ("pstride", ctypes.c_size_t),
    ]


class p1a_pool_cfg(ctypes.Structure):
    _fields_ = [
        ("kv_type", ctypes.c_uint32), ("n_kv_layers", ctypes.c_int), ("Hkv", ctypes.c_int), ("D", ctypes.c_int),
        ("psh", ctypes.c_int), ("n_ctx", ctypes.c_int), ("max_slots", ctypes.c_int), ("tokens", ctypes.c_int64),
        ("reserve_mb", ctypes.c_size_t), ("state_bytes", ctypes.c_size_t), ("host_budget", ctypes.c_size_t),
        ("host_memory", ctypes.c_int),
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
    L.p1a_attn_prep_mrope.restype = i32
    L.p1a_attn_prep_mrope.argtypes = [vp] * 8 + [kvp, i32, i32, i32, i32, f32, f32, i32, i32, i32, vp, i32, i32, i32, i32, i32, vp]
    L.p1a_attn_decode_a16.restype = i32
    L.p1a_attn_decode_a16.argtypes = [vp, kvp, vp, vp, vp, i32, i32, vp, vp, i32, i32, f32, vp]
    L.p1a_attn_decode_noalloc.restype = i32
    L.p1a_attn_decode_noalloc.argtypes = [vp, kvp, vp, vp, vp, i32, i32, vp, vp, i32, i32, f32, vp]
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
    L.p1a_kv_fill_random.restype = i32
    L.p1a_kv_fill_random.argtypes = [kvp, i32, i32, ctypes.c_uint32, vp]
    L.p1a_attn_prefill_key_splits.restype = i32
    L.p1a_attn_prefill_key_splits.argtypes = [i32, i32, i32]
    L.p1a_sigmoid_mul.restype = i32
    L.p1a_sigmoid_mul.argtypes = [vp, vp, sz, vp]
    L.p1a_warmup.restype = i32
    L.p1a_warmup.argtypes = [i32, i32, i32, i32, vp]
    L.p1a_get_nsplit.restype = i32
    L.p1a_get_nsplit.argtypes = [i32]
    L.p1a_decode_scratch_bytes.restype = sz
    L.p1a_decode_scratch_bytes.argtypes = [kvp, i32, i32, i32]
    L.p1a_decode_footprint_bytes.restype = sz
    L.p1a_decode_footprint_bytes.argtypes = [i32, i32, i32]
    L.p1a_numerics_id.restype = ctypes.c_uint64
    L.p1a_numerics_id.argtypes = [i32, i32]
    L.p1a_set_nsplit.restype = None
    L.p1a_set_nsplit.argtypes = [i32]
    L.p1a_reload_env.restype = i32
    L.p1a_reload_env.argtypes = []
    L.p1a_set_prefill_staging_limit.restype = None
    L.p1a_set_prefill_staging_limit.argtypes = [sz]
    L.p1a_warmup_prefill.restype = i32
    L.p1a_warmup_prefill.argtypes = [i32, i32, i32, i32, i32, vp]
    L.p1a_bench_decode_split_only.restype = i32
    L.p1a_bench_decode_split_only.argtypes = [vp, kvp, vp, i32, i32, vp, vp, i32, i32, f32, vp]
    L.p1a_bench_stream_read.restype = i32
    L.p1a_bench_stream_read.argtypes = [vp, sz, vp]
    L.p1a_release.restype = None
    L.p1a_last_error.restype = ctypes.c_char_p
    L.p1a_version.restype = ctypes.c_char_p
    # pool / sequence manager (include/p1a_pool.h)
    pp, ip = ctypes.c_void_p, ctypes.POINTER(ctypes.c_int32)
    L.p1a_pool_create.restype = pp
    L.p1a_pool_create.argtypes = [ctypes.POINTER(p1a_pool_cfg), vp]
    L.p1a_pool_destroy.restype = None
    L.p1a_pool_destroy.argtypes = [pp]
    for name in ("p1a_pool_n_pages", "p1a_pool_free_pages", "p1a_pool_max_pages"):
        getattr(L, name).restype = i32
        getattr(L, name).argtypes = [pp]
    for name in ("p1a_pool_page_bytes", "p1a_pool_host_used"):
        getattr(L, name).restype = sz
        getattr(L, name).argtypes = [pp]
    L.p1a_pool_kv_seq.restype = i32
    L.p1a_pool_kv_seq.argtypes = [pp, i32, i32, kvp]
    L.p1a_pool_kv_rows.restype = i32
    L.p1a_pool_kv_rows.argtypes = [pp, i32, kvp]
    L.p1a_pool_set_rows.restype = i32
    L.p1a_pool_set_rows.argtypes = [pp, ip, i32]
    L.p1a_pool_state.restype = vp
    L.p1a_pool_state.argtypes = [pp, i32]
    L.p1a_seq_create.restype = i32
    L.p1a_seq_create.argtypes = [pp]
    for name in ("p1a_seq_free", "p1a_seq_len", "p1a_seq_resident", "p1a_seq_pages", "p1a_seq_offload", "p1a_seq_restore"):
        getattr(L, name).restype = i32
        getattr(L, name).argtypes = [pp, i32]
    for name in ("p1a_seq_ensure_pages", "p1a_seq_truncate", "p1a_seq_fork", "p1a_seq_restore_prefix"):
        getattr(L, name).restype = i32
        getattr(L, name).argtypes = [pp, i32, i32]
    L.p1a_seq_host_bytes.restype = sz
    L.p1a_seq_host_bytes.argtypes = [pp, i32]
    L.p1a_seq_advance.restype = i32
    L.p1a_seq_advance.argtypes = [pp, i32, ip, i32]
    L.p1a_seq_rollback.restype = i32
    L.p1a_seq_rollback.argtypes = [pp, i32, i32, i32]
    L.p1a_seq_pages_out.restype = i32
    L.p1a_seq_pages_out.argtypes = [pp, i32, i32, i32, vp]
    L.p1a_seq_tokens.restype = i32
    L.p1a_seq_tokens.argtypes = [pp, i32, ip, i32]
    L.p1a_pool_set_fingerprint.restype = i32
    L.p1a_pool_set_fingerprint.argtypes = [pp, ctypes.POINTER(ctypes.c_uint64)]
    L.p1a_pool_fingerprint.restype = i32
    L.p1a_pool_fingerprint.argtypes = [pp, ctypes.POINTER(ctypes.c_uint64)]
    L.p1a_seq_write.restype = i32
    L.p1a_seq_write.argtypes = [pp, i32, ctypes.c_char_p]
    L.p1a_seq_read.restype = i32
    L.p1a_seq_read.argtypes = [pp, ctypes.c_char_p]
    L.p1a_verify_accept.restype = i32
    L.p1a_verify_accept.argtypes = [ip, ip, i32, i32, ip, ip]
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

    Contiguous: KVCache.contiguous(type, n_ctx, Hkv, D). Paged: KVCache.paged(...) lays a test pool out as
    [page][layer][K|V][2^psh positions][row] - a page stride that spans other layers, as the reference's session test
    does (tests/fast_sessions_test.cu:75,91-92) - one layer selected by the k / v base pointers, a slot by its
    page-table row. (The engine's own pool layout is class Pool's.)
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


def kv_fill_random(c, p0, p1, seed):
    """src/fast/attn.cuh:70: benchmark fill of positions p0 .. p1 - 1 of one sequence."""
    _check(lib().p1a_kv_fill_random(ctypes.byref(c.struct()), p0, p1, seed & 0xffffffff, _stream()), "kv_fill_random")


def kv_append_dev(c, k, v, p0_dev, T):
    """src/fast/attn.cuh:58: the first position is read from device memory."""
    _check(lib().p1a_kv_append(ctypes.byref(c.struct()), _ptr(k), _ptr(v), 0, _ptr(p0_dev), None, T, _stream()), "kv_append_dev")


def kv_append_rows(c, k, v, pos_rows, T):
    """Cache-write half of attn_prep in device-position mode (src/fast/fused.cuh:101-113): row t -> pos_rows[t] of
    its own sequence (c.rtab)."""
    _check(lib().p1a_kv_append(ctypes.byref(c.struct()), _ptr(k), _ptr(v), -1, None, _ptr(pos_rows), T, _stream()), "kv_append_rows")


def attn_prep(qg, k, v, q_norm, k_norm, pos, q, gate, c, p0, T, Hq, n_rot, freq_base, eps, ldq=0, ldk=0, ldv=0, mrope=None):
    """src/fast/fused.cuh:101-113: q | gate split, per-head RMS norm * weight, NEOX rope, quantizing KV write (p0 < 0:
    cache row of token t = pos[t], its own page table). mrope = (positions int32 [3][stride] on the device, stride,
    (s0, s1, s2), sect): interleaved M-RoPE (src/fast/mrope.cuh)."""
    if mrope is not None:
        mp, stride, (s0, s1, s2), sect = mrope
        _check(lib().p1a_attn_prep_mrope(_ptr(qg), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm), _ptr(pos), _ptr(q), _ptr(gate),
                                         ctypes.byref(c.struct()), p0, T, Hq, n_rot, freq_base, eps, ldq, ldk, ldv,
                                         _ptr(mp), stride, s0, s1, s2, sect, _stream()), "attn_prep")
        return
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


def prefill_key_splits(T, p0, Hq):
    return int(lib().p1a_attn_prefill_key_splits(T, p0, Hq))


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


def decode_scratch_bytes(c, Hq, T, rows_per_seq=1):
    return int(lib().p1a_decode_scratch_bytes(ctypes.byref(c), Hq, T, rows_per_seq))


def decode_footprint_bytes(Hq, Hkv, D):
    return int(lib().p1a_decode_footprint_bytes(Hq, Hkv, D))


def numerics_id(Hq, Hkv):
    return int(lib().p1a_numerics_id(Hq, Hkv))


def reload_env():
    """src/fast/attn_dec2.cuh:21: True when the split-count environment switch changed (captured graphs must be dropped)."""
    return bool(lib().p1a_reload_env())


def set_prefill_staging_limit(nbytes):
    lib().p1a_set_prefill_staging_limit(nbytes)


def warmup_prefill(T, p0, Hq, Hkv, D):
    _check(lib().p1a_warmup_prefill(T, p0, Hq, Hkv, D, _stream()), "warmup_prefill")


def bench_decode_split_only(q, c, out, T, p0, Hq, scale, pos=None, rows_per_seq=0):
    """Benchmarks only: the split-K kernel of attn_decode / attn_decode_rows without the merge (out untouched)."""
    _check(lib().p1a_bench_decode_split_only(_ptr(q), ctypes.byref(c.struct()), _ptr(out), T, p0, None, _ptr(pos), rows_per_seq, Hq, scale, _stream()), "bench_decode_split_only")


def bench_stream_read(t):
    """Benchmarks only: a plain streaming read of the tensor's bytes on the current stream."""
    _check(lib().p1a_bench_stream_read(_ptr(t), t.numel() * t.element_size(), _stream()), "p1a_bench_stream_read")


class KVDesc:
    """A p1a_kv descriptor that somebody else owns the memory of (the pool's)."""

    def __init__(self, st):
        self._st = st

    def struct(self):
        return self._st


class Pool:
    """The paged KV pool + sequence manager of include/p1a_pool.h (the reference's tp_model pool / seq_* members).

    Methods keep the reference's names; a refusal raises P1AError with the reference's message. host_memory=True keeps
    the pool in host memory (no GPU call): `memory()` then returns a numpy view of it."""

    def __init__(self, kv_type, n_kv_layers, Hkv, D, psh, n_ctx, max_slots, tokens, state_bytes=0, host_budget=0,
                 reserve_mb=0, host_memory=False, stream=None):
        cfg = p1a_pool_cfg(kv_type, n_kv_layers, Hkv, D, psh, n_ctx, max_slots, tokens, reserve_mb, state_bytes, host_budget,
                           1 if host_memory else 0)
        self.cfg, self.host_memory = cfg, host_memory
        self._p = lib().p1a_pool_create(ctypes.byref(cfg), stream)
        if not self._p:
            raise P1AError("alloc_pool refused: " + lib().p1a_last_error().decode())

    def close(self):
        if self._p:
            lib().p1a_pool_destroy(self._p)
            self._p = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _rc(self, rc, what):
        if rc < 0:
            raise P1AError(f"{what} refused (rc={rc}): {lib().p1a_last_error().decode()}")
        return rc

    n_pages = property(lambda self: lib().p1a_pool_n_pages(self._p))
    free_pages = property(lambda self: lib().p1a_pool_free_pages(self._p))
    max_pages = property(lambda self: lib().p1a_pool_max_pages(self._p))
    page_bytes = property(lambda self: int(lib().p1a_pool_page_bytes(self._p)))
    host_used = property(lambda self: int(lib().p1a_pool_host_used(self._p)))

    def cache_seq(self, layer, seq):
        """kv_seq as an object the attention entry points of this module take"""
        return KVDesc(self.kv_seq(layer, seq))

    def cache_rows(self, layer):
        return KVDesc(self.kv_rows(layer))

    def kv_seq(self, layer, seq):
        c = p1a_kv()
        self._rc(lib().p1a_pool_kv_seq(self._p, layer, seq, ctypes.byref(c)), "kv_seq")
        return c

    def kv_rows(self, layer):
        c = p1a_kv()
        self._rc(lib().p1a_pool_kv_rows(self._p, layer, ctypes.byref(c)), "kv_rows")
        return c

    def set_rows(self, ids):
        a = (ctypes.c_int32 * len(ids))(*ids)
        self._rc(lib().p1a_pool_set_rows(self._p, a, len(ids)), "set_rows")

    def state(self, seq):
        return lib().p1a_pool_state(self._p, seq)

    def seq_create(self):
        return self._rc(lib().p1a_seq_create(self._p), "seq_create")

    def seq_free(self, seq):
        self._rc(lib().p1a_seq_free(self._p, seq), "seq_free")

    def ensure_pages(self, seq, n):
        self._rc(lib().p1a_seq_ensure_pages(self._p, seq, n), "ensure_pages")

    def seq_len(self, seq):
        return self._rc(lib().p1a_seq_len(self._p, seq), "seq_len")

    def seq_resident(self, seq):
        return bool(lib().p1a_seq_resident(self._p, seq))

    def seq_pages(self, seq):
        return self._rc(lib().p1a_seq_pages(self._p, seq), "seq_pages")

    def seq_host_bytes(self, seq):
        return int(lib().p1a_seq_host_bytes(self._p, seq))

    def seq_advance(self, seq, toks=None, T=None):
        if toks is None:
            return self._rc(lib().p1a_seq_advance(self._p, seq, None, T), "seq_advance")
        a = (ctypes.c_int32 * len(toks))(*toks)
        return self._rc(lib().p1a_seq_advance(self._p, seq, a, len(toks)), "seq_advance")

    def rollback(self, seq, T, n_keep):
        return self._rc(lib().p1a_seq_rollback(self._p, seq, T, n_keep), "rollback")

    def seq_truncate(self, seq, n):
        self._rc(lib().p1a_seq_truncate(self._p, seq, n), "seq_truncate")

    def seq_fork(self, src, n):
        return self._rc(lib().p1a_seq_fork(self._p, src, n), "seq_fork")

    def seq_offload(self, seq):
        self._rc(lib().p1a_seq_offload(self._p, seq), "seq_offload")

    def seq_restore(self, seq):
        self._rc(lib().p1a_seq_restore(self._p, seq), "seq_restore")

    def seq_restore_prefix(self, seq, n):
        self._rc(lib().p1a_seq_restore_prefix(self._p, seq, n), "seq_restore_prefix")

    def pages_out(self, seq, p0, n, dst_ptr):
        self._rc(lib().p1a_seq_pages_out(self._p, seq, p0, n, dst_ptr), "pages_out")

    def seq_tokens(self, seq):
        n = self._rc(lib().p1a_seq_tokens(self._p, seq, None, 0), "seq_tokens")
        a = (ctypes.c_int32 * max(n, 1))()
        lib().p1a_seq_tokens(self._p, seq, a, n)
        return list(a[:n])

    def set_fingerprint(self, fp):
        a = (ctypes.c_uint64 * 15)(*fp)
        self._rc(lib().p1a_pool_set_fingerprint(self._p, a), "set_fingerprint")

    def fingerprint(self):
        a = (ctypes.c_uint64 * 15)()
        self._rc(lib().p1a_pool_fingerprint(self._p, a), "fingerprint")
        return list(a)

    def seq_write(self, seq, path):
        self._rc(lib().p1a_seq_write(self._p, seq, os.fsencode(path)), "seq_write")

    def seq_read(self, path):
        return self._rc(lib().p1a_seq_read(self._p, os.fsencode(path)), "seq_read")

    def memory(self, c=None):
        """host-memory pools only: the whole pool as a numpy byte array (a view)"""
        import numpy as np
        if not self.host_memory:
            raise P1AError("memory(): not a host-memory pool")
        c = c or self.kv_rows(0)
        n = self.n_pages * self.page_bytes
        return np.ctypeslib.as_array((ctypes.c_uint8 * n).from_address(c.k))


def verify_accept(tokens, greedy, budget):
    """(rows to keep, accepted drafts, next token) of one verify step: include/p1a_pool.h p1a_verify_accept"""
    T = len(tokens)
    a, b = (ctypes.c_int32 * T)(*tokens), (ctypes.c_int32 * T)(*greedy)
    na, nt = ctypes.c_int32(0), ctypes.c_int32(0)
    q = lib().p1a_verify_accept(a, b, T, budget, ctypes.byref(na), ctypes.byref(nt))
    if q < 0:
        raise P1AError("verify_accept refused: " + lib().p1a_last_error().decode())
    return q, na.value, nt.value
