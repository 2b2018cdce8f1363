"""The C-ABI library loads without a GPU and exports every function include/*.h declares; refusals launch nothing."""
import ctypes
import glob
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared():
    names = []
    for h in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        names += re.findall(r"\b(p1a_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_exports_match_header(p1a):
    names = declared()
    assert len(names) >= 10
    L = ctypes.CDLL(p1a.lib_path())
    for n in names:
        assert hasattr(L, n), n
    assert sorted(p1a.EXPORTS) == names


def test_row_bytes_and_version(p1a):
    assert p1a.kv_row_bytes(p1a.KV_F16, 4, 256) == 2048
    assert p1a.kv_row_bytes(p1a.KV_Q8_0, 4, 256) == 1088
    assert p1a.kv_row_bytes(p1a.KV_Q4_0, 4, 256) == 576
    assert b"gfx950" in p1a.lib().p1a_version()


def test_refusals_do_not_launch(p1a):
    # argument validation happens before any HIP call, so it can be exercised without a GPU
    from importlib import import_module
    b = import_module("p100e-engine_amd.binding")
    kv = b.p1a_kv()
    L = p1a.lib()
    assert L.p1a_kv_append(ctypes.byref(kv), None, None, 0, None, None, 1, None) == -2      # null cache
    kv.k = kv.v = 4096
    kv.type, kv.Hkv, kv.D = 77, 4, 256
    assert L.p1a_attn_decode(4096, ctypes.byref(kv), 4096, None, 1, 0, None, None, 0, 24, 0.0625, None) == -2   # unknown type
    kv.type = p1a.KV_Q8_0
    assert L.p1a_attn_decode(4096, ctypes.byref(kv), 4096, None, 1, 0, None, None, 0, 25, 0.0625, None) == -1   # Hq % Hkv
    assert L.p1a_attn_decode(4096, ctypes.byref(kv), 4096, None, 33, 0, None, None, 0, 24, 0.0625, None) == -1  # too many rows
    assert L.p1a_attn_decode(4100, ctypes.byref(kv), 4096, None, 1, 0, None, None, 0, 24, 0.0625, None) == -1   # misaligned q
    assert b"aligned" in L.p1a_last_error()


def test_cpp_mirror_header_compiles():
    """include/p100e_fast_attn.hpp is self-contained C++17 over the C ABI (host compile only, no GPU needed)"""
    import subprocess
    src = '#include "p100e_fast_attn.hpp"\nint main() { p100e::fast::kv_cache c; return (int) p100e::fast::kv_row_bytes(c.type, 4, 256) == 2048 ? 0 : 1; }\n'
    r = subprocess.run(["/opt/rocm/bin/hipcc", "-std=c++17", "-fsyntax-only", "-x", "c++", "-I" + os.path.join(ROOT, "include"),
                        "-I/opt/rocm/include", "-D__HIP_PLATFORM_AMD__", "-"], input=src, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]


def test_reload_env(p1a):
    """attn_dec2_reload_env (src/fast/attn_dec2.cuh:21): true exactly when the baked-in switch changed"""
    import os
    Hkv = 2
    old = os.environ.pop("P1A_DEC_SPLIT", None)
    try:
        p1a.reload_env()
        n0 = p1a.get_nsplit(Hkv)
        assert not p1a.reload_env()
        os.environ["P1A_DEC_SPLIT"] = "24"
        assert p1a.reload_env()
        assert p1a.get_nsplit(Hkv) == 24
        assert not p1a.reload_env()
        del os.environ["P1A_DEC_SPLIT"]
        assert p1a.reload_env()
        assert p1a.get_nsplit(Hkv) == n0
    finally:
        if old is not None:
            os.environ["P1A_DEC_SPLIT"] = old
        p1a.reload_env()


def test_decode_scratch_need_never_exceeds_footprint(p1a):
    """The per-(device, stream) buffers are sized once, at the footprint of a head shape. Whatever cache a later call of
    that head shape brings - short pages, a misaligned base or page stride (the generic kernel: more partials per row),
    any row grouping - its partials must fit that footprint. Host arithmetic only."""
    from importlib import import_module
    b = import_module("p100e-engine_amd.binding")
    worst = 0
    for Hq, Hkv, D in ((24, 4, 256), (4, 4, 256), (16, 2, 128), (8, 8, 64), (32, 2, 256), (4, 1, 64)):
        fp = p1a.decode_footprint_bytes(Hq, Hkv, D)
        assert fp > 0
        for ty in (p1a.KV_F16, p1a.KV_Q8_0, p1a.KV_Q4_0):
            for psh in range(0, 9):
                for base, pstride_extra in ((4096, 0), (4096 + 8, 0), (4096, 8), (4096 + 2, 2)):
                    for T, rps in ((1, 1), (9, 1), (32, 1), (32, 4), (12, 3), (16, 2)):
                        kv = b.p1a_kv()
                        kv.type, kv.Hkv, kv.D, kv.n_ctx = ty, Hkv, D, 1 << 14
                        kv.k = kv.v = base
                        kv.pt = 4096
                        kv.psh = psh
                        kv.pstride = (p1a.kv_row_bytes(ty, Hkv, D) << psh) + pstride_extra
                        need = p1a.decode_scratch_bytes(kv, Hq, T, rps)
                        assert 0 < need <= fp, (Hq, Hkv, D, ty, psh, base, T, rps, need, fp)
                        worst = max(worst, need / fp)
    assert worst > 0.5          # the footprint is not wildly oversized either


def test_numerics_id_follows_the_split_count(p1a):
    a = p1a.numerics_id(24, 4)
    assert a == p1a.numerics_id(24, 4) and a != 0
    try:
        p1a.set_nsplit(24)
        assert p1a.numerics_id(24, 4) != a
    finally:
        p1a.set_nsplit(0)
    assert p1a.numerics_id(24, 4) == a
