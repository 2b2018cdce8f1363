"""Seeded synthetic inputs shared by the CPU and GPU tests, the smoke check and the benchmark.

Generator: numpy Philox (counter-based) keyed by the seed; N(0,1) via Generator.standard_normal. "RMS-normed per head"
is x * rsqrt(mean(x^2) + 1e-6) with unit weight, computed by the oracle (orc_rmsnorm_heads).
"""
import numpy as np

import _oracle as O


def rng(seed):
    return np.random.Generator(np.random.Philox(seed))


def normal(g, shape, f16=False):
    x = g.standard_normal(shape).astype(np.float32)
    return x.astype(np.float16).astype(np.float32) if f16 else x


def qkv(seed, n_ctx, T, Hq, Hkv, D, f16_inputs=False, norm=True):
    """K, V [n_ctx][Hkv][D], Q [T][Hq][D], gate [T][Hq*D]; Q and K per-head RMS-normed."""
    g = rng(seed)
    k = normal(g, (n_ctx, Hkv, D), f16_inputs)
    v = normal(g, (n_ctx, Hkv, D), f16_inputs)
    q = normal(g, (T, Hq, D), f16_inputs)
    gate = normal(g, (T, Hq * D))
    if norm:
        k = O.rmsnorm_heads(k, D)
        q = O.rmsnorm_heads(q, D)
        if f16_inputs:
            k = k.astype(np.float16).astype(np.float32)
            q = q.astype(np.float16).astype(np.float32)
    return q, k, v, gate


def perm_table(seed, n_pages_pool, n_pages_used):
    g = rng(seed ^ 0x5EED)
    return g.permutation(n_pages_pool)[:n_pages_used].astype(np.int32)


def errors(out, ref):
    out = np.asarray(out, np.float64)
    ref = np.asarray(ref, np.float64)
    max_abs = float(np.max(np.abs(out - ref)))
    rel_l2 = float(np.linalg.norm(out - ref) / max(np.linalg.norm(ref), 1e-30))
    return max_abs, rel_l2


MAX_ABS_TOL = 2e-3   # the path's stated tolerance vs the fp32 reference (scaled by max|ref| where that exceeds 1, see _gpu.check)
REL_L2_TOL = 1e-3
