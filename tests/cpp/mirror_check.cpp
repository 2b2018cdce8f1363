// Drives the library through the C++ mirror of the reference surface (include/p100e_fast_attn.hpp), the way the
// reference's own standalone test executables do (tests/fast_sessions_test.cu:69-175 of the reference tree): a pool of
// pages with a random page permutation and a stride spanning other layers, the same appends to a contiguous and to a
// paged cache, then bitwise checks: cache rows, attn_decode T = 1..4 paged vs contiguous, attn_decode_rows vs one
// T = 1 call per row, prefill paged vs contiguous. Prints one line per check, exits non-zero on failure.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <string>
#include <vector>

#include "p100e_fast_attn.hpp"
#include "p100e_kv_pool.hpp"

namespace F = p100e::fast;
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); exit(2); } } while (0)

static int g_fail = 0, g_checks = 0;
static uint32_t g_rng = 12345;
static uint32_t urand() { g_rng = g_rng * 1664525u + 1013904223u; return g_rng >> 8; }
static float frand(float s) { return ((urand() & 0xffff) + (urand() & 0xffff) + (urand() & 0xffff)) * (s / 32768.0f) - 3.0f * s; }
static float * dev_rand(size_t n, float s) {
    std::vector<float> h(n);
    for (auto & x : h) x = frand(s);
    float * d; CK(hipMalloc(&d, n * 4)); CK(hipMemcpy(d, h.data(), n * 4, hipMemcpyHostToDevice));
    return d;
}
static std::vector<char> bytes_of(const void * d, size_t n) { std::vector<char> h(n); CK(hipMemcpy(h.data(), d, n, hipMemcpyDeviceToHost)); return h; }
static void check(const char * name, bool ok) { ++g_checks; if (!ok) ++g_fail; printf("    %-62s %s\n", name, ok ? "identical" : "FAIL"); }
static const char * tname(uint32_t t) { return t == F::KV_F16 ? "f16" : t == F::KV_Q8_0 ? "q8_0" : "q4_0"; }

static void test_type(uint32_t type, hipStream_t s) {
    printf("paged KV cache, %s\n", tname(type));
    const int Hkv = 2, D = 256, Hq = 12, PSH = 8, PS = 1 << PSH, NP = 64, MAXP = 48, NLAY = 2;
    const float scale = 1.0f / 16.0f;
    const size_t rowb = F::kv_row_bytes(type, Hkv, D);
    const size_t pstride = (size_t) NLAY * 2 * PS * rowb;
    char * pool; CK(hipMalloc(&pool, (size_t) NP * pstride)); CK(hipMemset(pool, 0, (size_t) NP * pstride));
    const int NS = 3, len[NS] = {700, 11000, 300};
    std::vector<int> perm(NP);
    std::iota(perm.begin(), perm.end(), 0);
    for (int i = NP - 1; i > 0; --i) std::swap(perm[i], perm[urand() % (i + 1)]);
    std::vector<int32_t> tabs((size_t) NS * MAXP, 0);
    int used = 0;
    for (int q = 0; q < NS; ++q)
        for (int p = 0; p < (len[q] + PS - 1) / PS + 1; ++p) tabs[(size_t) q * MAXP + p] = perm[used++];
    int32_t * dtab; CK(hipMalloc(&dtab, tabs.size() * 4)); CK(hipMemcpy(dtab, tabs.data(), tabs.size() * 4, hipMemcpyHostToDevice));
    auto paged = [&](int q) {
        F::kv_cache c; c.type = type; c.n_ctx = MAXP * PS; c.Hkv = Hkv; c.D = D;
        c.k = pool + (size_t) 1 * 2 * PS * rowb; c.v = pool + (size_t) 1 * 2 * PS * rowb + PS * rowb;   // layer 1 of the pool
        c.pt = dtab + (size_t) q * MAXP; c.psh = PSH; c.pstride = pstride;
        return c;
    };
    std::vector<F::kv_cache> cc(NS);
    for (int q = 0; q < NS; ++q) {
        cc[q] = F::kv_alloc(type, MAXP * PS, Hkv, D);
        float * ks = dev_rand((size_t) len[q] * Hkv * D, 1.0f), * vs = dev_rand((size_t) len[q] * Hkv * D, 1.0f);
        F::kv_cache pc = paged(q);
        for (int p = 0; p < len[q]; p += 64) {
            const int T = std::min(64, len[q] - p);
            F::kv_append(cc[q], ks + (size_t) p * Hkv * D, vs + (size_t) p * Hkv * D, p, T, s);
            F::kv_append(pc, ks + (size_t) p * Hkv * D, vs + (size_t) p * Hkv * D, p, T, s);
        }
        CK(hipStreamSynchronize(s));
        CK(hipFree(ks)); CK(hipFree(vs));
    }
    {
        bool ok = true;
        auto hpool = bytes_of(pool, (size_t) NP * pstride);
        for (int q = 0; q < NS; ++q) {
            auto hk = bytes_of(cc[q].k, (size_t) len[q] * rowb), hv = bytes_of(cc[q].v, (size_t) len[q] * rowb);
            for (int p = 0; p < len[q]; ++p) {
                const size_t o = (size_t) tabs[(size_t) q * MAXP + (p >> PSH)] * pstride + (size_t) 2 * PS * rowb + (size_t) (p & (PS - 1)) * rowb;
                ok = ok && !memcmp(hk.data() + (size_t) p * rowb, hpool.data() + o, rowb);
                ok = ok && !memcmp(hv.data() + (size_t) p * rowb, hpool.data() + o + PS * rowb, rowb);
            }
        }
        check("kv_append paged vs contiguous (every position, K and V)", ok);
    }
    float * q = dev_rand((size_t) 256 * Hq * D, 1.5f);
    float * o1, * o2; CK(hipMalloc(&o1, (size_t) 256 * Hq * D * 4)); CK(hipMalloc(&o2, (size_t) 256 * Hq * D * 4));
    {
        int bad = 0, n = 0;
        for (int sq = 0; sq < NS; ++sq) {
            const F::kv_cache pc = paged(sq);
            for (int T = 1; T <= 4; ++T)
                for (int p0 : {0, 1, 31, 32, 127, 128, 255, 256, 257, 511, 600, 4223, 4224, 5000, 8191, 10000, len[sq] - T}) {
                    if (p0 < 0 || p0 + T > len[sq]) continue;
                    const bool a1 = F::attn_decode(q, cc[sq], o1, T, p0, Hq, scale, s), a2 = F::attn_decode(q, pc, o2, T, p0, Hq, scale, s);
                    CK(hipStreamSynchronize(s));
                    auto a = bytes_of(o1, (size_t) T * Hq * D * 4), b = bytes_of(o2, (size_t) T * Hq * D * 4);
                    ++n; if (!a1 || !a2 || memcmp(a.data(), b.data(), a.size())) ++bad;
                }
        }
        printf("    (%d cases) ", n);
        check("attn_decode T=1..4 paged vs contiguous", bad == 0);
    }
    {
        struct row { int s, p; };
        const std::vector<std::vector<row>> sets = {
            {{0, 699}}, {{0, 699}, {1, 1499}, {2, 299}}, {{1, 10999}, {0, 600}, {1, 9000}, {2, 250}, {1, 4300}},
            {{1, 1200}, {1, 1201}, {1, 1202}, {1, 1203}},
            {{0, 650}, {0, 651}, {1, 1496}, {1, 1497}, {1, 1498}, {2, 100}, {2, 101}, {2, 102}},
            {{2, 0}, {0, 0}, {1, 255}, {1, 256}, {0, 31}, {0, 32}},
        };
        int32_t * dpos, * drt; CK(hipMalloc(&dpos, 64)); CK(hipMalloc(&drt, 64));
        int bad = 0;
        for (const auto & set : sets) {
            const int T = (int) set.size();
            std::vector<int32_t> hp(T), hr(T);
            for (int t = 0; t < T; ++t) { hp[t] = set[t].p; hr[t] = set[t].s * MAXP; }
            CK(hipMemcpy(dpos, hp.data(), T * 4, hipMemcpyHostToDevice)); CK(hipMemcpy(drt, hr.data(), T * 4, hipMemcpyHostToDevice));
            F::kv_cache pc = paged(0);
            pc.pt = dtab; pc.rtab = drt;
            if (!F::attn_decode_rows(q, pc, o2, T, dpos, Hq, scale, s)) { ++bad; continue; }
            CK(hipStreamSynchronize(s));
            auto b = bytes_of(o2, (size_t) T * Hq * D * 4);
            for (int t = 0; t < T; ++t) {
                F::attn_decode(q + (size_t) t * Hq * D, cc[set[t].s], o1, 1, set[t].p, Hq, scale, s);
                CK(hipStreamSynchronize(s));
                auto a = bytes_of(o1, (size_t) Hq * D * 4);
                if (memcmp(a.data(), b.data() + (size_t) t * Hq * D * 4, a.size())) ++bad;
            }
        }
        check("attn_decode_rows (3 sequences, 1..8 rows) vs T=1 per row", bad == 0);
        CK(hipFree(dpos)); CK(hipFree(drt));
    }
    {
        const int sq = 1, T = 200, p0 = 1300;
        const bool a1 = F::attn_prefill(q, cc[sq], o1, T, p0, Hq, scale, s), a2 = F::attn_prefill(q, paged(sq), o2, T, p0, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        auto a = bytes_of(o1, (size_t) T * Hq * D * 4), b = bytes_of(o2, (size_t) T * Hq * D * 4);
        check("attn_prefill T=200 p0=1300 paged vs contiguous", a1 && a2 && !memcmp(a.data(), b.data(), a.size()));
    }
    {   // attn_fold on a short chunk over a long context (the library splits it over the keys): with the scratch of
        // attn_fold_scratch_bytes, with a scratch that is too small and through attn_prefill - one result, bit for bit
        const int sq = 1, T = 100, p0 = len[sq] - T;
        const size_t nb = F::attn_fold_scratch_bytes(T, Hkv, 2048, 8, p0);
        void * scr; CK(hipMalloc(&scr, nb)); CK(hipMemset(scr, 0xff, nb));
        const bool a1 = F::attn_prefill(q, cc[sq], o1, T, p0, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        auto a = bytes_of(o1, (size_t) T * Hq * D * 4);
        const bool a2 = F::attn_fold(q, paged(sq), o2, T, p0, Hq, scale, scr, nb, s);
        CK(hipStreamSynchronize(s));
        auto b = bytes_of(o2, (size_t) T * Hq * D * 4);
        const bool a3 = F::attn_fold(q, cc[sq], o2, T, p0, Hq, scale, scr, 4096, s);
        CK(hipStreamSynchronize(s));
        auto c3 = bytes_of(o2, (size_t) T * Hq * D * 4);
        printf("    (%d key splits) ", p1a_attn_prefill_key_splits(T, p0, Hq));
        check("attn_fold (scratch, paged) vs attn_fold (small scratch) vs attn_prefill", a1 && a2 && a3 && p1a_attn_prefill_key_splits(T, p0, Hq) > 1 &&
              !memcmp(a.data(), b.data(), a.size()) && !memcmp(a.data(), c3.data(), a.size()));
        CK(hipFree(scr));
    }
    {   // kv_fill_random: a function of (position range, seed) alone, touching nothing else
        F::kv_cache f1 = F::kv_alloc(type, 512, Hkv, D), f2 = F::kv_alloc(type, 512, Hkv, D);
        F::kv_fill_random(f1, 10, 300, 42u, s);
        F::kv_fill_random(f2, 10, 150, 42u, s);
        F::kv_fill_random(f2, 150, 300, 42u, s);
        CK(hipStreamSynchronize(s));
        auto a = bytes_of(f1.k, 512 * rowb), b = bytes_of(f2.k, 512 * rowb), va = bytes_of(f1.v, 512 * rowb), vb = bytes_of(f2.v, 512 * rowb);
        bool ok = a == b && va == vb;
        for (size_t i = 0; i < 10 * rowb; ++i) ok = ok && a[i] == 0;
        for (size_t i = 300 * rowb; i < 512 * rowb; ++i) ok = ok && a[i] == 0 && va[i] == 0;
        F::kv_fill_random(f2, 10, 300, 43u, s);
        CK(hipStreamSynchronize(s));
        ok = ok && bytes_of(f2.k, 512 * rowb) != a;
        check("kv_fill_random: ranges add up, other rows untouched, seed matters", ok);
        F::kv_free(f1); F::kv_free(f2);
    }
    {   // attn_prep: host positions on the contiguous cache vs device positions through the page table (one sequence)
        const int sq = 2, T = 4, p0 = len[sq] - T, n_rot = 64;
        float * qg = dev_rand((size_t) T * Hq * 2 * D, 1.0f), * kk = dev_rand((size_t) T * Hkv * D, 1.0f), * vv = dev_rand((size_t) T * Hkv * D, 1.0f);
        float * wn = dev_rand((size_t) D, 1.0f), * g1, * g2;
        CK(hipMalloc(&g1, (size_t) T * Hq * D * 4)); CK(hipMalloc(&g2, (size_t) T * Hq * D * 4));
        int32_t * dpos, * drt; CK(hipMalloc(&dpos, 64)); CK(hipMalloc(&drt, 64));
        std::vector<int32_t> hp(T), hr(T, sq * MAXP);
        for (int t = 0; t < T; ++t) hp[t] = p0 + t;
        CK(hipMemcpy(dpos, hp.data(), T * 4, hipMemcpyHostToDevice)); CK(hipMemcpy(drt, hr.data(), T * 4, hipMemcpyHostToDevice));
        F::kv_cache pc = paged(0);
        pc.pt = dtab; pc.rtab = drt;
        const bool a1 = F::attn_prep(qg, kk, vv, wn, wn, dpos, o1, g1, cc[sq], p0, T, Hq, Hkv, D, n_rot, 1e7f, 1e-6f, s);
        const bool a2 = F::attn_prep(qg, kk, vv, wn, wn, dpos, o2, g2, pc, -1, T, Hq, Hkv, D, n_rot, 1e7f, 1e-6f, s);
        CK(hipStreamSynchronize(s));
        bool ok = a1 && a2;
        auto qa = bytes_of(o1, (size_t) T * Hq * D * 4), qb = bytes_of(o2, (size_t) T * Hq * D * 4);
        auto ga = bytes_of(g1, (size_t) T * Hq * D * 4), gb = bytes_of(g2, (size_t) T * Hq * D * 4);
        ok = ok && !memcmp(qa.data(), qb.data(), qa.size()) && !memcmp(ga.data(), gb.data(), ga.size());
        auto hpool = bytes_of(pool, (size_t) NP * pstride);
        auto hk = bytes_of(cc[sq].k, (size_t) len[sq] * rowb), hv = bytes_of(cc[sq].v, (size_t) len[sq] * rowb);
        for (int p = p0; p < p0 + T; ++p) {
            const size_t o = (size_t) tabs[(size_t) sq * MAXP + (p >> PSH)] * pstride + (size_t) 2 * PS * rowb + (size_t) (p & (PS - 1)) * rowb;
            ok = ok && !memcmp(hk.data() + (size_t) p * rowb, hpool.data() + o, rowb);
            ok = ok && !memcmp(hv.data() + (size_t) p * rowb, hpool.data() + o + PS * rowb, rowb);
        }
        check("attn_prep host positions vs device positions + page table", ok);
        {   // text rows through the M-RoPE argument (t = h = w = p) give the plain call's bits
            int32_t * d3; CK(hipMalloc(&d3, 3 * T * 4));
            for (int i = 0; i < 3; ++i) CK(hipMemcpy(d3 + i * T, hp.data(), T * 4, hipMemcpyHostToDevice));
            F::mrope_pos mr; mr.p = d3; mr.stride = T; mr.s0 = 11; mr.s1 = 11; mr.s2 = 10; mr.sect = 32;
            const bool a3 = F::attn_prep(qg, kk, vv, wn, wn, dpos, o2, g2, cc[sq], p0, T, Hq, Hkv, D, n_rot, 1e7f, 1e-6f, s, 0, 0, 0, mr);
            CK(hipStreamSynchronize(s));
            auto qc = bytes_of(o2, (size_t) T * Hq * D * 4);
            check("attn_prep with M-RoPE positions of text rows == plain", a3 && !memcmp(qa.data(), qc.data(), qa.size()));
            CK(hipFree(d3));
        }
        CK(hipFree(qg)); CK(hipFree(kk)); CK(hipFree(vv)); CK(hipFree(wn)); CK(hipFree(g1)); CK(hipFree(g2)); CK(hipFree(dpos)); CK(hipFree(drt));
    }
    {   // the rest of the surface the reference headers declare: the device-position and v2 entry points, the standalone
        // gate and gate + a16 emit, the split-count and environment knobs - each against the call it must equal
        const int sq = 1, T = 3, p0 = 5000;
        int32_t * dp0; CK(hipMalloc(&dp0, 16));
        const int32_t hp0 = p0;
        CK(hipMemcpy(dp0, &hp0, 4, hipMemcpyHostToDevice));
        const size_t ob = (size_t) T * Hq * D * 4;
        F::attn_decode(q, cc[sq], o1, T, p0, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        const auto base = bytes_of(o1, ob);
        const bool d1 = F::attn_decode_dev(q, paged(sq), o2, T, dp0, MAXP * PS, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        check("attn_decode_dev == attn_decode", d1 && bytes_of(o2, ob) == base);
        CK(hipMemset(o2, 0, ob));
        const bool d2 = F::attn_decode2(q, cc[sq], o2, T, p0, nullptr, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        const bool d2a = d2 && bytes_of(o2, ob) == base;
        CK(hipMemset(o2, 0, ob));
        const bool d3 = F::attn_decode2(q, paged(sq), o2, T, 0, dp0, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        check("attn_decode2 (host and device p0) == attn_decode", d2a && d3 && bytes_of(o2, ob) == base);
        {   // kv_append_dev writes the rows kv_append writes
            F::kv_cache a1 = F::kv_alloc(type, 64, Hkv, D), a2 = F::kv_alloc(type, 64, Hkv, D);
            float * ks = dev_rand((size_t) T * Hkv * D, 1.0f), * vs = dev_rand((size_t) T * Hkv * D, 1.0f);
            const int32_t h7 = 7;
            CK(hipMemcpy(dp0, &h7, 4, hipMemcpyHostToDevice));
            F::kv_append(a1, ks, vs, 7, T, s);
            F::kv_append_dev(a2, ks, vs, dp0, T, s);
            CK(hipStreamSynchronize(s));
            check("kv_append_dev == kv_append", bytes_of(a1.k, 64 * rowb) == bytes_of(a2.k, 64 * rowb) && bytes_of(a1.v, 64 * rowb) == bytes_of(a2.v, 64 * rowb));
            F::kv_free(a1); F::kv_free(a2); CK(hipFree(ks)); CK(hipFree(vs));
        }
        {   // the fused gate of attn_decode == attn_decode followed by sigmoid_mul; ew_quant(EW_SIGMOID_MUL) writes the same rows
            float * gt = dev_rand((size_t) T * Hq * D, 1.0f), * o3;
            void * qb; CK(hipMalloc(&qb, p1a_a16_bytes(T, Hq * D))); CK(hipMalloc(&o3, ob));
            F::attn_decode(q, cc[sq], o2, T, p0, Hq, scale, s, gt);
            F::sigmoid_mul(o1, gt, (int64_t) T * Hq * D, s);      // o1 holds the ungated rows
            CK(hipStreamSynchronize(s));
            const auto fused = bytes_of(o2, ob);
            check("attn_decode with gate == attn_decode + sigmoid_mul", fused == bytes_of(o1, ob));
            CK(hipMemcpy(o1, base.data(), ob, hipMemcpyHostToDevice));
            const bool e1 = F::ew_quant(F::EW_SIGMOID_MUL, o1, gt, o3, qb, T, Hq * D, s);
            CK(hipStreamSynchronize(s));
            check("ew_quant(EW_SIGMOID_MUL) rows == the fused gate's", e1 && bytes_of(o3, ob) == fused);
            CK(hipFree(gt)); CK(hipFree(qb)); CK(hipFree(o3));
        }
        {   // attn_prefill_variant is attn_prefill; the split-count knobs; the environment re-read
            const int Tp = 70, pp = 900;
            const bool v1 = F::attn_prefill(q, cc[sq], o1, Tp, pp, Hq, scale, s), v2 = F::attn_prefill_variant(q, cc[sq], o2, Tp, pp, Hq, scale, s, 2);
            CK(hipStreamSynchronize(s));
            check("attn_prefill_variant == attn_prefill", v1 && v2 && bytes_of(o1, (size_t) Tp * Hq * D * 4) == bytes_of(o2, (size_t) Tp * Hq * D * 4));
            const int n0 = F::attn_dec2_nsplit(Hkv);
            F::attn_dec2_set_nsplit(16);
            const bool k1 = F::attn_dec2_nsplit(Hkv) == 16;
            F::attn_dec2_set_nsplit(0);
            const bool k2 = F::attn_dec2_nsplit(Hkv) == n0 && n0 >= 8;
            (void) F::attn_dec2_reload_env();
            setenv("P1A_DEC_SPLIT", "24", 1);
            const bool r1 = F::attn_dec2_reload_env(), k3 = F::attn_dec2_nsplit(Hkv) == 24, r2 = F::attn_dec2_reload_env();
            unsetenv("P1A_DEC_SPLIT");
            const bool r3 = F::attn_dec2_reload_env(), k4 = F::attn_dec2_nsplit(Hkv) == n0;
            check("attn_dec2_nsplit / set_nsplit / reload_env", k1 && k2 && r1 && k3 && !r2 && r3 && k4);
        }
        {   // kv_append_rows: rows of two sequences at their own positions == kv_append into each
            int32_t * dpos, * drt; CK(hipMalloc(&dpos, 64)); CK(hipMalloc(&drt, 64));
            const int32_t hp[2] = {len[0], len[2]}, hr[2] = {0 * MAXP, 2 * MAXP};
            CK(hipMemcpy(dpos, hp, 8, hipMemcpyHostToDevice)); CK(hipMemcpy(drt, hr, 8, hipMemcpyHostToDevice));
            float * ks = dev_rand((size_t) 2 * Hkv * D, 1.0f), * vs = dev_rand((size_t) 2 * Hkv * D, 1.0f);
            F::kv_cache pc = paged(0);
            pc.pt = dtab; pc.rtab = drt;
            const bool a = F::kv_append_rows(pc, ks, vs, dpos, 2, s);
            F::kv_append(cc[0], ks, vs, len[0], 1, s);
            F::kv_append(cc[2], ks + (size_t) Hkv * D, vs + (size_t) Hkv * D, len[2], 1, s);
            CK(hipStreamSynchronize(s));
            auto hpool = bytes_of(pool, (size_t) NP * pstride);
            bool ok = a;
            for (int i = 0; i < 2; ++i) {
                const int sq2 = i ? 2 : 0, p = len[sq2];
                const size_t o = (size_t) tabs[(size_t) sq2 * MAXP + (p >> PSH)] * pstride + (size_t) 2 * PS * rowb + (size_t) (p & (PS - 1)) * rowb;
                auto hk = bytes_of((char *) cc[sq2].k + (size_t) p * rowb, rowb), hv = bytes_of((char *) cc[sq2].v + (size_t) p * rowb, rowb);
                ok = ok && !memcmp(hk.data(), hpool.data() + o, rowb) && !memcmp(hv.data(), hpool.data() + o + PS * rowb, rowb);
            }
            check("kv_append_rows == kv_append per sequence", ok);
            CK(hipFree(dpos)); CK(hipFree(drt)); CK(hipFree(ks)); CK(hipFree(vs));
        }
        CK(hipFree(dp0));
    }
    {   // a refusal launches nothing and leaves out untouched
        CK(hipMemset(o1, 0x5a, 4096));
        const bool r = F::attn_decode(q, cc[0], o1, 1, 10, Hq + 1, scale, s);
        CK(hipStreamSynchronize(s));
        auto a = bytes_of(o1, 4096);
        check("unsupported shape is refused, out untouched", !r && std::all_of(a.begin(), a.end(), [](char x) { return x == 0x5a; }));
    }
    for (int i = 0; i < NS; ++i) F::kv_free(cc[i]);
    CK(hipFree(q)); CK(hipFree(o1)); CK(hipFree(o2)); CK(hipFree(pool)); CK(hipFree(dtab));
}

// The pool / sequence manager (include/p100e_kv_pool.hpp) under the attention entry points, in the manner of the
// reference's tests/fast_sessions_test.cu: two sequences grown in turns (interleaved pages), every step appended to the
// pool's descriptors and to a contiguous cache; then bitwise checks of decode results across fork, offload + restore
// (onto other pages) and a session file read into a pool of another size.
static void test_pool(uint32_t type, hipStream_t s) {
    printf("  pool %s\n", tname(type));
    const int L = 2, Hq = 8, Hkv = 2, D = 256, PSH = 4, NCTX = 400, il = 1;
    const float scale = 0.0625f;
    p100e::kv_pool pool(type, L, Hkv, D, PSH, NCTX, 3, s, 64);
    pool.alloc_pool(16 * 40);
    pool.set_fingerprint({1, 2, 3, 4, 5000, 0, 0, 0, 0, 0, 0, 1, 7, 8, 9});
    const int a = pool.seq_create(), b = pool.seq_create();
    F::kv_cache ca = F::kv_alloc(type, NCTX, Hkv, D), cb = F::kv_alloc(type, NCTX, Hkv, D);
    const int steps[] = {37, 1, 20, 64, 3, 51};
    int na = 0, nb = 0;
    for (int st = 0; st < 6; ++st) {
        const int T = steps[st];
        for (int which = 0; which < 2; ++which) {
            const int id = which ? b : a;
            int & n = which ? nb : na;
            float * k = dev_rand((size_t) T * Hkv * D, 1.0f), * v = dev_rand((size_t) T * Hkv * D, 1.0f);
            pool.advance(id, std::vector<int32_t>(T, 100 + st));
            for (int l = 0; l < L; ++l) { F::kv_cache pc = pool.kv_seq(l, id); F::kv_append(pc, l == il ? k : v, l == il ? v : k, n, T, s); }
            F::kv_append(which ? cb : ca, k, v, n, T, s);
            CK(hipStreamSynchronize(s));
            CK(hipFree(k)); CK(hipFree(v));
            n += T;
        }
    }
    float * q = dev_rand((size_t) 4 * Hq * D, 0.3f);
    float * o1, * o2;
    CK(hipMalloc(&o1, (size_t) 4 * Hq * D * 4)); CK(hipMalloc(&o2, (size_t) 4 * Hq * D * 4));
    auto dec = [&](const F::kv_cache & c, float * o, int T, int p0) {
        const bool ok = F::attn_decode(q, c, o, T, p0, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        return ok;
    };
    auto same = [&](int T) { auto x = bytes_of(o1, (size_t) T * Hq * D * 4), y = bytes_of(o2, (size_t) T * Hq * D * 4); return !memcmp(x.data(), y.data(), x.size()); };
    bool ok = dec(ca, o1, 4, na - 4) && dec(pool.kv_seq(il, a), o2, 4, na - 4);
    check("pool descriptors: decode == contiguous cache (interleaved pages)", ok && same(4));
    ok = dec(cb, o1, 1, nb - 1) && dec(pool.kv_seq(il, b), o2, 1, nb - 1);
    check("second sequence", ok && same(1));
    {   // rows of both sequences in one call through the row table
        pool.set_rows({b, a, a});
        int32_t hp[3] = {nb - 1, na - 2, na - 1}, * dpos;
        CK(hipMalloc(&dpos, 12)); CK(hipMemcpy(dpos, hp, 12, hipMemcpyHostToDevice));
        ok = F::attn_decode_rows(q, pool.kv_rows(il), o2, 3, dpos, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        auto rows = bytes_of(o2, (size_t) 3 * Hq * D * 4);
        const size_t rb = (size_t) Hq * D * 4;
        const F::kv_cache * cc[3] = {&cb, &ca, &ca};
        for (int t = 0; t < 3 && ok; ++t) {
            float * qt = q + (size_t) t * Hq * D;
            ok = F::attn_decode(qt, *cc[t], o1, 1, hp[t], Hq, scale, s);
            CK(hipStreamSynchronize(s));
            auto one = bytes_of(o1, rb);
            ok = ok && !memcmp(one.data(), rows.data() + t * rb, rb);
        }
        check("kv_rows + set_rows: batched rows == one call per row", ok);
        CK(hipFree(dpos));
    }
    const int nf = 100;
    const int f = pool.seq_fork(a, nf);
    ok = dec(ca, o1, 1, nf - 1) && dec(pool.kv_seq(il, f), o2, 1, nf - 1);
    check("seq_fork: the copy decodes like the source", ok && same(1) && pool.seq_len(f) == nf);
    ok = dec(ca, o1, 4, na - 4);
    pool.seq_free(f);
    pool.seq_offload(a);
    const int filler = pool.seq_create();
    pool.ensure_pages(filler, 16 * 5);            // the restored sequence lands on other pages
    pool.seq_restore(a);
    ok = ok && dec(pool.kv_seq(il, a), o2, 4, na - 4);
    check("seq_offload + seq_restore onto other pages", ok && same(4) && pool.host_used() == 0);
    {
        const std::string path = "/tmp/p1a_mirror_check.p100esq";
        pool.seq_write(a, path);
        p100e::kv_pool pool2(type, L, Hkv, D, PSH, 1000, 2, s, 64);
        pool2.alloc_pool(16 * 64);
        pool2.set_fingerprint({1, 2, 3, 4, 5000, 0, 0, 0, 0, 0, 0, 1, 7, 8, 9});
        const int x = pool2.seq_create();
        pool2.ensure_pages(x, 50);
        const int r = pool2.seq_read(path);
        pool2.seq_restore(r);
        ok = dec(ca, o1, 4, na - 4) && dec(pool2.kv_seq(il, r), o2, 4, na - 4);
        check("seq_write -> seq_read into a pool of another size", ok && same(4) && pool2.seq_len(r) == na);
        bool refused = false;
        p100e::kv_pool pool3(type, L, Hkv, D, PSH + 1, 1000, 2, s, 64);
        pool3.alloc_pool(32 * 8);
        pool3.set_fingerprint({1, 2, 3, 4, 5000, 0, 0, 0, 0, 0, 0, 1, 7, 8, 9});
        try { pool3.seq_read(path); } catch (const std::runtime_error & e) { refused = strstr(e.what(), "page shift") != nullptr; }
        check("a file of another page size is refused by name", refused);
        remove(path.c_str());
    }
    bool threw = false;
    try { pool.ensure_pages(a, NCTX + 1); } catch (const std::runtime_error & e) { threw = !strcmp(e.what(), "context full"); }
    check("refusals throw the engine's messages", threw);
    F::kv_free(ca); F::kv_free(cb);
    CK(hipFree(q)); CK(hipFree(o1)); CK(hipFree(o2));
}

int main() {
    hipStream_t s; CK(hipStreamCreate(&s));
    for (uint32_t type : {F::KV_F16, F::KV_Q8_0, F::KV_Q4_0}) test_type(type, s);
    for (uint32_t type : {F::KV_F16, F::KV_Q8_0, F::KV_Q4_0}) test_pool(type, s);
    p1a_release();
    printf("%d checks, %d failed\n", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
