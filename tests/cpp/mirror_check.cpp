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
#include <vector>

#include "p100e_fast_attn.hpp"

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
        CK(hipFree(qg)); CK(hipFree(kk)); CK(hipFree(vv)); CK(hipFree(wn)); CK(hipFree(g1)); CK(hipFree(g2)); CK(hipFree(dpos)); CK(hipFree(drt));
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

int main() {
    hipStream_t s; CK(hipStreamCreate(&s));
    for (uint32_t type : {F::KV_F16, F::KV_Q8_0, F::KV_Q4_0}) test_type(type, s);
    p1a_release();
    printf("%d checks, %d failed\n", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
