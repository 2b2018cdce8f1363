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
// test inputs: a xorshift generator; values are a centred sum of four uniforms (bell-shaped, |x| < 2 s)
static uint64_t g_state = 0x9e3779b97f4a7c15ull;
static uint32_t next_u32() { g_state ^= g_state << 13; g_state ^= g_state >> 7; g_state ^= g_state << 17; return (uint32_t) (g_state >> 24); }
static float bell(float s) {
    float a = 0.0f;
    for (int i = 0; i < 4; ++i) a += (float) (next_u32() & 0xfffffu) * (1.0f / 1048576.0f);
    return (a - 2.0f) * s;
}
static float * upload_noise(size_t n, float s) {
    std::vector<float> h(n);
    for (size_t i = 0; i < n; ++i) h[i] = bell(s);
    float * d = nullptr;
    CK(hipMalloc(&d, n * sizeof(float)));
    CK(hipMemcpy(d, h.data(), n * sizeof(float), hipMemcpyHostToDevice));
    return d;
}
static std::vector<char> fetch(const void * d, size_t n) {
    std::vector<char> h(n);
    CK(hipMemcpy(h.data(), d, n, hipMemcpyDeviceToHost));
    return h;
}
static void check(const char * name, bool ok) { ++g_checks; if (!ok) ++g_fail; printf("    %-62s %s\n", name, ok ? "identical" : "FAIL"); }
static const char * kv_name(uint32_t t) { return t == F::KV_Q8_0 ? "q8_0" : t == F::KV_Q4_0 ? "q4_0" : "f16"; }

// One KV type end to end through the reference-shaped calls. Four sequences of unequal length live in one pool of
// 64-token pages that interleaves three layers (the third is used); pages are dealt to the sequences in turns through a
// stride-37 scatter, so neighbouring pages of a sequence are far apart and belong to different sequences in between.
// Every sequence also has a contiguous twin (kv_alloc) that receives the same appends.
static void test_type(uint32_t type, hipStream_t s) {
    printf("paged KV cache, %s\n", kv_name(type));
    const int Hkv = 4, D = 256, Hq = 16, PSH = 6, PS = 1 << PSH, NLAY = 3, LAYER = 2;
    const int NS = 4, n_tok[NS] = {433, 9100, 1290, 77};
    const int MAXP = 160, NP = 192;
    const float scale = 1.0f / 16.0f;
    const size_t rowb = F::kv_row_bytes(type, Hkv, D);
    const size_t pstride = (size_t) NLAY * 2 * PS * rowb;            // a page of every layer's K and V, back to back
    const size_t k_off = (size_t) LAYER * 2 * PS * rowb, v_off = k_off + (size_t) PS * rowb;
    char * pool = nullptr;
    CK(hipMalloc(&pool, (size_t) NP * pstride));
    CK(hipMemset(pool, 0, (size_t) NP * pstride));
    std::vector<int32_t> page_rows((size_t) NS * MAXP, 0);
    {
        int dealt = 0, have[NS] = {0, 0, 0, 0};
        for (bool more = true; more;) {
            more = false;
            for (int q = 0; q < NS; ++q) {
                if (have[q] > n_tok[q] / PS + 1) continue;            // one page beyond the last token
                page_rows[(size_t) q * MAXP + have[q]++] = (int32_t) ((dealt++ * 37) % NP);
                more = true;
            }
        }
        if (dealt > NP) { printf("pool too small\n"); exit(2); }
    }
    int32_t * d_page_rows = nullptr;
    CK(hipMalloc(&d_page_rows, page_rows.size() * 4));
    CK(hipMemcpy(d_page_rows, page_rows.data(), page_rows.size() * 4, hipMemcpyHostToDevice));
    // where position p of sequence q sits in the pool (K; V is v_off - k_off further)
    auto row_at = [&](int q, int p) { return (size_t) page_rows[(size_t) q * MAXP + (p >> PSH)] * pstride + k_off + (size_t) (p & (PS - 1)) * rowb; };
    auto slot_view = [&](int q) {
        F::kv_cache c;
        c.type = type; c.n_ctx = MAXP * PS; c.Hkv = Hkv; c.D = D;
        c.k = pool + k_off; c.v = pool + v_off;
        c.pt = d_page_rows + (size_t) q * MAXP; c.psh = PSH; c.pstride = pstride;
        return c;
    };
    std::vector<F::kv_cache> flat(NS);
    for (int q = 0; q < NS; ++q) {
        flat[q] = F::kv_alloc(type, MAXP * PS, Hkv, D);
        const size_t n = (size_t) n_tok[q] * Hkv * D;
        float * ks = upload_noise(n, 1.0f), * vs = upload_noise(n, 1.0f);
        F::kv_cache pc = slot_view(q);
        for (int p = 0; p < n_tok[q]; p += 48) {                      // chunks that straddle pages
            const int T = std::min(48, n_tok[q] - p);
            F::kv_append(flat[q], ks + (size_t) p * Hkv * D, vs + (size_t) p * Hkv * D, p, T, s);
            F::kv_append(pc, ks + (size_t) p * Hkv * D, vs + (size_t) p * Hkv * D, p, T, s);
        }
        CK(hipStreamSynchronize(s));
        CK(hipFree(ks)); CK(hipFree(vs));
    }
    {
        const auto hpool = fetch(pool, (size_t) NP * pstride);
        bool same = true;
        for (int q = 0; q < NS; ++q) {
            const auto hk = fetch(flat[q].k, (size_t) n_tok[q] * rowb), hv = fetch(flat[q].v, (size_t) n_tok[q] * rowb);
            for (int p = 0; p < n_tok[q]; ++p)
                same = same && !memcmp(&hk[(size_t) p * rowb], &hpool[row_at(q, p)], rowb) &&
                       !memcmp(&hv[(size_t) p * rowb], &hpool[row_at(q, p) + (v_off - k_off)], rowb);
        }
        check("kv_append paged vs contiguous (every position, K and V)", same);
    }
    float * q = upload_noise((size_t) 256 * Hq * D, 1.5f);
    float * o1 = nullptr, * o2 = nullptr;
    CK(hipMalloc(&o1, (size_t) 256 * Hq * D * 4));
    CK(hipMalloc(&o2, (size_t) 256 * Hq * D * 4));
    {   // decode / verify blocks of 1 .. 4 rows, at depths on both sides of page and split-unit boundaries
        int cases = 0, differ = 0;
        const int depths[] = {0, 1, 62, 63, 64, 65, 127, 128, 400, 2047, 2048, 4095, 4100, 9000};
        for (int sq = 0; sq < NS; ++sq)
            for (int T = 1; T <= 4; ++T) {
                std::vector<int> at(depths, depths + sizeof depths / sizeof depths[0]);
                at.push_back(n_tok[sq] - T);
                for (int p0 : at) {
                    if (p0 < 0 || p0 + T > n_tok[sq]) continue;
                    const bool r1 = F::attn_decode(q, flat[sq], o1, T, p0, Hq, scale, s);
                    const bool r2 = F::attn_decode(q, slot_view(sq), o2, T, p0, Hq, scale, s);
                    CK(hipStreamSynchronize(s));
                    ++cases;
                    if (!r1 || !r2 || fetch(o1, (size_t) T * Hq * D * 4) != fetch(o2, (size_t) T * Hq * D * 4)) ++differ;
                }
            }
        printf("    (%d cases) ", cases);
        check("attn_decode T=1..4 paged vs contiguous", differ == 0);
    }
    {   // attn_decode_rows: rows of several sequences in one call, each at its own depth, against one T = 1 call per row
        struct at { int seq, pos; };
        const std::vector<std::vector<at>> batches = {
            {{3, 76}},
            {{1, 9099}, {0, 432}, {3, 0}, {2, 1289}},
            {{2, 640}, {2, 641}, {2, 642}, {1, 63}, {1, 64}},
            {{0, 100}, {1, 5000}, {2, 1000}, {3, 50}, {0, 101}, {1, 5001}, {2, 1001}, {3, 51}},
            {{1, 8191}, {1, 8192}},
        };
        int32_t * dpos = nullptr, * drt = nullptr;
        CK(hipMalloc(&dpos, 64)); CK(hipMalloc(&drt, 64));
        int differ = 0;
        for (const auto & batch : batches) {
            const int T = (int) batch.size();
            std::vector<int32_t> hp, hr;
            for (const at & r : batch) { hp.push_back(r.pos); hr.push_back(r.seq * MAXP); }
            CK(hipMemcpy(dpos, hp.data(), T * 4, hipMemcpyHostToDevice));
            CK(hipMemcpy(drt, hr.data(), T * 4, hipMemcpyHostToDevice));
            F::kv_cache all = slot_view(0);
            all.pt = d_page_rows; all.rtab = drt;
            if (!F::attn_decode_rows(q, all, o2, T, dpos, Hq, scale, s)) { ++differ; continue; }
            CK(hipStreamSynchronize(s));
            const auto rows = fetch(o2, (size_t) T * Hq * D * 4);
            for (int t = 0; t < T; ++t) {
                F::attn_decode(q + (size_t) t * Hq * D, flat[batch[t].seq], o1, 1, batch[t].pos, Hq, scale, s);
                CK(hipStreamSynchronize(s));
                const auto one = fetch(o1, (size_t) Hq * D * 4);
                if (memcmp(one.data(), &rows[(size_t) t * Hq * D * 4], one.size())) ++differ;
            }
        }
        check("attn_decode_rows (4 sequences, 1..8 rows) vs T=1 per row", differ == 0);
        CK(hipFree(dpos)); CK(hipFree(drt));
    }
    {
        const int sq = 1, T = 150, p0 = 2000;
        const bool r1 = F::attn_prefill(q, flat[sq], o1, T, p0, Hq, scale, s), r2 = F::attn_prefill(q, slot_view(sq), o2, T, p0, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        check("attn_prefill T=150 p0=2000 paged vs contiguous", r1 && r2 && fetch(o1, (size_t) T * Hq * D * 4) == fetch(o2, (size_t) T * Hq * D * 4));
    }
    {   // attn_fold on a short chunk over a long context (the library splits it over the keys): with the scratch of
        // attn_fold_scratch_bytes, with a scratch that is too small and through attn_prefill - one result, bit for bit
        const int sq = 1, T = 100, p0 = n_tok[sq] - T;
        const size_t nb = F::attn_fold_scratch_bytes(T, Hkv, 2048, 8, p0);
        void * scr; CK(hipMalloc(&scr, nb)); CK(hipMemset(scr, 0xff, nb));
        const bool a1 = F::attn_prefill(q, flat[sq], o1, T, p0, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        auto a = fetch(o1, (size_t) T * Hq * D * 4);
        const bool a2 = F::attn_fold(q, slot_view(sq), o2, T, p0, Hq, scale, scr, nb, s);
        CK(hipStreamSynchronize(s));
        auto b = fetch(o2, (size_t) T * Hq * D * 4);
        const bool a3 = F::attn_fold(q, flat[sq], o2, T, p0, Hq, scale, scr, 4096, s);
        CK(hipStreamSynchronize(s));
        auto c3 = fetch(o2, (size_t) T * Hq * D * 4);
        printf("    (%d key splits) ", p1a_attn_prefill_key_splits(T, p0, Hq));
        check("attn_fold (scratch, slot_view) vs attn_fold (small scratch) vs attn_prefill", a1 && a2 && a3 && p1a_attn_prefill_key_splits(T, p0, Hq) > 1 &&
              !memcmp(a.data(), b.data(), a.size()) && !memcmp(a.data(), c3.data(), a.size()));
        CK(hipFree(scr));
    }
    {   // kv_fill_random: a function of (position range, seed) alone, touching nothing else
        F::kv_cache f1 = F::kv_alloc(type, 512, Hkv, D), f2 = F::kv_alloc(type, 512, Hkv, D);
        F::kv_fill_random(f1, 10, 300, 42u, s);
        F::kv_fill_random(f2, 10, 150, 42u, s);
        F::kv_fill_random(f2, 150, 300, 42u, s);
        CK(hipStreamSynchronize(s));
        auto a = fetch(f1.k, 512 * rowb), b = fetch(f2.k, 512 * rowb), va = fetch(f1.v, 512 * rowb), vb = fetch(f2.v, 512 * rowb);
        bool ok = a == b && va == vb;
        for (size_t i = 0; i < 10 * rowb; ++i) ok = ok && a[i] == 0;
        for (size_t i = 300 * rowb; i < 512 * rowb; ++i) ok = ok && a[i] == 0 && va[i] == 0;
        F::kv_fill_random(f2, 10, 300, 43u, s);
        CK(hipStreamSynchronize(s));
        ok = ok && fetch(f2.k, 512 * rowb) != a;
        check("kv_fill_random: ranges add up, other rows untouched, seed matters", ok);
        F::kv_free(f1); F::kv_free(f2);
    }
    {   // attn_prep: host positions on the contiguous cache vs device positions through the page table (one sequence)
        const int sq = 2, T = 4, p0 = n_tok[sq] - T, n_rot = 64;
        float * qg = upload_noise((size_t) T * Hq * 2 * D, 1.0f), * kk = upload_noise((size_t) T * Hkv * D, 1.0f), * vv = upload_noise((size_t) T * Hkv * D, 1.0f);
        float * wn = upload_noise((size_t) D, 1.0f), * g1, * g2;
        CK(hipMalloc(&g1, (size_t) T * Hq * D * 4)); CK(hipMalloc(&g2, (size_t) T * Hq * D * 4));
        int32_t * dpos, * drt; CK(hipMalloc(&dpos, 64)); CK(hipMalloc(&drt, 64));
        std::vector<int32_t> hp(T), hr(T, sq * MAXP);
        for (int t = 0; t < T; ++t) hp[t] = p0 + t;
        CK(hipMemcpy(dpos, hp.data(), T * 4, hipMemcpyHostToDevice)); CK(hipMemcpy(drt, hr.data(), T * 4, hipMemcpyHostToDevice));
        F::kv_cache pc = slot_view(0);
        pc.pt = d_page_rows; pc.rtab = drt;
        const bool a1 = F::attn_prep(qg, kk, vv, wn, wn, dpos, o1, g1, flat[sq], p0, T, Hq, Hkv, D, n_rot, 1e7f, 1e-6f, s);
        const bool a2 = F::attn_prep(qg, kk, vv, wn, wn, dpos, o2, g2, pc, -1, T, Hq, Hkv, D, n_rot, 1e7f, 1e-6f, s);
        CK(hipStreamSynchronize(s));
        bool ok = a1 && a2;
        auto qa = fetch(o1, (size_t) T * Hq * D * 4), qb = fetch(o2, (size_t) T * Hq * D * 4);
        auto ga = fetch(g1, (size_t) T * Hq * D * 4), gb = fetch(g2, (size_t) T * Hq * D * 4);
        ok = ok && !memcmp(qa.data(), qb.data(), qa.size()) && !memcmp(ga.data(), gb.data(), ga.size());
        auto hpool = fetch(pool, (size_t) NP * pstride);
        auto hk = fetch(flat[sq].k, (size_t) n_tok[sq] * rowb), hv = fetch(flat[sq].v, (size_t) n_tok[sq] * rowb);
        for (int p = p0; p < p0 + T; ++p) {
            const size_t o = row_at(sq, p);
            ok = ok && !memcmp(hk.data() + (size_t) p * rowb, hpool.data() + o, rowb);
            ok = ok && !memcmp(hv.data() + (size_t) p * rowb, hpool.data() + o + (v_off - k_off), rowb);
        }
        check("attn_prep host positions vs device positions + page table", ok);
        {   // text rows through the M-RoPE argument (t = h = w = p) give the plain call's bits
            int32_t * d3; CK(hipMalloc(&d3, 3 * T * 4));
            for (int i = 0; i < 3; ++i) CK(hipMemcpy(d3 + i * T, hp.data(), T * 4, hipMemcpyHostToDevice));
            F::mrope_pos mr; mr.p = d3; mr.stride = T; mr.s0 = 11; mr.s1 = 11; mr.s2 = 10; mr.sect = 32;
            const bool a3 = F::attn_prep(qg, kk, vv, wn, wn, dpos, o2, g2, flat[sq], p0, T, Hq, Hkv, D, n_rot, 1e7f, 1e-6f, s, 0, 0, 0, mr);
            CK(hipStreamSynchronize(s));
            auto qc = fetch(o2, (size_t) T * Hq * D * 4);
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
        F::attn_decode(q, flat[sq], o1, T, p0, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        const auto base = fetch(o1, ob);
        const bool d1 = F::attn_decode_dev(q, slot_view(sq), o2, T, dp0, MAXP * PS, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        check("attn_decode_dev == attn_decode", d1 && fetch(o2, ob) == base);
        CK(hipMemset(o2, 0, ob));
        const bool d2 = F::attn_decode2(q, flat[sq], o2, T, p0, nullptr, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        const bool d2a = d2 && fetch(o2, ob) == base;
        CK(hipMemset(o2, 0, ob));
        const bool d3 = F::attn_decode2(q, slot_view(sq), o2, T, 0, dp0, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        check("attn_decode2 (host and device p0) == attn_decode", d2a && d3 && fetch(o2, ob) == base);
        {   // kv_append_dev writes the rows kv_append writes
            F::kv_cache a1 = F::kv_alloc(type, 64, Hkv, D), a2 = F::kv_alloc(type, 64, Hkv, D);
            float * ks = upload_noise((size_t) T * Hkv * D, 1.0f), * vs = upload_noise((size_t) T * Hkv * D, 1.0f);
            const int32_t h7 = 7;
            CK(hipMemcpy(dp0, &h7, 4, hipMemcpyHostToDevice));
            F::kv_append(a1, ks, vs, 7, T, s);
            F::kv_append_dev(a2, ks, vs, dp0, T, s);
            CK(hipStreamSynchronize(s));
            check("kv_append_dev == kv_append", fetch(a1.k, 64 * rowb) == fetch(a2.k, 64 * rowb) && fetch(a1.v, 64 * rowb) == fetch(a2.v, 64 * rowb));
            F::kv_free(a1); F::kv_free(a2); CK(hipFree(ks)); CK(hipFree(vs));
        }
        {   // the fused gate of attn_decode == attn_decode followed by sigmoid_mul; ew_quant(EW_SIGMOID_MUL) writes the same rows
            float * gt = upload_noise((size_t) T * Hq * D, 1.0f), * o3;
            void * qb; CK(hipMalloc(&qb, p1a_a16_bytes(T, Hq * D))); CK(hipMalloc(&o3, ob));
            F::attn_decode(q, flat[sq], o2, T, p0, Hq, scale, s, gt);
            F::sigmoid_mul(o1, gt, (int64_t) T * Hq * D, s);      // o1 holds the ungated rows
            CK(hipStreamSynchronize(s));
            const auto fused = fetch(o2, ob);
            check("attn_decode with gate == attn_decode + sigmoid_mul", fused == fetch(o1, ob));
            CK(hipMemcpy(o1, base.data(), ob, hipMemcpyHostToDevice));
            const bool e1 = F::ew_quant(F::EW_SIGMOID_MUL, o1, gt, o3, qb, T, Hq * D, s);
            CK(hipStreamSynchronize(s));
            check("ew_quant(EW_SIGMOID_MUL) rows == the fused gate's", e1 && fetch(o3, ob) == fused);
            CK(hipFree(gt)); CK(hipFree(qb)); CK(hipFree(o3));
        }
        {   // attn_prefill_variant is attn_prefill; the split-count knobs; the environment re-read
            const int Tp = 70, pp = 900;
            const bool v1 = F::attn_prefill(q, flat[sq], o1, Tp, pp, Hq, scale, s), v2 = F::attn_prefill_variant(q, flat[sq], o2, Tp, pp, Hq, scale, s, 2);
            CK(hipStreamSynchronize(s));
            check("attn_prefill_variant == attn_prefill", v1 && v2 && fetch(o1, (size_t) Tp * Hq * D * 4) == fetch(o2, (size_t) Tp * Hq * D * 4));
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
            const int32_t hp[2] = {n_tok[0], n_tok[2]}, hr[2] = {0 * MAXP, 2 * MAXP};
            CK(hipMemcpy(dpos, hp, 8, hipMemcpyHostToDevice)); CK(hipMemcpy(drt, hr, 8, hipMemcpyHostToDevice));
            float * ks = upload_noise((size_t) 2 * Hkv * D, 1.0f), * vs = upload_noise((size_t) 2 * Hkv * D, 1.0f);
            F::kv_cache pc = slot_view(0);
            pc.pt = d_page_rows; pc.rtab = drt;
            const bool a = F::kv_append_rows(pc, ks, vs, dpos, 2, s);
            F::kv_append(flat[0], ks, vs, n_tok[0], 1, s);
            F::kv_append(flat[2], ks + (size_t) Hkv * D, vs + (size_t) Hkv * D, n_tok[2], 1, s);
            CK(hipStreamSynchronize(s));
            auto hpool = fetch(pool, (size_t) NP * pstride);
            bool ok = a;
            for (int i = 0; i < 2; ++i) {
                const int sq2 = i ? 2 : 0, p = n_tok[sq2];
                const size_t o = row_at(sq2, p);
                auto hk = fetch((char *) flat[sq2].k + (size_t) p * rowb, rowb), hv = fetch((char *) flat[sq2].v + (size_t) p * rowb, rowb);
                ok = ok && !memcmp(hk.data(), hpool.data() + o, rowb) && !memcmp(hv.data(), hpool.data() + o + (v_off - k_off), rowb);
            }
            check("kv_append_rows == kv_append per sequence", ok);
            CK(hipFree(dpos)); CK(hipFree(drt)); CK(hipFree(ks)); CK(hipFree(vs));
        }
        CK(hipFree(dp0));
    }
    {   // a refusal launches nothing and leaves out untouched
        CK(hipMemset(o1, 0x5a, 4096));
        const bool r = F::attn_decode(q, flat[0], o1, 1, 10, Hq + 1, scale, s);
        CK(hipStreamSynchronize(s));
        auto a = fetch(o1, 4096);
        check("unsupported shape is refused, out untouched", !r && std::all_of(a.begin(), a.end(), [](char x) { return x == 0x5a; }));
    }
    for (int i = 0; i < NS; ++i) F::kv_free(flat[i]);
    CK(hipFree(q)); CK(hipFree(o1)); CK(hipFree(o2)); CK(hipFree(pool)); CK(hipFree(d_page_rows));
}

// The pool / sequence manager (include/p100e_kv_pool.hpp) under the attention entry points, in the manner of the
// reference's tests/fast_sessions_test.cu: two sequences grown in turns (interleaved pages), every step appended to the
// pool's descriptors and to a contiguous cache; then bitwise checks of decode results across fork, offload + restore
// (onto other pages) and a session file read into a pool of another size.
static void test_pool(uint32_t type, hipStream_t s) {
    printf("  pool %s\n", kv_name(type));
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
            float * k = upload_noise((size_t) T * Hkv * D, 1.0f), * v = upload_noise((size_t) T * Hkv * D, 1.0f);
            pool.advance(id, std::vector<int32_t>(T, 100 + st));
            for (int l = 0; l < L; ++l) { F::kv_cache pc = pool.kv_seq(l, id); F::kv_append(pc, l == il ? k : v, l == il ? v : k, n, T, s); }
            F::kv_append(which ? cb : ca, k, v, n, T, s);
            CK(hipStreamSynchronize(s));
            CK(hipFree(k)); CK(hipFree(v));
            n += T;
        }
    }
    float * q = upload_noise((size_t) 4 * Hq * D, 0.3f);
    float * o1, * o2;
    CK(hipMalloc(&o1, (size_t) 4 * Hq * D * 4)); CK(hipMalloc(&o2, (size_t) 4 * Hq * D * 4));
    auto dec = [&](const F::kv_cache & c, float * o, int T, int p0) {
        const bool ok = F::attn_decode(q, c, o, T, p0, Hq, scale, s);
        CK(hipStreamSynchronize(s));
        return ok;
    };
    auto same = [&](int T) { auto x = fetch(o1, (size_t) T * Hq * D * 4), y = fetch(o2, (size_t) T * Hq * D * 4); return !memcmp(x.data(), y.data(), x.size()); };
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
        auto rows = fetch(o2, (size_t) 3 * Hq * D * 4);
        const size_t rb = (size_t) Hq * D * 4;
        const F::kv_cache * cc[3] = {&cb, &ca, &ca};
        for (int t = 0; t < 3 && ok; ++t) {
            float * qt = q + (size_t) t * Hq * D;
            ok = F::attn_decode(qt, *cc[t], o1, 1, hp[t], Hq, scale, s);
            CK(hipStreamSynchronize(s));
            auto one = fetch(o1, rb);
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
