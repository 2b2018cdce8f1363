// Chunked causal prefill attention over a paged f16 / q8_0 / q4_0 KV cache for gfx950 (MI355X).
//
// One workgroup (4 waves, one per SIMD) owns 128 consecutive query tokens of ONE q head; wave w owns 32 of them as the
// N = 32 columns of v_mfma_f32_32x32x16_f16 tiles. Keys are walked in tiles of 64: all 256 threads fetch the raw tile
// of the head's kv head (16-byte loads, page table looked up per key), dequantize it in registers and store it to LDS
// as f16 [key][dim]; the tile after the current one is fetched and converted while the current one is multiplied
// (two LDS buffers, one barrier per tile).
//   S^T = K Q^T : A = K rows straight from LDS (ds_read_b128), B = Q^T held in registers (pre-multiplied by
//                 scale * log2 e, rounded to f16). A lane then holds 16 keys of ONE query row, so the row maximum
//                 needs no cross-lane work beyond one half-wave swap.
//   O^T = V^T P^T : A = V^T read with the transposing ds_read_b64_tr_b16, B = P^T straight from the S^T registers.
// fp32 accumulation; the softmax denominator is accumulated by an MFMA against an all-ones operand so that it sums the
// same rounded P that multiplies V. Key tiles above the diagonal are skipped, only tiles that straddle a wave's
// diagonal are masked, and the sigmoid output gate is applied in the epilogue.
// Workgroup order: the q heads of one kv head, for one token block, get consecutive dispatch slots on the same XCD,
// so they stream the same K/V tiles through one L2.
#include "p1a_common.hpp"

namespace p1a {
namespace {

constexpr int BM = 128;   // query tokens per workgroup
constexpr int BN = 64;    // keys per tile
constexpr int NTHR = 256;
constexpr float NEG_INF = -__builtin_inff();

template <int D> struct pf_cfg {
    static constexpr int KSTR = D * 2 + 16;    // K tile row stride (odd multiple of 16 B: conflict-free b128 reads)
    static constexpr int VSTR = D * 2 + 32;    // V tile row stride (4 consecutive rows cover disjoint banks for tr16)
    static constexpr int KT_B = BN * KSTR, VT_B = BN * VSTR;
    static constexpr int STAGE_B = KT_B + VT_B;
    static constexpr int NKS = D / 16;         // k-steps of S^T (16 dims each)
    static constexpr int NDT = D / 32;         // 32-dim tiles of O^T
};

#ifdef P1A_TRACE
__device__ long long * g_pf_trace = nullptr;   // development build only: per-workgroup phase cycle totals
#define PT(i) do { const long long t_ = clock64(); acc_t[i] += t_ - last_t; last_t = t_; } while (0)
#else
#define PT(i) do { } while (0)
#endif

struct pf_params {
    const float * q;
    float * out;
    const float * gate;
    const char * kc;
    const char * vc;
    kv_view pg;
    int T, p0, Hq, Hkv, GQA;
    float qscale;
    int nblk;     // token blocks
};

__device__ __forceinline__ uint32_t perm_b(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }

// 4 int8 codes -> 4 halves (code * d), packed
struct pair32 { uint32_t lo, hi; };
__device__ __forceinline__ pair32 deq8x4(uint32_t w, h2 dd) {
    const uint32_t x = w ^ 0x80808080u;
    const h2 off = {(half_t) 1152, (half_t) 1152};
    const h2 a = __builtin_bit_cast(h2, perm_b(0x64646464u, x, 0x04010400u));
    const h2 b = __builtin_bit_cast(h2, perm_b(0x64646464u, x, 0x04030402u));
    return pair32{__builtin_bit_cast(uint32_t, (a - off) * dd), __builtin_bit_cast(uint32_t, (b - off) * dd)};
}
// 4 nibbles (in the low nibbles of the 4 bytes of w) -> 4 halves ((n - 8) * d)
__device__ __forceinline__ pair32 deq4x4(uint32_t w, h2 dd) {
    const h2 off = {(half_t) 1032, (half_t) 1032};
    const h2 a = __builtin_bit_cast(h2, perm_b(0x64646464u, w, 0x04010400u));
    const h2 b = __builtin_bit_cast(h2, perm_b(0x64646464u, w, 0x04030402u));
    return pair32{__builtin_bit_cast(uint32_t, (a - off) * dd), __builtin_bit_cast(uint32_t, (b - off) * dd)};
}

// The output accumulators (O^T and the softmax denominator) live in accumulation registers (AGPRs): MFMA reads and
// writes them there, which leaves the 256 architectural VGPRs to S and the staging data. VALU cannot touch an AGPR, so
// the (rare) rescale of a column goes through a scratch VGPR by hand. Each accumulator tile is pinned to a fixed AGPR
// range while it is rescaled (tile n in a[16n : 16n+15]), which lets the assembly name the registers one by one and
// keeps the register allocator from shuttling all of them through VGPRs on every loop iteration.
#define P1A_RS1(n) "v_accvgpr_read_b32 %1, a" #n "\n\tv_mul_f32 %1, %1, %2\n\tv_accvgpr_write_b32 a" #n ", %1\n\t"
#define P1A_RS16(a, b, c, d, e, f, g, h, i, j, k, l, m, n, o, p) \
    P1A_RS1(a) P1A_RS1(b) P1A_RS1(c) P1A_RS1(d) P1A_RS1(e) P1A_RS1(f) P1A_RS1(g) P1A_RS1(h) \
    P1A_RS1(i) P1A_RS1(j) P1A_RS1(k) P1A_RS1(l) P1A_RS1(m) P1A_RS1(n) P1A_RS1(o) P1A_RS1(p)
#define P1A_ACC_SCALE(vec, range, ...)                                                                        \
    do {                                                                                                      \
        float t_;                                                                                             \
        asm volatile(P1A_RS16(__VA_ARGS__) "s_nop 4" : "+{" range "}"(vec), "=&v"(t_) : "v"(alpha));       \
    } while (0)
// O^T += A B on a pinned accumulator tile. Consecutive calls name different tiles, so no two dependent MFMAs are ever
// closer than eight independent ones; the operands come from LDS reads and conversions the compiler has waited for.
#define P1A_ACC_MFMA(vec, range, a_, b_) \
    asm volatile("v_mfma_f32_32x32x16_f16 " range ", %1, %2, " range : "+{" range "}"(vec) : "v"(a_), "v"(b_))
__device__ __forceinline__ float acc_get(float x) {
#ifndef P1A_PF_PIN
    return x;
#endif
    float t;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t) : "a"(x));
    return t;
}
// MFMA results must have left the matrix pipeline before v_accvgpr_read may name them
__device__ __forceinline__ void acc_settle() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }
constexpr float RESCALE_STEP = 8.0f;   // log2 units: the reference maximum of a row only moves in steps larger than this

// ---- per-type staging: raw tile of one kv head -> registers -> f16 rows in LDS ----
// Every thread owns a fixed set of (key, 16-dim chunk) pairs of the tile; `raw` keeps what was loaded for them.
template <uint32_t KT, int D> struct stager;

template <int D> struct stager<P1A_KV_Q8_0, D> {
    static constexpr int CPK = D / 16;                    // 16-code chunks per key
    static constexpr int NPT = BN * CPK / NTHR;           // chunks per thread
    static_assert(BN * CPK % NTHR == 0, "tile must split evenly over the threads");
    struct raw { u4 w[NPT]; uint16_t d[NPT]; };
    static __device__ __forceinline__ void load(raw & r, const char * base, const size_t * rowoff, int tid) {
#pragma unroll
        for (int x = 0; x < NPT; ++x) {
            const int i = x * NTHR + tid, key = i / CPK, cc = i - key * CPK;
            const char * row = base + rowoff[x];
            (void) key;
            r.w[x] = *reinterpret_cast<const u4 *>(row + (D / 32) * 2 + cc * 16);
            r.d[x] = *reinterpret_cast<const uint16_t *>(row + (cc >> 1) * 2);
        }
    }
    static __device__ __forceinline__ void store(const raw & r, char * tile, int stride, int tid) {
#pragma unroll
        for (int x = 0; x < NPT; ++x) {
            const int i = x * NTHR + tid, key = i / CPK, cc = i - key * CPK;
            const uint32_t d16 = r.d[x];
            const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
            const pair32 x0 = deq8x4(r.w[x][0], dd), x1 = deq8x4(r.w[x][1], dd);
            const pair32 x2 = deq8x4(r.w[x][2], dd), x3 = deq8x4(r.w[x][3], dd);
            const u4 a = {x0.lo, x0.hi, x1.lo, x1.hi}, b = {x2.lo, x2.hi, x3.lo, x3.hi};
            u4 * dst = reinterpret_cast<u4 *>(tile + key * stride + cc * 32);
            dst[0] = a;
            dst[1] = b;
        }
    }
};

template <int D> struct stager<P1A_KV_F16, D> {
    static constexpr int CPK = D / 8;                     // 16-byte chunks (8 halves) per key
    static constexpr int NPT = BN * CPK / NTHR;
    static_assert(BN * CPK % NTHR == 0, "tile must split evenly over the threads");
    struct raw { u4 w[NPT]; };
    static __device__ __forceinline__ void load(raw & r, const char * base, const size_t * rowoff, int tid) {
#pragma unroll
        for (int x = 0; x < NPT; ++x) {
            const int i = x * NTHR + tid, key = i / CPK, cc = i - key * CPK;
            (void) key;
            r.w[x] = *reinterpret_cast<const u4 *>(base + rowoff[x] + cc * 16);
        }
    }
    static __device__ __forceinline__ void store(const raw & r, char * tile, int stride, int tid) {
#pragma unroll
        for (int x = 0; x < NPT; ++x) {
            const int i = x * NTHR + tid, key = i / CPK, cc = i - key * CPK;
            *reinterpret_cast<u4 *>(tile + key * stride + cc * 16) = r.w[x];
        }
    }
};

template <int D> struct stager<P1A_KV_Q4_0, D> {
    static constexpr int CPK = D / 32;                    // 18-byte blocks per key: one block (32 values) per item
    static constexpr int NPT = (BN * CPK + NTHR - 1) / NTHR;
    struct raw { uint16_t h[NPT][9]; };
    static __device__ __forceinline__ void load(raw & r, const char * base, const size_t * rowoff, int tid) {
#pragma unroll
        for (int x = 0; x < NPT; ++x) {
            const int i = x * NTHR + tid, key = i / CPK, b = i - key * CPK;
            if (BN * CPK % NTHR == 0 || key < BN) {
                const uint16_t * blk = reinterpret_cast<const uint16_t *>(base + rowoff[x] + b * 18);   // 2-byte aligned
#pragma unroll
                for (int k = 0; k < 9; ++k) r.h[x][k] = blk[k];
            }
        }
    }
    static __device__ __forceinline__ void store(const raw & r, char * tile, int stride, int tid) {
#pragma unroll
        for (int x = 0; x < NPT; ++x) {
            const int i = x * NTHR + tid, key = i / CPK, b = i - key * CPK;
            if (!(BN * CPK % NTHR == 0 || key < BN)) continue;
            const uint32_t d16 = r.h[x][0];
            const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
            // byte j of the block: low nibble = value j, high nibble = value j + 16
            pair32 lo[4], hi[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t w = (uint32_t) r.h[x][1 + 2 * k] | ((uint32_t) r.h[x][2 + 2 * k] << 16);   // bytes 4k..4k+3
                lo[k] = deq4x4(w & 0x0f0f0f0fu, dd);
                hi[k] = deq4x4((w >> 4) & 0x0f0f0f0fu, dd);
            }
            u4 * dst = reinterpret_cast<u4 *>(tile + key * stride + b * 64);
            dst[0] = u4{lo[0].lo, lo[0].hi, lo[1].lo, lo[1].hi};
            dst[1] = u4{lo[2].lo, lo[2].hi, lo[3].lo, lo[3].hi};
            dst[2] = u4{hi[0].lo, hi[0].hi, hi[1].lo, hi[1].hi};
            dst[3] = u4{hi[2].lo, hi[2].hi, hi[3].lo, hi[3].hi};
        }
    }
};

template <uint32_t KT, int D>
__global__ void __launch_bounds__(NTHR, 1) prefill_k(const pf_params P) {
    using C = pf_cfg<D>;
    using S = stager<KT, D>;
    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 31, g = lane >> 5;
    // blockIdx.x -> (token block, kv head, q head of the group): the GQA heads of one (block, kv head) share an XCD
    const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
    const int unit = (slot / P.GQA) * 8 + xcd, hh = slot % P.GQA;
    if (unit >= P.nblk * P.Hkv) return;
    // longest blocks (most keys) first
    const int tb = P.nblk - 1 - unit / P.Hkv, hk = unit % P.Hkv;
    const int h = hk * P.GQA + hh;

    const int tok0 = tb * BM;                                 // first token of the block
    const int wtok0 = tok0 + 32 * wave;                       // first token of this wave
    const int my_tok = wtok0 + c;                             // this lane's query row
    const bool live = my_tok < P.T;
    const int my_pos = P.p0 + (live ? my_tok : P.T - 1);
    const int pmax = P.p0 + min(P.T, tok0 + BM) - 1;          // last position any row of the block sees
    const int wave_pmin = P.p0 + wtok0;                       // smallest limit among this wave's rows
    const int wave_pmax = P.p0 + min(P.T - 1, wtok0 + 31);
    const bool wave_live = wtok0 < P.T;
    const int ntiles = pmax / BN + 1;

    const int32_t * ptab = P.pg.pt ? (P.pg.rtab ? P.pg.pt + P.pg.rtab[0] : P.pg.pt) : nullptr;
    const size_t hb = KT == P1A_KV_F16 ? (size_t) D * 2 : KT == P1A_KV_Q8_0 ? (size_t) (D / 32) * 34 : (size_t) (D / 32) * 18;
    const size_t head_off = (size_t) hk * hb;

    // ---- Q^T operands (B: k = 16 dims per step, n = query row): lane (row c, half g) holds dims 16 ks + 8 g .. + 7 ----
    h8 qf[C::NKS];
    {
        const float * qr = P.q + ((size_t) (live ? my_tok : 0) * P.Hq + h) * D;
#pragma unroll
        for (int ks = 0; ks < C::NKS; ++ks) {
            float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
            if (live) { a = *reinterpret_cast<const float4 *>(qr + 16 * ks + 8 * g); b = *reinterpret_cast<const float4 *>(qr + 16 * ks + 8 * g + 4); }
            const float s = P.qscale;
            qf[ks] = h8{(half_t) (a.x * s), (half_t) (a.y * s), (half_t) (a.z * s), (half_t) (a.w * s),
                        (half_t) (b.x * s), (half_t) (b.y * s), (half_t) (b.z * s), (half_t) (b.w * s)};
        }
    }

    f16x o[C::NDT];
    f16x ol;
    float m_run = NEG_INF;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        ol[i] = 0.f;
#pragma unroll
        for (int dt = 0; dt < C::NDT; ++dt) o[dt][i] = 0.f;
    }
    const h8 ones = {(half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1};

#ifdef P1A_TRACE
    long long acc_t[12] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    long long last_t = clock64();
#endif
    // Row offsets of a tile. A tile is four groups of 16 keys; with pages of >= 16 positions (or a contiguous cache) a
    // group lies in one page, so its base is wave-uniform: the page-table entries are fetched once per tile, one tile
    // ahead of their use, instead of once per thread and key in front of every load. Keys past pmax are clamped onto it.
    const bool grouped = !ptab || P.pg.psh >= 4;
    // The table entries are fetched with hand-issued scalar loads (s_load_dword): they do not share the in-order
    // vector-memory counter with the tile loads in flight, and they are issued where written - one iteration before
    // rowoffs() waits for them - instead of wherever the scheduler would sink an ordinary load to.
    const int pmask = (1 << P.pg.psh) - 1;
    struct gpages { int pg[BN / 16]; };
    auto group_pages = [&](int k0) {
        gpages r;
#pragma unroll
        for (int gq = 0; gq < BN / 16; ++gq) r.pg[gq] = 0;
        if (ptab && grouped) {
#pragma unroll
            for (int gq = 0; gq < BN / 16; ++gq) {
                const int32_t * e = ptab + (__builtin_amdgcn_readfirstlane(min(k0 + 16 * gq, pmax)) >> P.pg.psh);
                asm volatile("s_load_dword %0, %1, 0x0" : "=s"(r.pg[gq]) : "s"(e));
            }
        }
        return r;
    };
    auto rowoffs = [&](int k0, gpages & gp, size_t * ro) {
        size_t go[BN / 16];
        static_assert(BN / 16 == 4, "the wait below names four entries");
        asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(gp.pg[0]), "+s"(gp.pg[1]), "+s"(gp.pg[2]), "+s"(gp.pg[3]));
        PT(9);
        if (grouped) {
#pragma unroll
            for (int gq = 0; gq < BN / 16; ++gq) {
                const int p = __builtin_amdgcn_readfirstlane(min(k0 + 16 * gq, pmax));
                go[gq] = (ptab ? (size_t) gp.pg[gq] * P.pg.pstride + (size_t) (p & pmask) * P.pg.rowb : (size_t) p * P.pg.rowb) + head_off;
            }
        }
        PT(10);
#pragma unroll
        for (int x = 0; x < S::NPT; ++x) {
            const int i = x * NTHR + tid, key = min(i / S::CPK, BN - 1);
            if (grouped) {
                const int gq = key >> 4, room = pmax - (k0 + 16 * gq);      // keys of the group before pmax (< 0: none)
                size_t base = go[0];
#pragma unroll
                for (int j = 1; j < BN / 16; ++j) base = gq == j ? go[j] : base;
                ro[x] = base + (size_t) (min(key & 15, max(room, 0)) * (int) P.pg.rowb);
            } else {
                ro[x] = kv_off_tab(P.pg, ptab, min(k0 + key, pmax)) + head_off;
            }
        }
    };

    // Workgroups that share a kv head would otherwise walk the keys in lock-step and ask one L2 channel for the same
    // line at the same instant. Each starts at its own tile and wraps around (softmax does not care about key order);
    // the q heads of one group stay one tile apart, so all but the first still find the tile in L2.
    const int rot = (int) (((unsigned) unit * 29u + (unsigned) hh) % (unsigned) ntiles);
    auto tile_of = [&](int it) { const int t = it + rot; return t >= ntiles ? t - ntiles : t; };
    typename S::raw rk, rv;
    {
        size_t ro[S::NPT];
        gpages g0 = group_pages(tile_of(0) * BN);
        rowoffs(tile_of(0) * BN, g0, ro);
        S::load(rk, P.kc, ro, tid);
        S::load(rv, P.vc, ro, tid);
    }
    gpages go_next = group_pages(tile_of(ntiles > 1 ? 1 : 0) * BN);   // pages of the second tile, consumed in iteration 0
    S::store(rk, lds, C::KSTR, tid);
    S::store(rv, lds + C::KT_B, C::VSTR, tid);
    __syncthreads();

    for (int it = 0; it < ntiles; ++it) {
        const int k0 = tile_of(it) * BN;
        char * kt = lds + (it & 1) * C::STAGE_B;
        char * vt = kt + C::KT_B;
        char * nkt = lds + ((it + 1) & 1) * C::STAGE_B;
        const bool more = it + 1 < ntiles;
        PT(8);
        if (more) {   // raw loads of the next tile fly while this one is multiplied
            size_t ro[S::NPT];
            rowoffs(tile_of(it + 1) * BN, go_next, ro);
            PT(6);
            S::load(rk, P.kc, ro, tid);
            PT(7);
            S::load(rv, P.vc, ro, tid);
            if (it + 2 < ntiles) go_next = group_pages(tile_of(it + 2) * BN);   // page entries needed one iteration on
        }
        PT(0);
        const bool active = wave_live && k0 <= wave_pmax;     // tiles above this wave's diagonal contribute nothing
        h8 pb[BN / 16];
        if (active) {
            // ---- S^T = K Q^T: two 32-key sub-tiles ----
            f16x s[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
#pragma unroll
                for (int i = 0; i < 16; ++i) s[u][i] = 0.f;
                const char * krow = kt + (32 * u + c) * C::KSTR + g * 16;
#pragma unroll
                for (int ks = 0; ks < C::NKS; ++ks) {
                    const h8 a = *reinterpret_cast<const h8 *>(krow + ks * 32);
                    s[u] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[ks], s[u], 0, 0, 0);
                }
            }
            PT(1);
            // ---- online softmax: this lane holds keys k0 + 32 u + 8 (i / 4) + 4 g + (i % 4) of its own row ----
            float mloc = NEG_INF;
            if (k0 + BN - 1 > wave_pmin) {                     // the tile straddles the diagonal of some row: mask
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int kp = k0 + 32 * u + 8 * (i >> 2) + 4 * g + (i & 3);
                        s[u][i] = kp <= my_pos ? s[u][i] : NEG_INF;
                    }
            }
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 16; ++i) mloc = fmaxf(mloc, s[u][i]);
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
            // Lazy reference maximum: m_run follows the row maximum only when it has grown by more than RESCALE_STEP, so
            // P stays below 2^RESCALE_STEP (exact in f16 range) and the accumulators are rescaled a handful of times per
            // row instead of at every tile. A row that has seen no visible key yet (m_run = -inf) just adopts the maximum.
            const bool fresh = m_run == NEG_INF;
            const bool move = mloc > m_run + RESCALE_STEP || fresh;      // mloc = -inf never moves anything
            const float mnew = (move && mloc != NEG_INF) ? mloc : m_run;
            const bool dead = mnew == NEG_INF;
            const float alpha = (fresh || mnew == m_run) ? 1.0f : __builtin_amdgcn_exp2f(m_run - mnew);
            m_run = mnew;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int i = 0; i < 16; ++i) s[u][i] = dead ? 0.0f : __builtin_amdgcn_exp2f(s[u][i] - mnew);
#pragma unroll
            for (int ps = 0; ps < BN / 16; ++ps) {
                const int u = ps >> 1, b = 8 * (ps & 1);
                pb[ps] = h8{(half_t) s[u][b], (half_t) s[u][b + 1], (half_t) s[u][b + 2], (half_t) s[u][b + 3],
                            (half_t) s[u][b + 4], (half_t) s[u][b + 5], (half_t) s[u][b + 6], (half_t) s[u][b + 7]};
            }
            if (__builtin_expect(__any(alpha != 1.0f), 0)) {
#ifndef P1A_PF_PIN
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    ol[i] *= alpha;
#pragma unroll
                    for (int dt = 0; dt < C::NDT; ++dt) o[dt][i] *= alpha;
                }
#else
                acc_settle();
                P1A_ACC_SCALE(o[0], "a[0:15]", 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
                P1A_ACC_SCALE(o[1], "a[16:31]", 16, 17, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28, 29, 30, 31);
                if constexpr (C::NDT > 2) {
                    P1A_ACC_SCALE(o[2], "a[32:47]", 32, 33, 34, 35, 36, 37, 38, 39, 40, 41, 42, 43, 44, 45, 46, 47);
                    P1A_ACC_SCALE(o[3], "a[48:63]", 48, 49, 50, 51, 52, 53, 54, 55, 56, 57, 58, 59, 60, 61, 62, 63);
                }
                if constexpr (C::NDT > 4) {
                    P1A_ACC_SCALE(o[4], "a[64:79]", 64, 65, 66, 67, 68, 69, 70, 71, 72, 73, 74, 75, 76, 77, 78, 79);
                    P1A_ACC_SCALE(o[5], "a[80:95]", 80, 81, 82, 83, 84, 85, 86, 87, 88, 89, 90, 91, 92, 93, 94, 95);
                    P1A_ACC_SCALE(o[6], "a[96:111]", 96, 97, 98, 99, 100, 101, 102, 103, 104, 105, 106, 107, 108, 109, 110, 111);
                    P1A_ACC_SCALE(o[7], "a[112:127]", 112, 113, 114, 115, 116, 117, 118, 119, 120, 121, 122, 123, 124, 125, 126, 127);
                }
                P1A_ACC_SCALE(ol, "a[128:143]", 128, 129, 130, 131, 132, 133, 134, 135, 136, 137, 138, 139, 140, 141, 142, 143);
#endif
            }
        }
        PT(2);
        if (more) {   // convert the next tile into the other buffer
            S::store(rk, nkt, C::KSTR, tid);
            S::store(rv, nkt + C::KT_B, C::VSTR, tid);
        }
        PT(3);
        if (active) {
            // ---- O^T += V^T P^T. Slot e of lane half g in k-step ps is key 16 ps + 4 g + e (e < 4) or 16 ps + 8 + 4 g + e - 4 ----
            const int i16 = lane & 15, blk = lane >> 4;        // 16-lane block: dims 16 (blk & 1) .., lane half blk >> 1 == g
            const int kk = i16 >> 2, jq = i16 & 3;
            const char * vbase = vt + (4 * g + kk) * C::VSTR + (16 * (blk & 1) + 4 * jq) * 2;
#pragma unroll
            for (int ps = 0; ps < BN / 16; ++ps) {
#pragma unroll
                for (int dt = 0; dt < C::NDT; ++dt) {
                    const char * p0_ = vbase + (16 * ps) * C::VSTR + dt * 64;
                    const s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *) p0_);
                    const s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *) (p0_ + 8 * C::VSTR));
                    const h4 l4 = __builtin_bit_cast(h4, lo), h4_ = __builtin_bit_cast(h4, hi);
                    const h8 a = {l4[0], l4[1], l4[2], l4[3], h4_[0], h4_[1], h4_[2], h4_[3]};
#ifndef P1A_PF_PIN
                    o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb[ps], o[dt], 0, 0, 0);
                }
                ol = __builtin_amdgcn_mfma_f32_32x32x16_f16(ones, pb[ps], ol, 0, 0, 0);
            }
#else
                    if (dt == 0) P1A_ACC_MFMA(o[0], "a[0:15]", a, pb[ps]);
                    if (dt == 1) P1A_ACC_MFMA(o[1], "a[16:31]", a, pb[ps]);
                    if constexpr (C::NDT > 2) {
                        if (dt == 2) P1A_ACC_MFMA(o[2], "a[32:47]", a, pb[ps]);
                        if (dt == 3) P1A_ACC_MFMA(o[3], "a[48:63]", a, pb[ps]);
                    }
                    if constexpr (C::NDT > 4) {
                        if (dt == 4) P1A_ACC_MFMA(o[4], "a[64:79]", a, pb[ps]);
                        if (dt == 5) P1A_ACC_MFMA(o[5], "a[80:95]", a, pb[ps]);
                        if (dt == 6) P1A_ACC_MFMA(o[6], "a[96:111]", a, pb[ps]);
                        if (dt == 7) P1A_ACC_MFMA(o[7], "a[112:127]", a, pb[ps]);
                    }
                }
                P1A_ACC_MFMA(ol, "a[128:143]", ones, pb[ps]);
            }
#endif
            acc_settle();   // the compiler does not know these are MFMAs: let them retire before it may copy a tile
        }
        PT(4);
        __syncthreads();
        PT(5);
    }
#ifdef P1A_TRACE
    if (g_pf_trace && tid == 0) for (int i = 0; i < 12; ++i) g_pf_trace[(size_t) blockIdx.x * 12 + i] = acc_t[i];
#endif

    // ---- epilogue: normalise, gate, store. Lane (row c, half g) holds dims 32 dt + 8 (i / 4) + 4 g + (i % 4) ----
    if (live) {
        acc_settle();
        const float inv = 1.0f / acc_get(ol[0]);
        float * orow = P.out + ((size_t) my_tok * P.Hq + h) * D;
        const float * grow = P.gate ? P.gate + ((size_t) my_tok * P.Hq + h) * D : nullptr;
#pragma unroll
        for (int dt = 0; dt < C::NDT; ++dt)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int d0 = 32 * dt + 8 * q4 + 4 * g;
                f4 r = {acc_get(o[dt][4 * q4]) * inv, acc_get(o[dt][4 * q4 + 1]) * inv, acc_get(o[dt][4 * q4 + 2]) * inv,
                        acc_get(o[dt][4 * q4 + 3]) * inv};
                if (grow) {
                    const f4 gt = *reinterpret_cast<const f4 *>(grow + d0);
#pragma unroll
                    for (int x = 0; x < 4; ++x) r[x] *= 1.0f / (1.0f + expf(-gt[x]));
                }
                *reinterpret_cast<f4 *>(orow + d0) = r;
            }
    }
}

template <uint32_t KT, int D>
int launch_pf(const pf_params & P, hipStream_t s) {
    using C = pf_cfg<D>;
    const int lds = 2 * C::STAGE_B;
    static bool attr_set = false;
    if (!attr_set) {
        if (hipFuncSetAttribute((const void *) prefill_k<KT, D>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
            (void) hipGetLastError();
            set_error("p1a_attn_prefill: cannot reserve %d bytes of LDS", lds);
            return P1A_E_LAUNCH;
        }
        attr_set = true;
    }
    const int units = P.nblk * P.Hkv;
    const int slots = ((units + 7) / 8) * P.GQA;
    prefill_k<KT, D><<<slots * 8, NTHR, lds, s>>>(P);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

}   // namespace

int launch_prefill(const p1a_kv & c, const float * q, float * out, const float * gate, int T, int p0, int Hq,
                   float scale, void * scratch, size_t scratch_bytes, hipStream_t s) {
    (void) scratch; (void) scratch_bytes;
    if (c.D != 64 && c.D != 128 && c.D != 256) { set_error("p1a_attn_prefill: unsupported head size D=%d", c.D); return P1A_E_SHAPE; }
    if ((((uintptr_t) c.k | (uintptr_t) c.v) & 15) || (c.pt && (c.pstride & 15))) { set_error("p1a_attn_prefill: cache base / page stride must be 16-byte aligned"); return P1A_E_SHAPE; }
    pf_params P;
    P.q = q; P.out = out; P.gate = gate; P.kc = (const char *) c.k; P.vc = (const char *) c.v; P.pg = view_of(c);
    P.T = T; P.p0 = p0; P.Hq = Hq; P.Hkv = c.Hkv; P.GQA = Hq / c.Hkv;
    P.qscale = scale * 1.4426950408889634f;
    P.nblk = (T + BM - 1) / BM;
#define PF(KT_) (c.D == 256 ? launch_pf<KT_, 256>(P, s) : c.D == 128 ? launch_pf<KT_, 128>(P, s) : launch_pf<KT_, 64>(P, s))
    if (c.type == P1A_KV_F16) return PF(P1A_KV_F16);
    if (c.type == P1A_KV_Q8_0) return PF(P1A_KV_Q8_0);
    return PF(P1A_KV_Q4_0);
#undef PF
}

}   // namespace p1a

#ifdef P1A_TRACE
extern "C" void p1a_set_pf_trace(long long * buf) { (void) hipMemcpyToSymbol(HIP_SYMBOL(p1a::g_pf_trace), &buf, sizeof buf); }
#endif

extern "C" size_t p1a_attn_prefill_scratch_bytes(int T, int p0, int Hq, int Hkv, int D) {
    (void) T; (void) p0; (void) Hq; (void) Hkv; (void) D;
    return 0;   // the kernel keeps every intermediate in registers and LDS
}
