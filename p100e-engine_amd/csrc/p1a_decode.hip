// Split-K paged-KV decode / MTP-verify attention for gfx950 (MI355X).
//
// Work decomposition
//   grid = (nsplit, Hkv / HPW, row groups), block = 4 waves. A row group is up to 4 query rows of ONE sequence (the
//   tokens of a verify block); its GQA * rows query rows are the columns of 16-wide MFMA tiles, so the group's KV is
//   read once. Wave w owns kv head (w % HPW) and key sub-tile (w / HPW): it walks 32-key tiles of that head, the
//   tiles of split stream s being the units s, s + nsplit, ... of 32 * (4 / HPW) positions. The partition depends
//   only on the device and Hkv, never on T, the depth or the batch, so every row is computed by the same sequence of
//   operations whichever call it is part of (T-invariance, rows == single, paged == contiguous).
//   A wave's tile (32 keys x one head, K and V) is fetched with 16-byte loads in memory order (17 consecutive lanes
//   cover one q8_0 head row), parked in a wave-private LDS tile and read back in MFMA operand order; no workgroup
//   barrier is needed inside the key loop.
// Arithmetic
//   S^T = K Q^T and O^T = V^T P^T on v_mfma_f32_16x16x32_f16: q8_0 codes are expanded to f16 in registers with a
//   byte-permute (0x6400 | code ^ 0x80 = 1152 + code) and multiplied by the f16 block scale; V is read from LDS with
//   the transposing ds_read_b64_tr_b8 / _tr_b16 so that a lane holds 8 keys of one output dim. Q is pre-multiplied by
//   scale * log2(e) and rounded to f16, P = 2^(S - m) is rounded to f16, all accumulation is fp32. The softmax
//   denominator is one more MFMA against an all-ones operand, so it sums exactly the P that multiplies V.
//   Partials (m, l, O) go to scratch and merge_k folds them in split order and applies the sigmoid gate.
#include "p1a_common.hpp"

#include <cstdlib>

namespace p1a {
namespace {

constexpr float NEG_INF = -__builtin_inff();

template <uint32_t KT, int D> struct tile_cfg {
    static constexpr int HB = (int) head_bytes(KT, D);
    static constexpr int CPK = HB / 16;                        // 16-byte chunks per (key, head)
    static constexpr int KSTR = (CPK & 1) ? HB : HB + 16;      // LDS row stride: an odd number of 16-byte units
    static constexpr int NCH = 32 * CPK;                       // chunks per 32-key tile
    static constexpr int NRND = (NCH + 63) / 64;               // load rounds per tile
    static constexpr int TILE_B = 32 * KSTR;
    static constexpr int TAB_B = KT == P1A_KV_F16 ? 0 : (D / 32) * 64;   // transposed V scale table
    static constexpr int WAVE_B = 2 * TILE_B + TAB_B;
    static constexpr int NMF = D / 32;                         // QK MFMAs per 16-key sub-tile
    static constexpr int NDT = D / 16;                         // output dim tiles
    static_assert(HB % 16 == 0, "head row must be a whole number of 16-byte chunks");
};

#ifdef P1A_TRACE
// development build only: per-wave phase timestamps (shader clock) in a caller-visible buffer
__device__ long long * g_trace = nullptr;
#define TS(i) do { if (g_trace && lane == 0) g_trace[((size_t) blockIdx.x * NWV + wave) * 16 + (i)] = clock64(); } while (0)
#else
#define TS(i) do { } while (0)
#endif

struct dec_params {
    const float * q;
    const char * kc;
    const char * vc;
    float * part_o;
    float * part_ml;
    kv_view pg;
    int p0;
    const int32_t * p0_dev;
    const int32_t * pos_rows;
    int T, RG, Hq, Hkv, GQA, HPW;
    float qscale;     // softmax scale * log2(e)
    int nsplit;       // split streams (grid.x)
};

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }

// 4 int8 codes (one dword) -> 4 halves holding 1152 + code, as two packed pairs
__device__ __forceinline__ void codes4_to_h(uint32_t w, h2 & a, h2 & b) {
    const uint32_t x = w ^ 0x80808080u;
    a = __builtin_bit_cast(h2, perm(0x64646464u, x, 0x04010400u));
    b = __builtin_bit_cast(h2, perm(0x64646464u, x, 0x04030402u));
}

// 16-byte global load that the compiler cannot turn into something narrower
__device__ __forceinline__ i4 ldg16(const char * p) { return *reinterpret_cast<const i4 *>(p); }

__device__ __forceinline__ int rfl(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ size_t rfl64(size_t x) {
    const uint32_t lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) x);
    const uint32_t hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (x >> 32));
    return ((size_t) hi << 32) | lo;
}

// 4 int8 codes -> (code * d) as two packed f16 pairs, returned as raw dwords so that MFMA operands are built in place
struct u2 { uint32_t lo, hi; };
__device__ __forceinline__ u2 deq4(uint32_t w, h2 d01, h2 d23) {
    const h2 off = {(half_t) 1152, (half_t) 1152};
    h2 a, b;
    codes4_to_h(w, a, b);
    return u2{__builtin_bit_cast(uint32_t, (a - off) * d01), __builtin_bit_cast(uint32_t, (b - off) * d23)};
}

template <uint32_t KT, int D, int NT, int NWV>
__global__ void __launch_bounds__(NWV * 64, NWV == 4 ? 2 : 1) dec_mfma_k(const dec_params P) {
    using C = tile_cfg<KT, D>;
    __shared__ __attribute__((aligned(16))) char lds[NWV * C::WAVE_B];

    const int lane = threadIdx.x & 63, wave = rfl(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    // blockIdx.x -> (split stream, head group). Workgroups are dealt to the 8 XCDs round-robin by linear index, so
    // the head groups of one split stream (which share cache lines when HPW < Hkv) are given the same index mod 8.
    const int HG = P.Hkv / P.HPW;
    int split, hg;
    if ((P.nsplit & 7) == 0) {
        const int i = blockIdx.x, j = i >> 3;
        hg = j % HG;
        split = (j / HG) * 8 + (i & 7);
    } else {
        split = blockIdx.x / HG;
        hg = blockIdx.x - split * HG;
    }
    const int hslot = wave % P.HPW;
    const int hk = hg * P.HPW + hslot;
    const int sub = wave / P.HPW, WPH = NWV / P.HPW;
    const int U = 32 * WPH;                                   // positions per unit
    const int row0 = blockIdx.y * P.RG;
    const int nr = min(P.RG, P.T - row0);                     // rows of this group
    const int R = nr * P.GQA;                                 // live MFMA columns
    const int p0v = P.pos_rows ? 0 : (P.p0_dev ? *P.p0_dev : P.p0);

    TS(0);
    char * kt = lds + wave * C::WAVE_B;
    char * vt = kt + C::TILE_B;
    char * tab = vt + C::TILE_B;

    // visible-position limit of each of this lane's columns, and the group's maximum
    int plim[NT];
    int n_max = 0;
    for (int t = 0; t < nr; ++t) {
        const int pt_ = P.pos_rows ? P.pos_rows[row0 + t] : p0v + row0 + t;
        n_max = max(n_max, pt_ + 1);
    }
    n_max = rfl(n_max);
#pragma unroll
    for (int r = 0; r < NT; ++r) {
        const int col = 16 * r + c;
        plim[r] = -1;
        if (col < R) {
            const int t = col / P.GQA;
            plim[r] = P.pos_rows ? P.pos_rows[row0 + t] : p0v + row0 + t;
        }
    }
    const int32_t * ptab = kv_tab(P.pg, P.pos_rows ? row0 : 0);
    const size_t head_off = (size_t) hk * C::HB;
    const int rowb = (int) P.pg.rowb;
    // a 32-key tile lies in one page (or in a contiguous cache): one base per tile, static per-lane offsets
    const bool onepage = !ptab || P.pg.psh >= 5;

    int lofs[C::NRND], soff[C::NRND];
#pragma unroll
    for (int rd = 0; rd < C::NRND; ++rd) {
        const int i = rd * 64 + lane;
        const int key = i / C::CPK, cir = i - key * C::CPK;
        lofs[rd] = key * C::KSTR + cir * 16;
        soff[rd] = key * rowb + (int) head_off + cir * 16;
    }

    // 16 bytes per lane in memory order; keys past `last` (beyond every row's visible range) are clamped onto it, so
    // nothing outside the sequence is ever read
    auto issue = [&](i4 * regs, const char * base, int ts, int last) {
        const size_t off0 = rfl64(kv_off_tab(P.pg, ptab, ts));
        if (onepage && last >= 31) {
            const char * b0 = base + off0;
#pragma unroll
            for (int rd = 0; rd < C::NRND; ++rd)
                if (C::NCH % 64 == 0 || rd * 64 + lane < C::NCH) regs[rd] = ldg16(b0 + soff[rd]);
        } else {
            const size_t off1 = last >= 16 ? rfl64(kv_off_tab(P.pg, ptab, ts + 16)) : off0;
#pragma unroll
            for (int rd = 0; rd < C::NRND; ++rd) {
                const int i = rd * 64 + lane;
                const int key = i / C::CPK, cir = i - key * C::CPK;
                const int kcl = min(key, last);
                const size_t go = ((kcl & 16) ? off1 : off0) + (size_t) ((kcl & 15) * rowb) + head_off + (size_t) (cir * 16);
                if (C::NCH % 64 == 0 || i < C::NCH) regs[rd] = ldg16(base + go);
            }
        }
    };
    // the same loads written straight into an LDS tile (global_load_lds_dwordx4: lane i of a round lands at
    // tile + round * 1024 + 16 i), usable when the tile is the linear image of the head rows (KSTR == HB)
    auto issue_lds = [&](char * tile, const char * base, int ts, int last) {
        const size_t off0 = rfl64(kv_off_tab(P.pg, ptab, ts));
        if (onepage && last >= 31) {
            const char * b0 = base + off0;
#pragma unroll
            for (int rd = 0; rd < C::NRND; ++rd)
                if (C::NCH % 64 == 0 || rd * 64 + lane < C::NCH)
                    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *) (b0 + soff[rd]),
                                                     (void __attribute__((address_space(3))) *) (tile + rd * 1024), 16, 0, 0);
        } else {
            const size_t off1 = last >= 16 ? rfl64(kv_off_tab(P.pg, ptab, ts + 16)) : off0;
#pragma unroll
            for (int rd = 0; rd < C::NRND; ++rd) {
                const int i = rd * 64 + lane;
                const int key = i / C::CPK, cir = i - key * C::CPK;
                const int kcl = min(key, last);
                const char * src = base + ((kcl & 16) ? off1 : off0) + (size_t) ((kcl & 15) * rowb) + head_off + (size_t) (cir * 16);
                if (C::NCH % 64 == 0 || i < C::NCH)
                    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *) src,
                                                     (void __attribute__((address_space(3))) *) (tile + rd * 1024), 16, 0, 0);
            }
        }
    };
    auto park = [&](char * tile, const i4 * regs) {
#pragma unroll
        for (int rd = 0; rd < C::NRND; ++rd)
            if (C::NCH % 64 == 0 || rd * 64 + lane < C::NCH) *reinterpret_cast<i4 *>(tile + lofs[rd]) = regs[rd];
    };

    f4 o[NT][C::NDT];
    f4 ol[NT];
    float m_run[NT];
#pragma unroll
    for (int r = 0; r < NT; ++r) {
        m_run[r] = NEG_INF;
        ol[r] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < C::NDT; ++j) o[r][j] = f4{0.f, 0.f, 0.f, 0.f};
    }
    const h8 ones = {(half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1};

    // software pipeline: the loads of tile n + 1 are issued into the registers tile n has just vacated
    constexpr bool KDMA = C::KSTR == C::HB;   // K tiles go global -> LDS directly, V tiles through registers
    i4 kr[KDMA ? 1 : C::NRND], vr[C::NRND];
    int u = split;
    bool have = u * U + sub * 32 < n_max;
    TS(15);
    if (have) {
        const int ts = u * U + sub * 32;
#ifdef P1A_TRACE
        { const size_t o_ = rfl64(kv_off_tab(P.pg, ptab, ts)); if (o_ == 1) return; TS(9); }
#endif
        if constexpr (KDMA) issue_lds(kt, P.kc, ts, n_max - 1 - ts);
        else issue(kr, P.kc, ts, n_max - 1 - ts);
        TS(10);
        issue(vr, P.vc, ts, n_max - 1 - ts);
    }
    TS(14);
    // Q^T operands: column = query row (token t, head hh of the group), 8 consecutive dims per MFMA slot group
    h8 qf[NT][C::NMF];
#pragma unroll
    for (int r = 0; r < NT; ++r) {
        const int col = 16 * r + c;
        const bool livec = col < R;
        const int t = livec ? col / P.GQA : 0, hh = livec ? col - t * P.GQA : 0;
        const float * qr = P.q + ((size_t) (row0 + t) * P.Hq + (size_t) hk * P.GQA + hh) * D;
#pragma unroll
        for (int m = 0; m < C::NMF; ++m) {
            const int d0 = KT == P1A_KV_F16 ? 32 * m + 8 * g : 16 * (4 * (m >> 1) + g) + 8 * (m & 1);
            float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
            if (livec) { a = *reinterpret_cast<const float4 *>(qr + d0); b = *reinterpret_cast<const float4 *>(qr + d0 + 4); }
            const float s = P.qscale;
            qf[r][m] = h8{(half_t) (a.x * s), (half_t) (a.y * s), (half_t) (a.z * s), (half_t) (a.w * s),
                          (half_t) (b.x * s), (half_t) (b.y * s), (half_t) (b.z * s), (half_t) (b.w * s)};
        }
    }

    TS(1);
    int it_ = 0;
    while (have) {
        const int ts = u * U + sub * 32;                      // first position of this wave's tile
        const int un = u + P.nsplit;
        const int tsn = un * U + sub * 32;
        const bool have_n = tsn < n_max;

        if constexpr (!KDMA) {
            park(kt, kr);
            if (have_n) issue(kr, P.kc, tsn, n_max - 1 - tsn);
        }

        // ---- S^T = K Q^T for the two 16-key sub-tiles ----
        if (it_ < 1) TS(2 + 5 * it_);
        f4 s[NT][2];
#pragma unroll
        for (int st = 0; st < 2; ++st) {
#pragma unroll
            for (int r = 0; r < NT; ++r) s[r][st] = f4{0.f, 0.f, 0.f, 0.f};
            const char * krow = kt + (16 * st + c) * C::KSTR;
            if constexpr (KT == P1A_KV_F16) {
#pragma unroll
                for (int m = 0; m < C::NMF; ++m) {
                    const h8 a = *reinterpret_cast<const h8 *>(krow + (4 * m + g) * 16);
#pragma unroll
                    for (int r = 0; r < NT; ++r) s[r][st] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qf[r][m], s[r][st], 0, 0, 0);
                }
            } else {   // q8_0: 16 B of scales, then 16 chunks of 16 codes
                const i4 sc = *reinterpret_cast<const i4 *>(krow);
#pragma unroll
                for (int jj = 0; jj < C::NMF / 2; ++jj) {
                    const i4 w = *reinterpret_cast<const i4 *>(krow + 16 + (4 * jj + g) * 16);
                    const uint32_t sw = (uint32_t) sc[jj];
                    const uint32_t d16 = (g & 2) ? (sw >> 16) : (sw & 0xffffu);
                    const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
                    const u2 x0 = deq4((uint32_t) w[0], dd, dd), x1 = deq4((uint32_t) w[1], dd, dd);
                    const u2 x2 = deq4((uint32_t) w[2], dd, dd), x3 = deq4((uint32_t) w[3], dd, dd);
                    const u4 a0 = {x0.lo, x0.hi, x1.lo, x1.hi}, a1 = {x2.lo, x2.hi, x3.lo, x3.hi};
#pragma unroll
                    for (int r = 0; r < NT; ++r) {
                        s[r][st] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a0), qf[r][2 * jj], s[r][st], 0, 0, 0);
                        s[r][st] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a1), qf[r][2 * jj + 1], s[r][st], 0, 0, 0);
                    }
                }
            }
        }

        if (it_ < 1) TS(3 + 5 * it_);
        if constexpr (KDMA) {   // the K tile has been consumed: fetch the next one into it
            if (have_n) issue_lds(kt, P.kc, tsn, n_max - 1 - tsn);
        }

        // ---- online softmax (log2 domain); column = query row, this lane holds keys 16 st + 4 g + i ----
        h8 pb[NT];
        float alpha[NT];
        bool rescale = false;
#pragma unroll
        for (int r = 0; r < NT; ++r) {
            float mloc = NEG_INF;
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int kp = ts + 16 * st + 4 * g + i;
                    s[r][st][i] = kp <= plim[r] ? s[r][st][i] : NEG_INF;
                    mloc = fmaxf(mloc, s[r][st][i]);
                }
            mloc = fmaxf(mloc, __shfl_xor(mloc, 16));
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
            const float mnew = fmaxf(m_run[r], mloc);
            const bool dead = mnew == NEG_INF;
            // nothing accumulated yet (m = -inf): the accumulators are zero and need no rescale
            alpha[r] = (dead || m_run[r] == NEG_INF) ? 1.0f : __builtin_amdgcn_exp2f(m_run[r] - mnew);
            m_run[r] = mnew;
            float p[8];
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int i = 0; i < 4; ++i) p[4 * st + i] = dead ? 0.0f : __builtin_amdgcn_exp2f(s[r][st][i] - mnew);
            pb[r] = h8{(half_t) p[0], (half_t) p[1], (half_t) p[2], (half_t) p[3], (half_t) p[4], (half_t) p[5], (half_t) p[6], (half_t) p[7]};
            rescale = rescale || alpha[r] != 1.0f;
        }
        if (__any(rescale)) {
#pragma unroll
            for (int r = 0; r < NT; ++r) {
                ol[r] *= alpha[r];
#pragma unroll
                for (int j = 0; j < C::NDT; ++j) o[r][j] *= alpha[r];
            }
        }

        // ---- V tile to LDS, next V loads into the vacated registers ----
        if (it_ < 1) TS(4 + 5 * it_);
        park(vt, vr);
        if (it_ < 1) TS(5 + 5 * it_);
        if (have_n) issue(vr, P.vc, tsn, n_max - 1 - tsn);

        // slot e of lane group g is key 4 g + e (e < 4) or 16 + 4 g + e - 4: the keys this lane's P values belong to
        if constexpr (KT == P1A_KV_F16) {
            const int kk = c >> 2, jq = c & 3;
            const char * r0 = vt + (4 * g + kk) * C::KSTR + jq * 8;
            const char * r1 = vt + (16 + 4 * g + kk) * C::KSTR + jq * 8;
#pragma unroll
            for (int j = 0; j < C::NDT; ++j) {
                const s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *) (r0 + j * 32));
                const s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *) (r1 + j * 32));
                const h4 l4 = __builtin_bit_cast(h4, lo), h4_ = __builtin_bit_cast(h4, hi);
                const h8 a = {l4[0], l4[1], l4[2], l4[3], h4_[0], h4_[1], h4_[2], h4_[3]};
#pragma unroll
                for (int r = 0; r < NT; ++r) o[r][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pb[r], o[r][j], 0, 0, 0);
            }
        } else {
            {   // transposed scale table tab[b][g][e] (f16): one 16-byte row per (block, lane group)
                const int key = lane & 31, hf = lane >> 5;
                const i2 sc = *reinterpret_cast<const i2 *>(vt + key * C::KSTR + 8 * hf);
                const int st = key >> 4, kk = key & 15;
                char * dst = tab + (kk >> 2) * 16 + ((kk & 3) + 4 * st) * 2;
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const uint32_t wv = (uint32_t) sc[x >> 1];
                    *reinterpret_cast<uint16_t *>(dst + (4 * hf + x) * 64) = (uint16_t) ((x & 1) ? (wv >> 16) : wv);
                }
            }
            const int kk = c >> 1, jb = c & 1;
            const int key = kk < 4 ? 4 * g + kk : 16 + 4 * g + (kk - 4);
            const char * vrow = vt + key * C::KSTR + 16 + 8 * jb;
#pragma unroll
            for (int j = 0; j < C::NDT; ++j) {
                const i2 w = __builtin_amdgcn_ds_read_tr8_b64_v2i32((i2 __attribute__((address_space(3))) *) (vrow + j * 16));
                const h8 dv = *reinterpret_cast<const h8 *>(tab + (j >> 1) * 64 + g * 16);
                const u2 x0 = deq4((uint32_t) w[0], h2{dv[0], dv[1]}, h2{dv[2], dv[3]});
                const u2 x1 = deq4((uint32_t) w[1], h2{dv[4], dv[5]}, h2{dv[6], dv[7]});
                const u4 a = {x0.lo, x0.hi, x1.lo, x1.hi};
#pragma unroll
                for (int r = 0; r < NT; ++r) o[r][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a), pb[r], o[r][j], 0, 0, 0);
            }
        }
#pragma unroll
        for (int r = 0; r < NT; ++r) ol[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pb[r], ol[r], 0, 0, 0);
        u = un;
        have = have_n;
        if (it_ < 1) TS(6 + 5 * it_);
        ++it_;
    }
    TS(12);

    // ---- fold the WPH waves of each head (in sub order) and write one partial per (workgroup, head); the 16
    // columns of one MFMA tile at a time, so that a column is merged the same way whatever NT is. A wave parks its
    // state in its own (now idle) tile region, so no barrier is needed before the first write ----
    float * wreg = reinterpret_cast<float *>(lds + wave * C::WAVE_B);   // [16 m][16 l][16 columns][D]
#pragma unroll
    for (int r = 0; r < NT; ++r) {
        const int Rr = min(16, R - 16 * r);                  // live columns of this tile
        if (r) __syncthreads();
        if (c < Rr) {
#pragma unroll
            for (int j = 0; j < C::NDT; ++j) *reinterpret_cast<f4 *>(wreg + 32 + c * D + 16 * j + 4 * g) = o[r][j];
            if (g == 0) { wreg[c] = m_run[r]; wreg[16 + c] = ol[r][0]; }
        }
        __syncthreads();
        const int items = P.HPW * Rr * (D / 4);
        for (int it = threadIdx.x; it < items; it += NWV * 64) {
            const int d4 = it % (D / 4), rest = it / (D / 4);
            const int cc = rest % Rr, hs = rest / Rr;
            float M = NEG_INF;
            for (int sb = 0; sb < WPH; ++sb)
                M = fmaxf(M, reinterpret_cast<const float *>(lds + (hs + sb * P.HPW) * C::WAVE_B)[cc]);
            f4 acc = {0.f, 0.f, 0.f, 0.f};
            float l = 0.f;
            for (int sb = 0; sb < WPH; ++sb) {
                const float * wr = reinterpret_cast<const float *>(lds + (hs + sb * P.HPW) * C::WAVE_B);
                const float ms = wr[cc];
                if (ms == NEG_INF) continue;
                const float f = __builtin_amdgcn_exp2f(ms - M);
                const f4 a = *reinterpret_cast<const f4 *>(wr + 32 + cc * D + 4 * d4);
                acc += a * f;
                l += wr[16 + cc] * f;
            }
            const int col = 16 * r + cc;
            const int t = col / P.GQA, hh = col - t * P.GQA;
            const size_t row = (size_t) (row0 + t) * P.Hq + (size_t) (hg * P.HPW + hs) * P.GQA + hh;
            if (M != NEG_INF) *reinterpret_cast<f4 *>(P.part_o + (row * P.nsplit + split) * D + 4 * d4) = acc;
            if (d4 == 0) {
                float * pm = P.part_ml + (row * P.nsplit + split) * 2;
                pm[0] = M;
                pm[1] = l;
            }
        }
    }
    TS(13);
}

// ---- generic path: any D % 32 == 0 (<= 512), any GQA, every type; one wave per (split stream, q head, row) ----
template <uint32_t KT>
__device__ __forceinline__ float kv_elem(const char * head, int D, int d) {
    if constexpr (KT == P1A_KV_F16) return (float) reinterpret_cast<const half_t *>(head)[d];
    else if constexpr (KT == P1A_KV_Q8_0) {
        const float sc = (float) reinterpret_cast<const half_t *>(head)[d >> 5];
        return sc * (float) reinterpret_cast<const int8_t *>(head + (D / 32) * 2)[d];
    } else {
        const char * b = head + (d >> 5) * 18;
        const float sc = (float) *reinterpret_cast<const half_t *>(b);
        const int i = d & 31;
        const uint32_t by = (uint8_t) b[2 + (i & 15)];
        return (float) ((int) (i < 16 ? (by & 15) : (by >> 4)) - 8) * sc;
    }
}

struct gen_params {
    const float * q;
    const char * kc;
    const char * vc;
    float * part_o;
    float * part_ml;
    kv_view pg;
    int p0;
    const int32_t * p0_dev;
    const int32_t * pos_rows;
    int RG, Hq, Hkv, D;
    float qscale;
    int nsplit;
};

constexpr int GEN_MAXV = 8;   // dims per lane: D <= 512

template <uint32_t KT>
__global__ void __launch_bounds__(256) dec_generic_k(const gen_params P) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = blockIdx.y, t = blockIdx.z, D = P.D;
    const int hk = h / (P.Hq / P.Hkv);
    const int pos = P.pos_rows ? P.pos_rows[t] : (P.p0_dev ? *P.p0_dev : P.p0) + t;
    const int grow = P.pos_rows ? (t / P.RG) * P.RG : 0;   // the row whose page table the group uses
    const int32_t * ptab = kv_tab(P.pg, grow);
    const size_t hb = KT == P1A_KV_F16 ? (size_t) D * 2 : KT == P1A_KV_Q8_0 ? (size_t) (D / 32) * 34 : (size_t) (D / 32) * 18;
    const int nv = D / 64 + (D % 64 ? 1 : 0);
    float qv[GEN_MAXV], acc[GEN_MAXV];
    const float * qr = P.q + ((size_t) t * P.Hq + h) * D;
#pragma unroll
    for (int x = 0; x < GEN_MAXV; ++x) {
        const int d = x * 64 + lane;
        qv[x] = (x < nv && d < D) ? (float) (half_t) (qr[d] * P.qscale) : 0.f;
        acc[x] = 0.f;
    }
    float m = NEG_INF, l = 0.f;
    const int sp = blockIdx.x * 4 + wave, NS = P.nsplit * 4;
    for (int j = sp; j <= pos; j += NS) {
        const size_t o = kv_off_tab(P.pg, ptab, j) + (size_t) hk * hb;
        float dot = 0.f;
#pragma unroll
        for (int x = 0; x < GEN_MAXV; ++x) {
            const int d = x * 64 + lane;
            if (x < nv && d < D) dot += qv[x] * kv_elem<KT>(P.kc + o, D, d);
        }
#pragma unroll
        for (int w = 32; w > 0; w >>= 1) dot += __shfl_xor(dot, w);
        const float mn = fmaxf(m, dot);
        const float a = __builtin_amdgcn_exp2f(m - mn), p = __builtin_amdgcn_exp2f(dot - mn);
        l = l * a + p;
#pragma unroll
        for (int x = 0; x < GEN_MAXV; ++x) {
            const int d = x * 64 + lane;
            if (x < nv && d < D) acc[x] = acc[x] * a + p * kv_elem<KT>(P.vc + o, D, d);
        }
        m = mn;
    }
    const size_t row = (size_t) t * P.Hq + h;
    float * po = P.part_o + (row * NS + sp) * D;
#pragma unroll
    for (int x = 0; x < GEN_MAXV; ++x) {
        const int d = x * 64 + lane;
        if (x < nv && d < D) po[d] = acc[x];
    }
    if (lane == 0) {
        P.part_ml[(row * NS + sp) * 2] = m;
        P.part_ml[(row * NS + sp) * 2 + 1] = l;
    }
}

// ---- merge of the split partials, in a fixed order, with the fused sigmoid gate ----
// out[row][d] = sum_s 2^(m_s - M) O_s[d] / sum_s 2^(m_s - M) l_s; empty streams (m = -inf or l = 0) are skipped.
// One wave per (row, 32 dims): lane = (slice of the splits, 4 dims); slice k folds splits k, k + 8, ... in order and
// the 8 slices are then added in order, so the result depends on nothing but the partials.
__global__ void __launch_bounds__(64) merge_k(const float * __restrict__ part_o, const float * __restrict__ part_ml,
                                              float * __restrict__ out, const float * __restrict__ gate, int NS, int D) {
    __shared__ f4 sacc[8][8];
    __shared__ float sden[8];
    const size_t row = blockIdx.x;
    const int tid = threadIdx.x, q4 = tid & 7, sl = tid >> 3;
    const int d = blockIdx.y * 32 + q4 * 4;
    const float * ml = part_ml + row * NS * 2;
    float M = NEG_INF;
    for (int s = tid; s < NS; s += 64) M = fmaxf(M, ml[2 * s]);
#pragma unroll
    for (int w = 32; w > 0; w >>= 1) M = fmaxf(M, __shfl_xor(M, w));
    f4 num = {0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
    for (int s = sl; s < NS; s += 8) {
        const float ms = ml[2 * s], ls = ml[2 * s + 1];
        if (ms == NEG_INF || ls == 0.f) continue;
        const float f = __builtin_amdgcn_exp2f(ms - M);
        const f4 a = *reinterpret_cast<const f4 *>(part_o + (row * NS + s) * D + d);
        den = fmaf(f, ls, den);
        num[0] = fmaf(f, a[0], num[0]); num[1] = fmaf(f, a[1], num[1]);
        num[2] = fmaf(f, a[2], num[2]); num[3] = fmaf(f, a[3], num[3]);
    }
    sacc[sl][q4] = num;
    if (q4 == 0) sden[sl] = den;
    __syncthreads();
    if (sl == 0) {
        f4 n = sacc[0][q4];
        float dn = sden[0];
#pragma unroll
        for (int k = 1; k < 8; ++k) { n += sacc[k][q4]; dn += sden[k]; }
        f4 r = {n[0] / dn, n[1] / dn, n[2] / dn, n[3] / dn};
        if (gate) {
            const f4 gt = *reinterpret_cast<const f4 *>(gate + row * D + d);
#pragma unroll
            for (int x = 0; x < 4; ++x) r[x] *= 1.0f / (1.0f + expf(-gt[x]));
        }
        *reinterpret_cast<f4 *>(out + row * D + d) = r;
    }
}

__global__ void __launch_bounds__(256) sigmoid_mul_k(float * __restrict__ x, const float * __restrict__ g, size_t n) {
    for (size_t i = (size_t) blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t) gridDim.x * 256)
        x[i] *= 1.0f / (1.0f + expf(-g[i]));
}

// ---- launch plan: which kernel a shape takes, and how the keys are split ----
// The MFMA kernel needs 16-byte aligned head rows (f16: D in {64, 128, 256}; q8_0: D == 256), 16-byte aligned
// bases and strides, pages of >= 16 positions and GQA <= 16. Everything else takes the generic kernel.
struct dec_plan {
    bool mfma;
    int GQA, HPW, NW, NT, RG;
    int nsplit;    // split streams
    int NS;        // partials per output row (what merge_k folds)
};

bool mfma_ok(const p1a_kv & c, int GQA) {
    if (GQA < 1 || GQA > 16) return false;
    if (c.type == P1A_KV_F16) { if (c.D != 64 && c.D != 128 && c.D != 256) return false; }
    else if (c.type == P1A_KV_Q8_0) { if (c.D != 256) return false; }
    else return false;
    if (((uintptr_t) c.k | (uintptr_t) c.v) & 15) return false;
    if (c.pt && ((c.pstride & 15) || c.psh < 4)) return false;
    return true;
}

int env_int(const char * name, int dflt) {
    const char * e = getenv(name);
    return e && *e ? atoi(e) : dflt;
}

dec_plan make_plan(const p1a_kv & c, int Hq, int rows_per_group, int nsplit_req, int cus) {
    dec_plan p;
    p.GQA = Hq / c.Hkv;
    p.mfma = mfma_ok(c, p.GQA);
    if (!p.mfma) {
        p.HPW = 1; p.NW = 4; p.NT = 1;
        p.RG = rows_per_group < 1 ? 1 : rows_per_group;   // no sharing here: the group only selects the page table
        int n = nsplit_req > 0 ? nsplit_req : 2 * cus / Hq;
        p.nsplit = n < 1 ? 1 : (n > 1024 ? 1024 : n);
        p.NS = p.nsplit * 4;
        return p;
    }
    const int cap = 32 / p.GQA < 4 ? 32 / p.GQA : 4;
    p.RG = rows_per_group < 1 ? 1 : (rows_per_group > cap ? cap : rows_per_group);
    // tuning knobs (development A/B switches, read once): heads per workgroup and waves per workgroup
    static const int env_hpw = env_int("P1A_DEC_HPW", 0), env_nw = env_int("P1A_DEC_NW", 0);
    int hpw = c.Hkv % 4 == 0 ? 4 : c.Hkv % 2 == 0 ? 2 : 1;
    if (env_hpw > 0 && env_hpw <= hpw && hpw % env_hpw == 0) hpw = env_hpw;
    p.HPW = hpw;
    const bool big_tiles = c.type == P1A_KV_F16 && c.D == 256;   // 34 KB of LDS per wave
    p.NW = big_tiles ? 4 : 8;
    if (env_nw == 4 || (env_nw == 8 && !big_tiles)) p.NW = env_nw;
    const int HG = c.Hkv / p.HPW;
    const int wg_per_cu = p.NW == 8 ? 1 : 2;
    int n = nsplit_req > 0 ? nsplit_req : wg_per_cu * cus / HG;
    if (n >= 8) n &= ~7;
    p.nsplit = n < 1 ? 1 : (n > 1024 ? 1024 : n);
    return p;
}

void finish_plan(dec_plan & p) {
    p.NT = p.RG * p.GQA <= 16 ? 1 : 2;
    if (p.mfma) p.NS = p.nsplit;
}

template <uint32_t KT, int D>
int launch_mfma(const p1a_kv & c, const decode_args & a, const dec_plan & pl, hipStream_t s) {
    dec_params P;
    P.q = a.q; P.kc = (const char *) c.k; P.vc = (const char *) c.v;
    P.part_o = a.part_o; P.part_ml = a.part_ml; P.pg = view_of(c);
    P.p0 = a.p0; P.p0_dev = a.p0_dev; P.pos_rows = a.pos_rows;
    P.T = a.T; P.RG = pl.RG; P.Hq = a.Hq; P.Hkv = c.Hkv; P.GQA = pl.GQA; P.HPW = pl.HPW;
    P.qscale = a.scale * 1.4426950408889634f; P.nsplit = pl.nsplit;
    const dim3 grid(pl.nsplit * (c.Hkv / pl.HPW), (a.T + pl.RG - 1) / pl.RG);
    constexpr bool big_tiles = KT == P1A_KV_F16 && D == 256;
    if (pl.NW == 8) {
        if constexpr (!big_tiles) {
            if (pl.NT == 1) dec_mfma_k<KT, D, 1, 8><<<grid, 512, 0, s>>>(P);
            else dec_mfma_k<KT, D, 2, 8><<<grid, 512, 0, s>>>(P);
        }
    } else {
        if (pl.NT == 1) dec_mfma_k<KT, D, 1, 4><<<grid, 256, 0, s>>>(P);
        else dec_mfma_k<KT, D, 2, 4><<<grid, 256, 0, s>>>(P);
    }
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

}   // namespace

// bytes of split scratch (accumulators, then (m, l) pairs) a call with these arguments needs
void decode_scratch_need(const p1a_kv & c, int Hq, int rows, int rows_per_group, int nsplit_req, int cus,
                         size_t & bytes_o, size_t & bytes_ml) {
    dec_plan pl = make_plan(c, Hq, rows_per_group, nsplit_req, cus);
    finish_plan(pl);
    bytes_o = (size_t) rows * Hq * pl.NS * c.D * sizeof(float);
    bytes_ml = (size_t) rows * Hq * pl.NS * 2 * sizeof(float);
}

int decode_rows_per_group(const p1a_kv & c, int Hq, int want) {
    return make_plan(c, Hq, want, 0, 256).RG;
}

int decode_nsplit(const p1a_kv & c, int Hq, int nsplit_req, int cus) { return make_plan(c, Hq, 1, nsplit_req, cus).nsplit; }

int launch_decode(const p1a_kv & c, const decode_args & a, hipStream_t s) {
    dec_plan pl = make_plan(c, a.Hq, a.rows_per_group, a.nsplit, a.cus);
    pl.RG = a.rows_per_group;
    finish_plan(pl);
    int rc;
    if (pl.mfma) {
        if (c.type == P1A_KV_Q8_0) rc = launch_mfma<P1A_KV_Q8_0, 256>(c, a, pl, s);
        else if (c.D == 256) rc = launch_mfma<P1A_KV_F16, 256>(c, a, pl, s);
        else if (c.D == 128) rc = launch_mfma<P1A_KV_F16, 128>(c, a, pl, s);
        else rc = launch_mfma<P1A_KV_F16, 64>(c, a, pl, s);
    } else {
        gen_params P;
        P.q = a.q; P.kc = (const char *) c.k; P.vc = (const char *) c.v;
        P.part_o = a.part_o; P.part_ml = a.part_ml; P.pg = view_of(c);
        P.p0 = a.p0; P.p0_dev = a.p0_dev; P.pos_rows = a.pos_rows; P.RG = pl.RG;
        P.Hq = a.Hq; P.Hkv = c.Hkv; P.D = c.D; P.qscale = a.scale * 1.4426950408889634f; P.nsplit = pl.nsplit;
        const dim3 grid(pl.nsplit, a.Hq, a.T);
        if (c.type == P1A_KV_F16) dec_generic_k<P1A_KV_F16><<<grid, 256, 0, s>>>(P);
        else if (c.type == P1A_KV_Q8_0) dec_generic_k<P1A_KV_Q8_0><<<grid, 256, 0, s>>>(P);
        else dec_generic_k<P1A_KV_Q4_0><<<grid, 256, 0, s>>>(P);
        rc = hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
    }
    if (rc != P1A_OK) return rc;
    merge_k<<<dim3(a.T * a.Hq, c.D / 32), 64, 0, s>>>(a.part_o, a.part_ml, a.out, a.gate, pl.NS, c.D);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

#ifdef P1A_TRACE
extern "C" void p1a_set_trace(long long * buf) { (void) hipMemcpyToSymbol(HIP_SYMBOL(g_trace), &buf, sizeof buf); }
#endif

int launch_sigmoid_mul(float * x, const float * g, size_t n, hipStream_t s) {
    const size_t nb = (n + 255) / 256;
    sigmoid_mul_k<<<(unsigned) (nb > 4096 ? 4096 : (nb ? nb : 1)), 256, 0, s>>>(x, g, n);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

}   // namespace p1a
