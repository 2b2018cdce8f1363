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

namespace p1a {
namespace {

constexpr int NW = 4;           // waves per workgroup
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

template <uint32_t KT, int D, int NT>
__global__ void __launch_bounds__(NW * 64, 2) dec_mfma_k(const dec_params P) {
    using C = tile_cfg<KT, D>;
    __shared__ __attribute__((aligned(16))) char lds[NW * C::WAVE_B];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int hk = blockIdx.y * P.HPW + (wave % P.HPW);
    const int sub = wave / P.HPW, WPH = NW / P.HPW;
    const int U = 32 * WPH;                                   // positions per unit
    const int row0 = blockIdx.z * P.RG;
    const int nr = min(P.RG, P.T - row0);                     // rows of this group
    const int R = nr * P.GQA;                                 // live MFMA columns
    const int p0v = P.pos_rows ? 0 : (P.p0_dev ? *P.p0_dev : P.p0);

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
#pragma unroll
    for (int r = 0; r < NT; ++r) {
        const int col = 16 * r + c;
        plim[r] = -1;
        if (col < R) {
            const int t = col / P.GQA;
            plim[r] = P.pos_rows ? P.pos_rows[row0 + t] : p0v + row0 + t;
        }
    }

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
    const int32_t * ptab = kv_tab(P.pg, P.pos_rows ? row0 : 0);
    const size_t head_off = (size_t) hk * C::HB;

    for (int u = blockIdx.x; u * U + sub * 32 < n_max; u += P.nsplit) {
        const int ts = u * U + sub * 32;                      // first position of this wave's tile
        const int last = n_max - 1 - ts;                      // keys past `last` are clamped onto it (never weighted)
        // ---- global loads of the K and V tiles, 16 bytes per lane in memory order ----
        const size_t off0 = kv_off_tab(P.pg, ptab, ts);
        const size_t off1 = last >= 16 ? kv_off_tab(P.pg, ptab, ts + 16) : off0;
        i4 kr[C::NRND], vr[C::NRND];
        int lofs[C::NRND];
#pragma unroll
        for (int rd = 0; rd < C::NRND; ++rd) {
            const int i = rd * 64 + lane;
            const int key = i / C::CPK, cir = i - key * C::CPK;
            const int kcl = min(key, last);
            const size_t go = ((kcl & 16) ? off1 : off0) + (size_t) (kcl & 15) * P.pg.rowb + head_off + (size_t) cir * 16;
            lofs[rd] = key * C::KSTR + cir * 16;
            if (C::NCH % 64 == 0 || i < C::NCH) { kr[rd] = ldg16(P.kc + go); vr[rd] = ldg16(P.vc + go); }
        }
        // ---- K tile to LDS ----
#pragma unroll
        for (int rd = 0; rd < C::NRND; ++rd)
            if (C::NCH % 64 == 0 || rd * 64 + lane < C::NCH) *reinterpret_cast<i4 *>(kt + lofs[rd]) = kr[rd];

        // ---- S^T = K Q^T for the two 16-key sub-tiles ----
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
                    const h2 off = {(half_t) 1152, (half_t) 1152};
                    h2 v[8];
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        codes4_to_h((uint32_t) w[x], v[2 * x], v[2 * x + 1]);
                        v[2 * x] = (v[2 * x] - off) * dd;
                        v[2 * x + 1] = (v[2 * x + 1] - off) * dd;
                    }
                    const h8 a0 = {v[0][0], v[0][1], v[1][0], v[1][1], v[2][0], v[2][1], v[3][0], v[3][1]};
                    const h8 a1 = {v[4][0], v[4][1], v[5][0], v[5][1], v[6][0], v[6][1], v[7][0], v[7][1]};
#pragma unroll
                    for (int r = 0; r < NT; ++r) {
                        s[r][st] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, qf[r][2 * jj], s[r][st], 0, 0, 0);
                        s[r][st] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, qf[r][2 * jj + 1], s[r][st], 0, 0, 0);
                    }
                }
            }
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
            alpha[r] = dead ? 1.0f : __builtin_amdgcn_exp2f(m_run[r] - mnew);
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

        // ---- V tile to LDS (the loads were issued with K's) ----
#pragma unroll
        for (int rd = 0; rd < C::NRND; ++rd)
            if (C::NCH % 64 == 0 || rd * 64 + lane < C::NCH) *reinterpret_cast<i4 *>(vt + lofs[rd]) = vr[rd];

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
                const h2 off = {(half_t) 1152, (half_t) 1152};
                h2 v0, v1, v2, v3;
                codes4_to_h((uint32_t) w[0], v0, v1);
                codes4_to_h((uint32_t) w[1], v2, v3);
                v0 = (v0 - off) * h2{dv[0], dv[1]};
                v1 = (v1 - off) * h2{dv[2], dv[3]};
                v2 = (v2 - off) * h2{dv[4], dv[5]};
                v3 = (v3 - off) * h2{dv[6], dv[7]};
                const h8 a = {v0[0], v0[1], v1[0], v1[1], v2[0], v2[1], v3[0], v3[1]};
#pragma unroll
                for (int r = 0; r < NT; ++r) o[r][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pb[r], o[r][j], 0, 0, 0);
            }
        }
#pragma unroll
        for (int r = 0; r < NT; ++r) ol[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pb[r], ol[r], 0, 0, 0);
    }

    // ---- partial results: split index = stream * WPH + sub ----
    const int NS = P.nsplit * WPH;
    const int sp = blockIdx.x * WPH + sub;
#pragma unroll
    for (int r = 0; r < NT; ++r) {
        const int col = 16 * r + c;
        if (col >= R) continue;
        const int t = col / P.GQA, hh = col - t * P.GQA;
        const size_t row = (size_t) (row0 + t) * P.Hq + (size_t) hk * P.GQA + hh;
        float * po = P.part_o + (row * NS + sp) * D;
        if (m_run[r] != NEG_INF) {   // merge_k never reads the accumulator of an empty stream
#pragma unroll
            for (int j = 0; j < C::NDT; ++j) *reinterpret_cast<f4 *>(po + 16 * j + 4 * g) = o[r][j];
        }
        if (g == 0) {
            float * pm = P.part_ml + (row * NS + sp) * 2;
            pm[0] = m_run[r];
            pm[1] = ol[r][0];
        }
    }
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

// ---- merge of the split partials, in split order, with the fused sigmoid gate ----
// out[row][d] = sum_s 2^(m_s - M) O_s[d] / sum_s 2^(m_s - M) l_s; empty streams (l == 0) are skipped.
__global__ void __launch_bounds__(256) merge_k(const float * __restrict__ part_o, const float * __restrict__ part_ml,
                                               float * __restrict__ out, const float * __restrict__ gate, int NS, int D) {
    const size_t row = blockIdx.x;
    const float * ml = part_ml + row * NS * 2;
    float M = NEG_INF;
    for (int s = 0; s < NS; ++s) M = fmaxf(M, ml[2 * s]);
    for (int d = threadIdx.x * 4; d < D; d += blockDim.x * 4) {
        float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
        float den = 0.f;
        for (int s = 0; s < NS; ++s) {
            const float ms = ml[2 * s], ls = ml[2 * s + 1];
            if (ms == NEG_INF || ls == 0.f) continue;
            const float f = __builtin_amdgcn_exp2f(ms - M);
            const float4 a = *reinterpret_cast<const float4 *>(part_o + (row * NS + s) * D + d);
            den = fmaf(f, ls, den);
            num.x = fmaf(f, a.x, num.x); num.y = fmaf(f, a.y, num.y); num.z = fmaf(f, a.z, num.z); num.w = fmaf(f, a.w, num.w);
        }
        float4 r = make_float4(num.x / den, num.y / den, num.z / den, num.w / den);
        if (gate) {
            const float4 gt = *reinterpret_cast<const float4 *>(gate + row * D + d);
            r.x *= 1.0f / (1.0f + expf(-gt.x)); r.y *= 1.0f / (1.0f + expf(-gt.y));
            r.z *= 1.0f / (1.0f + expf(-gt.z)); r.w *= 1.0f / (1.0f + expf(-gt.w));
        }
        *reinterpret_cast<float4 *>(out + row * D + d) = r;
    }
}

__global__ void __launch_bounds__(256) sigmoid_mul_k(float * __restrict__ x, const float * __restrict__ g, size_t n) {
    for (size_t i = (size_t) blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t) gridDim.x * 256)
        x[i] *= 1.0f / (1.0f + expf(-g[i]));
}

template <uint32_t KT, int D>
int launch_mfma(const p1a_kv & c, const decode_args & a, int HPW, int GQA, hipStream_t s) {
    dec_params P;
    P.q = a.q; P.kc = (const char *) c.k; P.vc = (const char *) c.v;
    P.part_o = a.part_o; P.part_ml = a.part_ml; P.pg = view_of(c);
    P.p0 = a.p0; P.p0_dev = a.p0_dev; P.pos_rows = a.pos_rows;
    P.T = a.T; P.RG = a.rows_per_group; P.Hq = a.Hq; P.Hkv = c.Hkv; P.GQA = GQA; P.HPW = HPW;
    P.qscale = a.scale * 1.4426950408889634f; P.nsplit = a.nsplit;
    const dim3 grid(a.nsplit, c.Hkv / HPW, (a.T + a.rows_per_group - 1) / a.rows_per_group);
    if (a.rows_per_group * GQA <= 16) dec_mfma_k<KT, D, 1><<<grid, NW * 64, 0, s>>>(P);
    else dec_mfma_k<KT, D, 2><<<grid, NW * 64, 0, s>>>(P);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

}   // namespace

// Which kernel a shape takes. The MFMA kernel needs 16-byte aligned head rows (f16: D in {64, 128, 256}; q8_0:
// D == 256), 16-byte aligned bases and strides, pages of >= 16 positions and GQA <= 16.
static bool mfma_ok(const p1a_kv & c, int GQA) {
    if (GQA < 1 || GQA > 16) return false;
    if (c.type == P1A_KV_F16) { if (c.D != 64 && c.D != 128 && c.D != 256) return false; }
    else if (c.type == P1A_KV_Q8_0) { if (c.D != 256) return false; }
    else return false;
    if (((uintptr_t) c.k | (uintptr_t) c.v) & 15) return false;
    if (c.pt && ((c.pstride & 15) || c.psh < 4)) return false;
    return true;
}

// Split bookkeeping shared with the API layer: the partial buffers hold nsplit * streams_per_split entries per row,
// and the default nsplit puts about two workgroups on every compute unit for one row group.
int decode_streams_per_split(const p1a_kv & c, int Hq) {
    const int GQA = Hq / c.Hkv;
    if (!mfma_ok(c, GQA)) return 4;
    const int HPW = c.Hkv % 4 == 0 ? 4 : c.Hkv % 2 == 0 ? 2 : 1;
    return NW / HPW;
}

int decode_default_nsplit(const p1a_kv & c, int Hq, int cus) {
    const int GQA = Hq / c.Hkv;
    int per_split;   // workgroups per split stream and row group
    if (mfma_ok(c, GQA)) per_split = c.Hkv / (c.Hkv % 4 == 0 ? 4 : c.Hkv % 2 == 0 ? 2 : 1);
    else per_split = Hq;
    int n = 2 * cus / (per_split < 1 ? 1 : per_split);
    return n < 1 ? 1 : (n > 1024 ? 1024 : n);
}

int decode_rows_per_group(const p1a_kv & c, int Hq, int want) {
    const int GQA = Hq / c.Hkv;
    if (!mfma_ok(c, GQA)) return want < 1 ? 1 : want;   // the generic kernel has no sharing; the group only picks the table
    const int cap = 32 / GQA < 4 ? 32 / GQA : 4;
    return want < 1 ? 1 : (want > cap ? cap : want);
}

int launch_decode(const p1a_kv & c, const decode_args & a, hipStream_t s) {
    const int GQA = a.Hq / c.Hkv;
    int rc;
    int NS;
    if (mfma_ok(c, GQA)) {
        const int HPW = c.Hkv % 4 == 0 ? 4 : c.Hkv % 2 == 0 ? 2 : 1;
        NS = a.nsplit * (NW / HPW);
        if (c.type == P1A_KV_Q8_0) rc = launch_mfma<P1A_KV_Q8_0, 256>(c, a, HPW, GQA, s);
        else if (c.D == 256) rc = launch_mfma<P1A_KV_F16, 256>(c, a, HPW, GQA, s);
        else if (c.D == 128) rc = launch_mfma<P1A_KV_F16, 128>(c, a, HPW, GQA, s);
        else rc = launch_mfma<P1A_KV_F16, 64>(c, a, HPW, GQA, s);
    } else {
        gen_params P;
        P.q = a.q; P.kc = (const char *) c.k; P.vc = (const char *) c.v;
        P.part_o = a.part_o; P.part_ml = a.part_ml; P.pg = view_of(c);
        P.p0 = a.p0; P.p0_dev = a.p0_dev; P.pos_rows = a.pos_rows; P.RG = a.rows_per_group;
        P.Hq = a.Hq; P.Hkv = c.Hkv; P.D = c.D; P.qscale = a.scale * 1.4426950408889634f; P.nsplit = a.nsplit;
        NS = a.nsplit * 4;
        const dim3 grid(a.nsplit, a.Hq, a.T);
        if (c.type == P1A_KV_F16) dec_generic_k<P1A_KV_F16><<<grid, 256, 0, s>>>(P);
        else if (c.type == P1A_KV_Q8_0) dec_generic_k<P1A_KV_Q8_0><<<grid, 256, 0, s>>>(P);
        else dec_generic_k<P1A_KV_Q4_0><<<grid, 256, 0, s>>>(P);
        rc = hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
    }
    if (rc != P1A_OK) return rc;
    merge_k<<<a.T * a.Hq, c.D >= 256 ? 64 : 32, 0, s>>>(a.part_o, a.part_ml, a.out, a.gate, NS, c.D);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

int launch_sigmoid_mul(float * x, const float * g, size_t n, hipStream_t s) {
    const size_t nb = (n + 255) / 256;
    sigmoid_mul_k<<<(unsigned) (nb > 4096 ? 4096 : (nb ? nb : 1)), 256, 0, s>>>(x, g, n);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

}   // namespace p1a
