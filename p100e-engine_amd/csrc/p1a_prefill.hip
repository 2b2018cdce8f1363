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

    // byte offsets of the rows this thread stages, for a tile starting at k0 (keys past pmax are clamped onto pmax)
    auto rowoffs = [&](int k0, size_t * ro) {
#pragma unroll
        for (int x = 0; x < S::NPT; ++x) {
            const int i = x * NTHR + tid, key = i / S::CPK;
            const int p = min(k0 + min(key, BN - 1), pmax);
            ro[x] = kv_off_tab(P.pg, ptab, p) + head_off;
        }
    };

    typename S::raw rk, rv;
    {
        size_t ro[S::NPT];
        rowoffs(0, ro);
        S::load(rk, P.kc, ro, tid);
        S::load(rv, P.vc, ro, tid);
    }
    S::store(rk, lds, C::KSTR, tid);
    S::store(rv, lds + C::KT_B, C::VSTR, tid);
    __syncthreads();

    for (int tile = 0; tile < ntiles; ++tile) {
        const int k0 = tile * BN;
        char * kt = lds + (tile & 1) * C::STAGE_B;
        char * vt = kt + C::KT_B;
        char * nkt = lds + ((tile + 1) & 1) * C::STAGE_B;
        const bool more = tile + 1 < ntiles;
        if (more) {   // raw loads of the next tile fly while this one is multiplied
            size_t ro[S::NPT];
            rowoffs(k0 + BN, ro);
            S::load(rk, P.kc, ro, tid);
            S::load(rv, P.vc, ro, tid);
        }
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
            const float mnew = fmaxf(m_run, mloc);             // finite: key k0 <= wave_pmin... is visible to every live row
            const bool dead = mnew == NEG_INF;
            const float alpha = (dead || m_run == NEG_INF) ? 1.0f : __builtin_amdgcn_exp2f(m_run - mnew);
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
            if (__any(alpha != 1.0f)) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    ol[i] *= alpha;
#pragma unroll
                    for (int dt = 0; dt < C::NDT; ++dt) o[dt][i] *= alpha;
                }
            }
        }
        if (more) {   // convert the next tile into the other buffer
            S::store(rk, nkt, C::KSTR, tid);
            S::store(rv, nkt + C::KT_B, C::VSTR, tid);
        }
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
                    o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb[ps], o[dt], 0, 0, 0);
                }
                ol = __builtin_amdgcn_mfma_f32_32x32x16_f16(ones, pb[ps], ol, 0, 0, 0);
            }
        }
        __syncthreads();
    }

    // ---- epilogue: normalise, gate, store. Lane (row c, half g) holds dims 32 dt + 8 (i / 4) + 4 g + (i % 4) ----
    if (live) {
        const float inv = 1.0f / ol[0];
        float * orow = P.out + ((size_t) my_tok * P.Hq + h) * D;
        const float * grow = P.gate ? P.gate + ((size_t) my_tok * P.Hq + h) * D : nullptr;
#pragma unroll
        for (int dt = 0; dt < C::NDT; ++dt)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int d0 = 32 * dt + 8 * q4 + 4 * g;
                f4 r = {o[dt][4 * q4] * inv, o[dt][4 * q4 + 1] * inv, o[dt][4 * q4 + 2] * inv, o[dt][4 * q4 + 3] * inv};
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

extern "C" size_t p1a_attn_prefill_scratch_bytes(int T, int p0, int Hq, int Hkv, int D) {
    (void) T; (void) p0; (void) Hq; (void) Hkv; (void) D;
    return 0;   // the kernel keeps every intermediate in registers and LDS
}
