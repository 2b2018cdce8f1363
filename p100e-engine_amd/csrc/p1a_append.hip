// Quantize-on-append KV write for gfx950: f32 K/V rows -> f16 / q8_0 / q4_0 cache rows, paged or contiguous.
// The arithmetic is the reference's (src/fast/kv_q8.cuh:20-49 = ggml quantize_row_q8_0_ref / quantize_row_q4_0_ref)
// and must stay bit-exact: this file is compiled with -ffp-contract=off, because x * id + 8.5f must round the product
// and the sum separately, and uses IEEE division for amax / 127 and 1 / d.
// Mapping: one lane owns 4 consecutive values (one 16-byte load for K, one for V), 8 lanes own a 32-value block and
// reduce over it with three xor-shuffles; a 256-thread workgroup covers 1024 values of one position row.
// The attention-layer input prep (q | gate split, per-head RMS norm * weight, NEOX rope, the same quantizing write) lives
// here too: its K codes depend on the last bit of the normed, rotated values, so it keeps a fixed operation order under
// the same no-contraction rule.
#include "p1a_common.hpp"

#pragma clang fp contract(off)

namespace p1a {
namespace {

// the maximum over the 8 lanes of a block, in every one of them: lane ^ 1, lane ^ 2 within the quad, then the mirrored
// half row (quad 0 <-> quad 1 of the 8) - on the data-parallel-primitive path, no LDS round trip; a maximum does not
// care about the order it is taken in
__device__ __forceinline__ float xor8_max(float a) {
    a = max_dpp<0xB1>(a);     // quad_perm [1, 0, 3, 2]
    a = max_dpp<0x4E>(a);     // quad_perm [2, 3, 0, 1]
    a = max_dpp<0x141>(a);    // row_half_mirror
    return a;
}

__device__ __forceinline__ uint16_t f16_bits(float f) {
    const half_t h = (half_t) f;   // v_cvt_f16_f32, round-to-nearest-even
    return __builtin_bit_cast(uint16_t, h);
}

// q8_0 block: head = first byte of the (position, kv head) row, b = block index, nb = blocks per head
__device__ __forceinline__ void q8_block(const float4 x, int j, char * head, int b, int nb) {
    const float amax = xor8_max(fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w))));
    const float d = amax / 127.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const int q0 = (int) roundf(x.x * id), q1 = (int) roundf(x.y * id), q2 = (int) roundf(x.z * id), q3 = (int) roundf(x.w * id);
    const uint32_t w = (uint32_t) (q0 & 0xff) | ((uint32_t) (q1 & 0xff) << 8) | ((uint32_t) (q2 & 0xff) << 16) | ((uint32_t) (q3 & 0xff) << 24);
    *reinterpret_cast<uint32_t *>(head + nb * 2 + b * 32 + j * 4) = w;
    if (j == 0) *reinterpret_cast<uint16_t *>(head + b * 2) = f16_bits(d);
}

// q4_0 block: blk = the 18-byte ggml block
__device__ __forceinline__ void q4_block(const float4 x, int j, char * blk) {
    // signed value of largest magnitude, first index on ties (strict > keeps the earlier one)
    float a = fabsf(x.x), xm = x.x;
    int idx = 4 * j;
    if (fabsf(x.y) > a) { a = fabsf(x.y); xm = x.y; idx = 4 * j + 1; }
    if (fabsf(x.z) > a) { a = fabsf(x.z); xm = x.z; idx = 4 * j + 2; }
    if (fabsf(x.w) > a) { a = fabsf(x.w); xm = x.w; idx = 4 * j + 3; }
#pragma unroll
    for (int o = 1; o < 8; o <<= 1) {
        const float oa = __shfl_xor(a, o), ox = __shfl_xor(xm, o);
        const int oi = __shfl_xor(idx, o);
        if (oa > a || (oa == a && oi < idx)) { a = oa; xm = ox; idx = oi; }
    }
    const float mx = a > 0.0f ? xm : 0.0f;
    const float d = mx / -8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    const float p0 = x.x * id, p1 = x.y * id, p2 = x.z * id, p3 = x.w * id;   // rounded products
    const int q0 = min(15, (int) (p0 + 8.5f)), q1 = min(15, (int) (p1 + 8.5f));
    const int q2 = min(15, (int) (p2 + 8.5f)), q3 = min(15, (int) (p3 + 8.5f));
    const int mine = q0 | (q1 << 8) | (q2 << 16) | (q3 << 24);
    const int hi = __shfl_down(mine, 4);   // lanes 4..7 of the block hold values 16..31 = the high nibbles
    if (j < 4) {
        const uint32_t w = (uint32_t) mine | ((uint32_t) hi << 4);
        uint16_t * dst = reinterpret_cast<uint16_t *>(blk + 2 + 4 * j);   // 2-byte aligned only
        dst[0] = (uint16_t) w;
        dst[1] = (uint16_t) (w >> 16);
    }
    if (j == 0) *reinterpret_cast<uint16_t *>(blk) = f16_bits(d);
}

template <uint32_t KT>
__global__ void __launch_bounds__(256) append_k(const float * __restrict__ k, const float * __restrict__ v, char * kc,
                                                char * vc, int p0, const int32_t * __restrict__ p0_dev,
                                                const int32_t * __restrict__ pos_rows, int Hkv, int D, kv_view pg) {
    const int t = blockIdx.y;
    const int i4 = blockIdx.x * 256 + threadIdx.x;   // index of this lane's 4 values within the row
    const int n4 = Hkv * D / 4;
    // lanes past the row still take part in the shuffles of their (non-existent) block; n4 % 8 == 0 so a block is
    // never split between live and dead lanes
    const bool live = i4 < n4;
    int pos;
    if (pos_rows) pos = pos_rows[t];
    else pos = (p0_dev ? *p0_dev : p0) + t;
    const size_t o = kv_off_tab(pg, kv_tab(pg, pos_rows ? t : 0), pos);
    float4 xk = make_float4(0.f, 0.f, 0.f, 0.f), xv = xk;
    if (live) {
        xk = reinterpret_cast<const float4 *>(k + (size_t) t * Hkv * D)[i4];
        xv = reinterpret_cast<const float4 *>(v + (size_t) t * Hkv * D)[i4];
    }
    if constexpr (KT == P1A_KV_F16) {
        if (live) {
            h4 hk = {(half_t) xk.x, (half_t) xk.y, (half_t) xk.z, (half_t) xk.w};
            h4 hv = {(half_t) xv.x, (half_t) xv.y, (half_t) xv.z, (half_t) xv.w};
            reinterpret_cast<h4 *>(kc + o)[i4] = hk;
            reinterpret_cast<h4 *>(vc + o)[i4] = hv;
        }
    } else {
        const int nb = D / 32;
        const int blk = i4 >> 3, j = i4 & 7;   // block over Hkv * nb, lane within the block
        const int h = blk / nb, b = blk - h * nb;
        if constexpr (KT == P1A_KV_Q8_0) {
            const size_t ho = o + (size_t) h * nb * 34;
            if (live) { q8_block(xk, j, kc + ho, b, nb); q8_block(xv, j, vc + ho, b, nb); }
            else { xor8_max(0.f); xor8_max(0.f); }
        } else {
            const size_t bo = o + (size_t) blk * 18;
            // dead lanes form whole 8-lane groups, so the live groups' shuffles never read them
            if (live) { q4_block(xk, j, kc + bo); q4_block(xv, j, vc + bo); }
        }
    }
}

// ---- attention-layer input prep: one wave per (head, token); lane i owns dims 4 i .. 4 i + 3 of the head ----
// Replaces the front half of the reference's attn_prep kernel (src/fast/fused.cu:512-573). Heads b < Hq are q heads
// (gate copy, norm, rope, store), Hq <= b < Hq + Hkv k heads (norm, rope, quantizing write), the rest v heads (write).
// Operation order (the CPU oracle keeps the same one, so K codes compare bit for bit): the squares of a lane's 4 values
// are added left to right, the 64 lane sums in a butterfly (a balanced binary tree); scale = 1 / sqrtf(ss / D + eps)
// with IEEE division and square root; angle = pos * (float) base^(-2 j / n_rot) in fp32, its cosine and sine rounded to
// fp32 - power, cosine and sine through the fixed recipes below, not through a math library; every product and sum
// rounded on its own.
//
// The elementary functions of the rotary angle are spelled out in IEEE double additions, multiplications, divisions and
// round-to-integer, in a fixed order without contraction, so that any IEEE machine gets the same bits (two math
// libraries differ in the last bit now and then, and a last bit moves a K code):
//   ln x    : x = m 2^e with m in [sqrt(1/2), sqrt(2)); s = (m - 1) / (m + 1); ln m = 2 s (1 + s^2/3 + ... + s^24/25) (host)
//   e^x     : k = rint(x log2 e); r = (x - k LN2_HI) - k LN2_LO; Taylor to r^13 in Horner form; scaled by 2^k
//   sin, cos: n = rint(t 2/pi); r = t - n pi/2 with pi/2 in four 24-bit pieces (n a_i is exact for n < 2^29);
//             the fdlibm kernel polynomials on |r| <= pi/4; quadrant n mod 4
// each is within an ulp or two of double precision; the results are then rounded to fp32.
__host__ __device__ inline double det_exp(double x) {
    const double LOG2E = 1.44269504088896338700e+00, LN2_HI = 6.93147180369123816490e-01, LN2_LO = 1.90821492927058770002e-10;
    const double k = __builtin_rint(x * LOG2E);
    const double r = (x - k * LN2_HI) - k * LN2_LO;
    double p = 1.0 / 6227020800.0;
    p = p * r + 1.0 / 479001600.0;
    p = p * r + 1.0 / 39916800.0;
    p = p * r + 1.0 / 3628800.0;
    p = p * r + 1.0 / 362880.0;
    p = p * r + 1.0 / 40320.0;
    p = p * r + 1.0 / 5040.0;
    p = p * r + 1.0 / 720.0;
    p = p * r + 1.0 / 120.0;
    p = p * r + 1.0 / 24.0;
    p = p * r + 1.0 / 6.0;
    p = p * r + 0.5;
    p = p * r + 1.0;
    p = p * r + 1.0;
    return __builtin_ldexp(p, (int) k);
}
__host__ __device__ inline void det_sincos(double t, float & c, float & s) {
    const double TWO_OVER_PI = 6.36619772367581382433e-01;
    const double A1 = 1.57079625129699707031e+00, A2 = 7.54978941586159635335e-08, A3 = 5.39030252995776476554e-15, A4 = 3.28200341580791294123e-22;
    const double n = __builtin_rint(t * TWO_OVER_PI);
    double r = t - n * A1;
    r = r - n * A2;
    r = r - n * A3;
    r = r - n * A4;
    const double z = r * r;
    const double S1 = -1.66666666666666324348e-01, S2 = 8.33333333332248946124e-03, S3 = -1.98412698298579493134e-04;
    const double S4 = 2.75573137070700676789e-06, S5 = -2.50507602534068634195e-08, S6 = 1.58969099521155010221e-10;
    const double C1 = 4.16666666666666019037e-02, C2 = -1.38888888888741095749e-03, C3 = 2.48015872894767294178e-05;
    const double C4 = -2.75573143513906633035e-07, C5 = 2.08757232129817482790e-09, C6 = -1.13596475577881948265e-11;
    double ps = S5 + z * S6;
    ps = S4 + z * ps;
    ps = S3 + z * ps;
    ps = S2 + z * ps;
    ps = S1 + z * ps;
    const double sn = r + (z * r) * ps;
    double pc = C5 + z * C6;
    pc = C4 + z * pc;
    pc = C3 + z * pc;
    pc = C2 + z * pc;
    pc = C1 + z * pc;
    const double cs = 1.0 - (0.5 * z - (z * z) * pc);
    const int q = (int) ((long long) n & 3);
    const double cc = q == 0 ? cs : q == 1 ? -sn : q == 2 ? -cs : sn;
    const double ss = q == 0 ? sn : q == 1 ? cs : q == 2 ? -sn : -cs;
    c = (float) cc;
    s = (float) ss;
}
inline double det_log(double x) {
    const double LN2_HI = 6.93147180369123816490e-01, LN2_LO = 1.90821492927058770002e-10;
    int e = 0;
    double m = __builtin_frexp(x, &e);                        // m in [1/2, 1)
    if (m < 7.07106781186547524401e-01) { m = m * 2.0; e -= 1; }
    const double s = (m - 1.0) / (m + 1.0), z = s * s;
    double p = 1.0 / 25.0;
    for (int k = 23; k >= 1; k -= 2) p = p * z + 1.0 / (double) k;
    const double lm = (2.0 * s) * p;
    return (double) e * LN2_HI + ((double) e * LN2_LO + lm);
}
template <uint32_t KT>
__global__ void __launch_bounds__(64) prep_k(const float * __restrict__ qg, const float * __restrict__ k,
                                             const float * __restrict__ v, const float * __restrict__ qn,
                                             const float * __restrict__ kn, const int32_t * __restrict__ pos,
                                             float * __restrict__ q, float * __restrict__ gate, char * kc, char * vc, int p0,
                                             int Hq, int Hkv, int D, int n_rot, double ln_base, float eps, int ldq, int ldk,
                                             int ldv, kv_view pg, mrope_view mr) {
    const int t = blockIdx.y, b = blockIdx.x, i = threadIdx.x;
    const bool live = 4 * i < D;                               // dead lanes form whole 8-lane groups (D % 32 == 0)
    const int row = p0 < 0 ? pos[t] : p0 + t;                  // cache position of token t (src/fast/fused.cu:520)
    const size_t o = kv_off_tab(pg, kv_tab(pg, t), row);
    const int nb = D / 32, blk = i >> 3, j8 = i & 7;
    auto write_head = [&](char * cache, int h, float4 x) {
        if constexpr (KT == P1A_KV_F16) {
            if (live) reinterpret_cast<h4 *>(cache + o + (size_t) h * D * 2)[i] = h4{(half_t) x.x, (half_t) x.y, (half_t) x.z, (half_t) x.w};
        } else if constexpr (KT == P1A_KV_Q8_0) {
            if (live) q8_block(x, j8, cache + o + (size_t) h * nb * 34, blk, nb);
            else xor8_max(0.f);
        } else {
            if (live) q4_block(x, j8, cache + o + ((size_t) h * nb + blk) * 18);
        }
    };
    if (b >= Hq + Hkv) {                                       // v head: the plain quantizing write
        const int h = b - Hq - Hkv;
        float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) x = reinterpret_cast<const float4 *>(v + (size_t) t * ldv + (size_t) h * D)[i];
        write_head(vc, h, x);
        return;
    }
    const bool isq = b < Hq;
    const int h = isq ? b : b - Hq;
    const float * src = isq ? qg + (size_t) t * ldq + (size_t) h * 2 * D : k + (size_t) t * ldk + (size_t) h * D;
    const float * w = isq ? qn : kn;
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) {
        a = reinterpret_cast<const float4 *>(src)[i];
        if (isq) reinterpret_cast<float4 *>(gate + ((size_t) t * Hq + h) * D)[i] = reinterpret_cast<const float4 *>(src + D)[i];
    }
    float ss = a.x * a.x;
    ss = ss + a.y * a.y;
    ss = ss + a.z * a.z;
    ss = ss + a.w * a.w;
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) ss = ss + __shfl_xor(ss, m);
    const float sc = 1.0f / sqrtf(ss / (float) D + eps);
    float x[4] = {a.x * sc, a.y * sc, a.z * sc, a.w * sc};
    if (w && live) {
        const float4 ww = reinterpret_cast<const float4 *>(w)[i];
        x[0] = x[0] * ww.x; x[1] = x[1] * ww.y; x[2] = x[2] * ww.z; x[3] = x[3] * ww.w;
    }
    // NEOX rope: dims d < n_rot / 2 pair with d + n_rot / 2, which lane i + n_rot / 8 holds in the same slot
    const int half = n_rot >> 1, hl = half >> 2;
    const bool lo = i < hl, rot = i < 2 * hl;
    const int partner = lo ? i + hl : i - hl;
    // interleaved M-RoPE (src/fast/mrope.cuh:25-33): pair j rotates by the position of the stream its sector selects
    auto pair_pos = [&](int j) {
        if (!mr.p) return pos[t];
        const int sector = j % mr.sect;
        int st;
        if (sector % 3 == 1 && sector < 3 * mr.s1) st = 1;
        else if (sector % 3 == 2 && sector < 3 * mr.s2) st = 2;
        else if (sector % 3 == 0 && sector < 3 * mr.s0) st = 0;
        else return 0;
        return mr.p[(size_t) st * mr.stride + t];
    };
    // the angle tables of the head: pair j is computed once, by lane j & 63 (slot j >> 6), and handed round by shuffle
    float tc[2] = {1.f, 1.f}, tsn[2] = {0.f, 0.f};
#pragma unroll
    for (int sl = 0; sl < 2; ++sl) {
        const int jj = i + 64 * sl;
        if (jj < half) {
            const float inv = (float) det_exp(((-2.0 * (double) jj) / (double) n_rot) * ln_base);
            const float theta = (float) pair_pos(jj) * inv;
            det_sincos((double) theta, tc[sl], tsn[sl]);
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float other = __shfl(x[e], rot ? partner : i);
        const int jj = rot ? 4 * (lo ? i : i - hl) + e : 0;
        const float c0 = __shfl(tc[0], jj & 63), c1 = __shfl(tc[1], jj & 63);
        const float s0 = __shfl(tsn[0], jj & 63), s1 = __shfl(tsn[1], jj & 63);
        if (rot) {
            const float c = jj < 64 ? c0 : c1, sn = jj < 64 ? s0 : s1;
            const float x0 = lo ? x[e] : other, x1 = lo ? other : x[e];
            const float p0_ = x0 * (lo ? c : sn), p1_ = x1 * (lo ? sn : c);
            x[e] = lo ? p0_ - p1_ : p0_ + p1_;
        }
    }
    const float4 r = make_float4(x[0], x[1], x[2], x[3]);
    if (isq) {
        if (live) reinterpret_cast<float4 *>(q + ((size_t) t * Hq + h) * D)[i] = r;
    } else {
        write_head(kc, h, r);
    }
}

}   // namespace

int launch_append(const p1a_kv & c, const float * k, const float * v, int p0, const int32_t * p0_dev,
                  const int32_t * pos_rows, int T, hipStream_t s) {
    const kv_view pg = view_of(c);
    const int n4 = c.Hkv * c.D / 4;
    const dim3 grid((n4 + 255) / 256, T);
    char * kc = (char *) c.k, * vc = (char *) c.v;
    if (c.type == P1A_KV_F16) append_k<P1A_KV_F16><<<grid, 256, 0, s>>>(k, v, kc, vc, p0, p0_dev, pos_rows, c.Hkv, c.D, pg);
    else if (c.type == P1A_KV_Q8_0) append_k<P1A_KV_Q8_0><<<grid, 256, 0, s>>>(k, v, kc, vc, p0, p0_dev, pos_rows, c.Hkv, c.D, pg);
    else append_k<P1A_KV_Q4_0><<<grid, 256, 0, s>>>(k, v, kc, vc, p0, p0_dev, pos_rows, c.Hkv, c.D, pg);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

namespace {
// Benchmark fill of positions p0 .. p1 - 1 of one sequence with hashed 16-bit words (src/fast/attn.cu:538-581): word w of
// the contiguous cache - or of the page, for a paged one, whose logical page g then adds g * 0x632be5ab to the seed - gets
// a 32-bit mix of (w, seed); f16 caches take its halves as values in [-1, 1], the quantized ones as codes, with every
// scale word set to f16(1/127) (q8_0) or f16(0.125) (q4_0). The page table is read on the device: nothing is copied back
// to the host, and the call can be captured.
__global__ void __launch_bounds__(256) fill_random_k(uint16_t * kc, uint16_t * vc, kv_view pg, uint32_t type, int D, int p0, size_t nw,
                                                     int row_words, int head_words, uint32_t seed) {
    const int32_t * ptab = pg.pt ? (pg.rtab ? pg.pt + pg.rtab[0] : pg.pt) : nullptr;
    for (size_t i = (size_t) blockIdx.x * 256 + threadIdx.x; i < nw; i += (size_t) gridDim.x * 256) {
        const int p = p0 + (int) (i / (size_t) row_words), wr = (int) (i % (size_t) row_words);
        size_t w, base = 0;                                   // word index the hash takes; where that view starts (bytes)
        uint32_t sd = seed;
        if (ptab) {
            const int g = p >> pg.psh;
            w = (size_t) (p - (g << pg.psh)) * row_words + wr;
            base = (size_t) ptab[g] * pg.pstride;
            sd = seed + (uint32_t) g * 0x632be5abu;
        } else w = (size_t) p * row_words + wr;
        uint32_t h = (uint32_t) w * 2654435761u ^ sd;
        h ^= h >> 16; h *= 0x7feb352du; h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 16;
        const int hw = wr % head_words;
        uint16_t a, b;
        if (type == P1A_KV_F16) {
            a = __builtin_bit_cast(uint16_t, (half_t) ((float) (h & 0xffffu) / 32768.0f - 1.0f));
            b = __builtin_bit_cast(uint16_t, (half_t) ((float) (h >> 16) / 32768.0f - 1.0f));
        } else if ((type == P1A_KV_Q8_0 && hw < D / 32) || (type == P1A_KV_Q4_0 && hw % 9 == 0)) {
            a = b = __builtin_bit_cast(uint16_t, (half_t) (type == P1A_KV_Q8_0 ? 1.0f / 127.0f : 0.125f));
        } else {
            a = (uint16_t) h;
            b = (uint16_t) (h >> 16);
        }
        reinterpret_cast<uint16_t *>(reinterpret_cast<char *>(kc) + base)[w] = a;
        reinterpret_cast<uint16_t *>(reinterpret_cast<char *>(vc) + base)[w] = b;
    }
}
}   // namespace

int launch_fill_random(const p1a_kv & c, int p0, int p1, uint32_t seed, hipStream_t s) {
    const size_t rowb = p1a_kv_row_bytes(c.type, c.Hkv, c.D);
    const int row_words = (int) (rowb / 2), head_words = row_words / c.Hkv;
    const size_t nw = (size_t) (p1 - p0) * row_words;
    const unsigned blocks = (unsigned) (nw / 256 + 1 < 4096 ? nw / 256 + 1 : 4096);
    fill_random_k<<<blocks, 256, 0, s>>>((uint16_t *) c.k, (uint16_t *) c.v, view_of(c), c.type, c.D, p0, nw, row_words, head_words, seed);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

namespace {
// elementwise gate + a16 quantize, one float4 per lane, 8 lanes per 32-value group (src/fast/fused.cu:478-496):
// OP 0: y = silu(a) * b (the MLP gate); OP 1: y = a * sigmoid(b) (the attention output gate). y may alias a.
template <int OP>
__global__ void __launch_bounds__(256) ew_q_k(const float * a, const float * b, float * y, void * qbuf, int n, int lda, int ldb) {
    const int n4 = n >> 2, t = blockIdx.y, T = gridDim.y;
    const int i = blockIdx.x * 256 + threadIdx.x;
    const bool act = i < n4;
    f4 o = {0.f, 0.f, 0.f, 0.f};
    if (act) {
        const f4 av = reinterpret_cast<const f4 *>(a + (size_t) t * lda)[i], bv = reinterpret_cast<const f4 *>(b + (size_t) t * ldb)[i];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = OP == 0 ? (av[e] / (1.0f + expf(-av[e]))) * bv[e] : av[e] * (1.0f / (1.0f + expf(-bv[e])));
        reinterpret_cast<f4 *>(y + (size_t) t * n)[i] = o;
    }
    a16_quant8(o, i & 7, qbuf, t, i >> 3, n >> 5, T, act);   // n % 32 == 0: dead lanes form whole groups
}
}   // namespace

int launch_ew_quant(int op, const float * a, const float * b, float * y, void * qbuf, int T, int n, int lda, int ldb, hipStream_t s) {
    const dim3 grid((n / 4 + 255) / 256, T);
    if (op == 0) ew_q_k<0><<<grid, 256, 0, s>>>(a, b, y, qbuf, n, lda, ldb);
    else ew_q_k<1><<<grid, 256, 0, s>>>(a, b, y, qbuf, n, lda, ldb);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

int launch_prep(const p1a_kv & c, const float * qg, const float * k, const float * v, const float * q_norm, const float * k_norm,
                const int32_t * pos, float * q, float * gate, int p0, int T, int Hq, int n_rot, float freq_base, float eps,
                int ldq, int ldk, int ldv, const mrope_view & mr, hipStream_t s) {
    const kv_view pg = view_of(c);
    const dim3 grid(Hq + 2 * c.Hkv, T);
    char * kc = (char *) c.k, * vc = (char *) c.v;
    const double ln_base = det_log((double) freq_base);
#define P1A_PREP(KT_) prep_k<KT_><<<grid, 64, 0, s>>>(qg, k, v, q_norm, k_norm, pos, q, gate, kc, vc, p0, Hq, c.Hkv, c.D, n_rot, \
                                                      ln_base, eps, ldq, ldk, ldv, pg, mr)
    if (c.type == P1A_KV_F16) P1A_PREP(P1A_KV_F16);
    else if (c.type == P1A_KV_Q8_0) P1A_PREP(P1A_KV_Q8_0);
    else P1A_PREP(P1A_KV_Q4_0);
#undef P1A_PREP
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

}   // namespace p1a
