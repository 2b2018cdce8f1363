// Chunked causal prefill attention over a paged f16 / q8_0 / q4_0 KV cache for gfx950 (MI355X).
//
// One workgroup (4 waves, one per SIMD, 512 registers each) owns 128 consecutive query tokens of ONE q head; wave w owns
// 32 of them as the N = 32 columns of v_mfma_f32_32x32x16_f16 tiles. Keys are walked in tiles of 64, kept in LDS as f16
// (two K and two V tiles). f16 rows of 512 bytes are moved from global memory straight into LDS
// (global_load_lds_dwordx4); everything else is fetched into registers with 16-byte loads off a wave-uniform page base,
// dequantized and stored to the same LDS places.
//   S^T = K Q^T : A = K rows straight from LDS (ds_read_b128), B = Q^T held in accumulation registers (pre-multiplied
//                 by scale * log2 e, rounded to f16). A lane then holds 16 keys of ONE query row, so the row maximum
//                 needs no cross-lane work beyond one half-wave swap.
//   O^T = V^T P^T : A = V^T read with the transposing ds_read_b64_tr_b16, B = P^T straight from the S^T registers.
//                 Waves pair up: each wave of a pair accumulates half the dims for the 64 rows of both, so a V^T
//                 fragment feeds two MFMAs; the partner's P^T comes through LDS.
// The loop is software-pipelined so that every iteration holds two independent instruction streams side by side: the
// MFMAs of S^T for tile j+1 next to exp2 / f16 conversion of tile j, then the MFMAs of O^T for tile j next to masking and
// the row maximum of tile j+1 (and the dequantization of the tiles that come after). With one wave per SIMD nothing
// else can hide one pipe behind the other.
// fp32 accumulation; the softmax denominator is a packed dot product of the rounded P with ones, so that it sums the same
// rounded P that multiplies V. The reference maximum of a row moves lazily (only when the row maximum has grown
// by more than 2^RESCALE_STEP), so the accumulators are rescaled a handful of times per row. Keys above a row's
// diagonal are masked; the sigmoid output gate is applied in the epilogue.
// Workgroup order: the q heads of one kv head, for one token block, get consecutive dispatch slots on the same XCD,
// so they stream the same K/V tiles through one L2.
#include "p1a_common.hpp"

#include <atomic>

namespace p1a {
size_t prefill_stage_bytes(int n, int Hkv, int D);
namespace {

constexpr int BM = 128;   // query tokens per workgroup
constexpr int BN = 64;    // keys per tile
constexpr int NTHR = 256;
constexpr float NEG_INF = -__builtin_inff();

template <int D> struct pf_cfg {
    static constexpr int NKS = D / 16;         // k-steps of S^T (16 dims each)
    static constexpr int NDT = D / 32;         // 32-dim tiles of O^T
};

// Where the f16 tiles sit in LDS: in blocks of two rows (2 x 2 D bytes, then padding). Block (key & 7) + 8 (key >> 4)
// holds key in its half (key >> 3) & 1 - two keys of the same 16-key group. For D = 256 a block is exactly what one
// global_load_lds_dwordx4 moves (64 lanes x 16 bytes to 1 KB of consecutive LDS), and one page base serves it; tiles
// staged through registers use the same places. The padding puts the rows that are read together into disjoint banks:
// S^T row c of half u is the key of block 16 u + (c & 15), half c >> 4 (16 consecutive lanes: 16 blocks, 4 banks
// apart); the transposing V reads take 4 consecutive blocks of one half (16 banks apart). Every read address is
// (per-lane base) + (compile-time offset).
template <int D> struct pf_lay {
    static constexpr int RB = 2 * D;                            // bytes of a row
    static constexpr int KB = 2 * RB + 16, VB = 2 * RB + 64;   // block strides
    static constexpr int KT_B = 32 * KB, VT_B = 32 * VB;
    static constexpr int STAGE_B = KT_B + VT_B;
    static __device__ __forceinline__ int key_off(int key, int bstride) { return ((key & 7) + 8 * (key >> 4)) * bstride + ((key >> 3) & 1) * RB; }
    // S^T operand rows: lane base of row c, offset of half u
    static __device__ __forceinline__ int k_lane(int c) { return (c & 15) * KB + (c >> 4) * RB; }
    static constexpr int k_half(int u) { return 16 * u * KB; }
    // which key of the tile value i of half u of a lane's S^T column is, without the lane's 4 g
    static constexpr int key_of(int u, int i) { return 32 * u + 16 * ((i >> 2) & 1) + 8 * (i >> 3) + (i & 3); }
    // V^T operand of k-step ps: rows r = 4 g + kk (lane part), then the step's two row groups:
    // keys 32 (ps / 2) + 8 (ps % 2) + r and the same + 16
    static __device__ __forceinline__ int v_lane(int r) { return r * VB; }
    static constexpr int v_lo(int ps) { return 16 * (ps >> 1) * VB + (ps & 1) * RB; }
    static constexpr int v_hi(int ps) { return v_lo(ps) + 8 * VB; }
};


struct pf_params {
    const float * q;
    float * out;
    const float * gate;
    const char * kc;
    const char * vc;
    kv_view pg;
    int T, p0, Hq, Hkv, GQA;
    int n_rows;   // positions the cache holds (contiguous caches: rows that may be read)
    float qscale;
    int nblk;     // token blocks
    // key splits: with nks > 1 workgroup (block, head, ks) walks its share of the block's tiles and leaves an unnormalised
    // partial (O relative to m, and (m, l)) per row in part_o [T*Hq][nks][D] / part_ml [T*Hq][nks][2] for the merge
    int nks;
    float * part_o;
    float * part_ml;
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

constexpr float RESCALE_STEP = 8.0f;   // log2 units: the reference maximum of a row only moves in steps larger than this

// ---- per-type staging: raw tile of one kv head -> registers -> f16 rows in LDS ----
// Every thread owns a fixed set of items (key, chunk) of the tile: item x of thread tid is i = x * NTHR + tid,
// key = i / CPK, chunk = i % CPK. `raw` keeps what was loaded for them. A load names its address as
// gb[x] + vo[x][n]: gb = cache base + the base of the item's 16-key group (wave-uniform whenever 16 * CPK is a multiple
// of the wave size, so it sits in scalar registers), vo = the loop-invariant 32-bit offset of the item inside its group
// (row in the group * row bytes + offs()[n]); the loads then need no address arithmetic at all.
typedef unsigned u2v __attribute__((ext_vector_type(2)));
typedef float f2v __attribute__((ext_vector_type(2)));
typedef uint32_t __attribute__((may_alias)) u32a;   // the parked scale blocks are written as dwords and read as halves
typedef uint16_t __attribute__((may_alias)) u16a;
typedef const __attribute__((address_space(1))) char * gptr;      // global memory, so the loads are global_load (vmcnt only)
#define P1A_GLOAD(T, p) (*(const __attribute__((address_space(1))) T *) (p))
template <uint32_t KT, int D> struct stager;
// Which (key, chunk) of the 64-key tile item x of thread tid is. Wave-major whenever the chunks of a key divide a wave
// evenly: wave w owns keys 16 w .. 16 w + 15 - exactly one 16-key group, so one page base serves all its loads - and
// item x covers KPW = 64 / CPK of them. (Otherwise: items dealt out thread by thread over the whole tile.)
template <int CPK> struct item_map {
    static constexpr bool WAVE_MAJOR = CPK % 4 == 0 && CPK <= 64;
    static constexpr int KPW = WAVE_MAJOR ? 64 / CPK : 1;
    static __device__ __forceinline__ int key(int x, int tid) { return WAVE_MAJOR ? 16 * (tid >> 6) + x * KPW + (tid & 63) / CPK : (x * NTHR + tid) / CPK; }
    static __device__ __forceinline__ int cc(int x, int tid) { return WAVE_MAJOR ? (tid & 63) % CPK : (x * NTHR + tid) % CPK; }
};

template <int D> struct stager<P1A_KV_Q8_0, D> {
    static constexpr int CPK = D / 16;                    // 16-code chunks per key
    static constexpr int NPT = BN * CPK / NTHR;           // items per thread
    static constexpr int NOFF = 1;                        // codes
    // Sub-dword loads cost twice the issue time of a 16-byte one, so an item does not fetch its own f16 scale: each wave
    // fetches the scale blocks (D/32 scales) of the 16 keys its items belong to with ONE load per tile, parks them in a
    // small LDS area of its own and every lane picks its scales up from there.
    static constexpr bool SCALES_VIA_LDS = true;
    static constexpr int SB = (D / 32) * 2;               // bytes of scales per key head
    static_assert(BN * CPK % NTHR == 0, "tile must split evenly over the threads");
    struct raw { u4 w[NPT]; uint32_t d[NPT]; };           // d: one zero-extended f16 scale per item
    static __device__ __forceinline__ void offs(uint32_t * o, int cc) { o[0] = (D / 32) * 2 + cc * 16; }
    static __device__ __forceinline__ void load_item(raw & r, gptr gb, const uint32_t * vo, int x, int) {
        r.w[x] = P1A_GLOAD(u4, gb + vo[0]);
    }
    static constexpr int PARTS = 2;                       // 16-byte LDS stores per item
    static __device__ __forceinline__ void store_part(const raw & r, char * tile, int stride, int tid, int x, int part) {
        const int key = item_map<CPK>::key(x, tid), cc = item_map<CPK>::cc(x, tid);
        const uint32_t d16 = r.d[x];
        const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
        const pair32 x0 = deq8x4(r.w[x][2 * part], dd), x1 = deq8x4(r.w[x][2 * part + 1], dd);
        *reinterpret_cast<u4 *>(tile + pf_lay<D>::key_off(key, stride) + cc * 32 + part * 16) = u4{x0.lo, x0.hi, x1.lo, x1.hi};
    }
};

template <int D> struct stager<P1A_KV_F16, D> {
    static constexpr int CPK = D / 8;                     // 16-byte chunks (8 halves) per key
    static constexpr int NPT = BN * CPK / NTHR;
    static constexpr int NOFF = 1;
    static constexpr bool SCALES_VIA_LDS = false;
    static constexpr int SB = 4;
    static_assert(BN * CPK % NTHR == 0, "tile must split evenly over the threads");
    struct raw { u4 w[NPT]; };
    static __device__ __forceinline__ void offs(uint32_t * o, int cc) { o[0] = cc * 16; }
    static __device__ __forceinline__ void load_item(raw & r, gptr gb, const uint32_t * vo, int x, int) {
        r.w[x] = P1A_GLOAD(u4, gb + vo[0]);
    }
    static constexpr int PARTS = 1;
    static __device__ __forceinline__ void store_part(const raw & r, char * tile, int stride, int tid, int x, int) {
        const int key = item_map<CPK>::key(x, tid), cc = item_map<CPK>::cc(x, tid);
        *reinterpret_cast<u4 *>(tile + pf_lay<D>::key_off(key, stride) + cc * 16) = r.w[x];
    }
};

template <int D> struct stager<P1A_KV_Q4_0, D> {
    static constexpr int CPK = D / 32;                    // 18-byte blocks per key: one block (32 values) per item
    static constexpr int NPT = (BN * CPK + NTHR - 1) / NTHR;
    static constexpr int NOFF = 1;
    static constexpr bool SCALES_VIA_LDS = false;
    static constexpr int SB = 4;
    struct raw { uint16_t h[NPT][9]; };
    static __device__ __forceinline__ void offs(uint32_t * o, int cc) { o[0] = cc * 18; }
    static __device__ __forceinline__ void load_item(raw & r, gptr gb, const uint32_t * vo, int x, int tid) {
        const int key = item_map<CPK>::key(x, tid);
        if (BN * CPK % NTHR == 0 || key < BN) {
            const gptr blk = gb + vo[0];   // 2-byte aligned
#pragma unroll
            for (int k = 0; k < 9; ++k) r.h[x][k] = P1A_GLOAD(uint16_t, blk + 2 * k);
        }
    }
    static constexpr int PARTS = 4;                       // part 0, 1: values 0..15 (low nibbles), part 2, 3: values 16..31
    static __device__ __forceinline__ void store_part(const raw & r, char * tile, int stride, int tid, int x, int part) {
        const int key = item_map<CPK>::key(x, tid), b = item_map<CPK>::cc(x, tid);
        if (!(BN * CPK % NTHR == 0 || key < BN)) return;
        const uint32_t d16 = r.h[x][0];
        const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
        // byte j of the block: low nibble = value j, high nibble = value j + 16; this part covers bytes 8 (part & 1) .. + 7
        pair32 q[2];
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int kb = 2 * (part & 1) + k;
            const uint32_t w = (uint32_t) r.h[x][1 + 2 * kb] | ((uint32_t) r.h[x][2 + 2 * kb] << 16);   // bytes 4 kb .. 4 kb + 3
            q[k] = deq4x4((part & 2 ? w >> 4 : w) & 0x0f0f0f0fu, dd);
        }
        *reinterpret_cast<u4 *>(tile + pf_lay<D>::key_off(key, stride) + b * 64 + part * 16) = u4{q[0].lo, q[0].hi, q[1].lo, q[1].hi};
    }
};

// whole-tile store (prologue): every part of every item
template <class S> __device__ __forceinline__ void store_tile(const typename S::raw & r, char * tile, int stride, int tid) {
#pragma unroll
    for (int x = 0; x < S::NPT; ++x)
#pragma unroll
        for (int part = 0; part < S::PARTS; ++part) S::store_part(r, tile, stride, tid, x, part);
}

// GROUPED: pages hold at least 16 positions (or the cache is contiguous), so a 16-key group has one base
__device__ __forceinline__ uint32_t lds_addr(const char * p) { return (uint32_t) (size_t) (const __attribute__((address_space(3))) char *) p; }
// 64 lanes x 16 bytes, global (scalar base + 32-bit lane offset) -> LDS at `lds` + 16 * lane, no registers in between
__device__ __forceinline__ void dma16(const char * sbase, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(voff), "s"(sbase), "s"(lds) : "memory", "m0");
}

template <uint32_t KT, int D, bool GROUPED, bool DMA>
__global__ void __launch_bounds__(NTHR, 1) prefill_k(const pf_params P) {
    static_assert(!DMA || (KT == P1A_KV_F16 && GROUPED && D == 256), "the LDS-direct loads are laid out for f16 rows of 512 bytes");
    using C = pf_cfg<D>;
    using L = pf_lay<D>;
    using S = stager<KT, D>;
    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 31, g = lane >> 5;
    // blockIdx.x -> (token block, kv head, q head of the group): the GQA heads of one (block, kv head) share an XCD
    const int id = blockIdx.x, xcd = id & 7, slot = id >> 3;
    // (with key splits a unit is (key split, token block, kv head): the splits spread over the XCDs like the blocks do)
    const int vunit = (slot / P.GQA) * 8 + xcd, hh = slot % P.GQA;
    const int nunits = P.nblk * P.Hkv;
    if (vunit >= nunits * P.nks) return;
    const int ksp = vunit / nunits, unit = vunit - ksp * nunits;
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
    const int ntiles_all = pmax / BN + 1;                     // tiles the block sees
    // this workgroup's share of them: tiles tile_a .. tile_a + ntiles - 1
    int tile_a = 0, ntiles = ntiles_all;
    if (P.nks > 1) {
        const int tps = (ntiles_all + P.nks - 1) / P.nks;
        tile_a = ksp * tps;
        ntiles = min(tps, ntiles_all - tile_a);
        if (ntiles <= 0) {   // nothing left for this split: an empty partial (the merge skips it)
            if (g == 0 && live) {
                float * ml = P.part_ml + (((size_t) my_tok * P.Hq + h) * P.nks + ksp) * 2;
                ml[0] = NEG_INF;
                ml[1] = 0.f;
            }
            return;
        }
    }

    const int32_t * ptab = P.pg.pt ? (P.pg.rtab ? P.pg.pt + P.pg.rtab[0] : P.pg.pt) : nullptr;
    const size_t hb = KT == P1A_KV_F16 ? (size_t) D * 2 : KT == P1A_KV_Q8_0 ? (size_t) (D / 32) * 34 : (size_t) (D / 32) * 18;
    const size_t head_off = (size_t) hk * hb;

    // ---- Q^T operands (B: k = 16 dims per step, n = query row): lane (row c, half g) holds dims 16 ks + 8 g .. + 7 ----
    h8 qf[C::NKS];
    // (all the loads first, then the conversions: a load that is waited for before the next one is asked for costs a
    // memory round trip each - 16 of them in a row were most of what a workgroup spent outside its key loop. With
    // LDS-direct tiles the rows are asked for right behind the first tiles (the compiler drains its own loads in front of
    // hand-issued ones, so asking earlier would put the two latencies in a row): one latency, not two.)
    auto load_q = [&]() {
        float4 qa[C::NKS], qb[C::NKS];
        const float * qr = P.q + ((size_t) (live ? my_tok : 0) * P.Hq + h) * D;
#pragma unroll
        for (int ks = 0; ks < C::NKS; ++ks) {
            qa[ks] = make_float4(0.f, 0.f, 0.f, 0.f);
            qb[ks] = qa[ks];
            if (live) { qa[ks] = *reinterpret_cast<const float4 *>(qr + 16 * ks + 8 * g); qb[ks] = *reinterpret_cast<const float4 *>(qr + 16 * ks + 8 * g + 4); }
        }
#pragma unroll
        for (int ks = 0; ks < C::NKS; ++ks) {
            const float4 a = qa[ks], b = qb[ks];
            const float s = P.qscale;
            qf[ks] = h8{(half_t) (a.x * s), (half_t) (a.y * s), (half_t) (a.z * s), (half_t) (a.w * s),
                        (half_t) (b.x * s), (half_t) (b.y * s), (half_t) (b.z * s), (half_t) (b.w * s)};
            // Q stays in accumulation registers for the whole kernel: the matrix instructions read them in place, and
            // the vector registers are left to the tiles in flight
            asm volatile("" : "+a"(qf[ks]));
        }
    };
    if constexpr (!DMA) load_q();

    // Waves pair up for O^T: the pair (w, w ^ 1) shares its 64 query rows, each wave accumulating HALF the dims
    // (tiles HD * (w & 1) ..) for ALL 64 rows: a V^T fragment read from LDS then feeds two MFMAs (own rows, partner's
    // rows) instead of one, which halves the transposing reads - the slowest LDS traffic of the kernel. The price is
    // that P^T (and the rare rescale factors) of the partner come through LDS, behind one more barrier per tile.
    constexpr int HD = C::NDT / 2;                            // dim tiles per wave
    static_assert(C::NDT % 2 == 0, "the dims split over a pair of waves");
    const int dh = wave & 1;                                  // which half of the dims
    f16x o[2][HD];                                            // [0]: own rows, [1]: the partner's rows
    // softmax denominator of the own rows: this lane's share, per key half of a tile - the sum of the ROUNDED P values
    // (a packed dot product with ones, fp32 accumulation: v_dot2 keeps f16 denormals), so that it matches what
    // multiplies V. 16 vector instructions in the shadow of the S^T products instead of four more matrix instructions
    // per tile (-1.3 % of the call). Kept per (key half, lane half) and added up once, in a fixed order, at the end.
    float lp[2] = {0.f, 0.f};
    float m_run = NEG_INF;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
#pragma unroll
        for (int dt = 0; dt < HD; ++dt) { o[0][dt][i] = 0.f; o[1][dt][i] = 0.f; }
    }
    // exchange areas behind the tile stages: P^T of every wave (BN / 16 k-steps x 64 lanes x 16 bytes), then one float
    // per query row (rescale factor during the loop, denominator at the end)
    char * const xbase = lds + 2 * L::STAGE_B + (S::SCALES_VIA_LDS ? 2 * 4 * 16 * S::SB : 0);
    constexpr int PX_B = (BN / 16) * 64 * 16;
    char * const px_own = xbase + wave * PX_B, * const px_par = xbase + (wave ^ 1) * PX_B;
    float * const ax_own = reinterpret_cast<float *>(xbase + 4 * PX_B) + wave * 32;
    float * const ax_par = reinterpret_cast<float *>(xbase + 4 * PX_B) + (wave ^ 1) * 32;
    const h2 one2 = {(half_t) 1, (half_t) 1};

    // ---- addressing of the raw tile ----
    // A tile is four groups of 16 keys, one per wave. With pages of >= 16 positions (or a contiguous cache) a group lies
    // in one page, so its base is a scalar: one page-table entry per wave and tile, fetched with a hand-issued scalar
    // load (s_load_dword does not share the in-order vector-memory counter with the tile loads in flight) well before the
    // base is formed. Inside the group an item sits at a loop-invariant offset; only the tile that holds pmax clamps the
    // rows past it (they would otherwise read rows nobody has written); that tile's offsets are prepared once, up front.
    constexpr bool grouped = GROUPED;
    const int pmask = (1 << P.pg.psh) - 1;
    const int last_tile = ntiles_all - 1;                     // the tile that holds pmax
    using IM = item_map<S::CPK>;
    uint32_t voff[S::NPT][S::NOFF], voff_last[S::NPT][S::NOFF];
    int grp[S::NPT];                                             // (wave-major: all equal to the wave number)
#pragma unroll
    for (int x = 0; x < S::NPT; ++x) {
        const int key = min(IM::key(x, tid), BN - 1), cc = IM::cc(x, tid);
        grp[x] = key >> 4;
        uint32_t co[S::NOFF];
        S::offs(co, cc);
        const int room = pmax - (last_tile * BN + 16 * grp[x]);         // keys of the group before pmax (< 0: none)
        const int kl = min(key & 15, max(room, 0));
#pragma unroll
        for (int n = 0; n < S::NOFF; ++n) {
            voff[x][n] = (uint32_t) (key & 15) * (uint32_t) P.pg.rowb + co[n];
            voff_last[x][n] = (uint32_t) kl * (uint32_t) P.pg.rowb + co[n];
        }
    }
    // FAST: the wave's 16 keys of a tile lie in one page (or the cache is contiguous): one table entry, one scalar base
    constexpr bool FAST = GROUPED && IM::WAVE_MAJOR;
    struct gpages { int pg; };
    struct gbases { size_t go; };
    // a group past the last position takes the base of the last one that holds a position: the LDS-direct loads then
    // fetch that group's 16 rows (all inside its page) instead of clamping row by row
    const int gclamp = DMA ? (pmax & ~15) : pmax;
    auto group_pages = [&](int tile) {
        gpages r;
        r.pg = 0;
        if (FAST && ptab) {
            // (a load from the constant address space at a wave-uniform address is an s_load_dword whose wait the compiler
            // places itself, before the first use; the table does not change while the kernel runs)
            const int32_t * e = ptab + (__builtin_amdgcn_readfirstlane(min(tile * BN + 16 * wave, gclamp)) >> P.pg.psh);
            const size_t eu = (size_t) e;
            const uint32_t elo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) eu);
            const uint32_t ehi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (eu >> 32));
            r.pg = *reinterpret_cast<const __attribute__((address_space(4))) int32_t *>(((size_t) ehi << 32) | elo);
        }
        return r;
    };
    auto group_bases = [&](int tile, gpages & gp) {
        gbases r;
        const int p = __builtin_amdgcn_readfirstlane(min(tile * BN + 16 * wave, gclamp));
        r.go = (ptab ? (size_t) gp.pg * P.pg.pstride + (size_t) (p & pmask) * P.pg.rowb : (size_t) p * P.pg.rowb) + head_off;
        return r;
    };
    // where item x of `tile` starts: base (scalar registers when GROUPED) + 32-bit offsets
    struct iaddr { gptr base; uint32_t vo[S::NOFF]; };
    auto item_addr = [&](const char * cache, int tile, const gbases & gb, int x) {
        iaddr r;
        if constexpr (FAST) {
            r.base = (gptr) cache + gb.go;
            const bool is_last = tile == last_tile;
#pragma unroll
            for (int n = 0; n < S::NOFF; ++n) r.vo[n] = is_last ? voff_last[x][n] : voff[x][n];
        } else {   // pages shorter than a group (or items not dealt out wave by wave): every key looks its page up
            const int key = min(IM::key(x, tid), BN - 1);
            r.base = (gptr) cache + (kv_off_tab(P.pg, ptab, min(tile * BN + key, pmax)) + head_off);
#pragma unroll
            for (int n = 0; n < S::NOFF; ++n) r.vo[n] = voff[x][n] - (uint32_t) (key & 15) * (uint32_t) P.pg.rowb;
        }
        return r;
    };
    auto load_tile = [&](typename S::raw & r, const char * cache, int tile, const gbases & gb) {
#pragma unroll
        for (int x = 0; x < S::NPT; ++x) {
            const iaddr ia = item_addr(cache, tile, gb, x);
            S::load_item(r, ia.base, ia.vo, x, tid);
        }
    };

    // ---- scale blocks (types that keep their scales apart from the codes) ----
    // Lane l of a wave (l mod 16) fetches the block of the l-th of the wave's 16 keys; all four quarters of the wave fetch
    // and park the same 16 blocks, which saves masking lanes off.
    constexpr bool SVL = S::SCALES_VIA_LDS;
    static_assert(!SVL || IM::WAVE_MAJOR, "parked scale blocks are per wave");
    constexpr int KPW = IM::KPW;
    struct sblk { uint32_t w[S::SB / 4]; };
    const int l16 = lane & 15;
    const int lkey = 16 * wave + l16;
    const uint32_t sb_full = (uint32_t) l16 * (uint32_t) P.pg.rowb;
    const uint32_t sb_last = (uint32_t) min(l16, max(pmax - (last_tile * BN + 16 * wave), 0)) * (uint32_t) P.pg.rowb;
    char * const ksc = lds + 2 * L::STAGE_B + wave * 16 * S::SB;           // this wave's parking area: K blocks
    char * const vsc = ksc + 4 * 16 * S::SB;                               // ... V blocks
    auto load_sblk = [&](const char * cache, int tile, const gbases & gb) {
        sblk r;
        size_t off;
        if constexpr (FAST) {
            off = gb.go + (tile == last_tile ? sb_last : sb_full);
        } else {
            off = kv_off_tab(P.pg, ptab, min(tile * BN + lkey, pmax)) + head_off;
        }
        const gptr p_ = (gptr) cache + off;
        if constexpr (S::SB == 16) { const u4 t = P1A_GLOAD(u4, p_); r.w[0] = t[0]; r.w[1] = t[1]; r.w[2] = t[2]; r.w[3] = t[3]; }
        else if constexpr (S::SB == 8) { const u2v t = P1A_GLOAD(u2v, p_); r.w[0] = t[0]; r.w[1] = t[1]; }
        else r.w[0] = P1A_GLOAD(uint32_t, p_);
        return r;
    };
    auto park_sblk = [&](char * area, const sblk & b) {
#pragma unroll
        for (int j = 0; j < S::SB / 4; ++j) reinterpret_cast<u32a *>(area + l16 * S::SB)[j] = b.w[j];
    };
    auto pick_scales = [&](typename S::raw & r, const char * area) {
        if constexpr (SVL) {
#pragma unroll
            for (int x = 0; x < S::NPT; ++x)
                r.d[x] = *reinterpret_cast<const u16a *>(area + (x * KPW + lane / S::CPK) * S::SB + ((lane % S::CPK) >> 1) * 2);
        }
    };
    // prologue helper: a whole raw tile, scales included
    auto fetch_tile = [&](typename S::raw & r, const char * cache, char * area, int tile, const gbases & gb) {
        load_tile(r, cache, tile, gb);
        if constexpr (SVL) {
            const sblk b = load_sblk(cache, tile, gb);
            park_sblk(area, b);
            pick_scales(r, area);
        }
    };

    // Workgroups that share a kv head would otherwise walk the keys in lock-step and ask one L2 channel for the same
    // line at the same instant. Each starts at its own tile and wraps around (softmax does not care about key order);
    // the q heads of one group stay one tile apart, so all but the first still find the tile in L2.
    // Steps past the last one (the pipeline looks up to three tiles ahead) repeat the last tile; nothing uses them.
    const int rot = (int) (((unsigned) unit * 29u + (unsigned) hh) % (unsigned) ntiles);
    auto tile_of = [&](int it) { const int t = min(it, ntiles - 1) + rot; return tile_a + (t >= ntiles ? t - ntiles : t); };

    // S^T of one tile: 32-key halves u = 0, 1
    auto qk = [&](const char * kt, f16x (&s)[2]) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s[u][i] = 0.f;
            const char * krow = kt + L::k_lane(c) + L::k_half(u) + g * 16;
#pragma unroll
            for (int ks = 0; ks < C::NKS; ++ks) {
                const h8 a = *reinterpret_cast<const h8 *>(krow + ks * 32);
                s[u] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[ks], s[u], 0, 0, 0);
            }
        }
    };

    // ---- LDS-direct tile loads (DMA): wave w moves the 8 blocks of its 16-key group; instruction j takes keys j and
    // j + 8 of the group (lanes 0-31 / 32-63, 16 bytes of the row each): a scalar base that advances by one row per
    // instruction and ONE loop-invariant lane offset. Rows past the last position are fetched as they are (the group lies
    // inside one page, or inside the cache when it is contiguous - the host checks): as K they only make scores that the
    // mask replaces; as V they are overwritten with zeros in LDS once the tile has landed (P = 0 times anything finite).
    const uint32_t dma_vo = (uint32_t) (8 * g) * (uint32_t) P.pg.rowb + (uint32_t) (lane & 31) * 16u;
    auto dma_block = [&](const char * cache, const gbases & gb, char * dst_tile, int bstride, int j) {
        dma16(cache + gb.go + (size_t) j * P.pg.rowb, dma_vo, lds_addr(dst_tile + (8 * wave + j) * bstride));
    };
    auto zero_v_tail = [&](int tile, char * vtile) {
        if (tile != last_tile) return;
        const int room = pmax - (last_tile * BN + 16 * wave);             // the wave's last key that exists (< 0: none)
        for (int kg = max(room + 1, 0); kg < 16; ++kg)
            *reinterpret_cast<u2v *>(vtile + L::key_off(16 * wave + kg, L::VB) + lane * 8) = u2v{0u, 0u};
    };

    // ---- prologue: K(0), V(0), K(1) in LDS; (staged through registers: V(1) and K(2) on their way); S^T(0) ----
    typename S::raw rk, rv;
    sblk sk, sv;                                           // scale blocks that belong to rk, rv
    gbases gb_prev;                                        // group bases of the tile whose V is fetched next
    gpages gp_ahead;                                       // (DMA) table entry of the K tile fetched in the next step
    if constexpr (DMA) {
        gpages g0 = group_pages(tile_of(0)), g1 = group_pages(tile_of(1));
        const gbases b0 = group_bases(tile_of(0), g0);
        gb_prev = group_bases(tile_of(1), g1);
        gp_ahead = group_pages(tile_of(2));
#pragma unroll
        for (int j = 0; j < 8; ++j) dma_block(P.kc, b0, lds, L::KB, j);
#pragma unroll
        for (int j = 0; j < 8; ++j) dma_block(P.vc, b0, lds + L::KT_B, L::VB, j);
#pragma unroll
        for (int j = 0; j < 8; ++j) dma_block(P.kc, gb_prev, lds + L::STAGE_B, L::KB, j);
        load_q();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        zero_v_tail(tile_of(0), lds + L::KT_B);
    } else {
        gpages g0 = group_pages(tile_of(0)), g1 = group_pages(tile_of(1)), g2 = group_pages(tile_of(2));
        const gbases b0 = group_bases(tile_of(0), g0), b1 = group_bases(tile_of(1), g1);
        gb_prev = group_bases(tile_of(2), g2);
        fetch_tile(rk, P.kc, ksc, tile_of(0), b0);
        fetch_tile(rv, P.vc, vsc, tile_of(0), b0);
        store_tile<S>(rk, lds, L::KB, tid);
        store_tile<S>(rv, lds + L::KT_B, L::VB, tid);
        fetch_tile(rk, P.kc, ksc, tile_of(1), b1);
        store_tile<S>(rk, lds + L::STAGE_B, L::KB, tid);
        load_tile(rv, P.vc, tile_of(1), b1);
        load_tile(rk, P.kc, tile_of(2), gb_prev);
        if constexpr (SVL) { sv = load_sblk(P.vc, tile_of(1), b1); sk = load_sblk(P.kc, tile_of(2), gb_prev); }
    }
    __syncthreads();
    f16x s_next[2];
    qk(lds, s_next);
    // Masking and the row maximum of a tile are done one step ahead of its softmax (in the shadow of the O^T products of
    // the tile before it): value i of half u of a lane's S^T column is key k0 + key_of(u, i) + 4 g of the lane's own row.
    auto mask_max = [&](f16x (&sv_)[2], int k0_, int idx, float m) {
        const int su = idx >> 4, i = idx & 15;
        sv_[su][i] = L::key_of(su, i) <= my_pos - k0_ - 4 * g ? sv_[su][i] : NEG_INF;
        return fmaxf(m, sv_[su][i]);
    };
    // both lane halves of a row -> the row's maximum
    auto row_max = [&](float m) { return max_swap32(m); };
    float mloc = NEG_INF;
#pragma unroll
    for (int idx = 0; idx < 32; ++idx) mloc = mask_max(s_next, tile_of(0) * BN, idx, mloc);
    mloc = row_max(mloc);
    // (the first step overwrites K(0) while it runs; every wave has to be done reading it)
    if constexpr (DMA) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    for (int it = 0; it < ntiles; ++it) {
        const int k0 = tile_of(it) * BN;
        char * const st_cur = lds + (it & 1) * L::STAGE_B;             // holds K(it) (done with) and V(it)
        char * const st_nxt = lds + ((it + 1) & 1) * L::STAGE_B;       // holds K(it+1); V(it-1) is done with
        gpages gp_k;
        gbases gb_dma;
        if constexpr (DMA) {
            gb_dma = group_bases(tile_of(it + 2), gp_ahead);           // K(it+2) goes over K(it), V(it+1) over V(it-1):
            gp_ahead = group_pages(tile_of(it + 3));                   // requested between the S^T steps below
        } else gp_k = group_pages(tile_of(it + 3));                    // entries for the K fetch at the end of this step
        f16x s[2] = {s_next[0], s_next[1]};                            // S^T(it), masked; mloc = its row maximum

        // Lazy reference maximum: m_run follows the row maximum only when it has grown by more than RESCALE_STEP, so P
        // stays below 2^RESCALE_STEP (well inside f16) and the accumulators are rescaled a handful of times per row
        // instead of at every tile. A row that has seen no visible key yet (m_run = -inf) just adopts the maximum.
        const bool fresh = m_run == NEG_INF;
        const bool move = mloc > m_run + RESCALE_STEP || fresh;      // mloc = -inf never moves anything
        const float mnew = (move && mloc != NEG_INF) ? mloc : m_run;
        const bool dead = mnew == NEG_INF;
        const float alpha = (fresh || mnew == m_run) ? 1.0f : __builtin_amdgcn_exp2f(m_run - mnew);
        m_run = mnew;
        const float msub = dead ? 0.0f : mnew;                       // a row with no visible key yet: exp2(-inf - 0) = 0
        lp[0] *= alpha;
        lp[1] *= alpha;
        if (__builtin_expect(__any(alpha != 1.0f), 0)) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
#pragma unroll
                for (int dt = 0; dt < HD; ++dt) o[0][dt][i] *= alpha;
            }
        }
        // ---- stream 1: S^T(it+1) on the matrix pipe; stream 2: P^T(it) = exp2(S^T(it) - m) on the vector pipe ----
        // Written step by step, one MFMA per step, with a scheduling fence after each: the LDS read of the K fragment
        // PF_K steps ahead, the MFMA, and a slice of the softmax that fits in the MFMA's shadow.
        h8 pb[BN / 16];
        constexpr int NQK = 2 * C::NKS, VPS = 32 / NQK, PF_K = 4;
        static_assert(32 % NQK == 0 && (VPS == 1 || VPS % 2 == 0), "softmax slices must tile the 32 values of a lane");
        const char * krow = st_nxt + L::k_lane(c) + g * 16;
        auto kfrag = [&](int k) { return *reinterpret_cast<const h8 *>(krow + L::k_half(k / C::NKS) + (k % C::NKS) * 32); };
        h8 fr[NQK];
#pragma unroll
        for (int k = 0; k < PF_K; ++k) fr[k] = kfrag(k);
#pragma unroll
        for (int k = 0; k < NQK; ++k) {
            if (k + PF_K < NQK) fr[k + PF_K] = kfrag(k + PF_K);
            if constexpr (DMA) {   // one tile load every other step: K(it+2) first (it is needed first), then V(it+1)
                if (k % 2 == 0) {
                    const int j = k / 2;
                    if (j < 8) dma_block(P.kc, gb_dma, st_cur, L::KB, j);
                    else if (j < 16) dma_block(P.vc, gb_prev, st_nxt + L::KT_B, L::VB, j - 8);
                }
            }
            const int u = k / C::NKS;
            if (k % C::NKS == 0) {
#pragma unroll
                for (int i = 0; i < 16; ++i) s_next[u][i] = 0.f;
            }
            s_next[u] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fr[k], qf[k % C::NKS], s_next[u], 0, 0, 0);
            if constexpr (SVL) {   // the scales of the raw tiles fetched one step ago: through LDS to the lanes that use them
                if (k == NQK - 4) { park_sblk(ksc, sk); park_sblk(vsc, sv); }
                if (k == NQK - 2) { pick_scales(rk, ksc); pick_scales(rv, vsc); }
            }
#pragma unroll
            for (int v = 0; v < VPS; ++v) {
                const int idx = k * VPS + v, su = idx >> 4, i = idx & 15;
                s[su][i] = __builtin_amdgcn_exp2f(s[su][i] - msub);
                if (idx & 1) {   // packed conversion (round to nearest even), two values per instruction
                    const h2 pr = __builtin_convertvector(f2v{s[su][i - 1], s[su][i]}, h2);
                    lp[su] = __builtin_amdgcn_fdot2(pr, one2, lp[su], false);
                    pb[idx >> 3][(idx & 7) - 1] = pr[0];
                    pb[idx >> 3][idx & 7] = pr[1];
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- O^T += V^T(it) P^T: set-up. V(it) has been in LDS since the last barrier, so its first fragments are asked
        // for ahead of the exchange: their latency hides behind it ----
        // Slot e of lane half g in k-step ps is key 32 (ps / 2) + 8 (ps % 2) + 4 g + e (e < 4), or that + 16 for e - 4
        const int i16 = lane & 15, blk = lane >> 4;        // 16-lane block: dims 16 (blk & 1) .., lane half blk >> 1 == g
        const int kk = i16 >> 2, jq = i16 & 3;
        const char * vbase = st_cur + L::KT_B + L::v_lane(4 * g + kk) + (16 * (blk & 1) + 4 * jq) * 2 + dh * HD * 64;
        // per k-step: HD fragments of V^T, each multiplied with the own and the partner's P^T, then the denominator
        constexpr int NFR = (BN / 16) * HD, PF_V = 3;
        constexpr int NP = 2 * S::NPT * S::PARTS;                             // store parts: K items, then V items
        struct vfrag { s4 lo, hi; };
        auto vread = [&](int f) {
            const char * p0_ = vbase + (f % HD) * 64;
            return vfrag{__builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *) (p0_ + L::v_lo(f / HD))),
                         __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *) (p0_ + L::v_hi(f / HD)))};
        };
        vfrag vf[NFR];
#pragma unroll
        for (int f = 0; f < PF_V && f < NFR; ++f) vf[f] = vread(f);
        // ---- hand P^T and the rescale factor of the own rows to the partner ----
#pragma unroll
        for (int ps = 0; ps < BN / 16; ++ps) *reinterpret_cast<h8 *>(px_own + (ps * 64 + lane) * 16) = pb[ps];
        if (g == 0) ax_own[c] = alpha;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        // ---- stream 1: O^T += V^T(it) P^T on the matrix pipe; stream 2: masking and row maximum of S^T(it+1) (and K(it+2),
        // V(it+1) -> f16 tiles in LDS when they are staged through registers) ----
        {
            const float alpha_p = ax_par[c];                                      // (needed before the partner's first product)
            h8 pp[BN / 16];
            constexpr int MPS = 32 / NFR;                                          // next tile's values masked per step
            static_assert(32 % NFR == 0, "mask slices must tile the 32 values of a lane");
            const int k0n = tile_of(it + 1) * BN;
            mloc = NEG_INF;
            pp[0] = *reinterpret_cast<const h8 *>(px_par + lane * 16);
#pragma unroll
            for (int f = 0; f < NFR; ++f) {
                if (f + PF_V < NFR) vf[f + PF_V] = vread(f + PF_V);
                const int ps = f / HD, dt = f % HD;
                if (dt == 0 && ps + 1 < BN / 16) pp[ps + 1] = *reinterpret_cast<const h8 *>(px_par + ((ps + 1) * 64 + lane) * 16);
                const h4 l4 = __builtin_bit_cast(h4, vf[f].lo), h4_ = __builtin_bit_cast(h4, vf[f].hi);
                const h8 a = {l4[0], l4[1], l4[2], l4[3], h4_[0], h4_[1], h4_[2], h4_[3]};
                o[0][dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb[ps], o[0][dt], 0, 0, 0);
                if (f == 0 && __builtin_expect(__any(alpha_p != 1.0f), 0)) {       // the partner's rows moved their reference maximum
#pragma unroll
                    for (int i = 0; i < 16; ++i)
#pragma unroll
                        for (int d2 = 0; d2 < HD; ++d2) o[1][d2][i] *= alpha_p;
                }
                o[1][dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pp[ps], o[1][dt], 0, 0, 0);
#pragma unroll
                for (int v = 0; v < MPS; ++v) mloc = mask_max(s_next, k0n, f * MPS + v, mloc);
#pragma unroll
                for (int pt = DMA ? NP : f * NP / NFR; pt < (f + 1) * NP / NFR; ++pt) {
                    const int item = pt / S::PARTS, part = pt % S::PARTS;
                    if (item < S::NPT) S::store_part(rk, st_cur, L::KB, tid, item, part);                          // K(it+2) over K(it)
                    else               S::store_part(rv, st_nxt + L::KT_B, L::VB, tid, item - S::NPT, part);       // V(it+1) over V(it-1)
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        mloc = row_max(mloc);
        // ---- raw loads of K(it+3), V(it+2): one whole step to arrive. Issued back to back: a vector memory instruction
        // holds the wave for as long as the CU's address path needs for it, wherever it is placed ----
        if constexpr (DMA) {
            gb_prev = gb_dma;
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // this step's tile loads have landed
            zero_v_tail(tile_of(it + 1), st_nxt + L::KT_B);
        } else {
            const gbases gb_k = group_bases(tile_of(it + 3), gp_k);
            load_tile(rk, P.kc, tile_of(it + 3), gb_k);
            load_tile(rv, P.vc, tile_of(it + 2), gb_prev);
            if constexpr (SVL) { sk = load_sblk(P.kc, tile_of(it + 3), gb_k); sv = load_sblk(P.vc, tile_of(it + 2), gb_prev); }
            gb_prev = gb_k;
        }
        // LDS stores retired, then the barrier (without the global-memory fence of __syncthreads())
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }

    // ---- epilogue: the pair swaps denominators, then each wave normalises, gates and stores its half of the dims of
    // all 64 rows. Lane (row c, half g) holds dims 32 dt + 8 (i / 4) + 4 g + (i % 4) of tile dt ----
    const float l_own = (lp[0] + __shfl_xor(lp[0], 32)) + (lp[1] + __shfl_xor(lp[1], 32));
    if (g == 0) ax_own[c] = l_own;
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");   // (also: no tile load is left in flight)
    if (P.nks > 1) {   // one of several key splits: the unnormalised partial of every row, for the merge
        if (g == 0 && live) {
            float * ml = P.part_ml + (((size_t) my_tok * P.Hq + h) * P.nks + ksp) * 2;
            ml[0] = m_run;
            ml[1] = l_own;
        }
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int tok = tok0 + 32 * (r ? wave ^ 1 : wave) + c;
            if (tok >= P.T) continue;
            float * orow = P.part_o + (((size_t) tok * P.Hq + h) * P.nks + ksp) * D;
#pragma unroll
            for (int dt = 0; dt < HD; ++dt)
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4)
                    *reinterpret_cast<f4 *>(orow + 32 * (dh * HD + dt) + 8 * q4 + 4 * g) =
                        f4{o[r][dt][4 * q4], o[r][dt][4 * q4 + 1], o[r][dt][4 * q4 + 2], o[r][dt][4 * q4 + 3]};
        }
        return;
    }
    const float l_par = ax_par[c];
    // (the gate values of both row blocks are asked for before the first is used: one memory round trip, not one per 16
    // bytes or per block)
    f4 gt[2][HD][4];
    if (P.gate) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int tok = tok0 + 32 * (r ? wave ^ 1 : wave) + c;
            const float * grow = P.gate + ((size_t) min(tok, P.T - 1) * P.Hq + h) * D;
#pragma unroll
            for (int dt = 0; dt < HD; ++dt)
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) gt[r][dt][q4] = *reinterpret_cast<const f4 *>(grow + 32 * (dh * HD + dt) + 8 * q4 + 4 * g);
        }
    }
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const int tok = tok0 + 32 * (r ? wave ^ 1 : wave) + c;
        if (tok >= P.T) continue;
        const float inv = 1.0f / (r ? l_par : l_own);
        float * orow = P.out + ((size_t) tok * P.Hq + h) * D;
#pragma unroll
        for (int dt = 0; dt < HD; ++dt)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int d0 = 32 * (dh * HD + dt) + 8 * q4 + 4 * g;
                f4 rr = {o[r][dt][4 * q4] * inv, o[r][dt][4 * q4 + 1] * inv, o[r][dt][4 * q4 + 2] * inv, o[r][dt][4 * q4 + 3] * inv};
                if (P.gate) {
                    // sigmoid through the hardware exponential and reciprocal (each within an ulp or two; exact at g = 0): the
                    // library's full-range expf and IEEE division are some twenty instructions per value, 128 values per lane
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        rr[x] *= __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * gt[r][dt][q4][x]));
                }
                *reinterpret_cast<f4 *>(orow + d0) = rr;
            }
    }
}

template <uint32_t KT, int D, bool GROUPED, bool DMA = false>
int launch_pf_g(const pf_params & P, hipStream_t s) {
    using L = pf_lay<D>;
    const int lds = 2 * L::STAGE_B + (stager<KT, D>::SCALES_VIA_LDS ? 2 * 4 * 16 * stager<KT, D>::SB : 0) + 4 * (BN / 16) * 64 * 16 + 4 * 32 * 4;
    // (the attribute belongs to the function on ONE device: remembered per device, set again on another)
    static std::atomic<uint32_t> attr_set{0};
    int dev = 0;
    (void) hipGetDevice(&dev);
    const uint32_t bit = 1u << (dev & 31);
    if (!(attr_set.load(std::memory_order_acquire) & bit)) {
        if (hipFuncSetAttribute((const void *) prefill_k<KT, D, GROUPED, DMA>, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
            (void) hipGetLastError();
            set_error("p1a_attn_prefill: cannot reserve %d bytes of LDS", lds);
            return P1A_E_LAUNCH;
        }
        attr_set.fetch_or(bit, std::memory_order_release);
    }
    const int units = P.nblk * P.Hkv * P.nks;
    const int slots = ((units + 7) / 8) * P.GQA;
    prefill_k<KT, D, GROUPED, DMA><<<slots * 8, NTHR, lds, s>>>(P);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}
template <uint32_t KT, int D>
int launch_pf(const pf_params & P, hipStream_t s) {
    const bool grouped = !P.pg.pt || P.pg.psh >= 4;
    if constexpr (KT == P1A_KV_F16 && D == 256) {
        // (rows of whole 16-byte units at 16-byte aligned addresses: what a 16-byte load per lane needs)
        // and whole 16-key groups that can be read: always inside a page; inside a contiguous cache when it holds them
        const bool groups_ok = P.pg.pt || ((P.p0 + P.T - 1) | 15) < P.n_rows;
        if (grouped && groups_ok && P.pg.rowb % 16 == 0 && P.pg.rowb * 16 < (1ull << 32)) return launch_pf_g<KT, D, true, true>(P, s);
    }
    return grouped ? launch_pf_g<KT, D, true>(P, s) : launch_pf_g<KT, D, false>(P, s);
}

}   // namespace

namespace {
// Staging pass of the scratch variant: positions 0 .. n-1 of one sequence of a q8_0 / q4_0 cache -> contiguous f16 rows
// [n][Hkv][D] (K, then V). Same conversion as the in-kernel stagers (code * f16 scale, rounded once to f16), so the
// attention kernel sees the very tiles it would have built itself. One thread per 16 codes (q8_0) / per block (q4_0).
template <uint32_t KT>
__global__ void __launch_bounds__(256) dq_k(const char * kc, const char * vc, kv_view pg, int n, int Hkv, int D, char * ko, char * vo) {
    const int32_t * ptab = pg.pt ? (pg.rtab ? pg.pt + pg.rtab[0] : pg.pt) : nullptr;
    const int per = KT == P1A_KV_Q8_0 ? 16 : 32;               // values per item
    const int ipr = Hkv * D / per;                             // items per position
    const long long idx = (long long) blockIdx.x * 256 + threadIdx.x;
    const int row = (int) (idx / ipr), it = (int) (idx - (long long) row * ipr);
    if (row >= n) return;
    const size_t off = kv_off_tab(pg, ptab, row);
    const int iph = D / per, h = it / iph, cc = it - h * iph;
    const size_t orow = ((size_t) row * Hkv + h) * D * 2;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const char * src = (which ? vc : kc) + off;
        char * dst = (which ? vo : ko) + orow;
        if constexpr (KT == P1A_KV_Q8_0) {
            const char * head = src + (size_t) h * (D / 32) * 34;
            const u4 w = *reinterpret_cast<const u4 *>(head + (D / 32) * 2 + cc * 16);
            const uint32_t d16 = *reinterpret_cast<const uint16_t *>(head + (cc >> 1) * 2);
            const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
            const pair32 x0 = deq8x4(w[0], dd), x1 = deq8x4(w[1], dd), x2 = deq8x4(w[2], dd), x3 = deq8x4(w[3], dd);
            u4 * o = reinterpret_cast<u4 *>(dst + cc * 32);
            o[0] = u4{x0.lo, x0.hi, x1.lo, x1.hi};
            o[1] = u4{x2.lo, x2.hi, x3.lo, x3.hi};
        } else {
            const uint16_t * blk = reinterpret_cast<const uint16_t *>(src + ((size_t) h * (D / 32) + cc) * 18);
            const uint32_t d16 = blk[0];
            const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
            pair32 lo[4], hi[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t w = (uint32_t) blk[1 + 2 * k] | ((uint32_t) blk[2 + 2 * k] << 16);
                lo[k] = deq4x4(w & 0x0f0f0f0fu, dd);
                hi[k] = deq4x4((w >> 4) & 0x0f0f0f0fu, dd);
            }
            u4 * o = reinterpret_cast<u4 *>(dst + cc * 64);
            o[0] = u4{lo[0].lo, lo[0].hi, lo[1].lo, lo[1].hi};
            o[1] = u4{lo[2].lo, lo[2].hi, lo[3].lo, lo[3].hi};
            o[2] = u4{hi[0].lo, hi[0].hi, hi[1].lo, hi[1].hi};
            o[3] = u4{hi[2].lo, hi[2].hi, hi[3].lo, hi[3].hi};
        }
    }
}
}   // namespace

// Key splits of a call: a chunk of few token blocks over a long context would leave most of the device idle (one
// workgroup per block and q head, each walking every tile), so the tiles of a block are dealt to nks workgroups and the
// partials merged. Chosen from the shape and the device alone (never from what scratch the caller brought: the result
// bits depend on the split): the count that minimises rounds of workgroups x tiles per workgroup, a split being at least
// 8 tiles and paying about 6 tiles' worth of set-up and partial traffic; 1 unless that saves 15 %.
int prefill_key_splits(int T, int p0, int Hq, int cus) {
    const long units = (long) ((T + BM - 1) / BM) * Hq, nt = (p0 + T - 1) / BN + 1;
    if (cus < 1) cus = 1;
    auto cost = [&](long k) { return ((units * k + cus - 1) / cus) * ((nt + k - 1) / k + 6); };
    long best = 1, cbest = cost(1);
    for (long k = 2; k <= 64 && nt / k >= 8; ++k)
        if (cost(k) < cbest) { best = k; cbest = cost(k); }
    return cbest * 100 <= cost(1) * 85 ? (int) best : 1;
}
size_t prefill_part_bytes_o(int T, int Hq, int D, int nks) { return nks > 1 ? (size_t) T * Hq * nks * D * 4 : 0; }
size_t prefill_part_bytes_ml(int T, int Hq, int nks) { return nks > 1 ? (((size_t) T * Hq * nks * 2 * 4) + 255) & ~(size_t) 255 : 0; }
void prefill_part_need(int T, int p0, int Hq, int D, size_t & bytes_o, size_t & bytes_ml) {
    const int nks = prefill_key_splits(T, p0, Hq, cu_count());
    bytes_o = prefill_part_bytes_o(T, Hq, D, nks);
    bytes_ml = prefill_part_bytes_ml(T, Hq, nks);
}

// bytes of the f16 staging copy of the first n positions (K and V)
// (rows rounded up to whole 16-key groups: the attention kernel fetches whole groups)
size_t prefill_stage_bytes(int n, int Hkv, int D) { return 2 * (size_t) ((n + 15) & ~15) * Hkv * D * 2; }

int launch_prefill(const p1a_kv & c, const float * q, float * out, const float * gate, int T, int p0, int Hq,
                   float scale, void * scratch, size_t scratch_bytes, hipStream_t s) {
    if (c.D != 64 && c.D != 128 && c.D != 256) { set_error("p1a_attn_prefill: unsupported head size D=%d", c.D); return P1A_E_SHAPE; }
    if ((((uintptr_t) c.k | (uintptr_t) c.v) & 15) || (c.pt && (c.pstride & 15))) { set_error("p1a_attn_prefill: cache base / page stride must be 16-byte aligned"); return P1A_E_SHAPE; }
    pf_params P;
    P.q = q; P.out = out; P.gate = gate; P.kc = (const char *) c.k; P.vc = (const char *) c.v; P.pg = view_of(c);
    P.T = T; P.p0 = p0; P.Hq = Hq; P.Hkv = c.Hkv; P.GQA = Hq / c.Hkv;
    P.n_rows = c.n_ctx;
    P.qscale = scale * 1.4426950408889634f;
    P.nblk = (T + BM - 1) / BM;
    P.nks = 1; P.part_o = nullptr; P.part_ml = nullptr;
    // the caller's scratch: first the f16 staging copy of a quantized cache (when it fits), then the split partials (when
    // they fit behind it); partials that do not fit go to the library's own per-stream buffers
    const int n = p0 + T;
    const bool aligned = scratch && !((uintptr_t) scratch & 255);
    const bool stage_caller = c.type != P1A_KV_F16 && aligned && scratch_bytes >= prefill_stage_bytes(n, c.Hkv, c.D);
    const size_t used = stage_caller ? (prefill_stage_bytes(n, c.Hkv, c.D) + 255) & ~(size_t) 255 : 0;
    // no room in the caller's scratch (the reference's attn_prefill brings none): the library's own staging copy, if it has one
    void * stage_own = nullptr;
    if (c.type != P1A_KV_F16 && !stage_caller) stage_own = stage_scratch(s, prefill_stage_bytes(n, c.Hkv, c.D));
    const bool stage = stage_caller || stage_own;
    const int nks = prefill_key_splits(T, p0, Hq, cu_count());
    if (nks > 1) {
        const size_t bo = prefill_part_bytes_o(T, Hq, c.D, nks), bm = prefill_part_bytes_ml(T, Hq, nks);
        if (aligned && scratch_bytes >= used + bm + bo) {
            P.part_ml = reinterpret_cast<float *>((char *) scratch + used);
            P.part_o = reinterpret_cast<float *>((char *) scratch + used + bm);
        } else if (!split_scratch(s, bo, bm, P.part_o, P.part_ml)) return P1A_E_SCRATCH;   // (the split count fixes the result bits: never fewer splits for want of room)
    }
    P.nks = nks;
    auto finish = [&](int rc) {
        if (rc != P1A_OK || P.nks == 1) return rc;
        return launch_merge(P.part_o, P.part_ml, out, gate, P.nks, c.D, Hq, T, s);
    };
#define PF(KT_) finish(c.D == 256 ? launch_pf<KT_, 256>(P, s) : c.D == 128 ? launch_pf<KT_, 128>(P, s) : launch_pf<KT_, 64>(P, s))
    if (c.type == P1A_KV_F16) return PF(P1A_KV_F16);
    // A quantized cache with enough caller scratch: convert the visible positions to f16 once (tens of microseconds, the
    // copy stays in the Infinity Cache) and run the f16 kernel on it - every workgroup then skips the dequantization it
    // would otherwise repeat per 128 query rows. Same tiles, same products, same bits as the direct kernel.
    if (stage) {
        const int n16 = (n + 15) & ~15;
        char * ko = (char *) (stage_caller ? scratch : stage_own), * vo = ko + (size_t) n16 * c.Hkv * c.D * 2;
        const long long items = (long long) n * (c.Hkv * c.D / (c.type == P1A_KV_Q8_0 ? 16 : 32));
        const unsigned blocks = (unsigned) ((items + 255) / 256);
        if (c.type == P1A_KV_Q8_0) dq_k<P1A_KV_Q8_0><<<blocks, 256, 0, s>>>(P.kc, P.vc, P.pg, n, c.Hkv, c.D, ko, vo);
        else dq_k<P1A_KV_Q4_0><<<blocks, 256, 0, s>>>(P.kc, P.vc, P.pg, n, c.Hkv, c.D, ko, vo);
        if (hipPeekAtLastError() != hipSuccess) return P1A_E_LAUNCH;
        P.kc = ko; P.vc = vo;
        P.pg.pt = nullptr; P.pg.rtab = nullptr; P.pg.psh = 0; P.pg.pstride = 0;
        P.pg.rowb = (size_t) c.Hkv * c.D * 2;
        P.n_rows = n16;
        return PF(P1A_KV_F16);
    }
    if (c.type == P1A_KV_Q8_0) return PF(P1A_KV_Q8_0);
    return PF(P1A_KV_Q4_0);
#undef PF
}

}   // namespace p1a


extern "C" size_t p1a_attn_prefill_scratch_bytes(int T, int p0, int Hq, int Hkv, int D) {
    if (T < 1 || p0 < 0 || Hkv < 1 || D < 1) return 0;
    // optional: with this much scratch a quantized cache is converted to f16 once per call instead of once per
    // workgroup, and the partials of a key-split call (few token blocks over a long context) live in it; with less (or
    // none) the kernel converts on the fly and the partials go to the library's own per-stream buffers
    const int nks = Hq >= 1 ? p1a::prefill_key_splits(T, p0, Hq, p1a::cu_count()) : 1;
    return ((p1a::prefill_stage_bytes(p0 + T, Hkv, D) + 255) & ~(size_t) 255) + p1a::prefill_part_bytes_ml(T, Hq, nks) +
           p1a::prefill_part_bytes_o(T, Hq, D, nks);
}

extern "C" int p1a_attn_prefill_key_splits(int T, int p0, int Hq) {
    if (T < 1 || p0 < 0 || Hq < 1) return 1;
    return p1a::prefill_key_splits(T, p0, Hq, p1a::cu_count());
}
