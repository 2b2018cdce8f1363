// Split-K paged-KV decode / MTP-verify attention for gfx950 (MI355X).
//
// Work decomposition
//   grid = (nsplit * kv heads, row groups), block = NW waves (8, or 4 when a tile is large). A row group is up to 4
//   query rows of ONE sequence (the tokens of a verify block); its GQA * rows query rows are the columns of 16-wide
//   MFMA tiles, so the group's KV is read once. A workgroup owns one kv head; in unit u (32 * NW positions) wave w owns
//   the 32 consecutive positions 32 w .., which it walks as two 16-key tiles; split stream s owns the units s,
//   s + nsplit, ... . The partition depends only on the device and Hkv, never on T, the depth or the batch, so a row
//   is computed by the same sequence of operations whichever call it is part of (T-invariance, rows == single,
//   paged == contiguous).
// Data movement
//   A 16-key tile of one head (K or V) is fetched by global_load_lds_dwordx4: 16 bytes per lane in memory order (17
//   consecutive lanes cover one q8_0 head row), written by the memory pipeline straight into a wave-private LDS slot
//   that is the linear image of those rows - no staging registers, no workgroup barrier in the key loop. K and V have
//   two slots each; the loads of tile t + 1 are issued between the products of tile t, and the in-order vector-memory
//   counter tells which tile has landed. (A second build of the kernel, SB, has one slot each and half the registers, so
//   that two workgroups share a CU: calls of many workgroups take it, see dec_mfma_k.) The Q rows are the same for all waves of a workgroup: they are requested
//   first (older than every tile request), once, straight into LDS, and scaled and rounded into an f16 table that the
//   lanes pick their MFMA operands from.
// Arithmetic
//   S^T = K Q^T on v_mfma_f32_16x16x32_f16 and O^T = V^T P^T on v_mfma_f32_16x16x16_f16: q8_0 codes are expanded to
//   f16 in registers with a byte-permute (0x6400 | code ^ 0x80 = 1152 + code) and multiplied by the f16 block scale;
//   V is read from LDS with the transposing ds_read_b64_tr_b8 / _tr_b16 so that a lane holds 4 keys of one output
//   dim. Q is pre-multiplied by scale * log2(e) and rounded to f16, P = 2^(S - m) is rounded to f16, all accumulation
//   is fp32. The softmax denominator is one more MFMA against an all-ones operand, so it sums exactly the P that
//   multiplies V. The waves of one head fold their (m, l, O) through LDS; one partial per (workgroup, head) goes to
//   scratch and merge_k folds the splits in a fixed order and applies the sigmoid gate.
#include "p1a_common.hpp"

#include <cstdlib>
#include <type_traits>

namespace p1a {
namespace {

constexpr float NEG_INF = -__builtin_inff();
constexpr float RESCALE_STEP = 8.0f;   // log2 of the largest P the running maximum lets through

template <uint32_t KT, int D> struct tile_cfg {
    static constexpr int HB = (int) head_bytes(KT, D);
    static constexpr int CPK = HB / 16;                        // 16-byte chunks per (key, head)
    static constexpr int NCH = 16 * CPK;                       // chunks per 16-key tile
    static constexpr int NRND = (NCH + 63) / 64;               // load rounds per tile
    static constexpr int TILE_B = 16 * HB;                     // the linear image of 16 head rows
    static constexpr int QDP = D / 4 + 4;                      // floats per column of a parked dim quarter: padded, or the 16
                                                               // columns of a store would all start in the same LDS bank
    static constexpr int QTR_B = 16 * QDP * 4;                 // one dim quarter of a wave's accumulators (merge epilogue)
    static constexpr int SLOT_B = TILE_B > QTR_B ? TILE_B : QTR_B;   // one LDS slot
    static constexpr int VA_B = KT == P1A_KV_Q4_0 ? 16 * 144 : 0;    // q4_0: 8-byte aligned copy of a V tile's nibbles
    static constexpr int TAB_B = 256;                          // per wave: transposed V scales, later (m, l) of the merge
    static constexpr int QRS = D * 2 + 16;                     // row stride of the f16 Q table (padded: no bank conflicts)
    static constexpr int NMF = D / 32;                         // QK MFMAs per tile
    static constexpr int NDT = D / 16;                         // output dim tiles
    static_assert(HB % 16 == 0, "head row must be a whole number of 16-byte chunks");
};


// Staged source (q8_0 / q4_0 head rows that are not whole 16-byte chunks, i.e. D = 64 or 128): the raw image of 16 head
// rows is fetched 4 bytes per lane, converted by its wave into the f16 tile the f16 kernel reads, and computed on as f16.
template <uint32_t KS, int D> struct raw_cfg {
    static constexpr int HB = (int) head_bytes(KS, D);
    static constexpr int RAW_B = 16 * HB;                      // the linear image of 16 raw head rows
    static constexpr int NDW = RAW_B / 4;
    static constexpr int NRND = (NDW + 63) / 64;               // load rounds per tile (4 bytes per lane)
    static_assert(HB % 4 == 0, "raw head rows are whole dwords");
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
    int T, RG, Hq, Hkv, GQA;
    float qscale;     // softmax scale * log2(e)
    int nsplit;       // split streams
    int hkv_sh;       // log2(Hkv) when Hkv is a power of two, else -1
    int npt;          // page-table entries of one sequence (ceil(n_ctx / page positions)); 0 = contiguous
};

__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) { return __builtin_amdgcn_perm(hi, lo, sel); }
__device__ __forceinline__ int rfl(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ size_t rfl64(size_t x) {
    const uint32_t lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) x);
    const uint32_t hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (x >> 32));
    return ((size_t) hi << 32) | lo;
}

// 4 int8 codes (one dword) -> (code * d) as two packed f16 pairs, returned as raw dwords so MFMA operands are built in place
struct u2 { uint32_t lo, hi; };
__device__ __forceinline__ u2 deq4(uint32_t w, h2 d01, h2 d23) {
    const h2 off = {(half_t) 1152, (half_t) 1152};
    const uint32_t x = w ^ 0x80808080u;
    const h2 a = __builtin_bit_cast(h2, perm(0x64646464u, x, 0x04010400u));
    const h2 b = __builtin_bit_cast(h2, perm(0x64646464u, x, 0x04030402u));
    return u2{__builtin_bit_cast(uint32_t, (a - off) * d01), __builtin_bit_cast(uint32_t, (b - off) * d23)};
}

// q * scale rounded to fp32, then to f16: two roundings, spelled out. Left to itself the compiler turns (half) (q * s) into
// a fused multiply-convert (one rounding) in some places and into a multiply and a convert in others, and two kernel
// variants could then disagree in the last bit of a Q operand - rows must not depend on the variant that ran.
__device__ __forceinline__ half_t scale_to_half(float q, float s) {
    float p = q * s;
    asm volatile("" : "+v"(p));
    return (half_t) p;
}

// the maximum over the four lanes that share (lane & 15): the two 16-lane rows of each half, then the two halves
__device__ __forceinline__ float max_over_groups(float m) { return max_swap32(max_swap16(m)); }

// 4 nibbles (the low nibbles of the 4 bytes of w) -> ((n - 8) * d) as two packed f16 pairs (0x6400 | n = 1024 + n)
__device__ __forceinline__ u2 deq4n2(uint32_t w, h2 d01, h2 d23) {
    const h2 off = {(half_t) 1032, (half_t) 1032};
    const h2 a = __builtin_bit_cast(h2, perm(0x64646464u, w, 0x04010400u));
    const h2 b = __builtin_bit_cast(h2, perm(0x64646464u, w, 0x04030402u));
    return u2{__builtin_bit_cast(uint32_t, (a - off) * d01), __builtin_bit_cast(uint32_t, (b - off) * d23)};
}
__device__ __forceinline__ u2 deq4n(uint32_t w, h2 dd) { return deq4n2(w, dd, dd); }

// ---- hand-issued memory operations of the tile ring ----
// The tile loads are global_load_lds_dwordx4 (global -> LDS, 16 bytes per lane, lane i lands at M0 + 16 i). They are
// written as inline assembly so that the waits on them can be partial: the vector-memory counter retires in order,
// so "at most n newer loads outstanding" (s_waitcnt vmcnt(n)) is exactly "tile x has landed" when every tile is NR
// loads. For the same reason nothing else in the key loop may be a vector load: the page-table entry of a tile is
// fetched with a scalar load, issued one step ahead.
__device__ __forceinline__ uint32_t lds_addr(const char * p) { return (uint32_t) (size_t) (const __attribute__((address_space(3))) char *) p; }
__device__ __forceinline__ void dma16(const char * sbase, uint32_t voff, uint32_t lds) {
    // (the destination is wave-uniform by construction; say so, or a value the compiler happens to keep in a vector
    // register cannot be given to s_mov)
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(voff), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane((int) lds)) : "memory", "m0");
}
__device__ __forceinline__ void dma16v(const char * vaddr, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(vaddr), "s"(lds) : "memory", "m0");
}
// 4 bytes per lane: lane i lands at M0 + 4 i
__device__ __forceinline__ void dma4(const char * sbase, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" :: "v"(voff), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane((int) lds)) : "memory", "m0");
}
template <int N> __device__ __forceinline__ void wait_vm_imm() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }
// wait until at most `newer` tile fetches (NR loads each) issued after the wanted one are still in flight
template <int NR> __device__ __forceinline__ void wait_tiles(int newer) {
    if (newer <= 0) wait_vm_imm<0>();
    else if (newer == 1) wait_vm_imm<NR>();
    else if (newer == 2) wait_vm_imm<2 * NR>();
    else wait_vm_imm<3 * NR>();
}
// A page-table entry through the scalar cache: a load from the constant address space at a wave-uniform address is an
// s_load_dword, and the compiler itself places the wait for it before the first use of the value (a hand-written
// s_load whose result the compiler may copy before a hand-written wait is a race). The table does not change while a
// kernel runs.
__device__ __forceinline__ int sload_i32(const int32_t * p) {
    return *reinterpret_cast<const __attribute__((address_space(4))) int32_t *>(rfl64((size_t) p));
}

// SB ("single-buffered"): one K and one V slot per wave instead of two, so that two workgroups fit a CU's LDS (and register
// file: 128 registers per lane) - for calls of many workgroups, where a second resident workgroup covers the start-up,
// the fold and the memory round trips of the first. Tile t + 1 of K is then requested once the products with tile t of K
// are done, V likewise; everything a lane computes, and the order it computes it in, is the same as in the double-buffered
// kernel, so the partials are the same bits. One column tile only (NT == 1, at most 16 live columns).
// KS (when it differs from KT = f16): the type the cache holds - its raw tiles are staged (raw_cfg) and converted to f16
template <uint32_t KT, int D, int NT, int NWV, bool SB, uint32_t KS = KT>
__global__ void __launch_bounds__(NWV * 64, SB ? NWV / 2 : 1) dec_mfma_k(const dec_params P) {
    using C = tile_cfg<KT, D>;
    using RW = raw_cfg<KS, D>;
    constexpr bool STG = KS != KT;
    static_assert(!SB || NT == 1, "the single-buffered variant has one column tile");
    static_assert(!STG || (KT == P1A_KV_F16 && !SB && D <= 128), "staged tiles are converted to f16 and take the double-buffered build");
    constexpr int NLD = STG ? RW::NRND : C::NRND;             // vector-memory operations per tile fetch
    // STG: slot array 0 = the f16 K tile of every wave, 1 = the f16 V tile, 2 = two raw K tiles, 3 = two raw V tiles
    constexpr int SLOTX = STG ? (C::SLOT_B > 2 * RW::RAW_B ? C::SLOT_B : 2 * RW::RAW_B) : C::SLOT_B;
    // four tile slots per wave (K and V, two each), plus a small per-wave table. SB: one pool that holds one K slot, one
    // V slot (and the q4_0 copy) per wave at the size of a tile, and is handed over to the fold as a whole afterwards:
    // wave w parks 8 columns at a time, dim quarter k at PARK_B (4 w + k)
    constexpr int SLB = SB ? C::TILE_B : SLOTX;                // bytes per slot
    constexpr int PARK_B = 8 * C::QDP * 4;                     // SB: one dim quarter of 8 parked columns
    constexpr int POOL_T = NWV * (2 * C::TILE_B + C::VA_B), POOL_P = NWV * 4 * PARK_B;
    __shared__ __attribute__((aligned(16))) char pool[SB ? (POOL_T > POOL_P ? POOL_T : POOL_P) : 16];
    // (one array, slot array k at k NWV SLOT_B: K slot 0, K slot 1, V slot 0, V slot 1 - the fold addresses them by number)
    __shared__ __attribute__((aligned(16))) char slots[SB ? 16 : 4 * NWV * SLOTX];
    __shared__ __attribute__((aligned(16))) char qown[SB ? 16 * C::QRS : 16];          // SB: the f16 Q table (first the fp32 copy of up to 8 rows)
    // (STG: "K slot 1" / "V slot 1" - where the Q copies go before any tile is converted - are the f16 tile arrays themselves)
    char * const kb0 = SB ? pool : slots, * const vb0 = SB ? pool + NWV * C::TILE_B : STG ? slots + NWV * SLOTX : slots + 2 * NWV * SLOTX;
    char * const kb1 = SB || STG ? kb0 : slots + NWV * SLOTX, * const vb1 = SB || STG ? vb0 : slots + 3 * NWV * SLOTX;
    static_assert(SB || (32 * D * 4 <= NWV * SLOTX && 32 * C::QRS <= NWV * SLOTX), "the Q copies (at most 32 columns) fit over the second K and V slots");
    static_assert(!SB || 8 * D * 4 <= 16 * C::QRS, "SB: the fp32 copy of 8 rows fits where the f16 table of 16 goes");
    // q8_0 with two column tiles has no registers left for 64 dwords of Q operands (spills there cost more than their
    // traffic: the compiler can only wait for a reload with "no vector memory operation outstanding", tiles included):
    // that variant keeps the f16 Q table and reads its operands from it tile after tile
    // (SB, 128 registers: likewise, whatever the type; with at most 8 live columns its table has 8 and lanes c and c + 8
    // read the same one - the columns past the live ones are never weighted)
    constexpr bool QLDS = (KT == P1A_KV_Q8_0 && NT == 2) || SB;
    __shared__ __attribute__((aligned(16))) char qtab[QLDS && !SB ? 32 * C::QRS : 16];
    __shared__ __attribute__((aligned(16))) char tabs[NWV * C::TAB_B];
    __shared__ __attribute__((aligned(16))) char vab[SB ? 16 : NWV * C::VA_B + 16];

    const int lane = threadIdx.x & 63, wave = rfl(threadIdx.x >> 6);
    const int c = lane & 15, g = lane >> 4;
    // blockIdx.x -> (split stream, head group). Workgroups are dealt to the 8 XCDs round-robin by linear index, so
    // the kv heads of one split stream (which share cache lines) are given the same index mod 8.
    const int HG = P.Hkv;
    int split, hg;
    if ((P.nsplit & 7) == 0) {
        const int i = blockIdx.x, j = i >> 3;
        const int jq = P.hkv_sh >= 0 ? j >> P.hkv_sh : j / HG;
        hg = j - jq * HG;
        split = jq * 8 + (i & 7);
    } else {
        split = blockIdx.x / HG;
        hg = blockIdx.x - split * HG;
    }
    const int hk = hg, sub = wave;
    constexpr int U = 32 * NWV;                               // positions per unit
    const int row0 = blockIdx.y * P.RG;
    const int nr = min(P.RG, P.T - row0);                     // rows of this group
    const int R = nr * P.GQA;                                 // live MFMA columns
    // the page-table entry of this wave's first tile is asked for before anything else (it is the first link of the
    // chain entry -> tile address -> tile); the index is clamped into the table, the entry is only used if the tile exists
    // (the group's first position and its page-table row hang on the kernel arguments only: both scalar loads are issued
    // before either value is used - one round trip for the two)
    const bool has_rt = P.pg.pt && P.pg.rtab;
    const int rt0 = has_rt ? sload_i32(P.pg.rtab + (P.pos_rows ? row0 : 0)) : 0;
    const int pos_first = P.pos_rows ? sload_i32(P.pos_rows + row0) : 0;
    const int32_t * ptab = P.pg.pt ? P.pg.pt + rt0 : nullptr;
    // (n_ctx only bounds the read here: an entry fetched through a clamped index is fetched again, unclamped, once the
    // tile is known to exist)
    const int idx_early = max(0, min((split * U + sub * 32) >> P.pg.psh, P.npt - 1));
    int pg0_early = 0;
    if (ptab) pg0_early = sload_i32(ptab + idx_early);
    const int p0v = P.pos_rows ? 0 : (P.p0_dev ? *P.p0_dev : P.p0);
    char * const ks0 = kb0 + wave * SLB, * const ks1 = kb1 + wave * SLB;
    char * const vs0 = vb0 + wave * SLB, * const vs1 = vb1 + wave * SLB;
    char * const tab = tabs + wave * C::TAB_B;
    char * const va = (SB ? pool + 2 * NWV * C::TILE_B : vab) + wave * C::VA_B;
    char * const rawk = slots + (2 * NWV + wave) * SLOTX, * const rawv = slots + (3 * NWV + wave) * SLOTX;   // STG: two raw tiles each

    // column -> row of the group (at most 4 rows: three comparisons instead of a division)
    auto row_of = [&](int col) { return (col >= P.GQA) + (col >= 2 * P.GQA) + (col >= 3 * P.GQA); };
    // visible-position limit of each of this lane's columns, and the group's maximum
    int plim[NT];
    int n_max = 0, p_min = 0x7fffffff;
    for (int t = 0; t < nr; ++t) {
        const int pt_ = P.pos_rows ? (t ? P.pos_rows[row0 + t] : pos_first) : p0v + row0 + t;
        n_max = max(n_max, pt_ + 1);
        p_min = min(p_min, pt_);
    }
    n_max = rfl(n_max);
    p_min = rfl(p_min);
    // A workgroup none of whose streams holds a visible key (a short sequence in a batch: stream s is empty once s units
    // cover the sequence) is done before it asks for anything else - a wide call of short sequences launches several of
    // these for every workgroup that has work. It leaves the empty partials its stream would have ended with, unless the
    // rows carry their own positions: merge_k then knows from those which streams to skip and never reads them.
    if (split * U >= n_max) {
        if (!P.pos_rows) {
            for (int col = threadIdx.x; col < R; col += NWV * 64) {
                const int t = row_of(col), hh = col - t * P.GQA;
                const size_t row = (size_t) (row0 + t) * P.Hq + (size_t) hg * P.GQA + hh;
                float * pm = P.part_ml + (row * P.nsplit + split) * 2;
                pm[0] = NEG_INF;
                pm[1] = 0.f;
            }
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < NT; ++r) {
        const int col = 16 * r + c;
        plim[r] = -1;
        if (col < R) {
            const int t = row_of(col);
            plim[r] = P.pos_rows ? P.pos_rows[row0 + t] : p0v + row0 + t;
        }
    }
    // The limits are wanted HERE, before the first tile request: the compiler waits for its own loads with a plain
    // "nothing outstanding", and placed after the requests such a wait would also wait for the tiles.
#pragma unroll
    for (int r = 0; r < NT; ++r) asm volatile("" : "+v"(plim[r]));
    const size_t head_off = (size_t) hk * (STG ? RW::HB : C::HB);
    const int rowb = (int) P.pg.rowb;

    // chunk i = 64 * round + lane of a tile is bytes [16 cir, +16) of key i / CPK; static per-lane source offsets
    // (STG: dword i of the raw image is dword i % (HB / 4) of key i / (HB / 4))
    constexpr int IPK = STG ? RW::HB / 4 : C::CPK, ISZ = STG ? 4 : 16;     // items per key, bytes per item
    unsigned soff[NLD];
#pragma unroll
    for (int rd = 0; rd < NLD; ++rd) {
        const int i = rd * 64 + lane;
        const int key = i / IPK, cir = i - key * IPK;
        soff[rd] = (unsigned) (key * rowb + (int) head_off + cir * ISZ);
    }

    // Tile t of this wave (t = 0, 1, ...): unit split + (t >> 1) * nsplit, keys [ts, ts + 16) with
    // ts = unit * U + sub * 32 + 16 * (t & 1). A 16-key tile never straddles a page (pages hold >= 16 positions).
    auto tile_start = [&](int t) { return (split + (t >> 1) * P.nsplit) * U + sub * 32 + 16 * (t & 1); };
    // One of the NR loads of a tile: round rd of the tile at `ts` into `slot`. Keys past the last visible position are
    // clamped onto it (never weighted), so nothing outside the sequence is read. A tile is always exactly NR loads.
    auto tile_off = [&](int ts, int page) -> size_t {
        if (!ptab) return (size_t) ts * P.pg.rowb;
        return (size_t) page * P.pg.pstride + (size_t) (ts & ((1 << P.pg.psh) - 1)) * P.pg.rowb;
    };
    auto fetch_round = [&](char * slot, const char * b0, int ts, int rd) {
        const int last = n_max - 1 - ts;
        const int i = rd * 64 + lane;
        uint32_t off = soff[rd];
        if (last < 15) {   // (the last tile of a sequence only)
            if constexpr (SB) {   // worked out from scratch rather than from values kept in registers through the key loop
                int ii = i;
                asm volatile("" : "+v"(ii));
                off -= (uint32_t) (max(ii / C::CPK - last, 0) * rowb);
            } else {
                const int key = i / IPK, cir = i - key * IPK;
                off = (uint32_t) (min(key, last) * rowb + (int) head_off + cir * ISZ);
            }
        }
        if constexpr (STG) { if (RW::NDW % 64 == 0 || i < RW::NDW) dma4(b0, off, lds_addr(slot) + rd * 256); }
        else if (C::NCH % 64 == 0 || i < C::NCH) dma16(b0, off, lds_addr(slot) + rd * 1024);
    };
    // STG: the raw image of 16 head rows at `raw` -> the f16 tile at `dst` (row c at c * 2 D bytes), by this wave alone. The
    // values are code * f16 scale rounded once to f16 - what the D = 256 kernels feed their products and the prefill stages.
    auto convert = [&](const char * raw, char * dst) {
        if constexpr (STG && KS == P1A_KV_Q8_0) {
            // item = 8 codes of one key: D / 8 items per key; codes start behind the D / 32 scales
            constexpr int IPR = D / 8, NIT = 16 * IPR / 64;
#pragma unroll
            for (int x = 0; x < NIT; ++x) {
                const int it = x * 64 + lane, key = it / IPR, p8 = it - key * IPR;
                const char * row = raw + key * RW::HB;
                const uint32_t * cw = reinterpret_cast<const uint32_t *>(row + (D / 32) * 2 + 8 * p8);   // (4-byte aligned)
                const uint32_t w0 = cw[0], w1 = cw[1];
                const uint32_t d16 = *reinterpret_cast<const uint16_t *>(row + 2 * (p8 >> 2));
                const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
                const u2 a = deq4(w0, dd, dd), b = deq4(w1, dd, dd);
                *reinterpret_cast<u4 *>(dst + key * (2 * D) + 16 * p8) = u4{a.lo, a.hi, b.lo, b.hi};
            }
        } else if constexpr (STG) {
            // item = one 18-byte block of one key (2-byte aligned): values 0 .. 15 are its low nibbles, 16 .. 31 the high ones
            constexpr int BPR = D / 32, NIT = (16 * BPR + 63) / 64;
#pragma unroll
            for (int x = 0; x < NIT; ++x) {
                const int it = x * 64 + lane, key = it / BPR, b = it - key * BPR;
                if (16 * BPR % 64 == 0 || it < 16 * BPR) {
                    const uint16_t * blk = reinterpret_cast<const uint16_t *>(raw + key * RW::HB + 18 * b);
                    const uint32_t d16 = blk[0];
                    const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
                    u4 lo[2], hi[2];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const uint32_t w = (uint32_t) blk[1 + 2 * q] | ((uint32_t) blk[2 + 2 * q] << 16);
                        const u2 l = deq4n(w & 0x0f0f0f0fu, dd), h = deq4n((w >> 4) & 0x0f0f0f0fu, dd);
                        lo[q >> 1][2 * (q & 1)] = l.lo; lo[q >> 1][2 * (q & 1) + 1] = l.hi;
                        hi[q >> 1][2 * (q & 1)] = h.lo; hi[q >> 1][2 * (q & 1) + 1] = h.hi;
                    }
                    u4 * o = reinterpret_cast<u4 *>(dst + key * (2 * D) + 64 * b);
                    o[0] = lo[0]; o[1] = lo[1]; o[2] = hi[0]; o[3] = hi[1];
                }
            }
        }
    };
    auto page_of = [&](int ts) -> const int32_t * { return ptab + (ts >> P.pg.psh); };

    // first requests: K, then V of tile 0; every later tile is requested, one load at a time, from inside the step
    // before it, so that a wave is never parked on the memory pipeline for long while it has products to compute
    size_t off0 = 0;                                          // where tile 0 starts
    auto request_k0 = [&](bool first) {
        if (tile_start(0) >= n_max) return;
        int pg0 = pg0_early;
        if (ptab && (!first || (tile_start(0) >> P.pg.psh) != idx_early)) pg0 = sload_i32(page_of(tile_start(0)));
        off0 = tile_off(tile_start(0), pg0);
#pragma unroll
        for (int rd = 0; rd < NLD; ++rd) fetch_round(STG ? rawk : ks0, P.kc + off0, tile_start(0), rd);
    };
    auto request_v0 = [&]() {
        if (tile_start(0) >= n_max) return;
#pragma unroll
        for (int rd = 0; rd < NLD; ++rd) fetch_round(STG ? rawv : vs0, P.vc + off0, tile_start(0), rd);
    };
    // This wave's share of the Q rows -> LDS (fp32, column col at col * 4 D bytes of K slot 1; lane i brings floats
    // 4 i .. 4 i + 3). These requests are OLDER than the tile requests that follow, so waiting for them below does not
    // wait for a tile.
    // (SB with more than 8 live columns has no room for their fp32 copy: every thread fetches its pieces itself, scales and
    // rounds them and writes them to the table - ahead of the tile requests, since the compiler's wait for such a load is a
    // wait for everything outstanding)
    const bool q_direct = SB && R > 8;
    if (q_direct) {
        constexpr int NPC = (16 * (D / 4) + NWV * 64 - 1) / (NWV * 64);
        float4 a[NPC];
#pragma unroll
        for (int k = 0; k < NPC; ++k) {
            const int i = threadIdx.x + k * NWV * 64, col = i / (D / 4), d4 = i - col * (D / 4);
            a[k] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (col < R) {
                const int t = row_of(col), hh = col - t * P.GQA;
                a[k] = *reinterpret_cast<const float4 *>(P.q + ((size_t) (row0 + t) * P.Hq + (size_t) hk * P.GQA + hh) * D + 4 * d4);
            }
        }
#pragma unroll
        for (int k = 0; k < NPC; ++k) {
            const int i = threadIdx.x + k * NWV * 64, col = i / (D / 4), d4 = i - col * (D / 4);
            const float s = P.qscale;
            if (col < 16) *reinterpret_cast<h4 *>(qown + col * C::QRS + d4 * 8) = h4{scale_to_half(a[k].x, s), scale_to_half(a[k].y, s), scale_to_half(a[k].z, s), scale_to_half(a[k].w, s)};
        }
    } else {
    for (int col = wave; col < R; col += NWV) {
        const int t = row_of(col), hh = col - t * P.GQA;
        const float * qr = P.q + ((size_t) (row0 + t) * P.Hq + (size_t) hk * P.GQA + hh) * D;
        if (lane < D / 4) dma16(reinterpret_cast<const char *>(qr), lane * 16, lds_addr(SB ? qown : kb1) + col * (D * 4));
    }
    }
    request_k0(true);
    request_v0();
    // Q^T operands: column = query row (token t, head hh of the group), 8 consecutive dims per MFMA slot group. The
    // rows are the same for every wave of the workgroup, so the workgroup scales and rounds them once - every thread its
    // piece - into an f16 table over V slot 1 (rows padded: conflict-free reads), and every lane picks its operands
    // out of that. (While a workgroup's requests queue up at the memory pipeline a wave cannot issue anything else:
    // what little work there is before the first tile is best kept short.)
    if (!q_direct) { if (tile_start(0) < n_max) wait_vm_imm<2 * NLD>(); else wait_vm_imm<0>(); }
    __syncthreads();
    char * const qt = SB ? qown : QLDS ? qtab : vb1;
    if constexpr (SB) {   // in place (8 columns): every piece is read, by the thread that will write it, before any is written
        if (!q_direct) {
            constexpr int NPQ = (8 * (D / 4) + NWV * 64 - 1) / (NWV * 64);
            float4 a[NPQ];
#pragma unroll
            for (int k = 0; k < NPQ; ++k) {
                const int i = threadIdx.x + k * NWV * 64, col = i / (D / 4);
                a[k] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (col < R) a[k] = *reinterpret_cast<const float4 *>(qown + (size_t) i * 16);
            }
            __syncthreads();
            const float s = P.qscale;
#pragma unroll
            for (int k = 0; k < NPQ; ++k) {
                const int i = threadIdx.x + k * NWV * 64, col = i / (D / 4), d = 4 * (i - col * (D / 4));
                if (col < 8) *reinterpret_cast<h4 *>(qt + col * C::QRS + d * 2) = h4{scale_to_half(a[k].x, s), scale_to_half(a[k].y, s), scale_to_half(a[k].z, s), scale_to_half(a[k].w, s)};
            }
        }
    } else {
    for (int i = threadIdx.x; i < (QLDS ? 32 : R) * (D / 4); i += NWV * 64) {
        const int col = i / (D / 4), d = 4 * (i - col * (D / 4));
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f);          // (columns past the live ones: zero operands)
        if (col < R) a = *reinterpret_cast<const float4 *>(kb1 + (size_t) i * 16);
        const float s = P.qscale;
        *reinterpret_cast<h4 *>(qt + col * C::QRS + d * 2) = h4{scale_to_half(a.x, s), scale_to_half(a.y, s), scale_to_half(a.z, s), scale_to_half(a.w, s)};
    }
    }
    __syncthreads();
    h8 qf[QLDS ? 1 : NT][QLDS ? 1 : C::NMF];
#pragma unroll
    for (int r = 0; r < (QLDS ? 0 : NT); ++r) {
        const int col = 16 * r + c;
        const bool livec = col < R;
        const char * qr = vb1 + (livec ? col : 0) * C::QRS;
#pragma unroll
        for (int m = 0; m < C::NMF; ++m) {
            // the 8 dims of k-slot group g of product m: f16 a run of 8; q8_0 half of a 16-code chunk; q4_0 the values
            // of nibble bytes 4 g .. 4 g + 3 of block m (low nibbles = values 4 g .., high nibbles = values 16 + 4 g ..)
            const int d0 = KT == P1A_KV_F16 ? 32 * m + 8 * g : KT == P1A_KV_Q8_0 ? 16 * (4 * (m >> 1) + g) + 8 * (m & 1) : 32 * m + 4 * g;
            const int d1 = KT == P1A_KV_Q4_0 ? d0 + 16 : d0 + 4;
            const h4 a = *reinterpret_cast<const h4 *>(qr + d0 * 2), b = *reinterpret_cast<const h4 *>(qr + d1 * 2);
            const half_t z = (half_t) 0;
            qf[r][m] = livec ? h8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]} : h8{z, z, z, z, z, z, z, z};
        }
    }
    if constexpr (!SB) __syncthreads();                       // both copies are done with: tile 1 may be requested
    const char * qrow[NT];                                    // QLDS: this lane's row of the table, per column tile
#pragma unroll
    for (int r = 0; r < NT; ++r) qrow[r] = qt + (SB ? (R > 8 ? c : (c & 7)) : 16 * r + c) * C::QRS;
    f4 o[NT][C::NDT];
    f4 ol[NT];
    float m_run[NT];
    const h4 ones = {(half_t) 1, (half_t) 1, (half_t) 1, (half_t) 1};
#pragma unroll
    for (int r = 0; r < NT; ++r) {
        m_run[r] = NEG_INF;
        ol[r] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < C::NDT; ++j) o[r][j] = f4{0.f, 0.f, 0.f, 0.f};
    }

    // one 16-key tile from slots (ks, vs); the loads of tile t + 1 into (ksn, vsn) are issued between its products
    auto step = [&](char * ks, char * vs, char * ksn_, char * vsn_, int t) {
        // (STG: ks / vs are the wave's f16 tiles; the raw tiles alternate between the two halves of its raw areas)
        char * const ksn = STG ? rawk + ((t + 1) & 1) * RW::RAW_B : ksn_, * const vsn = STG ? rawv + ((t + 1) & 1) * RW::RAW_B : vsn_;
        const int ts = tile_start(t);
        const int tn = tile_start(t + 1);
        const bool have_n = tn < n_max;
        // the two waves of a SIMD take turns at the higher issue priority: the older wave would otherwise win every tie,
        // finish its stream some 2 us before the younger one and wait for it at the fold
        if ((t ^ (wave >> 2)) & 1) __builtin_amdgcn_s_setprio(1); else __builtin_amdgcn_s_setprio(0);
        int pgn = 0;
        if (ptab && have_n) pgn = sload_i32(page_of(tn));
        wait_vm_imm<NLD>();                                   // K of tile t has landed (only its V is younger)
        if constexpr (STG) convert(rawk + (t & 1) * RW::RAW_B, ks);
        const size_t on = have_n ? tile_off(tn, pgn) : 0;
        const char * const kn = P.kc + on, * const vn = P.vc + on;
        // ---- S^T = K Q^T ----
        f4 s[NT];
#pragma unroll
        for (int r = 0; r < NT; ++r) s[r] = f4{0.f, 0.f, 0.f, 0.f};
        const char * krow = ks + c * C::HB;
        if constexpr (KT == P1A_KV_F16) {
#pragma unroll
            for (int m = 0; m < C::NMF; ++m) {
                const h8 a = *reinterpret_cast<const h8 *>(krow + (4 * m + g) * 16);
#pragma unroll
                for (int r = 0; r < NT; ++r) {
                    h8 qo;
                    if constexpr (QLDS) qo = *reinterpret_cast<const h8 *>(qrow[r] + (32 * m + 8 * g) * 2);
                    else qo = qf[r][m];
                    s[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qo, s[r], 0, 0, 0);
                }
                if (!SB && have_n && m < NLD) fetch_round(ksn, kn, tn, m);
            }
        } else if constexpr (KT == P1A_KV_Q4_0) {   // 8 blocks of 18 B: f16 scale, then 16 nibble bytes (2-byte aligned)
            // nibble bytes 4 g .. 4 g + 3 of block b sit at 18 b + 2 + 4 g: a whole dword in odd blocks, the upper and
            // lower halves of two neighbouring dwords in even ones (head rows start 16-byte aligned). The reads of block
            // b + 1 are asked for before block b is expanded, so that an LDS round trip hides behind the expansion.
            struct kraw { uint32_t d16, w0, w1; };
            auto kread = [&](int b) {
                kraw r;
                r.d16 = *reinterpret_cast<const uint16_t *>(krow + 18 * b);
                if (b & 1) { r.w0 = *reinterpret_cast<const uint32_t *>(krow + 18 * b + 2 + 4 * g); r.w1 = 0; }   // (b is a constant once unrolled)
                else { const uint32_t * pw = reinterpret_cast<const uint32_t *>(krow + 18 * b + 4 * g); r.w0 = pw[0]; r.w1 = pw[1]; }
                return r;
            };
            kraw kcur = kread(0);
#pragma unroll
            for (int b = 0; b < C::NMF; ++b) {
                kraw knxt = kcur;
                if (b + 1 < C::NMF) knxt = kread(b + 1);
                const uint32_t d16 = kcur.d16;
                const uint32_t w = (b & 1) ? kcur.w0 : __builtin_amdgcn_alignbit(kcur.w1, kcur.w0, 16);
                const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
                const u2 lo = deq4n(w & 0x0f0f0f0fu, dd), hi = deq4n((w >> 4) & 0x0f0f0f0fu, dd);
                const u4 a = {lo.lo, lo.hi, hi.lo, hi.hi};
#pragma unroll
                for (int r = 0; r < NT; ++r) {
                    h8 qo;
                    if constexpr (QLDS) {
                        const h4 x = *reinterpret_cast<const h4 *>(qrow[r] + (32 * b + 4 * g) * 2), y = *reinterpret_cast<const h4 *>(qrow[r] + (32 * b + 16 + 4 * g) * 2);
                        qo = h8{x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]};
                    } else qo = qf[r][b];
                    s[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a), qo, s[r], 0, 0, 0);
                }
                if (!SB && have_n && b < NLD) fetch_round(ksn, kn, tn, b);
                kcur = knxt;
            }
        } else {   // q8_0: 16 B of scales, then 16 chunks of 16 codes
            const i4 sc = *reinterpret_cast<const i4 *>(krow);
            i4 wcur = *reinterpret_cast<const i4 *>(krow + 16 + g * 16);
#pragma unroll
            for (int jj = 0; jj < C::NMF / 2; ++jj) {
                const i4 w = wcur;
                if (jj + 1 < C::NMF / 2) wcur = *reinterpret_cast<const i4 *>(krow + 16 + (4 * (jj + 1) + g) * 16);
                const uint32_t sw = (uint32_t) sc[jj];
                const uint32_t d16 = (g & 2) ? (sw >> 16) : (sw & 0xffffu);
                const h2 dd = __builtin_bit_cast(h2, d16 | (d16 << 16));
                const u2 x0 = deq4((uint32_t) w[0], dd, dd), x1 = deq4((uint32_t) w[1], dd, dd);
                const u2 x2 = deq4((uint32_t) w[2], dd, dd), x3 = deq4((uint32_t) w[3], dd, dd);
                const u4 a0 = {x0.lo, x0.hi, x1.lo, x1.hi}, a1 = {x2.lo, x2.hi, x3.lo, x3.hi};
#pragma unroll
                for (int r = 0; r < NT; ++r) {
                    h8 q0, q1;
                    if constexpr (QLDS) {   // operands 2 jj and 2 jj + 1 of column 16 r + c: 16 consecutive halves of its table row
                        const char * qr = qrow[r] + 32 * (4 * jj + g);
                        q0 = *reinterpret_cast<const h8 *>(qr);
                        q1 = *reinterpret_cast<const h8 *>(qr + 16);
                    } else { q0 = qf[r][2 * jj]; q1 = qf[r][2 * jj + 1]; }
                    s[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a0), q0, s[r], 0, 0, 0);
                    s[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, a1), q1, s[r], 0, 0, 0);
                }
                if (!SB && have_n && jj < NLD) fetch_round(ksn, kn, tn, jj);
            }
        }
        if (!SB && have_n) {   // the rounds the product loop had no place for
#pragma unroll
            for (int rd = (KT == P1A_KV_Q8_0 ? C::NMF / 2 : C::NMF); rd < NLD; ++rd) fetch_round(ksn, kn, tn, rd);
        }
        if (SB && have_n) {    // the K slot is free once its last fragment has been read
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int rd = 0; rd < NLD; ++rd) fetch_round(ksn, kn, tn, rd);
        }

        // ---- online softmax (log2 domain); column = query row, this lane holds keys ts + 4 g + i ----
        h4 pb[NT];
        float alpha[NT];
        bool rescale = false;
        const bool need_mask = ts + 15 > p_min;               // only the last tiles of a sequence hold hidden keys
#pragma unroll
        for (int r = 0; r < NT; ++r) {
            float mloc = NEG_INF;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (need_mask) s[r][i] = ts + 4 * g + i <= plim[r] ? s[r][i] : NEG_INF;
                else if (plim[r] < 0) s[r][i] = NEG_INF;
                mloc = fmaxf(mloc, s[r][i]);
            }
            mloc = max_over_groups(mloc);
            // the running maximum only moves when a tile exceeds it by more than 2^RESCALE_STEP: P stays below that
            // (f16 holds it, the sums are fp32) and the accumulators are rescaled far less often
            const float mnew = mloc > m_run[r] + RESCALE_STEP ? mloc : m_run[r];
            const bool dead = mnew == NEG_INF;
            // nothing accumulated yet (m = -inf): the accumulators are zero and need no rescale
            alpha[r] = (dead || m_run[r] == NEG_INF) ? 1.0f : __builtin_amdgcn_exp2f(m_run[r] - mnew);
            m_run[r] = mnew;
            float p[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = dead ? 0.0f : __builtin_amdgcn_exp2f(s[r][i] - mnew);
            pb[r] = h4{(half_t) p[0], (half_t) p[1], (half_t) p[2], (half_t) p[3]};
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

        if (have_n) wait_vm_imm<NLD>(); else wait_vm_imm<0>();   // V of tile t has landed (only K of t + 1 is younger)
        if constexpr (STG) convert(rawv + (t & 1) * RW::RAW_B, vs);
        // ---- O^T += V^T P^T: k-slot i of lane group g is key ts + 4 g + i, the key of this lane's P value i ----
        if constexpr (KT == P1A_KV_F16) {
            const int kk = c >> 2, jq = c & 3;
            const char * vr0 = vs + (4 * g + kk) * C::HB + jq * 8;
#pragma unroll
            for (int j = 0; j < C::NDT; ++j) {
                const s4 w = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *) (vr0 + j * 32));
                const h4 a = __builtin_bit_cast(h4, w);
#pragma unroll
                for (int r = 0; r < NT; ++r) o[r][j] = __builtin_amdgcn_mfma_f32_16x16x16f16(a, pb[r], o[r][j], 0, 0, 0);
                if (!SB && have_n && j < NLD) fetch_round(vsn, vn, tn, j);
            }
            if (!SB && have_n) {   // (staged tiles can take more rounds than the loop has places)
#pragma unroll
                for (int rd = C::NDT; rd < NLD; ++rd) fetch_round(vsn, vn, tn, rd);
            }
        } else if constexpr (KT == P1A_KV_Q4_0) {
            {   // re-align: nibble bytes of block bb of a key -> va[key][bb][16] (8-byte aligned for the transposing read);
                // scales -> tab[block][key]
                const int key = lane & 15, q2 = lane >> 4;
                // block 2 q2 starts dword-aligned (its 16 nibble bytes straddle 5 dwords), block 2 q2 + 1 two bytes past a dword
                // (its nibble bytes are 4 whole dwords)
                {
                    const int bb = 2 * q2;
                    const uint32_t * pw = reinterpret_cast<const uint32_t *>(vs + key * C::HB + 18 * bb);
                    const uint32_t d0 = pw[0], d1 = pw[1], d2 = pw[2], d3 = pw[3], d4 = pw[4];
                    *reinterpret_cast<uint16_t *>(tab + bb * 32 + key * 2) = (uint16_t) d0;
                    const u4 n = {__builtin_amdgcn_alignbit(d1, d0, 16), __builtin_amdgcn_alignbit(d2, d1, 16),
                                  __builtin_amdgcn_alignbit(d3, d2, 16), __builtin_amdgcn_alignbit(d4, d3, 16)};
                    *reinterpret_cast<u4 *>(va + key * 144 + 16 * bb) = n;
                }
                {
                    const int bb = 2 * q2 + 1;
                    const char * pb_ = vs + key * C::HB + 18 * bb;
                    *reinterpret_cast<uint16_t *>(tab + bb * 32 + key * 2) = *reinterpret_cast<const uint16_t *>(pb_);
                    const uint32_t * pw = reinterpret_cast<const uint32_t *>(pb_ + 2);
                    const u4 n = {pw[0], pw[1], pw[2], pw[3]};
                    *reinterpret_cast<u4 *>(va + key * 144 + 16 * bb) = n;
                }
            }
            // one transposing read returns 8 rows: rows 0-3 = keys 4 g .. 4 g + 3, nibble bytes of block 2 p; rows 4-7 =
            // the same keys, block 2 p + 1. Low nibbles are dims 32 b + c, high nibbles dims 32 b + 16 + c.
            const int kk = c >> 1, jb = c & 1;
            const char * vrow = va + (4 * g + (kk & 3)) * 144 + 16 * (kk >> 2) + 8 * jb;
            i2 wvc = __builtin_amdgcn_ds_read_tr8_b64_v2i32((i2 __attribute__((address_space(3))) *) vrow);
            h4 dvc[2] = {*reinterpret_cast<const h4 *>(tab + g * 8), *reinterpret_cast<const h4 *>(tab + 32 + g * 8)};
#pragma unroll
            for (int p = 0; p < C::NMF / 2; ++p) {
                const i2 w = wvc;
                const h4 dvp[2] = {dvc[0], dvc[1]};
                if (p + 1 < C::NMF / 2) {
                    wvc = __builtin_amdgcn_ds_read_tr8_b64_v2i32((i2 __attribute__((address_space(3))) *) (vrow + (p + 1) * 32));
                    dvc[0] = *reinterpret_cast<const h4 *>(tab + (2 * p + 2) * 32 + g * 8);
                    dvc[1] = *reinterpret_cast<const h4 *>(tab + (2 * p + 3) * 32 + g * 8);
                }
#pragma unroll
                for (int x = 0; x < 2; ++x) {
                    const int b = 2 * p + x;
                    const h4 dv = dvp[x];
                    const uint32_t wx = (uint32_t) w[x];
                    const u2 lo = deq4n2(wx & 0x0f0f0f0fu, h2{dv[0], dv[1]}, h2{dv[2], dv[3]});
                    const u2 hi = deq4n2((wx >> 4) & 0x0f0f0f0fu, h2{dv[0], dv[1]}, h2{dv[2], dv[3]});
                    const i2 a0 = {(int) lo.lo, (int) lo.hi}, a1 = {(int) hi.lo, (int) hi.hi};
#pragma unroll
                    for (int r = 0; r < NT; ++r) {
                        o[r][2 * b] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h4, a0), pb[r], o[r][2 * b], 0, 0, 0);
                        o[r][2 * b + 1] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h4, a1), pb[r], o[r][2 * b + 1], 0, 0, 0);
                    }
                }
                if (!SB && have_n && p < NLD) fetch_round(vsn, vn, tn, p);
            }
        } else {
            {   // transposed scale table tab[block][key] (f16, 32 B per block)
                const int key = lane & 15, q2 = lane >> 4;    // this lane moves blocks 2 q2 and 2 q2 + 1 of its key
                const uint32_t sc = *reinterpret_cast<const uint32_t *>(vs + key * C::HB + 4 * q2);
                *reinterpret_cast<uint16_t *>(tab + (2 * q2) * 32 + key * 2) = (uint16_t) sc;
                *reinterpret_cast<uint16_t *>(tab + (2 * q2 + 1) * 32 + key * 2) = (uint16_t) (sc >> 16);
            }
            // one transposing read returns 8 rows: rows 0-3 = keys 4 g .. 4 g + 3 at dims 16 j .., rows 4-7 = the
            // same keys at dims 16 (j + 1) ..
            const int kk = c >> 1, jb = c & 1;
            const char * vrow = vs + (4 * g + (kk & 3)) * C::HB + 16 + 16 * (kk >> 2) + 8 * jb;
            i2 wvc = __builtin_amdgcn_ds_read_tr8_b64_v2i32((i2 __attribute__((address_space(3))) *) vrow);
            h4 dvc = *reinterpret_cast<const h4 *>(tab + g * 8);
#pragma unroll
            for (int j = 0; j < C::NDT; j += 2) {
                const i2 w = wvc;
                const h4 dv = dvc;
                if (j + 2 < C::NDT) {
                    wvc = __builtin_amdgcn_ds_read_tr8_b64_v2i32((i2 __attribute__((address_space(3))) *) (vrow + (j + 2) * 16));
                    dvc = *reinterpret_cast<const h4 *>(tab + ((j + 2) >> 1) * 32 + g * 8);
                }
                const u2 x0 = deq4((uint32_t) w[0], h2{dv[0], dv[1]}, h2{dv[2], dv[3]});
                const u2 x1 = deq4((uint32_t) w[1], h2{dv[0], dv[1]}, h2{dv[2], dv[3]});
                const i2 a0 = {(int) x0.lo, (int) x0.hi}, a1 = {(int) x1.lo, (int) x1.hi};
#pragma unroll
                for (int r = 0; r < NT; ++r) {
                    o[r][j] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h4, a0), pb[r], o[r][j], 0, 0, 0);
                    o[r][j + 1] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h4, a1), pb[r], o[r][j + 1], 0, 0, 0);
                }
                if (!SB && have_n && j / 2 < NLD) fetch_round(vsn, vn, tn, j / 2);
            }
        }
        static_assert(KT == P1A_KV_F16 || NLD <= (KT == P1A_KV_Q8_0 ? C::NDT / 2 : C::NMF / 2), "the PV loop must have room for every V load");
        if (SB && have_n) {    // the V slot likewise
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int rd = 0; rd < NLD; ++rd) fetch_round(vsn, vn, tn, rd);
        }
#pragma unroll
        for (int r = 0; r < NT; ++r) ol[r] = __builtin_amdgcn_mfma_f32_16x16x16f16(ones, pb[r], ol[r], 0, 0, 0);
    };

    for (int t = 0; tile_start(t) < n_max; t += 2) {
        step(ks0, vs0, ks1, vs1, t);
        if (tile_start(t + 1) < n_max) step(ks1, vs1, ks0, vs0, t + 1);
    }
    // ---- fold the waves of the workgroup (in wave order) and write one partial per (workgroup, head); the 16
    // columns of one MFMA tile at a time, so that a column is merged the same way whatever NT is. A wave parks its
    // accumulators in its own (now idle) slots, dim quarter k in slot array k (SB: in its share of the pool, 8 columns at
    // a time), and (m, l) in its table ----
    constexpr int QD = D / 4;                                 // dims per quarter
    constexpr int PC = SB ? 8 : 16;                           // columns parked at a time
    // (lane coordinates worked out afresh: what is derived from them here need not live in registers through the key loop)
    int tid_f = threadIdx.x;
    asm volatile("" : "+v"(tid_f));
    const int c_f = tid_f & 15, g_f = (tid_f >> 4) & 3;
    auto park = [&](int w, int k) -> float * {                // dim quarter k of wave w
        if constexpr (SB) return reinterpret_cast<float *>(pool + (4 * w + k) * PARK_B);
        else return reinterpret_cast<float *>(slots + (k * NWV + w) * SLOTX);
    };
#pragma unroll
    for (int r = 0; r < NT; ++r) {
        const int Rr = min(16, R - 16 * r);                  // live columns of this tile
        for (int h0 = 0; h0 < Rr; h0 += PC) {                // (one round unless SB)
        const int he = min(h0 + PC, Rr);
        if (r || h0 || SB) __syncthreads();                   // (SB: the pool changes hands once every wave is done with its tiles)
        if (c_f >= h0 && c_f < he) {
#pragma unroll
            for (int j = 0; j < C::NDT; ++j)
                *reinterpret_cast<f4 *>(park(wave, j / (C::NDT / 4)) + (c_f - h0) * C::QDP + 16 * (j % (C::NDT / 4)) + 4 * g_f) = o[r][j];
        }
        if (h0 == 0 && c_f < Rr && g_f == 0) {
            reinterpret_cast<float *>(tab)[c_f] = m_run[r];
            reinterpret_cast<float *>(tab)[16 + c_f] = ol[r][0];
        }
        __syncthreads();
        // LPC lanes per column: the factors of a column (one per wave; a wave that saw no visible key parked zeros and
        // gets the factor 0) are worked out once per lane and serve all the dims the lane folds. 64 lanes when the columns of
        // the round are few enough for that to keep every thread busy (a single row of 6 heads: 384 threads fold one
        // float4 each instead of 192 folding two), else 32; the sums are the same either way
        auto fold_round = [&](auto lpc_tag) {
        constexpr int LPC = decltype(lpc_tag)::value;
        for (int cc = h0 + tid_f / LPC; cc < he; cc += NWV * 64 / LPC) {
            const int dl = tid_f % LPC;
            // the parked accumulators are asked for first: they do not depend on the factors, whose table reads and
            // exponentials then run under their LDS round trip instead of in front of it
            constexpr int NIT = (D / 4 + LPC - 1) / LPC;
            f4 aw[NIT][NWV];
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                const int d4 = dl + it * LPC;
                if (D / 4 % LPC == 0 || d4 < D / 4) {
                    const int qtr = (4 * d4) / QD, dq = 4 * d4 - qtr * QD;
#pragma unroll
                    for (int w = 0; w < NWV; ++w) aw[it][w] = *reinterpret_cast<const f4 *>(park(w, qtr) + (cc - h0) * C::QDP + dq);
                }
            }
            float mw[NWV], lw[NWV], fw[NWV];
#pragma unroll
            for (int w = 0; w < NWV; ++w) {
                const float * tw = reinterpret_cast<const float *>(tabs + w * C::TAB_B);
                mw[w] = tw[cc];
                lw[w] = tw[16 + cc];
            }
            float M = NEG_INF;
#pragma unroll
            for (int w = 0; w < NWV; ++w) M = fmaxf(M, mw[w]);
            float l = 0.f;
#pragma unroll
            for (int w = 0; w < NWV; ++w) {
                fw[w] = mw[w] == NEG_INF ? 0.f : __builtin_amdgcn_exp2f(mw[w] - M);
                l += lw[w] * fw[w];
            }
            const int col = 16 * r + cc;
            const int t = row_of(col), hh = col - t * P.GQA;
            const size_t row = (size_t) (row0 + t) * P.Hq + (size_t) hg * P.GQA + hh;
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                const int d4 = dl + it * LPC;
                if (D / 4 % LPC == 0 || d4 < D / 4) {
                    f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int w = 0; w < NWV; ++w) acc += aw[it][w] * fw[w];
                    // (two column tiles = several rows per group: the partials are tens of megabytes and nothing here reads
                    // them again, so they go past the cache - measured -3 ... -5 % on 4-row verify calls, +6 % on a single row)
                    f4 * const po = reinterpret_cast<f4 *>(P.part_o + (row * P.nsplit + split) * D + 4 * d4);
                    if (M != NEG_INF) { if constexpr (NT == 2) __builtin_nontemporal_store(acc, po); else *po = acc; }
                }
            }
            if (dl == 0) {
                float * pm = P.part_ml + (row * P.nsplit + split) * 2;
                pm[0] = M;
                pm[1] = l;
            }
        }
        };
        if (SB || he - h0 <= NWV) fold_round(std::integral_constant<int, 64>{}); else fold_round(std::integral_constant<int, 32>{});
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

// ---- merge of the split partials, in a fixed order, with the fused sigmoid gate ----
// out[row][d] = sum_s 2^(m_s - M) O_s[d] / sum_s 2^(m_s - M) l_s; empty streams (m = -inf or l = 0) are skipped.
// One workgroup of 256 threads per (row, 128 dims): thread = (slice of the splits, 4 dims); slice k folds splits k, k + 8,
// ... in order and the 8 slices are then added in order, so the result depends on nothing but the partials. A wave holds
// two slices, so each of its loads covers two contiguous half-rows of 512 bytes. The (m, l) pairs are fetched once per
// wave - lane i brings the pair of split i - and handed round by lane shuffles; the maximum is a wave reduction.
// pos_rows / U (optional): row t of a batched call sits at position pos_rows[t] and its split stream s holds keys only when
// s units of U positions do not cover the sequence yet - the streams past that are known to be empty and are not fetched.
constexpr int MRG_DIMS = 128;
__global__ void __launch_bounds__(256) merge_k(const float * __restrict__ part_o, const float * __restrict__ part_ml,
                                               float * __restrict__ out, const float * __restrict__ gate, int NS_all, int D,
                                               void * qbuf, int Hq, int T, const int32_t * __restrict__ pos_rows, int U) {
    __shared__ f4 sacc[8][32];
    __shared__ float sden[8];
    const size_t row = blockIdx.x;
    const int NS_row = NS_all;                                // (the row stride of the partials)
    int NS = NS_all;
    // (a row at a negative position - an idle slot - sees no key: no stream is read, and 0 / 0 gives the NaN row the
    // reference's combine gives for n = 0)
    if (pos_rows && U > 0) { const int pr_ = pos_rows[row / Hq]; NS = pr_ < 0 ? 0 : min(NS_all, pr_ / U + 1); }
    const int tid = threadIdx.x, lane = tid & 63, qd = tid & 31, sl = tid >> 5;
    const int d = blockIdx.y * MRG_DIMS + qd * 4;
    const bool live = d < D;
    const float * ml = part_ml + row * NS_row * 2;
    constexpr int CH = 8;                                     // splits of a slice fetched together
    // the gate depends on nothing here: its load rides along with the first batch of partials
    f4 gt = {0.f, 0.f, 0.f, 0.f};
    if (gate && sl == 0 && live) gt = *reinterpret_cast<const f4 *>(gate + row * D + d);
    f4 num = {0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
    // the maximum over all splits first: batches of 64 pairs, lane i of every wave the pair of split s0 + i
    float M = NEG_INF;
    float2 pr = make_float2(NEG_INF, 0.f);                    // the pair of split `lane` of the first batch
    if (lane < NS) pr = *reinterpret_cast<const float2 *>(ml + 2 * lane);
    // the first batch of partials (all of them when NS <= 64) is requested before anything is known about the maximum
    f4 a[CH];
#pragma unroll
    for (int k = 0; k < CH; ++k) {
        const int s = sl + 8 * k;
        a[k] = f4{0.f, 0.f, 0.f, 0.f};
        if (s < NS && live) a[k] = *reinterpret_cast<const f4 *>(part_o + (row * NS_row + s) * D + d);
    }
    M = pr.x;
    for (int s0 = 64; s0 < NS; s0 += 64) if (s0 + lane < NS) M = fmaxf(M, ml[2 * (s0 + lane)]);
    M = wave_max(M);
    for (int s0 = 0; s0 < NS; s0 += 8 * CH) {
        if (s0) {
            pr = make_float2(NEG_INF, 0.f);
            if (s0 + lane < NS) pr = *reinterpret_cast<const float2 *>(ml + 2 * (s0 + lane));
#pragma unroll
            for (int k = 0; k < CH; ++k) {
                const int s = s0 + sl + 8 * k;
                if (s < NS && live) a[k] = *reinterpret_cast<const f4 *>(part_o + (row * NS_row + s) * D + d);
            }
        }
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            const float msk = __shfl(pr.x, sl + 8 * k), lsk = __shfl(pr.y, sl + 8 * k);
            if (msk == NEG_INF || lsk == 0.f) continue;       // empty stream: its accumulator was never written
            const float f = __builtin_amdgcn_exp2f(msk - M);
            den = fmaf(f, lsk, den);
            num[0] = fmaf(f, a[k][0], num[0]); num[1] = fmaf(f, a[k][1], num[1]);
            num[2] = fmaf(f, a[k][2], num[2]); num[3] = fmaf(f, a[k][3], num[3]);
        }
    }
    sacc[sl][qd] = num;
    if (qd == 0) sden[sl] = den;
    __syncthreads();
    if (sl == 0) {
        f4 n = sacc[0][qd];
        float dn = sden[0];
#pragma unroll
        for (int k = 1; k < 8; ++k) { n += sacc[k][qd]; dn += sden[k]; }
        f4 r = {n[0] / dn, n[1] / dn, n[2] / dn, n[3] / dn};
        if (gate) {
#pragma unroll
            for (int x = 0; x < 4; ++x) r[x] *= 1.0f / (1.0f + expf(-gt[x]));
        }
        if (live) *reinterpret_cast<f4 *>(out + row * D + d) = r;
        // 8 consecutive lanes of slice 0 hold one 32-value group of the output row: its a16 activation quantize rides
        // along (what the engine's ew_quant emits for the output projection, src/fast/fused.cu:478-496)
        if (qbuf) {
            const int t = (int) (row / Hq), h = (int) (row - (size_t) t * Hq);
            a16_quant8(r, qd & 7, qbuf, t, h * (D >> 5) + (d >> 5), (Hq * D) >> 5, T, live);
        }
    }
}

__global__ void __launch_bounds__(256) sigmoid_mul_k(float * __restrict__ x, const float * __restrict__ g, size_t n) {
    for (size_t i = (size_t) blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t) gridDim.x * 256)
        x[i] *= 1.0f / (1.0f + expf(-g[i]));
}

// ---- launch plan: which kernel a shape takes, and how the keys are split ----
// The MFMA kernel needs 16-byte aligned head rows (f16: D in {64, 128, 256}; q8_0 / q4_0: D == 256), 16-byte aligned
// bases and strides, pages of >= 16 positions and GQA <= 16; q8_0 / q4_0 at D = 64 or 128 (head rows of whole dwords)
// take its staged build, which fetches 4 bytes per lane and only needs 4-byte alignment. Everything else takes the
// generic kernel.
struct dec_plan {
    bool mfma;
    int GQA, NW, NT, RG;
    int nsplit;    // split streams
    int NS;        // partials per output row (what merge_k folds)
};

bool mfma_ok(const p1a_kv & c, int GQA) {
    if (GQA < 1 || GQA > 16) return false;
    if (c.D != 64 && c.D != 128 && c.D != 256) return false;
    const bool staged = c.type != P1A_KV_F16 && c.D != 256;   // q8_0 / q4_0 head rows are whole 16-byte chunks only at D = 256
    const uintptr_t al = staged ? 3 : 15;
    if (((uintptr_t) c.k | (uintptr_t) c.v) & al) return false;
    if (c.pt && ((c.pstride & al) || c.psh < 4)) return false;
    return true;
}

dec_plan make_plan(const p1a_kv & c, int Hq, int rows_per_group, int nsplit_req, int cus) {
    dec_plan p;
    p.GQA = Hq / c.Hkv;
    p.mfma = mfma_ok(c, p.GQA);
    if (!p.mfma) {
        p.NW = 4; p.NT = 1;
        p.RG = rows_per_group < 1 ? 1 : rows_per_group;   // no sharing here: the group only selects the page table
        int n = nsplit_req > 0 ? nsplit_req : 2 * cus / Hq;
        p.nsplit = n < 1 ? 1 : (n > 1024 ? 1024 : n);
        p.NS = p.nsplit * 4;
        return p;
    }
    const int cap = 32 / p.GQA < 4 ? 32 / p.GQA : 4;
    p.RG = rows_per_group < 1 ? 1 : (rows_per_group > cap ? cap : rows_per_group);
    // One kv head per workgroup: its waves fold into ONE partial, which keeps the split traffic at a few percent of the KV
    // bytes; the heads of a split stream are placed on one XCD so shared cache lines meet in its L2.
    const bool big_tiles = c.type == P1A_KV_F16 && c.D == 256;   // 34 KB of LDS per wave
    p.NW = big_tiles ? 4 : 8;
    const int HG = c.Hkv;
    // (one workgroup per CU for every variant: the four-wave one keeps 128 KB of f16 tiles in LDS; measured for f16 at
    // 32 K: 64 streams 27.2 us, 128 streams - two rounds of workgroups - 30.2 us)
    int n = nsplit_req > 0 ? nsplit_req : cus / HG;
    if (n >= 8) n &= ~7;
    p.nsplit = n < 1 ? 1 : (n > 1024 ? 1024 : n);
    return p;
}

void finish_plan(dec_plan & p) {
    p.NT = p.RG * p.GQA <= 16 ? 1 : 2;
    if (p.mfma) p.NS = p.nsplit;
}

template <uint32_t KT, int D, uint32_t KS = KT>
int launch_mfma(const p1a_kv & c, const decode_args & a, const dec_plan & pl, hipStream_t s) {
    dec_params P;
    P.q = a.q; P.kc = (const char *) c.k; P.vc = (const char *) c.v;
    P.part_o = a.part_o; P.part_ml = a.part_ml; P.pg = view_of(c);
    P.p0 = a.p0; P.p0_dev = a.p0_dev; P.pos_rows = a.pos_rows;
    P.T = a.T; P.RG = pl.RG; P.Hq = a.Hq; P.Hkv = c.Hkv; P.GQA = pl.GQA;
    P.qscale = a.scale * 1.4426950408889634f; P.nsplit = pl.nsplit;
    P.hkv_sh = -1;
    for (int sh = 0; sh < 16; ++sh) if ((1 << sh) == c.Hkv) P.hkv_sh = sh;
    P.npt = c.pt ? (int) (((long long) c.n_ctx + (1LL << c.psh) - 1) >> c.psh) : 0;
    constexpr bool big_tiles = KT == P1A_KV_F16 && D == 256;
    // A call of at least two workgroups per CU whose row groups fit one column tile takes the single-buffered variant, two
    // workgroups to a CU (same partials, bit for bit; measured at 24 / 4 heads, D = 256: 8 q8_0 slots of 1 K ... 27 K 56 ->
    // 47 us, 4 x 64 K q4_0 single rows 92 -> 73 us, 16 x 2 rows q4_0 at 16 K 143 -> 115 us, 32 slots of 2 ... 5 K 104 -> 71 us).
    // (A workgroup walks ONE split stream whatever the call: letting it walk several in turn - fewer, longer workgroups
    // for calls of many - measured slower on every shape tried, e.g. 8 x 4 rows q4_0 at 8 K 72 -> 60 us with one.)
    const long long wgs_all = (long long) pl.nsplit * c.Hkv * ((a.T + pl.RG - 1) / pl.RG);
    const bool sb = KS == KT && pl.NT == 1 && wgs_all >= 2LL * (a.cus > 0 ? a.cus : 256);
    const dim3 grid(pl.nsplit * c.Hkv, (a.T + pl.RG - 1) / pl.RG);
#define P1A_DEC(NT_, NW_) dec_mfma_k<KT, D, NT_, NW_, false, KS><<<grid, NW_ * 64, 0, s>>>(P)
    if constexpr (KS != KT) {
        if (pl.NT == 1) P1A_DEC(1, 8);
        else P1A_DEC(2, 8);
    } else if constexpr (big_tiles) {
        if (sb) dec_mfma_k<KT, D, 1, 4, true><<<grid, 256, 0, s>>>(P);
        else if (pl.NT == 1) P1A_DEC(1, 4);
        else P1A_DEC(2, 4);
    } else {
        if (sb) dec_mfma_k<KT, D, 1, 8, true><<<grid, 512, 0, s>>>(P);
        else if (pl.NT == 1) P1A_DEC(1, 8);
        else P1A_DEC(2, 8);
    }
#undef P1A_DEC
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
    // the partials of this launch: [T * Hq][NS][D] accumulators and [T * Hq][NS][2] (m, l) pairs
    const size_t need_o = (size_t) a.T * a.Hq * pl.NS * c.D * sizeof(float), need_ml = (size_t) a.T * a.Hq * pl.NS * 2 * sizeof(float);
    if (need_o > a.cap_o || need_ml > a.cap_ml) {
        set_error("p1a_attn_decode: split partials of %zu + %zu bytes do not fit the scratch of %zu + %zu", need_o, need_ml, a.cap_o, a.cap_ml);
        return P1A_E_SCRATCH;
    }
    int rc;
    if (pl.mfma) {
        if (c.type == P1A_KV_Q8_0 && c.D == 256) rc = launch_mfma<P1A_KV_Q8_0, 256>(c, a, pl, s);
        else if (c.type == P1A_KV_Q4_0 && c.D == 256) rc = launch_mfma<P1A_KV_Q4_0, 256>(c, a, pl, s);
        else if (c.type == P1A_KV_Q8_0 && c.D == 128) rc = launch_mfma<P1A_KV_F16, 128, P1A_KV_Q8_0>(c, a, pl, s);
        else if (c.type == P1A_KV_Q8_0) rc = launch_mfma<P1A_KV_F16, 64, P1A_KV_Q8_0>(c, a, pl, s);
        else if (c.type == P1A_KV_Q4_0 && c.D == 128) rc = launch_mfma<P1A_KV_F16, 128, P1A_KV_Q4_0>(c, a, pl, s);
        else if (c.type == P1A_KV_Q4_0) rc = launch_mfma<P1A_KV_F16, 64, P1A_KV_Q4_0>(c, a, pl, s);
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
    if (rc != P1A_OK || a.skip_merge) return rc;
    merge_k<<<dim3(a.T * a.Hq, (c.D + MRG_DIMS - 1) / MRG_DIMS), 256, 0, s>>>(a.part_o, a.part_ml, a.out, a.gate, pl.NS, c.D, a.qbuf, a.Hq, a.T,
                                                       pl.mfma ? a.pos_rows : nullptr, 32 * pl.NW);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

int launch_merge(const float * part_o, const float * part_ml, float * out, const float * gate, int NS, int D, int Hq, int T, hipStream_t s) {
    merge_k<<<dim3((unsigned) T * Hq, (D + MRG_DIMS - 1) / MRG_DIMS), 256, 0, s>>>(part_o, part_ml, out, gate, NS, D, nullptr, Hq, T, nullptr, 0);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}


// Benchmarks only: a plain streaming read. Workgroup b reads one contiguous span, every lane 16 bytes at a time with four
// loads in flight, four workgroups of 512 threads per compute unit (measured on a 71 MB read inside a graph: 13.4 us
// with one workgroup per unit, 11.5 with two, 11.25 with four; deeper per-lane queues instead of more waves do worse);
// the sum is kept so that the loads cannot be dropped, and stored nowhere (it never equals the sentinel for the inputs a
// benchmark uses; one float of static device memory takes it if it ever does).
__device__ float g_stream_read_sink;
__global__ void __launch_bounds__(512) stream_read_k(const f4 * __restrict__ p, size_t n16) {
    const size_t per = n16 / gridDim.x;
    const f4 * b = p + per * blockIdx.x;
    const size_t n = blockIdx.x + 1 == gridDim.x ? n16 - per * blockIdx.x : per;
    f4 acc = {0.f, 0.f, 0.f, 0.f};
    size_t i = threadIdx.x;
    for (; i + 3 * 512 < n; i += 4 * 512) {
        const f4 v0 = __builtin_nontemporal_load(b + i), v1 = __builtin_nontemporal_load(b + i + 512);
        const f4 v2 = __builtin_nontemporal_load(b + i + 1024), v3 = __builtin_nontemporal_load(b + i + 1536);
        acc += (v0 + v1) + (v2 + v3);
    }
    for (; i < n; i += 512) acc += __builtin_nontemporal_load(b + i);
    if (acc[0] + acc[1] + acc[2] + acc[3] == -1.2345678e38f) g_stream_read_sink = acc[0];
}

int launch_stream_read(const void * src, size_t bytes, hipStream_t s) {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void) hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    stream_read_k<<<4 * (cus > 0 ? cus : 256), 512, 0, s>>>(reinterpret_cast<const f4 *>(src), bytes / 16);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

int launch_sigmoid_mul(float * x, const float * g, size_t n, hipStream_t s) {
    const size_t nb = (n + 255) / 256;
    sigmoid_mul_k<<<(unsigned) (nb > 4096 ? 4096 : (nb ? nb : 1)), 256, 0, s>>>(x, g, n);
    return hipPeekAtLastError() == hipSuccess ? P1A_OK : P1A_E_LAUNCH;
}

}   // namespace p1a
