// Shared device/host helpers of the gfx950 paged-KV attention library (internal header).
#pragma once
#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>
#include "p1a_attn.h"

namespace p1a {

typedef _Float16 half_t;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16x __attribute__((ext_vector_type(16)));
typedef int i2 __attribute__((ext_vector_type(2)));
typedef int i4 __attribute__((ext_vector_type(4)));
typedef short s4 __attribute__((ext_vector_type(4)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));

// Paged addressing: the device twin of the reference's kv_pg helpers (src/fast/kv_page.cuh:11-31), with 64-bit
// page bases throughout.
struct kv_view {
    const int32_t * pt;     // page table(s); nullptr = contiguous
    const int32_t * rtab;   // per-row element offsets into pt; nullptr = 0
    int psh;
    size_t pstride;
    size_t rowb;            // bytes of one position (all kv heads)
};

inline kv_view view_of(const p1a_kv & c) {
    return kv_view{c.pt, c.rtab, c.psh, c.pstride, p1a_kv_row_bytes(c.type, c.Hkv, c.D)};
}

__device__ __forceinline__ const int32_t * kv_tab(const kv_view & g, int t) {
    return g.pt ? (g.rtab ? g.pt + g.rtab[t] : g.pt) : nullptr;
}
__device__ __forceinline__ size_t kv_off_tab(const kv_view & g, const int32_t * tab, int p) {
    if (!tab) return (size_t) p * g.rowb;
    return (size_t) tab[p >> g.psh] * g.pstride + (size_t) (p & ((1 << g.psh) - 1)) * g.rowb;
}

constexpr size_t head_bytes(uint32_t type, int D) {
    return type == P1A_KV_F16 ? (size_t) D * 2 : type == P1A_KV_Q8_0 ? (size_t) (D / 32) * 34 : (size_t) (D / 32) * 18;
}

// ---- a16 activation quantize of one 32-value group (src/fast/a16q.cuh:21-45 of the reference) ----
// Lane l8 (0..7) of an aligned 8-lane segment holds values 4 l8 .. 4 l8 + 3 of the group; all 8 lanes call together.
// qbuf layout: half2 words; word (t * ng + g) * 16 + slot = two scaled values (slot order of the engine), word
// T * ng * 16 + t * ng + g = (amax, sum of the scaled values). Products and sums are rounded one by one (no contraction),
// the sum runs over a lane's 4 values in order from +0 and then over the lanes in an xor butterfly with strides 4, 2, 1.
#if defined(__HIPCC__)
// v_permlane16_swap / v_permlane32_swap exchange the odd 16-lane rows (the upper 32 lanes) of the first register with the
// even rows (the lower 32 lanes) of the second; BOTH registers are results. They are issued through inline assembly: the
// compiler's builtin for them hands back its first result twice (the second register - the other half of the exchange -
// is dropped), so a maximum built on it silently kept the even rows' / lower lanes' value only. The instruction needs two
// wait states after a vector write of either operand, which the compiler does not know to insert around assembly; the maximum of the two results rides in the same block.
__device__ __forceinline__ float max_swap16(float m) {
    float a = m, b = m;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 0\n\tv_max_f32 %0, %0, %1" : "+v"(a), "+v"(b));
    return a;
}
__device__ __forceinline__ float max_swap32(float m) {
    float a = m, b = m;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 0\n\tv_max_f32 %0, %0, %1" : "+v"(a), "+v"(b));
    return a;
}
// the maximum over all 64 lanes, in every lane: four steps inside a row of 16 lanes on the data-parallel-primitive path
// (lane ^ 1, lane ^ 2, mirrored halves of 8, mirrored row - no LDS round trip), then the four rows by the two swaps
template <int CTRL> __device__ __forceinline__ float max_dpp(float x) {
    const int xi = __builtin_bit_cast(int, x);
    return fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(xi, xi, CTRL, 0xf, 0xf, false)));
}
__device__ __forceinline__ float wave_max(float x) {
    x = max_dpp<0xB1>(x);     // quad_perm [1, 0, 3, 2]
    x = max_dpp<0x4E>(x);     // quad_perm [2, 3, 0, 1]
    x = max_dpp<0x141>(x);    // row_half_mirror
    x = max_dpp<0x140>(x);    // row_mirror
    return max_swap32(max_swap16(x));
}
__device__ __forceinline__ void a16_quant8(const f4 v4, int l8, void * qbuf, int t, int g, int ng, int T, bool store) {
#pragma clang fp contract(off)
    float v[4] = {v4[0], v4[1], v4[2], v4[3]};
    float amax = fmaxf(0.0f, fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
#pragma unroll
    for (int st = 4; st > 0; st >>= 1) amax = fmaxf(amax, __shfl_xor(amax, st));
    amax = amax < 65520.0f ? amax : 65504.0f;               // a finite f16 scale
    const float id = amax > 0.0f ? 1.0f / amax : 0.0f;
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[i] = v[i] * id;
        sum = sum + v[i];
    }
#pragma unroll
    for (int st = 4; st > 0; st >>= 1) sum = sum + __shfl_xor(sum, st);
    if (!store) return;
    h2 * qs = reinterpret_cast<h2 *>(qbuf) + ((size_t) t * ng + g) * 16;
    if (l8 == 0) reinterpret_cast<h2 *>(qbuf)[(size_t) T * ng * 16 + (size_t) t * ng + g] = h2{(half_t) amax, (half_t) sum};
    const int off = l8 >= 4 ? 1 : 0, k = l8 - 4 * off;
    qs[4 * k + 0 + off] = h2{(half_t) v[0], (half_t) v[2]};
    qs[4 * k + 2 + off] = h2{(half_t) v[1], (half_t) v[3]};
}
#endif

// host-side launch entry points implemented in the .hip files
int launch_append(const p1a_kv & c, const float * k, const float * v, int p0, const int32_t * p0_dev,
                  const int32_t * pos_rows, int T, hipStream_t s);

int launch_fill_random(const p1a_kv & c, int p0, int p1, uint32_t seed, hipStream_t s);

struct decode_args {
    const float * q;
    float * out;
    const float * gate;
    int T, p0;
    const int32_t * p0_dev;
    const int32_t * pos_rows;
    int rows_per_group;   // rows sharing one KV read
    int Hq;
    float scale;
    int nsplit;           // requested split streams (0 = default for the device)
    int cus;              // compute units of the device
    bool skip_merge;      // benchmarks only: stop after the split-K kernel
    float * part_o;       // [T*Hq][nsplit][D]
    float * part_ml;      // [T*Hq][nsplit][2]
    size_t cap_o, cap_ml; // bytes behind part_o / part_ml (a launch that would write past them is refused)
    void * qbuf;          // optional: a16 activation buffer of the (gated) output, [T][Hq*D] values
};
int launch_decode(const p1a_kv & c, const decode_args & a, hipStream_t s);
int decode_rows_per_group(const p1a_kv & c, int Hq, int want);
int decode_nsplit(const p1a_kv & c, int Hq, int nsplit_req, int cus);
void decode_scratch_need(const p1a_kv & c, int Hq, int rows, int rows_per_group, int nsplit_req, int cus,
                         size_t & bytes_o, size_t & bytes_ml);
// interleaved M-RoPE positions of a batch (src/fast/mrope.cuh:14-19): [3][stride] t / h / w, sections in rotary pairs
struct mrope_view { const int32_t * p; int stride, s0, s1, s2, sect; };
int launch_prep(const p1a_kv & c, const float * qg, const float * k, const float * v, const float * q_norm, const float * k_norm,
                const int32_t * pos, float * q, float * gate, int p0, int T, int Hq, int n_rot, float freq_base, float eps,
                int ldq, int ldk, int ldv, const mrope_view & mr, hipStream_t s);
int launch_ew_quant(int op, const float * a, const float * b, float * y, void * qbuf, int T, int n, int lda, int ldb, hipStream_t s);
int launch_prefill(const p1a_kv & c, const float * q, float * out, const float * gate, int T, int p0, int Hq,
                   float scale, void * scratch, size_t scratch_bytes, hipStream_t s);
// fold of split partials [rows][NS][D] + (m, l) [rows][NS][2] into out [rows][D] (rows = T * Hq), sigmoid gate fused
int launch_merge(const float * part_o, const float * part_ml, float * out, const float * gate, int NS, int D, int Hq, int T, hipStream_t s);
// the library's own buffers for the partials of a key-split prefill on (current device, stream), at least these sizes;
// false (error set) when that is not possible now, e.g. the stream is being captured and they would have to be allocated
bool split_scratch(hipStream_t s, size_t bytes_o, size_t bytes_ml, float *& o, float *& ml);
// the library's own f16 staging copy of (current device, stream) for a prefill over a quantized cache (nullptr: none now)
void * stage_scratch(hipStream_t s, size_t bytes);
size_t prefill_stage_bytes(int n, int Hkv, int D);
// bytes of partials a key-split prefill of this shape needs on the current device (0, 0 = one split)
void prefill_part_need(int T, int p0, int Hq, int D, size_t & bytes_o, size_t & bytes_ml);
int cu_count();   // compute units of the current device
int launch_sigmoid_mul(float * x, const float * g, size_t n, hipStream_t s);
int launch_stream_read(const void * src, size_t bytes, hipStream_t s);   // benchmarks only

void set_error(const char * fmt, ...);

}   // namespace p1a
