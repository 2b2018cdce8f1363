// placeholder until the MFMA prefill kernel lands
#include "p1a_common.hpp"
namespace p1a {
int launch_prefill(const p1a_kv &, const float *, float *, const float *, int, int, int, float, void *, size_t, hipStream_t) {
    set_error("p1a_attn_prefill: not built");
    return P1A_E_SHAPE;
}
}
extern "C" size_t p1a_attn_prefill_scratch_bytes(int, int, int, int, int) { return 0; }
