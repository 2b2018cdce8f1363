"""MI355X (gfx950) paged-KV attention path of the qwen35 full-attention layers.

The product is the C-ABI shared library ``libp1a_attn.so`` (sources in ``csrc/``, declarations in
``include/p1a_attn.h``) and its C++ mirror of the reference surface (``include/p100e_fast_attn.hpp``).
This Python package is only the ctypes binding the tests, the smoke check and the benchmark use to drive that
library with torch tensors as device memory. It never computes anything itself: if the library is missing or a
call is refused, it raises.
"""
from .binding import (  # noqa: F401
    KV_F16, KV_Q4_0, KV_Q8_0, KVCache, P1AError, attn_prep, a16_bytes, ew_quant, attn_decode, attn_decode_dev, attn_decode_rows, attn_prefill,
    get_nsplit, kv_append, kv_append_dev, kv_append_rows, kv_fill_random, kv_row_bytes, lib, lib_path, prefill_scratch_bytes, prefill_key_splits,
    set_nsplit, sigmoid_mul, warmup, reload_env, decode_scratch_bytes, decode_footprint_bytes, numerics_id, warmup_prefill, set_prefill_staging_limit, bench_decode_split_only, bench_stream_read, EXPORTS, Pool, verify_accept, p1a_kv,
)
