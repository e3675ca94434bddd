"""The package's own kernel modules: source name, entry points with their argument types, the variants
built ahead of time and extra compiler flags.  Registered with the loader on import; a part that brings a
kernel of its own registers it the same way (library.register_kernel_module)."""
from ctypes import c_float, c_int, c_long, c_void_p

from .library import register_kernel_module
from .variants import HEAD_DIMS

P, I, L, F = c_void_p, c_int, c_long, c_float
_head_variants = [(f"-DHEAD_DIM={d}",) for d in HEAD_DIMS]

register_kernel_module("embed_norm", {
    "mie_embedding": [P, P, I, P, I, I, I, P, P, P],
    "mie_add_rmsnorm": [P, I, P, P, I, P, I, P, I, I, F, P],
})
register_kernel_module("rope_kv", {
    "mie_rotary_kv_store": [P, I, L, P, P, P, I, I, I, I, P, P, P, I, I, P],
    "mie_rotary_kv_store_sums": [P, L, P, L, P, P, P, P, P, P, I, I, I, I, I, P],
})
register_kernel_module("gemm", {
    "mie_gemm_nt": [P, I, L, P, I, L, P, I, L, P, I, I, I, P],
    "mie_silu_mul": [P, L, P, L, I, I, I, P],
})
register_kernel_module("attention", {
    "mie_paged_attention": [P, L, P, P, P, I, P, I, P, P, I, I, I, I, I, F, I, P],
})
register_kernel_module("sampling", {
    "mie_sample": [P, L, P, P, P, P, I, I, P],
})
register_kernel_module("gemm_bf16", {
    "mie_skinny_gemm": [P, L, P, L, P, L, I, I, I, I, P, I, P, L, P, P, I, F, P, P],
    "mie_skinny_qkv_rope": [P, L, P, L, P, L, P, P, P, P, P, P, I, I, I, I, I, I, P, I, F, P],
    "mie_skinny_max_rows": [],
})
register_kernel_module("gemm_mid_bf16", {
    "mie_mid_gemm": [P, L, P, L, P, I, I, I, I, P, P],
    "mie_mid_reduce": [P, I, I, I, I, P, L, P, P, I, P, L, F, P],
    "mie_mid_reduce_rope_kv": [P, I, I, P, L, P, P, P, P, P, P, I, I, I, I, P],
    "mie_mid_splits": [I, I],
    "mie_mid_max_rows": [],
})
register_kernel_module("attention_bf16", {
    "mie_decode_attention": [P, L, P, P, P, P, P, P, I, P, I, I, I, I, I, F, I, I, I, P],
    "mie_decode_attention_from_sums": [P, I, L, L, P, P, P, P, P, P, P, I, P, I, I, I, I, I, F, I, I, P],
    "mie_decode_attention_static": [P, L, P, P, P, P, I, P, I, I, I, I, I, F, I, I, I, P],
    "mie_decode_attention_static_setup": [],
    "mie_decode_block_keys": [],
    "mie_attention_bf16_head_dim": [],
}, variants=_head_variants)
# prefill_attention_bf16: matrix instructions keep their accumulators in ordinary vector registers; otherwise
# the compiler parks the outputs in accumulation registers and copies all of them back and forth around
# every key block for the sake of the (rare) rescaling.
register_kernel_module("prefill_attention_bf16", {
    "mie_prefill_attention": [P, L, P, P, P, P, I, P, P, I, I, I, I, I, I, I, F, I, P],
}, variants=_head_variants, flags=["-mllvm", "-amdgpu-mfma-vgpr-form"])
# lt_gemm: host code only, the engine's own way into the library's matrix products (hipBLASLt) with the choice of
# kernel per shape kept here.
register_kernel_module("lt_gemm", {
    "mie_lt_gemm": [P, L, P, L, P, L, I, I, I, I, P, L, P],
    "mie_lt_is_tuned": [L, L, L, I, I, I, I],
    "mie_lt_tune": [P, L, P, L, P, L, I, I, I, I, P, L, I, I, P, L, P, P, P],
}, flags=["-L/opt/rocm/lib", "-lhipblaslt", "-Wl,-rpath,/opt/rocm/lib"])
# stream_read: a measurement for bench.py (the rate at which memory that is only read streams in); no model uses it.
register_kernel_module("stream_read", {
    "mie_stream_read": [P, L, P, I, I, P],
})
