"""The package's own kernel modules: source name, entry points with their argument types, the variants
built ahead of time and extra compiler flags.  Registered with the loader on import; a part that brings a
kernel of its own registers it the same way (library.register_kernel_module)."""
from ctypes import c_float, c_int, c_long, c_void_p

from .library import register_kernel_module
from .variants import HEAD_DIMS

P, I, L, F = c_void_p, c_int, c_long, c_float
_head_variants = [(f"-DHEAD_DIM={d}",) for d in HEAD_DIMS]

register_kernel_module("embed_norm", {
    "mie_embedding": [P, P, I, P, I, I, I, P, P, F, P],
    "mie_add_rmsnorm": [P, I, P, P, I, P, I, P, I, I, F, P],
    "mie_branch_norm_add": [P, I, P, P, I, P, I, I, I, F, P],
    "mie_rmsnorm_columns": [P, L, P, I, P, I, I, I, F, P],
    "mie_scale": [P, L, F, P],
    "mie_normed_sum_add": [P, P, P, P, P, I, I, F, F, P],
    "mie_norm_pair_conv": [P, P, P, P, P, P, P, P, P, P, I, P, I, I, I, I, F, P],
    "mie_branch_norm_conv_single": [P, P, P, F, P, P, P, P, P, I, I, I, I, F, P],
})
register_kernel_module("layer_norm", {
    "mie_add_layernorm": [P, I, P, P, P, P, I, P, I, I, F, P],
    "mie_branch_layernorm_add": [P, I, P, P, P, F, P, P, F, P, I, I, I, P],
    "mie_scale_softcap": [P, L, F, F, P],
})
register_kernel_module("rope_kv", {
    "mie_rotary_kv_store": [P, I, L, P, P, P, I, I, I, I, P, P, P, I, I, P],
    "mie_rotary_kv_store_sums": [P, L, P, L, P, P, P, P, P, P, I, I, I, I, I, P],
})
register_kernel_module("gemm", {
    "mie_gemm_nt": [P, I, L, P, I, L, P, I, L, P, I, I, I, P],
    "mie_silu_mul": [P, L, P, L, I, I, I, P],
    "mie_act_mul": [P, L, P, L, I, I, I, I, P],
    "mie_act_store": [P, L, P, L, I, I, I, I, P],
    "mie_clamped_glu": [P, L, P, L, I, I, I, F, F, F, I, P],
})
register_kernel_module("grouped_gemm", {
    "mie_grouped_linear": [P, I, L, L, I, P, I, L, L, P, I, L, L, P, P, L, P, P, I, I, I, I, I, I, P, P],
    "mie_grouped_glu": [P, I, L, P, I, L, L, P, I, L, P, P, I, I, I, I, I, F, F, F, P, P],
    "mie_route_topk": [P, L, P, P, P, I, I, I, P],
    "mie_route_topk_all": [P, L, P, P, P, P, I, I, I, I, P],
    "mie_moe_align": [P, I, I, P, P, P, P],
    "mie_moe_combine": [P, P, P, P, I, I, I, P],
    "mie_moe_combine_identity": [P, P, P, P, I, I, I, P, I, P, I, L, P],
})
register_kernel_module("latent_attention", {
    "mie_latent_kv_store": [P, L, P, I, F, P, P, I, P, P, I, P, I, I, I, I, I, P, P, P, I, I, P],
    "mie_latent_query_rotate": [P, L, I, P, P, I, I, I, I, I, I, P],
})
register_kernel_module("recurrence", {
    "mie_causal_conv": [P, L, P, P, P, P, P, P, P, P, I, I, I, P],
    "mie_rglru_scan": [P, P, P, P, L, P, P, L, P, P, P, P, P, P, I, I, I, I, F, P],
    "mie_rglru_scan_chunked": [P, P, P, P, L, P, P, L, P, P, P, P, P, P, I, I, I, I, F, I, I, P, P, P, P],
    "mie_residual_conv": [P, P, P, P, P, P, P, I, I, I, I, I, P],
})
register_kernel_module("attention_prep", {
    "mie_qkv_finish": [P, L, I, I, I, P, P, F, I, P, I, I, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P, F, I, P],
    "mie_head_gate": [P, I, P, L, I, I, I, P],
})
register_kernel_module("delta_rule", {
    "mie_delta_rule": [P, L, I, I, I, I, I, I, P, I, P, F, P, P, F, P, P, P, P, P, I, I, I, I, I, I, I, P, P, P],
})
register_kernel_module("gla", {
    "mie_gla": [P, L, I, I, I, I, I, P, I, P, F, F, P, F, P, P, P, P, P, I, I, I, I, I, I, I, I, P, P, P, P],
})
register_kernel_module("attention", {
    "mie_paged_attention": [P, L, P, P, P, I, P, I, P, P, I, I, I, I, I, F, I, I, F, P],
    "mie_paged_attention_scored": [P, L, P, P, P, I, P, I, P, P, I, I, I, I, I, F, I, I, F, I, F, I, P, P, I, P],
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
    "mie_decode_attention_sink": [P, L, P, P, P, P, P, P, I, P, I, I, I, I, I, F, I, I, I, F, P],
    "mie_decode_attention_sigmoid": [P, L, P, P, P, P, P, P, I, P, I, I, I, I, I, F, I, I, I, I, F, P, P],
    "mie_decode_attention_biased": [P, L, P, P, P, P, P, P, I, P, I, I, I, I, I, F, I, I, I, P, I, P],
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
    "mie_prefill_attention_sink": [P, L, P, P, P, P, I, P, P, I, I, I, I, I, I, I, F, I, F, P],
    "mie_prefill_attention_sigmoid": [P, L, P, P, P, P, I, P, P, I, I, I, I, I, I, I, F, I, I, F, P, P],
    "mie_prefill_attention_biased": [P, L, P, P, P, P, I, P, P, I, I, I, I, I, I, I, F, I, P, I, P],
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
