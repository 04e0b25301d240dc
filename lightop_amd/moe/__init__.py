"""Mixture-of-Experts APIs of the block-INT8 path (reference: python/lightop/moe/__init__.py)."""
from importlib import import_module

from .cache import get_moe_cache
from .routing import moe_align_block_size, moe_align_block_size_out, moe_fused_gate, moe_sum, topk_softmax

# resolved on first access, like the reference's lazily imported "LMSlim native" entry points
# (moe/__init__.py:57-78)
_NATIVE_APIS = {
    "fused_experts_impl_int8",
    "fused_experts_impl_w4a8",
    "preshuffle_moe_weight_int4",
    "preshuffle_moe_scale_int4",
    "get_w8a8moe_json",
    "get_moe_cuda_config",
    "invoke_fused_moe_kernel_int8",
    "invoke_fused_moe_kernel_w4a8",
    "invoke_fused_moe_gemm1_silu_quant",
    "silu_and_mul",
    "gelu_and_mul",
    "act_and_mul_group_quant",
    "fused_experts_workspace_bytes",
    "fused_experts_workspace_views",
    "preshuffle_moe_weight",
    "moe_gemm_w8a8",
}


def __getattr__(name):
    if name not in _NATIVE_APIS:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
    value = getattr(import_module(f"{__name__}.native"), name)
    globals()[name] = value
    return value


__all__ = [
    "act_and_mul_group_quant",
    "fused_experts_impl_int8",
    "fused_experts_impl_w4a8",
    "fused_experts_workspace_bytes",
    "fused_experts_workspace_views",
    "get_moe_cache",
    "get_moe_cuda_config",
    "gelu_and_mul",
    "get_w8a8moe_json",
    "invoke_fused_moe_gemm1_silu_quant",
    "invoke_fused_moe_kernel_int8",
    "invoke_fused_moe_kernel_w4a8",
    "moe_align_block_size",
    "moe_align_block_size_out",
    "moe_fused_gate",
    "moe_gemm_w8a8",
    "moe_sum",
    "preshuffle_moe_weight",
    "preshuffle_moe_weight_int4",
    "preshuffle_moe_scale_int4",
    "silu_and_mul",
    "topk_softmax",
]
