"""lightop_amd - MI355X-native (gfx950) drop-in for LightOp's block-INT8 fused-MoE path.

Public surface (same names, argument order and defaults as the reference package):

    lightop_amd.moe.fused_experts_impl_int8      (reference: lightop.moe.fused_experts_impl_int8)
    lightop_amd.moe.moe_align_block_size         (lightop.moe.moe_align_block_size)
    lightop_amd.moe.moe_align_block_size_out     (lightop.moe.moe_align_block_size_out)
    lightop_amd.moe.moe_sum                      (lightop.moe.moe_sum)
    lightop_amd.moe.get_moe_cache                (vllm_compat.fused_moe_cache.get_moe_cache)
    lightop_amd.quant.per_token_group_quant_int8 (lightop.quant.per_token_group_quant_int8)
    lightop_amd.quant.per_token_quant_int8       (lightop.quant.per_token_quant_int8)
    lightop_amd.fuse_silu_mul_quant              (lightop.fuse_silu_mul_quant)
    lightop_amd.gemmopt.moe_gemm_w8a8            (lightop.gemmopt.moe_gemm_w8a8)
    lightop_amd.moe.fused_experts_impl_w4a8      (lightop.moe.fused_experts_impl_w4a8, K-group form)
    lightop_amd.op                               (lightop.op: moe_align_block_size, moe_sum)
    lightop_amd.envs                             (lightop.envs: LMSLIM_* flags, read lazily)

The repository also ships a package named ``lightop`` whose modules ARE these modules (``lightop.moe is
lightop_amd.moe``), so that a caller of the reference keeps its imports.

Importing the package touches neither the GPU nor the HIP library; the library
(lightop_amd/csrc/liblightop_mi355.so, built by ``python -m lightop_amd.build``) is
loaded on the first call and a missing library is a hard error - there is no CPU or
PyTorch fallback.
"""
from . import envs  # noqa: F401
from . import op  # noqa: F401
from . import moe  # noqa: F401
from . import quant  # noqa: F401
from .moe.routing import moe_align_block_size_out, moe_sum  # noqa: F401
from .fuse_silu_mul_quant import fuse_silu_mul_quant  # noqa: F401

__version__ = "0.1.0"
__all__ = ["envs", "op", "moe", "quant", "moe_sum", "moe_align_block_size_out", "fuse_silu_mul_quant"]
