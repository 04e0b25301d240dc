"""``lightop`` as an importable name for the MI355X build of the fused-MoE path.

A program written against the reference imports ``lightop.moe``, ``lightop.quant``, ``lightop.op``,
``lightop.envs``, ``lightop.gemmopt`` and ``lightop.fuse_silu_mul_quant`` (python/lightop/__init__.py,
python/lightop/moe/__init__.py:57-78).  This package makes those names resolve to the modules of
``lightop_amd`` themselves - the same module objects, so the lazily resolved entry points
(``lightop.moe.fused_experts_impl_int8`` and friends) are the same functions and module state (caches,
flags) exists once.  Only the operators of the block-INT8 fused-MoE path, its per-channel and W4A8 forms and
the two routers exist; every other name of the reference package raises AttributeError / ImportError.

Importing it touches neither the GPU nor the HIP library.
"""
import sys as _sys

import lightop_amd as _impl
from lightop_amd import envs, gemmopt, moe, op, quant  # noqa: F401
from lightop_amd import fuse_silu_mul_quant as _fsq_module  # the module; the package attribute is the function
from lightop_amd.fuse_silu_mul_quant import fuse_silu_mul_quant  # noqa: F401
from lightop_amd.gemmopt import moe_gemm_w8a8  # noqa: F401
from lightop_amd.moe import cache as _moe_cache, native as _moe_native, routing as _moe_routing
from lightop_amd.moe.routing import moe_align_block_size_out, moe_fused_gate, moe_sum  # noqa: F401

__version__ = _impl.__version__

# module paths of the reference -> the module that serves them here
_ALIASES = {
    "lightop.envs": envs,
    "lightop.op": op,
    "lightop.gemmopt": gemmopt,
    "lightop.quant": quant,
    "lightop.quant.int8": quant,                       # python/lightop/quant/int8.py
    "lightop.moe": moe,
    "lightop.moe.native": _moe_native,                 # python/lightop/moe/native.py:9
    "lightop.moe.routing": _moe_routing,               # python/lightop/moe/routing.py
    "lightop.moe.cache": _moe_cache,
    "lightop.moe_fused_gate": _moe_routing,            # python/lightop/moe_fused_gate.py:10-31
    "lightop.moe_align_sum": _moe_routing,             # python/lightop/moe_align_sum.py:12-29 (moe_sum)
    "lightop.fuse_silu_mul_quant": _sys.modules["lightop_amd.fuse_silu_mul_quant"],
}
for _name, _module in _ALIASES.items():
    _sys.modules.setdefault(_name, _module)
del _name, _module, _fsq_module

__all__ = ["envs", "op", "moe", "quant", "gemmopt", "moe_sum", "moe_align_block_size_out", "moe_fused_gate",
           "fuse_silu_mul_quant", "moe_gemm_w8a8"]
