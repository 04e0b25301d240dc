"""Quantisation APIs of the fused-MoE path (reference: python/lightop/quant/int8.py:13-16, :35)."""
from .int8 import per_token_group_quant_int8, per_token_quant_int8

__all__ = ["per_token_group_quant_int8", "per_token_quant_int8"]
