"""Grouped-GEMM stage of the per-channel W8A8 MoE (reference: python/lightop/gemmopt.py:437-457)."""
from .moe.native import moe_gemm_w8a8

__all__ = ["moe_gemm_w8a8"]
