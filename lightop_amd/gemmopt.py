"""Grouped-GEMM stage of the per-channel W8A8 MoE (reference: lightop.gemmopt.moe_gemm_w8a8,
python/lightop/gemmopt.py:437-457; native side csrc/moe_gemm/w8a8/moe_w8a8.cu:2389-2536)."""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from . import _lib
from .op import _act_dtype, _on_device, _require_cuda


def moe_gemm_w8a8(input: torch.Tensor, b_qweight: torch.Tensor, output: torch.Tensor, a_scale: torch.Tensor,
                  b_scale: torch.Tensor, topk_weights: Optional[torch.Tensor], sorted_token_ids: torch.Tensor,
                  experts_ids: torch.Tensor, num_tokens_post_pad: torch.Tensor, top_k: int,
                  config: Dict[str, Any], flags: int = 0, global_num_experts: int = 0) -> torch.Tensor:
    """One grouped GEMM stage in the per-channel form (reference: moe_gemm_w8a8, gemmopt.py:437-457):
    output[f] = T((sum_k input[f // top_k] * b_qweight[e]) * ts * b_scale[e]) with
    ts = a_scale[f // top_k], times topk_weights[f] when they are given (the second stage).
    ``a_scale`` [rows(, 1)], ``b_scale`` [E, N(, 1)]; ``config`` needs ``BLOCK_SIZE_M`` (the reference's
    ``MODE`` / ``DELTA`` pick among its tuned kernels and are ignored)."""
    _require_cuda(input, b_qweight, output, a_scale, b_scale, topk_weights, sorted_token_ids, experts_ids,
                  num_tokens_post_pad)
    assert input.dtype == torch.int8 and b_qweight.dtype == torch.int8
    assert input.is_contiguous() and b_qweight.is_contiguous() and output.is_contiguous()
    E, N, K = b_qweight.shape
    assert input.shape[1] == K and output.shape[-1] == N
    assert a_scale.dtype == torch.float32 and a_scale.is_contiguous() and a_scale.numel() == input.shape[0]
    assert b_scale.dtype == torch.float32 and b_scale.is_contiguous() and b_scale.numel() == E * N
    assert sorted_token_ids.dtype == torch.int32 and experts_ids.dtype == torch.int32
    num_valid = output.numel() // N
    tw = None
    if topk_weights is not None:
        tw = topk_weights if topk_weights.dtype == torch.float32 and topk_weights.is_contiguous() \
            else topk_weights.to(torch.float32).contiguous()
    with _on_device(input):
        _lib.check(_lib.lib().lo_moe_gemm_w8a8(
            _lib.ptr(input), _lib.ptr(a_scale), _lib.ptr(b_qweight), _lib.ptr(b_scale), _lib.ptr(output),
            _act_dtype(output), _lib.ptr(tw), _lib.ptr(sorted_token_ids), _lib.ptr(experts_ids),
            _lib.ptr(num_tokens_post_pad), sorted_token_ids.numel(), num_valid, input.shape[0], E,
            int(global_num_experts or 0), N, K, int(top_k),
            int(config["BLOCK_SIZE_M"]), 1 if tw is not None else 0,
            flags | (_lib.LO_GEMM_W_PRESHUFFLED if bool(getattr(b_qweight, "lo_preshuffled", False)) else 0), _lib.stream_of(input)))
    return output


__all__ = ["moe_gemm_w8a8"]
