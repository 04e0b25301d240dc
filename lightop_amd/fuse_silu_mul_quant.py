"""SiLU-and-mul with per-token int8 quantisation (reference: python/lightop/fuse_silu_mul_quant.py:45-62)."""
from typing import Optional, Tuple

import torch

from . import op


def fuse_silu_mul_quant(input: torch.Tensor,
                        num_local_tokens_tensor: Optional[torch.Tensor] = None,
                        topk: int = 1,
                        expect_m: int = -1,
                        output: Optional[torch.Tensor] = None,
                        scales: Optional[torch.Tensor] = None,
                        expert_ids: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    leading, d2 = input.shape  # d2 == 2 * d
    d = d2 // 2
    if output is None:
        output = torch.empty(leading, d, dtype=torch.int8, device=input.device)
    if scales is None:
        scales = torch.empty((leading, 1), device=input.device, dtype=torch.float32)
    op.fuse_silu_mul_quant(input, output, scales, num_local_tokens_tensor, topk, expect_m, expert_ids)
    return output, scales
