"""SiLU-and-mul followed by per-token int8 quantisation, the activation stage of the per-channel
W8A8 path (reference: lightop.fuse_silu_mul_quant, python/lightop/fuse_silu_mul_quant.py:45-62; kernel
csrc/kernels/gated_activation/fuse_silu_mul_quant.cu:90-199)."""
from __future__ import annotations

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
    """``input`` [rows, 2I] holds gate and up halves side by side.  Every row becomes
    ``act = T(T(silu(gate)) * up)``, then ``scale = max|act| / 127`` and ``q = round(act / scale)``
    (ties to even).  Returns ``(q [rows, I] int8, scale [rows, 1] f32)``, written into ``output`` /
    ``scales`` when the caller brings them.  With ``num_local_tokens_tensor`` only the first
    ``num_local_tokens * topk`` rows are touched; rows whose ``expert_ids`` entry is negative are skipped."""
    if input.dim() != 2 or input.shape[1] % 2:
        raise RuntimeError(f"fuse_silu_mul_quant: input must be [rows, 2 * I], got {tuple(input.shape)}")
    rows, width = input.shape[0], input.shape[1] // 2
    q = output if output is not None else input.new_empty((rows, width), dtype=torch.int8)
    s = scales if scales is not None else input.new_empty((rows, 1), dtype=torch.float32)
    op.fuse_silu_mul_quant(input, q, s, num_local_tokens_tensor, topk, expect_m, expert_ids)
    return q, s
