"""Routers, expert alignment and expert reduction (reference: python/lightop/moe/routing.py,
python/lightop/_lmslim_native/vllm_compat/moe_align_block_size.py,
python/lightop/moe_align_sum.py:12-29)."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import op

# reference: moe/routing.py:20
topk_softmax = op.topk_softmax


def moe_fused_gate(x, bias, num_expert_group, topk_group, topk, n_share_experts_fusion, routed_scaling_factor,
                   apply_routed_scaling_factor_on_output=True, output_indices_int64=False):
    """Grouped top-k router of DeepSeek-style layers: sigmoid scores plus ``bias`` pick ``topk_group`` of
    ``num_expert_group`` expert groups (a group's score is the sum of its two best experts) and then ``topk``
    experts inside them; the weights are the unbiased sigmoid scores, renormalised and, when
    ``apply_routed_scaling_factor_on_output``, multiplied by ``routed_scaling_factor``.  Returns
    ``(topk_weights [T, topk] f32, topk_ids [T, topk] int32 or int64)``.  Same arguments as the reference's
    lightop.moe_fused_gate (python/lightop/moe_fused_gate.py:10-31; kernel
    csrc/kernels/moe_gate/moe_fused_gate.cu:76-312)."""
    return op.moe_fused_gate(x, bias, num_expert_group, topk_group, topk, n_share_experts_fusion,
                             routed_scaling_factor, apply_routed_scaling_factor_on_output, output_indices_int64)


def round_up(x: int, y: int) -> int:
    return ((x + y - 1) // y) * y


def cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def moe_align_block_size(
    topk_ids: torch.Tensor,
    block_size: int,
    num_experts: int,
    expert_map: Optional[torch.Tensor] = None,
    pad_sorted_ids: bool = False,
    ignore_invalid_experts: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Sort the flat (token, k) slots by expert and pad every expert to a multiple of
    ``block_size`` (moe_align_block_size.py:17-120).

    Returns ``(sorted_token_ids, expert_ids, num_tokens_post_padded)``, all int32:
    slot ids grouped by expert with ``topk_ids.numel()`` as the pad value, the expert of
    every block (mapped through ``expert_map``; -1 = not on this rank), and the padded
    total.  ``num_experts`` is the global expert count.  Within an expert, slot ids are
    ascending.  With ``ignore_invalid_experts`` ids whose map entry is -1 are dropped
    instead of being kept as -1 blocks.
    """
    numel = topk_ids.numel()
    max_num_tokens_padded = numel + num_experts * (block_size - 1)
    if pad_sorted_ids:
        max_num_tokens_padded = round_up(max_num_tokens_padded, block_size)
    if numel < num_experts:
        max_num_tokens_padded = min(numel * block_size, max_num_tokens_padded)
    sorted_ids = torch.empty((max_num_tokens_padded,), dtype=torch.int32, device=topk_ids.device)
    expert_ids = torch.empty((cdiv(max_num_tokens_padded, block_size),), dtype=torch.int32,
                             device=topk_ids.device)
    num_tokens_post_pad = torch.empty((1,), dtype=torch.int32, device=topk_ids.device)
    op._align(topk_ids, num_experts, block_size, sorted_ids, expert_ids, num_tokens_post_pad,
              expert_map, ignore_invalid=ignore_invalid_experts and expert_map is not None)
    return sorted_ids, expert_ids, num_tokens_post_pad


def moe_align_block_size_out(
    topk_ids,
    num_experts,
    block_size,
    sorted_ids,
    expert_ids,
    num_tokens_post_pad,
    expert_map=None,
    expert_mask=None,
    num_local_tokens=None,
    is_ep=False,
    is_fuse_fill=True,
):
    """Run expert alignment into caller-provided output tensors (moe/routing.py:23-49)."""
    return op.moe_align_block_size(
        topk_ids,
        num_experts,
        block_size,
        sorted_ids,
        expert_ids,
        num_tokens_post_pad,
        expert_map,
        expert_mask,
        num_local_tokens,
        is_ep,
        is_fuse_fill,
    )


def moe_sum(
    input: torch.Tensor,
    output: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    expert_mask: Optional[torch.Tensor] = None,
    num_local_tokens: Optional[torch.Tensor] = None,
    factor: float = 1.0,
    expect_m: int = -1,
) -> None:
    """output[t] = factor * sum_k input[t, k] (+ bias[t])  (moe_align_sum.py:12-29)."""
    op.moe_sum(input, output, bias, expert_mask, num_local_tokens, factor, expect_m)


__all__ = ["moe_align_block_size", "moe_align_block_size_out", "moe_sum"]
