"""Flat native-op namespace (reference: the pybind module ``lightop.op``,
csrc/pybind/export.cpp:1437, :1508, :1584-1605).  Only the operators of the block-INT8
fused-MoE path, its per-channel form and the two routers that feed it exist here.
"""
from __future__ import annotations

import contextlib
from typing import Optional

import torch

from . import _lib


def _require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("lightop_amd: tensors must live on the GPU (there is no CPU path)")


@contextlib.contextmanager
def _on_device(t: torch.Tensor):
    if torch.cuda.current_device() == t.device.index:
        yield
    else:
        with torch.cuda.device(t.device):
            yield


def _ids_dtype(t: torch.Tensor) -> int:
    if t.dtype == torch.int32:
        return _lib.LO_I32
    if t.dtype == torch.int64:
        return _lib.LO_I64
    raise RuntimeError(f"lightop_amd: topk_ids must be int32 or int64, got {t.dtype}")


def _act_dtype(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return _lib.LO_BF16
    if t.dtype == torch.float16:
        return _lib.LO_F16
    if t.dtype == torch.float32:  # the block form's stages; entry points without an fp32 form say so
        return _lib.LO_F32
    raise RuntimeError(f"lightop_amd: unsupported activation dtype {t.dtype}")


def _align(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids, num_tokens_post_pad,
           expert_map, ignore_invalid, expert_mask=None, num_local_tokens=None):
    _require_cuda(topk_ids, sorted_token_ids, experts_ids, num_tokens_post_pad, expert_map, expert_mask,
                  num_local_tokens)
    if not topk_ids.is_contiguous():
        topk_ids = topk_ids.contiguous()
    for t, name in ((sorted_token_ids, "sorted_token_ids"), (experts_ids, "experts_ids"),
                    (num_tokens_post_pad, "num_tokens_post_pad")):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError(f"lightop_amd: {name} must be a contiguous int32 tensor")
    if expert_map is not None and (expert_map.dtype != torch.int32 or not expert_map.is_contiguous()):
        expert_map = expert_map.to(torch.int32).contiguous()
    if expert_mask is not None:
        if expert_mask.dtype not in (torch.bool, torch.uint8) or not expert_mask.is_contiguous() \
                or expert_mask.numel() != topk_ids.numel():
            raise RuntimeError("lightop_amd: expert_mask must be a contiguous bool tensor with one entry per slot")
        expert_mask = expert_mask.view(torch.uint8)
    top_k = 1
    if num_local_tokens is not None:
        if num_local_tokens.dtype != torch.int32 or num_local_tokens.numel() < 1:
            raise RuntimeError("lightop_amd: num_local_tokens must be an int32 tensor with one element")
        if topk_ids.dim() != 2:
            raise RuntimeError("lightop_amd: num_local_tokens needs topk_ids of shape [num_tokens, topk]")
        top_k = topk_ids.shape[1]
    lib = _lib.lib()
    # large inputs are aligned by many workgroups; their per-chunk counters live in a
    # scratch tensor (the reference allocates one too, moe_align_sum_kernels.cu:1175)
    nscratch = int(lib.lo_moe_align_scratch_bytes(topk_ids.numel(), int(num_experts)))
    scratch = torch.empty(nscratch, dtype=torch.uint8, device=topk_ids.device) if nscratch > 0 else None
    with _on_device(topk_ids):
        _lib.check(lib.lo_moe_align_block_size_local(
            _lib.ptr(topk_ids), _ids_dtype(topk_ids), topk_ids.numel(), int(num_experts), int(block_size),
            _lib.ptr(expert_map), 1 if ignore_invalid else 0, _lib.ptr(sorted_token_ids),
            sorted_token_ids.numel(), _lib.ptr(experts_ids), experts_ids.numel(),
            _lib.ptr(num_tokens_post_pad), _lib.ptr(expert_mask), _lib.ptr(scratch), max(nscratch, 0),
            _lib.ptr(num_local_tokens), top_k, _lib.stream_of(topk_ids)))


def moe_align_block_size(topk_ids: torch.Tensor, num_experts: int, block_size: int,
                         sorted_token_ids: torch.Tensor, experts_ids: torch.Tensor,
                         num_tokens_post_pad: torch.Tensor,
                         expert_map: Optional[torch.Tensor] = None,
                         expert_mask: Optional[torch.Tensor] = None,
                         num_local_tokens: Optional[torch.Tensor] = None,
                         Is_EP: bool = False, Is_fuse_fill: bool = True) -> None:
    """``op.moe_align_block_size`` (export.cpp:1593-1605; kernel semantics
    csrc/kernels/moe_align_sum_kernels.cu:25-150).  With an ``expert_map`` the block expert ids
    are the mapped (local) ids, -1 for experts of other ranks; ``Is_EP`` drops the slots of those
    experts instead of keeping them as -1 blocks; ``expert_mask`` (bool, one entry per slot) is an
    output: True where the slot's expert is on this rank; ``num_local_tokens`` (device int32[1])
    limits the work to the first that many tokens, whose padding successors get mask False."""
    del Is_fuse_fill  # the pad value is always written
    _align(topk_ids, num_experts, block_size, sorted_token_ids, experts_ids, num_tokens_post_pad,
           expert_map, ignore_invalid=bool(Is_EP) and expert_map is not None, expert_mask=expert_mask,
           num_local_tokens=num_local_tokens)


def moe_sum(input: torch.Tensor, output: torch.Tensor, bias: Optional[torch.Tensor] = None,
            expert_mask: Optional[torch.Tensor] = None, num_local_tokens: Optional[torch.Tensor] = None,
            factor: float = 1.0, expect_m: int = -1) -> None:
    """``op.moe_sum`` (export.cpp:1584-1592): output[t] = factor * sum_k input[t, k] (+ bias[t]).
    Slots whose ``expert_mask`` entry is False are skipped; rows from ``num_local_tokens[0]`` on
    (device int32[1]) are left untouched."""
    del expect_m
    _require_cuda(input, output, bias, num_local_tokens)
    if num_local_tokens is not None and (num_local_tokens.dtype != torch.int32 or num_local_tokens.numel() < 1):
        raise RuntimeError("lightop_amd.op.moe_sum: num_local_tokens must be an int32 tensor with one element")
    if input.dim() != 3:
        raise RuntimeError("lightop_amd.op.moe_sum: input must be [num_tokens, topk, hidden]")
    if not input.is_contiguous():
        input = input.contiguous()
    M, k, H = input.shape
    if not output.is_contiguous() or output.numel() != M * H or output.dtype != input.dtype:
        raise RuntimeError("lightop_amd.op.moe_sum: output must be a contiguous [num_tokens, hidden] "
                           "tensor of the input dtype")
    if bias is not None and (not bias.is_contiguous() or bias.numel() != M * H or bias.dtype != input.dtype):
        raise RuntimeError("lightop_amd.op.moe_sum: bias must match output")
    if expert_mask is not None:
        _require_cuda(expert_mask)
        if expert_mask.numel() != M * k or expert_mask.dtype not in (torch.bool, torch.uint8):
            raise RuntimeError("lightop_amd.op.moe_sum: expert_mask must be a bool tensor of M*topk elements")
        expert_mask = expert_mask.contiguous().view(torch.uint8)
    with _on_device(input):
        _lib.check(_lib.lib().lo_moe_sum(_lib.ptr(input), _lib.ptr(output), _lib.ptr(bias),
                                         _lib.ptr(expert_mask), _act_dtype(input), M, k, H, float(factor),
                                         _lib.ptr(num_local_tokens), _lib.stream_of(input)))


def fuse_silu_mul_quant(input: torch.Tensor, output: torch.Tensor, scales: torch.Tensor,
                        num_local_tokens_tensor: Optional[torch.Tensor] = None, topk: int = 1, expect_m: int = -1,
                        expert_ids: Optional[torch.Tensor] = None) -> None:
    """``op.fuse_silu_mul_quant`` (export.cpp:1532; fuse_silu_mul_quant.cu:90-199): SiLU(gate) * up of
    ``input`` [rows, 2d], then one int8 scale per row: ``output`` [rows, d] int8, ``scales`` [rows(, 1)] f32.
    With ``num_local_tokens_tensor`` (device int32[1]) only the first ``n * topk`` rows are processed; with
    ``expert_ids`` (int32 [rows]; fuse_silu_mul_quant.cu:269-283) rows whose entry is -1 are skipped and their
    ``output`` / ``scales`` left untouched."""
    del expect_m
    _require_cuda(input, output, scales, num_local_tokens_tensor, expert_ids)
    if input.dim() != 2 or not input.is_contiguous() or input.shape[1] % 16:
        raise RuntimeError("lightop_amd.op.fuse_silu_mul_quant: input must be a contiguous [rows, 2*d] tensor, d % 8 == 0")
    rows, d = input.shape[0], input.shape[1] // 2
    if output.dtype != torch.int8 or not output.is_contiguous() or output.numel() != rows * d:
        raise RuntimeError("lightop_amd.op.fuse_silu_mul_quant: output must be a contiguous int8 [rows, d] tensor")
    if scales.dtype != torch.float32 or not scales.is_contiguous() or scales.numel() != rows:
        raise RuntimeError("lightop_amd.op.fuse_silu_mul_quant: scales must be a contiguous float32 [rows, 1] tensor")
    if num_local_tokens_tensor is not None and (num_local_tokens_tensor.dtype != torch.int32
                                                or num_local_tokens_tensor.numel() < 1):
        raise RuntimeError("lightop_amd.op.fuse_silu_mul_quant: num_local_tokens_tensor must be int32 with one element")
    if expert_ids is not None and (expert_ids.dtype != torch.int32 or not expert_ids.is_contiguous()
                                   or expert_ids.numel() < rows):
        raise RuntimeError("lightop_amd.op.fuse_silu_mul_quant: expert_ids must be a contiguous int32 tensor with one "
                           "entry per row")
    with _on_device(input):
        _lib.check(_lib.lib().lo_fuse_silu_mul_quant_ids(_lib.ptr(input), _act_dtype(input), rows, d, _lib.ptr(output),
                                                         _lib.ptr(scales), _lib.ptr(num_local_tokens_tensor), int(topk),
                                                         _lib.ptr(expert_ids), _lib.stream_of(input)))


def _float_dtype(t: torch.Tensor, what: str) -> int:
    if t.dtype == torch.float32:
        return _lib.LO_F32
    if t.dtype == torch.float16:
        return _lib.LO_F16
    if t.dtype == torch.bfloat16:
        return _lib.LO_BF16
    raise RuntimeError(f"lightop_amd: {what} must be float32, float16 or bfloat16, got {t.dtype}")


def topk_softmax(topk_weights: torch.Tensor, topk_indices: torch.Tensor,
                 token_expert_indices: Optional[torch.Tensor], gating_output: torch.Tensor,
                 Is_renormalize: bool = False) -> None:
    """Softmax top-k router into caller-allocated outputs (op.topk_softmax, export.cpp:546, :1437;
    topk_softmax_kernels.cu:1716-1790).  Winners in descending order, equal logits are won by
    the lower expert id; ``token_expert_indices[t, j] = j * num_tokens + t``."""
    _require_cuda(topk_weights, topk_indices, token_expert_indices, gating_output)
    if gating_output.dim() != 2 or not gating_output.is_contiguous():
        raise RuntimeError("lightop_amd: gating_output must be a contiguous [num_tokens, num_experts] tensor")
    T, E = gating_output.shape
    k = topk_weights.shape[-1]
    if topk_weights.dtype != torch.float32 or not topk_weights.is_contiguous() or topk_weights.numel() != T * k:
        raise RuntimeError("lightop_amd: topk_weights must be a contiguous float32 [num_tokens, topk] tensor")
    if not topk_indices.is_contiguous() or topk_indices.numel() != T * k:
        raise RuntimeError("lightop_amd: topk_indices must be a contiguous [num_tokens, topk] tensor")
    if token_expert_indices is not None and (token_expert_indices.dtype != torch.int32
                                             or not token_expert_indices.is_contiguous()
                                             or token_expert_indices.numel() != T * k):
        raise RuntimeError("lightop_amd: token_expert_indices must be a contiguous int32 [num_tokens, topk] tensor")
    with _on_device(gating_output):
        _lib.check(_lib.lib().lo_topk_softmax(
            _lib.ptr(gating_output), _float_dtype(gating_output, "gating_output"), T, E, k, int(bool(Is_renormalize)),
            _lib.ptr(topk_weights), _lib.ptr(topk_indices), _ids_dtype(topk_indices),
            _lib.ptr(token_expert_indices), _lib.stream_of(gating_output)))


def moe_fused_gate(input: torch.Tensor, bias: torch.Tensor, num_expert_group: int, topk_group: int, topk: int,
                   n_share_experts_fusion: int, routed_scaling_factor: float,
                   apply_routed_scaling_factor_on_output: bool = True, output_indices_int64: bool = False):
    """Grouped sigmoid top-k with correction bias; returns ``[weights f32 [T, topk], indices [T, topk]]``
    (op.moe_fused_gate, export.cpp:566, :1508; moe_fused_gate.cu:1331-1530)."""
    _require_cuda(input, bias)
    if input.dim() != 2 or not input.is_contiguous():
        raise RuntimeError("lightop_amd: input must be a contiguous [num_tokens, num_experts] tensor")
    T, E = input.shape
    if bias.dim() != 1 or bias.numel() != E or not bias.is_contiguous():
        raise RuntimeError("lightop_amd: bias must be a contiguous [num_experts] tensor")
    weights = torch.empty(T, topk, dtype=torch.float32, device=input.device)
    indices = torch.empty(T, topk, dtype=torch.int64 if output_indices_int64 else torch.int32, device=input.device)
    with _on_device(input):
        _lib.check(_lib.lib().lo_moe_fused_gate(
            _lib.ptr(input), _float_dtype(input, "input"), _lib.ptr(bias), _float_dtype(bias, "bias"), T, E,
            int(num_expert_group), int(topk_group), int(topk), int(n_share_experts_fusion),
            float(routed_scaling_factor), int(bool(apply_routed_scaling_factor_on_output)),
            _lib.ptr(weights), _lib.ptr(indices), _ids_dtype(indices), _lib.stream_of(input)))
    return [weights, indices]
