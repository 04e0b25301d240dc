"""torch-CPU restatement of the reference's test-side block-INT8 MoE.  TEST INFRASTRUCTURE ONLY.

This is the "repo's torch CPU reference of the same path": the structure of
``native_per_token_group_quant_int8`` (test/moe_w8a8/benchmark_moe_int8.py:60-83),
``native_w8a8_block_int8_matmul`` (:87-139) and the per-expert MoE loop of
``torch_w8a8_per_column_moe`` (:163-201, block-quantised as in the sglang test the
reference points to, :225-234).  It is written from the description of those
functions, is an independent second opinion for the C oracle (different
summation order: ``dot * (a_s * b_s)`` accumulated block by block with fp32
matmuls) and is what ``bench.py`` times as the CPU baseline.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def native_per_token_group_quant_int8(x: torch.Tensor, group_size: int = 128, eps: float = 1e-10):
    """amax over each 1 x group_size group, s = amax / 127, q = trunc(clamp(x / s))."""
    assert x.shape[-1] % group_size == 0 and x.is_contiguous()
    xg = x.reshape(-1, group_size).to(torch.float32)
    amax = xg.abs().amax(dim=-1, keepdim=True).clamp(min=eps)
    s = amax / 127.0
    q = (xg / s).clamp(min=-128, max=127).to(torch.int8)
    return q.reshape(x.shape), s.reshape(x.shape[:-1] + (x.shape[-1] // group_size,))


def native_w8a8_block_int8_matmul(A, B, As, Bs, block_size=(128, 128), output_dtype=torch.bfloat16):
    """C = sum over K-blocks of (A_blk @ B_blk^T) * (As[:, kb] * Bs[nb, kb]); A [M,K], B [N,K]."""
    block_n, block_k = block_size
    A = A.to(torch.float32)
    B = B.to(torch.float32)
    M, K = A.shape
    N = B.shape[0]
    n_tiles = (N + block_n - 1) // block_n
    k_tiles = (K + block_k - 1) // block_k
    assert Bs.shape == (n_tiles, k_tiles) and As.shape == (M, k_tiles)
    C = torch.zeros(M, N, dtype=torch.float32)
    for kb in range(k_tiles):
        a = A[:, kb * block_k:(kb + 1) * block_k]
        for nb in range(n_tiles):
            b = B[nb * block_n:(nb + 1) * block_n, kb * block_k:(kb + 1) * block_k]
            C[:, nb * block_n:(nb + 1) * block_n] += (a @ b.t()) * (As[:, kb:kb + 1] * Bs[nb, kb])
    return C.to(output_dtype)


def unpack_int4(wp: torch.Tensor) -> torch.Tensor:
    """Packed signed int4 [..., K/2] (even k in the high nibble, w4a8.py:341, :375-377) -> int8 [..., K]."""
    b = wp.view(torch.uint8).to(torch.int16)
    hi, lo = b >> 4, b & 15
    w = torch.stack([hi, lo], dim=-1).reshape(*wp.shape[:-1], wp.shape[-1] * 2)
    return torch.where(w >= 8, w - 16, w).to(torch.int8)


def native_w4a8_group_matmul(A, B, As, Bs, output_dtype=torch.bfloat16):
    """C = sum over K-blocks of (A_blk @ B_blk^T) * As[:, kb] * Bs[:, kb]; A [M,K] int8, B [N,K] int8 holding
    int4 values, Bs [N, K/128]: one scale per output row and K group."""
    A = A.to(torch.float32)
    B = B.to(torch.float32)
    M, K = A.shape
    C = torch.zeros(M, B.shape[0], dtype=torch.float32)
    for kb in range(K // 128):
        C += (A[:, kb * 128:(kb + 1) * 128] @ B[:, kb * 128:(kb + 1) * 128].t()) * As[:, kb:kb + 1] * Bs[:, kb][None, :]
    return C.to(output_dtype)


def torch_w4a8_group_moe(x, w1_packed, w2_packed, w1_s, w2_s, topk_weight, topk_ids, expert_map=None,
                         routed_scaling_factor: float = 1.0):
    """The loop of torch_w8a8_block_int8_moe with packed int4 weights and K-group row scales."""
    return torch_w8a8_block_int8_moe(x, unpack_int4(w1_packed), unpack_int4(w2_packed), w1_s, w2_s, topk_weight,
                                     topk_ids, expert_map, routed_scaling_factor, matmul=native_w4a8_group_matmul)


def native_per_token_quant_int8(x: torch.Tensor):
    """One scale per row, round half to even: s = absmax / 127, q = round(x * (127 / absmax))
    (the torch form of int8_utils.py:20-44; vLLM's dynamic scaled_int8_quant, which the reference's
    test of fuse_silu_mul_quant compares with, test/test_fuse_silu_mul_quant.py:11-14, is the same rule)."""
    xf = x.to(torch.float32)
    absmax = xf.abs().amax(dim=-1, keepdim=True).clamp(min=1e-10)
    # torch evaluates `127.0 / t` as reciprocal-times-127; the rule is a true division
    q = torch.round(xf * (torch.full_like(absmax, 127.0) / absmax)).clamp(min=-128, max=127).to(torch.int8)
    return q, absmax / 127.0


def native_w8a8_per_token_matmul(A, B, As, Bs, output_dtype=torch.bfloat16):
    """C = As * (A @ B^T) * Bs: per-token scale As [M, 1], per-row weight scale Bs [N(, 1)]
    (test/moe_w8a8/fuse_moegemm_correctness.py:825-844)."""
    C = torch.matmul(A.to(torch.float32), B.to(torch.float32).t())  # exact below 2^24, else ~1e-7 relative
    return (As * C * Bs.reshape(1, -1)).to(output_dtype)


def torch_w8a8_per_column_moe(x, w1, w2, w1_s, w2_s, topk_weight, topk_ids, expert_map=None,
                              routed_scaling_factor: float = 1.0):
    """The per-expert loop of test/moe_w8a8/fuse_moegemm_correctness.py:847-885 (per-token activation
    scales, per-row weight scales), with the optional ``expert_map`` of the block version."""
    M, H = x.shape
    k = topk_ids.shape[1]
    a_q, a_s = native_per_token_quant_int8(x)
    a_q = a_q.view(M, 1, H).repeat(1, k, 1).reshape(-1, H)
    a_s = a_s.view(M, 1, 1).repeat(1, k, 1).reshape(-1, 1)
    out = torch.zeros(M * k, w2.shape[1], dtype=x.dtype)
    flat_ids = topk_ids.reshape(-1).long()
    local = flat_ids if expert_map is None else expert_map.long()[flat_ids]
    for e in range(w1.shape[0]):
        mask = local == e
        if not bool(mask.any()):
            continue
        inter = native_w8a8_per_token_matmul(a_q[mask], w1[e], a_s[mask], w1_s[e], output_dtype=x.dtype)
        d = inter.shape[-1] // 2
        act = F.silu(inter[..., :d]) * inter[..., d:]
        act_q, act_s = native_per_token_quant_int8(act)
        out[mask] = native_w8a8_per_token_matmul(act_q, w2[e], act_s, w2_s[e], output_dtype=x.dtype)
    res = (out.view(M, k, -1) * topk_weight.view(M, k, 1).to(out.dtype)).sum(dim=1)
    if routed_scaling_factor != 1.0:
        res = res * routed_scaling_factor
    return res


def torch_w8a8_block_int8_moe(x, w1, w2, w1_s, w2_s, topk_weight, topk_ids, expert_map=None,
                              routed_scaling_factor: float = 1.0, matmul=None):
    """Per-expert loop: quant -> GEMM1 -> silu*mul -> quant -> GEMM2 -> * weight -> sum over k.

    ``expert_map`` (global id -> local id or -1) restricts the loop to local
    experts; slots of non-local experts contribute zero.
    """
    matmul = matmul or native_w8a8_block_int8_matmul
    M, H = x.shape
    k = topk_ids.shape[1]
    a_q, a_s = native_per_token_group_quant_int8(x)
    a_q = a_q.view(M, 1, H).repeat(1, k, 1).reshape(-1, H)
    a_s = a_s.view(M, 1, -1).repeat(1, k, 1).reshape(M * k, -1)
    out = torch.zeros(M * k, w2.shape[1], dtype=x.dtype)
    flat_ids = topk_ids.reshape(-1).long()
    local = flat_ids if expert_map is None else expert_map.long()[flat_ids]
    for e in range(w1.shape[0]):
        mask = local == e
        if not bool(mask.any()):
            continue
        inter = matmul(a_q[mask], w1[e], a_s[mask], w1_s[e], output_dtype=x.dtype)
        d = inter.shape[-1] // 2
        act = F.silu(inter[..., :d]) * inter[..., d:]
        act_q, act_s = native_per_token_group_quant_int8(act.contiguous())
        out[mask] = matmul(act_q, w2[e], act_s, w2_s[e], output_dtype=x.dtype)
    res = (out.view(M, k, -1) * topk_weight.view(M, k, 1).to(out.dtype)).sum(dim=1)
    if routed_scaling_factor != 1.0:
        res = res * routed_scaling_factor
    return res
