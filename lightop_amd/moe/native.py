"""Block-INT8 fused experts (reference:
python/lightop/_lmslim_native/layers/fused_moe/int8.py:543-908)."""
from __future__ import annotations

import ctypes
import functools
from typing import Any, Dict, List, Optional, Tuple

import torch

from .. import _lib, envs
from ..gemmopt import moe_gemm_w8a8
from ..op import _act_dtype, _ids_dtype, _on_device, _require_cuda


def get_w8a8moe_json(m: int, E: int, n1: int, n2: int, k: int, use_int8_w8a8: bool,
                     block_shape: Optional[List[int]], topk: int,
                     global_num_experts: int = -1, preshuffled: bool = True,
                     int4: bool = False, dtype: torch.dtype = torch.bfloat16,
                     activation: str = "silu") -> Tuple[Dict[str, Any], Dict[str, Any]]:
    """Tile configuration of both GEMMs for ``m`` tokens (reference: get_w8a8moe_json,
    int8.py:220-256, backed there by per-device JSON files).  ``n1`` = 2*I, ``n2`` = H, ``k`` = I.
    ``block_shape=None`` asks for the per-channel form (the reference consults get_moe_cuda_config first
    there, int8.py:735-741), ``[1, 128]`` for W4A8 with K-group scales.  ``int4`` with ``block_shape=None``:
    the reference's own W4A8 form (w4a8.py:587, which passes only the first five arguments).

    The block size comes from a tuning file when ``TRITON_JSON_DIR`` names a directory that holds one for
    this layer shape (``lightop_amd.moe.tile_files``: the reference's file names and keys, written by
    ``python -m lightop_amd.tune --out``), else from the table compiled into the library.  The dictionaries
    keep the reference's keys; ``kernel`` / ``num_warps`` / ``BLOCK_SIZE_N`` describe the kernel the
    whole-path call launches for that block size, ``source`` says where the block size came from.
    ``preshuffled``: the weights are in the load-time layout of ``preshuffle_moe_weight`` (the table
    differs for row-major weights); ``dtype`` / ``activation``: rows other than bfloat16 and GELU take the
    path without the fused epilogue."""
    del use_int8_w8a8
    from . import tile_files

    t1, t2 = _lib.LoMoeTile(), _lib.LoMoeTile()
    Eg = E if global_num_experts in (-1, None) else global_num_experts
    form = _lib.LO_FORM_CHANNEL if block_shape is None else (
        _lib.LO_FORM_W4 if list(block_shape) == [1, 128] else _lib.LO_FORM_BLOCK)
    flags = _lib.LO_GEMM_W_PRESHUFFLED if preshuffled else 0
    if int4 and block_shape is None:
        flags |= _lib.LO_GEMM_W4 | _lib.LO_GEMM_W_PRESHUFFLED
    if activation == "gelu":
        flags |= _lib.LO_FUSED_ACT_GELU
    dt = {torch.bfloat16: _lib.LO_BF16, torch.float16: _lib.LO_F16, torch.float32: _lib.LO_F32}[dtype]
    bs_file = tile_files.block_size_m(m, E, n1, n2, k, topk, block_shape, int4=int4 or form == _lib.LO_FORM_W4)
    _lib.check(_lib.lib().lo_moe_tile_query_path(form, flags, dt, bs_file, m, E, Eg, topk, n2, k, t1, t2))

    def as_dict(t):
        return {"BLOCK_SIZE_M": t.block_size_m, "BLOCK_SIZE_N": t.block_n, "BLOCK_SIZE_K": 128,
                "GROUP_SIZE_M": 1, "num_warps": t.waves, "num_stages": 0, "kernel": t.kernel,
                "kernel_name": _lib.KERNEL_NAMES.get(t.kernel, "?"),
                "source": "file" if bs_file else "compiled"}

    return as_dict(t1), as_dict(t2)


def get_moe_cuda_config(E: int, M: int, N1: int, K1: int, N2: int, K2: int, topk: int,
                        device_name: Optional[str] = None, num_cus: Optional[int] = None,
                        dtype: Optional[str] = None, block_n: Optional[int] = None,
                        block_k: Optional[int] = None, is_ep: Optional[bool] = False,
                        ep_size: Optional[int] = 16) -> Tuple[Dict[str, Any], Dict[str, Any], bool]:
    """Configurations of the two per-channel GEMMs for ``M`` tokens and whether they were found
    (reference: lightop.moe.get_moe_cuda_config, python/lightop/config.py:33-131, which reads per-device
    JSON files keyed by GEMM shape and token count; the per-channel branch of fused_experts_impl_int8
    asks it first, int8.py:735-741).  ``N1, K1`` = 2*I, H and ``N2, K2`` = H, I.  The table is the one
    compiled into the library, so the answer is always found; ``MODE`` and ``DELTA``, which select among
    the reference's per-gfx kernels, are carried as 0 and read by nothing here.  ``is_ep``: ``E`` experts
    are resident out of ``E * ep_size`` that the router chooses from."""
    del device_name, num_cus, dtype, block_n, block_k
    assert N1 % 2 == 0 and K1 == N2 and K2 == N1 // 2, "shapes of one gated layer: N1 = 2*I, K1 = N2 = H, K2 = I"
    c1, c2 = get_w8a8moe_json(M, E, N1, N2, K2, True, None, topk,
                              global_num_experts=E * int(ep_size) if is_ep else E)
    for c in (c1, c2):
        c.update(MODE=0, DELTA=0)
    return c1, c2, True


def _scale_flags(fused_scale: Optional[bool]) -> int:
    """None or False: the library's default order, acc = fma(f32(d) * a_s, b_s, acc) per K block;
    True: acc = fma(f32(d), a_s * b_s, acc) everywhere (last-ulp differences).  The order without
    fp fusion, acc + (f32(d) * a_s) * b_s, is ``flags=LO_GEMM_SEPARATE_ORDER``."""
    return _lib.LO_GEMM_FUSED_SCALE if fused_scale else 0


def preshuffle_moe_weight(w: torch.Tensor) -> torch.Tensor:
    """Return expert weights ``w`` [E, N, K] (int8, row-major) in the load-time layout of the
    gfx950 GEMM kernels: each 16-row x 128-byte block stored as [8 x 16-byte K chunks][16 rows].
    Same shape and dtype as ``w``; the result carries ``lo_preshuffled = True`` and is what
    ``fused_experts_impl_int8`` wants for ``w1`` / ``w2`` when full speed matters.  Do this
    once when the checkpoint is loaded.  N % 16 == 0 and K % 128 == 0 are required."""
    _require_cuda(w)
    assert w.dtype == torch.int8 and w.dim() == 3 and w.is_contiguous()
    E, N, K = w.shape
    out = torch.empty_like(w)
    with _on_device(w):
        _lib.check(_lib.lib().lo_preshuffle_weight_int8(_lib.ptr(w), _lib.ptr(out), E, N, K,
                                                        _lib.stream_of(w)))
    out.lo_preshuffled = True
    return out


def preshuffle_moe_weight_int4(w_packed: torch.Tensor) -> torch.Tensor:
    """Packed signed int4 expert weights [E, N, K/2] (two per byte along K, even k in the high
    nibble: the reference's order, w4a8.py:341, :375-377) in the load-time layout of the gfx950
    kernels.  Same shape and dtype; the result carries ``lo_preshuffled = True`` and
    ``lo_int4 = True``.  N % 16 == 0 and K % 128 == 0 are required."""
    _require_cuda(w_packed)
    assert w_packed.dtype in (torch.int8, torch.uint8) and w_packed.dim() == 3 and w_packed.is_contiguous()
    E, N, K2 = w_packed.shape
    out = torch.empty_like(w_packed)
    with _on_device(w_packed):
        _lib.check(_lib.lib().lo_preshuffle_weight_int4(_lib.ptr(w_packed), _lib.ptr(out), E, N, 2 * K2,
                                                        _lib.stream_of(w_packed)))
    out.lo_preshuffled = True
    out.lo_int4 = True
    return out


def preshuffle_moe_scale_int4(scale: torch.Tensor) -> torch.Tensor:
    """K-group scales of packed int4 weights, [E, N, K/128] -> [E, K/128, N] contiguous fp32 (the four
    rows a lane accumulates become one 16-byte load).  Once at load time; the result carries
    ``lo_kmajor = True``."""
    assert scale.dim() == 3
    out = scale.to(torch.float32).transpose(1, 2).contiguous()
    out.lo_kmajor = True
    return out


def _is_preshuffled(w: torch.Tensor) -> bool:
    return bool(getattr(w, "lo_preshuffled", False))


def _check_gemm_inputs(A, A_scale, B, B_scale, sorted_token_ids, expert_ids, num_tokens_post_padded, w4=False):
    _require_cuda(A, A_scale, B, B_scale, sorted_token_ids, expert_ids, num_tokens_post_padded)
    assert A.dtype == torch.int8 and B.dtype in ((torch.int8, torch.uint8) if w4 else (torch.int8,)), \
        "A must be int8, B int8 (packed int4: int8 or uint8)"
    assert A.is_contiguous() and A_scale.is_contiguous() and A_scale.dtype == torch.float32
    assert B.is_contiguous(), "weights must be contiguous [E, N, K]"
    assert B_scale.is_contiguous() and B_scale.dtype == torch.float32
    assert sorted_token_ids.stride(0) == 1 and sorted_token_ids.dtype == torch.int32
    assert expert_ids.dtype == torch.int32 and num_tokens_post_padded.dtype == torch.int32
    E, N, K = B.shape
    if w4:
        K *= 2
        assert _is_preshuffled(B), "packed int4 weights must go through preshuffle_moe_weight_int4"
        assert getattr(B_scale, "lo_kmajor", False) and B_scale.shape == (E, K // 128, N), \
            "int4 weight scales must go through preshuffle_moe_scale_int4 ([E, K/128, N])"
    else:
        assert B_scale.shape == (E, (N + 127) // 128, K // 128), "weight scales must be [E, N/128, K/128]"
    assert A.shape[1] == K and A_scale.shape == (A.shape[0], K // 128)
    return E, N, K


def _check_block_extents(sorted_token_ids, expert_ids, block_size_m, num_valid):
    """``expert_ids`` must cover every token block the launch's grid can reach (the blocks ``sorted_token_ids``
    has room for, at most one per routed slot): a kernel may read a block's entry before it knows how many
    blocks are in use."""
    blocks = min(sorted_token_ids.numel() // int(block_size_m), int(num_valid))
    if expert_ids.numel() < blocks:
        raise ValueError(f"expert_ids holds {expert_ids.numel()} entries, the {sorted_token_ids.numel()} sorted ids "
                         f"span {blocks} blocks of {int(block_size_m)}")


def invoke_fused_moe_kernel_int8(A: torch.Tensor, B: torch.Tensor, C: torch.Tensor,
                                 A_scale: torch.Tensor, B_scale: torch.Tensor,
                                 topk_weights: Optional[torch.Tensor],
                                 sorted_token_ids: torch.Tensor, expert_ids: torch.Tensor,
                                 num_tokens_post_padded: torch.Tensor, mul_routed_weight: bool,
                                 top_k: int, config: Dict[str, Any], fused_scale: Optional[bool] = None,
                                 flags: int = 0, global_num_experts: int = 0) -> None:
    """One grouped block-INT8 GEMM stage: C[f] = bf16(sum_kb dot(A[f // top_k], B[e])_kb *
    A_scale * B_scale) (* topk_weights[f]) for every routed slot f (reference:
    invoke_fused_moe_kernel_int8, int8.py:543-626).  ``C`` is [M, topk, N] or [S, N].
    With ``flags=LO_GEMM_W4`` ``B`` is packed int4 from ``preshuffle_moe_weight_int4`` and
    ``B_scale`` is [E, N, K/128] (the stage of w4a8.py:406-478 with K-group scales)."""
    assert topk_weights is not None or not mul_routed_weight
    E, N, K = _check_gemm_inputs(A, A_scale, B, B_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
                                 w4=bool(flags & _lib.LO_GEMM_W4))
    assert C.is_contiguous() and C.shape[-1] == N
    num_valid = C.numel() // N
    _check_block_extents(sorted_token_ids, expert_ids, config["BLOCK_SIZE_M"], num_valid)
    tw = None
    if topk_weights is not None:
        tw = topk_weights
        if tw.dtype != torch.float32 or not tw.is_contiguous():
            tw = tw.to(torch.float32).contiguous()
    with _on_device(A):
        _lib.check(_lib.lib().lo_moe_gemm_block_int8(
            _lib.ptr(A), _lib.ptr(A_scale), _lib.ptr(B), _lib.ptr(B_scale), _lib.ptr(C), _act_dtype(C),
            _lib.ptr(tw), _lib.ptr(sorted_token_ids), _lib.ptr(expert_ids),
            _lib.ptr(num_tokens_post_padded), sorted_token_ids.numel(), num_valid, A.shape[0], E,
            int(global_num_experts or 0), N, K,
            int(top_k), int(config["BLOCK_SIZE_M"]), 1 if mul_routed_weight else 0,
            _scale_flags(fused_scale) | flags | (_lib.LO_GEMM_W_PRESHUFFLED if _is_preshuffled(B) else 0),
            _lib.stream_of(A)))


def invoke_fused_moe_gemm1_silu_quant(A: torch.Tensor, B: torch.Tensor, A_scale: torch.Tensor,
                                      B_scale: torch.Tensor, topk_weights: Optional[torch.Tensor],
                                      sorted_token_ids: torch.Tensor, expert_ids: torch.Tensor,
                                      num_tokens_post_padded: torch.Tensor, mul_routed_weight: bool,
                                      top_k: int, num_valid: int, config: Dict[str, Any],
                                      fused_scale: Optional[bool] = None, flags: int = 0,
                                      global_num_experts: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    """First GEMM with SiLU-and-mul and the 1x128 re-quantisation in its epilogue: the
    sequence int8.py:784-823 in one kernel.  Returns (A2q [num_valid, I] int8,
    A2s [num_valid, I/128] f32); rows of slots routed to non-local experts are not written."""
    assert topk_weights is not None or not mul_routed_weight
    E, N, K = _check_gemm_inputs(A, A_scale, B, B_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
                                 w4=bool(flags & _lib.LO_GEMM_W4))
    I = N // 2
    _check_block_extents(sorted_token_ids, expert_ids, config["BLOCK_SIZE_M"], num_valid)
    a2q = torch.empty(num_valid, I, dtype=torch.int8, device=A.device)
    a2s = torch.empty(num_valid, I // 128, dtype=torch.float32, device=A.device)
    tw = None
    if topk_weights is not None:
        tw = topk_weights
        if tw.dtype != torch.float32 or not tw.is_contiguous():
            tw = tw.to(torch.float32).contiguous()
    with _on_device(A):
        _lib.check(_lib.lib().lo_moe_gemm1_silu_quant_block_int8(
            _lib.ptr(A), _lib.ptr(A_scale), _lib.ptr(B), _lib.ptr(B_scale), _lib.ptr(a2q), _lib.ptr(a2s),
            _lib.LO_BF16, _lib.ptr(tw), _lib.ptr(sorted_token_ids), _lib.ptr(expert_ids),
            _lib.ptr(num_tokens_post_padded), sorted_token_ids.numel(), num_valid, A.shape[0], E,
            int(global_num_experts or 0), I, K,
            int(top_k), int(config["BLOCK_SIZE_M"]), 1 if mul_routed_weight else 0,
            _scale_flags(fused_scale) | flags | (_lib.LO_GEMM_W_PRESHUFFLED if _is_preshuffled(B) else 0),
            _lib.stream_of(A)))
    return a2q, a2s


def invoke_fused_moe_kernel_w4a8(A: torch.Tensor, B: torch.Tensor, C: torch.Tensor, A_scale: torch.Tensor,
                                 B_scale: torch.Tensor, B_zp: Optional[torch.Tensor],
                                 topk_weights: Optional[torch.Tensor], sorted_token_ids: torch.Tensor,
                                 expert_ids: torch.Tensor, num_tokens_post_padded: torch.Tensor,
                                 mul_routed_weight: bool, top_k: int, config: Dict[str, Any],
                                 compute_type=None, block_shape: Optional[List[int]] = None,
                                 global_num_experts: int = 0) -> None:
    """One grouped GEMM stage of the reference's own int4 form (invoke_fused_moe_kernel_w4a8,
    w4a8.py:405-478; kernel :202-401): ``A`` int8 [rows, K], ``B`` packed int4 [E, N, K/2] from
    ``preshuffle_moe_weight_int4``, ``A_scale`` one per row, ``B_scale`` one per weight row.
    C[f] = T(((sum_k A[f // top_k] * w16[e]) [* topk_weights[f]]) * A_scale[f // top_k] * B_scale[e]),
    w16 = int8(nibble << 4).  ``config`` needs ``BLOCK_SIZE_M``."""
    del B_zp  # the reference's kernel takes the pointer and never reads it (b_qzero_ptr, w4a8.py:218)
    assert block_shape is None, "the K-group form goes through fused_experts_impl_w4a8(block_shape=[1, 128])"
    del compute_type
    _require_cuda(A, B, C, A_scale, B_scale, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded)
    assert A.dtype == torch.int8 and B.dtype in (torch.int8, torch.uint8)
    assert A.is_contiguous() and B.is_contiguous() and C.is_contiguous()
    if not getattr(B, "lo_int4", False):
        raise RuntimeError("lightop_amd: pass the weights through preshuffle_moe_weight_int4 once at load time")
    E, N, K2 = B.shape
    K = 2 * K2
    assert A.shape[1] == K and C.shape[-1] == N
    assert A_scale.dtype == torch.float32 and A_scale.is_contiguous() and A_scale.numel() == A.shape[0]
    assert B_scale.dtype == torch.float32 and B_scale.is_contiguous() and B_scale.numel() == E * N
    assert sorted_token_ids.dtype == torch.int32 and expert_ids.dtype == torch.int32
    assert topk_weights is not None or not mul_routed_weight
    num_valid = C.numel() // N
    _check_block_extents(sorted_token_ids, expert_ids, config["BLOCK_SIZE_M"], num_valid)
    tw = None
    if mul_routed_weight:
        tw = topk_weights if topk_weights.dtype == torch.float32 and topk_weights.is_contiguous() \
            else topk_weights.to(torch.float32).contiguous()
    with _on_device(A):
        _lib.check(_lib.lib().lo_moe_gemm_w8a8(
            _lib.ptr(A), _lib.ptr(A_scale), _lib.ptr(B), _lib.ptr(B_scale), _lib.ptr(C), _act_dtype(C),
            _lib.ptr(tw), _lib.ptr(sorted_token_ids), _lib.ptr(expert_ids), _lib.ptr(num_tokens_post_padded),
            sorted_token_ids.numel(), num_valid, A.shape[0], E, int(global_num_experts or 0), N, K, int(top_k),
            int(config["BLOCK_SIZE_M"]), 1 if mul_routed_weight else 0,
            _lib.LO_GEMM_W4 | _lib.LO_GEMM_W_PRESHUFFLED, _lib.stream_of(A)))


def silu_and_mul(out: torch.Tensor, x: torch.Tensor) -> None:
    """out[:, i] = T(T(silu(x[:, i])) * x[:, d + i])  (the op called at int8.py:811)."""
    _require_cuda(out, x)
    assert x.is_contiguous() and out.is_contiguous() and x.shape[-1] == 2 * out.shape[-1]
    I = out.shape[-1]
    rows = out.numel() // I
    with _on_device(x):
        _lib.check(_lib.lib().lo_silu_and_mul(_lib.ptr(x), _act_dtype(x), rows, I, _lib.ptr(out),
                                              _lib.stream_of(x)))


def gelu_and_mul(out: torch.Tensor, x: torch.Tensor) -> None:
    """out[:, i] = T(T(gelu(x[:, i])) * x[:, d + i]), gelu in its erf form (the op called at int8.py:826;
    in-repo twin gelu_and_mul_opt, csrc/kernels/activation_kernels_opt.cu:234-242)."""
    _require_cuda(out, x)
    assert x.is_contiguous() and out.is_contiguous() and x.shape[-1] == 2 * out.shape[-1]
    I = out.shape[-1]
    rows = out.numel() // I
    with _on_device(x):
        _lib.check(_lib.lib().lo_gelu_and_mul(_lib.ptr(x), _act_dtype(x), rows, I, _lib.ptr(out),
                                              _lib.stream_of(x)))


def act_and_mul_group_quant(x: torch.Tensor, activation: str = "silu", row_mask: Optional[torch.Tensor] = None,
                            out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
                            ) -> Tuple[torch.Tensor, torch.Tensor]:
    """The gated activation of ``x`` [rows, 2I] and the 1x128 group quantisation of the result in one
    launch: (q [rows, I] int8, s [rows, I/128] f32).  The pair silu_and_mul / gelu_and_mul +
    per_token_group_quant_int8 of int8.py:811-838.  ``row_mask`` (bool or uint8 [rows], as the alignment
    writes its slot mask): rows whose entry is 0 are neither read nor written.  ``out``: (q, s) to write
    into."""
    _require_cuda(x)
    assert x.is_contiguous() and x.dim() == 2 and x.shape[1] % 256 == 0
    assert activation in ("silu", "gelu")
    rows, I = x.shape[0], x.shape[1] // 2
    if out is None:
        q = torch.empty(rows, I, dtype=torch.int8, device=x.device)
        s = torch.empty(rows, I // 128, dtype=torch.float32, device=x.device)
    else:
        q, s = out
        assert q.is_contiguous() and s.is_contiguous() and q.dtype == torch.int8 and s.dtype == torch.float32
        assert q.shape == (rows, I) and s.shape == (rows, I // 128)
    if row_mask is not None:
        assert row_mask.is_contiguous() and row_mask.numel() == rows and row_mask.element_size() == 1
    with _on_device(x):
        _lib.check(_lib.lib().lo_act_mul_group_quant(
            _lib.ptr(x), _act_dtype(x), _lib.LO_ACT_GELU if activation == "gelu" else _lib.LO_ACT_SILU, rows, I,
            _lib.ptr(q), _lib.ptr(s), None if row_mask is None else _lib.ptr(row_mask), _lib.stream_of(x)))
    return q, s


@functools.lru_cache(maxsize=256)
def fused_experts_workspace_bytes(M: int, top_k: int, H: int, I: int, num_experts: int,
                                  block_size_m: int = 0) -> int:
    """Bytes of scratch one whole-path call needs (0: enough for every block size)."""
    n = _lib.lib().lo_fused_experts_workspace_bytes(M, top_k, H, I, num_experts, block_size_m)
    _lib.check(n)
    return int(n)


def fused_experts_workspace_views(workspace: torch.Tensor, M: int, top_k: int, H: int, I: int, num_experts: int,
                                  block_size_m: int) -> Dict[str, torch.Tensor]:
    """The intermediates a whole-path call left in ``workspace`` (the uint8 tensor given to it as
    ``lightop_amd_workspace``), as tensors: a1q, a1s, sorted_ids, expert_ids, num_tokens_post_pad,
    a2q, a2s, slot_mask.  ``block_size_m`` must be the block size the call used."""
    lib = _lib.lib()
    base = (workspace.data_ptr() + 255) // 256 * 256 - workspace.data_ptr()
    S = M * top_k
    cap = S + num_experts * (block_size_m - 1)
    if S < num_experts:
        cap = min(cap, S * block_size_m)
    spec = [("a1q", torch.int8, (M, H)), ("a1s", torch.float32, (M, H // 128)), ("sorted_ids", torch.int32, (cap,)),
            ("expert_ids", torch.int32, ((cap + block_size_m - 1) // block_size_m,)),
            ("num_tokens_post_pad", torch.int32, (1,)), ("a2q", torch.int8, (S, I)),
            ("a2s", torch.float32, (S, I // 128)), ("slot_mask", torch.uint8, (S,))]
    views = {}
    for which, (name, dt, shape) in enumerate(spec):
        off = lib.lo_fused_experts_workspace_offset(which, M, top_k, H, I, num_experts, block_size_m)
        _lib.check(off)
        n = 1
        for d in shape:
            n *= d
        nbytes = n * torch.empty((), dtype=dt).element_size()
        views[name] = workspace[base + off: base + off + nbytes].view(dt).view(shape)
    return views


def fused_experts_impl_int8(hidden_states: torch.Tensor,
                            w1: torch.Tensor,
                            w2: torch.Tensor,
                            topk_weights: torch.Tensor,
                            topk_ids: torch.Tensor,
                            cache13: torch.Tensor,
                            inplace: bool = False,
                            activation: str = "silu",
                            apply_router_weight_on_input: bool = False,
                            use_fp8_w8a8: bool = False,
                            use_int8_w8a8: bool = False,
                            use_int8_w8a16: bool = False,
                            use_int4_w4a16: bool = False,
                            per_channel_quant: bool = False,
                            global_num_experts: int = -1,
                            expert_map: Optional[torch.Tensor] = None,
                            w1_scale: Optional[torch.Tensor] = None,
                            w2_scale: Optional[torch.Tensor] = None,
                            w1_zp: Optional[torch.Tensor] = None,
                            w2_zp: Optional[torch.Tensor] = None,
                            a1_scale: Optional[torch.Tensor] = None,
                            a2_scale: Optional[torch.Tensor] = None,
                            block_shape: Optional[List[int]] = None,
                            use_nn_moe: Optional[bool] = False,
                            routed_scaling_factor: Optional[float] = 1.0,
                            shared_output: Optional[torch.Tensor] = None,
                            i_q: Optional[torch.Tensor] = None,
                            i_s: Optional[torch.Tensor] = None, **_):
    """Fused MoE experts with block-quantised INT8 weights (128x128 blocks, fp32 scales) and
    activations quantised per 1x128 group on the fly.

    Same signature as the reference (int8.py:628-656).  This build implements the branches
    ``use_int8_w8a8=True, block_shape=[128, 128]`` and ``use_int8_w8a8=True,
    per_channel_quant=True, block_shape=None`` (one scale per token and per weight row,
    ``w1_scale`` [E, 2I, 1], ``w2_scale`` [E, H, 1]) with ``activation="silu"`` or ``"gelu"`` (the
    latter without the fused epilogue: one more launch and a bf16 round trip of [S, 2I]); every other
    combination raises.  ``hidden_states`` is bfloat16, float16 or, in the block form, float32 (float16 and
    float32 rows take the path without the fused epilogue as well; every value between the stages is rounded
    to float16, or not at all, as the reference's compute_type does, int8.py:689-696; float32 rows go
    through the weight-streaming kernel at every size); float32 with per-channel scales raises.
    ``cache13`` is the caller's workspace (dtype of ``hidden_states``,
    at least ``min(M, CHUNK) * topk * max(2I, H)`` elements); its first ``M*topk*H``
    elements receive the second GEMM's per-slot output.  The top-k reduction is always
    performed: ``out = routed_scaling_factor * sum_k(...) (+ shared_output)``.
    Unknown keyword arguments are ignored, as in the reference.
    """
    extra = _  # private knobs: lightop_amd_flags, lightop_amd_block_size_m, lightop_amd_workspace
    # Check constraints (int8.py:658-667).
    assert use_int8_w8a8 or use_fp8_w8a8
    assert hidden_states.shape[1] == w1.shape[2], "Hidden size mismatch"
    assert topk_weights.shape == topk_ids.shape, "topk shape mismatch"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.stride(-1) == 1, "Stride of last dimension must be 1"
    assert w2.stride(-1) == 1, "Stride of last dimension must be 1"
    assert hidden_states.dtype in [torch.float32, torch.float16, torch.bfloat16]
    if not use_int8_w8a8 or use_fp8_w8a8 or use_int8_w8a16 or use_int4_w4a16:
        raise NotImplementedError("lightop_amd: only use_int8_w8a8=True is built")
    channel = bool(per_channel_quant) and block_shape is None  # int8.py:285-295: per-token x per-channel
    if not channel and (per_channel_quant or block_shape is None or list(block_shape) != [128, 128]):
        raise NotImplementedError("lightop_amd: block_shape must be [128, 128], or None with per_channel_quant=True")
    if activation not in ("silu", "gelu"):
        raise ValueError(f"Unsupported FusedMoe activation: {activation}")
    if hidden_states.dtype == torch.float32 and channel:
        # the reference's per-channel GEMM refuses them too (moe_w8a8_gemm: bf16 or fp16 outputs only,
        # csrc/moe_gemm/w8a8/moe_w8a8.cu:2585-2784)
        raise NotImplementedError("lightop_amd: per-channel scales take bfloat16 or float16 hidden_states")
    assert w1_scale is not None and w2_scale is not None
    del w1_zp, w2_zp, a1_scale, a2_scale, use_nn_moe
    # int8.py:291-293: the per-channel form takes the caller's own per-token quantisation of the input
    # (the fused RMS-norm + quant upstream) when the flag is set; the block form never does (:297-301).
    prequant = None
    if channel and envs.LMSLIM_USE_FUSED_RMS_QUANT and i_q is not None and i_s is not None:
        assert i_q.dtype == torch.int8 and i_q.is_contiguous() and i_q.shape == hidden_states.shape
        assert i_s.numel() == hidden_states.shape[0]
        prequant = (i_q, i_s if i_s.dtype == torch.float32 and i_s.is_contiguous()
                    else i_s.to(torch.float32).contiguous())
        _require_cuda(*prequant)
    _require_cuda(hidden_states, w1, w2, topk_weights, topk_ids, cache13, w1_scale, w2_scale,
                  expert_map, shared_output)

    num_tokens, H = hidden_states.shape
    E, N = w1.shape[0], w1.shape[1]
    I = N // 2
    assert w2.shape == (E, H, I), "w2 must be [E, H, I]"
    assert w1.is_contiguous() and w2.is_contiguous(), "expert weights must be contiguous"
    assert w1.dtype == torch.int8 and w2.dtype == torch.int8
    if channel:  # one scale per weight row: [E, N, 1] as the reference's tests hold them, or [E, N]
        assert w1_scale.numel() == E * N and w2_scale.numel() == E * H, "per-channel scales must be [E, N(, 1)]"
        w1_scale, w2_scale = w1_scale.reshape(E, N), w2_scale.reshape(E, H)
    else:
        assert w1_scale.shape == (E, N // 128, H // 128) and w2_scale.shape == (E, H // 128, I // 128)
    if global_num_experts == -1:
        global_num_experts = E
    top_k_num = topk_ids.shape[1]
    CHUNK_SIZE = envs.LMSLIM_FUSED_MOE_CHUNK_SIZE
    M = min(num_tokens, CHUNK_SIZE)
    assert cache13.dtype == hidden_states.dtype and cache13.is_contiguous()
    assert cache13.numel() >= M * top_k_num * max(N, H), "cache13 is too small"

    flags = int(extra.get("lightop_amd_flags", 0)) | (_lib.LO_FUSED_ACT_GELU if activation == "gelu" else 0)
    if extra.get("lightop_amd_weights_preshuffled", False):
        flags |= _lib.LO_GEMM_W_PRESHUFFLED
    return _run_fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, cache13, inplace,
                              apply_router_weight_on_input, global_num_experts, expert_map, w1_scale, w2_scale,
                              routed_scaling_factor, shared_output, I, flags,
                              int(extra.get("lightop_amd_block_size_m", 0)), channel=channel,
                              workspace=extra.get("lightop_amd_workspace"), prequant=prequant, chunk_size=CHUNK_SIZE)


def fused_experts_impl_w4a8(hidden_states: torch.Tensor,
                            w1: torch.Tensor,
                            w2: torch.Tensor,
                            topk_weights: torch.Tensor,
                            topk_ids: torch.Tensor,
                            cache13: torch.Tensor,
                            inplace: bool = False,
                            activation: str = "silu",
                            apply_router_weight_on_input: bool = False,
                            global_num_experts: int = -1,
                            expert_map: Optional[torch.Tensor] = None,
                            w1_scale: Optional[torch.Tensor] = None,
                            w2_scale: Optional[torch.Tensor] = None,
                            w1_zp: Optional[torch.Tensor] = None,
                            w2_zp: Optional[torch.Tensor] = None,
                            a1_scale: Optional[torch.Tensor] = None,
                            a2_scale: Optional[torch.Tensor] = None,
                            block_shape: Optional[List[int]] = None,
                            use_nn_moe: Optional[bool] = False,
                            routed_scaling_factor: Optional[float] = 1.0,
                            shared_output: Optional[torch.Tensor] = None, **_):
    """Fused MoE experts with packed int4 weights and int8 activations (signature of the
    reference's fused_experts_impl_w4a8, w4a8.py:480-501).

    ``w1`` [E, 2I, H/2] and ``w2`` [E, H, I/2] hold two int4 per byte along K (even k in the high
    nibble, the reference's order) and have been passed through ``preshuffle_moe_weight_int4``.

    ``block_shape=None`` is the reference's own form (w4a8.py:480-658): activations quantised per
    token, ``w1_scale`` [E, 2I(, 1)] and ``w2_scale`` [E, H(, 1)] one fp32 scale per weight row,
    both applied in the epilogue of each stage to a sum that keeps the factor 16 of the nibbles
    (w4a8.py:375-395).

    ``block_shape=[1, 128]`` is the K-group form: one fp32 scale per weight row and 128-wide K
    group (``w1_scale`` [E, 2I, H/128], ``w2_scale`` [E, H, I/128], or their load-time form from
    ``preshuffle_moe_scale_int4``), activations quantised per 1x128 group on the fly.

    ``activation``: "silu" or "gelu"; the reduce is always performed.
    """
    extra = _
    assert hidden_states.shape[1] == w1.shape[2] * 2, "Hidden size mismatch"  # w4a8.py:503
    assert topk_weights.shape == topk_ids.shape, "topk shape mismatch"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.stride(-1) == 1, "Stride of last dimension must be 1"
    assert w2.stride(-1) == 1, "Stride of last dimension must be 1"
    assert hidden_states.dtype in [torch.float32, torch.float16, torch.bfloat16]
    channel = block_shape is None
    if not channel and list(block_shape) != [1, 128]:
        raise NotImplementedError("lightop_amd: W4A8 is built for block_shape=None (per token x per channel) "
                                  "and for K-group scales, block_shape=[1, 128]")
    if activation not in ("silu", "gelu"):
        raise ValueError(f"Unsupported FusedMoe activation: {activation}")
    if hidden_states.dtype == torch.float32:
        raise NotImplementedError("lightop_amd: hidden_states must be bfloat16 or float16")
    if not channel and (w1_zp is not None or w2_zp is not None):
        raise NotImplementedError("lightop_amd: W4A8 zero points are not built (symmetric int4 only)")
    # block_shape=None: the reference passes w1_zp / w2_zp to a kernel that never reads them
    # (b_qzero_ptr, w4a8.py:218): they are ignored here as well
    assert w1_scale is not None and w2_scale is not None
    del a1_scale, a2_scale, use_nn_moe
    _require_cuda(hidden_states, w1, w2, topk_weights, topk_ids, cache13, w1_scale, w2_scale, expert_map,
                  shared_output)
    num_tokens, H = hidden_states.shape
    E, N = w1.shape[0], w1.shape[1]
    I = N // 2
    assert w2.shape == (E, H, I // 2), "w2 must be packed [E, H, I/2]"
    assert w1.is_contiguous() and w2.is_contiguous(), "expert weights must be contiguous"
    assert w1.dtype in (torch.int8, torch.uint8) and w2.dtype == w1.dtype
    if not (getattr(w1, "lo_int4", False) and getattr(w2, "lo_int4", False)):
        raise RuntimeError("lightop_amd: pass w1 and w2 through preshuffle_moe_weight_int4 once at load time")
    if global_num_experts == -1:
        global_num_experts = E
    if channel:
        assert w1_scale.numel() == E * N and w2_scale.numel() == E * H, "scales must be [E, 2I] and [E, H]"
        M = min(num_tokens, envs.LMSLIM_FUSED_MOE_CHUNK_SIZE)
        assert cache13.dtype == hidden_states.dtype and cache13.is_contiguous()
        assert cache13.numel() >= M * topk_ids.shape[1] * max(N, H), "cache13 is too small"
        flags = int(extra.get("lightop_amd_flags", 0)) | _lib.LO_GEMM_W4 | (
        _lib.LO_FUSED_ACT_GELU if activation == "gelu" else 0)
        return _run_fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, cache13, inplace,
                                  apply_router_weight_on_input, global_num_experts, expert_map,
                                  w1_scale.reshape(E, N), w2_scale.reshape(E, H), routed_scaling_factor,
                                  shared_output, I, flags, int(extra.get("lightop_amd_block_size_m", 0)),
                                  channel=True, workspace=extra.get("lightop_amd_workspace"))
    # scales: [E, N, K/128] as a checkpoint holds them (transposed here, on every call) or, better,
    # already K-group-major from preshuffle_moe_scale_int4
    if not getattr(w1_scale, "lo_kmajor", False):
        assert w1_scale.shape == (E, N, H // 128), "w1_scale must be [E, 2I, H/128]"
        w1_scale = preshuffle_moe_scale_int4(w1_scale)
    if not getattr(w2_scale, "lo_kmajor", False):
        assert w2_scale.shape == (E, H, I // 128), "w2_scale must be [E, H, I/128]"
        w2_scale = preshuffle_moe_scale_int4(w2_scale)
    assert w1_scale.shape == (E, H // 128, N) and w2_scale.shape == (E, I // 128, H)
    M = min(num_tokens, envs.LMSLIM_FUSED_MOE_CHUNK_SIZE)
    assert cache13.dtype == hidden_states.dtype and cache13.is_contiguous()
    assert cache13.numel() >= M * topk_ids.shape[1] * max(N, H), "cache13 is too small"
    flags = int(extra.get("lightop_amd_flags", 0)) | _lib.LO_GEMM_W4 | (
        _lib.LO_FUSED_ACT_GELU if activation == "gelu" else 0)
    return _run_fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, cache13, inplace,
                              apply_router_weight_on_input, global_num_experts, expert_map, w1_scale, w2_scale,
                              routed_scaling_factor, shared_output, I, flags,
                              int(extra.get("lightop_amd_block_size_m", 0)), workspace=extra.get("lightop_amd_workspace"))


@functools.lru_cache(maxsize=256)
def _workspace_bytes_cached(M: int, top_k: int, H: int, I: int, num_experts: int) -> int:
    return fused_experts_workspace_bytes(M, top_k, H, I, num_experts, 0)


_ws_cache: Dict[Tuple[int, int], torch.Tensor] = {}


def _cached_workspace(nbytes: int, device: torch.device, stream_key: int) -> torch.Tensor:
    """The library's scratch for a whole-path call, kept per (device, stream) and grown on demand, so that a
    serving loop does not allocate on every call (the reference keeps its own workspace, cache13, in a
    process-wide cache the same way: vllm_compat/fused_moe_cache.py:19-24).  Calls on one stream run in
    order, so they can share it; calls on different streams get workspaces of their own."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream_key)
    ws = _ws_cache.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _ws_cache[key] = ws
    return ws


def _run_fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, cache13, inplace, apply_router_weight_on_input,
                       global_num_experts, expert_map, w1_scale, w2_scale, routed_scaling_factor, shared_output,
                       I, flags, block_size_m, channel=False, workspace=None, prequant=None, chunk_size=None):
    """Chunk loop shared by the block-INT8, per-channel and W4A8 entry points (int8.py:703-888)."""
    num_tokens, H = hidden_states.shape
    E = w1.shape[0]
    top_k_num = topk_ids.shape[1]
    CHUNK_SIZE = envs.LMSLIM_FUSED_MOE_CHUNK_SIZE if chunk_size is None else chunk_size
    M = min(num_tokens, CHUNK_SIZE)
    out_hidden_states = hidden_states if inplace else torch.empty_like(hidden_states)
    if num_tokens == 0:
        return out_hidden_states

    w1_scale = w1_scale if w1_scale.dtype == torch.float32 and w1_scale.is_contiguous() \
        else w1_scale.to(torch.float32).contiguous()
    w2_scale = w2_scale if w2_scale.dtype == torch.float32 and w2_scale.is_contiguous() \
        else w2_scale.to(torch.float32).contiguous()
    if topk_weights.dtype != torch.float32 or not topk_weights.is_contiguous():
        topk_weights = topk_weights.to(torch.float32).contiguous()
    if not topk_ids.is_contiguous():
        topk_ids = topk_ids.contiguous()
    if expert_map is not None and (expert_map.dtype != torch.int32 or not expert_map.is_contiguous()):
        expert_map = expert_map.to(torch.int32).contiguous()
    if shared_output is not None:
        assert shared_output.shape == hidden_states.shape and shared_output.dtype == hidden_states.dtype
        shared_output = shared_output.contiguous()

    lib = _lib.lib()
    ws_bytes = _workspace_bytes_cached(M, top_k_num, H, I, global_num_experts)
    stream_handle = torch.cuda.current_stream(hidden_states.device).cuda_stream
    if workspace is None:
        workspace = _cached_workspace(ws_bytes, hidden_states.device, stream_handle)
        ws_bytes = workspace.numel()
    else:  # the caller's own scratch (tests read the intermediates out of it afterwards)
        assert workspace.dtype == torch.uint8 and workspace.is_contiguous() and workspace.numel() >= ws_bytes
        assert workspace.device == hidden_states.device
        ws_bytes = workspace.numel()
    ws_ptr = (workspace.data_ptr() + 255) // 256 * 256
    ws_avail = ws_bytes - (ws_ptr - workspace.data_ptr())
    assert _is_preshuffled(w1) == _is_preshuffled(w2), "preshuffle both w1 and w2 or neither"
    if _is_preshuffled(w1):
        flags |= _lib.LO_GEMM_W_PRESHUFFLED

    from . import tile_files

    use_files = block_size_m == 0 and tile_files.json_dir() is not None
    w4 = bool(flags & _lib.LO_GEMM_W4)
    file_shape = None if channel else ([1, 128] if w4 else [128, 128])
    with _on_device(hidden_states):
        stream = ctypes_void(stream_handle)
        for chunk in range((num_tokens // CHUNK_SIZE) + 1):
            begin, end = chunk * CHUNK_SIZE, min((chunk + 1) * CHUNK_SIZE, num_tokens)
            m = end - begin
            if m <= 0:
                break
            x = hidden_states[begin:end]
            if use_files:  # a tuning file under TRITON_JSON_DIR wins over the compiled-in table
                block_size_m = tile_files.block_size_m(m, E, 2 * I, H, I, top_k_num, file_shape, int4=w4)
            if prequant is not None:  # the chunk's rows of the caller's quantised input
                entry = lib.lo_fused_experts_channel_int8_prequant
                head = (_lib.ptr(prequant[0][begin:end]), _lib.ptr(prequant[1].reshape(-1)[begin:end]))
            else:
                entry = lib.lo_fused_experts_channel_int8 if channel else lib.lo_fused_experts_block_int8
                head = (_lib.ptr(x),)
            _lib.check(entry(
                *head, _act_dtype(x), m, H, I, E, global_num_experts, top_k_num,
                _lib.ptr(w1), _lib.ptr(w1_scale), _lib.ptr(w2), _lib.ptr(w2_scale),
                _lib.ptr(topk_weights[begin:end]), _lib.ptr(topk_ids[begin:end]), _ids_dtype(topk_ids),
                _lib.ptr(expert_map), 1 if apply_router_weight_on_input else 0,
                float(routed_scaling_factor), _lib.ptr(None if shared_output is None else shared_output[begin:end]),
                _lib.ptr(cache13), _lib.ptr(out_hidden_states[begin:end]),
                ctypes_void(ws_ptr), ws_avail, block_size_m, flags, stream))
    return out_hidden_states


def ctypes_void(addr: int):
    return ctypes.c_void_p(addr)


__all__ = ["fused_experts_impl_int8", "fused_experts_impl_w4a8", "get_w8a8moe_json", "get_moe_cuda_config",
           "preshuffle_moe_weight",
           "preshuffle_moe_weight_int4", "preshuffle_moe_scale_int4", "invoke_fused_moe_kernel_int8",
           "invoke_fused_moe_kernel_w4a8",
           "invoke_fused_moe_gemm1_silu_quant", "silu_and_mul", "gelu_and_mul", "act_and_mul_group_quant", "fused_experts_workspace_bytes",
           "fused_experts_workspace_views", "moe_gemm_w8a8"]
