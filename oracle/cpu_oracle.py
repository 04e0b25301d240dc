"""ctypes front end of the C oracle (oracle/moe_oracle.c).  TEST INFRASTRUCTURE ONLY.

Nothing in ``lightop_amd`` may import this module: it is the checker used by
``tests/``, ``__graft_entry__.smoke()`` and the cpu-baseline leg of ``bench.py``.
All functions take and return torch CPU tensors; bf16 tensors are handed to C
as their raw 16-bit patterns.
"""
from __future__ import annotations

import contextlib
import ctypes
import os
import subprocess
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libmoe_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a few seconds).  Returns the .so path."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
        os.path.join(_HERE, "moe_oracle.c")
    ):
        subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_SO)
        _lib.orc_expf.restype = ctypes.c_float
        _lib.orc_expf.argtypes = [ctypes.c_float]
        _lib.orc_bf16_to_f32.restype = ctypes.c_float
        _lib.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.orc_f32_to_bf16.restype = ctypes.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.orc_silu_bf16.restype = ctypes.c_uint16
        _lib.orc_silu_bf16.argtypes = [ctypes.c_uint16]
        _lib.orc_silu_bf16_libm.restype = ctypes.c_uint16
        _lib.orc_silu_bf16_libm.argtypes = [ctypes.c_uint16]
    return _lib


SCALE_ORDERS = ("contract", "separate")


@contextlib.contextmanager
def scale_order(order: str):
    """Scale arithmetic of the block-form GEMMs per 128-wide K block inside the ``with`` block:
    "contract" (the default: acc = fma(f32(d) * a_s, b_s, acc)) or "separate"
    (acc = acc + (f32(d) * a_s) * b_s)."""
    assert order in SCALE_ORDERS, order
    lib().orc_set_scale_order(ctypes.c_int(1 if order == "contract" else 0))
    try:
        yield order
    finally:
        lib().orc_set_scale_order(ctypes.c_int(1))


def _p(t: Optional[torch.Tensor]):
    if t is None:
        return ctypes.c_void_p(0)
    assert t.device.type == "cpu" and t.is_contiguous(), "oracle wants contiguous CPU tensors"
    return ctypes.c_void_p(t.data_ptr())


def _i64(v):
    return ctypes.c_int64(int(v))


def _i32(v):
    return ctypes.c_int32(int(v))


def align_buffer_sizes(numel: int, num_experts: int, block_size: int, pad_sorted_ids: bool = False):
    """Buffer extents of moe_align_block_size.py:80-93."""
    max_pad = numel + num_experts * (block_size - 1)
    if pad_sorted_ids:
        max_pad = (max_pad + block_size - 1) // block_size * block_size
    if numel < num_experts:
        max_pad = min(numel * block_size, max_pad)
    return max_pad, (max_pad + block_size - 1) // block_size


def moe_align_block_size(topk_ids, block_size, num_experts, expert_map=None,
                         pad_sorted_ids=False, ignore_invalid_experts=False, num_local_tokens=None):
    """With num_local_tokens only the slots of the first that many tokens are aligned; the pad
    value and the buffer sizes stay those of the whole batch (moe_align_sum_kernels.cu:32-45)."""
    ids = topk_ids.reshape(-1).to(torch.int32).contiguous()
    S = ids.numel()
    n_eff = S if num_local_tokens is None else max(0, min(S, int(num_local_tokens) * topk_ids.shape[-1]))
    max_pad, max_blocks = align_buffer_sizes(S, num_experts, block_size, pad_sorted_ids)
    sorted_ids = torch.empty(max_pad, dtype=torch.int32)
    expert_ids = torch.empty(max_blocks, dtype=torch.int32)
    ntpp = torch.zeros(1, dtype=torch.int32)
    emap = None if expert_map is None else expert_map.to(torch.int32).contiguous()
    rc = lib().orc_moe_align_block_size(
        _p(ids[:n_eff].contiguous()), _i64(n_eff), _i32(num_experts), _i32(block_size), _p(emap),
        ctypes.c_int(1 if ignore_invalid_experts else 0), _p(sorted_ids), _i64(max_pad),
        _p(expert_ids), _i64(max_blocks), _p(ntpp))
    if rc != 0:
        raise RuntimeError("oracle moe_align_block_size: id out of range or buffer too small")
    if n_eff != S:
        sorted_ids[sorted_ids == n_eff] = S  # valid slot ids are below n_eff, so this only hits pads
    return sorted_ids, expert_ids, ntpp


def align_slot_mask(topk_ids, expert_map=None, num_local_tokens=None):
    """expert_mask output of the alignment op: True where the slot belongs to a local token and
    its expert is on this rank (moe_align_sum_kernels.cu:73-79, :147)."""
    ids = topk_ids.reshape(-1).long()
    S = ids.numel()
    n_eff = S if num_local_tokens is None else max(0, min(S, int(num_local_tokens) * topk_ids.shape[-1]))
    mask = torch.ones(S, dtype=torch.bool) if expert_map is None else expert_map.long()[ids] >= 0
    mask[n_eff:] = False
    return mask


@contextlib.contextmanager
def _elements_of(t):
    """The C oracle reads and writes 16-bit floats as bf16 unless told otherwise: switch it to IEEE half
    around a call whose tensors are torch.float16."""
    assert t.dtype in (torch.bfloat16, torch.float16)
    lib().orc_set_dtype(ctypes.c_int(1 if t.dtype == torch.float16 else 0))
    try:
        yield t.dtype
    finally:
        lib().orc_set_dtype(ctypes.c_int(0))


def per_token_group_quant_int8(x, group_size=128, eps=1e-10):
    assert group_size == 128
    x = x.contiguous()
    C = x.shape[-1]
    R = x.numel() // C
    q = torch.empty(x.shape, dtype=torch.int8)
    s = torch.empty(x.shape[:-1] + (C // 128,), dtype=torch.float32)
    if x.dtype == torch.float32:
        lib().orc_group_quant_int8_f32(_p(x), _i64(R), _i64(C), ctypes.c_float(eps), _p(q), _p(s))
        return q, s
    with _elements_of(x):
        lib().orc_group_quant_int8(_p(x), _i64(R), _i64(C), ctypes.c_float(eps), _p(q), _p(s))
    return q, s


def per_token_quant_int8(x):
    """One scale per row, round to nearest even (int8_utils.py:20-44): q [.., C] int8, s [.., 1] f32."""
    x = x.contiguous()
    C = x.shape[-1]
    R = x.numel() // C
    q = torch.empty(x.shape, dtype=torch.int8)
    s = torch.empty(x.shape[:-1] + (1,), dtype=torch.float32)
    with _elements_of(x):
        lib().orc_per_token_quant_int8(_p(x), _i64(R), _i64(C), _p(q), _p(s))
    return q, s


def fuse_silu_mul_quant(c1, return_act=False):
    """c1 [S, 2I] bf16 -> q [S, I] int8, s [S, 1] f32 (fuse_silu_mul_quant.cu:90-133)."""
    S, N = c1.shape
    q = torch.empty(S, N // 2, dtype=torch.int8)
    s = torch.empty(S, 1, dtype=torch.float32)
    act = torch.empty(S, N // 2, dtype=c1.dtype) if return_act else None
    with _elements_of(c1):
        lib().orc_fuse_silu_mul_quant(_p(c1.contiguous()), _i64(S), _i64(N // 2), _p(q), _p(s), _p(act))
    return (q, s, act) if return_act else (q, s)


def moe_gemm_w8a8(A, As, W, Ws, sorted_ids, expert_ids, ntpp, topk_w, mul_routed, top_k, num_valid,
                  block_size, dump_acc=False, out=None):
    """Per-channel grouped GEMM: As one scale per row of A, Ws [E, N(, 1)] one per weight row.
    Returns C [num_valid, N] bf16 (and the whole-K int32 sums when dump_acc)."""
    E, N, K = W.shape
    C = torch.zeros(num_valid, N, dtype=torch.bfloat16) if out is None else out
    acc = torch.zeros(num_valid, N, dtype=torch.int32) if dump_acc else None
    tw = None if topk_w is None else topk_w.reshape(-1).to(torch.float32).contiguous()
    lib().orc_moe_gemm_w8a8(
        _p(A.contiguous()), _p(As.reshape(-1).contiguous()), _p(W.contiguous()), _p(Ws.reshape(E, N).contiguous()),
        _p(sorted_ids), _p(expert_ids), _p(ntpp), _p(tw), ctypes.c_int(1 if mul_routed else 0),
        _i32(top_k), _i64(num_valid), _i64(N), _i64(K), _i32(block_size), _p(C), _p(acc))
    return (C, acc) if dump_acc else C


def unpack_int4(w4):
    """Packed signed int4 [..., K/2] (uint8 or int8; even k in the high nibble) -> int8 [..., K]."""
    p = w4.contiguous().view(torch.uint8)
    out = torch.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=torch.int8)
    lib().orc_unpack_int4(_p(p), _i64(p.numel()), _p(out))
    return out


def pack_int4(w):
    """int8 values in [-8, 7], [..., K] -> packed uint8 [..., K/2] in the reference's nibble order
    (inverse of unpack_int4; plain torch, used to build test inputs)."""
    u = (w.to(torch.int16) & 15).to(torch.uint8)
    return ((u[..., 0::2] << 4) | u[..., 1::2]).contiguous()


def moe_gemm_w4a8(A, As, W4, Ws, *args, **kwargs):
    """Grouped GEMM with packed int4 weights [E, N, K/2] and one scale per row and K group,
    Ws [E, N, K/128]; other arguments as moe_gemm_block_int8."""
    return moe_gemm_block_int8(A, As, unpack_int4(W4), Ws, *args, _fn="orc_moe_gemm_rowscale_int8", **kwargs)


def moe_gemm_w4a8_channel(A, As, W4, Ws, sorted_ids, expert_ids, ntpp, topk_w, mul_routed, top_k, num_valid,
                          block_size, dump_acc=False, out=None):
    """The reference's own int4 stage (w4a8.py:341-395): W4 [E, N, K/2] packed bytes, As one scale
    per row of A, Ws [E, N(, 1)].  Returns C [num_valid, N] bf16 (and the int32 sums, factor 16
    of the nibbles included, when dump_acc)."""
    E, N, K2 = W4.shape
    C = torch.zeros(num_valid, N, dtype=torch.bfloat16) if out is None else out
    acc = torch.zeros(num_valid, N, dtype=torch.int32) if dump_acc else None
    tw = None if topk_w is None else topk_w.reshape(-1).to(torch.float32).contiguous()
    lib().orc_moe_gemm_w4a8_channel(
        _p(A.contiguous()), _p(As.reshape(-1).contiguous()), _p(W4.contiguous().view(torch.uint8)),
        _p(Ws.reshape(E, N).contiguous()), _p(sorted_ids), _p(expert_ids), _p(ntpp), _p(tw),
        ctypes.c_int(1 if mul_routed else 0), _i32(top_k), _i64(num_valid), _i64(N), _i64(2 * K2),
        _i32(block_size), _p(C), _p(acc))
    return (C, acc) if dump_acc else C


def moe_gemm_block_int8(A, As, W, Ws, sorted_ids, expert_ids, ntpp, topk_w, mul_routed,
                        top_k, num_valid, block_size, dump_acc=False, out=None, _fn="orc_moe_gemm_block_int8"):
    """One grouped-GEMM stage.  Returns C[num_valid, N] bf16 (and the int32
    per-128-block dot products when dump_acc).  With a float32 ``out`` the sums are stored unrounded."""
    E, N, K = W.shape
    C = torch.zeros(num_valid, N, dtype=torch.bfloat16) if out is None else out
    if C.dtype == torch.float32:
        assert _fn == "orc_moe_gemm_block_int8"
        _fn = "orc_moe_gemm_block_int8_f32"
    acc = torch.zeros(num_valid, N, K // 128, dtype=torch.int32) if dump_acc else None
    tw = None if topk_w is None else topk_w.reshape(-1).to(torch.float32).contiguous()
    with (_elements_of(C) if C.dtype != torch.float32 else contextlib.nullcontext()):  # a float16 ``out``: rounded to half
        getattr(lib(), _fn)(
            _p(A.contiguous()), _p(As.contiguous()), _p(W.contiguous()), _p(Ws.contiguous()),
            _p(sorted_ids), _p(expert_ids), _p(ntpp), _p(tw), ctypes.c_int(1 if mul_routed else 0),
            _i32(top_k), _i64(num_valid), _i64(N), _i64(K), _i32(block_size), _p(C), _p(acc))
    return (C, acc) if dump_acc else C


def _act_and_mul_f32(c1, activation):
    S, N = c1.shape
    act = torch.empty(S, N // 2, dtype=torch.float32)
    lib().orc_act_and_mul_f32(_p(c1.contiguous()), _i64(S), _i64(N // 2), ctypes.c_int(activation), _p(act))
    return act


def silu_and_mul(c1):
    S, N = c1.shape
    if c1.dtype == torch.float32:
        return _act_and_mul_f32(c1, 0)
    act = torch.empty(S, N // 2, dtype=c1.dtype)
    with _elements_of(c1):
        lib().orc_silu_and_mul(_p(c1.contiguous()), _i64(S), _i64(N // 2), _p(act))
    return act


def gelu_and_mul(c1):
    """act = bf16(bf16(gelu(g)) * u), gelu with erf (activation_kernels_opt.cu:234-242)."""
    S, N = c1.shape
    if c1.dtype == torch.float32:
        return _act_and_mul_f32(c1, 1)
    act = torch.empty(S, N // 2, dtype=c1.dtype)
    with _elements_of(c1):
        lib().orc_gelu_and_mul(_p(c1.contiguous()), _i64(S), _i64(N // 2), _p(act))
    return act


def activation_table(activation="gelu", dtype=torch.bfloat16):
    """T(act(g)) for every 16-bit pattern g of the type T, as int16 [65536]."""
    fn = lib().orc_gelu_bf16 if activation == "gelu" else lib().orc_silu_bf16
    fn.restype = ctypes.c_uint16
    fn.argtypes = [ctypes.c_uint16]
    with _elements_of(torch.empty(0, dtype=dtype)):
        return torch.tensor([fn(i) for i in range(65536)], dtype=torch.int32).to(torch.int16)


def gelu_bf16_table():
    """bf16(gelu(g)) for every bf16 pattern g, as int16 [65536]."""
    return activation_table("gelu", torch.bfloat16)


def moe_sum(inp, bias=None, factor=1.0, num_local_tokens=None, out=None):
    """With num_local_tokens, rows from that index on keep what ``out`` held."""
    M, k, H = inp.shape
    res = torch.empty(M, H, dtype=inp.dtype)
    if inp.dtype == torch.float32:
        lib().orc_moe_sum_f32(_p(inp.contiguous()), _i64(M), _i32(k), _i64(H),
                              _p(None if bias is None else bias.contiguous()), ctypes.c_float(factor), _p(res))
    else:
        with _elements_of(inp):
            lib().orc_moe_sum(_p(inp.contiguous()), _i64(M), _i32(k), _i64(H),
                              _p(None if bias is None else bias.contiguous()), ctypes.c_float(factor), _p(res))
    if num_local_tokens is not None:
        n = max(0, min(M, int(num_local_tokens)))
        res[n:] = out[n:]
    return res


def topk_softmax(gating, topk, renormalize=False):
    """gating [T, E] (any float dtype; widened to fp32) -> weights [T,k] f32, indices [T,k] i32,
    source_rows [T,k] i32."""
    g = gating.to(torch.float32).contiguous()
    T, E = g.shape
    w = torch.empty(T, topk, dtype=torch.float32)
    idx = torch.empty(T, topk, dtype=torch.int32)
    src = torch.empty(T, topk, dtype=torch.int32)
    rc = lib().orc_topk_softmax(_p(g), _i64(T), _i32(E), _i32(topk), ctypes.c_int(int(renormalize)),
                                _p(w), _p(idx), _p(src))
    if rc:
        raise ValueError(f"orc_topk_softmax: rc={rc}")
    return w, idx, src


def moe_fused_gate(x, bias, num_expert_group, topk_group, topk, n_share_experts_fusion,
                   routed_scaling_factor, apply_routed_scaling_factor_on_output=True):
    """x [T, E], bias [E] (widened to fp32) -> weights [T, topk] f32, indices [T, topk] i32."""
    g = x.to(torch.float32).contiguous()
    b = bias.to(torch.float32).contiguous()
    T, E = g.shape
    w = torch.empty(T, topk, dtype=torch.float32)
    idx = torch.empty(T, topk, dtype=torch.int32)
    rc = lib().orc_moe_fused_gate(_p(g), _p(b), _i64(T), _i32(E), _i32(num_expert_group), _i32(topk_group),
                                  _i32(topk), _i32(n_share_experts_fusion),
                                  ctypes.c_double(routed_scaling_factor),
                                  ctypes.c_int(int(apply_routed_scaling_factor_on_output)), _p(w), _p(idx))
    if rc:
        raise ValueError(f"orc_moe_fused_gate: rc={rc}")
    return w, idx


def fused_experts_w4a8(x, w1_packed, w2_packed, w1_scale, w2_scale, *args, **kwargs):
    """Whole path with packed int4 weights ([E, 2I, H/2], [E, H, I/2]) and K-group row scales
    ([E, 2I, H/128], [E, H, I/128]); other arguments as fused_experts_block_int8."""
    return fused_experts_block_int8(x, unpack_int4(w1_packed), unpack_int4(w2_packed), w1_scale, w2_scale,
                                    *args, _fn="orc_fused_experts_w4a8", **kwargs)


def fused_experts_w4a8_channel(x, w1_packed, w2_packed, w1_scale, w2_scale, *args, **kwargs):
    """Whole path in the reference's own int4 form (w4a8.py:480-658): packed weights
    [E, 2I, H/2] and [E, H, I/2], w1_scale [E, 2I(, 1)], w2_scale [E, H(, 1)]; a1s and a2s hold one
    scale per row.  Other arguments as fused_experts_block_int8."""
    E = w1_packed.shape[0]
    return fused_experts_block_int8(x, w1_packed.contiguous().view(torch.uint8), w2_packed.contiguous().view(torch.uint8),
                                    w1_scale.reshape(E, -1), w2_scale.reshape(E, -1), *args,
                                    _fn="orc_fused_experts_w4a8_channel", **kwargs)


def fused_experts_channel_int8(x, w1, w2, w1_scale, w2_scale, *args, **kwargs):
    """Whole path in the per-channel form: w1_scale [E, 2I(, 1)], w2_scale [E, H(, 1)]; the
    intermediates a1s and a2s hold one scale per row.  Other arguments as fused_experts_block_int8."""
    E = w1.shape[0]
    return fused_experts_block_int8(x, w1, w2, w1_scale.reshape(E, -1), w2_scale.reshape(E, -1), *args,
                                    _fn="orc_fused_experts_channel_int8", **kwargs)


def fused_experts_block_int8(x, w1, w2, w1_scale, w2_scale, topk_weights, topk_ids, block_size_m,
                             global_num_experts=-1, expert_map=None,
                             apply_router_weight_on_input=False, routed_scaling_factor=1.0,
                             shared_output=None, return_intermediates=False, _fn="orc_fused_experts_block_int8",
                             activation="silu"):
    """Whole path; with return_intermediates a dict of every stage's output.  ``activation``:
    "silu" or "gelu"."""
    assert activation in ("silu", "gelu")
    M, H = x.shape
    E, N1, _ = w1.shape
    I = N1 // 2
    k = topk_ids.shape[1]
    S = M * k
    Eg = E if global_num_experts == -1 else global_num_experts
    max_pad, max_blocks = align_buffer_sizes(S, Eg, block_size_m)
    dt = x.dtype
    out = torch.empty(M, H, dtype=dt)
    sorted_ids = torch.empty(max_pad, dtype=torch.int32)
    expert_ids = torch.empty(max_blocks, dtype=torch.int32)
    ntpp = torch.zeros(1, dtype=torch.int32)
    inter = {}
    if return_intermediates:
        inter = dict(
            a1q=torch.empty(M, H, dtype=torch.int8), a1s=torch.empty(M, H // 128, dtype=torch.float32),
            c1=torch.zeros(S, 2 * I, dtype=dt), act=torch.empty(S, I, dtype=dt),
            a2q=torch.empty(S, I, dtype=torch.int8), a2s=torch.empty(S, I // 128, dtype=torch.float32),
            c3=torch.zeros(S, H, dtype=dt))
    ids = topk_ids.to(torch.int32).contiguous()
    tw = topk_weights.to(torch.float32).contiguous()
    emap = None if expert_map is None else expert_map.to(torch.int32).contiguous()
    assert shared_output is None or shared_output.dtype == dt
    if dt == torch.float32:
        assert _fn == "orc_fused_experts_block_int8", "fp32 rows: block form only"
        _fn = "orc_fused_experts_block_int8_f32"
    lib().orc_set_activation(ctypes.c_int(1 if activation == "gelu" else 0))
    lib().orc_set_dtype(ctypes.c_int(1 if dt == torch.float16 else 0))
    try:
        rc = _call_chain(_fn, x, M, H, I, E, Eg, k, w1, w1_scale, w2, w2_scale, tw, ids, emap, block_size_m,
                         apply_router_weight_on_input, routed_scaling_factor, shared_output, out, sorted_ids,
                         max_pad, expert_ids, max_blocks, ntpp, inter)
    finally:
        lib().orc_set_activation(ctypes.c_int(0))
        lib().orc_set_dtype(ctypes.c_int(0))
    if rc != 0:
        raise RuntimeError("oracle fused_experts: alignment failed")
    if return_intermediates:
        if _fn in ("orc_fused_experts_channel_int8", "orc_fused_experts_w4a8_channel"):  # one scale per row, written densely at the front
            inter["a1s"] = inter["a1s"].reshape(-1)[:M].reshape(M, 1).clone()
            inter["a2s"] = inter["a2s"].reshape(-1)[:S].reshape(S, 1).clone()
        inter.update(sorted_ids=sorted_ids, expert_ids=expert_ids, num_tokens_post_pad=ntpp, out=out)
        return inter
    return out


def _call_chain(_fn, x, M, H, I, E, Eg, k, w1, w1_scale, w2, w2_scale, tw, ids, emap, block_size_m,
                apply_router_weight_on_input, routed_scaling_factor, shared_output, out, sorted_ids, max_pad,
                expert_ids, max_blocks, ntpp, inter):
    return getattr(lib(), _fn)(
        _p(x.contiguous()), _i64(M), _i64(H), _i64(I), _i32(E), _i32(Eg), _i32(k),
        _p(w1.contiguous()), _p(w1_scale.contiguous()), _p(w2.contiguous()), _p(w2_scale.contiguous()),
        _p(tw), _p(ids), _p(emap), _i32(block_size_m),
        ctypes.c_int(1 if apply_router_weight_on_input else 0), ctypes.c_float(routed_scaling_factor),
        _p(None if shared_output is None else shared_output.contiguous()), _p(out),
        _p(sorted_ids), _i64(max_pad), _p(expert_ids), _i64(max_blocks), _p(ntpp),
        _p(inter.get("a1q")), _p(inter.get("a1s")), _p(inter.get("c1")), _p(inter.get("act")),
        _p(inter.get("a2q")), _p(inter.get("a2s")), _p(inter.get("c3")))
