"""ctypes binding of the C ABI declared in include/lightop_mi355.h."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.environ.get("LIGHTOP_AMD_LIB") or os.path.join(_CSRC, "liblightop_mi355.so")

LO_BF16, LO_F16, LO_F32 = 0, 1, 2
LO_I32, LO_I64 = 0, 1
LO_GEMM_DEFAULT, LO_GEMM_FUSED_SCALE, LO_GEMM_FORCE_STREAMING, LO_GEMM_SEPARATE_ORDER = 0, 1, 2, 4
LO_GEMM_W_PRESHUFFLED = 8
LO_GEMM_SKIP_NONLOCAL = 16
LO_GEMM_W4 = 32
LO_FUSED_NO_DECODE_PATH = 64
LO_FUSED_FORCE_DECODE_PATH = 128
LO_FUSED_ACT_GELU = 256
LO_ACT_SILU, LO_ACT_GELU = 0, 1
LO_FORM_BLOCK, LO_FORM_CHANNEL, LO_FORM_W4 = 0, 1, 2
LO_NOALLOC_SCRATCH_BYTES = 32 << 20
LO_KERNEL_WS, LO_KERNEL_TILE, LO_KERNEL_PC, LO_KERNEL_AS, LO_KERNEL_T128, LO_KERNEL_W4_TILE, LO_KERNEL_DEC = 0, 1, 2, 3, 4, 5, 6
KERNEL_NAMES = {LO_KERNEL_WS: "moe_gemm_ws_kernel", LO_KERNEL_TILE: "moe_gemm_tile_kernel",
                LO_KERNEL_PC: "moe_gemm_pc_kernel", LO_KERNEL_AS: "moe_gemm_as_kernel",
                LO_KERNEL_T128: "moe_gemm_t128_kernel", LO_KERNEL_W4_TILE: "moe_gemm_w4_tile_kernel",
                LO_KERNEL_DEC: "dec_gemm1_kernel / dec_gemm2_kernel"}


class LoMoeTile(ctypes.Structure):
    _fields_ = [("block_size_m", c_int32), ("kernel", c_int32), ("waves", c_int32), ("block_n", c_int32)]


# name -> (restype, argtypes); must list every symbol of include/lightop_mi355.h
SIGNATURES = {
    "lo_version": (c_int, []),
    "lo_last_error": (c_char_p, []),
    "lo_init": (c_int, [c_void_p]),
    "lo_moe_align_block_size": (c_int, [c_void_p, c_int, c_int64, c_int32, c_int32, c_void_p, c_int,
                                        c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p]),
    "lo_moe_align_block_size_mask": (c_int, [c_void_p, c_int, c_int64, c_int32, c_int32, c_void_p, c_int,
                                             c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "lo_moe_align_scratch_bytes": (c_int64, [c_int64, c_int32]),
    "lo_moe_align_block_size_ws": (c_int, [c_void_p, c_int, c_int64, c_int32, c_int32, c_void_p, c_int,
                                           c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
                                           c_int64, c_void_p]),
    "lo_moe_align_block_size_local": (c_int, [c_void_p, c_int, c_int64, c_int32, c_int32, c_void_p, c_int,
                                              c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
                                              c_int64, c_void_p, c_int32, c_void_p]),
    "lo_per_token_group_quant_int8": (c_int, [c_void_p, c_int, c_int64, c_int64, c_float, c_void_p,
                                              c_void_p, c_void_p]),
    "lo_moe_gemm_block_int8": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                       c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int32, c_int32,
                                       c_int64, c_int64, c_int32, c_int32, c_int, c_int, c_void_p]),
    "lo_moe_gemm1_silu_quant_block_int8": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                   c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                                   c_int64, c_int64, c_int64, c_int32, c_int32, c_int64, c_int64,
                                                   c_int32, c_int32, c_int, c_int, c_void_p]),
    "lo_preshuffle_weight_int8": (c_int, [c_void_p, c_void_p, c_int32, c_int64, c_int64, c_void_p]),
    "lo_preshuffle_weight_int4": (c_int, [c_void_p, c_void_p, c_int32, c_int64, c_int64, c_void_p]),
    "lo_silu_and_mul": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p]),
    "lo_gelu_and_mul": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p]),
    "lo_activation_table": (c_int, [c_int, c_int, c_void_p, c_void_p]),
    "lo_act_mul_group_quant": (c_int, [c_void_p, c_int, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "lo_moe_sum": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int32, c_int64, c_float,
                           c_void_p, c_void_p]),
    "lo_topk_softmax": (c_int, [c_void_p, c_int, c_int64, c_int32, c_int32, c_int, c_void_p, c_void_p, c_int,
                                c_void_p, c_void_p]),
    "lo_moe_fused_gate": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int64, c_int32, c_int32, c_int32, c_int32,
                                  c_int32, ctypes.c_double, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "lo_moe_tile_query": (c_int, [c_int64, c_int32, c_int32, c_int32, c_int64, c_int64,
                                  ctypes.POINTER(LoMoeTile), ctypes.POINTER(LoMoeTile)]),
    "lo_moe_tile_query_form": (c_int, [c_int, c_int, c_int64, c_int32, c_int32, c_int32, c_int64, c_int64,
                                       ctypes.POINTER(LoMoeTile), ctypes.POINTER(LoMoeTile)]),
    "lo_moe_tile_query_path": (c_int, [c_int, c_int, c_int, c_int32, c_int64, c_int32, c_int32, c_int32, c_int64,
                                       c_int64, ctypes.POINTER(LoMoeTile), ctypes.POINTER(LoMoeTile)]),
    "lo_measure_mfma_issue_rate": (c_int, [c_int, c_int, c_int, c_void_p, ctypes.POINTER(ctypes.c_double)]),
    "lo_fused_experts_workspace_bytes": (c_int64, [c_int64, c_int32, c_int64, c_int64, c_int32, c_int32]),
    "lo_fused_experts_workspace_offset": (c_int64, [c_int, c_int64, c_int32, c_int64, c_int64, c_int32, c_int32]),
    "lo_per_token_quant_int8": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p]),
    "lo_fuse_silu_mul_quant": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int32,
                                       c_void_p]),
    "lo_fuse_silu_mul_quant_ids": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int32,
                                           c_void_p, c_void_p]),
    "lo_moe_gemm_w8a8": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                 c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int32, c_int32,
                                 c_int64, c_int64, c_int32, c_int32, c_int, c_int, c_void_p]),
    "lo_fused_experts_channel_int8": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int32, c_int32,
                                              c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                              c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_int64, c_int32, c_int, c_void_p]),
    "lo_fused_experts_channel_int8_prequant": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int32,
                                                       c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
                                                       c_void_p, c_void_p, c_int, c_void_p, c_int, c_float, c_void_p,
                                                       c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int,
                                                       c_void_p]),
    "lo_fused_experts_block_int8": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int32, c_int32,
                                            c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p,
                                            c_void_p, c_void_p, c_int64, c_int32, c_int, c_void_p]),
    "lo_fused_experts_block_int8_noalloc": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int32, c_int32,
                                                    c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                    c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p,
                                                    c_void_p, c_int32, c_int, c_void_p]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """The loaded HIP library.  A missing library is an error: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m lightop_amd.build` "
                "(lightop_amd has no CPU or PyTorch fallback)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc: int) -> None:
    """Map a negative return code to RuntimeError, as TORCH_CHECK does in the reference."""
    if rc < 0:
        msg = lib().lo_last_error()
        raise RuntimeError(f"lightop_amd: {msg.decode() if msg else 'error'} (code {rc})")


def ptr(t) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


def stream_of(t) -> c_void_p:
    import torch

    return c_void_p(torch.cuda.current_stream(t.device).cuda_stream)
