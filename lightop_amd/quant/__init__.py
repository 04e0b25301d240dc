"""INT8 activation quantisation of the fused-MoE path: 1x128 groups and per token (reference:
python/lightop/_lmslim_native/layers/gemm/int8_utils.py:125-195 and :20-71; public names
lightop.quant.per_token_group_quant_int8 and lightop.quant.per_token_quant_int8,
python/lightop/quant/int8.py:13-16, :35)."""
from __future__ import annotations

from typing import Tuple

import torch

from .. import _lib
from ..op import _act_dtype, _on_device, _require_cuda


def per_token_group_quant_int8(
    x: torch.Tensor,
    group_size: int,
    eps: float = 1e-10,
    dtype: torch.dtype = torch.int8,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantise every ``group_size`` contiguous values of the last dimension to int8:
    ``amax = max(|x|.max(), eps); s = amax / 127; q = trunc(clamp(x / s, -128, 127))``.
    Returns ``(x_q, x_s)`` with ``x_s`` of shape ``x.shape[:-1] + (x.shape[-1] // group_size,)``
    in fp32.  The kernel is built for ``group_size == 128`` (int8_utils.py:112).
    """
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` cannot be divisible by `group_size`"
    if dtype != torch.int8:
        raise RuntimeError("per_token_group_quant_int8: only torch.int8 output is supported")
    if group_size != 128:
        raise RuntimeError("per_token_group_quant_int8: group_size must be 128")
    _require_cuda(x)
    if not x.is_contiguous():
        x = x.contiguous()
    x_q = torch.empty_like(x, dtype=torch.int8)
    x_s = torch.empty(x.shape[:-1] + (x.shape[-1] // group_size,), device=x.device, dtype=torch.float32)
    cols = x.shape[-1]
    rows = x.numel() // cols
    with _on_device(x):
        _lib.check(_lib.lib().lo_per_token_group_quant_int8(
            _lib.ptr(x), _act_dtype(x), rows, cols, float(eps), _lib.ptr(x_q), _lib.ptr(x_s),
            _lib.stream_of(x)))
    return x_q, x_s


def per_token_quant_int8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """One scale per row of the last dimension: ``absmax = max(|x|.max(), 1e-10); s = absmax / 127;
    q = round_half_even(x * (127 / absmax))``.  Returns ``(x_q, scales)`` with ``scales`` of shape
    ``x.shape[:-1] + (1,)`` in fp32 (reference: per_token_quant_int8, int8_utils.py:46-71;
    public name lightop.quant.per_token_quant_int8, python/lightop/quant/int8.py:35)."""
    _require_cuda(x)
    if not x.is_contiguous():
        x = x.contiguous()
    cols = x.shape[-1]
    rows = x.numel() // cols
    x_q = torch.empty_like(x, dtype=torch.int8)
    scales = torch.empty(x.shape[:-1] + (1,), device=x.device, dtype=torch.float32)
    with _on_device(x):
        _lib.check(_lib.lib().lo_per_token_quant_int8(_lib.ptr(x), _act_dtype(x), rows, cols, _lib.ptr(x_q),
                                                      _lib.ptr(scales), _lib.stream_of(x)))
    return x_q, scales


__all__ = ["per_token_group_quant_int8", "per_token_quant_int8"]

# ``quant.int8`` (python/lightop/quant/int8.py in the reference) is this module: the attribute makes
# ``import lightop.quant.int8 as q`` and ``from lightop_amd.quant import int8`` resolve as well.
import sys as _sys  # noqa: E402

int8 = _sys.modules[__name__]
_sys.modules.setdefault(__name__ + ".int8", int8)
