"""Activation quantisation entry points and the one-time weight quantisers.

The activation functions launch the fused HIP kernels through the C ABI; they
have no CPU implementation.  The weight quantisers are one-time host-side torch
code, as in the reference.
"""
from typing import Tuple

import torch
from torch import Tensor

from . import _ext
from .dtypes import DType, TORCH_TO_DTYPE

_FP4_POS_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
_FP4_THRESHOLDS = (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0)


def get_dtype_range(compute_dtype: torch.dtype):
    """(min, max) representable value (reference: gemlite/quant_utils.py:19-24)."""
    info = torch.finfo(compute_dtype) if compute_dtype.is_floating_point else torch.iinfo(compute_dtype)
    return info.min, info.max


# ---------------------------------------------------------------------------
# activations (GPU, fused kernels)
# ---------------------------------------------------------------------------
def scale_activations_per_token(tensor: Tensor, w_dtype: torch.dtype, fp32_scale: bool = True) -> Tuple[Tensor, Tensor]:
    """Per-row dynamic quantisation to int8 or fp8-e4m3fn.

    Returns ``(y, scales)`` with ``y`` shaped like the input and ``scales``
    ``[M, 1]`` fp32 (reference: gemlite/quant_utils.py:510-539).
    """
    if w_dtype not in (torch.int8, torch.float8_e4m3fn):
        raise NotImplementedError(f"per-token activation quantisation to {w_dtype} is not supported")
    if not fp32_scale:
        raise NotImplementedError("only fp32 activation scales are supported")
    x_shape = tensor.shape
    x2d = tensor.reshape(-1, x_shape[-1])
    if x2d.stride(-1) != 1:
        x2d = x2d.contiguous()
    M, K = x2d.shape
    y = torch.empty((M, K), dtype=w_dtype, device=tensor.device)
    scales = torch.empty((M, 1), dtype=torch.float32, device=tensor.device)
    _ext.scale_activations_per_token(x2d, y, scales)
    return y.view(x_shape), scales


BLOCK_QUANT_SIZE = 128  # (reference: gemlite/triton_kernels/config.py:12)


def scale_activations_per_block(tensor: Tensor, w_dtype: torch.dtype, block_size: int = BLOCK_QUANT_SIZE) -> Tuple[Tensor, Tensor]:
    """Dynamic quantisation to int8 or fp8-e4m3fn with one fp32 scale per (row, ``block_size``
    consecutive values).  Returns ``(y, scales)`` with ``y`` shaped like the input and ``scales``
    ``[M, K / block_size]`` fp32 (reference: gemlite/quant_utils.py:2654-2676)."""
    if w_dtype not in (torch.int8, torch.float8_e4m3fn):
        raise NotImplementedError(f"per-block activation quantisation to {w_dtype} is not supported")
    if block_size != BLOCK_QUANT_SIZE:
        raise NotImplementedError(f"only blocks of {BLOCK_QUANT_SIZE} values are supported")
    x_shape = tensor.shape
    x2d = tensor.reshape(-1, x_shape[-1])
    if x2d.stride(-1) != 1:
        x2d = x2d.contiguous()
    M, K = x2d.shape
    assert K % block_size == 0, "K must be divisible by block_size for per-block activation quantization."
    y = torch.empty((M, K), dtype=w_dtype, device=tensor.device)
    scales = torch.empty((M, K // block_size), dtype=torch.float32, device=tensor.device)
    _ext.scale_activations_per_block(x2d, y, scales)
    return y.view(x_shape), scales


def scale_activations_mxfp8(tensor: Tensor, w_dtype: torch.dtype = torch.float8_e4m3fn) -> Tuple[Tensor, Tensor]:
    """MXFP8 dynamic quantisation: ``([M, K] e4m3fn codes, [ceil32(M), K/32] uint8 e8m0)``
    (reference: gemlite/quant_utils.py:1025-1127)."""
    if w_dtype != torch.float8_e4m3fn:
        raise NotImplementedError(f"MXFP8 activations as {w_dtype}: only float8_e4m3fn is built")
    x2d = tensor.reshape(-1, tensor.shape[-1])
    if x2d.stride(-1) != 1:
        x2d = x2d.contiguous()
    M, K = x2d.shape
    M_pad = (M + 31) // 32 * 32
    out = torch.empty((M, K), dtype=torch.uint8, device=tensor.device)
    scales = torch.empty((M_pad, K // 32), dtype=torch.uint8, device=tensor.device)
    _ext.scale_activations_mxfp8(x2d, out, scales)
    return out.view(torch.float8_e4m3fn).view(tensor.shape), scales


def scale_activations_mxfp4(tensor: Tensor) -> Tuple[Tensor, Tensor]:
    """MXFP4 dynamic quantisation: ``([M, K/2] uint8 codes, [ceil32(M), K/32] uint8 e8m0)``
    (reference: gemlite/quant_utils.py:2108-2135)."""
    x2d = tensor.reshape(-1, tensor.shape[-1])
    if x2d.stride(-1) != 1:
        x2d = x2d.contiguous()
    M, K = x2d.shape
    M_pad = (M + 31) // 32 * 32
    out = torch.empty((M, K // 2), dtype=torch.uint8, device=tensor.device)
    scales = torch.empty((M_pad, K // 32), dtype=torch.uint8, device=tensor.device)
    _ext.scale_activations_mxfp4(x2d, out, scales)
    return out, scales


def _not_built(name):
    def fn(*args, **kwargs):
        raise NotImplementedError(f"{name} is not implemented in this build")

    fn.__name__ = name
    return fn


scale_activations_nvfp4 = _not_built("scale_activations_nvfp4")


# ---------------------------------------------------------------------------
# weights (one-time, torch)
# ---------------------------------------------------------------------------
class WeightQuantizerMXFP:
    """Weight-side MXFP4 quantiser (reference: gemlite/quant_utils.py:75-168)."""

    def __init__(self, compute_dtype=torch.bfloat16, device="cuda:0"):
        self.compute_dtype = compute_dtype
        self.device = device

    @staticmethod
    def round_to_closest_fp4(tensor: Tensor) -> Tensor:
        """Nearest e2m1 magnitude with ties toward zero, sign restored by multiplication
        (reference: gemlite/quant_utils.py:80-88)."""
        thr = torch.tensor(_FP4_THRESHOLDS, dtype=tensor.dtype, device=tensor.device)
        vals = torch.tensor(_FP4_POS_VALUES, dtype=torch.float32, device=tensor.device)
        out = vals[torch.searchsorted(thr, tensor.abs())].to(tensor.dtype)
        return out * tensor.sign()

    @staticmethod
    def to_index(W_q: Tensor) -> Tensor:
        """e2m1 value -> 4-bit code; +0 and -0 both map to 0
        (reference: gemlite/quant_utils.py:90-99)."""
        mag = W_q.abs()
        vals = torch.tensor(_FP4_POS_VALUES, dtype=W_q.dtype, device=W_q.device)
        idx = torch.searchsorted(vals, mag.contiguous()).to(torch.uint8)
        neg = (W_q < 0).to(torch.uint8) * 8
        return (idx + neg).to(torch.uint8).view(W_q.shape)

    def quantize_mxfp4(self, W: Tensor, window_size: int = 0, index: bool = False) -> Tuple[Tensor, Tensor]:
        """Blocks of 32 along the last axis: s = 2^ceil(log2(amax/6)) clamped to >= 2^-30
        (reference: gemlite/quant_utils.py:130-168, window_size=0 branch)."""
        if window_size != 0:
            raise NotImplementedError("scale search (window_size > 0) is not implemented")
        W_flat = W.reshape(-1, 32).float()
        ideal = W_flat.abs().amax(dim=1, keepdim=True) / 6
        scales = (2 ** torch.ceil(torch.log2(ideal))).clamp_(min=2.0 ** -30)
        W_q = self.round_to_closest_fp4(W_flat / scales)
        scales = scales.to(torch.float8_e8m0fnu)
        if index:
            W_q = self.to_index(W_q)
        return W_q, scales

    def quantize_mxfp8(self, W: Tensor, index: bool = False, mx_fp8_dtype: torch.dtype = torch.float8_e4m3fn) -> Tuple[Tensor, Tensor]:
        """Blocks of 32 along the last axis: s = 2^ceil(log2(amax/qmax)) clamped to >= 2^-30, values
        clamp(w/s) cast to fp8 (reference: gemlite/quant_utils.py:102-128)."""
        max_val = torch.finfo(mx_fp8_dtype).max
        W_flat = W.reshape(-1, 32).float()
        ideal = W_flat.abs().amax(dim=1, keepdim=True) / max_val
        scales = (2 ** torch.ceil(torch.log2(ideal))).clamp_(min=2.0 ** -30)
        W_q = (W_flat / scales).clamp_(min=-max_val, max=max_val)
        scales = scales.to(torch.float8_e8m0fnu)
        W_q = W_q.to(mx_fp8_dtype) if index else W_q.to(mx_fp8_dtype).to(W_flat.dtype)
        return W_q, scales

    def dequantize(self, W_q, scales, shape=None, dtype=None, meta_scales=None):
        """(reference: gemlite/quant_utils.py:220-232)"""
        if W_q.dtype == torch.uint8:
            table = torch.tensor(
                list(_FP4_POS_VALUES) + [-v for v in _FP4_POS_VALUES], dtype=torch.float32, device=W_q.device
            )
            W_q = table[W_q.int()]
        group_size = W_q.numel() // scales.numel()
        out = W_q.reshape(-1, group_size).float() * scales.float().reshape(-1, 1)
        if meta_scales is not None:
            out = out * meta_scales
        if shape is not None:
            out = out.view(shape)
        return out.to(self.compute_dtype if dtype is None else dtype)


def quantize_weights_per_channel(weight: Tensor, w_dtype: torch.dtype) -> Tuple[Tensor, Tensor]:
    """Per-output-channel symmetric quantisation to int8 / fp8:
    ``s = max(amax_row / qmax, 1e-6)``; int8 rounds half-to-even
    (reference: gemlite/helper.py:635-657)."""
    min_val, max_val = get_dtype_range(w_dtype)
    w32 = weight.to(torch.float32)
    scales = (w32.abs().amax(dim=1, keepdim=True) / max_val).clamp_(min=1e-6)
    W_q = (w32 / scales).clamp_(min=min_val, max=max_val)
    W_q = W_q.to(w_dtype) if w_dtype.is_floating_point else W_q.round_().to(w_dtype)
    return W_q, scales


__all__ = [
    "get_dtype_range",
    "scale_activations_per_token",
    "scale_activations_mxfp4",
    "scale_activations_per_block",
    "scale_activations_mxfp8",
    "scale_activations_nvfp4",
    "WeightQuantizerMXFP",
    "quantize_weights_per_channel",
]
