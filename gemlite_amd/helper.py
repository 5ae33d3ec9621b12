"""Processors: recipes that turn weights into packed ``GemLiteLinear`` layers.

Only the recipes the hot path is measured on are provided; each mirrors the
mode overrides of the reference class of the same name.
"""
import torch

from .core import GemLiteLinear
from .dtypes import DType, TORCH_TO_DTYPE
from .quant_utils import WeightQuantizerMXFP, quantize_weights_per_channel


class A16Wn:
    """fp16/bf16 activations x grouped 8/4/2/1-bit integer weights
    (reference: gemlite/helper.py:174-272).  ``post_scale`` defaults to True, the
    reference's default on AMD GPUs (reference: gemlite/helper.py:14-22)."""

    def __init__(self, device="cuda:0", dtype=None, packing_bitwidth=None, post_scale=True):
        self.device = device
        self.dtype = dtype
        self.packing_bitwidth = packing_bitwidth
        self.post_scale = post_scale

    def from_weights(self, W_q, scales, zeros, W_nbits, group_size, bias=None):
        dtype = scales.dtype if self.dtype is None else self.dtype
        assert dtype in (torch.float16, torch.bfloat16, torch.float32), "Invalid scales.dtype, should floating point."
        out_features, in_features = W_q.shape
        W_q = W_q.to(self.device)
        scales = scales.to(device=self.device, dtype=dtype)
        zeros = zeros.to(device=self.device, dtype=dtype) if isinstance(zeros, torch.Tensor) else zeros
        bias = bias.to(device=self.device, dtype=dtype) if bias is not None else None
        layer = GemLiteLinear(
            W_nbits, group_size=group_size, in_features=in_features, out_features=out_features,
            input_dtype=TORCH_TO_DTYPE[dtype], output_dtype=TORCH_TO_DTYPE[dtype], scaled_activations=False,
        )
        layer.pack(W_q, scales, zeros, bias=bias, packing_bitwidth=self.packing_bitwidth)
        if group_size == in_features:  # channel-wise: scale after or before the K sum
            if self.post_scale:
                layer.W_group_mode, layer.channel_scale_mode = 1, 1
            else:
                layer.W_group_mode, layer.channel_scale_mode = 3, 0
        return layer


class A16W8(A16Wn):
    def from_weights(self, W_q, scales, zeros, group_size, bias=None):
        return super().from_weights(W_q, scales, zeros, 8, group_size, bias)


class A16W4(A16Wn):
    def from_weights(self, W_q, scales, zeros, group_size, bias=None):
        return super().from_weights(W_q, scales, zeros, 4, group_size, bias)


class A16W2(A16Wn):
    def from_weights(self, W_q, scales, zeros, group_size, bias=None):
        return super().from_weights(W_q, scales, zeros, 2, group_size, bias)


A16W8_HQQ_INT, A16W4_HQQ_INT, A16W2_HQQ_INT = A16W8, A16W4, A16W2


class A8W8_dynamic:
    """Per-token dynamic activations x per-channel 8-bit weights, fp32 scales on both
    sides applied after the K sum (reference: gemlite/helper.py:509-691)."""

    def __init__(self, device="cuda:0", dtype=None, fp8=False, fp32_scale=True):
        self.device = device
        self.dtype = dtype
        self.fp8 = fp8
        self.fp32_scale = fp32_scale

    def from_weights(self, weight, bias=None, scales=None):
        w_dtype = self.fp8 if self.fp8 else torch.int8
        input_dtype = TORCH_TO_DTYPE[w_dtype]
        out_features, in_features = weight.shape
        if scales is None:
            dtype = weight.dtype if self.dtype is None else self.dtype
            assert dtype in (torch.float16, torch.bfloat16, torch.float32), "Invalid weight dtype, should be floating point."
            W_q, scales = quantize_weights_per_channel(weight.to(self.device), w_dtype)
        else:
            assert weight.dtype.itemsize == 1, "Invalid weight.dtype, should be 8-bit."
            dtype = self.dtype or (scales.dtype if scales.dtype in (torch.float16, torch.bfloat16) else torch.float16)
            W_q, scales = weight.to(self.device), scales.to(self.device)
        scales = scales.to(torch.float32 if self.fp32_scale else dtype)
        bias = bias.to(device=self.device, dtype=dtype) if bias is not None else None
        layer = GemLiteLinear(
            8, group_size=in_features, in_features=in_features, out_features=out_features,
            input_dtype=input_dtype, output_dtype=TORCH_TO_DTYPE[dtype], scaled_activations=True,
        )
        layer.pack(W_q, scales, zeros=None, bias=bias)
        layer.W_group_mode, layer.channel_scale_mode = 0, 3
        return layer

    def from_linear(self, linear_layer, del_orig=True):
        return self.from_weights(linear_layer.weight.data, None if linear_layer.bias is None else linear_layer.bias.data)


class A8W8_INT8_dynamic(A8W8_dynamic):
    def __init__(self, device="cuda:0", dtype=None):
        super().__init__(device=device, dtype=dtype, fp8=False)


class A8W8_FP8_dynamic(A8W8_dynamic):
    def __init__(self, device="cuda:0", dtype=None):
        super().__init__(device=device, dtype=dtype, fp8=torch.float8_e4m3fn)


A8W8_int8_dynamic, A8W8_fp8_dynamic = A8W8_INT8_dynamic, A8W8_FP8_dynamic


class A4W4_MXFP_dynamic:
    """MXFP4 activations (quantised on the fly) x MXFP4 weights
    (reference: gemlite/helper.py:1042-1114)."""

    def __init__(self, device="cuda:0", dtype=None):
        self.device = device
        self.dtype = dtype
        self.quantizer_mx = None

    def from_weights(self, weight, bias=None, scales=None, packed=False):
        out_features, in_features = weight.shape
        if packed:
            in_features *= 2
        assert scales is not None, "Scales parameter cannot be None. Use from_linear() call to pre-quantize the weights."
        assert weight.dtype == torch.uint8, f"Invalid weight.dtype, should be uint8 codes, got {weight.dtype}."
        assert scales.dtype in (torch.float8_e8m0fnu, torch.uint8), f"Invalid scales.dtype, got {scales.dtype}."
        assert self.dtype is not None, "Input dtype should be either torch.float16 or torch.bfloat16, not None."
        if scales.dtype == torch.uint8:
            scales = scales.view(torch.float8_e8m0fnu)
        bias = bias.to(device=self.device, dtype=self.dtype) if bias is not None else None
        layer = GemLiteLinear(
            4, group_size=32, in_features=in_features, out_features=out_features,
            input_dtype=DType.MXFP4, output_dtype=TORCH_TO_DTYPE[self.dtype], scaled_activations=True,
        )
        layer.pack(weight.to(self.device), scales.to(self.device), zeros=None, bias=bias, packed=packed)
        layer.W_group_mode, layer.channel_scale_mode = 0, 4
        return layer

    def from_linear(self, linear_layer, del_orig=True):
        if self.dtype is None:
            self.dtype = linear_layer.weight.dtype
        if self.quantizer_mx is None:
            self.quantizer_mx = WeightQuantizerMXFP(device=self.device, compute_dtype=linear_layer.weight.dtype)
        W = linear_layer.weight.data
        N, K = W.shape
        W_q, scales = self.quantizer_mx.quantize_mxfp4(W, index=True)
        bias = None if linear_layer.bias is None else linear_layer.bias.data.clone()
        return self.from_weights(W_q.view(N, K), scales=scales.view(N, K // 32), bias=bias)
