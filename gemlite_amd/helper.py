"""Processors: recipes that turn weights into packed ``GemLiteLinear`` layers.

Class names, constructor arguments and mode overrides follow the reference class of the same name
(reference: gemlite/helper.py).
"""
import gc

import torch

from .core import GemLiteLinear
from .dtypes import DType, TORCH_TO_DTYPE
from .quant_utils import BLOCK_QUANT_SIZE, WeightQuantizerMXFP, quantize_weights_per_channel


def cleanup_linear(linear_layer, del_orig=True):
    """Drop the tensors of a replaced layer (reference: gemlite/helper.py:26-32)."""
    if del_orig:
        for attr in ("weight", "bias", "weight_scale", "W_q", "meta"):
            val = getattr(linear_layer, attr, None)
            if val is not None and hasattr(val, "__len__") and len(val) > 0:
                setattr(linear_layer, attr, None)
    if torch.cuda.is_available():
        torch.cuda.empty_cache()


def patch_model(model, device, processor, skip_modules=("lm_head", "vision", "visual"), group_size=64):
    """Replace every ``torch.nn.Linear`` of ``model`` (outside ``skip_modules``) by
    ``processor.from_linear(layer)`` (reference: gemlite/helper.py:35-87).  Processors that start
    from an HQQ layer (``from_hqqlinear``) need the ``hqq`` package to quantize; without it they are
    refused here, as the reference does."""
    if hasattr(processor, "from_hqqlinear") and not hasattr(processor, "from_linear"):
        raise ImportError("This processor requires the `hqq` package to quantize nn.Linear layers; "
                          "quantize first and use from_weights().")
    for name, module in model.named_modules():
        module.name = name

    def patch(parent):
        for child_name, layer in parent.named_children():
            if isinstance(layer, torch.nn.Linear):
                layer = layer.to(device=device)
                if not any(s in layer.name for s in skip_modules):
                    layer = processor.from_linear(layer)
                setattr(parent, child_name, layer)
            else:
                patch(layer)

    patch(model)
    model = model.to(device=device)
    gc.collect()
    return model


class A16W8:
    """fp16/bf16 activations x int8 or fp8 weights, one scale per output channel, weights kept as
    unpacked bytes (reference: gemlite/helper.py:89-171).  ``post_scale``: multiply by the channel
    scale after the K sum (W_group_mode 0, channel_scale_mode 1) instead of dequantising the weights
    (W_group_mode 2, channel_scale_mode 0)."""

    def __init__(self, device="cuda:0", dtype=None, fp8=None, fp32_scale=True, post_scale=False):
        self.device = device
        self.dtype = dtype
        self.fp8 = fp8
        self.fp32_scale = fp32_scale
        self.post_scale = post_scale

    def from_weights(self, weight, bias=None, scales=None):
        if isinstance(weight, torch.nn.Parameter):
            weight = weight.data
        if isinstance(bias, torch.nn.Parameter):
            bias = bias.data
        out_features, in_features = weight.shape
        if scales is None:
            w_dtype = self.fp8 if self.fp8 else torch.int8
            dtype = weight.dtype if self.dtype is None else self.dtype
            assert dtype in (torch.float16, torch.bfloat16, torch.float32), \
                f"Invalid weight dtype, should be floating point, got {dtype}"
            W_q, scales = quantize_weights_per_channel(weight.to(self.device), w_dtype)
        else:
            assert weight.dtype.itemsize == 1, f"Invalid weight.dtype, should be 8-bit (INT8 or FP8), got {weight.dtype}"
            dtype = self.dtype or (scales.dtype if scales.dtype in (torch.float16, torch.bfloat16) else torch.float16)
            W_q, scales = weight.to(self.device), scales.to(self.device)
        bias = bias.to(device=self.device, dtype=dtype) if bias is not None else None
        layer = GemLiteLinear(
            8, group_size=in_features, in_features=in_features, out_features=out_features,
            input_dtype=TORCH_TO_DTYPE[dtype], output_dtype=TORCH_TO_DTYPE[dtype],
        )
        layer.pack(W_q, scales, zeros=None, bias=bias)
        if self.post_scale:
            layer.W_group_mode, layer.channel_scale_mode = 0, 1
        else:
            layer.W_group_mode, layer.channel_scale_mode = 2, 0
        return layer

    def from_linear(self, linear_layer, del_orig=True):
        out_layer = self.from_weights(weight=linear_layer.weight, bias=linear_layer.bias)
        cleanup_linear(linear_layer, del_orig)
        return out_layer


class A16W8_INT8(A16W8):
    def __init__(self, device="cuda:0", dtype=None, fp32_scale=True, post_scale=False):
        super().__init__(device=device, dtype=dtype, fp8=None, fp32_scale=fp32_scale, post_scale=post_scale)


class A16W8_FP8(A16W8):
    def __init__(self, device="cuda:0", dtype=None, fp8=torch.float8_e4m3fn, fp32_scale=True, post_scale=False):
        super().__init__(device=device, dtype=dtype, fp8=fp8, fp32_scale=fp32_scale, post_scale=post_scale)


class A16Wn:
    """fp16/bf16 activations x grouped 8/4/2/1-bit integer weights (``quant_type="INT"``) or x
    MXFP8 / MXFP4 weights with one e8m0 scale per 32 values (``quant_type="MXFP"``)
    (reference: gemlite/helper.py:174-332).  ``post_scale`` defaults to True, the reference's
    default on AMD GPUs (reference: gemlite/helper.py:14-22)."""

    def __init__(self, device="cuda:0", dtype=None, packing_bitwidth=None, post_scale=True):
        self.device = device
        self.dtype = dtype
        self.packing_bitwidth = packing_bitwidth
        self.post_scale = post_scale
        self.quantizer_mx = None
        self.mx_fp8_dtype = torch.float8_e4m3fn

    def from_packed_weights(self, W_q, scales, zeros, W_nbits, group_size, bias=None, quant_type="INT"):
        """Load pre-packed weights (already nibble/byte-packed)."""
        return self.from_weights_(W_q, scales, zeros, W_nbits, group_size, bias, quant_type, packed=True)

    def from_weights(self, W_q, scales, zeros, W_nbits, group_size, bias=None, quant_type="INT"):
        return self.from_weights_(W_q, scales, zeros, W_nbits, group_size, bias, quant_type)

    def from_weights_(self, W_q, scales, zeros, W_nbits, group_size, bias=None, quant_type="INT", packed=False):
        assert quant_type in ("INT", "MXFP"), f"Invalid quant_type. Got {quant_type}, valid values are INT, MXFP."
        if isinstance(W_q, torch.nn.Parameter):
            W_q = W_q.data
        if isinstance(bias, torch.nn.Parameter):
            bias = bias.data
        if quant_type == "MXFP":
            return self._from_mxfp_weights(W_q, scales, W_nbits, group_size, bias, packed)
        dtype = scales.dtype if self.dtype is None else self.dtype
        assert dtype in (torch.float16, torch.bfloat16, torch.float32), "Invalid scales.dtype, should floating point."
        out_features, in_features = W_q.shape
        if packed:
            in_features = in_features * 8 // W_nbits
        W_q = W_q.to(self.device)
        scales = scales.to(device=self.device, dtype=dtype)
        zeros = zeros.to(device=self.device, dtype=dtype) if isinstance(zeros, torch.Tensor) else zeros
        bias = bias.to(device=self.device, dtype=dtype) if bias is not None else None
        layer = GemLiteLinear(
            W_nbits, group_size=group_size, in_features=in_features, out_features=out_features,
            input_dtype=TORCH_TO_DTYPE[dtype], output_dtype=TORCH_TO_DTYPE[dtype], scaled_activations=False,
        )
        layer.pack(W_q, scales, zeros, bias=bias, packing_bitwidth=self.packing_bitwidth, packed=packed)
        if group_size == in_features:  # channel-wise: scale after or before the K sum
            if self.post_scale:
                layer.W_group_mode, layer.channel_scale_mode = 1, 1
            else:
                layer.W_group_mode, layer.channel_scale_mode = 3, 0
        return layer

    def _from_mxfp_weights(self, W_q, scales, W_nbits, group_size, bias, packed):
        """Weight-only MX layer: the activations stay fp16 / bf16, the layer's input and output
        types are MXFP16 / MXBF16 (reference: gemlite/helper.py:199-202, 222-237)."""
        assert W_nbits in (8, 4), "Unsupported W_nbit for MXFP quant_dtype."
        assert group_size == 32, "group_size should 32 for MXFP."
        if W_nbits == 8:
            assert W_q.dtype == self.mx_fp8_dtype, f"Unsupported dtype of W_q. got {W_q.dtype}"
        else:
            assert W_q.dtype == torch.uint8, f"Unsupported dtype of W_q. got {W_q.dtype}"
        dtype = torch.float16 if self.dtype is None else self.dtype
        if dtype == torch.float16:
            gemlite_dtype = DType.MXFP16
        elif dtype == torch.bfloat16:
            gemlite_dtype = DType.MXBF16
        else:
            raise Exception(f"Unsupported dtype for MXFP. Got {dtype}, supported [torch.float16, torch.bfloat16]")
        self.post_scale = False
        out_features, in_features = W_q.shape
        if packed and W_nbits == 4:
            in_features *= 2
        if scales.dtype == torch.uint8:
            scales = scales.view(torch.float8_e8m0fnu)
        scales = scales.view(out_features, in_features // group_size)
        bias = bias.to(device=self.device, dtype=dtype) if bias is not None else None
        layer = GemLiteLinear(
            W_nbits, group_size=group_size, in_features=in_features, out_features=out_features,
            input_dtype=gemlite_dtype, output_dtype=gemlite_dtype, scaled_activations=False,
        )
        layer.pack(W_q.to(self.device), scales.to(self.device), None, bias=bias,
                   packing_bitwidth=self.packing_bitwidth, packed=packed)
        return layer

    def mxfp_from_linear(self, linear_layer, W_nbits, del_orig=True):
        """Quantise a float layer to MXFP8 / MXFP4 weights (reference: gemlite/helper.py:304-332)."""
        if self.quantizer_mx is None:
            self.quantizer_mx = WeightQuantizerMXFP(device=self.device, compute_dtype=linear_layer.weight.dtype)
        W = linear_layer.weight.data
        bias = linear_layer.bias.clone() if linear_layer.bias is not None else None
        N, K = W.shape
        if W_nbits == 8:
            W_q, scales = self.quantizer_mx.quantize_mxfp8(W, index=True, mx_fp8_dtype=self.mx_fp8_dtype)
        else:
            W_q, scales = self.quantizer_mx.quantize_mxfp4(W, index=True)
        W_q, scales = W_q.view(N, K), scales.view(N, K // 32)
        cleanup_linear(linear_layer, del_orig)
        return self.from_weights_(W_q=W_q, scales=scales, zeros=None, W_nbits=W_nbits, group_size=32, bias=bias,
                                  quant_type="MXFP")

    def from_hqqlinear(self, hqq_layer, del_orig=True):
        """From an HQQ layer object: what it exposes (``unpack()``, ``meta['scale'|'zero'|'nbits'|
        'group_size'|'shape'|'axis']``, ``bias``) is all that is used (reference: gemlite/helper.py:274-302)."""
        assert hqq_layer.meta["axis"] == 1, "Only axis==1 is supported."
        self.device = hqq_layer.W_q.device
        W_nbits = hqq_layer.meta["nbits"]
        group_size = hqq_layer.meta["group_size"]
        if group_size is None:
            group_size = hqq_layer.in_features
        W_q = hqq_layer.unpack(dtype=torch.uint8).view(hqq_layer.meta["shape"])
        scales, zeros = hqq_layer.meta["scale"].clone(), hqq_layer.meta["zero"].clone()
        bias = hqq_layer.bias.clone() if hqq_layer.bias is not None else None
        cleanup_linear(hqq_layer, del_orig)
        return self.from_weights_(W_q=W_q, scales=scales, zeros=zeros, W_nbits=W_nbits, group_size=group_size,
                                  bias=bias, quant_type="INT")


class A16Wn_HQQ_INT(A16Wn):
    """The grouped-integer recipe with the bit width fixed; the group size follows from the shapes
    (reference: gemlite/helper.py:344-381)."""

    def __init__(self, device="cuda:0", dtype=None, W_nbits=None):
        super().__init__(device=device, dtype=dtype)
        self.W_nbits = W_nbits

    def from_packed_weights(self, W_q_packed, scales, zeros, bias=None):
        group_size = W_q_packed.numel() * (8 // self.W_nbits) // scales.numel()
        return super().from_packed_weights(W_q_packed, scales, zeros, self.W_nbits, group_size, bias=bias)

    def from_weights(self, W_q, scales, zeros, bias=None):
        group_size = W_q.numel() // scales.numel()
        return super().from_weights(W_q=W_q, scales=scales, zeros=zeros, W_nbits=self.W_nbits,
                                    group_size=group_size, bias=bias, quant_type="INT")


class A16W8_HQQ_INT(A16Wn_HQQ_INT):
    def __init__(self, device="cuda:0", dtype=None):
        super().__init__(device=device, dtype=dtype, W_nbits=8)


class A16W4_HQQ_INT(A16Wn_HQQ_INT):
    def __init__(self, device="cuda:0", dtype=None):
        super().__init__(device=device, dtype=dtype, W_nbits=4)


class A16W2_HQQ_INT(A16Wn_HQQ_INT):
    def __init__(self, device="cuda:0", dtype=None):
        super().__init__(device=device, dtype=dtype, W_nbits=2)


class A16W1_HQQ_INT(A16Wn_HQQ_INT):
    def __init__(self, device="cuda:0", dtype=None):
        super().__init__(device=device, dtype=dtype, W_nbits=1)


class A16Wn_MXFP(A16Wn):
    """Weight-only MXFP8 / MXFP4 with the bit width fixed (reference: gemlite/helper.py:384-412)."""

    def __init__(self, device="cuda:0", dtype=None, W_nbits=None):
        super().__init__(device=device, dtype=dtype)
        self.W_nbits = W_nbits

    def from_packed_weights(self, W_q_packed, scales, bias=None):
        """Load pre-packed MXFP weights (nibble/byte-packed)."""
        group_size = W_q_packed.numel() * (8 // self.W_nbits) // scales.numel()
        return super().from_packed_weights(W_q_packed, scales, zeros=None, W_nbits=self.W_nbits,
                                           group_size=group_size, bias=bias, quant_type="MXFP")

    def from_weights(self, W_q, scales, bias=None):
        group_size = W_q.numel() // scales.numel()
        return super().from_weights(W_q=W_q, scales=scales, zeros=None, W_nbits=self.W_nbits,
                                    group_size=group_size, bias=bias, quant_type="MXFP")

    def from_linear(self, linear_layer, del_orig=True):
        return super().mxfp_from_linear(linear_layer=linear_layer, W_nbits=self.W_nbits, del_orig=del_orig)


class A16W8_MXFP(A16Wn_MXFP):
    def __init__(self, device="cuda:0", dtype=None):
        super().__init__(device=device, dtype=dtype, W_nbits=8)


class A16W4_MXFP(A16Wn_MXFP):
    def __init__(self, device="cuda:0", dtype=None):
        super().__init__(device=device, dtype=dtype, W_nbits=4)


class A8W8_dynamic:
    """Per-token dynamic activations x per-channel 8-bit weights, fp32 scales on both
    sides applied after the K sum (reference: gemlite/helper.py:509-691)."""

    def __init__(self, device="cuda:0", dtype=None, fp8=False, fp32_scale=True, block_quant=False):
        self.device = device
        self.dtype = dtype
        self.fp8 = fp8
        self.fp32_scale = fp32_scale
        self.block_quant = block_quant

    def _from_weights_block_quant(self, weight, bias=None, scales=None):
        """128 x 128 block quantisation of the weights + one activation scale per (row, 128 values):
        ``channel_scale_mode`` 5.  With ``scales`` ([ceil(N/128), ceil(K/128)] fp32) the weight is
        taken as already quantised; otherwise it is quantised here per block
        (reference: gemlite/helper.py:517-617)."""
        B = BLOCK_QUANT_SIZE
        w_dtype = self.fp8 if self.fp8 else torch.int8
        input_dtype = TORCH_TO_DTYPE[w_dtype]
        info = torch.finfo(w_dtype) if w_dtype.is_floating_point else torch.iinfo(w_dtype)
        min_val, max_val = info.min, info.max
        out_features, in_features = weight.shape
        if scales is not None:
            assert weight.dtype == w_dtype, f"Pre-quantized weight must be {w_dtype}, got {weight.dtype}"
            want = ((out_features + B - 1) // B, (in_features + B - 1) // B)
            assert tuple(scales.shape) == want, f"Pre-quantized scales must have shape {want}, got {tuple(scales.shape)}"
            W_q = weight.contiguous().to(device=self.device)
            scales = scales.to(device=self.device, dtype=torch.float32)
            dtype = self.dtype if self.dtype is not None else torch.bfloat16
        else:
            dtype = weight.dtype if self.dtype is None else self.dtype
            assert dtype in (torch.float16, torch.bfloat16, torch.float32), "Invalid weight dtype, should be floating point."
            in_pad, out_pad = (in_features + B - 1) // B * B, (out_features + B - 1) // B * B
            w = weight.to(dtype=torch.float32, device=self.device)
            if in_pad != in_features or out_pad != out_features:
                w = torch.nn.functional.pad(w, (0, in_pad - in_features, 0, out_pad - out_features))
            w = w.view(out_pad // B, B, in_pad // B, B)
            scales = (w.abs().amax(dim=(1, 3)) / max_val).clamp_(min=1e-6)
            W_q = (w / scales[:, None, :, None]).clamp_(min=min_val, max=max_val)
            W_q = W_q.to(w_dtype) if w_dtype.is_floating_point else W_q.round_().to(w_dtype)
            W_q = W_q.view(out_pad, in_pad)[:out_features, :in_features].contiguous()
        bias = bias.to(device=self.device, dtype=dtype) if bias is not None else None
        layer = GemLiteLinear(
            8, group_size=in_features, in_features=in_features, out_features=out_features,
            input_dtype=input_dtype, output_dtype=TORCH_TO_DTYPE[dtype], acc_dtype=DType.FP32,
            scaled_activations=True,
        )
        # pack() lays out the weights; the block scales replace its per-channel placeholder
        layer.pack(W_q, torch.ones((out_features, 1), dtype=torch.float32, device=W_q.device), zeros=None, bias=bias)
        layer._set_param("scales", scales.t().contiguous())   # [K/128, N/128]
        layer.meta_dtype = DType.FP32
        layer.W_group_mode, layer.channel_scale_mode = 0, 5
        layer._set_param("metadata", torch.tensor(layer.get_meta_args(), device=W_q.device, dtype=torch.int32))
        return layer

    def from_weights(self, weight, bias=None, scales=None):
        if isinstance(weight, torch.nn.Parameter):
            weight = weight.data
        if isinstance(bias, torch.nn.Parameter):
            bias = bias.data
        if self.block_quant:
            return self._from_weights_block_quant(weight, bias=bias, scales=scales)
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
    def __init__(self, device="cuda:0", dtype=None, block_quant=False):
        super().__init__(device=device, dtype=dtype, fp8=False, block_quant=block_quant)


class A8W8_FP8_dynamic(A8W8_dynamic):
    def __init__(self, device="cuda:0", dtype=None, fp8=torch.float8_e4m3fn, block_quant=False):
        super().__init__(device=device, dtype=dtype, fp8=fp8, block_quant=block_quant)


A8W8_int8_dynamic, A8W8_fp8_dynamic = A8W8_INT8_dynamic, A8W8_FP8_dynamic


class A8Wn_HQQ_INT_dynamic(A16Wn):
    """fp8 activations quantised per token on the fly x grouped 8/4/2-bit integer weights
    (reference: gemlite/helper.py:712-871).  Runs the layout-agnostic kernel (no tuned kernel for
    fp8 activations against packed integer codes is built)."""

    def __init__(self, device="cuda:0", packing_bitwidth=None, dtype=None, post_scale=True,
                 fp8=torch.float8_e4m3fn, fp32_scale=False, W_nbits=None):
        assert W_nbits is not None, "W_nbits argument should be either 8, 4 or 2, not None."
        super().__init__(device=device, dtype=dtype, packing_bitwidth=packing_bitwidth, post_scale=post_scale)
        self.fp8 = fp8
        self.fp32_scale = fp32_scale
        self.W_nbits = W_nbits

    def from_packed_weights(self, W_q_packed, scales, zeros, bias=None):
        group_size = W_q_packed.numel() * (8 // self.W_nbits) // scales.numel()
        return self.from_weights_(W_q_packed, scales, zeros, self.W_nbits, group_size, bias=bias, packed=True)

    def from_weights(self, W_q, scales, zeros, bias=None):
        group_size = W_q.numel() // scales.numel()
        return self.from_weights_(W_q, scales, zeros, self.W_nbits, group_size, bias=bias)

    def from_weights_(self, W_q, scales, zeros, W_nbits, group_size, bias=None, quant_type="INT", packed=False):
        if isinstance(W_q, torch.nn.Parameter):
            W_q = W_q.data
        if isinstance(bias, torch.nn.Parameter):
            bias = bias.data
        if self.dtype is None:
            dtype = scales.dtype if scales.dtype in (torch.float16, torch.bfloat16) else torch.float16
        else:
            dtype = self.dtype
        assert dtype in (torch.float16, torch.bfloat16, torch.float32), "Invalid scales.dtype, should be floating point."
        out_features, in_features = W_q.shape
        if packed:
            in_features = in_features * 8 // W_nbits
        W_q = W_q.to(self.device)
        scales = scales.to(device=self.device, dtype=torch.float32 if self.fp32_scale else dtype) if scales is not None else None
        zeros = zeros.to(device=self.device, dtype=dtype) if isinstance(zeros, torch.Tensor) else zeros
        bias = bias.to(device=self.device, dtype=dtype) if bias is not None else None
        layer = GemLiteLinear(
            W_nbits, group_size=group_size, in_features=in_features, out_features=out_features,
            input_dtype=TORCH_TO_DTYPE[self.fp8], output_dtype=TORCH_TO_DTYPE[dtype], scaled_activations=True,
        )
        layer.pack(W_q, scales, zeros, bias=bias, packing_bitwidth=self.packing_bitwidth, fma_mode=False, packed=packed)
        if group_size == in_features:
            if self.post_scale:
                layer.W_group_mode, layer.channel_scale_mode = 1, 3
            else:
                layer.W_group_mode, layer.channel_scale_mode = 3, 2
        return layer


class A8W4_HQQ_INT_dynamic(A8Wn_HQQ_INT_dynamic):
    def __init__(self, device="cuda:0", packing_bitwidth=None, dtype=None, post_scale=True,
                 fp8=torch.float8_e4m3fn, fp32_scale=False):
        super().__init__(device=device, packing_bitwidth=packing_bitwidth, dtype=dtype, post_scale=post_scale,
                         fp8=fp8, fp32_scale=fp32_scale, W_nbits=4)


class A8W2_HQQ_INT_dynamic(A8Wn_HQQ_INT_dynamic):
    def __init__(self, device="cuda:0", packing_bitwidth=None, dtype=None, post_scale=True,
                 fp8=torch.float8_e4m3fn, fp32_scale=False):
        super().__init__(device=device, packing_bitwidth=packing_bitwidth, dtype=dtype, post_scale=post_scale,
                         fp8=fp8, fp32_scale=fp32_scale, W_nbits=2)


class A8Wn_MXFP_dynamic:
    """MXFP8 or MXFP4 weights (fp8-e4m3 bytes / e2m1 codes, one e8m0 scale per 32 values) x fp8
    activations quantised on the fly: per token with the scale applied after the K sum
    (``post_scale=True``, the default) or with MXFP8 micro-scales on the activations as well
    (``post_scale=False``) (reference: gemlite/helper.py:950-1032)."""

    def __init__(self, device="cuda:0", dtype=None, post_scale=True, fp8=torch.float8_e4m3fn, W_nbits=None):
        assert W_nbits is not None, "W_nbits argument should be either 8 or 4, not None."
        self.device = device
        self.dtype = dtype
        self.mx_fp8_dtype = fp8
        self.quantizer_mx = None
        self.post_scale = post_scale
        self.W_nbits = W_nbits

    def from_packed_weights(self, weight_packed, bias=None, scales=None):
        """Load pre-packed MXFP weights (nibble-packed [N, K//2] for 4-bit)."""
        return self.from_weights(weight_packed, bias=bias, scales=scales, packed=True)

    def from_weights(self, weight, bias=None, scales=None, packed=False):
        if isinstance(weight, torch.nn.Parameter):
            weight = weight.data
        if isinstance(bias, torch.nn.Parameter):
            bias = bias.data
        out_features, in_features = weight.shape
        if packed and self.W_nbits == 4:
            in_features *= 2
        assert scales is not None, "Scales parameter cannot be None. Use from_linear() call to pre-quantize the weights."
        if self.W_nbits == 8:
            assert weight.is_floating_point() and weight.dtype.itemsize == 1, \
                f"Invalid weight.dtype, should be an MXFP8 dtype, got {weight.dtype}."
        if self.W_nbits == 4:
            assert weight.dtype == torch.uint8, f"Invalid weight.dtype, should be uint8 codes, got {weight.dtype}."
        assert scales.dtype in (torch.float8_e8m0fnu, torch.uint8), f"Invalid scales.dtype, got {scales.dtype}."
        assert self.dtype is not None, "Input dtype should be either torch.float16 or torch.bfloat16, not None."
        if scales.dtype == torch.uint8:
            scales = scales.view(torch.float8_e8m0fnu)
        bias = bias.to(device=self.device, dtype=self.dtype) if bias is not None else None
        layer = GemLiteLinear(
            self.W_nbits, group_size=32, in_features=in_features, out_features=out_features,
            input_dtype=DType.MXFP8, output_dtype=TORCH_TO_DTYPE[self.dtype], scaled_activations=True,
        )
        layer.pack(weight.to(self.device), scales.to(self.device), zeros=None, bias=bias, packed=packed)
        layer.W_group_mode = 0
        layer.channel_scale_mode = 2 if self.post_scale else 4
        return layer

    def from_linear(self, linear_layer, del_orig=True):
        if self.dtype is None:
            self.dtype = linear_layer.weight.dtype
        if self.quantizer_mx is None:
            self.quantizer_mx = WeightQuantizerMXFP(device=self.device, compute_dtype=linear_layer.weight.dtype)
        W = linear_layer.weight.data
        bias = linear_layer.bias.clone() if linear_layer.bias is not None else None
        N, K = W.shape
        if self.W_nbits == 8:
            W_q, scales = self.quantizer_mx.quantize_mxfp8(W, index=True, mx_fp8_dtype=self.mx_fp8_dtype)
        else:
            W_q, scales = self.quantizer_mx.quantize_mxfp4(W, index=True)
        W_q, scales = W_q.view(N, K), scales.view(N, K // 32)
        cleanup_linear(linear_layer, del_orig)
        return self.from_weights(weight=W_q, scales=scales, bias=bias)


class A8W8_MXFP_dynamic(A8Wn_MXFP_dynamic):
    """(reference: gemlite/helper.py:1034-1036)"""

    def __init__(self, device="cuda:0", dtype=None, post_scale=True, fp8=torch.float8_e4m3fn):
        super().__init__(device=device, dtype=dtype, post_scale=post_scale, fp8=fp8, W_nbits=8)


class A8W4_MXFP_dynamic(A8Wn_MXFP_dynamic):
    """(reference: gemlite/helper.py:1038-1040)"""

    def __init__(self, device="cuda:0", dtype=None, post_scale=True, fp8=torch.float8_e4m3fn):
        super().__init__(device=device, dtype=dtype, post_scale=post_scale, fp8=fp8, W_nbits=4)


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


class A16W158_INT:
    """fp16/bf16 activations x ternary weights {-1, 0, 1} stored as 2-bit codes w + 1 with a scalar
    zero point of 1 and one weight scale applied after the K sum (W_group_mode 1, channel_scale_mode 1)
    (reference: gemlite/helper.py:1208-1262)."""

    def __init__(self, device="cuda:0", dtype=None, fp32_scale=True):
        self.device = device
        self.dtype = dtype
        self.fp32_scale = fp32_scale

    def _layer(self, weight, weight_scale, bias, input_dtype, scaled_activations, csm):
        if isinstance(weight, torch.nn.Parameter):
            weight = weight.data
        if isinstance(bias, torch.nn.Parameter):
            bias = bias.data
        dtype = weight.dtype if self.dtype is None else self.dtype
        assert dtype in (torch.float16, torch.bfloat16, torch.float32), "Invalid weight.dtype, should be floating point."
        weight = weight.to(dtype=dtype, device=self.device)
        W_q = (weight + 1).to(torch.uint8)
        out_features, in_features = W_q.shape
        scale = float(weight_scale.item()) if isinstance(weight_scale, torch.Tensor) else float(weight_scale)
        scales = torch.full((out_features, 1), scale, dtype=torch.float32 if self.fp32_scale else dtype, device=W_q.device)
        bias = bias.to(device=self.device, dtype=dtype) if bias is not None else None
        layer = GemLiteLinear(
            2, group_size=in_features, in_features=in_features, out_features=out_features,
            input_dtype=TORCH_TO_DTYPE[dtype] if input_dtype is None else input_dtype,
            output_dtype=TORCH_TO_DTYPE[dtype], scaled_activations=scaled_activations,
        )
        layer.pack(W_q, scales=scales, zeros=1, bias=bias)
        layer.W_group_mode, layer.channel_scale_mode = 1, csm
        return layer

    def from_weights(self, weight, weight_scale, bias=None):
        return self._layer(weight, weight_scale, bias, None, False, 1)

    def from_bitlinear(self, linear_layer, del_orig=True):
        out_layer = self.from_weights(weight=linear_layer.weight, weight_scale=linear_layer.weight_scale,
                                      bias=linear_layer.bias)
        cleanup_linear(linear_layer, del_orig)
        return out_layer


class A8W158_INT_dynamic(A16W158_INT):
    """int8 activations quantised per token x ternary weights, INT8 x INT8 -> INT32 accumulation, both
    scales applied after the K sum (W_group_mode 1, channel_scale_mode 3)
    (reference: gemlite/helper.py:1264-1321)."""

    def from_weights(self, weight, weight_scale, bias=None):
        return self._layer(weight, weight_scale, bias, DType.INT8, True, 3)


default_batch_sizes = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048, 4096]


def warmup(processor, shapes, batch_sizes=default_batch_sizes, group_size=64, dtype=torch.float16):
    """Build a layer of every ``(out_features, in_features)`` shape with ``processor`` and tune it at
    every batch size, filling the config cache that ``GemLiteLinear.cache_config`` saves.  The
    reference's function of the same name runs each shape once so that Triton autotunes it
    (reference: gemlite/helper.py:1326-1376); here the offline tuner times the few tile alternatives
    of the kernel family instead.  Processors that start from an HQQ layer need weights quantised
    elsewhere and are refused."""
    from .tune import tune_layer
    if not hasattr(processor, "from_linear"):
        raise ImportError("warmup() needs a processor with from_linear(); HQQ-based ones need the `hqq` package")
    device = torch.device("cuda", torch.cuda.current_device())
    results = {}
    for out_features, in_features in shapes:
        linear = torch.nn.Linear(in_features, out_features, bias=False, dtype=dtype, device=device)
        layer = processor.from_linear(linear)
        results[(out_features, in_features)] = tune_layer(layer, batch_sizes)
        del layer, linear
        torch.cuda.empty_cache()
        gc.collect()
    return results
