"""``GemLiteLinear``: the packed quantized linear layer and its functional forward.

Host-side mirror of the reference module (reference: gemlite/core.py).  The
public surface - constructor, ``pack``, ``forward`` / ``forward_manual``,
``get_meta_args`` / ``get_tensor_args``, the state-dict schema and the
config-cache helpers - keeps the reference's names, argument meaning and error
behaviour; the kernels underneath are HIP kernels reached through the C ABI
(``gemlite_amd._ext``).
"""
import json
import logging
import threading
from typing import List, Optional, Union

import torch
from torch import Tensor

from . import _ext
from .bitpack import pack_weights_over_cols
from .dtypes import (
    DType,
    DTYPE_TO_TORCH,
    FP8_INT8_DTYPES,
    TORCH_TO_DTYPE,
    is_mx_dtype,
)
from .quant_utils import (scale_activations_mxfp4, scale_activations_mxfp8, scale_activations_per_block,
                          scale_activations_per_token)

logger = logging.getLogger(__name__)
_FILE_LOCK = threading.Lock()

# Accumulator type per input type (reference: gemlite/core.py:40-55).
GEMLITE_ACC_DTYPE = {
    DType.FP16: DType.FP32,
    DType.BF16: DType.FP32,
    DType.FP32: DType.FP32,
    DType.FP8: DType.FP32,
    DType.FP8e4nuz: DType.FP32,
    DType.FP8e5: DType.FP32,
    DType.FP8e5nuz: DType.FP32,
    DType.INT8: DType.INT32,
    DType.MXFP16: DType.FP32,
    DType.MXBF16: DType.FP32,
    DType.MXFP8: DType.FP32,
    DType.MXFP4: DType.FP32,
    DType.NVFP4: DType.FP32,
}

# Kernel-family names, in the order the integer ids are serialised
# (reference: gemlite/core.py:57-67).
GEMLITE_MATMUL_TYPES = ["GEMV", "GEMV_REVSPLITK", "GEMV_SPLITK", "GEMM_SPLITK", "GEMM"]
GEMLITE_MATMUL_TYPES_MAPPING = {name: i for i, name in enumerate(GEMLITE_MATMUL_TYPES)}

# {matmul_type: {"(Mc, N, K, group_size, e, type_id)": tile config}}; same key
# format as the reference's autotune cache (reference: gemlite/core.py:68,
# gemlite/triton_kernels/gemm_kernels.py:31-34).
GEMLITE_CONFIG_CACHE = {}


# ---------------------------------------------------------------------------
# global settings
# ---------------------------------------------------------------------------
def set_packing_bitwidth(packing_bitwidth: int):
    """Default word width used by ``pack`` (reference: gemlite/core.py:96-97)."""
    GemLiteLinear.PACKING_BITWIDTH = packing_bitwidth


def set_acc_dtype(dtype):
    """Only fp32 accumulation exists in this build (reference: gemlite/core.py:100-103)."""
    if dtype != DType.FP32:
        raise NotImplementedError("only DType.FP32 accumulation is available for floating-point inputs")


def get_default_gemv(W_nbits: int, mx_dtype: bool = False) -> str:
    """(reference: gemlite/core.py:163-168)"""
    if mx_dtype:
        return "GEMM_SPLITK"
    return "GEMV_REVSPLITK" if W_nbits < 8 else "GEMV_SPLITK"


def get_matmul_type(batch_size: int, W_nbits: int, mx_dtype: bool = False) -> str:
    """Kernel family for a batch size (reference: gemlite/core.py:171-179)."""
    if batch_size >= 64:
        return "GEMM"
    gemv_limit = 4 if (W_nbits < 8 and not mx_dtype) else 2
    if batch_size > gemv_limit:
        return "GEMM_SPLITK"
    return get_default_gemv(W_nbits, mx_dtype)


_CLOSEST_M_VALUES = sorted(
    {2 ** i for i in range(13)}
    | {(2 ** i + 2 ** (i + 1)) // d for i in range(5, 12) for d in (2, 4)}
)


def get_closest_m(M: int) -> int:
    """Batch-size bucket used in config keys: next value in {2^i} U {0.75, 1.5 * 2^i for
    2^i >= 32}, capped at 4096 (reference: gemlite/triton_kernels/utils.py:185-220)."""
    if M > 4096:
        return 4096
    for v in _CLOSEST_M_VALUES:
        if v >= M:
            return v
    return 4096


def get_type_id(input_dtype: int, W_nbits: int) -> int:
    """``input_dtype * 100 + W_nbits`` with bf16 folded onto fp16 (reference: gemlite/core.py:206-210)."""
    if input_dtype == DType.BF16.value:
        input_dtype = DType.FP16.value
    if input_dtype == DType.MXBF16.value:
        input_dtype = DType.MXFP16.value
    return input_dtype * 100 + W_nbits


def config_key(M: int, N: int, K: int, group_size: int, elements_per_sample: int, type_id: int) -> str:
    return str((get_closest_m(M), N, K, group_size, elements_per_sample, type_id))


def _cached_tile_config(matmul_type: str, key: str) -> int:
    entry = GEMLITE_CONFIG_CACHE.get(matmul_type, {}).get(key)
    if entry is None:
        return -1
    if isinstance(entry, dict):
        return int(entry.get("tile_config", -1))
    return int(entry)


# rows up to which forward() asks the matmul to quantise the activations itself (the library may still decline)
_FUSED_QUANT_ROWS = 4


def _bias_is_fusable(bias, output_dtype, x2d):
    return bias is not None and bias.dtype in _BIAS_DTYPES and DTYPE_TO_TORCH[output_dtype] in _BIAS_DTYPES \
        and bias.dim() == 1 and bias.is_contiguous() and bias.device == x2d.device


# ---------------------------------------------------------------------------
# functional forward
# ---------------------------------------------------------------------------
def forward_functional(
    x: Tensor,
    bias: Optional[Tensor],
    tensor_args: List[Tensor],
    meta_args: List[int],
    matmul_type: int = -1,
) -> Tensor:
    """``out = x @ dequant(W).T (+ bias)`` (reference: gemlite/core.py:193-274).

    ``tensor_args = [W_q, scales, zeros, meta_scale]``; ``meta_args`` are the 12
    ints of ``get_meta_args``; ``matmul_type`` indexes ``GEMLITE_MATMUL_TYPES``
    (-1 = choose from the batch size).
    """
    W_q, scales, zeros = tensor_args[0], tensor_args[1], tensor_args[2]
    (scaled_activations, W_nbits, group_size, unpack_mask, elements_per_sample, input_dtype, output_dtype,
     acc_dtype, meta_dtype, channel_scale_mode, W_group_mode, data_contiguous) = [int(v) for v in meta_args]

    if x.device.type != "cuda":
        raise RuntimeError("GemLiteLinear.forward runs on the GPU only (input is on '%s')" % x.device)

    out_features = W_q.shape[1]
    if not x.is_contiguous():
        x = x.contiguous()
    out_shape = x.shape[:-1] + (out_features,)
    x2d = x.view(-1, x.shape[-1])

    scales_x = None
    kernel_input_dtype = input_dtype
    if scaled_activations and x2d.shape[0] <= _FUSED_QUANT_ROWS and x2d.dtype in (torch.float16, torch.bfloat16):
        # decode sizes: the streaming kernels quantise the rows themselves (same codes and scales as the quantiser
        # launch, one launch less); the library says whether the call at hand is one they take
        in_dt = DType(input_dtype)
        if (in_dt in FP8_INT8_DTYPES and channel_scale_mode in (2, 3)) or (in_dt == DType.MXFP4 and channel_scale_mode == 4):
            fused_bias = _bias_is_fusable(bias, output_dtype, x2d)
            type_str = GEMLITE_MATMUL_TYPES[matmul_type] if matmul_type >= 0 else get_matmul_type(
                x2d.shape[0], W_nbits, is_mx_dtype(input_dtype))
            out = _KERNEL_FORWARD[type_str](
                x2d, W_q, scales, zeros, None, W_nbits, group_size, unpack_mask, elements_per_sample,
                input_dtype, output_dtype, acc_dtype, meta_dtype, channel_scale_mode, W_group_mode,
                data_contiguous, get_type_id(input_dtype, W_nbits), bias=bias if fused_bias else None,
                x_quant_from=TORCH_TO_DTYPE[x2d.dtype].value,
            )
            if out is not None:
                out = out.view(out_shape)
                if bias is not None and not fused_bias:
                    out += bias
                return out
    if scaled_activations:
        in_dt = DType(input_dtype)
        if in_dt in FP8_INT8_DTYPES and channel_scale_mode == 5:  # 128 x 128 block quantisation
            x2d, scales_x = scale_activations_per_block(x2d, w_dtype=DTYPE_TO_TORCH[input_dtype])
        elif in_dt in FP8_INT8_DTYPES:
            x2d, scales_x = scale_activations_per_token(x2d, w_dtype=DTYPE_TO_TORCH[input_dtype])
        elif in_dt == DType.MXFP4 and channel_scale_mode == 4:
            x2d, scales_x = scale_activations_mxfp4(x2d)
        elif in_dt == DType.MXFP8 and channel_scale_mode == 4:  # MXFP8 micro-scales on both sides
            x2d, scales_x = scale_activations_mxfp8(x2d)
        elif in_dt == DType.MXFP8 and channel_scale_mode == 2:  # MXFP8 weights, per-token post-scaled activations
            x2d, scales_x = scale_activations_per_token(x2d, w_dtype=torch.float8_e4m3fn)
        else:
            raise NotImplementedError(
                f"dynamic activation quantisation for input_dtype={in_dt}, channel_scale_mode={channel_scale_mode}"
            )
    elif x2d.dtype in TORCH_TO_DTYPE and not is_mx_dtype(input_dtype):
        # the kernels read x as the element type it actually has
        kernel_input_dtype = TORCH_TO_DTYPE[x2d.dtype].value
    elif input_dtype in (DType.MXFP16.value, DType.MXBF16.value):
        # weight-only MX layer: the 16-bit activations go to the kernel as they are
        if x2d.dtype == torch.float16:
            kernel_input_dtype = DType.MXFP16.value
        elif x2d.dtype == torch.bfloat16:
            kernel_input_dtype = DType.MXBF16.value
        else:
            raise NotImplementedError(f"weight-only MX layers take fp16 or bf16 activations, got {x2d.dtype}")

    M = x2d.shape[0]
    mx = is_mx_dtype(input_dtype)
    if matmul_type >= 0:
        matmul_type_str = GEMLITE_MATMUL_TYPES[matmul_type]
    else:
        matmul_type_str = get_matmul_type(M, W_nbits, mx)

    # the library adds a floating-point bias itself (in the GEMV epilogue, or with one small launch after
    # the other kernels); anything else is added here like the reference does (gemlite/core.py:271-272)
    fused_bias = _bias_is_fusable(bias, output_dtype, x2d)
    out = _KERNEL_FORWARD[matmul_type_str](
        x2d, W_q, scales, zeros, scales_x, W_nbits, group_size, unpack_mask, elements_per_sample,
        kernel_input_dtype, output_dtype, acc_dtype, meta_dtype, channel_scale_mode, W_group_mode,
        data_contiguous, get_type_id(input_dtype, W_nbits), bias=bias if fused_bias else None,
    )

    out = out.view(out_shape)
    if bias is not None and not fused_bias:
        out += bias
    return out


# ---------------------------------------------------------------------------
# kernel plug-in level: one class per matmul type with the reference's interface
# (reference: gemlite/core.py:57-67; gemlite/triton_kernels/gemm_kernels.py:741-799 and the
# matching classes of the GEMV / split-K files).  All five run gla_matmul; the type is a hint the
# library's dispatcher may override (up to 16 rows the streaming kernels run whatever was asked for).
# ---------------------------------------------------------------------------
# Prepared launches: filling and bounds-checking a gla_matmul_args costs more host time than a
# decode-sized kernel runs, so a filled struct is kept per (weight tensor object, shapes, strides,
# dtypes, modes, tile) and later calls only refresh the activation / output addresses.  An entry is
# trusted only while the weight, scale and zero tensors still sit at the addresses it was built for.
# Entries are per thread: the struct is rewritten in place on every call.
_PREPARED = {}
_PREPARED_LIMIT = 8192
_DECLINED = object()  # cached answer: the library has no kernel for this (optional) form of the call
_thread_id = threading.get_ident


def _kernel_forward(matmul_type_str):
    matmul_type_id = GEMLITE_MATMUL_TYPES_MAPPING[matmul_type_str]

    def forward(x, W_q, scales, zeros, scales_x, W_nbits, group_size, unpack_mask, elements_per_sample,
                input_dtype, output_dtype, acc_dtype, meta_dtype, channel_scale_mode, W_group_mode,
                data_contiguous, type_id, meta_scale=0.0, bias=None, x_quant_from=0):
        """``x_quant_from``: DType value of the 16-bit rows in ``x`` that the kernel is to quantise to ``input_dtype``
        itself; returns None when the library has no kernel that does so for this call."""
        M, K, N = x.shape[0], W_q.shape[0] * elements_per_sample, W_q.shape[1]
        out = torch.empty((M, N), dtype=DTYPE_TO_TORCH[int(output_dtype)], device=x.device)
        if M == 0:
            return out
        if GEMLITE_CONFIG_CACHE:
            tile = _cached_tile_config(matmul_type_str, config_key(M, N, K, group_size, elements_per_sample, type_id))
        else:
            tile = -1
        sx_key = None if scales_x is None else (scales_x.shape, scales_x.stride(), scales_x.dtype)
        key = (id(W_q), W_q.shape, W_q.stride(), _thread_id(), matmul_type_id, x.shape, x.stride(), x.dtype, sx_key,
               x.device.index, W_nbits, group_size,
               unpack_mask, elements_per_sample, input_dtype, output_dtype, acc_dtype, meta_dtype, channel_scale_mode,
               W_group_mode, data_contiguous, tile, None if bias is None else (bias.data_ptr(), bias.dtype), x_quant_from)
        hit = _PREPARED.get(key)
        if hit is _DECLINED:
            return None
        if hit is not None:
            args, need, w_ptr, s_ptr, z_ptr = hit
            if (W_q.data_ptr() == w_ptr and (scales is None or scales.data_ptr() == s_ptr)
                    and (zeros is None or zeros.data_ptr() == z_ptr)):
                _ext.matmul_prepared(args, need, x.data_ptr(), out.data_ptr(),
                                     None if scales_x is None else scales_x.data_ptr(), x.device)
                return out
        args = _ext.build_matmul_args(
            x, W_q, scales, zeros, scales_x, out,
            W_nbits=W_nbits, group_size=group_size, unpack_mask=unpack_mask,
            elements_per_sample=elements_per_sample, input_dtype=input_dtype, output_dtype=output_dtype,
            acc_dtype=acc_dtype, meta_dtype=meta_dtype, channel_scale_mode=channel_scale_mode,
            W_group_mode=W_group_mode, data_contiguous=data_contiguous,
            matmul_type=matmul_type_id, tile_config=tile, bias=bias, x_quant_from=x_quant_from,
        )
        if x_quant_from and not _ext.matmul_is_supported(args):
            if len(_PREPARED) >= _PREPARED_LIMIT:
                _PREPARED.clear()
            _PREPARED[key] = _DECLINED
            return None
        need = _ext.matmul_workspace_need(args)
        _ext.matmul_prepared(args, need, args.x, args.out, args.scales_x, x.device)
        if len(_PREPARED) >= _PREPARED_LIMIT:
            _PREPARED.clear()
        _PREPARED[key] = (args, need, W_q.data_ptr(), None if scales is None else scales.data_ptr(),
                          None if zeros is None else zeros.data_ptr())
        return out
    return forward


_BIAS_DTYPES = (torch.float16, torch.bfloat16, torch.float32)
_KERNEL_FORWARD = {}  # matmul type -> forward with the extra `bias` argument (what forward_functional calls)


def _kernel_class(matmul_type_str):
    inner = _KERNEL_FORWARD[matmul_type_str] = _kernel_forward(matmul_type_str)

    def forward(x, W_q, scales, zeros, scales_x, W_nbits, group_size, unpack_mask, elements_per_sample,
                input_dtype, output_dtype, acc_dtype, meta_dtype, channel_scale_mode, W_group_mode,
                data_contiguous, type_id, meta_scale=0.0):
        # the reference's argument list, which has no bias
        return inner(x, W_q, scales, zeros, scales_x, W_nbits, group_size, unpack_mask, elements_per_sample,
                     input_dtype, output_dtype, acc_dtype, meta_dtype, channel_scale_mode, W_group_mode,
                     data_contiguous, type_id, meta_scale)

    return type(matmul_type_str.lower(), (), {
        "kernel": ["gla_matmul"],
        "matmul_type": matmul_type_str,
        "forward": staticmethod(forward),
        "__doc__": f"Kernel plug-in for matmul type {matmul_type_str}: forward(x, W_q, scales, zeros, scales_x, "
                   "W_nbits, ..., type_id) -> Tensor[M, N], backed by the C ABI.",
    })


GEMLITE_TRITON_MAPPING = {name: _kernel_class(name) for name in GEMLITE_MATMUL_TYPES}


# The same function as a torch custom op with a fake (meta) implementation, so that graphs traced
# by torch.compile hold it as one opaque node instead of tracing into ctypes
# (reference: gemlite/core.py:193-200, :276-285).  The module's forward goes through the op while
# a graph is being traced and calls the plain function otherwise: eager decode steps do not pay the
# op dispatch (~10 us per call against a ~7 us kernel).
def _make_custom_op():
    try:
        @torch.library.custom_op("gemlite::forward_functional", mutates_args=())
        def forward_functional_op(x: Tensor, bias: Optional[Tensor], tensor_args: List[Tensor], meta_args: List[int],
                                  matmul_type: int = -1) -> Tensor:
            return forward_functional(x, bias, tensor_args, meta_args, matmul_type)

        @forward_functional_op.register_fake
        def _(x, bias, tensor_args, meta_args, matmul_type=-1):
            # the dtype forward_functional really returns (the reference's fake says x.dtype, which
            # is the same thing for every processor it ships: output type = activation type)
            out_features = tensor_args[0].shape[1]
            return torch.empty(x.shape[:-1] + (out_features,), device=x.device, dtype=DTYPE_TO_TORCH[int(meta_args[6])])

        return forward_functional_op
    except Exception as exc:  # the name is taken (the reference package is loaded in this process) or torch is too old
        logger.warning("gemlite_amd: torch custom op gemlite::forward_functional was not registered (%s); "
                       "torch.compile will trace into the plain Python forward", exc)
        return None


forward_functional_op = _make_custom_op()


def _dispatch_forward(x, bias, tensor_args, meta_args, matmul_type=-1):
    if forward_functional_op is not None and torch.compiler.is_compiling():
        return forward_functional_op(x, bias, tensor_args, meta_args, matmul_type)
    return forward_functional(x, bias, tensor_args, meta_args, matmul_type)


# ---------------------------------------------------------------------------
# module
# ---------------------------------------------------------------------------
class GemLiteLinear(torch.nn.Module):
    """Quantized linear layer (reference: gemlite/core.py:289-836)."""

    SUPPORTED_BITS = [1, 2, 4, 8, 16]
    SUPPORTED_BITS_TRITON = SUPPORTED_BITS  # name kept for callers of the reference
    SUPPORTED_DTYPES = [
        DType.FP16, DType.BF16, DType.FP32, DType.FP8, DType.FP8e4nuz, DType.FP8e5, DType.FP8e5nuz,
        DType.INT8, DType.MXFP16, DType.MXBF16, DType.MXFP8, DType.MXFP4, DType.NVFP4,
    ]
    MIN_SIZE = 32
    PACKING_BITWIDTH = 32

    _SCHEMA = ("W_q", "bias", "scales", "zeros", "metadata", "orig_shape", "meta_scale")

    def __init__(
        self,
        W_nbits=4,
        group_size=64,
        in_features=None,
        out_features=None,
        input_dtype=DType.FP16,
        output_dtype=DType.FP16,
        acc_dtype=None,
        scaled_activations=False,
    ):
        super().__init__()
        # validation (reference: gemlite/core.py:325-350)
        if W_nbits not in self.SUPPORTED_BITS:
            raise NotImplementedError("Only " + str(self.SUPPORTED_BITS) + " W_nbits are supported.")
        if in_features is not None and out_features is not None:
            bad_k = in_features % self.MIN_SIZE != 0
            bad_g = group_size is not None and W_nbits < 16 and in_features % group_size != 0
            if bad_k or bad_g:
                raise NotImplementedError(
                    f"Invalid input shapes: {in_features} , {out_features}. "
                    "in_features should be divisible by 32 or the group_size"
                )
        if input_dtype not in self.SUPPORTED_DTYPES:
            raise NotImplementedError("Unsupport input dtype: " + str(input_dtype))
        if group_size is not None and group_size < 16:
            raise NotImplementedError("Only group_size >= 16 is supported.")

        self.in_features = in_features
        self.out_features = out_features
        self.W_nbits = W_nbits
        self.group_size = 1 if group_size is None else group_size
        self.unpack_mask = 2 ** W_nbits - 1
        self.elements_per_sample = None
        self.signature = (in_features, out_features, W_nbits, self.group_size)

        self.input_dtype = input_dtype
        self.output_dtype = output_dtype
        self.compute_dtype = DTYPE_TO_TORCH[input_dtype.value]
        self.meta_dtype = input_dtype
        self.acc_dtype = GEMLITE_ACC_DTYPE[input_dtype] if acc_dtype is None else acc_dtype

        # float inputs are never re-quantised (reference: gemlite/core.py:371-374)
        float_in = self.compute_dtype in (torch.float16, torch.bfloat16, torch.float32)
        self.scaled_activations = False if float_in else scaled_activations

        self.forward = self.forward_auto_no_warmup

        # checkpoint schema advertised by a fresh module (reference: gemlite/core.py:382-389)
        self.register_buffer("W_q", torch.empty(0, dtype=torch.uint8))
        self.register_buffer("scales", torch.empty(0, dtype=torch.uint8))
        self.register_buffer("zeros", torch.empty(0, dtype=torch.int32))
        self.register_buffer("metadata", torch.empty(0, dtype=torch.int32))
        self.register_buffer("orig_shape", torch.empty(0, dtype=torch.int32))
        self.register_buffer("meta_scale", torch.tensor(0.0, dtype=torch.float32))
        self.register_parameter("bias", None)

    # -- slot management: schema entries switch between buffers, parameters and plain values
    def _drop(self, name):
        self._buffers.pop(name, None)
        self._parameters.pop(name, None)
        self.__dict__.pop(name, None)

    def _set_param(self, name, tensor):
        self._drop(name)
        if tensor is None:
            self.register_parameter(name, None)
        else:
            self.register_parameter(name, torch.nn.Parameter(tensor, requires_grad=False))

    # ------------------------------------------------------------------ pack
    def pack(
        self,
        W_q: Tensor,
        scales: Optional[Tensor],
        zeros: Union[Tensor, int, None],
        bias: Optional[Tensor] = None,
        fma_mode: bool = True,
        contiguous: Optional[bool] = None,
        packing_bitwidth: Optional[int] = None,
        packed: bool = False,
    ):
        """Lay out the weights and choose the dequant / scaling modes
        (reference: gemlite/core.py:559-795)."""
        N, K = self.out_features, self.in_features
        mx = is_mx_dtype(self.input_dtype)

        if zeros is not None and self.input_dtype == DType.INT8:
            fractional = (isinstance(zeros, Tensor) and bool(zeros.mean() != zeros.int().float().mean())) or isinstance(
                zeros, float
            )
            if fractional:
                raise Exception("INT8 inputs is not compatible with floating-point zeros.")

        if packing_bitwidth is None:
            packing_bitwidth = GemLiteLinear.PACKING_BITWIDTH
        if mx:
            packing_bitwidth = 8  # micro-scaled formats are byte packed

        # ---- weight layout
        w_view, e = None, None
        if W_q.dtype == torch.int8 or W_q.is_floating_point():
            expect = {torch.float32: 32, torch.float16: 16, torch.bfloat16: 16}.get(W_q.dtype, 8)
            assert self.W_nbits == expect, f"Invalid {W_q.dtype} weights for W_nbits={self.W_nbits}."
            w_view, e = W_q.t(), 1
            if contiguous is None:
                contiguous = False
        if packed and W_q.dtype == torch.uint8:
            e = packing_bitwidth // self.W_nbits
            w_view = W_q.view(N, K // e).t()
            if contiguous is None:
                contiguous = not mx
        elif W_q.dtype == torch.uint8:
            w_view, e = pack_weights_over_cols(
                W_q.view((N, K)), W_nbits=self.W_nbits, packing_bitwidth=packing_bitwidth, transpose=True
            )
            if contiguous is None:
                contiguous = not mx
        if w_view is None:
            raise Exception("Weights were not packed, please check your W_q.dtype")

        device = w_view.device
        bias_t = None if bias is None else bias.to(device=device)

        # ---- dequant / channel-scale modes (reference: gemlite/core.py:647-703)
        scales_t = None if scales is None else scales.view((N, -1)).t()
        channelwise = scales_t is not None and scales_t.numel() == N
        csm = 0
        if scales is None and zeros is None:
            csm = 2 if self.scaled_activations else 0

        if zeros is None:
            zeros_t = None
            wgm = 2 if scales_t is not None else 0
        elif isinstance(zeros, Tensor):
            if fma_mode and not channelwise:
                # w = q * s + z'  with z' = -z * s rounded once to the zeros dtype
                zeros_t = (-zeros.float() * scales.float()).to(zeros.dtype).view((N, -1)).t()
                wgm = 4
            else:
                zeros_t = zeros.view((N, -1)).t()
                wgm = 3
        else:
            zeros_t = int(zeros)
            wgm = 3 if scales_t is not None else 1

        if channelwise and not self.scaled_activations:
            csm = 1
            wgm = 1 if zeros_t is not None else 0
        if self.scaled_activations and not channelwise:
            csm = 2
        if self.scaled_activations and channelwise:
            csm = 3
            wgm = 1 if zeros_t is not None else 0
        if csm in (1, 3):
            assert wgm not in (3, 4), "Can't use channel_scale_mode with W_group_mode == 3 or 4."

        # ---- placeholders for absent metadata, contiguity
        if isinstance(zeros_t, int):
            zeros_t = torch.tensor(zeros_t, dtype=torch.int32, device=device)
        if zeros_t is None:
            zeros_t = torch.tensor([[]], dtype=torch.int32, device=device)
        if scales_t is None:
            scales_t = torch.tensor([[]], dtype=torch.int32, device=device)

        self.data_contiguous = bool(contiguous)
        if contiguous:
            w_view = w_view.contiguous()
        scales_t = scales_t.contiguous()
        zeros_t = zeros_t.contiguous()

        # ---- micro-scaled formats: e8m0 scales handed over as the [N, K/gs] view
        if self.input_dtype in (DType.MXFP16, DType.MXBF16, DType.MXFP8, DType.MXFP4):
            scales_t = scales_t.to(torch.float8_e8m0fnu).view(torch.uint8)
        if self.input_dtype == DType.NVFP4:
            scales_t = scales_t.to(torch.float8_e4m3fn)
        if mx:
            wgm, csm = 2, 0
            # [N, K/gs] like the reference's view (gemlite/core.py:719), but materialised row-major
            # so that the block scales of one output row are consecutive bytes for the MFMA kernel
            scales_t = scales_t.T.contiguous()

        self.W_group_mode = wgm
        self.channel_scale_mode = csm
        self.elements_per_sample = e
        self.device = device
        self.meta_is_channelwise = channelwise
        if scales_t is not None:
            self.meta_dtype = TORCH_TO_DTYPE[scales_t.dtype]

        ms = self.meta_scale
        ms_val = float(ms.item()) if isinstance(ms, Tensor) else float(ms)

        self._set_param("W_q", w_view)
        self._set_param("scales", scales_t)
        self._set_param("zeros", zeros_t)
        self._set_param("bias", bias_t)
        self._set_param("metadata", torch.tensor(self.get_meta_args(), device=device, dtype=torch.int32))
        self._set_param("orig_shape", torch.tensor([N, K], device=device, dtype=torch.int32))
        self._set_param("meta_scale", torch.tensor(ms_val, device=device, dtype=torch.float32))
        return self

    # ------------------------------------------------------------- accessors
    def get_tensor_args(self):
        """(reference: gemlite/core.py:798-802)"""
        meta_scale = self.meta_scale
        if not isinstance(meta_scale, Tensor):
            meta_scale = torch.tensor(meta_scale, dtype=torch.float32, device=self.W_q.device)
        return [self.W_q, self.scales, self.zeros, meta_scale]

    def get_meta_args(self):
        """The 12 serialised ints, in the reference's order (reference: gemlite/core.py:804-817)."""
        return [
            int(self.scaled_activations),
            self.W_nbits,
            self.group_size,
            self.unpack_mask,
            self.elements_per_sample,
            self.input_dtype.value,
            self.output_dtype.value,
            self.acc_dtype.value,
            self.meta_dtype.value,
            self.channel_scale_mode,
            self.W_group_mode,
            int(self.data_contiguous),
        ]

    # --------------------------------------------------------------- forward
    def forward_manual(self, x: Tensor, matmul_type: str = "GEMM") -> Tensor:
        """(reference: gemlite/core.py:820-827)"""
        return _dispatch_forward(
            x, self.bias, self.get_tensor_args(), self.get_meta_args(), GEMLITE_MATMUL_TYPES_MAPPING[matmul_type]
        )

    def forward_auto_no_warmup(self, x: Tensor) -> Tensor:
        """(reference: gemlite/core.py:830-836)"""
        return _dispatch_forward(x, self.bias, self.get_tensor_args(), self.get_meta_args())

    # ------------------------------------------------------------ state dict
    def _save_to_state_dict(self, destination, prefix, keep_vars):
        # Modes may have been overridden after pack(); serialise the live values
        # (reference: gemlite/core.py:419-430).
        w = getattr(self, "W_q", None)
        if isinstance(w, Tensor) and w.numel() > 0 and self.elements_per_sample is not None:
            self._set_param("metadata", torch.tensor(self.get_meta_args(), device=w.device, dtype=torch.int32))
        super()._save_to_state_dict(destination, prefix, keep_vars)
        # Micro-scaled layers keep their e8m0 scales [N, K/32] row-major in memory (K-contiguous, what the
        # MFMA kernels read).  The reference holds the same shape as the transposed view of a
        # [K/32, N] buffer (gemlite/core.py:752) and torch.save keeps strides, so the checkpoint
        # gets that stride order; loading accepts either (_apply_state_dict).
        sc = destination.get(prefix + "scales")
        if (isinstance(sc, Tensor) and sc.dim() == 2 and sc.numel() > 0 and self.elements_per_sample is not None
                and is_mx_dtype(self.input_dtype) and sc.stride(-1) == 1 and sc.shape[0] > 1):
            destination[prefix + "scales"] = sc.detach().t().contiguous().t()

    def _apply_state_dict(self, sd):
        """Populate the module from short-keyed checkpoint tensors
        (reference: gemlite/core.py:432-512)."""
        W_q, metadata, orig_shape = sd.get("W_q"), sd.get("metadata"), sd.get("orig_shape")
        if W_q is None or metadata is None or orig_shape is None:
            raise RuntimeError(
                "GemLite checkpoint is missing required keys (W_q / metadata / orig_shape). "
                f"Got keys: {sorted(k for k, v in sd.items() if v is not None)}"
            )
        meta = [int(v) for v in metadata.tolist()]
        (sa, self.W_nbits, self.group_size, self.unpack_mask, self.elements_per_sample, in_dt, out_dt, acc_dt,
         meta_dt, self.channel_scale_mode, self.W_group_mode, dc) = meta
        self.scaled_activations = bool(sa)
        self.data_contiguous = bool(dc)
        self.input_dtype, self.output_dtype = DType(in_dt), DType(out_dt)
        self.acc_dtype, self.meta_dtype = DType(acc_dt), DType(meta_dt)
        self.out_features, self.in_features = (int(v) for v in orig_shape.tolist())
        self.compute_dtype = DTYPE_TO_TORCH[self.input_dtype.value]

        ms = sd.get("meta_scale")
        if ms is None:
            ms_val = 0.05 if self.input_dtype == DType.NVFP4 else 0.0
        else:
            ms_val = float(ms.float().item()) if isinstance(ms, Tensor) else float(ms)

        device = W_q.device
        self.device = device
        self._set_param("W_q", W_q)
        self._set_param("bias", sd.get("bias"))
        scales = sd.get("scales")
        if scales is not None and is_mx_dtype(self.input_dtype) and scales.dim() == 2 and scales.stride(-1) != 1:
            scales = scales.contiguous()  # checkpoints written by the reference hold the transposed view
        self._set_param("scales", scales)
        self._set_param("zeros", sd.get("zeros"))
        self._set_param("metadata", torch.tensor(self.get_meta_args(), device=device, dtype=torch.int32))
        self._set_param(
            "orig_shape", torch.tensor([self.out_features, self.in_features], device=device, dtype=torch.int32)
        )
        self._set_param("meta_scale", torch.tensor(ms_val, device=device, dtype=torch.float32))

    def load_state_dict(self, state_dict, strict=True, assign=False):
        """Direct load from a raw checkpoint dict (reference: gemlite/core.py:514-527)."""
        sd = {k: state_dict.pop(k, None) for k in self._SCHEMA}
        state_dict.pop("scales_5d", None)
        self._apply_state_dict(sd)

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        """Load through a parent module (reference: gemlite/core.py:529-554)."""
        sd = {k: state_dict.pop(prefix + k) for k in self._SCHEMA if (prefix + k) in state_dict}
        state_dict.pop(prefix + "scales_5d", None)
        if "W_q" not in sd:
            super()._load_from_state_dict(
                state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs
            )
            return
        try:
            self._apply_state_dict(sd)
        except Exception as exc:  # reported through nn.Module's error list
            error_msgs.append(f"GemLite load error at prefix '{prefix}': {exc}")

    # ---------------------------------------------------------- config cache
    @staticmethod
    def cache_config(filename: str):
        """Merge the in-memory tile-config cache into a JSON file
        (reference: gemlite/core.py:838-877)."""
        with _FILE_LOCK:
            try:
                with open(filename, "r") as f:
                    config = json.load(f)
            except Exception:
                config = {}
            for name in GEMLITE_MATMUL_TYPES:
                config.setdefault(name, {})
                config[name].update(GEMLITE_CONFIG_CACHE.get(name, {}))
            with open(filename, "w") as f:
                json.dump(config, f)

    @staticmethod
    def load_config(filename: str, print_error: bool = True, overwrite: bool = False):
        """(reference: gemlite/core.py:879-901)"""
        global GEMLITE_CONFIG_CACHE
        if filename is None:
            return False
        try:
            with _FILE_LOCK, open(filename, "r") as f:
                config = json.load(f)
            if overwrite:
                GEMLITE_CONFIG_CACHE.clear()
            for name, entries in config.items():
                GEMLITE_CONFIG_CACHE.setdefault(name, {}).update(entries)
        except Exception as exc:
            if print_error:
                logger.error(f"Failed to load the cache file '{filename}': {exc}")
            return False
        return True

    @staticmethod
    def reset_config():
        """(reference: gemlite/core.py:903-906)"""
        GEMLITE_CONFIG_CACHE.clear()


GemLiteLinearTriton = GemLiteLinear  # name kept for callers of the reference

__all__ = [
    "GemLiteLinear",
    "GemLiteLinearTriton",
    "DType",
    "TORCH_TO_DTYPE",
    "DTYPE_TO_TORCH",
    "forward_functional",
    "get_matmul_type",
    "get_default_gemv",
    "get_closest_m",
    "get_type_id",
    "config_key",
    "set_packing_bitwidth",
    "set_acc_dtype",
    "GEMLITE_ACC_DTYPE",
    "GEMLITE_MATMUL_TYPES",
    "GEMLITE_MATMUL_TYPES_MAPPING",
    "GEMLITE_TRITON_MAPPING",
    "GEMLITE_CONFIG_CACHE",
]
