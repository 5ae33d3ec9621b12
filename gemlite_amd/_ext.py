"""ctypes binding of ``libgemlite_amd.so`` (the C ABI in ``include/gemlite_amd.h``).

The library is built in-tree by ``gemlite_amd/csrc/Makefile`` (or
``gemlite_amd.build.build_library``).  There is no fallback: if the shared
object is missing, or a call returns a non-zero status, the caller gets an
exception.
"""
import ctypes
import os
import threading
from typing import Optional

import torch

from .dtypes import DType, TORCH_TO_DTYPE, is_mx_dtype

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgemlite_amd.so")

GLA_OK = 0
_ERR_TO_EXC = {
    -1: ValueError,            # GLA_ERR_INVALID_ARGUMENT
    -2: NotImplementedError,   # GLA_ERR_UNSUPPORTED_DTYPE
    -3: NotImplementedError,   # GLA_ERR_UNSUPPORTED_MODE
    -4: ValueError,            # GLA_ERR_MISALIGNED_SHAPE
    -5: RuntimeError,          # GLA_ERR_WORKSPACE_TOO_SMALL
    -6: RuntimeError,          # GLA_ERR_LAUNCH_FAILED
    -7: RuntimeError,          # GLA_ERR_NO_DEVICE
}

MATMUL_AUTO = -1


class MatmulArgs(ctypes.Structure):
    """Mirror of ``gla_matmul_args``; field order and types must match the header."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("matmul_type", ctypes.c_int32),
        ("x", ctypes.c_void_p),
        ("w", ctypes.c_void_p),
        ("scales", ctypes.c_void_p),
        ("zeros", ctypes.c_void_p),
        ("scales_x", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_uint64),
        ("M", ctypes.c_int32),
        ("N", ctypes.c_int32),
        ("K", ctypes.c_int32),
        ("x_stride_m", ctypes.c_int64),
        ("x_stride_k", ctypes.c_int64),
        ("w_stride_k", ctypes.c_int64),
        ("w_stride_n", ctypes.c_int64),
        ("out_stride_m", ctypes.c_int64),
        ("out_stride_n", ctypes.c_int64),
        ("meta_stride_g", ctypes.c_int64),
        ("meta_stride_n", ctypes.c_int64),
        ("sx_stride_m", ctypes.c_int64),
        ("sx_stride_g", ctypes.c_int64),
        ("W_nbits", ctypes.c_int32),
        ("group_size", ctypes.c_int32),
        ("unpack_mask", ctypes.c_int32),
        ("elements_per_sample", ctypes.c_int32),
        ("input_dtype", ctypes.c_int32),
        ("output_dtype", ctypes.c_int32),
        ("acc_dtype", ctypes.c_int32),
        ("meta_dtype", ctypes.c_int32),
        ("channel_scale_mode", ctypes.c_int32),
        ("W_group_mode", ctypes.c_int32),
        ("data_contiguous", ctypes.c_int32),
        ("w_dtype", ctypes.c_int32),
        ("zeros_dtype", ctypes.c_int32),
        ("zero_is_scalar", ctypes.c_int32),
        ("sx_dtype", ctypes.c_int32),
        ("tile_config", ctypes.c_int32),
        ("bias", ctypes.c_void_p),
        ("bias_dtype", ctypes.c_int32),
        ("x_quant_from", ctypes.c_int32),
    ]


_lib = None
_lib_lock = threading.Lock()

# name -> (restype, argtypes); every symbol include/gemlite_amd.h declares
SYMBOLS = {
    "gla_abi_version": (ctypes.c_int, []),
    "gla_last_error": (ctypes.c_char_p, []),
    "gla_get_matmul_type": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "gla_get_closest_m": (ctypes.c_int, [ctypes.c_int]),
    "gla_select_config": (ctypes.c_int, [ctypes.POINTER(MatmulArgs)]),
    "gla_matmul_family": (ctypes.c_int, [ctypes.POINTER(MatmulArgs)]),
    "gla_probe_mfma": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                      ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]),
    "gla_probe_read": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
    "gla_probe_read_cfg": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_int, ctypes.c_void_p]),
    "gla_prefetch": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]),
    "gla_matmul_workspace_bytes": (ctypes.c_int64, [ctypes.POINTER(MatmulArgs)]),
    "gla_matmul": (ctypes.c_int, [ctypes.POINTER(MatmulArgs), ctypes.c_void_p]),
    "gla_matmul_static": (ctypes.c_int, [ctypes.POINTER(MatmulArgs), ctypes.c_void_p]),
    "gla_static_scratch_bytes": (ctypes.c_int64, []),
    "gla_scale_activations_per_token": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_void_p],
    ),
    "gla_scale_activations_per_block": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_void_p],
    ),
    "gla_scale_activations_mxfp4": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p],
    ),
    "gla_scale_activations_mxfp8": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p],
    ),
    "gla_pack_over_cols": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p],
    ),
    "gla_unpack_over_cols": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p],
    ),
}


def load_library(path: Optional[str] = None):
    """Load the shared object and declare prototypes.  Raises if it is missing."""
    global _lib
    with _lib_lock:
        if _lib is not None and path is None:
            return _lib
        p = path or LIB_PATH
        if not os.path.exists(p):
            raise RuntimeError(
                f"{p} not found: the HIP extension is not built. "
                "Run `make -C gemlite_amd/csrc` (or `python -c 'import __graft_entry__ as g; g.build()'`)."
            )
        lib = ctypes.CDLL(p)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.gla_abi_version() != 1:
            raise RuntimeError(f"{p}: ABI version {lib.gla_abi_version()} != 1")
        if path is None:
            _lib = lib
        return lib


def is_available() -> bool:
    return os.path.exists(LIB_PATH)


def _check(status: int, what: str):
    if status == GLA_OK:
        return
    lib = load_library()
    msg = lib.gla_last_error().decode("utf-8", "replace")
    exc = _ERR_TO_EXC.get(status, RuntimeError)
    raise exc(f"{what} failed (status {status}): {msg}")


def _stream_ptr(device) -> int:
    """Raw handle of torch's current stream on ``device`` (the capture stream inside torch.cuda.graph)."""
    index = device.index
    if index is None:
        index = torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(index)


def _require_cuda(*tensors):
    for t in tensors:
        if t is not None and t.device.type != "cuda":
            raise RuntimeError(
                "gemlite_amd kernels run on the GPU only; got a tensor on device '%s'" % t.device
            )


# ---------------------------------------------------------------------------
# dispatcher helpers (host-only, usable without a GPU)
# ---------------------------------------------------------------------------
def get_matmul_type_id(M: int, W_nbits: int, is_mx: bool) -> int:
    return load_library().gla_get_matmul_type(int(M), int(W_nbits), int(bool(is_mx)))


def get_closest_m(M: int) -> int:
    return load_library().gla_get_closest_m(int(M))


# ---------------------------------------------------------------------------
# workspace: one zero-initialised scratch tensor per (device, stream), grown on demand
# ---------------------------------------------------------------------------
_workspaces = {}
_retired_workspaces = []  # outgrown buffers stay allocated: a captured HIP graph may still point at them
_workspace_lock = threading.Lock()
_last_eager_key = {}  # (thread, device index) -> key of the stream that thread last launched on outside a capture


def _workspace_key(device: torch.device, stream: int):
    index = device.index if device.index is not None else torch.cuda.current_device()
    return (device.type, index, int(stream))


def get_workspace(device: torch.device, nbytes: int, stream: Optional[int] = None) -> torch.Tensor:
    """Scratch memory for split-K partials, ticket counters and regrouped block scales.

    Keyed by the device and the raw handle of the stream the launch goes to (the current stream when
    ``stream`` is None): kernels on one stream run in order and may share scratch, kernels on
    different streams may overlap and must not, so each stream that launches a matmul needing
    scratch gets a buffer of its own.

    While a graph is being captured nothing can be allocated or zero-filled (the fill would become a
    node of the graph).  A capture stream that has no buffer of its own (torch.cuda.graph captures
    on an internal stream) therefore takes the buffer of the stream this thread last launched on
    outside a capture - the stream the layer was warmed up on, and normally the one that replays the
    graph, so the two stay ordered.  A graph replayed on another stream while that stream is busy
    with matmuls would race with them; capture on an explicit, warmed-up stream in that case.  If no
    buffer is large enough the capture is refused: run the layer once at this shape first.

    Growing replaces the buffer (at least doubling, so the outgrown ones add up to less than the
    live one) and never frees the old one: a captured graph may still point at it.
    """
    if stream is None:
        stream = _stream_ptr(device)
    key = _workspace_key(device, stream)
    capturing = torch.cuda.is_current_stream_capturing()
    owner = (threading.get_ident(), key[1])
    if not capturing:
        _last_eager_key[owner] = key
    ws = _workspaces.get(key)
    if ws is not None and ws.numel() >= nbytes:
        return ws
    if capturing:
        fallback = _workspaces.get(_last_eager_key.get(owner))
        if fallback is not None and fallback.numel() >= nbytes:
            return fallback
        raise RuntimeError(
            f"gemlite_amd: a workspace of {int(nbytes)} bytes is needed while a graph is being captured and none "
            "that large exists yet; run the layer once at this shape before capturing"
        )
    with _workspace_lock:
        ws = _workspaces.get(key)
        if ws is None or ws.numel() < nbytes:
            size = max(int(nbytes), 8 << 20, 0 if ws is None else 2 * ws.numel())
            if ws is not None:
                _retired_workspaces.append(ws)
            ws = _new_workspace(size, device)
            _workspaces[key] = ws
    return ws


def _new_workspace(size: int, device: torch.device) -> torch.Tensor:
    return torch.zeros(size, dtype=torch.uint8, device=device)


def _dt(t: Optional[torch.Tensor], default: int = 0) -> int:
    if t is None:
        return default
    return TORCH_TO_DTYPE[t.dtype].value


def build_matmul_args(
    x, W_q, scales, zeros, scales_x, out, *,
    W_nbits, group_size, unpack_mask, elements_per_sample, input_dtype, output_dtype, acc_dtype, meta_dtype,
    channel_scale_mode, W_group_mode, data_contiguous, matmul_type=MATMUL_AUTO, tile_config=-1, bias=None,
    x_quant_from=0,
) -> MatmulArgs:
    """Fill a ``gla_matmul_args`` from tensors and the reference's meta ints.  ``x_quant_from``: the DType value of
    the 16-bit rows in ``x`` when the kernel is to quantise them to ``input_dtype`` itself (``scales_x`` is then None)."""
    a = MatmulArgs()
    a.struct_size = ctypes.sizeof(MatmulArgs)
    a.matmul_type = int(matmul_type)
    M = x.shape[0]
    N = W_q.shape[1]
    K = W_q.shape[0] * elements_per_sample
    a.M, a.N, a.K = int(M), int(N), int(K)
    a.x = x.data_ptr()
    a.w = W_q.data_ptr()
    has_scales = scales is not None and scales.numel() > 0
    has_zeros = zeros is not None and zeros.numel() > 0
    a.scales = scales.data_ptr() if has_scales else None
    a.zeros = zeros.data_ptr() if has_zeros else None
    a.scales_x = scales_x.data_ptr() if scales_x is not None else None
    a.out = out.data_ptr()
    a.x_stride_m, a.x_stride_k = x.stride(0), x.stride(1)
    a.w_stride_k, a.w_stride_n = W_q.stride(0), W_q.stride(1)
    a.out_stride_m, a.out_stride_n = out.stride(0), out.stride(1)
    mx = is_mx_dtype(int(input_dtype))
    if has_scales and scales.dim() == 2:
        if mx:  # micro-scaled formats hand the scales over as the [N, K/group] view
            a.meta_stride_n, a.meta_stride_g = scales.stride(0), scales.stride(1)
        else:   # [K/group, N]
            a.meta_stride_g, a.meta_stride_n = scales.stride(0), scales.stride(1)
    elif has_zeros and zeros.dim() == 2:
        a.meta_stride_g, a.meta_stride_n = zeros.stride(0), zeros.stride(1)
    else:
        a.meta_stride_g, a.meta_stride_n = N, 1
    if scales_x is not None and scales_x.dim() == 2:
        a.sx_stride_m, a.sx_stride_g = scales_x.stride(0), scales_x.stride(1)
    else:
        a.sx_stride_m, a.sx_stride_g = 1, 1
    a.W_nbits = int(W_nbits)
    a.group_size = int(group_size)
    a.unpack_mask = int(unpack_mask)
    a.elements_per_sample = int(elements_per_sample)
    a.input_dtype = int(input_dtype)
    a.output_dtype = int(output_dtype)
    a.acc_dtype = int(acc_dtype)
    a.meta_dtype = _dt(scales, int(meta_dtype)) if has_scales else int(meta_dtype)
    a.channel_scale_mode = int(channel_scale_mode)
    a.W_group_mode = int(W_group_mode)
    a.data_contiguous = int(bool(data_contiguous))
    a.w_dtype = _dt(W_q)
    a.zeros_dtype = _dt(zeros, DType.INT32.value) if has_zeros else DType.INT32.value
    a.zero_is_scalar = int(has_zeros and zeros.numel() == 1)
    a.sx_dtype = _dt(scales_x, DType.FP32.value)
    a.tile_config = int(tile_config)
    a.x_quant_from = int(x_quant_from)
    if bias is not None:
        if bias.numel() < N or bias.stride(-1) != 1:
            raise ValueError(f"bias: need {N} contiguous elements, got shape {tuple(bias.shape)} strides {bias.stride()}")
        a.bias = bias.data_ptr()
        a.bias_dtype = _dt(bias)
    else:
        a.bias = None
        a.bias_dtype = 0
    _check_operand_bounds(a, x, W_q, scales if has_scales else None, zeros if has_zeros else None, scales_x, out, mx)
    return a


def _span(t: torch.Tensor) -> int:
    """Elements addressable from the tensor's first element to the end of its storage."""
    return t.untyped_storage().nbytes() // t.element_size() - t.storage_offset()


def _check_operand_bounds(a, x, W_q, scales, zeros, scales_x, out, mx):
    """The kernels trust strides: refuse any operand whose last addressed element would fall
    outside the memory its tensor owns."""
    def need(*terms):
        return 1 + sum((n - 1) * abs(s) for n, s in terms if n > 0)

    def check(name, t, required):
        if t is not None and required > _span(t):
            raise ValueError(
                f"{name}: kernel would address {required} elements but the tensor spans {_span(t)} "
                f"(shape {tuple(t.shape)}, strides {t.stride()})"
            )

    M, N, K, e = a.M, a.N, a.K, a.elements_per_sample
    kx = K // 2 if (a.input_dtype == DType.MXFP4.value and not a.x_quant_from) else K
    check("x", x, need((M, a.x_stride_m), (kx, a.x_stride_k)))
    check("W_q", W_q, need((K // e, a.w_stride_k), (N, a.w_stride_n)))
    check("out", out, need((M, a.out_stride_m), (N, a.out_stride_n)))
    wgm, csm = a.W_group_mode, a.channel_scale_mode
    groups = K // 32 if mx else (K // a.group_size if a.group_size > 0 else 1)
    if csm == 5:  # 128 x 128 weight blocks, (row, 128) activation blocks
        kb, nb = (K + 127) // 128, (N + 127) // 128
        if scales is not None:
            check("scales", scales, need((kb, a.meta_stride_g), (nb, a.meta_stride_n)))
        if scales_x is not None:
            check("scales_x", scales_x, need((M, a.sx_stride_m), (kb, a.sx_stride_g)))
        return
    if scales is not None:
        if mx or wgm >= 2:
            check("scales", scales, need((groups, a.meta_stride_g), (N, a.meta_stride_n)))
        if csm in (1, 3):
            check("scales", scales, N)
    if zeros is not None and not a.zero_is_scalar and wgm in (1, 3, 4):
        check("zeros", zeros, need((groups, a.meta_stride_g), (N, a.meta_stride_n)))
    if scales_x is not None:
        if csm == 4:
            check("scales_x", scales_x, need((M, a.sx_stride_m), (K // 32, a.sx_stride_g)))
        elif csm in (2, 3):
            check("scales_x", scales_x, need((M, a.sx_stride_m)))


def matmul(args: MatmulArgs, device: torch.device):
    """Launch ``gla_matmul`` on the current stream of ``device``; attaches workspace if needed."""
    lib = load_library()
    need = lib.gla_matmul_workspace_bytes(ctypes.byref(args))
    if need < 0:
        _check(int(need), "gla_matmul_workspace_bytes")
    stream = _stream_ptr(device)
    if need > 0:
        ws = get_workspace(device, need, stream)
        args.workspace = ws.data_ptr()
        args.workspace_bytes = ws.numel()
    _check(lib.gla_matmul(ctypes.byref(args), stream), "gla_matmul")


def matmul_prepared(args: MatmulArgs, need: int, x_ptr: int, out_ptr: int, sx_ptr, device: torch.device):
    """Launch a ``gla_matmul_args`` that ``build_matmul_args`` filled and checked before, for the
    same shapes, strides and weight tensors: only the activation, output and activation-scale
    addresses (and the workspace, which may have grown) are refreshed.  ``need`` is what
    ``gla_matmul_workspace_bytes`` returned for it."""
    args.x = x_ptr
    args.out = out_ptr
    args.scales_x = sx_ptr
    stream = _stream_ptr(device)
    if need > 0:
        ws = get_workspace(device, need, stream)
        args.workspace = ws.data_ptr()
        args.workspace_bytes = ws.numel()
    status = load_library().gla_matmul(ctypes.byref(args), stream)
    if status != GLA_OK:
        _check(status, "gla_matmul")


def matmul_workspace_need(args: MatmulArgs) -> int:
    need = load_library().gla_matmul_workspace_bytes(ctypes.byref(args))
    if need < 0:
        _check(int(need), "gla_matmul_workspace_bytes")
    return int(need)


def matmul_is_supported(args: MatmulArgs) -> bool:
    """Whether the library has a kernel for ``args`` as they are (host logic only; no exception, no launch)."""
    return load_library().gla_matmul_family(ctypes.byref(args)) >= 0


FAMILIES = ["GENERIC", "GEMV_PACKED", "GEMV_KMAJOR", "GEMM_WN", "GEMM_8BIT", "GEMM_MXFP4", "GEMM_KBYTES", "GEMM_MXFP8", "MX_STREAM", "BLOCKQ_STREAM", "GEMM_BLOCKQ", "GEMM_KBYTES_MX", "MX_SKINNY", "K_SKINNY", "WN_MID", "GEMM_16BIT"]


def matmul_family(args: MatmulArgs) -> str:
    """Name of the kernel family ``gla_matmul`` would run for ``args`` (host logic only)."""
    f = load_library().gla_matmul_family(ctypes.byref(args))
    if f < 0:
        _check(f, "gla_matmul_family")
    return FAMILIES[f]


def select_config(args: MatmulArgs) -> int:
    return load_library().gla_select_config(ctypes.byref(args))


# ---------------------------------------------------------------------------
# activation quantisation and bit packing
# ---------------------------------------------------------------------------
def scale_activations_per_token(x2d: torch.Tensor, y: torch.Tensor, scales: torch.Tensor):
    _require_cuda(x2d, y, scales)
    lib = load_library()
    M, K = x2d.shape
    _check(
        lib.gla_scale_activations_per_token(
            x2d.data_ptr(), _dt(x2d), x2d.stride(0), M, K, y.data_ptr(), _dt(y), scales.data_ptr(),
            _stream_ptr(x2d.device),
        ),
        "gla_scale_activations_per_token",
    )


def scale_activations_per_block(x2d: torch.Tensor, y: torch.Tensor, scales: torch.Tensor):
    _require_cuda(x2d, y, scales)
    lib = load_library()
    M, K = x2d.shape
    _check(
        lib.gla_scale_activations_per_block(
            x2d.data_ptr(), _dt(x2d), x2d.stride(0), M, K, y.data_ptr(), _dt(y), scales.data_ptr(),
            _stream_ptr(x2d.device),
        ),
        "gla_scale_activations_per_block",
    )


def scale_activations_mxfp4(x2d: torch.Tensor, y: torch.Tensor, scales: torch.Tensor):
    _require_cuda(x2d, y, scales)
    lib = load_library()
    M, K = x2d.shape
    _check(
        lib.gla_scale_activations_mxfp4(
            x2d.data_ptr(), _dt(x2d), x2d.stride(0), M, K, y.data_ptr(), scales.data_ptr(), _stream_ptr(x2d.device)
        ),
        "gla_scale_activations_mxfp4",
    )


def scale_activations_mxfp8(x2d: torch.Tensor, y: torch.Tensor, scales: torch.Tensor):
    _require_cuda(x2d, y, scales)
    lib = load_library()
    M, K = x2d.shape
    _check(
        lib.gla_scale_activations_mxfp8(
            x2d.data_ptr(), _dt(x2d), x2d.stride(0), M, K, y.data_ptr(), scales.data_ptr(), _stream_ptr(x2d.device)
        ),
        "gla_scale_activations_mxfp8",
    )


def pack_over_cols(codes: torch.Tensor, out: torch.Tensor, rows: int, cols: int, W_nbits: int, width: int):
    _require_cuda(codes, out)
    lib = load_library()
    _check(
        lib.gla_pack_over_cols(codes.data_ptr(), out.data_ptr(), rows, cols, W_nbits, width, _stream_ptr(codes.device)),
        "gla_pack_over_cols",
    )


def unpack_over_cols(packed: torch.Tensor, out: torch.Tensor, rows: int, pcols: int, W_nbits: int, width: int):
    _require_cuda(packed, out)
    lib = load_library()
    _check(
        lib.gla_unpack_over_cols(
            packed.data_ptr(), out.data_ptr(), rows, pcols, W_nbits, width, _stream_ptr(packed.device)
        ),
        "gla_unpack_over_cols",
    )
