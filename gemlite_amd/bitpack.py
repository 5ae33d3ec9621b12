"""Bit-packing of low-bit weight codes into machine words.

Layout contract (reference: gemlite/bitpack.py:36-60 for packing,
gemlite/bitpack.py:146-162 for unpacking): with ``e = packing_bitwidth //
W_nbits`` codes per word, code ``j`` of a row lands in word ``j // e`` at bit
offset ``(j % e) * W_nbits``.  Words use the signed storage types of
``PACKING_BITWIDTH_TO_TORCH_DTYPE`` (uint8 for 8-bit words), so a code in the
top slot may set the sign bit.

On a GPU tensor the packing runs as a HIP kernel through the C ABI
(``gla_pack_over_cols``); on a CPU tensor it runs as vectorised torch integer
arithmetic.  Both produce identical bits.
"""
from typing import Tuple

import torch

from .dtypes import PACKING_BITWIDTH_TO_TORCH_DTYPE

_VALID_WIDTHS = (8, 16, 32, 64)
_VALID_NBITS = (8, 4, 2, 1)


def _check(W_nbits: int, packing_bitwidth: int) -> int:
    if packing_bitwidth not in _VALID_WIDTHS:
        raise AssertionError("Unsuported bitpacking width")
    if W_nbits not in _VALID_NBITS:
        raise AssertionError("Unsuported nbits")
    return packing_bitwidth // W_nbits


def _to_storage(words64: torch.Tensor, packing_bitwidth: int) -> torch.Tensor:
    """Reinterpret the low ``packing_bitwidth`` bits of int64 words as the storage type."""
    dtype = PACKING_BITWIDTH_TO_TORCH_DTYPE[packing_bitwidth]
    if packing_bitwidth == 64:
        return words64
    if packing_bitwidth == 8:
        return words64.to(torch.uint8)
    # Two's-complement wrap into the signed storage type.
    half = 1 << (packing_bitwidth - 1)
    wrapped = ((words64 + half) % (1 << packing_bitwidth)) - half
    return wrapped.to(dtype)


def pack_weights_over_cols_torch(
    W_q: torch.Tensor, W_nbits: int, packing_bitwidth: int, transpose: bool
) -> Tuple[torch.Tensor, int]:
    """Pack along the column (K) axis of a ``[rows, cols]`` code matrix.

    Returns ``([rows, cols // e] words, e)``; with ``transpose`` the result is
    the ``[cols // e, rows]`` transposed *view* (reference:
    gemlite/bitpack.py:36-60).
    """
    e = _check(W_nbits, packing_bitwidth)
    rows, cols = W_q.shape
    if cols % e != 0:
        raise ValueError(f"number of columns ({cols}) must be divisible by {e}")
    codes = W_q.to(torch.int64).reshape(rows, cols // e, e)
    shifts = torch.arange(e, dtype=torch.int64, device=W_q.device) * W_nbits
    if packing_bitwidth == 64:
        # Avoid overflow in the sum: OR the slots together one at a time.
        words = torch.zeros((rows, cols // e), dtype=torch.int64, device=W_q.device)
        for slot in range(e):
            words |= codes[:, :, slot] << (W_nbits * slot)
    else:
        words = (codes << shifts).sum(dim=-1)
    out = _to_storage(words, packing_bitwidth)
    if transpose:
        out = out.t()
    return out, e


def pack_weights_over_rows_torch(
    W_q: torch.Tensor, W_nbits: int, packing_bitwidth: int, transpose: bool
) -> Tuple[torch.Tensor, int]:
    """Pack along the row axis (reference: gemlite/bitpack.py:10-34)."""
    out, e = pack_weights_over_cols_torch(W_q.t(), W_nbits, packing_bitwidth, transpose=False)
    out = out.t()
    if transpose:
        out = out.t()
    return out, e


def unpack_over_cols_torch(
    W_q_packed: torch.Tensor,
    W_nbits: int,
    num_output_cols: int,
    dtype: torch.dtype = torch.uint8,
) -> torch.Tensor:
    """Inverse of :func:`pack_weights_over_cols_torch` (before the transpose)
    (reference: gemlite/bitpack.py:146-162)."""
    rows, cols = W_q_packed.shape
    e = num_output_cols // cols
    mask = (1 << W_nbits) - 1
    shifts = torch.arange(e, dtype=torch.int64, device=W_q_packed.device) * W_nbits
    words = W_q_packed.to(torch.int64)
    codes = (words.unsqueeze(-1) >> shifts) & mask  # arithmetic shift then mask
    return codes.to(dtype).reshape(rows, num_output_cols)


def unpack_over_rows_torch(
    W_q_packed: torch.Tensor,
    W_nbits: int,
    num_output_rows: int,
    dtype: torch.dtype = torch.uint8,
) -> torch.Tensor:
    """Inverse of :func:`pack_weights_over_rows_torch` (reference:
    gemlite/bitpack.py:207-224)."""
    return unpack_over_cols_torch(W_q_packed.t(), W_nbits, num_output_rows, dtype).t()


def pack_weights_over_cols_hip(
    W_q: torch.Tensor, W_nbits: int, packing_bitwidth: int, transpose: bool
) -> Tuple[torch.Tensor, int]:
    """GPU packing through the C ABI; same contract as the torch version
    (takes the place of the reference's Triton launcher, gemlite/bitpack.py:112-144)."""
    from . import _ext

    e = _check(W_nbits, packing_bitwidth)
    rows, cols = W_q.shape
    if cols % e != 0:
        raise ValueError(f"number of columns ({cols}) must be divisible by {e}")
    src = W_q.contiguous()
    if src.dtype != torch.uint8:
        src = src.to(torch.uint8)
    out = torch.empty(
        (rows, cols // e), dtype=PACKING_BITWIDTH_TO_TORCH_DTYPE[packing_bitwidth], device=W_q.device
    )
    _ext.pack_over_cols(src, out, rows, cols, W_nbits, packing_bitwidth)
    if transpose:
        out = out.t()
    return out, e


def unpack_over_cols_hip(
    W_q_packed: torch.Tensor, W_nbits: int, num_output_cols: int, dtype: torch.dtype = torch.uint8
) -> torch.Tensor:
    """GPU unpacking through the C ABI (takes the place of gemlite/bitpack.py:164-205)."""
    from . import _ext

    rows, cols = W_q_packed.shape
    src = W_q_packed.contiguous()
    out = torch.empty((rows, num_output_cols), dtype=torch.uint8, device=src.device)
    _ext.unpack_over_cols(src, out, rows, cols, W_nbits, src.element_size() * 8)
    return out if dtype == torch.uint8 else out.to(dtype)


def pack_weights_over_cols(W_q, W_nbits, packing_bitwidth, transpose):
    """Device dispatch used by ``GemLiteLinear.pack`` (reference: gemlite/core.py:624)."""
    if W_q.device.type == "cuda":
        return pack_weights_over_cols_hip(W_q, W_nbits, packing_bitwidth, transpose)
    return pack_weights_over_cols_torch(W_q, W_nbits, packing_bitwidth, transpose)


def unpack_over_cols(W_q_packed, W_nbits, num_output_cols, dtype=torch.uint8):
    if W_q_packed.device.type == "cuda":
        return unpack_over_cols_hip(W_q_packed, W_nbits, num_output_cols, dtype)
    return unpack_over_cols_torch(W_q_packed, W_nbits, num_output_cols, dtype)


# Names kept for callers of the reference package.
pack_weights_over_cols_triton = pack_weights_over_cols
unpack_over_cols_triton = unpack_over_cols

__all__ = [
    "pack_weights_over_cols",
    "pack_weights_over_cols_torch",
    "pack_weights_over_cols_hip",
    "pack_weights_over_cols_triton",
    "pack_weights_over_rows_torch",
    "unpack_over_cols",
    "unpack_over_cols_torch",
    "unpack_over_cols_hip",
    "unpack_over_cols_triton",
    "unpack_over_rows_torch",
]
