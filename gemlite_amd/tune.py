"""Offline tile tuner: fills the dispatcher's config cache for given layers and batch sizes.

The reference finds tile configurations by Triton autotuning on first use and can save them with
``GemLiteLinear.cache_config`` (reference: gemlite/core.py:838-906, gemlite/helper.py:1326-1376).
Here kernels derive their geometry from the shape in closed form; this tuner times the few
alternatives each kernel family accepts (``tile_config``) and records a winner only where it
beats the built-in choice.  Entries live under the reference's cache key, so ``cache_config`` /
``load_config`` files keep their format: ``{matmul_type: {key: {"tile_config": id, "us": t}}}``.
"""
import ctypes
from typing import Iterable, List, Optional

import torch

from . import _ext
from .core import (
    GEMLITE_CONFIG_CACHE,
    GEMLITE_MATMUL_TYPES_MAPPING,
    GemLiteLinear,
    config_key,
    get_matmul_type,
    get_type_id,
)
from .dtypes import DTYPE_TO_TORCH, DType, is_mx_dtype
from .quant_utils import (scale_activations_mxfp4, scale_activations_mxfp8, scale_activations_per_block,
                          scale_activations_per_token)


PREFER_STREAMING, PREFER_MATRIX, PREFER_MID, PREFER_UNPACKED = -2, -3, -4, -5   # GLA_TILE_PREFER_* of the C header
HAND_OFF_ROWS = 128                        # batch sizes up to which both kinds of kernel are timed


def candidate_configs(family: str, M: int, K: int) -> List[int]:
    """``tile_config`` ids worth timing for a kernel family (-1, the built-in heuristic, comes first)."""
    if family == "GEMV_PACKED":      # waves per workgroup * 1000 + batches of loads per wave
        return [-1, 4001, 8001, 16001, 4002, 4004]
    if family == "GEMM_WN":          # BM + 1000 * K splits
        bms = [32, 64] if M <= 32 else ([64, 128] if M <= 128 else [128, 256])
        splits = [1, 2, 4, 8, 16] if M <= 256 else [1, 2]
        return [-1] + [bm + 1000 * s for bm in bms for s in splits if s <= max(1, K // 512)]
    if family == "WN_MID":           # waves per workgroup + 1000 * K splits
        return [-1] + [nw + 1000 * s for nw in (4, 8) for s in (2, 4, 8, 16) if s <= max(1, K // 512)]
    if family in ("GEMM_KBYTES", "GEMM_KBYTES_MX"):      # BM + 1000 * K splits
        bms = [64] if M <= 64 else ([64, 128] if M <= 128 else [128, 256])
        splits = [1, 2, 4, 8, 16] if M <= 256 else [1, 2]
        return [-1] + [bm + 1000 * s for bm in bms for s in splits if s <= max(1, K // 512)]
    if family in ("GEMM_8BIT", "GEMM_MXFP4", "GEMM_MXFP8", "GEMM_16BIT"):
        bms = [64] if M <= 64 else ([64, 128] if M <= 128 else [128, 256])
        splits = [1, 2, 4, 8, 16] if M <= 256 else [1, 2]
        return [-1] + [bm + 1000 * s for bm in bms for s in splits if s <= max(1, K // 1024)]
    if family == "GEMM_BLOCKQ":      # the second accumulator rules out the 256-row tile
        bms = [64] if M <= 64 else [64, 128]
        splits = [1, 2, 4, 8, 16] if M <= 256 else [1, 2]
        return [-1] + [bm + 1000 * s for bm in bms for s in splits if s <= max(1, K // 1024)]
    return [-1]


def _prepare_inputs(layer: GemLiteLinear, M: int, device):
    """Synthetic activations of the type the layer's kernels see (quantised on the fly where the layer does)."""
    g = torch.Generator(device="cpu").manual_seed(M)
    in_dt = DType(layer.input_dtype)
    if layer.scaled_activations:
        x = torch.randn((M, layer.in_features), generator=g).to(torch.bfloat16).to(device)
        if in_dt == DType.MXFP4:
            return scale_activations_mxfp4(x)
        if in_dt == DType.MXFP8:
            if layer.channel_scale_mode == 4:
                return scale_activations_mxfp8(x)
            return scale_activations_per_token(x, w_dtype=torch.float8_e4m3fn)
        if layer.channel_scale_mode == 5:
            return scale_activations_per_block(x, w_dtype=DTYPE_TO_TORCH[in_dt.value])
        return scale_activations_per_token(x, w_dtype=DTYPE_TO_TORCH[in_dt.value])
    if layer.compute_dtype == torch.int8:
        return torch.randint(-128, 128, (M, layer.in_features), generator=g, dtype=torch.int32).to(torch.int8).to(device), None
    dt = layer.compute_dtype if layer.compute_dtype in (torch.float16, torch.bfloat16, torch.float32) else torch.bfloat16
    return torch.randn((M, layer.in_features), generator=g).to(dt).to(device), None


def tune_layer(layer: GemLiteLinear, batch_sizes: Iterable[int], reps: int = 20, min_gain: float = 0.03,
               verbose: bool = False) -> dict:
    """Time every candidate tile of ``layer`` at each batch size on its device and store the
    winners in ``GEMLITE_CONFIG_CACHE``.  Returns ``{M: (tile_config, microseconds, family)}``."""
    device = layer.W_q.device
    if device.type != "cuda":
        raise RuntimeError("tuning runs on the GPU the layer lives on")
    lib = _ext.load_library()
    m = layer.get_meta_args()
    results = {}
    for M in batch_sizes:
        x, scales_x = _prepare_inputs(layer, M, device)
        out = torch.empty((M, layer.out_features), dtype=DTYPE_TO_TORCH[m[6]], device=device)
        input_dtype = m[5]
        if not layer.scaled_activations and not is_mx_dtype(input_dtype):
            input_dtype = _ext_dtype_of(x)
        matmul_type = get_matmul_type(M, m[1], is_mx_dtype(m[5]))

        def build(tile):
            return _ext.build_matmul_args(
                x, layer.W_q, layer.scales, layer.zeros, scales_x, out, W_nbits=m[1], group_size=m[2],
                unpack_mask=m[3], elements_per_sample=m[4], input_dtype=input_dtype, output_dtype=m[6],
                acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                data_contiguous=m[11], matmul_type=GEMLITE_MATMUL_TYPES_MAPPING[matmul_type], tile_config=tile)

        family = _ext.matmul_family(build(-1))
        stream = torch.cuda.current_stream(device).cuda_stream
        runnable = []
        candidates = candidate_configs(family, M, layer.in_features)
        if M <= HAND_OFF_ROWS:
            # around the hand-off between the streaming kernels and the matrix-core GEMMs the other side is timed too;
            # the library's thresholds there were fitted on one machine
            candidates += [t for t in (PREFER_STREAMING, PREFER_MATRIX, PREFER_MID) if _ext.matmul_family(build(t)) != family]
        if M >= 512 and family in ("GEMM_WN", "GEMM_16BIT"):
            # prefill of packed layers: the fused kernel against weight unpacking + the 16-bit GEMM
            candidates += [t for t in (PREFER_MATRIX, PREFER_UNPACKED) if _ext.matmul_family(build(t)) != family]
        for tile in candidates:
            args = build(tile)
            need = lib.gla_matmul_workspace_bytes(ctypes.byref(args))
            if need < 0:
                continue  # this tile does not fit the shape
            if need > 0:
                ws = _ext.get_workspace(device, need)
                args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel()
            if lib.gla_matmul(ctypes.byref(args), stream) != 0:
                continue
            runnable.append((tile, args))
        torch.cuda.synchronize(device)
        best_of = {}
        for _ in range(2):  # two rounds over all candidates, best of both: the first timings of a run are slower
            for tile, args in runnable:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _r in range(reps):
                    lib.gla_matmul(ctypes.byref(args), stream)
                e1.record()
                torch.cuda.synchronize(device)
                us = e0.elapsed_time(e1) * 1e3 / reps
                best_of[tile] = min(us, best_of.get(tile, us))
        timings = [(us, tile) for tile, us in best_of.items()]
        if verbose:
            for us, tile in timings:
                print(f"  M={M} {family} tile={tile}: {us:.1f} us")
        if not timings:
            continue
        base = next((t for t, tile in timings if tile == -1), None)
        best_us, best_tile = min(timings)
        if base is not None and best_us > base * (1.0 - min_gain):
            best_us, best_tile = base, -1  # not clearly better than the built-in choice
        results[M] = (best_tile, best_us, family)
        if best_tile != -1:
            key = config_key(M, layer.out_features, layer.in_features, m[2], m[4], get_type_id(m[5], m[1]))
            GEMLITE_CONFIG_CACHE.setdefault(matmul_type, {})[key] = {"tile_config": int(best_tile), "us": round(best_us, 2)}
    return results


def _ext_dtype_of(x: torch.Tensor) -> int:
    from .dtypes import TORCH_TO_DTYPE
    return TORCH_TO_DTYPE[x.dtype].value


def tune_model(model: torch.nn.Module, batch_sizes: Iterable[int], filename: Optional[str] = None, **kw) -> dict:
    """Tune every ``GemLiteLinear`` in ``model`` (one representative per distinct shape / format)
    and optionally write the cache file."""
    seen, report = set(), {}
    for name, mod in model.named_modules():
        if not isinstance(mod, GemLiteLinear):
            continue
        sig = (mod.in_features, mod.out_features, mod.W_nbits, mod.group_size, int(mod.input_dtype), mod.W_group_mode,
               mod.channel_scale_mode)
        if sig in seen:
            continue
        seen.add(sig)
        report[name] = tune_layer(mod, batch_sizes, **kw)
    if filename is not None:
        GemLiteLinear.cache_config(filename)
    return report
