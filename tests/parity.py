"""Shared helpers of the parity tests: build seeded cases, run the oracle on the tensors a
packed layer holds, and compare."""
import numpy as np
import torch

from gemlite_amd import DType, GemLiteLinear
from gemlite_amd.dtypes import DTYPE_TO_TORCH
from oracle import oracle as orc

FROB_TOL = 1e-2  # max relative Frobenius error allowed for float outputs


def to_np(t):
    """Tensor -> float32 / integer numpy array on the CPU (bf16/fp16/fp8 widened exactly)."""
    t = t.detach().cpu()
    if t.dtype in (torch.bfloat16, torch.float16, torch.float8_e4m3fn):
        return t.float().numpy()
    return t.numpy()


def rel_frob(y, y_ref):
    y = np.asarray(y, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    denom = np.linalg.norm(y_ref)
    return float(np.linalg.norm(y - y_ref) / (denom if denom > 0 else 1.0))


# Elementwise bound next to the global norm: |y - y_ref| <= atol_rms * rms(y_ref) + rtol * |y_ref|.
# A correct kernel's error is output rounding (half an ulp: 2^-9 bf16, 2^-12 fp16, relative to the
# element) plus fp32 accumulation noise and, where weights are dequantised to 16 bits before the MFMA,
# their rounding (a few 1e-4 of the rms in fp16, 2e-3 in bf16).  A wrong tail column, row tile or MFMA
# tile is off by about the rms itself and fails this whatever its share of the whole norm.
ELEMENTWISE = {"bf16": (2.5e-2, 2.0 ** -7), "fp16": (5e-3, 2.0 ** -10), "fp32": (1e-3, 1e-4)}


def elementwise_excess(y, y_ref, kind):
    """Largest |y - y_ref| / (atol_rms * rms + rtol * |y_ref|); <= 1 passes."""
    atol_rms, rtol = ELEMENTWISE[kind]
    y = np.asarray(y, dtype=np.float64)
    y_ref = np.asarray(y_ref, dtype=np.float64)
    if y_ref.size == 0:
        return 0.0
    rms = float(np.sqrt(np.mean(y_ref * y_ref)))
    bound = atol_rms * (rms if rms > 0 else 1.0) + rtol * np.abs(y_ref)
    return float(np.max(np.abs(y - y_ref) / bound))


def kind_of(dtype):
    return {torch.bfloat16: "bf16", torch.float16: "fp16", torch.float32: "fp32"}[dtype]


def gen_int_case(N, K, W_nbits, group_size, dtype, seed=0, scale_std=0.02, channelwise=False):
    """Seeded weights in the distributions of the benchmark configs: codes uniform over the
    bit range, scales |N(0, std)|, zeros uniform over the middle of the range."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    W_q = torch.randint(0, 2 ** W_nbits, (N, K), generator=g, dtype=torch.int32).to(torch.uint8)
    groups = N if channelwise else N * K // group_size
    scales = (torch.randn((groups, 1), generator=g) * scale_std).abs().clamp_(min=1e-4).to(dtype)
    lo, hi = (2 ** W_nbits) * 3 / 8, (2 ** W_nbits) * 9 / 16
    zeros = (torch.rand((groups, 1), generator=g) * (hi - lo) + lo).to(dtype)
    return W_q, scales, zeros


def gen_x(M, K, dtype, seed=1, std=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return (torch.randn((M, K), generator=g) * std).to(dtype)


def layer_codes_kn(layer):
    """[K, N] integer codes (or float weights) held by a packed layer, via the oracle's unpack."""
    W = layer.W_q.detach().cpu()
    e = layer.elements_per_sample
    if e == 1:
        return to_np(W)  # [K, N] view of the [N, K] tensor
    packed_nk = W.t().contiguous().numpy()  # [N, K/e]
    K = packed_nk.shape[1] * e
    return orc.unpack_over_cols(packed_nk, layer.W_nbits, K).T.copy()


def oracle_forward(layer, x, matmul_x=None, scales_x=None):
    """What forward(x) must return, computed by the oracle from the tensors the layer holds.
    `matmul_x` / `scales_x` override the activation operand (already quantised codes)."""
    wgm, csm = layer.W_group_mode, layer.channel_scale_mode
    in_dt = layer.input_dtype
    xin = to_np(x).reshape(-1, x.shape[-1])
    if csm == 5:   # 128 x 128 block-quantised int8 / fp8
        to_int8 = in_dt == DType.INT8
        if matmul_x is None:
            matmul_x, scales_x = orc.scale_activations_per_block(xin, to_int8)
        Wb = layer.W_q.detach().cpu().t().contiguous()            # [N, K]
        b = Wb.numpy() if to_int8 else orc.e4m3fn_decode(Wb.view(torch.uint8).numpy())
        a = matmul_x if to_int8 else orc.e4m3fn_decode(matmul_x)
        out = orc.matmul_block_quant(a, scales_x, b, to_np(layer.scales).T)
    elif in_dt in (DType.MXFP16, DType.MXBF16):   # weight-only MX: activations as they are, unit scales
        sb = layer.scales.detach().cpu().contiguous().numpy()        # [N, K/32]
        if layer.elements_per_sample == 2:
            b, kind = orc.unpack_fp4_bytes(layer.W_q.detach().cpu().t().contiguous().numpy()), "e2m1"
        else:
            b, kind = layer.W_q.detach().cpu().t().contiguous().view(torch.uint8).numpy(), "e4m3"
        out = orc.matmul_mx_mixed(xin, "float", None, b, kind, sb)
    elif in_dt == DType.MXFP8 and layer.elements_per_sample == 2:   # fp8 activations x MXFP4 weights
        b = orc.unpack_fp4_bytes(layer.W_q.detach().cpu().t().contiguous().numpy())
        sb = layer.scales.detach().cpu().contiguous().numpy()
        if csm == 2:
            if matmul_x is None:
                matmul_x, scales_x = orc.scale_activations_per_token(xin, False)
            out = orc.matmul_mx_mixed(matmul_x, "e4m3", None, b, "e2m1", sb, scales_x=scales_x)
        else:
            if matmul_x is None:
                matmul_x, scales_x = orc.scale_activations_mxfp8(xin)
            out = orc.matmul_mx_mixed(matmul_x, "e4m3", scales_x[: matmul_x.shape[0]], b, "e2m1", sb)
    elif in_dt == DType.MXFP4:
        if matmul_x is None:
            matmul_x, scales_x = orc.scale_activations_mxfp4(xin)
        a_codes = orc.unpack_fp4_bytes(matmul_x)
        Wb = layer.W_q.detach().cpu().t().contiguous().numpy()      # [N, K/2] bytes
        b_codes = orc.unpack_fp4_bytes(Wb)
        sb = layer.scales.detach().cpu().contiguous().numpy()        # [N, K/32]
        out = orc.matmul_mx(a_codes, scales_x[: a_codes.shape[0]], b_codes, sb)
    elif in_dt == DType.MXFP8:
        Wb = layer.W_q.detach().cpu().t().contiguous().view(torch.uint8).numpy()   # [N, K] e4m3fn bytes
        sb = layer.scales.detach().cpu().contiguous().numpy()                        # [N, K/32] e8m0 bytes
        if csm == 2:   # per-token activations, scale applied after the K sum
            if matmul_x is None:
                matmul_x, scales_x = orc.scale_activations_per_token(xin, False)
            out = orc.matmul_mxfp8_weights(orc.e4m3fn_decode(matmul_x), scales_x, Wb, sb)
        else:          # micro-scales on both sides
            if matmul_x is None:
                matmul_x, scales_x = orc.scale_activations_mxfp8(xin)
            out = orc.matmul_mxfp8(matmul_x, scales_x[: matmul_x.shape[0]], Wb, sb)
    else:
        if layer.scaled_activations:
            if matmul_x is None:
                matmul_x, scales_x = orc.scale_activations_per_token(xin, in_dt == DType.INT8)
            a = matmul_x if in_dt == DType.INT8 else orc.e4m3fn_decode(matmul_x)
        else:
            a = xin
        q_kn = layer_codes_kn(layer)
        has_s = layer.scales.numel() > 0
        has_z = layer.zeros.numel() > 0
        s_gn = to_np(layer.scales) if has_s else None
        z_gn = to_np(layer.zeros) if has_z else None
        scales_n = s_gn.reshape(-1) if (csm in (1, 3)) else None
        int_acc = layer.acc_dtype == DType.INT32
        out = orc.matmul_int(
            a, q_kn, s_gn if wgm >= 2 else None, z_gn, scales_x, wgm, csm, layer.group_size,
            int_acc=int_acc, scales_n=scales_n,
        )
    out = np.asarray(out)
    if layer.bias is not None:
        out = out + to_np(layer.bias).reshape(1, -1)
    return out


def round_like(out, dtype):
    """Round an fp32 oracle result to the layer's output dtype (still as float32 / int)."""
    t = torch.from_numpy(np.asarray(out))
    if dtype in (torch.float16, torch.bfloat16):
        return t.float().to(dtype).float().numpy()
    return t.numpy()
