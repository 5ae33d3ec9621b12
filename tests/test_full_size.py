"""Parity at the full sizes of the benchmark configurations.  The whole output is too large for the
CPU oracle, so the HIP result is checked on a seeded sample of output columns, for which the oracle
computes every row exactly (float64 / int64 accumulation) from the same weights and activations."""
import numpy as np
import pytest
import torch

import gemlite_amd
from gemlite_amd import DType, GemLiteLinear, helper
from oracle import oracle as orc
from parity import FROB_TOL, elementwise_excess, gen_int_case, gen_x, rel_frob, to_np

pytestmark = pytest.mark.gpu
TIGHT_BF16, TIGHT_FP16 = 6e-3, 1.5e-3


def sample_cols(N, count=48, seed=0):
    rng = np.random.default_rng(seed)
    cols = np.unique(np.concatenate([rng.integers(0, N, size=count), [0, N - 1]]))
    return cols


@pytest.mark.parametrize("nbits,gs,M", [(8, 16384, 1), (8, 16384, 16), (8, 16384, 64), (8, 16384, 256), (8, 16384, 512),
                                        (2, 64, 1), (2, 64, 16), (2, 64, 64), (2, 64, 256), (2, 64, 512)])
def test_a16wn_bf16_16384_square(device, nbits, gs, M):
    """bf16 activations x 8-bit channel-wise / 2-bit group-64 weights, N = K = 16384 (at 256 and 512 rows the tiled
    GEMM splits K under 256-row tiles for 8-bit codes and runs 128-row tiles two to a CU for 2-bit ones)."""
    N = K = 16384
    W_q, scales, zeros = gen_int_case(N, K, nbits, gs, torch.bfloat16, seed=nbits, scale_std=0.01)
    layer = helper.A16Wn(device=device, post_scale=True).from_weights(W_q, scales, zeros, nbits, gs)
    x = gen_x(M, K, torch.bfloat16, seed=M)
    y = to_np(layer(x.to(device)))
    cols = sample_cols(N, seed=M + nbits)
    gpn = K // gs   # groups per output row
    idx = (cols[:, None] * gpn + np.arange(gpn)[None, :]).reshape(-1)
    want = orc.hqq_dequant_matmul(to_np(x), W_q.numpy()[cols], to_np(scales)[idx], to_np(zeros)[idx], gs)
    err = rel_frob(y[:, cols], want)
    assert err <= FROB_TOL and err <= TIGHT_BF16, err
    assert elementwise_excess(y[:, cols], want, "bf16") <= 1.0


@pytest.mark.parametrize("fp8", [False, True])
def test_a8w8_dynamic_4096x8192x8192(device, fp8):
    """Per-token dynamic activations x per-channel 8-bit weights at M = 4096, N = K = 8192: the
    activation codes and scales are the oracle's bit for bit; sampled output columns follow from exact
    integer (float64) sums of those codes."""
    M, N, K = 4096, 8192, 8192
    W = gen_x(N, K, torch.bfloat16, seed=3, std=0.02)
    wq, sw = gemlite_amd.quantize_weights_per_channel(W, torch.float8_e4m3fn if fp8 else torch.int8)
    proc = (helper.A8W8_FP8_dynamic if fp8 else helper.A8W8_INT8_dynamic)(device=device)
    proc.dtype = torch.bfloat16
    layer = proc.from_weights(wq, scales=sw)
    x = gen_x(M, K, torch.bfloat16, seed=4)
    y = to_np(layer(x.to(device)))
    xq, sx = gemlite_amd.scale_activations_per_token(x.to(device), torch.float8_e4m3fn if fp8 else torch.int8)
    rows = np.arange(0, M, 61)   # the quantiser on a subset of rows, against the oracle
    want_q, want_s = orc.scale_activations_per_token(to_np(x)[rows], not fp8)
    got_q = xq.view(torch.uint8).cpu().numpy()[rows] if fp8 else xq.cpu().numpy()[rows]
    assert np.array_equal(got_q, want_q) and np.array_equal(sx.cpu().numpy()[rows], want_s)
    cols = sample_cols(N, seed=7)
    a = orc.e4m3fn_decode(xq.view(torch.uint8).cpu().numpy()) if fp8 else xq.cpu().numpy()
    wsub = wq.view(torch.uint8).numpy()[cols] if fp8 else wq.numpy()[cols]
    b = orc.e4m3fn_decode(wsub) if fp8 else wsub
    acc = a.astype(np.float64) @ b.astype(np.float64).T
    want = acc * sx.cpu().numpy().astype(np.float64) * to_np(sw).astype(np.float64).reshape(-1)[cols][None, :]
    assert rel_frob(y[:, cols], want.astype(np.float32)) <= TIGHT_BF16
    assert elementwise_excess(y[:, cols], want, "bf16") <= 1.0


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("shape", [(4096, 4096), (14336, 4096), (4096, 14336)])
def test_a8w8_dynamic_medium_batches_on_small_layers(device, fp8, shape):
    """Layers of a 4096-wide model at prefill chunks of a few hundred to a few thousand rows: the tile height and K
    split are chosen per layer size there (64- and 128-row tiles, with and without a split), and the first rows go
    through the streaming kernel.  Sampled output columns against exact sums of the GPU quantiser's own codes."""
    N, K = shape
    W = gen_x(N, K, torch.bfloat16, seed=13, std=0.02)
    wq, sw = gemlite_amd.quantize_weights_per_channel(W, torch.float8_e4m3fn if fp8 else torch.int8)
    proc = (helper.A8W8_FP8_dynamic if fp8 else helper.A8W8_INT8_dynamic)(device=device)
    proc.dtype = torch.bfloat16
    layer = proc.from_weights(wq, scales=sw)
    cols = sample_cols(N, seed=17)
    wsub = wq.view(torch.uint8).numpy()[cols] if fp8 else wq.numpy()[cols]
    b = (orc.e4m3fn_decode(wsub) if fp8 else wsub).astype(np.float64)
    swc = to_np(sw).astype(np.float64).reshape(-1)[cols][None, :]
    for M in (2, 40, 300, 1024, 2048):
        x = gen_x(M, K, torch.bfloat16, seed=M)
        y = to_np(layer(x.to(device)))
        xq, sx = gemlite_amd.scale_activations_per_token(x.to(device), torch.float8_e4m3fn if fp8 else torch.int8)
        a = orc.e4m3fn_decode(xq.view(torch.uint8).cpu().numpy()) if fp8 else xq.cpu().numpy()
        want = (a.astype(np.float64) @ b.T) * sx.cpu().numpy().astype(np.float64) * swc
        assert rel_frob(y[:, cols], want.astype(np.float32)) <= TIGHT_BF16, M
        assert elementwise_excess(y[:, cols], want, "bf16") <= 1.0, M


def test_int8_x_int8_int32_exact_4096x8192x8192(device):
    """INT8 x INT8 -> INT32 at M = 4096, N = K = 8192 with the accumulators as the output: sampled
    columns, all rows, bit for bit against exact sums (|sum| <= 8192 * 2^14 < 2^53, so float64 BLAS is
    exact) (reference epilogue: gemlite/triton_kernels/gemm_kernels.py:479-488 with channel_scale_mode 0)."""
    M, N, K = 4096, 8192, 8192
    g = torch.Generator().manual_seed(41)
    W = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    x = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
    layer = GemLiteLinear(8, None, K, N, DType.INT8, DType.INT32).pack(W.to(device), None, None)
    assert layer.acc_dtype == DType.INT32 and layer.W_group_mode == 0 and layer.channel_scale_mode == 0
    y = layer(x.to(device))
    assert y.dtype == torch.int32 and y.shape == (M, N)
    y = y.cpu().numpy()
    cols = sample_cols(N, count=96, seed=42)
    want = (x.numpy().astype(np.float64) @ W.numpy()[cols].astype(np.float64).T).astype(np.int64)
    assert np.array_equal(y[:, cols].astype(np.int64), want)
    # every tile of the output is touched by a cheap invariant too: the row sums over all columns
    # equal x @ (sum of weight rows), exactly
    wsum = W.numpy().astype(np.float64).sum(axis=0)
    assert np.array_equal(y.astype(np.int64).sum(axis=1), (x.numpy().astype(np.float64) @ wsum).astype(np.int64))


@pytest.mark.parametrize("M", [1, 32, 1024, 8192])
def test_a4w4_mxfp4_16384_square(device, M):
    N = K = 16384
    W = gen_x(N, K, torch.bfloat16, seed=9, std=0.02)
    codes, e8 = orc.quantize_mxfp4_weights(to_np(W))
    layer = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_weights(
        torch.from_numpy(codes), scales=torch.from_numpy(e8))
    x = gen_x(M, K, torch.bfloat16, seed=M)
    y = to_np(layer(x.to(device)))
    # the activation quantiser works row by row, so at the largest batch the oracle follows a sample of
    # rows: the first and last 256-row tiles whole, every 13th row between
    rows = np.arange(M) if M <= 1024 else np.unique(np.concatenate([np.arange(256), np.arange(256, M - 256, 13),
                                                                     np.arange(M - 256, M)]))
    a_packed, sa = orc.scale_activations_mxfp4(to_np(x)[rows])
    cols = sample_cols(N, seed=M)
    want = orc.matmul_mx(orc.unpack_fp4_bytes(a_packed), sa[:len(rows)], codes[cols], e8[cols])
    got = y[rows][:, cols]
    assert rel_frob(got, want) <= TIGHT_BF16
    assert elementwise_excess(got, want, "bf16") <= 1.0


@pytest.mark.parametrize("M", [1, 1024])
def test_a8w8_mxfp8_8192_square(device, M):
    N = K = 8192
    W = gen_x(N, K, torch.bfloat16, seed=10, std=0.02)
    codes, e8 = orc.quantize_mxfp8_weights(to_np(W))
    layer = helper.A8W8_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_weights(
        torch.from_numpy(codes).view(torch.float8_e4m3fn), scales=torch.from_numpy(e8))
    x = gen_x(M, K, torch.bfloat16, seed=M)
    y = to_np(layer(x.to(device)))
    aq, sx = orc.scale_activations_per_token(to_np(x), False)
    cols = sample_cols(N, seed=M)
    want = orc.matmul_mxfp8_weights(orc.e4m3fn_decode(aq), sx, codes[cols], e8[cols])
    assert rel_frob(y[:, cols], want) <= TIGHT_BF16
    assert elementwise_excess(y[:, cols], want, "bf16") <= 1.0


def test_a16w4_prefill_4096_cubed(device):
    """fp16 activations x 4-bit group-128 weights at M = N = K = 4096 (the GEMM point of the headline metric)."""
    M = N = K = 4096
    W_q, scales, zeros = gen_int_case(N, K, 4, 128, torch.float16, seed=12)
    layer = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
    x = gen_x(M, K, torch.float16, seed=13)
    y = to_np(layer(x.to(device)))
    cols = sample_cols(N, seed=14)
    gpn = K // 128
    idx = (cols[:, None] * gpn + np.arange(gpn)[None, :]).reshape(-1)
    want = orc.hqq_dequant_matmul(to_np(x), W_q.numpy()[cols], to_np(scales)[idx], to_np(zeros)[idx], 128)
    err = rel_frob(y[:, cols], want)
    assert err <= FROB_TOL and err <= TIGHT_FP16, err
    assert elementwise_excess(y[:, cols], want, "fp16") <= 1.0


@pytest.mark.parametrize("nbits,gs", [(4, 128), (8, 4096), (2, 64), (1, 128)])
@pytest.mark.parametrize("shape", [(4096, 4096), (11008, 4096)])
def test_a16wn_medium_batches_on_small_layers(device, nbits, gs, shape):
    """Packed-code layers of a 4096-wide model between decode and prefill: row chunks of 16 through the streaming
    kernel up to 64 rows (1-bit codes: chunks of 4 at any row count), the tiled GEMM above with the tile height and
    K split its cost model picks (32- and 64-row tiles with 4 to 8 splits, some ragged, up to 128 rows; 128-row tiles
    two to a CU at 1024)."""
    N, K = shape
    W_q, scales, zeros = gen_int_case(N, K, nbits, gs, torch.float16, seed=37 + nbits)
    layer = GemLiteLinear(nbits, gs, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
    cols = sample_cols(N, seed=3)
    gpn = K // gs
    idx = (cols[:, None] * gpn + np.arange(gpn)[None, :]).reshape(-1)
    for M in (5, 20, 48, 64, 65, 100, 128, 300, 1024):
        x = gen_x(M, K, torch.float16, seed=M)
        y = to_np(layer(x.to(device)))
        want = orc.hqq_dequant_matmul(to_np(x), W_q.numpy()[cols], to_np(scales)[idx], to_np(zeros)[idx], gs)
        err = rel_frob(y[:, cols], want)
        assert err <= FROB_TOL and err <= TIGHT_FP16, (M, err)
        assert elementwise_excess(y[:, cols], want, "fp16") <= 1.0, M


@pytest.mark.parametrize("to_int8", [True, False])
def test_a8w8_block_quantised_4096x8192x8192(device, to_int8):
    """128 x 128 block-quantised int8 / fp8 at M = 4096, N = K = 8192 (the matrix-core kernel, 128-row tiles):
    activation codes and scales bit for bit on a row sample; sampled output columns from exact sums per block."""
    M, N, K = 4096, 8192, 8192
    W = gen_x(N, K, torch.bfloat16, seed=21, std=0.02)
    codes, sw = orc.quantize_block_weights(to_np(W), to_int8)          # [N, K], [N/128, K/128]
    wdt = torch.int8 if to_int8 else torch.float8_e4m3fn
    wq = torch.from_numpy(codes) if to_int8 else torch.from_numpy(codes).view(torch.float8_e4m3fn)
    proc = (helper.A8W8_INT8_dynamic if to_int8 else helper.A8W8_FP8_dynamic)(device=device, dtype=torch.bfloat16, block_quant=True)
    layer = proc.from_weights(wq, scales=torch.from_numpy(sw))
    x = gen_x(M, K, torch.bfloat16, seed=22)
    y = to_np(layer(x.to(device)))
    xq, sx = gemlite_amd.scale_activations_per_block(x.to(device), wdt)
    rows = np.arange(0, M, 61)
    want_q, want_s = orc.scale_activations_per_block(to_np(x)[rows], to_int8)
    got_q = xq.cpu().numpy()[rows] if to_int8 else xq.view(torch.uint8).cpu().numpy()[rows]
    assert np.array_equal(got_q, want_q) and np.array_equal(sx.cpu().numpy()[rows], want_s)
    cols = sample_cols(N, seed=23)
    a = xq.cpu().numpy() if to_int8 else orc.e4m3fn_decode(xq.view(torch.uint8).cpu().numpy())
    b = codes[cols] if to_int8 else orc.e4m3fn_decode(codes[cols])
    sa = np.repeat(sx.cpu().numpy().astype(np.float64), 128, axis=1)
    sb = np.repeat(sw[cols // 128].astype(np.float64), 128, axis=1)
    want = (a.astype(np.float64) * sa) @ (b.astype(np.float64) * sb).T
    assert rel_frob(y[:, cols], want.astype(np.float32)) <= TIGHT_BF16
    assert elementwise_excess(y[:, cols], want, "bf16") <= 1.0


@pytest.mark.parametrize("M", [1, 4, 16])
def test_a16w4_mxfp_weight_only_16384_square(device, M):
    """bf16 activations x MXFP4 weights, N = K = 16384 (the streaming MX kernel)."""
    N = K = 16384
    W = gen_x(N, K, torch.bfloat16, seed=9, std=0.02)
    codes, e8 = orc.quantize_mxfp4_weights(to_np(W))
    layer = helper.A16W4_MXFP(device=device, dtype=torch.bfloat16).from_weights(torch.from_numpy(codes), torch.from_numpy(e8))
    x = gen_x(M, K, torch.bfloat16, seed=M)
    y = to_np(layer(x.to(device)))
    cols = sample_cols(N, seed=M)
    want = orc.matmul_mx_mixed(to_np(x), "float", None, codes[cols], "e2m1", e8[cols])
    assert rel_frob(y[:, cols], want) <= TIGHT_BF16
    assert elementwise_excess(y[:, cols], want, "bf16") <= 1.0


@pytest.mark.parametrize("post_scale,M", [(True, 1), (True, 1024), (False, 32), (False, 1024)])
def test_a8w4_mxfp_16384_square(device, post_scale, M):
    """MXFP8 activations (per token / micro-scaled) x MXFP4 weights, N = K = 16384: streaming kernel at M = 1,
    the mixed fp8 x fp4 MFMA above."""
    N = K = 16384
    W = gen_x(N, K, torch.bfloat16, seed=9, std=0.02)
    codes, e8 = orc.quantize_mxfp4_weights(to_np(W))
    layer = helper.A8W4_MXFP_dynamic(device=device, dtype=torch.bfloat16, post_scale=post_scale).from_weights(
        torch.from_numpy(codes), scales=torch.from_numpy(e8))
    x = gen_x(M, K, torch.bfloat16, seed=M)
    y = to_np(layer(x.to(device)))
    cols = sample_cols(N, seed=M)
    if post_scale:
        aq, sx = orc.scale_activations_per_token(to_np(x), False)
        want = orc.matmul_mx_mixed(aq, "e4m3", None, codes[cols], "e2m1", e8[cols], scales_x=sx)
    else:
        aq, sa = orc.scale_activations_mxfp8(to_np(x))
        want = orc.matmul_mx_mixed(aq, "e4m3", sa[:M], codes[cols], "e2m1", e8[cols])
    assert rel_frob(y[:, cols], want) <= TIGHT_BF16
    assert elementwise_excess(y[:, cols], want, "bf16") <= 1.0
