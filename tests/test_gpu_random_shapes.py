"""Seeded sweeps over shapes the hand-picked cases do not name: ragged N, K that ends inside a
pipeline stage or a K-slab, every row count up to a few tiles.  Same bar as the other GPU parity
tests: the C ABI against the CPU oracle on the same inputs."""
import numpy as np
import pytest
import torch

import gemlite_amd
from gemlite_amd import DType, GemLiteLinear, helper
from parity import FROB_TOL, gen_int_case, gen_x, oracle_forward, rel_frob, to_np

pytestmark = pytest.mark.gpu

TIGHT = {torch.float16: 1.5e-3, torch.bfloat16: 6e-3, torch.float32: 2e-4}


def check(layer, x, dtype, tag):
    print("case:", tag, flush=True)
    y_ref = oracle_forward(layer, x)
    y = layer(x)
    torch.cuda.synchronize()
    err = rel_frob(to_np(y).reshape(y_ref.shape), y_ref)
    assert err <= FROB_TOL and err <= TIGHT[dtype], (tag, err)


def row_counts(rng, n_small, n_large):
    return sorted({int(m) for m in rng.integers(1, 17, n_small)} | {int(m) for m in rng.integers(17, 301, n_large)})


@pytest.mark.parametrize("seed", range(12))
def test_packed_weight_only_random_shapes(device, seed):
    rng = np.random.default_rng(1000 + seed)
    nbits = int(rng.choice([1, 2, 4, 8]))
    gs = int(rng.choice([32, 64, 128, 256]))
    dtype = [torch.float16, torch.bfloat16][seed % 2]
    K = gs * int(rng.integers(1, 3072 // gs + 1))
    N = 8 * int(rng.integers(4, 200))
    channelwise = bool(rng.integers(0, 4) == 0)
    W_q, scales, zeros = gen_int_case(N, K, nbits, K if channelwise else gs, dtype, seed=seed, channelwise=channelwise)
    dt = gemlite_amd.TORCH_TO_DTYPE[dtype]
    layer = GemLiteLinear(nbits, K if channelwise else gs, K, N, dt, dt).pack(
        W_q.to(device), scales.to(device), zeros.to(device), fma_mode=bool(rng.integers(0, 2)))
    for M in row_counts(rng, 3, 3):
        check(layer, gen_x(M, K, dtype, seed=M).to(device), dtype,
              f"W{nbits} gs={gs} cw={channelwise} {dtype} M={M} N={N} K={K} mode={layer.W_group_mode}")


@pytest.mark.parametrize("seed", range(8))
def test_a8w8_dynamic_random_shapes(device, seed):
    rng = np.random.default_rng(2000 + seed)
    fp8 = bool(seed % 2)
    K = 32 * int(rng.integers(2, 96))
    N = 8 * int(rng.integers(4, 200))
    W = gen_x(N, K, torch.bfloat16, seed=seed, std=0.02)
    W_q, s = gemlite_amd.quantize_weights_per_channel(W, torch.float8_e4m3fn if fp8 else torch.int8)
    proc = helper.A8W8_FP8_dynamic(device=device) if fp8 else helper.A8W8_INT8_dynamic(device=device)
    proc.dtype = torch.bfloat16
    layer = proc.from_weights(W_q, scales=s)
    for M in row_counts(rng, 2, 3):
        check(layer, gen_x(M, K, torch.bfloat16, seed=M).to(device), torch.bfloat16,
              f"A8W8 {'fp8' if fp8 else 'int8'} M={M} N={N} K={K}")


@pytest.mark.parametrize("seed", range(6))
def test_a16w8_bytes_random_shapes(device, seed):
    rng = np.random.default_rng(3000 + seed)
    fp8 = bool(seed % 2)
    dtype = [torch.float16, torch.bfloat16][(seed // 2) % 2]
    K = 32 * int(rng.integers(2, 96))
    N = 8 * int(rng.integers(4, 200))
    W = gen_x(N, K, dtype, seed=seed, std=0.02)
    W_q, s = gemlite_amd.quantize_weights_per_channel(W, torch.float8_e4m3fn if fp8 else torch.int8)
    proc = (helper.A16W8_FP8 if fp8 else helper.A16W8_INT8)(device=device, dtype=dtype, post_scale=bool(rng.integers(0, 2)))
    layer = proc.from_weights(W_q, scales=s)
    for M in row_counts(rng, 3, 3):
        check(layer, gen_x(M, K, dtype, seed=M).to(device), dtype,
              f"A16W8 {'fp8' if fp8 else 'int8'} {dtype} M={M} N={N} K={K}")


@pytest.mark.parametrize("seed", range(6))
def test_mx_random_shapes(device, seed):
    rng = np.random.default_rng(4000 + seed)
    dtype = [torch.bfloat16, torch.float16][seed % 2]
    fp4 = seed % 3 != 2
    K = 128 * int(rng.integers(1, 33))
    N = 8 * int(rng.integers(4, 200))
    lin = torch.nn.Linear(K, N, bias=False, dtype=dtype)
    lin.weight.data = gen_x(N, K, dtype, seed=seed, std=0.02)
    proc = helper.A4W4_MXFP_dynamic(device=device, dtype=dtype) if fp4 else helper.A8W8_MXFP_dynamic(device=device, dtype=dtype)
    layer = proc.from_linear(lin.to(device))
    for M in row_counts(rng, 2, 3):
        check(layer, gen_x(M, K, dtype, seed=M).to(device), dtype, f"MX{'FP4' if fp4 else 'FP8'} {dtype} M={M} N={N} K={K}")


@pytest.mark.parametrize("seed", range(8))
def test_weight_only_mx_and_mixed_random_shapes(device, seed):
    """Weight-only MX layers (fp16 / bf16 x MXFP8 / MXFP4) and MXFP8 activations x MXFP4 weights: K a multiple of
    32 (streaming kernel at every batch size) or of 128 (matrix cores from 3 rows up)."""
    rng = np.random.default_rng(5000 + seed)
    dtype = [torch.bfloat16, torch.float16][seed % 2]
    kind = seed % 4   # 0: A16W4_MXFP, 1: A16W8_MXFP, 2: A8W4 per token, 3: A8W4 micro-scaled activations
    K = (128 if seed < 6 else 32) * int(rng.integers(1, 33))
    N = 8 * int(rng.integers(4, 200))
    lin = torch.nn.Linear(K, N, bias=bool(seed % 3 == 0), dtype=dtype)
    lin.weight.data = gen_x(N, K, dtype, seed=seed, std=0.02)
    if kind == 0:
        proc = helper.A16W4_MXFP(device=device, dtype=dtype)
    elif kind == 1:
        proc = helper.A16W8_MXFP(device=device, dtype=dtype)
    else:
        proc = helper.A8W4_MXFP_dynamic(device=device, dtype=dtype, post_scale=(kind == 2))
    layer = proc.from_linear(lin.to(device))
    for M in row_counts(rng, 3, 3):
        check(layer, gen_x(M, K, dtype, seed=M).to(device), dtype, f"MX kind {kind} {dtype} M={M} N={N} K={K}")


@pytest.mark.parametrize("seed", range(6))
def test_block_quantised_random_shapes(device, seed):
    rng = np.random.default_rng(6000 + seed)
    to_int8 = bool(seed % 2)
    dtype = [torch.bfloat16, torch.float16][(seed // 2) % 2]
    K = 128 * int(rng.integers(1, 40))
    N = 8 * int(rng.integers(4, 300))
    W = gen_x(N, K, dtype, seed=seed, std=0.02)
    proc = (helper.A8W8_INT8_dynamic if to_int8 else helper.A8W8_FP8_dynamic)(device=device, block_quant=True)
    layer = proc.from_weights(W)
    for M in row_counts(rng, 3, 3):
        check(layer, gen_x(M, K, dtype, seed=M).to(device), dtype, f"block-quant {'int8' if to_int8 else 'fp8'} {dtype} M={M} N={N} K={K}")
