"""GPU parity tests: every call goes through the C ABI (gemlite_amd._ext) and is compared with
the CPU oracle on the same seeded inputs.  Integer / code outputs must match bit for bit; float
outputs are gated at 1e-2 relative Frobenius error (and a tighter bound that a correct kernel
with fp32 accumulation meets with room to spare)."""
import numpy as np
import pytest
import torch

import gemlite_amd
from gemlite_amd import DType, GemLiteLinear, _ext, helper
from gemlite_amd.bitpack import pack_weights_over_cols_hip, unpack_over_cols_hip
from oracle import oracle as orc
from parity import (FROB_TOL, elementwise_excess, gen_int_case, gen_x, kind_of, oracle_forward, rel_frob, round_like,
                    to_np)

pytestmark = pytest.mark.gpu

ALL_TYPES = ["GEMV_REVSPLITK", "GEMV", "GEMV_SPLITK", "GEMM_SPLITK", "GEMM"]
TIGHT = {torch.float16: 1.5e-3, torch.bfloat16: 6e-3, torch.float32: 2e-4}


def check_layer(layer, x, tol_dtype, types=ALL_TYPES, exact=False):
    y_ref = oracle_forward(layer, x)
    for mt in types:
        M = x.numel() // x.shape[-1]
        if M > 16 and "GEMV" in mt:
            continue
        print(f"case: {mt} M={M} N={layer.out_features} K={layer.in_features}", flush=True)
        y = layer.forward_manual(x, matmul_type=mt)
        torch.cuda.synchronize()
        y_np = to_np(y).reshape(y_ref.shape)
        if exact:
            assert np.array_equal(y_np, y_ref), mt
        else:
            err = rel_frob(y_np, y_ref)
            assert err <= FROB_TOL, (mt, err)
            assert err <= TIGHT[tol_dtype], (mt, err)
            ex = elementwise_excess(y_np, y_ref, kind_of(y.dtype))
            assert ex <= 1.0, (mt, "elementwise", ex)
    y_auto = layer(x)
    torch.cuda.synchronize()
    if exact:
        assert np.array_equal(to_np(y_auto).reshape(y_ref.shape), y_ref)
    else:
        assert rel_frob(to_np(y_auto).reshape(y_ref.shape), y_ref) <= TIGHT[tol_dtype]
        assert elementwise_excess(to_np(y_auto).reshape(y_ref.shape), y_ref, kind_of(y_auto.dtype)) <= 1.0


# ------------------------------------------------------------------ bit packing
@pytest.mark.parametrize("nbits", [1, 2, 4, 8])
@pytest.mark.parametrize("width", [8, 16, 32, 64])
def test_pack_unpack_bit_exact(device, nbits, width):
    rng = np.random.default_rng(nbits * 7 + width)
    e = width // nbits
    W = rng.integers(0, 2 ** nbits, size=(37, 6 * e), dtype=np.uint8)
    packed, e_out = pack_weights_over_cols_hip(torch.from_numpy(W).to(device), nbits, width, transpose=False)
    assert e_out == e
    assert np.array_equal(packed.cpu().numpy(), orc.pack_over_cols(W, nbits, width))
    back = unpack_over_cols_hip(packed, nbits, 6 * e)
    assert np.array_equal(back.cpu().numpy(), W)


def test_pack_large_matches_torch(device):
    g = torch.Generator().manual_seed(0)
    W = torch.randint(0, 16, (2032, 3968), generator=g, dtype=torch.int32).to(torch.uint8)
    ref, _ = gemlite_amd.pack_weights_over_cols_torch(W, 4, 32, transpose=True)
    out, _ = pack_weights_over_cols_hip(W.to(device), 4, 32, transpose=True)
    assert torch.equal(out.cpu(), ref)


# ------------------------------------------------------------------ activation quant
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 64), (5, 4224), (33, 8192), (7, 16384 + 64)])
def test_per_token_quant_bit_exact(device, dtype, shape):
    x = gen_x(shape[0], shape[1], dtype, seed=shape[1]) * 3
    x[0, 0] = 0.0
    for w_dtype, to_int8 in ((torch.int8, True), (torch.float8_e4m3fn, False)):
        y, s = gemlite_amd.scale_activations_per_token(x.to(device), w_dtype)
        q_ref, s_ref = orc.scale_activations_per_token(to_np(x), to_int8)
        assert s.shape == (shape[0], 1) and np.array_equal(s.cpu().numpy(), s_ref)
        y_bits = y.cpu().numpy() if to_int8 else y.view(torch.uint8).cpu().numpy()
        assert np.array_equal(y_bits, q_ref)


def test_per_token_quant_edge_rows(device):
    x = torch.zeros((3, 128), dtype=torch.bfloat16)
    x[1, 5] = -7.0
    x[2, :8] = torch.tensor([127.0, 0.5, 1.5, -0.5, -1.5, 2.5, -2.5, 0.0]).bfloat16()
    y, s = gemlite_amd.scale_activations_per_token(x.to(device), torch.int8)
    q_ref, s_ref = orc.scale_activations_per_token(to_np(x), True)
    assert np.array_equal(y.cpu().numpy(), q_ref) and np.array_equal(s.cpu().numpy(), s_ref)
    assert y.cpu()[2, :8].tolist() == [127, 1, 2, 0, -1, 3, -2, 0]
    # 3-D input keeps its shape
    y3, s3 = gemlite_amd.scale_activations_per_token(x.view(3, 2, 64).to(device), torch.int8)
    assert y3.shape == (3, 2, 64) and s3.shape == (6, 1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 32), (3, 4224), (32, 1024), (45, 16384)])
def test_mxfp4_quant_bit_exact(device, dtype, shape):
    x = gen_x(shape[0], shape[1], dtype, seed=shape[0]) * (2.0 ** torch.randint(-6, 6, (shape[0], 1)).float()).to(dtype)
    x[0, :8] = torch.tensor([0.25, -0.25, 0.75, 2.5, -0.0, 0.0, 5.0, -6.0]).to(dtype)
    y, s = gemlite_amd.scale_activations_mxfp4(x.to(device))
    y_ref, s_ref = orc.scale_activations_mxfp4(to_np(x))
    assert y.shape == (shape[0], shape[1] // 2) and s.shape == ((shape[0] + 31) // 32 * 32, shape[1] // 32)
    assert np.array_equal(s.cpu().numpy(), s_ref)
    assert np.array_equal(y.cpu().numpy(), y_ref)


@pytest.mark.parametrize("w_dtype", [torch.int8, torch.float8_e4m3fn])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_per_token_quant_every_16_bit_value(device, dtype, w_dtype):
    """Rows that hold every finite value of the input type up to a row maximum (both zeros, subnormals), for row
    maxima across the type's range: codes and scales equal the oracle's bit for bit.  (The kernel divides
    through a reciprocal and one correction step; tests/test_division.py proves the quotients equal over all
    pairs on the CPU, this runs the kernel itself over 28 rows of them.)"""
    allv = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(dtype)
    allv = allv[torch.isfinite(allv.float())]
    g = torch.Generator().manual_seed(5)
    tops = [allv.float().abs().max().item(), 1.0, 448.0, 127.0, 3.0e-5, 1.0e-7, 0.3333] + \
        (torch.rand(21, generator=g) * 16 - 12).exp2().tolist()
    rows = []
    for top in tops:
        top = torch.tensor(top).to(dtype)
        row = torch.where(allv.float().abs() <= top.float(), allv, torch.zeros_like(allv))
        rows.append(torch.cat([top.view(1), row, torch.zeros((-row.numel() - 1) % 8, dtype=dtype)]))
    x = torch.stack(rows)
    to_int8 = w_dtype == torch.int8
    y, sc = gemlite_amd.scale_activations_per_token(x.to(device), w_dtype)
    q_ref, s_ref = orc.scale_activations_per_token(to_np(x), to_int8)
    assert np.array_equal(sc.cpu().numpy(), s_ref)
    got = y.cpu().numpy() if to_int8 else y.cpu().view(torch.uint8).numpy()
    assert np.array_equal(got, q_ref if to_int8 else q_ref.view(np.uint8))


@pytest.mark.parametrize("amax_exp", [-9, -3, 0, 4, 12])
def test_mxfp4_quant_every_bf16_value(device, amax_exp):
    """The same for bf16 inputs (8 significant bits, the exponent range of fp32)."""
    top = 6.0 * 2.0 ** amax_exp
    allv = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    allv = allv[torch.isfinite(allv.float()) & (allv.float().abs() <= top)]
    pad = (-allv.numel()) % 31
    allv = torch.cat([allv, torch.zeros(pad, dtype=torch.bfloat16)])
    groups = allv.view(-1, 31)
    x = torch.cat([torch.full((groups.shape[0], 1), top, dtype=torch.bfloat16), groups], dim=1).reshape(1, -1)
    cols = 32 * 128
    x = torch.cat([x, torch.zeros((1, (-x.shape[1]) % cols), dtype=torch.bfloat16)], dim=1).view(-1, cols)
    y, s = gemlite_amd.scale_activations_mxfp4(x.to(device))
    y_ref, s_ref = orc.scale_activations_mxfp4(to_np(x))
    assert np.array_equal(s.cpu().numpy(), s_ref)
    assert np.array_equal(y.cpu().numpy(), y_ref)


@pytest.mark.parametrize("amax_exp", [-9, -3, 0, 4, 12])
def test_mxfp4_quant_every_fp16_value(device, amax_exp):
    """Every finite fp16 value (both zeros, subnormals, every exact tie) up to the block maximum, under a block
    scale pinned by one element 6 * 2^amax_exp per group of 32: codes and scales equal the oracle's bit for bit."""
    top = 6.0 * 2.0 ** amax_exp
    allv = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    allv = allv[torch.isfinite(allv) & (allv.float().abs() <= top)]
    pad = (-allv.numel()) % 31
    allv = torch.cat([allv, torch.zeros(pad, dtype=torch.float16)])
    groups = allv.view(-1, 31)
    x = torch.cat([torch.full((groups.shape[0], 1), top, dtype=torch.float16), groups], dim=1).reshape(1, -1)
    # rows of 128 groups, so that several rows and wave steps are exercised
    cols = 32 * 128
    x = torch.cat([x, torch.zeros((1, (-x.shape[1]) % cols), dtype=torch.float16)], dim=1).view(-1, cols)
    for dtype in (torch.float16, torch.float32):
        y, s = gemlite_amd.scale_activations_mxfp4(x.to(dtype).to(device))
        y_ref, s_ref = orc.scale_activations_mxfp4(to_np(x))
        assert np.array_equal(s.cpu().numpy(), s_ref)
        assert np.array_equal(y.cpu().numpy(), y_ref)


def test_mxfp4_quant_zero_and_tiny_groups(device):
    x = torch.zeros((2, 64), dtype=torch.bfloat16)
    x[1, 32:] = 1e-30
    y, s = gemlite_amd.scale_activations_mxfp4(x.to(device))
    y_ref, s_ref = orc.scale_activations_mxfp4(to_np(x))
    assert np.array_equal(s.cpu().numpy(), s_ref) and np.array_equal(y.cpu().numpy(), y_ref)
    assert s.cpu()[0].tolist() == [97, 97]


# ------------------------------------------------------------------ A16Wn
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("fma_mode", [True, False])
def test_a16w4_grouped_reference_test_shape(device, dtype, fma_mode):
    # the reference's own test shape: K = 3968, N = 2032 (edge tiles), 4-bit, group 128
    N, K, gs = 2032, 3968, 128
    W_q, scales, zeros = gen_int_case(N, K, 4, gs, dtype)
    dt = gemlite_amd.TORCH_TO_DTYPE[dtype]
    layer = GemLiteLinear(4, gs, K, N, dt, dt).pack(W_q.to(device), scales.to(device), zeros.to(device), fma_mode=fma_mode)
    assert layer.W_group_mode == (4 if fma_mode else 3) and layer.channel_scale_mode == 0 and layer.data_contiguous
    for M in (1, 3, 5, 16, 30, 65):
        check_layer(layer, gen_x(M, K, dtype, seed=M).to(device), dtype)


@pytest.mark.parametrize("M", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("shape", [(4096, 4096), (14336, 4096), (4096, 14336)])
def test_a16w4_benchmark_shapes(device, M, shape):
    N, K = shape
    W_q, scales, zeros = gen_int_case(N, K, 4, 128, torch.float16, seed=N + K)
    layer = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
    x = gen_x(M, K, torch.float16, seed=M)
    y_ref = oracle_forward(layer, x)
    y = layer(x.to(device))
    torch.cuda.synchronize()
    err = rel_frob(to_np(y), y_ref)
    assert err <= TIGHT[torch.float16], err
    # against the baseline's CPU path on the unpacked tensors: fp32 (W_q - z) * s, then matmul
    y_hqq = orc.hqq_dequant_matmul(to_np(x), W_q.numpy(), to_np(scales), to_np(zeros), 128)
    assert rel_frob(to_np(y), y_hqq) <= FROB_TOL


def test_split_k_hand_off_repeats_bit_for_bit(device):
    """The split-K hand-off of the packed-code GEMV (tagged slots, ticket counters that the last arriver resets) over
    many column tiles and slabs, launched 150 times in a row, two layers and several batch sizes taking turns on
    one stream and one workspace: every launch must reproduce the layer's first result bit for bit, and that
    result must match the oracle.  A counter or slot left dirty by one launch shows up in a later one."""
    layers = []
    for (N, K, seed) in ((4096, 14336, 3), (1024, 8192, 4)):   # 64 tiles x 4 slabs; 16 tiles with more slabs
        W_q, scales, zeros = gen_int_case(N, K, 4, 128, torch.float16, seed=seed)
        layers.append(GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device)))
    cases = []
    for li, layer in enumerate(layers):
        for M in (1, 3, 16):
            x = gen_x(M, layer.in_features, torch.float16, seed=10 * li + M)
            first = layer(x.to(device))
            torch.cuda.synchronize()
            assert rel_frob(to_np(first), oracle_forward(layer, x)) <= TIGHT[torch.float16]
            cases.append((layer, x.to(device), first.clone()))
    outs = []
    for it in range(150):
        layer, x, _ = cases[(7 * it) % len(cases)]
        outs.append(((7 * it) % len(cases), layer(x)))
    torch.cuda.synchronize()
    for ci, y in outs:
        assert torch.equal(y, cases[ci][2]), ci


@pytest.mark.parametrize("nbits,gs", [(2, 64), (1, 64), (4, 32), (4, 64), (8, 128), (2, 32), (4, 16)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_a16wn_bits_and_groups(device, nbits, gs, dtype):
    N, K = 1024, 2048
    W_q, scales, zeros = gen_int_case(N, K, nbits, gs, dtype, seed=nbits * 10 + gs)
    dt = gemlite_amd.TORCH_TO_DTYPE[dtype]
    layer = GemLiteLinear(nbits, gs, K, N, dt, dt).pack(W_q.to(device), scales.to(device), zeros.to(device))
    for M in (1, 4, 7, 24, 64, 100, 200):   # above 16 rows: every tile height of the MFMA GEMM
        check_layer(layer, gen_x(M, K, dtype, seed=M).to(device), dtype)


@pytest.mark.parametrize("nbits,gs", [(2, 16), (4, 16), (8, 16), (1, 32), (1, 64), (1, 128), (1, 256), (2, 32), (4, 32), (8, 32), (2, 64), (2, 128), (4, 64), (4, 128), (4, 256), (8, 64), (8, 128), (4, None), (8, None)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_packed_codes_at_17_to_64_rows(device, nbits, gs, dtype):
    """The mid-batch kernel (weights from registers into the MFMA, activations shared through an LDS ring): every code
    width and activation type, groups of 16, of a quarter of a stage, half a stage, one stage and several stages, channel-wise
    scales (gs None), 1..4 row tiles with ragged last tiles, batches above 64 rows as row chunks, N that ends inside a wave's 64 columns and inside a workgroup's 512, K of
    few and many stages (with and without a K split, splits of unequal length), a bias."""
    dt = gemlite_amd.TORCH_TO_DTYPE[dtype]
    for (N, K) in ((1000, 1280), (520, 4352), (2112, 512)):
        g = K if gs is None else gs
        W_q, scales, zeros = gen_int_case(N, K, nbits, g, dtype, seed=nbits * 100 + g % 1000 + N)
        layer = GemLiteLinear(nbits, g, K, N, dt, dt).pack(W_q.to(device), scales.to(device), zeros.to(device),
                                                           bias=gen_x(1, N, dtype, seed=5).reshape(-1).to(device) if N == 520 else None)
        m = layer.get_meta_args()
        for M in (5, 17, 32, 33, 47, 64, 150):
            x = gen_x(M, K, dtype, seed=M)
            y_ref = oracle_forward(layer, x)
            x = x.to(device)
            for tile in (-4, 2008, 1004):   # the library's plan; 8 waves and 2 splits; 4 waves, K in one piece
                out = torch.empty(M, N, dtype=dtype, device=device)
                a = _ext.build_matmul_args(x, layer.W_q, layer.scales, layer.zeros, None, out, W_nbits=m[1], group_size=m[2],
                                           unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                           acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                           data_contiguous=m[11], tile_config=tile, bias=layer.bias)
                assert _ext.matmul_family(a) == "WN_MID", (N, K, M, tile, _ext.matmul_family(a))
                print(f"case: WN_MID tile={tile} M={M} N={N} K={K}", flush=True)
                _ext.matmul(a, device)
                torch.cuda.synchronize()
                err = rel_frob(to_np(out), y_ref)
                assert err <= TIGHT[dtype], (N, K, M, tile, err)
                assert elementwise_excess(to_np(out), y_ref, kind_of(dtype)) <= 1.0, (N, K, M, tile)


@pytest.mark.parametrize("nbits,gs", [(4, 128), (4, 64), (2, 64), (8, 128), (8, None), (4, None), (4, 32), (2, 32), (1, 64), (1, 32), (1, 128),
                                      (2, 16), (4, 16), (8, 16)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_packed_layers_at_prefill_size_unpack_their_weights_first(device, nbits, gs, dtype):
    """From 2048 rows of bf16, 4096 of fp16 (or on request) the packed codes are written out once as 16-bit weights and the 16-bit
    matrix-core GEMM runs on them.  Every code width of the fused GEMM, groups of one and two 64-K chunks and one group
    per channel (scales after the K sum), both activation types; N ends inside a wave's 64 columns, K inside a
    workgroup's four chunks; a bias; the five dequantisation forms; and that the weights come out exactly as the fused
    kernel makes them (one-hot rows: bit-identical outputs of both paths).  Groups of 16 / 32 and 1-bit codes, which have
    no tiled GEMM and would run the mid-batch kernel once per 64 rows, take the same path (from 512 rows unasked)."""
    dt = gemlite_amd.TORCH_TO_DTYPE[dtype]
    N, K = (2032, 1088) if gs == 64 and nbits > 1 else (520, 1152)
    g = K if gs is None else gs
    W_q, scales, zeros = gen_int_case(N, K, nbits, g, dtype, seed=nbits * 100 + g % 1000)
    layer = GemLiteLinear(nbits, g, K, N, dt, dt).pack(W_q.to(device), scales.to(device), zeros.to(device),
                                                       bias=gen_x(1, N, dtype, seed=5).reshape(-1).to(device))
    l_scale = GemLiteLinear(nbits, g, K, N, dt, dt).pack(W_q.to(device), scales.to(device), None)                  # scales only
    l_zero = GemLiteLinear(nbits, g, K, N, dt, dt).pack(W_q.to(device), scales.to(device), 1 if nbits < 4 else 3)   # one integer zero
    l_shift = GemLiteLinear(nbits, g, K, N, dt, DType.FP32).pack(W_q.to(device), None, 1)                           # shift only

    def run(l, x, tile):
        m = l.get_meta_args()
        out = torch.empty(x.shape[0], N, dtype=dtype if l is not l_shift else torch.float32, device=device)
        a = _ext.build_matmul_args(x, l.W_q, l.scales, l.zeros, None, out, W_nbits=m[1], group_size=m[2], unpack_mask=m[3],
                                   elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6], acc_dtype=m[7], meta_dtype=m[8],
                                   channel_scale_mode=m[9], W_group_mode=m[10], data_contiguous=m[11], tile_config=tile, bias=l.bias)
        fam = _ext.matmul_family(a)
        print(f"case: {fam} tile={tile} M={x.shape[0]} N={N} K={K} W{nbits} gs={gs} mode={l.W_group_mode}", flush=True)
        _ext.matmul(a, device)
        torch.cuda.synchronize()
        return fam, out

    for M, tile in ((40, -5), (300, -5), (2048 if dtype == torch.bfloat16 else 4096, -1)):
        x = gen_x(M, K, dtype, seed=M)
        y_ref = oracle_forward(layer, x)
        fam, out = run(layer, x.to(device), tile)
        assert fam == "GEMM_16BIT", (M, tile, fam)
        err = rel_frob(to_np(out), y_ref)
        assert err <= TIGHT[dtype], (M, err)
        assert elementwise_excess(to_np(out), y_ref, kind_of(dtype)) <= 1.0, M
    for l, tol in ((l_scale, dtype), (l_zero, dtype), (l_shift, torch.float32)):
        x = (gen_x(70, K, dtype, seed=7) / 10)
        fam, out = run(l, x.to(device), -5)
        assert fam == "GEMM_16BIT", (l.W_group_mode, fam)
        y_ref = oracle_forward(l, x)
        assert rel_frob(to_np(out), y_ref) <= TIGHT[tol], l.W_group_mode
    # one-hot rows read single weights: the fused kernel and this path must agree to the bit
    x = torch.zeros(48, K, dtype=dtype)
    for r in range(48):
        x[r, (53 * r + 11) % K] = 1.0
    layer.bias = None
    tiled = (gs is None or gs % 64 == 0) and nbits > 1
    (fa, ya), (fb, yb) = run(layer, x.to(device), -3 if tiled else -4), run(layer, x.to(device), -5)
    assert (fa, fb) == ("GEMM_WN" if tiled else "WN_MID", "GEMM_16BIT")
    assert torch.equal(ya, yb)


@pytest.mark.parametrize("nbits,gs", [(1, 32), (1, 64), (2, 16), (2, 32), (4, 16), (8, 16)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_packed_codes_in_short_groups(device, nbits, gs, dtype):
    """Groups shorter than a step of the tuned kernels: the generic family's K-split packed-word kernel.  N is not a
    multiple of 64 (lanes past N), K gives some waves no word row (1-bit: 10 word rows for 16 waves) or splits groups
    between waves, rows 1 / 2 / 4 per lane and a ragged last block; scale-only, shift-only and scalar-zero modes."""
    dt = gemlite_amd.TORCH_TO_DTYPE[dtype]
    for N, K in ((200, 320), (1000, 2112)):
        if nbits == 8:
            K += 32  # not a whole number of the mid-batch kernel's 64-K stages either
        W_q, scales, zeros = gen_int_case(N, K, nbits, gs, dtype, seed=nbits * 100 + gs)
        layer = GemLiteLinear(nbits, gs, K, N, dt, dt).pack(W_q.to(device), scales.to(device), zeros.to(device))
        x1 = gen_x(1, K, dtype, seed=1).to(device)
        a = _ext.build_matmul_args(x1, layer.W_q, layer.scales, layer.zeros, None, torch.empty(1, N, dtype=dtype, device=device),
                                   **dict(zip(("W_nbits", "group_size", "unpack_mask", "elements_per_sample", "input_dtype", "output_dtype",
                                               "acc_dtype", "meta_dtype", "channel_scale_mode", "W_group_mode", "data_contiguous"),
                                              layer.get_meta_args()[1:12])))
        assert _ext.matmul_family(a) == "GENERIC"
        for M in (1, 2, 3, 4, 9, 21):
            check_layer(layer, gen_x(M, K, dtype, seed=M).to(device), dtype, types=())
    N, K = 328, 1088
    W_q, scales, _ = gen_int_case(N, K, nbits, gs, dtype, seed=5)
    l2 = GemLiteLinear(nbits, gs, K, N, dt, dt).pack(W_q.to(device), scales.to(device), None)                 # scales only
    l3 = GemLiteLinear(nbits, gs, K, N, dt, dt).pack(W_q.to(device), scales.to(device), 1 if nbits < 4 else 3)  # one integer zero
    l1 = GemLiteLinear(nbits, gs, K, N, dt, DType.FP32).pack(W_q.to(device), None, 1)                          # shift only
    assert (l2.W_group_mode, l3.W_group_mode, l1.W_group_mode) == (2, 3, 1)
    for layer, tol in ((l2, dtype), (l3, dtype), (l1, torch.float32)):
        for M in (1, 6):
            check_layer(layer, (gen_x(M, K, dtype, seed=M) / 10).to(device), tol, types=())


@pytest.mark.parametrize("nbits,gs", [(1, 32), (2, 16)])
def test_short_group_codes_at_prefill_size(device, nbits, gs):
    """1024 rows on packings the tiled GEMM does not take: the weights are unpacked into the workspace and the 16-bit GEMM runs
    (below 1024 rows: row chunks of the mid-batch kernel)."""
    N, K, M = 256, 1024, 1024
    W_q, scales, zeros = gen_int_case(N, K, nbits, gs, torch.float16, seed=nbits + gs)
    layer = GemLiteLinear(nbits, gs, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
    check_layer(layer, gen_x(M, K, torch.float16, seed=M).to(device), torch.float16, types=())


def test_int32_accumulator_on_4_bit_codes_stays_exact(device):
    """int8 activations x shift-only 4-bit codes with an int32 accumulator (reference: tests/test_int.py:173-199),
    every activation 127 and every code at the top of its range: the sums of 127 * 8 over K are exact integers at
    K = 8192, where the widened 16-bit kernels run them in fp32 (K * 128 * 15 < 2^24), and at K = 16384, which is
    past that bound and goes to the integer loop of the generic kernel."""
    N = 256
    for K in (8192, 16384):
        W_q = torch.full((N, K), 15, dtype=torch.uint8)
        W_q[::2, ::3] = 3
        layer = GemLiteLinear(4, 128, K, N, DType.INT8, DType.FP32, scaled_activations=True).pack(W_q.to(device), None, 7)
        layer.meta_dtype = DType.FP32
        assert (layer.W_group_mode, layer.channel_scale_mode, layer.acc_dtype) == (1, 2, DType.INT32)
        for M in (1, 20, 100):
            x = torch.full((M, K), 127.0, dtype=torch.float16)
            x[:, 1::2] = -127.0
            x[:, ::5] = 127.0
            y = layer(x.to(device))
            torch.cuda.synchronize()
            want = x.double() @ (W_q.double() - 7.0).T
            assert np.array_equal(to_np(y).astype(np.float64), want.numpy()), (K, M)


@pytest.mark.parametrize("post_scale", [True, False])
@pytest.mark.parametrize("nbits", [8, 4])
def test_a16wn_channelwise(device, nbits, post_scale):
    N, K = 768, 1536
    W_q, scales, zeros = gen_int_case(N, K, nbits, K, torch.bfloat16, seed=nbits, scale_std=0.01, channelwise=True)
    layer = helper.A16Wn(device=device, post_scale=post_scale).from_weights(W_q, scales, zeros, nbits, K)
    assert (layer.W_group_mode, layer.channel_scale_mode) == ((1, 1) if post_scale else (3, 0))
    for M in (1, 2, 16, 65):
        check_layer(layer, gen_x(M, K, torch.bfloat16, seed=M).to(device), torch.bfloat16)


def test_symmetric_and_shift_only_modes(device):
    N, K, gs = 512, 1024, 128
    W_q, scales, _ = gen_int_case(N, K, 4, gs, torch.float16)
    # mode 2: scales only
    l2 = GemLiteLinear(4, gs, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), None)
    assert l2.W_group_mode == 2
    # mode 3 with an integer zero point
    l3 = GemLiteLinear(4, gs, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), 8)
    assert l3.W_group_mode == 3 and l3.zeros.numel() == 1
    # mode 1: shift only, fp32 output
    l1 = GemLiteLinear(4, gs, K, N, DType.FP16, DType.FP32).pack(W_q.to(device), None, 7)
    assert l1.W_group_mode == 1
    for layer, dt in ((l2, torch.float16), (l3, torch.float16), (l1, torch.float32)):
        for M in (1, 5):
            check_layer(layer, (gen_x(M, K, torch.float16, seed=M) / 10).to(device), dt)


def test_unpacked_fp16_weights_and_bias(device):
    N, K = 1000, 2048
    W = gen_x(N, K, torch.float16, seed=3, std=0.05)
    bias = gen_x(1, N, torch.float16, seed=4).view(N)
    layer = GemLiteLinear(16, None, K, N, DType.FP16, DType.FP16).pack(W.to(device), None, None, bias.to(device))
    assert layer.W_group_mode == 0 and layer.elements_per_sample == 1 and not layer.data_contiguous
    for M in (1, 3, 17):
        x = gen_x(M, K, torch.float16, seed=M).to(device)
        check_layer(layer, x, torch.float16)
    # 3-D activations keep their leading dims
    y = layer(gen_x(6, K, torch.float16).view(2, 3, K).to(device))
    assert y.shape == (2, 3, N)


@pytest.mark.parametrize("contiguous", [None, True])
@pytest.mark.parametrize("w_dtype,x_dtype", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
                                             (torch.bfloat16, torch.float16), (torch.float16, torch.bfloat16)])
def test_unpacked_16_bit_weights_both_layouts(device, contiguous, w_dtype, x_dtype):
    """16-bit weights as the layer keeps them ([N, K], K contiguous: a wave per two columns, lanes along K) and as
    pack(contiguous=True) makes them ([K, N]: a lane per column, K split over the waves); N odd or not a multiple of
    64, K not a multiple of the 512 values a wave covers per step, 1 / 2 / 4 rows per lane and a ragged last block."""
    xdt = gemlite_amd.TORCH_TO_DTYPE[x_dtype]
    for N, K in ((1000, 2048), (77, 224), (4096, 4128)):
        W = gen_x(N, K, w_dtype, seed=N, std=0.05)
        layer = GemLiteLinear(16, None, K, N, xdt, xdt).pack(W.to(device), None, None, contiguous=contiguous)
        assert layer.data_contiguous == bool(contiguous) and layer.W_q.stride(1) == (1 if contiguous else K)
        for M in (1, 2, 3, 4, 9, 18):
            check_layer(layer, gen_x(M, K, x_dtype, seed=M).to(device), x_dtype, types=())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_unquantised_layers_above_16_rows_on_matrix_cores(device, dtype):
    """W_nbits = 16 at the reference's own test shape (tests/test_int.py:99-118: K = 3968, N = 2032) and its batch
    sizes above 16 rows, and at a shape whose K is a few stages: the MFMA GEMM on both operands as they lie ([rows, K],
    K contiguous), every tile height, with and without a K split, ragged M and N tiles, a bias."""
    dt = gemlite_amd.TORCH_TO_DTYPE[dtype]
    for (N, K, with_bias) in ((2032, 3968, False), (520, 160, True)):
        W = gen_x(N, K, dtype, seed=N, std=0.05)
        bias = gen_x(1, N, dtype, seed=4).view(N).to(device) if with_bias else None
        layer = GemLiteLinear(16, None, K, N, dt, dt).pack(W.to(device), None, None, bias)
        assert layer.W_group_mode == 0 and layer.channel_scale_mode == 0 and not layer.data_contiguous
        m = layer.get_meta_args()
        for M in (17, 30, 65, 100, 250, 600):
            x = gen_x(M, K, dtype, seed=M).to(device)
            out = torch.empty(M, N, dtype=dtype, device=device)
            a = _ext.build_matmul_args(x, layer.W_q, layer.scales, layer.zeros, None, out, W_nbits=m[1], group_size=m[2],
                                       unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                       acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                       data_contiguous=m[11])
            assert _ext.matmul_family(a) == "GEMM_16BIT", (N, K, M, _ext.matmul_family(a))
            check_layer(layer, x, dtype, types=["GEMM_SPLITK", "GEMM"])


@pytest.mark.parametrize("width", [8, 16, 64])
def test_other_packing_widths(device, width):
    N, K, gs = 256, 512, 64
    W_q, scales, zeros = gen_int_case(N, K, 4, gs, torch.float16, seed=width)
    layer = GemLiteLinear(4, gs, K, N, DType.FP16, DType.FP16).pack(
        W_q.to(device), scales.to(device), zeros.to(device), packing_bitwidth=width)
    assert layer.W_q.element_size() * 8 == width
    check_layer(layer, gen_x(3, K, torch.float16).to(device), torch.float16)


# ------------------------------------------------------------------ 8-bit activations
def test_int8_x_int8_accumulators_bit_exact(device):
    N, K = 520, 1024
    g = torch.Generator().manual_seed(0)
    W = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    layer = GemLiteLinear(8, None, K, N, DType.INT8, DType.INT32).pack(W.to(device), None, None)
    assert layer.acc_dtype == DType.INT32 and layer.W_group_mode == 0 and layer.channel_scale_mode == 0
    for M in (1, 2, 9, 70, 256):
        x = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
        ref = (x.long() @ W.long().t()).numpy()
        for mt in ALL_TYPES:
            y = layer.forward_manual(x.to(device), matmul_type=mt)
            assert y.dtype == torch.int32 and np.array_equal(y.cpu().numpy(), ref), (mt, M)


@pytest.mark.parametrize("fp8", [False, True])
def test_a8w8_dynamic(device, fp8):
    N, K = 1032, 2048
    W = gen_x(N, K, torch.bfloat16, seed=5, std=0.02)
    proc = helper.A8W8_FP8_dynamic(device=device) if fp8 else helper.A8W8_INT8_dynamic(device=device)
    # weights are quantised once on the host (CPU torch), then handed over pre-quantised
    W_q_cpu, s_cpu = gemlite_amd.quantize_weights_per_channel(W, torch.float8_e4m3fn if fp8 else torch.int8)
    proc.dtype = torch.bfloat16
    layer = proc.from_weights(W_q_cpu, scales=s_cpu)
    assert (layer.W_group_mode, layer.channel_scale_mode) == (0, 3) and layer.scales.dtype == torch.float32
    assert layer.W_q.stride() == (1, K)
    # the weight codes are the oracle's
    q_ref, s_ref = orc.quantize_per_channel(to_np(W), not fp8)
    got = layer.W_q.t().contiguous()
    got = got.view(torch.uint8).cpu().numpy() if fp8 else got.cpu().numpy()
    assert np.array_equal(got, q_ref) and np.array_equal(layer.scales.cpu().numpy().reshape(-1, 1), s_ref)
    for M in (1, 2, 33, 128):
        check_layer(layer, gen_x(M, K, torch.bfloat16, seed=M).to(device), torch.bfloat16)


@pytest.mark.parametrize("fp8", [False, True])
def test_a8w8_dynamic_streams_the_first_rows(device, fp8):
    """Dynamically quantised A8W8 layers at 1-2 rows (3-4 on small layers) take the K-major streaming kernel with
    8-bit activations, the matrix-core GEMM above.  Ragged N (last workgroup has 2 of 4 columns), K that does not
    fill the waves' last sweep, and the exact int32 sums of int8 x int8 against an int64 reference."""
    import ctypes
    from gemlite_amd import _ext
    N, K = 1030, 4160
    W = gen_x(N, K, torch.bfloat16, seed=15, std=0.02)
    proc = helper.A8W8_FP8_dynamic(device=device) if fp8 else helper.A8W8_INT8_dynamic(device=device)
    W_q_cpu, s_cpu = gemlite_amd.quantize_weights_per_channel(W, torch.float8_e4m3fn if fp8 else torch.int8)
    proc.dtype = torch.bfloat16
    layer = proc.from_weights(W_q_cpu, scales=s_cpu)
    for M, fam in ((1, "GEMV_KMAJOR"), (2, "GEMV_KMAJOR"), (3, "GEMV_KMAJOR"), (4, "GEMV_KMAJOR"), (5, "GEMM_8BIT")):
        x = gen_x(M, K, torch.bfloat16, seed=20 + M).to(device)
        xq, sx = gemlite_amd.scale_activations_per_token(x, torch.float8_e4m3fn if fp8 else torch.int8)
        m = layer.get_meta_args()
        out = torch.empty(M, N, dtype=torch.bfloat16, device=device)
        a = _ext.build_matmul_args(xq, layer.W_q, layer.scales, layer.zeros, sx, out, W_nbits=m[1], group_size=m[2],
                                   unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                   acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                   data_contiguous=m[11])
        assert _ext.matmul_family(a) == fam
        check_layer(layer, x, torch.bfloat16)
        if not fp8 and M <= 4:
            # fp32 output: every element is float(int32 sum) * (s_w * s_x), the sum exact
            y32 = torch.empty(M, N, dtype=torch.float32, device=device)
            a32 = _ext.build_matmul_args(xq, layer.W_q, layer.scales, layer.zeros, sx, y32, W_nbits=m[1], group_size=m[2],
                                         unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=DType.FP32.value,
                                         acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                         data_contiguous=m[11])
            assert _ext.matmul_family(a32) == "GEMV_KMAJOR"
            rc = _ext.load_library().gla_matmul(ctypes.byref(a32), torch.cuda.current_stream().cuda_stream)
            assert rc == 0
            torch.cuda.synchronize()
            acc = xq.cpu().to(torch.int64) @ layer.W_q.t().contiguous().cpu().to(torch.int64).t()
            want = acc.to(torch.float32) * (layer.scales.cpu().reshape(1, N).float() * sx.cpu().reshape(M, 1).float())
            assert torch.equal(y32.cpu(), want)
    # a larger layer hands over at 3 rows
    N2, K2 = 5120, 4096
    W2 = gen_x(N2, K2, torch.bfloat16, seed=16, std=0.02)
    l2 = proc.from_weights(*gemlite_amd.quantize_weights_per_channel(W2, torch.float8_e4m3fn if fp8 else torch.int8)[:1],
                           scales=gemlite_amd.quantize_weights_per_channel(W2, torch.float8_e4m3fn if fp8 else torch.int8)[1])
    for M in (2, 3):
        check_layer(l2, gen_x(M, K2, torch.bfloat16, seed=30 + M).to(device), torch.bfloat16)


@pytest.mark.parametrize("fp8", [False, True])
def test_a8w8_decode_batches_on_the_matrix_cores_in_one_launch(device, fp8):
    """fp8 x fp8 and int8 x int8 at 3..32 rows (K a multiple of 128): both operands are copied to LDS by lines and go
    into the MFMA as they are.  Ragged N, K with fewer turns than waves and with a last turn only some waves take,
    one and two activation tiles, every launch shape (1, 2 and 4 weight tiles per wave), a bias; for int8 the fp32
    output is float(exact int32 sum) * (s_w * s_x) and the int32 output the exact sum."""
    import ctypes
    from gemlite_amd import _ext
    lib = _ext.load_library()
    wdt = torch.float8_e4m3fn if fp8 else torch.int8
    for (N, K) in ((1040, 4096), (520, 2304), (72, 128), (7056, 768), (14096, 512)):
        W = gen_x(N, K, torch.bfloat16, seed=N + 1, std=0.02)
        proc = helper.A8W8_FP8_dynamic(device=device) if fp8 else helper.A8W8_INT8_dynamic(device=device)
        proc.dtype = torch.bfloat16
        W_q_cpu, s_cpu = gemlite_amd.quantize_weights_per_channel(W, wdt)
        layer = proc.from_weights(W_q_cpu, scales=s_cpu, bias=gen_x(1, N, torch.bfloat16, seed=2).reshape(-1) if N == 520 else None)
        for M in (3, 5, 16, 17, 32, 33):
            x = gen_x(M, K, torch.bfloat16, seed=80 + M).to(device)
            xq, sx = gemlite_amd.scale_activations_per_token(x, wdt)
            m = layer.get_meta_args()
            out = torch.empty(M, N, dtype=torch.bfloat16, device=device)
            a = _ext.build_matmul_args(xq, layer.W_q, layer.scales, layer.zeros, sx, out, W_nbits=m[1], group_size=m[2],
                                       unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                       acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                       data_contiguous=m[11])
            ring = M <= 16 or (M <= 32 and N < 7040)   # two activation tiles: only where N is short
            assert _ext.matmul_family(a) == ("K_SKINNY" if ring else "GEMM_8BIT"), (N, K, M, _ext.matmul_family(a))
            check_layer(layer, x, torch.bfloat16)
            if not fp8 and N != 520 and ring:
                y32 = torch.empty(M, N, dtype=torch.float32, device=device)
                a32 = _ext.build_matmul_args(xq, layer.W_q, layer.scales, layer.zeros, sx, y32, W_nbits=m[1], group_size=m[2],
                                             unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=DType.FP32.value,
                                             acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                             data_contiguous=m[11])
                assert lib.gla_matmul(ctypes.byref(a32), torch.cuda.current_stream().cuda_stream) == 0
                torch.cuda.synchronize()
                acc = xq.cpu().to(torch.int64) @ layer.W_q.t().contiguous().cpu().to(torch.int64).t()
                want = acc.to(torch.float32) * (layer.scales.cpu().reshape(1, N).float() * sx.cpu().reshape(M, 1).float())
                assert torch.equal(y32.cpu(), want), (N, K, M)
    if not fp8:
        # INT8 x INT8 -> INT32, no scales: the exact sums
        g = torch.Generator().manual_seed(3)
        N, K = 1048, 1536
        Wi = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
        li = GemLiteLinear(8, None, K, N, DType.INT8, DType.INT32).pack(Wi.to(device), None, None)
        for M in (3, 16, 20, 32):
            xi = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
            y = li.forward_manual(xi.to(device), matmul_type="GEMM_SPLITK")
            assert y.dtype == torch.int32 and np.array_equal(y.cpu().numpy(), (xi.long() @ Wi.long().t()).numpy()), M


def test_int8_activations_packed_weights(device):
    # int8 x 4-bit with an integer zero and channel-wise scales (reference: tests/test_int.py:146-171)
    N, K = 400, 1024
    W_q, _, _ = gen_int_case(N, K, 4, 128, torch.bfloat16)
    scales = (gen_x(N, 1, torch.bfloat16, seed=9) * 1e-2)
    layer = GemLiteLinear(4, 128, K, N, DType.INT8, DType.FP32).pack(W_q.to(device), scales.to(device), 7)
    assert (layer.W_group_mode, layer.channel_scale_mode) == (1, 1)
    g = torch.Generator().manual_seed(1)
    for M in (1, 5, 65):
        x = torch.randint(-10, 10, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
        check_layer(layer, x.to(device), torch.float32)
    # dynamic int8 activations x shifted 4-bit weights (reference: tests/test_int.py:173-199)
    layer = GemLiteLinear(4, 128, K, N, DType.INT8, DType.FP32, scaled_activations=True).pack(W_q.to(device), None, 7)
    layer.meta_dtype = DType.FP32
    assert (layer.W_group_mode, layer.channel_scale_mode) == (1, 2)
    for M in (1, 5, 65):
        check_layer(layer, (gen_x(M, K, torch.float16, seed=M) / 20).to(device), torch.float32)


def _forward_both_ways(layer, x):
    """(forward with the activations quantised inside the matmul, forward with the quantiser launch in front)."""
    from gemlite_amd import core
    y_fused = layer(x)
    rows = core._FUSED_QUANT_ROWS
    core._FUSED_QUANT_ROWS = 0
    try:
        y_two = layer(x)
    finally:
        core._FUSED_QUANT_ROWS = rows
    torch.cuda.synchronize()
    return y_fused, y_two


def _fused_family(layer, x):
    """Kernel family the library picks when asked to quantise `x` inside the matmul, or None if it declines."""
    m = layer.get_meta_args()
    out = torch.empty(x.shape[0], layer.out_features, dtype=gemlite_amd.DTYPE_TO_TORCH[m[6]], device=x.device)
    a = _ext.build_matmul_args(x, layer.W_q, layer.scales, layer.zeros, None, out, W_nbits=m[1], group_size=m[2],
                               unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                               acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                               data_contiguous=m[11], x_quant_from=gemlite_amd.TORCH_TO_DTYPE[x.dtype].value)
    return _ext.matmul_family(a) if _ext.matmul_is_supported(a) else None


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_a8w8_decode_rows_are_quantised_inside_the_matmul(device, fp8, dtype):
    """At the rows the K-major streaming kernel takes (up to 4 when K is not a multiple of 128, else 2: from 3 rows
    the one-launch matrix-core kernel wants ready-made codes) it takes the 16-bit rows and quantises them per token
    itself (reference: the quantiser call in front of the matmul, gemlite/core.py:220-250): the output must equal
    the quantiser launch followed by the matmul bit for bit, rows of very different magnitudes, an all-zero row
    (scale 1e-6) and a ragged K included; above those rows the library declines and forward() runs two launches."""
    for (N, K) in ((1030, 4160), (512, 8192)):
        W = gen_x(N, K, torch.bfloat16, seed=15, std=0.02)
        proc = helper.A8W8_FP8_dynamic(device=device) if fp8 else helper.A8W8_INT8_dynamic(device=device)
        W_q_cpu, s_cpu = gemlite_amd.quantize_weights_per_channel(W, torch.float8_e4m3fn if fp8 else torch.int8)
        proc.dtype = dtype
        layer = proc.from_weights(W_q_cpu, scales=s_cpu)
        for M in (1, 2, 3, 4, 5):
            x = gen_x(M, K, dtype, seed=40 + M)
            x[0] *= 37.0
            if M > 1:
                x[1] = 0.0
            if M > 2:
                x[2] *= 1e-3
            x = x.to(device)
            assert _fused_family(layer, x) == ("GEMV_KMAJOR" if M <= (4 if K % 128 else 2) else None), M
            y_fused, y_two = _forward_both_ways(layer, x)
            assert torch.equal(y_fused, y_two), (N, K, M)
            check_layer(layer, x, dtype)
    # a large layer keeps the streaming kernel, and with it the quantiser inside, for 2 rows only
    big = helper.A8W8_INT8_dynamic(device=device)
    big.dtype = torch.bfloat16
    Wb = gen_x(8192, 4096, torch.bfloat16, seed=3, std=0.02)
    Wq_b, s_b = gemlite_amd.quantize_weights_per_channel(Wb, torch.int8)
    layer = big.from_weights(Wq_b, scales=s_b)
    for M, fam in ((2, "GEMV_KMAJOR"), (3, None)):
        x = gen_x(M, 4096, torch.bfloat16, seed=M).to(device)
        assert _fused_family(layer, x) == fam
        y_fused, y_two = _forward_both_ways(layer, x)
        assert torch.equal(y_fused, y_two), M


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_a4w4_decode_rows_are_quantised_inside_the_matmul(device, dtype):
    """MXFP4 x MXFP4 at the rows the streaming kernel takes: the kernel makes the e2m1 codes and e8m0 bytes of its
    activation blocks itself; same output as the quantiser launch + matmul bit for bit (blocks of all zeros, of
    tiny and of huge values, ties of the e2m1 grid included)."""
    for (N, K) in ((520, 4224), (512, 4096)):   # K of the reference's MX tests (streams up to 4 rows); a K the matrix cores take
        W = gen_x(N, K, torch.bfloat16, seed=7, std=0.02)
        codes, e8 = orc.quantize_mxfp4_weights(to_np(W))
        layer = helper.A4W4_MXFP_dynamic(device=device, dtype=dtype).from_weights(torch.from_numpy(codes), scales=torch.from_numpy(e8))
        for M in (1, 2, 3, 4, 5):
            x = gen_x(M, K, dtype, seed=60 + M)
            x[0, :32] = 0.0
            x[0, 32:64] = torch.tensor([0.75, 1.75, 3.5, -0.75, -1.75, -3.5, 0.25, 6.0] * 4).to(dtype)  # ties at scale 1
            x[0, 64:96] *= 1e-4
            x[0, 96:128] *= 3e3
            x = x.to(device)
            if K % 256 == 0:   # from 3 rows the scaled-MFMA kernel takes ready-made codes: the fused call is declined
                assert _fused_family(layer, x) == ("MX_STREAM" if M <= 2 else None), M
            y_fused, y_two = _forward_both_ways(layer, x)
            assert torch.equal(y_fused, y_two), (K, M)
            check_layer(layer, x, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_a4w4_mxfp4_skinny_rows_on_the_scaled_mfma(device, dtype):
    """3..32 rows of MXFP4 x MXFP4 (K a multiple of 256): weight and activation codes are copied to LDS by lines and
    go into the scaled MFMA as they are.  Ragged N (last tile of 16 columns partly past N), K with fewer pairs of steps
    than waves and with a last turn only some waves take, one and two activation tiles, every launch shape (1, 2 and 4
    weight tiles per wave), a bias."""
    for (N, K) in ((1040, 4096), (520, 2304), (2056, 512), (72, 256), (7056, 768), (14096, 512)):
        W = gen_x(N, K, torch.bfloat16, seed=N, std=0.02)
        codes, e8 = orc.quantize_mxfp4_weights(to_np(W))
        layer = helper.A4W4_MXFP_dynamic(device=device, dtype=dtype).from_weights(
            torch.from_numpy(codes), scales=torch.from_numpy(e8), bias=gen_x(1, N, dtype, seed=1).reshape(-1) if N == 520 else None)
        for M in (3, 5, 16, 17, 32, 33):
            x = gen_x(M, K, dtype, seed=70 + M).to(device)
            xq, sx = gemlite_amd.scale_activations_mxfp4(x)
            m = layer.get_meta_args()
            out = torch.empty(M, N, dtype=dtype, device=device)
            a = _ext.build_matmul_args(xq, layer.W_q, layer.scales, layer.zeros, sx, out, W_nbits=m[1], group_size=m[2],
                                       unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                       acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                       data_contiguous=m[11])
            if M == 33:
                assert _ext.matmul_family(a) == "GEMM_MXFP4"
            else:
                assert _ext.matmul_family(a) == "K_SKINNY", (N, K, M, _ext.matmul_family(a))
            check_layer(layer, x, dtype)


# ------------------------------------------------------------------ MXFP4
@pytest.mark.parametrize("M", [1, 3, 32, 100, 128])
def test_a4w4_mxfp4(device, M):
    N, K = 512, 4224  # K of the reference's MX tests (reference: tests/test_mxfp.py:31)
    W = gen_x(N, K, torch.bfloat16, seed=6, std=0.02)
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.bfloat16)
    lin.weight.data = W
    layer = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_linear(lin.to(device))
    assert (layer.W_group_mode, layer.channel_scale_mode) == (0, 4)
    codes_ref, e_ref = orc.quantize_mxfp4_weights(to_np(W))
    assert np.array_equal(orc.unpack_fp4_bytes(layer.W_q.t().contiguous().cpu().numpy()), codes_ref)
    assert np.array_equal(layer.scales.contiguous().cpu().numpy(), e_ref)
    x = gen_x(M, K, torch.bfloat16, seed=M)
    check_layer(layer, x.to(device), torch.bfloat16, types=["GEMM", "GEMM_SPLITK"])
    # and close to the unquantised product (format error only)
    y = to_np(layer(x.to(device)))
    y_fp = to_np(x) @ to_np(W).T
    assert rel_frob(y, y_fp) < 0.2


@pytest.mark.parametrize("M", [64, 300])
def test_a4w4_mxfp4_wide(device, M):
    # K a multiple of the full 256-value step, N across several column tiles with a ragged last one
    N, K = 1352, 2048
    W = gen_x(N, K, torch.float16, seed=8, std=0.02)
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.float16)
    lin.weight.data = W
    layer = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.float16).from_linear(lin.to(device))
    assert layer.scales.stride() == (K // 32, 1)
    check_layer(layer, gen_x(M, K, torch.float16, seed=M).to(device), torch.float16, types=["GEMM"])


@pytest.mark.parametrize("K", [1056, 2240])
def test_int8_ragged_k_bit_exact(device, K):
    # K that is a multiple of 32 but not of the 128-byte pipeline step
    N = 300
    g = torch.Generator().manual_seed(K)
    W = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    layer = GemLiteLinear(8, None, K, N, DType.INT8, DType.INT32).pack(W.to(device), None, None)
    for M in (40, 130, 260):
        x = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int32).to(torch.int8)
        ref = (x.long() @ W.long().t()).numpy()
        y = layer.forward_manual(x.to(device), matmul_type="GEMM")
        assert np.array_equal(y.cpu().numpy(), ref), M


def test_fp8_ragged_k(device):
    N, K = 520, 2112  # 16.5 pipeline steps
    W = gen_x(N, K, torch.bfloat16, seed=11, std=0.02)
    W_q, s = gemlite_amd.quantize_weights_per_channel(W, torch.float8_e4m3fn)
    proc = helper.A8W8_FP8_dynamic(device=device)
    proc.dtype = torch.bfloat16
    layer = proc.from_weights(W_q, scales=s)
    for M in (70, 200):
        check_layer(layer, gen_x(M, K, torch.bfloat16, seed=M).to(device), torch.bfloat16, types=["GEMM"])


def test_tuner_fills_the_config_cache_and_results_stay_correct(device):
    from gemlite_amd import tune
    GemLiteLinear.reset_config()
    N, K = 1024, 4096
    W_q, scales, zeros = gen_int_case(N, K, 4, 128, torch.float16, seed=21)
    layer = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
    res = tune.tune_layer(layer, [1, 200], reps=5, min_gain=0.0)
    assert set(res) == {1, 200} and res[1][2] == "GEMV_PACKED" and res[200][2] == "GEMM_WN"
    for M in (1, 200):  # whatever tile won is now used by forward(), and the output is still right
        check_layer(layer, gen_x(M, K, torch.float16, seed=M).to(device), torch.float16, types=[])
    GemLiteLinear.reset_config()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype_id,flop_per_mfma", [(1, 2 * 32 * 32 * 16), (2, 2 * 32 * 32 * 16), (3, 2 * 32 * 32 * 64),
                                                   (4, 2 * 32 * 32 * 32), (17, 2 * 32 * 32 * 64)])
def test_mfma_probe_runs_and_reports_its_flops(device, dtype_id, flop_per_mfma):
    """The diagnostic MFMA loop launches for every matrix format, reports the flops of the launch
    (2 workgroups of 4 waves per CU, 8 MFMAs per iteration) and leaves its sink untouched."""
    import ctypes
    from gemlite_amd import _ext
    lib = _ext.load_library()
    sink = torch.zeros(1, dtype=torch.float32, device=device)
    flops = ctypes.c_double(0.0)
    for rnd in (0, 1):
        rc = lib.gla_probe_mfma(dtype_id, rnd, 50, sink.data_ptr(), ctypes.byref(flops), torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.gla_last_error().decode()
    torch.cuda.synchronize()
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    assert flops.value == cus * 2 * 4 * 50 * 8 * flop_per_mfma
    assert sink.item() == 0.0
    assert lib.gla_probe_mfma(0, 0, 50, sink.data_ptr(), None, None) == -2   # fp32: no such loop
    assert lib.gla_probe_mfma(1, 0, 0, sink.data_ptr(), None, None) == -1


@pytest.mark.gpu
@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("post_scale", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("K", [2080, 2112])   # 2112 = 33 x 64: the matrix-core variant (3..16 rows); 2080: the vector one
def test_a16w8_weight_only_unpacked_bytes(device, fp8, post_scale, dtype, K):
    """fp16/bf16 activations x int8 / fp8 weights kept as bytes, one scale per channel
    (reference processor: gemlite/helper.py:89-171, 336-342).  Up to 16 rows the K-major streaming
    kernel runs; the codes are the oracle's."""
    from gemlite_amd import _ext
    N = 1028                              # K % 32 == 0 as the module requires; neither a multiple of the kernels' tiles
    W = gen_x(N, K, dtype, seed=21, std=0.02)
    proc = (helper.A16W8_FP8 if fp8 else helper.A16W8_INT8)(device=device, post_scale=post_scale)
    # weights are quantised once on the host (CPU torch), then handed over pre-quantised
    W_q_cpu, s_cpu = gemlite_amd.quantize_weights_per_channel(W, torch.float8_e4m3fn if fp8 else torch.int8)
    proc.dtype = dtype
    layer = proc.from_weights(W_q_cpu, scales=s_cpu)
    assert (layer.W_group_mode, layer.channel_scale_mode) == ((0, 1) if post_scale else (2, 0))
    assert layer.W_q.stride() == (1, K) and layer.W_q.dtype == (torch.float8_e4m3fn if fp8 else torch.int8)
    q_ref, s_ref = orc.quantize_per_channel(to_np(W), not fp8)
    got = layer.W_q.t().contiguous()
    got = got.view(torch.uint8).cpu().numpy() if fp8 else got.cpu().numpy()
    assert np.array_equal(got, q_ref)
    for M in (1, 2, 3, 8, 16):
        x = gen_x(M, K, dtype, seed=M).to(device)
        out = torch.empty((M, N), dtype=dtype, device=device)
        m = layer.get_meta_args()
        args = _ext.build_matmul_args(x, layer.W_q, layer.scales, layer.zeros, None, out, W_nbits=m[1], group_size=m[2],
                                      unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                      acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                      data_contiguous=m[11])
        assert _ext.matmul_family(args) == "GEMV_KMAJOR"
        check_layer(layer, x, dtype)
    # above 16 rows: the MFMA GEMM for weight bytes where K is a multiple of its 64-value stage, else the generic kernel
    for M in (17, 40, 100, 130, 300):
        x = gen_x(M, K, dtype, seed=M).to(device)
        out = torch.empty((M, N), dtype=dtype, device=device)
        m = layer.get_meta_args()
        args = _ext.build_matmul_args(x, layer.W_q, layer.scales, layer.zeros, None, out, W_nbits=m[1], group_size=m[2],
                                      unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                      acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                      data_contiguous=m[11])
        assert _ext.matmul_family(args) == ("GEMM_KBYTES" if K % 64 == 0 else "GENERIC")
        check_layer(layer, x, dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("post_scale", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_byte_weights_at_prefill_size_are_converted_first(device, fp8, post_scale, dtype):
    """From 2048 rows (or on request) unpacked int8 / fp8 weight bytes are written out once as fp16 / bf16 values (exact)
    and the 16-bit GEMM runs on them with the per-channel scale in its epilogue, as the byte-weight GEMM has it.  N is
    no multiple of the kernels' tiles; one-hot rows: bit-identical outputs of both paths."""
    N, K = 1028, 2112
    W = gen_x(N, K, dtype, seed=21, std=0.02)
    proc = (helper.A16W8_FP8 if fp8 else helper.A16W8_INT8)(device=device, post_scale=post_scale)
    W_q_cpu, s_cpu = gemlite_amd.quantize_weights_per_channel(W, torch.float8_e4m3fn if fp8 else torch.int8)
    proc.dtype = dtype
    layer = proc.from_weights(W_q_cpu, scales=s_cpu)
    m = layer.get_meta_args()

    def run(x, tile):
        out = torch.empty((x.shape[0], N), dtype=dtype, device=device)
        a = _ext.build_matmul_args(x, layer.W_q, layer.scales, layer.zeros, None, out, W_nbits=m[1], group_size=m[2],
                                   unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                   acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                   data_contiguous=m[11], tile_config=tile)
        fam = _ext.matmul_family(a)
        print(f"case: {fam} tile={tile} M={x.shape[0]} N={N} K={K} fp8={fp8} post_scale={post_scale} {dtype}", flush=True)
        _ext.matmul(a, device)
        torch.cuda.synchronize()
        return fam, out

    for M, tile in ((40, -5), (300, -5), (2048, -1)):
        x = gen_x(M, K, dtype, seed=M)
        y_ref = oracle_forward(layer, x)
        fam, out = run(x.to(device), tile)
        assert fam == "GEMM_16BIT", (M, tile, fam)
        err = rel_frob(to_np(out), y_ref)
        assert err <= TIGHT[dtype], (M, err)
        assert elementwise_excess(to_np(out), y_ref, kind_of(dtype)) <= 1.0, M
    x = torch.zeros(48, K, dtype=dtype)
    for r in range(48):
        x[r, (53 * r + 11) % K] = 1.0
    (fa, ya), (fb, yb) = run(x.to(device), -3), run(x.to(device), -5)
    assert (fa, fb) == ("GEMM_KBYTES", "GEMM_16BIT")
    assert torch.equal(ya, yb)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("zeros_kind", ["tensor_fma", "tensor_shift_scale", "scalar"])
def test_int8_bytes_with_zero_point_channelwise(device, dtype, zeros_kind):
    """Unpacked int8 codes with a per-channel scale and a zero point: the K-major streaming kernels
    fold the zero point into s (D - z X) / s D + z' X after the K sum."""
    from gemlite_amd import _ext
    N, K = 520, 2112
    g = torch.Generator().manual_seed(3)
    W_q = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int32).to(torch.int8)
    scales = (torch.rand((N, 1), generator=g) * 0.02 + 0.005).to(dtype)
    if zeros_kind == "scalar":
        zeros, fma = 3, True
    else:
        zeros, fma = (torch.rand((N, 1), generator=g) * 8 - 4).to(dtype).to(device), zeros_kind == "tensor_fma"
    dt = DType.FP16 if dtype == torch.float16 else DType.BF16
    layer = GemLiteLinear(8, K, K, N, dt, dt).pack(W_q.to(device), scales.to(device), zeros, fma_mode=fma)
    assert layer.W_q.dtype == torch.int8 and layer.W_q.stride() == (1, K)
    for M in (1, 2, 5, 16):
        x = gen_x(M, K, dtype, seed=M).to(device)
        out = torch.empty((M, N), dtype=dtype, device=device)
        m = layer.get_meta_args()
        args = _ext.build_matmul_args(x, layer.W_q, layer.scales, layer.zeros, None, out, W_nbits=m[1], group_size=m[2],
                                      unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                      acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                      data_contiguous=m[11])
        assert _ext.matmul_family(args) == "GEMV_KMAJOR", (layer.W_group_mode, layer.channel_scale_mode)
        check_layer(layer, x, dtype)


@pytest.mark.gpu
def test_kernel_plugin_classes_match_the_module(device):
    """Calling a registry class's forward with the module's tensor / meta arguments gives what the
    module gives (the seam a maintainer of the reference would plug the library into)."""
    N, K = 512, 1024
    W_q, scales, zeros = gen_int_case(N, K, 4, 128, torch.float16)
    layer = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
    W, s, z, _ = layer.get_tensor_args()
    m = layer.get_meta_args()
    for M, name in ((1, "GEMV_REVSPLITK"), (8, "GEMM_SPLITK"), (64, "GEMM")):
        x = gen_x(M, K, torch.float16, seed=M).to(device)
        y = gemlite_amd.GEMLITE_TRITON_MAPPING[name].forward(x, W, s, z, None, *m[1:], type_id=0)
        assert torch.equal(y, layer.forward_manual(x, matmul_type=name))


@pytest.mark.gpu
@pytest.mark.parametrize("group_size", [128, None])
def test_a8w4_hqq_int_dynamic_fp8_activations(device, group_size):
    """fp8 activations quantised per token x 4-bit grouped weights (reference processor:
    gemlite/helper.py:712-851; modes as tests/test_int.py:173-199 asserts them)."""
    N, K = 256, 1024
    gs = group_size or K
    W_q, scales, zeros = gen_int_case(N, K, 4, gs, torch.float16)
    layer = helper.A8W4_HQQ_INT_dynamic(device=device).from_weights(W_q, scales, zeros)
    assert layer.scaled_activations and layer.input_dtype == DType.FP8
    if group_size is None:
        assert (layer.W_group_mode, layer.channel_scale_mode) == (1, 3)
    else:
        assert (layer.W_group_mode, layer.channel_scale_mode) == (3, 2)
    for M in (1, 7, 40):
        check_layer(layer, gen_x(M, K, torch.float16, seed=M).to(device), torch.bfloat16)


@pytest.mark.gpu
def test_a8w2_hqq_int_dynamic_groups_of_32_widened_onto_the_mid_batch_kernel(device):
    """fp8 activations quantised per token x 2-bit codes in groups of 32 (A8W2_HQQ_INT_dynamic): the activations are
    widened to fp16 in the workspace and the packed-code kernel that takes groups of 32 runs on them, the mid-batch
    one at every row count, per-token scales in its epilogue or split-K finishing launch."""
    N, K = 520, 2048
    W_q, scales, zeros = gen_int_case(N, K, 2, 32, torch.float16, seed=77)
    layer = helper.A8W2_HQQ_INT_dynamic(device=device).from_weights(W_q, scales, zeros)
    assert layer.scaled_activations and layer.input_dtype == DType.FP8 and layer.group_size == 32
    m = layer.get_meta_args()
    for M in (1, 7, 40, 100):
        x = gen_x(M, K, torch.float16, seed=M).to(device)
        xq, sx = gemlite_amd.scale_activations_per_token(x, torch.float8_e4m3fn)
        out = torch.empty(M, N, dtype=gemlite_amd.DTYPE_TO_TORCH[m[6]], device=device)
        a = _ext.build_matmul_args(xq, layer.W_q, layer.scales, layer.zeros, sx, out, W_nbits=m[1], group_size=m[2],
                                   unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                   acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                   data_contiguous=m[11])
        assert _ext.matmul_family(a) == "WN_MID", (M, _ext.matmul_family(a))
        check_layer(layer, x, torch.bfloat16)


@pytest.mark.gpu
@pytest.mark.parametrize("K", [384, 1024])
def test_a8w8_mxfp8_weights_per_token_activations(device, K):
    """MXFP8 weights x fp8 activations quantised per token, scale applied after the K sum
    (reference processor: gemlite/helper.py:876-923, its default post_scale=True)."""
    from gemlite_amd import _ext
    N = 520
    W = gen_x(N, K, torch.bfloat16, seed=31, std=0.03)
    W[7, 64:96] = 0.0
    codes, e8 = orc.quantize_mxfp8_weights(to_np(W))
    layer = helper.A8W8_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_weights(
        torch.from_numpy(codes).view(torch.float8_e4m3fn), scales=torch.from_numpy(e8))
    assert (layer.W_group_mode, layer.channel_scale_mode) == (0, 2)
    for M in (1, 5, 33, 64, 100, 130, 300):
        check_layer(layer, gen_x(M, K, torch.bfloat16, seed=M).to(device), torch.bfloat16)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("M", [1, 31, 64, 100])
def test_mxfp8_activation_quantizer_bit_exact(device, dtype, M):
    K = 1024
    x = gen_x(M, K, dtype, seed=M + 3)
    x[0, 32:64] = 0.0
    if M > 2:
        x[2, 0] = 448.0
        x[2, 1:32] = 0.25
    codes, e8 = gemlite_amd.scale_activations_mxfp8(x.to(device))
    want_codes, want_e8 = orc.scale_activations_mxfp8(to_np(x))
    assert codes.dtype == torch.float8_e4m3fn and e8.shape == ((M + 31) // 32 * 32, K // 32)
    assert np.array_equal(codes.view(torch.uint8).cpu().numpy(), want_codes)
    assert np.array_equal(e8.cpu().numpy(), want_e8)


@pytest.mark.gpu
def test_a8w8_mxfp8_block_scaled_both_sides(device):
    """MXFP8 x MXFP8 with micro-scales on the activations too (post_scale=False,
    channel_scale_mode 4; reference: gemlite/helper.py:917-919)."""
    N, K = 520, 1024
    W = gen_x(N, K, torch.bfloat16, seed=41, std=0.03)
    codes, e8 = orc.quantize_mxfp8_weights(to_np(W))
    layer = helper.A8W8_MXFP_dynamic(device=device, dtype=torch.bfloat16, post_scale=False).from_weights(
        torch.from_numpy(codes).view(torch.float8_e4m3fn), scales=torch.from_numpy(e8))
    assert (layer.W_group_mode, layer.channel_scale_mode) == (0, 4)
    for M in (1, 5, 33, 100, 130, 300):
        check_layer(layer, gen_x(M, K, torch.bfloat16, seed=M).to(device), torch.bfloat16)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("W_nbits", [8, 4])
def test_weight_only_mxfp_layers(device, dtype, W_nbits):
    """fp16 / bf16 activations x MXFP8 / MXFP4 weights (reference processors A16W8_MXFP / A16W4_MXFP,
    gemlite/helper.py:384-420), on the reference tests' ragged shapes (N=2032, K=3968 = 124 blocks)."""
    N, K = 2032, 3968
    W = gen_x(N, K, torch.bfloat16, seed=51, std=0.03)
    W[5, 32:64] = 0.0
    lin = torch.nn.Linear(K, N, bias=True, dtype=dtype)
    lin.weight.data = W.to(dtype)
    lin.bias.data = gen_x(1, N, dtype, seed=52).reshape(-1)
    cls = helper.A16W8_MXFP if W_nbits == 8 else helper.A16W4_MXFP
    layer = cls(device=device, dtype=dtype).from_linear(lin.to(device))
    want = orc.quantize_mxfp8_weights(to_np(W.to(dtype))) if W_nbits == 8 else orc.quantize_mxfp4_weights(to_np(W.to(dtype)))
    assert np.array_equal(layer.scales.cpu().numpy(), want[1])
    # streaming kernel up to 2 rows; 3..16 rows: weights straight into registers and to the matrix cores;
    # above, the tiled matrix-core kernel (64-, 128- and 256-row tiles, split K)
    for M in (1, 2, 3, 4, 5, 7, 11, 16, 17, 33, 70, 130, 300):
        check_layer(layer, gen_x(M, K, dtype, seed=M).to(device), dtype, types=["GEMV", "GEMM_SPLITK", "GEMM"])
    # a one-hot activation row picks out one dequantised weight column exactly
    x = torch.zeros(1, K, dtype=dtype)
    x[0, 37] = 1.0
    layer.bias = None
    y = layer(x.to(device))
    torch.cuda.synchronize()
    y_ref = oracle_forward(layer, x)
    assert np.array_equal(to_np(y), round_like(y_ref, dtype))
    # ... and through the matrix-core kernels (13 rows: the skinny one, 40: the tiled one): row r of the batch is
    # one-hot at a position of its own
    for rows in (13, 40):
        x = torch.zeros(rows, K, dtype=dtype)
        for r in range(rows):
            x[r, (97 * r + 5) % K] = 1.0
        y = layer(x.to(device))
        torch.cuda.synchronize()
        assert np.array_equal(to_np(y), round_like(oracle_forward(layer, x), dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("W_nbits", [8, 4])
def test_weight_only_mxfp_skinny_kernel_on_wide_layers(device, W_nbits):
    """3..16 rows on layers wide enough for two and four 16-row tiles per wave (N = 16400 leaves the last
    workgroup a ragged tile; K = 2560 ends inside the second chunk of activations)."""
    N, K = 16400, 2560
    dtype = torch.bfloat16
    lin = torch.nn.Linear(K, N, bias=True, dtype=dtype)
    lin.weight.data = gen_x(N, K, torch.bfloat16, seed=57, std=0.03)
    lin.weight.data[:, 64:96] *= 16.0   # block scales that differ along K
    lin.bias.data = gen_x(1, N, dtype, seed=58).reshape(-1)
    cls = helper.A16W8_MXFP if W_nbits == 8 else helper.A16W4_MXFP
    layer = cls(device=device, dtype=dtype).from_linear(lin.to(device))
    for M in (3, 9, 16):
        check_layer(layer, gen_x(M, K, dtype, seed=M).to(device), dtype, types=["GEMM"])
    x = torch.zeros(11, K, dtype=dtype)
    for r in range(11):
        x[r, (211 * r + 7) % K] = 1.0
    layer.bias = None
    y = layer(x.to(device))
    torch.cuda.synchronize()
    assert np.array_equal(to_np(y), round_like(oracle_forward(layer, x), dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("W_nbits", [8, 4])
def test_weight_only_mxfp_batches_as_sums_of_e4m3_terms(device, dtype, W_nbits):
    """3..16 rows (fp16: 10) of 16-bit activations on MX weights through the skinny kernel of the narrow formats: a launch
    in front writes every activation as two (fp16: three) e4m3 terms with block scales of their own, the scaled MFMA
    multiplies them with the weights as they are, the epilogue adds a row's terms.  Forced with the preference on a
    small ragged layer (N = 2032 ends inside a 16-row weight tile; one and two activation tiles, a last tile with one
    row; a bias), activations whose blocks differ by 2^12 in magnitude, a block of zeros, fp16 values down to the
    subnormals; then one-hot rows, which must come out exactly; then a layer large enough to take the path unasked."""
    N, K = 2032, 3840
    W = gen_x(N, K, torch.bfloat16, seed=71, std=0.03)
    W[:, 64:96] *= 16.0
    W[7, 128:160] = 0.0
    lin = torch.nn.Linear(K, N, bias=True, dtype=dtype)
    lin.weight.data = W.to(dtype)
    lin.bias.data = gen_x(1, N, dtype, seed=72).reshape(-1)
    cls = helper.A16W8_MXFP if W_nbits == 8 else helper.A16W4_MXFP
    layer = cls(device=device, dtype=dtype).from_linear(lin.to(device))
    m = layer.get_meta_args()

    def run(x, bias):
        out = torch.empty(x.shape[0], N, dtype=dtype, device=device)
        a = _ext.build_matmul_args(x, layer.W_q, layer.scales, layer.zeros, None, out, W_nbits=m[1], group_size=m[2],
                                   unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                   acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                   data_contiguous=m[11], tile_config=-4, bias=bias)
        assert _ext.matmul_family(a) == "K_SKINNY", (x.shape[0], _ext.matmul_family(a))
        print(f"case: K_SKINNY on e4m3 terms M={x.shape[0]} N={N} K={K} W{W_nbits} {dtype}", flush=True)
        _ext.matmul(a, device)
        torch.cuda.synchronize()
        return out

    rows = (3, 5, 8, 9, 16) if dtype == torch.bfloat16 else (3, 5, 6, 10)
    for M in rows:
        x = gen_x(M, K, dtype, seed=M)
        x[:, 96:160] *= 64.0
        x[:, 160:192] /= 64.0
        x[0, 256:288] = 0.0
        if dtype == torch.float16:
            x[1, 320:352] *= 2.0 ** -14      # down to fp16 subnormals
        y_ref = oracle_forward(layer, x)
        y = to_np(run(x.to(device), layer.bias))
        err = rel_frob(y, y_ref)
        assert err <= TIGHT[dtype], (M, err)
        assert elementwise_excess(y, y_ref, kind_of(dtype)) <= 1.0, M
    # one-hot rows pick single dequantised weights: exact, whatever the position inside its block and the row's slot
    layer_bias, layer.bias = layer.bias, None
    for M in rows[-2:]:
        x = torch.zeros(M, K, dtype=dtype)
        for r in range(M):
            x[r, (97 * r + 5) % K] = 1.0 if r % 2 == 0 else -0.375
        assert np.array_equal(to_np(run(x.to(device), None)), round_like(oracle_forward(layer, x), dtype))
    layer.bias = layer_bias
    # a wide layer (881 tiles of 16 weight rows, the last one ragged): four weight tiles per wave against two activation tiles
    if dtype == torch.bfloat16:
        N3, K3 = 14088, 512
        lin3 = torch.nn.Linear(K3, N3, bias=False, dtype=dtype)
        lin3.weight.data = gen_x(N3, K3, torch.bfloat16, seed=75, std=0.03).to(dtype)
        wide = cls(device=device, dtype=dtype).from_linear(lin3.to(device))
        m3 = wide.get_meta_args()
        for M in (7, 13):
            x = gen_x(M, K3, dtype, seed=M + 40)
            out = torch.empty(M, N3, dtype=dtype, device=device)
            a = _ext.build_matmul_args(x.to(device), wide.W_q, wide.scales, wide.zeros, None, out, W_nbits=m3[1], group_size=m3[2],
                                       unpack_mask=m3[3], elements_per_sample=m3[4], input_dtype=m3[5], output_dtype=m3[6],
                                       acc_dtype=m3[7], meta_dtype=m3[8], channel_scale_mode=m3[9], W_group_mode=m3[10],
                                       data_contiguous=m3[11], tile_config=-4)
            assert _ext.matmul_family(a) == "K_SKINNY"
            print(f"case: K_SKINNY on e4m3 terms M={M} N={N3} K={K3} W{W_nbits} {dtype}", flush=True)
            _ext.matmul(a, device)
            torch.cuda.synchronize()
            y_ref = oracle_forward(wide, x)
            assert rel_frob(to_np(out), y_ref) <= TIGHT[dtype], M
            assert elementwise_excess(to_np(out), y_ref, kind_of(dtype)) <= 1.0, M
    # unasked: a long-K layer at 8 rows (MXFP4: 58.7 M weights; MXFP8: K >= 8192 and N <= 8192)
    N2, K2 = 4096, 14336
    lin2 = torch.nn.Linear(K2, N2, bias=False, dtype=dtype, device=device)
    lin2.weight.data = gen_x(N2, K2, torch.bfloat16, seed=73, std=0.02).to(dtype).to(device)
    big = cls(device=device, dtype=dtype).from_linear(lin2)
    M = 8 if dtype == torch.bfloat16 else 5
    x = gen_x(M, K2, dtype, seed=74).to(device)
    m2 = big.get_meta_args()
    a = _ext.build_matmul_args(x, big.W_q, big.scales, big.zeros, None, torch.empty(M, N2, dtype=dtype, device=device), W_nbits=m2[1],
                               group_size=m2[2], unpack_mask=m2[3], elements_per_sample=m2[4], input_dtype=m2[5], output_dtype=m2[6],
                               acc_dtype=m2[7], meta_dtype=m2[8], channel_scale_mode=m2[9], W_group_mode=m2[10], data_contiguous=m2[11])
    assert _ext.matmul_family(a) == "K_SKINNY"
    check_layer(big, x, dtype, types=["GEMM"])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("W_nbits", [8, 4])
def test_weight_only_mxfp_layers_k_not_a_multiple_of_128(device, dtype, W_nbits):
    """K = 1056 (33 blocks): every batch size stays on the streaming kernel."""
    N, K = 264, 1056
    lin = torch.nn.Linear(K, N, bias=False, dtype=dtype)
    lin.weight.data = gen_x(N, K, torch.bfloat16, seed=53, std=0.03).to(dtype)
    cls = helper.A16W8_MXFP if W_nbits == 8 else helper.A16W4_MXFP
    layer = cls(device=device, dtype=dtype).from_linear(lin.to(device))
    for M in (1, 6, 9, 40):
        check_layer(layer, gen_x(M, K, dtype, seed=M).to(device), dtype, types=["GEMM_SPLITK", "GEMM"])


@pytest.mark.gpu
@pytest.mark.parametrize("post_scale", [True, False])
@pytest.mark.parametrize("K", [1056, 1024, 2432])
def test_a8w4_mxfp8_activations_mxfp4_weights(device, post_scale, K):
    """MXFP8 activations (per token, or with micro-scales) x MXFP4 weights
    (reference processor A8W4_MXFP_dynamic, gemlite/helper.py:950-1040).  K = 1056 is 33 blocks, not a
    multiple of the 128 the matrix-core kernel wants, and streams; the others run the mixed fp8 x fp4 MFMA
    (K = 2432 is 19 words of scales: an odd number of stage pairs)."""
    N = 520
    W = gen_x(N, K, torch.bfloat16, seed=61, std=0.03)
    W[:, 32:64] *= 8.0     # block scales that differ from block to block
    W[:, 96:128] *= 0.125
    codes, e8 = orc.quantize_mxfp4_weights(to_np(W))
    layer = helper.A8W4_MXFP_dynamic(device=device, dtype=torch.bfloat16, post_scale=post_scale).from_weights(
        torch.from_numpy(codes), scales=torch.from_numpy(e8))
    assert (layer.W_group_mode, layer.channel_scale_mode) == (0, 2 if post_scale else 4)
    for M in (1, 2, 3, 5, 33, 70, 130, 300):
        x = gen_x(M, K, torch.bfloat16, seed=M)
        x[:, 64:96] *= 16.0
        check_layer(layer, x.to(device), torch.bfloat16, types=["GEMM_SPLITK", "GEMM"])


@pytest.mark.gpu
@pytest.mark.parametrize("post_scale", [True, False])
@pytest.mark.parametrize("w4", [False, True])
def test_fp8_activations_on_mx_weights_decode_batches_in_one_launch(device, post_scale, w4):
    """fp8 activations (one scale per token, or MXFP8 micro-scales) x MXFP8 / MXFP4 weights at 3..32 rows: both
    operands copied to LDS by lines and fed to the scaled MFMA as they are (the mixed fp8 x fp4 form for MXFP4
    weights, whose activation rows are two tiles a turn).  Ragged N, few and many turns of K, block scales that
    differ from block to block, every launch shape, a bias."""
    from gemlite_amd import _ext
    proc = helper.A8W4_MXFP_dynamic if w4 else helper.A8W8_MXFP_dynamic
    for (N, K) in ((1040, 4096), (520, 2304), (72, 256), (7056, 768), (14096, 512)):
        W = gen_x(N, K, torch.bfloat16, seed=N + 2, std=0.03)
        W[:, 32:64] *= 8.0
        W[:, 96:128] *= 0.125
        if w4:
            codes, e8 = orc.quantize_mxfp4_weights(to_np(W))
            wq = torch.from_numpy(codes)
        else:
            codes, e8 = orc.quantize_mxfp8_weights(to_np(W))
            wq = torch.from_numpy(codes).view(torch.float8_e4m3fn)
        layer = proc(device=device, dtype=torch.bfloat16, post_scale=post_scale).from_weights(
            wq, scales=torch.from_numpy(e8), bias=gen_x(1, N, torch.bfloat16, seed=3).reshape(-1) if N == 520 else None)
        for M in (3, 5, 16, 17, 32, 33):
            x = gen_x(M, K, torch.bfloat16, seed=90 + M)
            x[:, 64:96] *= 16.0
            x = x.to(device)
            if post_scale:
                xq, sx = gemlite_amd.scale_activations_per_token(x, torch.float8_e4m3fn)
            else:
                xq, sx = gemlite_amd.scale_activations_mxfp8(x)
            m = layer.get_meta_args()
            out = torch.empty(M, N, dtype=torch.bfloat16, device=device)
            a = _ext.build_matmul_args(xq, layer.W_q, layer.scales, layer.zeros, sx, out, W_nbits=m[1], group_size=m[2],
                                       unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                       acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                       data_contiguous=m[11])
            ring = M <= 16 or (M <= 32 and N < 7040)
            assert _ext.matmul_family(a) == ("K_SKINNY" if ring else "GEMM_MXFP8"), (N, K, M, _ext.matmul_family(a))
            check_layer(layer, x, torch.bfloat16, types=["GEMM_SPLITK", "GEMM"])


@pytest.mark.gpu
def test_mxfp4_with_k_not_a_multiple_of_128_streams(device):
    """MXFP4 x MXFP4 at K = 96, 160: three and five 32-blocks (the matrix-core kernel needs K % 128 == 0)."""
    for K in (96, 160):
        N = 72
        W = gen_x(N, K, torch.bfloat16, seed=K, std=0.03)
        codes, e8 = orc.quantize_mxfp4_weights(to_np(W))
        layer = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_weights(
            torch.from_numpy(codes), scales=torch.from_numpy(e8))
        for M in (1, 6, 40):
            check_layer(layer, gen_x(M, K, torch.bfloat16, seed=M).to(device), torch.bfloat16, types=["GEMM_SPLITK", "GEMM"])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("to_int8", [True, False])
def test_per_block_activation_quantizer_bit_exact(device, dtype, to_int8):
    M, K = 37, 1024
    x = gen_x(M, K, dtype, seed=M)
    x[0, 128:256] = 0.0
    x[3, 0] = 1000.0
    codes, s = gemlite_amd.scale_activations_per_block(x.to(device), torch.int8 if to_int8 else torch.float8_e4m3fn)
    want_codes, want_s = orc.scale_activations_per_block(to_np(x), to_int8)
    assert s.shape == (M, K // 128) and np.array_equal(s.cpu().numpy(), want_s)
    got = codes.cpu().numpy() if to_int8 else codes.view(torch.uint8).cpu().numpy()
    assert np.array_equal(got, want_codes)


@pytest.mark.gpu
@pytest.mark.parametrize("to_int8", [True, False])
def test_a8w8_block_quantised(device, to_int8):
    """128 x 128 block-quantised int8 / fp8 layers (reference: gemlite/helper.py:517-617), N not a
    multiple of 128 or of the kernel's 16 columns per workgroup."""
    N, K = 2032 + 5, 1152
    W = gen_x(N, K, torch.bfloat16, seed=71, std=0.02)
    proc = helper.A8W8_INT8_dynamic if to_int8 else helper.A8W8_FP8_dynamic
    layer = proc(device=device, block_quant=True).from_weights(W, bias=gen_x(1, N, torch.bfloat16, seed=3).reshape(-1))
    assert (layer.W_group_mode, layer.channel_scale_mode) == (0, 5)
    codes, s = orc.quantize_block_weights(to_np(W), to_int8)
    # the one-time weight quantiser is torch code: its fp32 division on the GPU may differ from the CPU's in the
    # last place (the CPU test compares it exactly); the matmul is checked against the layer's own tensors
    assert np.allclose(layer.scales.cpu().numpy(), s.T, rtol=1e-6, atol=0)
    for M in (1, 2, 3, 4, 5, 8, 16, 21, 64, 100, 130, 300):   # streaming kernel up to 4 rows, MFMA GEMM above
        check_layer(layer, gen_x(M, K, torch.bfloat16, seed=M).to(device), torch.bfloat16, types=["GEMM_SPLITK", "GEMM"])


@pytest.mark.gpu
@pytest.mark.parametrize("to_int8", [True, False])
@pytest.mark.parametrize("K", [2176, 4096])
def test_a8w8_block_quantised_split_k(device, to_int8, K):
    """Few output tiles and a long K: the MFMA kernel splits K on whole 128-blocks (K = 2176 is 17
    blocks, split 9 + 8); block scales that differ a lot from block to block make a misplaced scale visible."""
    N = 520
    W = gen_x(N, K, torch.bfloat16, seed=73, std=0.02)
    W[:, 128:256] *= 16.0
    W[:, K - 128:] *= 0.125
    proc = helper.A8W8_INT8_dynamic if to_int8 else helper.A8W8_FP8_dynamic
    layer = proc(device=device, block_quant=True).from_weights(W)
    for M in (24, 70, 200):
        x = gen_x(M, K, torch.bfloat16, seed=M)
        x[:, 256:384] *= 8.0
        check_layer(layer, x.to(device), torch.bfloat16, types=["GEMM"])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_ternary_weight_layers(device, dtype):
    """A16W158_INT and A8W158_INT_dynamic: weights in {-1, 0, 1} as 2-bit codes with a scalar zero
    point of 1 (reference: gemlite/helper.py:1208-1321).  The int8 x ternary sums are exact integers."""
    N, K = 520, 2048
    g = torch.Generator(device="cpu").manual_seed(3)
    W = torch.randint(-1, 2, (N, K), generator=g).to(dtype)
    layer = helper.A16W158_INT(device=device).from_weights(W, torch.tensor(0.037), bias=gen_x(1, N, dtype, seed=5).reshape(-1))
    assert (layer.W_nbits, layer.W_group_mode, layer.channel_scale_mode) == (2, 1, 1)
    for M in (1, 3, 16, 70):
        check_layer(layer, gen_x(M, K, dtype, seed=M).to(device), dtype)
    dyn = helper.A8W158_INT_dynamic(device=device).from_weights(W, torch.tensor(0.037))
    assert (dyn.W_group_mode, dyn.channel_scale_mode, dyn.acc_dtype) == (1, 3, DType.INT32)
    for M in (1, 9, 70):
        x = gen_x(M, K, dtype, seed=M)
        check_layer(dyn, x.to(device), dtype, types=["GEMM_SPLITK", "GEMM"])
    # exact integer check of the accumulation: unit scales on both sides, int8-valued activations
    unit = helper.A8W158_INT_dynamic(device=device).from_weights(W, torch.tensor(1.0))
    unit.output_dtype = DType.FP32
    xi = torch.randint(-127, 128, (5, K), generator=g).to(dtype)
    xi[:, 0] = 127.0   # every row's amax is 127, so the activation scale is exactly 1
    y = unit(xi.to(device))
    torch.cuda.synchronize()
    want = xi.double() @ W.double().T
    assert np.array_equal(to_np(y).astype(np.float64), want.numpy())
    # the same at the extremes (every activation 127, long K) through each kernel the int8 activations are widened
    # for: the streaming kernel at 1, 5 and 20 rows (it folds its offset sums every 64 K-values for an int32
    # accumulator, so that no fp32 sum passes 2^24) and the tiled GEMM at 100 rows
    K2 = 8192
    W2 = torch.randint(-1, 2, (N, K2), generator=g).to(dtype)
    W2[:8] = 1.0
    unit2 = helper.A8W158_INT_dynamic(device=device).from_weights(W2, torch.tensor(1.0))
    unit2.output_dtype = DType.FP32
    for M in (1, 5, 20, 100):
        xa = torch.randint(-127, 128, (M, K2), generator=g).to(dtype)
        xa[0] = 127.0
        xa[:, 0] = 127.0
        y2 = unit2(xa.to(device))
        torch.cuda.synchronize()
        assert np.array_equal(to_np(y2).astype(np.float64), (xa.double() @ W2.double().T).numpy()), M


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_bias_is_added_to_the_rounded_output_like_the_reference(device, dtype):
    """`out += bias` on the output already rounded to its type (reference: gemlite/core.py:271-272): a layer with
    a bias must equal the same layer without one plus the bias, bit for bit, whether the kernel adds it in its
    epilogue or split-K finishing kernel (every family but the byte-weight MFMA GEMM) or the library adds it with a
    launch of its own."""
    N, K = 1032, 2048
    bias = gen_x(1, N, dtype, seed=77).reshape(-1).to(device)
    W_q, s, z = gen_int_case(N, K, 4, 128, dtype, seed=5)
    in_dt = DType.FP16 if dtype == torch.float16 else DType.BF16
    W = gen_x(N, K, torch.bfloat16, seed=6, std=0.02)
    lin = torch.nn.Linear(K, N, bias=False, dtype=dtype)
    lin.weight.data = W.to(dtype)

    def pair(make):
        a, b = make(), make()
        b.bias = torch.nn.Parameter(bias.clone(), requires_grad=False)
        return a, b

    cases = {
        "A16W4": pair(lambda: GemLiteLinear(4, 128, K, N, in_dt, in_dt).pack(W_q.to(device), s.to(device), z.to(device))),
        "A8W8 fp8": pair(lambda: helper.A8W8_FP8_dynamic(device=device).from_weights(W.to(dtype))),
        "A16W4_MXFP": pair(lambda: helper.A16W4_MXFP(device=device, dtype=dtype).from_linear(lin.to(device), del_orig=False)),
        "block-quantised": pair(lambda: helper.A8W8_FP8_dynamic(device=device, block_quant=True).from_weights(W.to(dtype))),
        "A8W8 int8": pair(lambda: helper.A8W8_INT8_dynamic(device=device).from_weights(W.to(dtype))),
        "A4W4 MXFP4": pair(lambda: helper.A4W4_MXFP_dynamic(device=device, dtype=dtype).from_linear(lin.to(device), del_orig=False)),
        "A8W8 MXFP8": pair(lambda: helper.A8W8_MXFP_dynamic(device=device, dtype=dtype).from_linear(lin.to(device), del_orig=False)),
        "A8W4 MXFP": pair(lambda: helper.A8W4_MXFP_dynamic(device=device, dtype=dtype).from_linear(lin.to(device), del_orig=False)),
        "A16W8 bytes": pair(lambda: helper.A16W8_INT8(device=device, dtype=dtype).from_weights(
            *gemlite_amd.quantize_weights_per_channel(W.to(dtype), torch.int8)[:1],
            scales=gemlite_amd.quantize_weights_per_channel(W.to(dtype), torch.int8)[1])),
    }
    for name, (plain, biased) in cases.items():
        for M in (1, 2, 5, 16, 70, 300):   # streaming kernels, split-K with a finishing kernel, 64- / 128- / 256-row tiles
            x = gen_x(M, K, dtype, seed=M).to(device)
            want = plain(x) + bias
            got = biased(x)
            torch.cuda.synchronize()
            assert got.dtype == want.dtype and torch.equal(got, want), (name, M)
    # a bias the library does not take (fp32 bias on an fp16 output is fine; an integer output is not) still works
    y32 = cases["A16W4"][1]
    y32.bias = torch.nn.Parameter(bias.float(), requires_grad=False)
    x = gen_x(3, K, dtype, seed=3).to(device)
    got = y32(x)
    torch.cuda.synchronize()
    assert torch.equal(got, (cases["A16W4"][0](x).float() + bias.float()).to(dtype))
