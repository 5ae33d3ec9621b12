"""`gla_matmul_static` (the entry point that takes its scratch from a device array inside the
library instead of a caller's workspace) against `gla_matmul`, through the C ABI: the same kernels
run, so the outputs must be identical bit for bit.  Each case makes two calls in a row, the second
on a smaller problem, so the second call finds the first one's partials, counters and regrouped
scales in the shared array."""
import ctypes

import numpy as np
import pytest
import torch

import gemlite_amd
from gemlite_amd import DType, GemLiteLinear, _ext, helper
from oracle import oracle as orc
from parity import gen_int_case, gen_x, oracle_forward, rel_frob, to_np

pytestmark = pytest.mark.gpu


def _args(layer, x, scales_x, out):
    m = layer.get_meta_args()
    in_dt = m[5]
    if scales_x is None and not gemlite_amd.dtypes.is_mx_dtype(in_dt):
        in_dt = gemlite_amd.TORCH_TO_DTYPE[x.dtype].value
    return _ext.build_matmul_args(
        x, layer.W_q, layer.scales, layer.zeros, scales_x, out,
        W_nbits=m[1], group_size=m[2], unpack_mask=m[3], elements_per_sample=m[4], input_dtype=in_dt,
        output_dtype=m[6], acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
        data_contiguous=m[11])


def _both(layer, x, scales_x, N, out_dtype, device):
    """(output of gla_matmul with a workspace, output of gla_matmul_static, scratch bytes the problem needs)."""
    lib = _ext.load_library()
    stream = torch.cuda.current_stream().cuda_stream
    out_a = torch.full((x.shape[0], N), float("nan"), dtype=out_dtype, device=device)
    out_b = torch.full((x.shape[0], N), float("nan"), dtype=out_dtype, device=device)
    a = _args(layer, x, scales_x, out_a)
    need = _ext.matmul_workspace_need(a)
    _ext.matmul(a, device)
    b = _args(layer, x, scales_x, out_b)
    b.workspace, b.workspace_bytes = None, 0          # ignored by the entry point under test
    rc = lib.gla_matmul_static(ctypes.byref(b), stream)
    assert rc == 0, lib.gla_last_error().decode()
    torch.cuda.synchronize()
    return out_a, out_b, need


def _same(a, b):
    return torch.equal(a.view(torch.int16 if a.element_size() == 2 else torch.int32),
                       b.view(torch.int16 if b.element_size() == 2 else torch.int32))


def test_static_entry_point_captured_into_a_graph(device):
    """A split-K GEMV and a split-K GEMM through gla_matmul_static, recorded into one HIP graph and replayed with new
    activations: every replay equals gla_matmul bit for bit.  When this file runs on its own, the capture holds the
    very first static call of the process on the device (the scratch address is looked up while capturing; nothing
    is cleared or allocated then)."""
    lib = _ext.load_library()
    W_q, scales, zeros = gen_int_case(1024, 8192, 4, 128, torch.float16, seed=21)
    layer = GemLiteLinear(4, 128, 8192, 1024, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
    xs = {M: gen_x(M, 8192, torch.float16, seed=30 + M).to(device) for M in (1, 70)}   # GEMV with K slabs; split-K GEMM
    outs = {M: torch.full((M, 1024), float("nan"), dtype=torch.float16, device=device) for M in xs}
    args = {M: _args(layer, xs[M], None, outs[M]) for M in xs}
    for M in xs:
        assert _ext.matmul_workspace_need(args[M]) > 0, "the case is meant to use scratch"
        args[M].workspace, args[M].workspace_bytes = None, 0
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for M in xs:
                rc = lib.gla_matmul_static(ctypes.byref(args[M]), torch.cuda.current_stream().cuda_stream)
                assert rc == 0, lib.gla_last_error().decode()
    for rep in range(4):
        for M in xs:
            xs[M].copy_(gen_x(M, 8192, torch.float16, seed=100 * rep + M).to(device))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for M in xs:
            want = torch.empty_like(outs[M])
            _ext.matmul(_args(layer, xs[M], None, want), device)   # eager work between the replays
            torch.cuda.synchronize()
            assert _same(outs[M], want), (M, rep)
            assert rel_frob(to_np(outs[M]), oracle_forward(layer, xs[M])) <= 1.5e-3


def test_streaming_split_k_twice(device):
    """A16W4 group 128 decode shapes whose K is cut into slabs (fp32 partials + ticket counters)."""
    for (N, K, M, seed) in ((4096, 14336, 1, 1), (1024, 4096, 3, 2)):
        print(f"case: static scratch, gemv N={N} K={K} M={M}", flush=True)
        W_q, scales, zeros = gen_int_case(N, K, 4, 128, torch.float16, seed=seed)
        layer = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
        x = gen_x(M, K, torch.float16, seed=seed + 10).to(device)
        ya, yb, need = _both(layer, x, None, N, torch.float16, device)
        assert need > 0, "the case is meant to use scratch"
        assert _same(ya, yb)
        assert rel_frob(to_np(yb), oracle_forward(layer, x)) <= 1.5e-3


def test_gemm_split_k_twice(device):
    """Packed-code MFMA GEMM at a batch small enough that K is split over workgroups (fp32 partials)."""
    for (N, K, M, seed) in ((4096, 4096, 100, 3), (2048, 2048, 70, 4)):   # above 64 rows: the tiled GEMM
        print(f"case: static scratch, gemm_wn N={N} K={K} M={M}", flush=True)
        W_q, scales, zeros = gen_int_case(N, K, 4, 128, torch.float16, seed=seed)
        layer = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
        x = gen_x(M, K, torch.float16, seed=seed + 10).to(device)
        ya, yb, need = _both(layer, x, None, N, torch.float16, device)
        assert need > 0, "the case is meant to use scratch"
        assert _same(ya, yb)
        assert rel_frob(to_np(yb), oracle_forward(layer, x)) <= 1.5e-3


def test_unpacked_weights_in_the_array_twice_and_the_fused_kernel_when_they_do_not_fit(device):
    """A packed layer at prefill size unpacks its weights into the scratch (N K 2 bytes) before the 16-bit GEMM; twice in
    a row, the second call on a smaller layer, which finds the first one's weights there.  A layer whose unpacked weights
    exceed the array is not refused: the entry point keeps it on the fused kernel, so it must equal gla_matmul with the
    preference for the tiled GEMM bit for bit."""
    lib = _ext.load_library()
    for (N, K, M, seed) in ((4096, 4096, 4096, 7), (4096, 1024, 4096, 8)):   # 256 output tiles: K in one piece
        print(f"case: static scratch, unpacked weights N={N} K={K} M={M}", flush=True)
        W_q, scales, zeros = gen_int_case(N, K, 4, 128, torch.float16, seed=seed)
        layer = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
        x = gen_x(M, K, torch.float16, seed=seed + 10).to(device)
        ya, yb, need = _both(layer, x, None, N, torch.float16, device)
        assert (4 << 20) + N * K * 2 <= need <= lib.gla_static_scratch_bytes(), "the case is meant to unpack the weights into the scratch"
        assert _same(ya, yb)
        assert rel_frob(to_np(yb), oracle_forward(layer, x)) <= 1.5e-3
    N, K, M = 8192, 4608, 4096    # 75.5 MB of fp16 weights: more than the array holds
    print(f"case: static scratch, fused kernel instead of unpacked weights N={N} K={K} M={M}", flush=True)
    W_q, scales, zeros = gen_int_case(N, K, 4, 128, torch.float16, seed=9)
    layer = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q.to(device), scales.to(device), zeros.to(device))
    x = gen_x(M, K, torch.float16, seed=19).to(device)
    out_a = torch.full((M, N), float("nan"), dtype=torch.float16, device=device)
    out_b = torch.full((M, N), float("nan"), dtype=torch.float16, device=device)
    a = _args(layer, x, None, out_a)
    assert _ext.matmul_family(a) == "GEMM_16BIT" and _ext.matmul_workspace_need(a) > lib.gla_static_scratch_bytes()
    a.tile_config = -3          # GLA_TILE_PREFER_MATRIX: the fused kernel
    assert _ext.matmul_family(a) == "GEMM_WN"
    _ext.matmul(a, device)
    b = _args(layer, x, None, out_b)
    b.workspace, b.workspace_bytes = None, 0
    rc = lib.gla_matmul_static(ctypes.byref(b), torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.gla_last_error().decode()
    torch.cuda.synchronize()
    assert _same(out_a, out_b)


def test_mxfp4_regrouped_scales_twice(device):
    """MXFP4 x MXFP4 with 128+-row tiles: both scale arrays are regrouped by stage into the scratch."""
    for (N, K, M, seed) in ((4096, 4096, 2048, 5), (4096, 4096, 1100, 6)):   # sizes at which the 128-row tile is the one chosen
        print(f"case: static scratch, mxfp4 N={N} K={K} M={M}", flush=True)
        W = gen_x(N, K, torch.bfloat16, seed=seed, std=0.02)
        codes, e8 = orc.quantize_mxfp4_weights(to_np(W))
        layer = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_weights(
            torch.from_numpy(codes), scales=torch.from_numpy(e8))
        x = gen_x(M, K, torch.bfloat16, seed=seed + 10).to(device)
        xq, sx = gemlite_amd.scale_activations_mxfp4(x)
        ya, yb, need = _both(layer, xq, sx, N, torch.bfloat16, device)
        assert need > 0, "the case is meant to use scratch"
        assert _same(ya, yb)
        assert rel_frob(to_np(yb), oracle_forward(layer, x)) <= 6e-3


def test_refuses_more_than_the_array_holds(device):
    lib = _ext.load_library()
    limit = lib.gla_static_scratch_bytes()
    assert limit == 72 << 20
    # a split-K GEMM whose partials exceed the array: refused before any pointer is used
    N = K = 16384
    M = 512
    W_q, scales, zeros = gen_int_case(64, 128, 2, 64, torch.bfloat16, seed=0)
    a = _ext.MatmulArgs()
    a.struct_size = ctypes.sizeof(a)
    a.matmul_type = 3   # GEMM_SPLITK
    a.M, a.N, a.K = M, N, K
    dummy = torch.zeros(64, dtype=torch.int32, device=device)
    for f in ("x", "w", "scales", "zeros", "out"):
        setattr(a, f, dummy.data_ptr())
    a.x_stride_m, a.x_stride_k, a.w_stride_k, a.w_stride_n = K, 1, N, 1
    a.out_stride_m, a.out_stride_n, a.meta_stride_g, a.meta_stride_n = N, 1, N, 1
    a.W_nbits, a.group_size, a.unpack_mask, a.elements_per_sample = 2, 64, 3, 16
    a.input_dtype = a.output_dtype = a.meta_dtype = a.zeros_dtype = DType.BF16.value
    a.acc_dtype, a.channel_scale_mode, a.W_group_mode, a.data_contiguous = DType.FP32.value, 0, 4, 1
    a.w_dtype, a.tile_config = DType.INT32.value, 4256   # 4 splits of K, 256-row tiles: 128 MiB of partials
    need = lib.gla_matmul_workspace_bytes(ctypes.byref(a))
    assert need > limit
    rc = lib.gla_matmul_static(ctypes.byref(a), torch.cuda.current_stream().cuda_stream)
    assert rc == -5
    msg = lib.gla_last_error().decode()
    assert "gla_matmul_static" in msg and str(need) in msg
