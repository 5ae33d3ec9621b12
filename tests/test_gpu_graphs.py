"""forward() under HIP graph capture: the launches of a layer (activation quantisation, the
matmul, a split-K finish) are recorded once and replayed with new inputs.  Every replay must equal
the eager result bit for bit - the kernels are deterministic, the ticket counters of the split-K
GEMV reset themselves, and nothing in the path allocates or clears memory once the layer has run
at that shape."""
import pytest
import torch

import gemlite_amd
from gemlite_amd import DType, GemLiteLinear, _ext, helper
from parity import gen_int_case, gen_x

pytestmark = pytest.mark.gpu


def _layers(device):
    W_q, s, z = gen_int_case(1024, 8192, 4, 128, torch.float16, seed=1)
    yield "A16W4", GemLiteLinear(4, 128, 8192, 1024, DType.FP16, DType.FP16).pack(W_q.to(device), s.to(device), z.to(device)), \
        torch.float16, (1, 5, 64)      # split-K GEMV with tickets; split-K MFMA GEMM with its finishing kernel
    W = gen_x(1032, 2048, torch.bfloat16, seed=2, std=0.02)
    W_q8, s8 = gemlite_amd.quantize_weights_per_channel(W, torch.int8)
    proc = helper.A8W8_INT8_dynamic(device=device)
    proc.dtype = torch.bfloat16
    yield "A8W8", proc.from_weights(W_q8, scales=s8), torch.bfloat16, (3, 70)   # activation quantiser + GEMM
    lin = torch.nn.Linear(2048, 1032, bias=True, dtype=torch.bfloat16)
    lin.weight.data = W
    yield "MXFP4", helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_linear(lin.to(device)), \
        torch.bfloat16, (40,)
    lin = torch.nn.Linear(2048, 1032, bias=True, dtype=torch.bfloat16)
    lin.weight.data = W
    yield "A16W4_MXFP", helper.A16W4_MXFP(device=device, dtype=torch.bfloat16).from_linear(lin.to(device), del_orig=False), \
        torch.bfloat16, (1, 6)         # streaming kernel; split-K matrix-core kernel with its finishing kernel
    yield "A8W4_MXFP", helper.A8W4_MXFP_dynamic(device=device, dtype=torch.bfloat16, post_scale=False).from_linear(
        lin.to(device), del_orig=False), torch.bfloat16, (2, 150)   # MXFP8 quantiser + streaming / mixed MFMA with staged scales
    yield "A8W8 block-quantised", helper.A8W8_FP8_dynamic(device=device, block_quant=True).from_weights(W.to(device)), \
        torch.bfloat16, (3, 40)        # per-block quantiser + streaming / split-K MFMA with the second accumulator


def test_forward_replays_from_a_graph(device):
    for name, layer, dtype, row_counts in _layers(device):
        K = layer.in_features
        for M in row_counts:
            print(f"case: {name} M={M}", flush=True)
            x_static = gen_x(M, K, dtype, seed=99).to(device)
            layer(x_static)  # first run at this shape: sizes the workspace
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                y_static = layer(x_static)
            for rep in range(4):
                x_new = gen_x(M, K, dtype, seed=rep).to(device)
                x_static.copy_(x_new)
                graph.replay()
                torch.cuda.synchronize()
                got = y_static.clone()
                want = layer(x_new)  # eager work between the replays
                torch.cuda.synchronize()
                assert torch.equal(got, want), (name, M, rep)


def test_workspace_growth_is_refused_during_capture_and_keeps_old_buffers(device, monkeypatch):
    ws = _ext.get_workspace(device, 1)
    bigger = ws.numel() + 1
    # the stream reports a capture in progress (no real capture: a failed one would outlive the test)
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    with pytest.raises(RuntimeError, match="before capturing"):
        _ext.get_workspace(device, bigger)
    assert _ext.get_workspace(device, ws.numel()).data_ptr() == ws.data_ptr()  # large enough: no growth, no refusal
    monkeypatch.undo()
    grown = _ext.get_workspace(device, bigger)
    assert grown.numel() >= 2 * ws.numel() and grown.data_ptr() != ws.data_ptr()
    assert any(r.data_ptr() == ws.data_ptr() for r in _ext._retired_workspaces)


def test_two_streams_use_separate_scratch(device):
    """Split-K launches (fp32 partials + ticket counters in the workspace) issued from two streams at the same
    time: each stream has a workspace of its own, so every result equals the single-stream one bit for bit."""
    W_q, s, z = gen_int_case(1024, 8192, 4, 128, torch.float16, seed=5)
    layer_a = GemLiteLinear(4, 128, 8192, 1024, DType.FP16, DType.FP16).pack(W_q.to(device), s.to(device), z.to(device))
    W_q, s, z = gen_int_case(2048, 4096, 4, 128, torch.float16, seed=6)
    layer_b = GemLiteLinear(4, 128, 4096, 2048, DType.FP16, DType.FP16).pack(W_q.to(device), s.to(device), z.to(device))
    xa, xb = gen_x(1, 8192, torch.float16, seed=7).to(device), gen_x(3, 4096, torch.float16, seed=8).to(device)
    want_a, want_b = layer_a(xa).clone(), layer_b(xb).clone()
    torch.cuda.synchronize()
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    outs_a, outs_b = [], []
    for _ in range(200):
        with torch.cuda.stream(sa):
            outs_a.append(layer_a(xa))
        with torch.cuda.stream(sb):
            outs_b.append(layer_b(xb))
    torch.cuda.synchronize()
    key_a = _ext._workspace_key(device, sa.cuda_stream)
    key_b = _ext._workspace_key(device, sb.cuda_stream)
    assert _ext._workspaces[key_a].data_ptr() != _ext._workspaces[key_b].data_ptr()
    assert all(torch.equal(o, want_a) for o in outs_a) and all(torch.equal(o, want_b) for o in outs_b)
