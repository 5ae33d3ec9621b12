"""Checkpoints on the GPU: pack -> state_dict() -> torch.save / torch.load -> a fresh GemLiteLinear()
(loaded directly, and inside an nn.Sequential with and without assign=True) must give the original
layer's output bit for bit and the oracle's within tolerance
(reference: gemlite/core.py:419-555, tests/test_serialization.py:28-56, :334-356, :442-491)."""
import io

import numpy as np
import pytest
import torch

import gemlite_amd
from gemlite_amd import DType, GemLiteLinear, helper
from oracle import oracle as orc
from parity import elementwise_excess, gen_int_case, gen_x, kind_of, oracle_forward, rel_frob, to_np

pytestmark = pytest.mark.gpu
TIGHT = {torch.float16: 1.5e-3, torch.bfloat16: 6e-3}


def _through_disk(sd):
    buf = io.BytesIO()
    torch.save(sd, buf)
    buf.seek(0)
    return torch.load(buf, weights_only=True)


def _bits(t):
    return t.contiguous().view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()])


def _check_round_trip(layer, x, device, matmul_types=("GEMM",), edit=None):
    """Loads the layer's checkpoint three ways and compares forward() with the original and the oracle."""
    y_ref = {mt: layer.forward_manual(x, matmul_type=mt) for mt in matmul_types}
    y_auto = layer(x)
    want = oracle_forward(layer, x)

    def fresh_direct():
        sd = _through_disk(layer.state_dict())
        if edit is not None:
            edit(sd, "")
        loaded = GemLiteLinear()
        loaded.load_state_dict(sd)
        return loaded

    def fresh_sequential(assign):
        sd = _through_disk(torch.nn.Sequential(layer).state_dict())
        if edit is not None:
            edit(sd, "0.")
        model = torch.nn.Sequential(GemLiteLinear()).to(device)
        model.load_state_dict(sd, strict=True, assign=assign)
        return model[0]

    for how, loaded in (("direct", fresh_direct()), ("sequential", fresh_sequential(False)),
                        ("sequential assign", fresh_sequential(True))):
        print(f"case: checkpoint {how}, {layer.input_dtype} W{layer.W_nbits} M={x.shape[0]}", flush=True)
        assert loaded.get_meta_args() == layer.get_meta_args(), how
        assert (loaded.in_features, loaded.out_features) == (layer.in_features, layer.out_features)
        for a, b in zip(layer.get_tensor_args(), loaded.get_tensor_args()):
            assert a.dtype == b.dtype and a.shape == b.shape and torch.equal(_bits(a) if a.numel() else a, _bits(b) if b.numel() else b), how
        if layer.bias is not None:
            assert torch.equal(layer.bias, loaded.bias)
        for mt in matmul_types:
            y = loaded.forward_manual(x, matmul_type=mt)
            assert torch.equal(_bits(y), _bits(y_ref[mt])), (how, mt)
        y = loaded(x)
        assert torch.equal(_bits(y), _bits(y_auto)), how
        got = to_np(y).reshape(want.shape)
        assert rel_frob(got, want) <= TIGHT[y.dtype], how
        assert elementwise_excess(got, want, kind_of(y.dtype)) <= 1.0, how


@pytest.mark.parametrize("width,word", [(8, torch.uint8), (16, torch.int16), (32, torch.int32)])
def test_a16w4_checkpoint_every_packing_width(device, width, word):
    N, K, gs = 1024, 2048, 128
    W_q, scales, zeros = gen_int_case(N, K, 4, gs, torch.bfloat16, seed=width)
    bias = gen_x(1, N, torch.bfloat16, seed=3).reshape(N) if width == 32 else None
    layer = GemLiteLinear(4, gs, K, N, DType.BF16, DType.BF16).pack(
        W_q.to(device), scales.to(device), zeros.to(device), None if bias is None else bias.to(device),
        packing_bitwidth=width)
    assert layer.W_q.dtype == word
    for M in (1, 32):
        _check_round_trip(layer, gen_x(M, K, torch.bfloat16, seed=M).to(device), device,
                          matmul_types=("GEMM",) if M > 16 else ("GEMV_REVSPLITK", "GEMM_SPLITK"))


def test_a8w8_fp8_dynamic_checkpoint(device):
    N, K = 1024, 2048
    W = gen_x(N, K, torch.bfloat16, seed=5, std=0.02)
    layer = helper.A8W8_FP8_dynamic(device=device, dtype=torch.bfloat16).from_weights(W.to(device))
    assert layer.scaled_activations and layer.channel_scale_mode == 3
    for M in (2, 48):
        _check_round_trip(layer, gen_x(M, K, torch.bfloat16, seed=M).to(device), device)


def test_a4w4_mxfp_checkpoint_in_both_scale_layouts(device):
    """The processor changes the modes after pack() (channel_scale_mode 4), which the save-time metadata
    rebuild must capture.  The checkpoint carries the scales as the reference does - shape [N, K/32],
    strides of a transposed [K/32, N] buffer - and loading accepts that, the row-major form, and a
    stray `scales_5d` key (the reference's TMA layout, which this build ignores)."""
    N, K = 1024, 2048
    W = gen_x(N, K, torch.bfloat16, seed=6, std=0.02)
    codes, e8 = orc.quantize_mxfp4_weights(to_np(W))
    layer = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_weights(
        torch.from_numpy(codes), scales=torch.from_numpy(e8))
    assert (layer.W_group_mode, layer.channel_scale_mode) == (0, 4)
    assert layer.scales.shape == (N, K // 32) and layer.scales.stride() == (K // 32, 1)
    sd = layer.state_dict()
    assert sd["scales"].shape == (N, K // 32) and sd["scales"].stride() == (1, N)       # the reference's stride order
    assert torch.equal(sd["scales"], layer.scales)
    assert sd["metadata"].tolist() == layer.get_meta_args()
    x_small, x_big = gen_x(2, K, torch.bfloat16, seed=1).to(device), gen_x(160, K, torch.bfloat16, seed=2).to(device)
    _check_round_trip(layer, x_big, device)
    _check_round_trip(layer, x_small, device, matmul_types=("GEMM_SPLITK",))

    def row_major(sd, prefix):          # what a safetensors round trip makes of it
        sd[prefix + "scales"] = sd[prefix + "scales"].contiguous()

    def with_5d(sd, prefix):
        sd[prefix + "scales_5d"] = torch.zeros((1, N // 128, K // 128, 2, 256), dtype=torch.uint8)

    _check_round_trip(layer, x_big, device, edit=row_major)
    _check_round_trip(layer, x_big, device, edit=with_5d)


def test_warmup_fills_the_config_cache(device, tmp_path):
    """helper.warmup() tunes a processor's layers at the given shapes and batch sizes; the winners land in the
    cache under the reference's key format and survive cache_config / load_config."""
    gemlite_amd.reset_config()
    try:
        res = helper.warmup(helper.A8W8_INT8_dynamic(device=device, dtype=torch.float16), shapes=[(512, 1024)],
                            batch_sizes=[1, 64], dtype=torch.float16)
        assert set(res[(512, 1024)]) == {1, 64}
        for M, (tile, us, family) in res[(512, 1024)].items():
            assert us > 0 and isinstance(family, str)
        f = str(tmp_path / "cfg.json")
        gemlite_amd.cache_config(f)
        snapshot = {k: dict(v) for k, v in gemlite_amd.GEMLITE_CONFIG_CACHE.items()}
        gemlite_amd.reset_config()
        assert gemlite_amd.load_config(f) is True
        for k, v in snapshot.items():
            assert gemlite_amd.GEMLITE_CONFIG_CACHE.get(k, {}) == v
    finally:
        gemlite_amd.reset_config()
