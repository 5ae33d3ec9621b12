"""CPU-side tests of the host layer: layout, mode logic, dispatcher, C-ABI surface, errors."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import gemlite_amd
from gemlite_amd import DType, GemLiteLinear, _ext
from gemlite_amd.bitpack import pack_weights_over_cols_torch, unpack_over_cols_torch
from gemlite_amd.dtypes import PACKING_BITWIDTH_TO_TORCH_DTYPE
from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_dtype_enum_values():
    # serialised integer ids (reference: gemlite/dtypes.py:8-29)
    expect = dict(FP32=0, FP16=1, BF16=2, FP8=3, FP8e4=3, INT8=4, UINT8=5, INT32=6, UINT32=7, FP8e5=8, INT16=9,
                  UINT16=10, INT64=11, FP8e4nuz=12, FP8e5nuz=13, MXFP16=14, MXBF16=15, MXFP8=16, MXFP4=17, NVFP4=18,
                  E8M0=19)
    for name, v in expect.items():
        assert DType[name].value == v
    assert gemlite_amd.is_mx_dtype(DType.MXFP4) and gemlite_amd.is_mx_dtype(17) and not gemlite_amd.is_mx_dtype(DType.FP8)


@pytest.mark.parametrize("nbits", [1, 2, 4, 8])
@pytest.mark.parametrize("width", [8, 16, 32, 64])
def test_torch_pack_matches_oracle(nbits, width):
    rng = np.random.default_rng(nbits + width)
    e = width // nbits
    W = rng.integers(0, 2 ** nbits, size=(6, 4 * e), dtype=np.uint8)
    packed, e_out = pack_weights_over_cols_torch(torch.from_numpy(W), nbits, width, transpose=False)
    assert e_out == e and packed.dtype == PACKING_BITWIDTH_TO_TORCH_DTYPE[width]
    assert np.array_equal(packed.numpy(), orc.pack_over_cols(W, nbits, width))
    packed_t, _ = pack_weights_over_cols_torch(torch.from_numpy(W), nbits, width, transpose=True)
    assert packed_t.shape == (4, 6) and not packed_t.is_contiguous()
    assert np.array_equal(unpack_over_cols_torch(packed, nbits, 4 * e).numpy(), W)


def _layer(nbits=4, gs=128, K=256, N=64, in_dt=DType.FP16, out_dt=DType.FP16, **kw):
    return GemLiteLinear(nbits, gs, K, N, in_dt, out_dt, **kw)


def test_pack_layout_a16w4():
    N, K, gs = 64, 256, 128
    g = torch.Generator().manual_seed(0)
    W_q = torch.randint(0, 16, (N, K), generator=g, dtype=torch.int32).to(torch.uint8)
    scales = torch.rand((N * K // gs, 1), generator=g).half()
    zeros = (torch.rand((N * K // gs, 1), generator=g) * 8).half()
    layer = _layer().pack(W_q, scales, zeros)
    # physical [K/8, N] int32, N fastest
    assert layer.W_q.shape == (K // 8, N) and layer.W_q.dtype == torch.int32 and layer.W_q.is_contiguous()
    assert layer.elements_per_sample == 8 and layer.data_contiguous is True
    k8, n = 5, 17
    word = sum(int(W_q[n, 8 * k8 + i]) << (4 * i) for i in range(8))
    assert int(layer.W_q[k8, n]) & 0xFFFFFFFF == word
    # scales [K/gs, N]; zeros pre-multiplied: z' = fp16(-z * s); mode 4
    assert layer.scales.shape == (K // gs, N) and layer.scales.is_contiguous()
    assert layer.W_group_mode == 4 and layer.channel_scale_mode == 0
    assert torch.equal(layer.scales, scales.view(N, -1).t())
    assert torch.equal(layer.zeros, (-zeros.float() * scales.float()).half().view(N, -1).t())
    assert layer.get_meta_args() == [0, 4, 128, 15, 8, 1, 1, 0, 1, 0, 4, 1]
    assert layer.metadata.tolist() == layer.get_meta_args() and layer.orig_shape.tolist() == [N, K]
    # fma_mode=False keeps the raw zeros and uses mode 3
    layer3 = _layer().pack(W_q, scales, zeros, fma_mode=False)
    assert layer3.W_group_mode == 3 and torch.equal(layer3.zeros, zeros.view(N, -1).t())


def test_pack_modes_like_reference_tests():
    N, K = 48, 256
    W_q = torch.randint(0, 15, (N, K)).to(torch.uint8)
    W = torch.randn(N, K).to(torch.bfloat16)
    # fp16 x fp16 (reference: tests/test_int.py:99-113)
    l = _layer(16, None, K, N, DType.BF16, DType.BF16).pack(W, None, None, None)
    assert (l.W_group_mode, l.channel_scale_mode, l.data_contiguous) == (0, 0, False)
    assert l.W_q.shape == (K, N) and l.W_q.stride() == (1, K) and l.elements_per_sample == 1
    # int8 x Wn, channel-wise scales + integer zero (reference: tests/test_int.py:146-163)
    l = _layer(4, 128, K, N, DType.INT8, DType.FP32).pack(W_q, torch.randn(N, 1).bfloat16() * 1e-4, 7)
    assert (l.W_group_mode, l.channel_scale_mode) == (1, 1) and l.zeros.item() == 7 and l.zeros.dtype == torch.int32
    assert l.acc_dtype == DType.INT32
    # dynamic activations only (reference: tests/test_int.py:173-190)
    l = _layer(4, 128, K, N, DType.INT8, DType.FP32, scaled_activations=True).pack(W_q, None, 7)
    assert (l.W_group_mode, l.channel_scale_mode) == (1, 2)
    assert l.meta_dtype == DType.INT32  # placeholder scales tensor is int32
    # both scaled (reference: tests/test_int.py:201-218)
    l = _layer(8, 128, K, N, DType.INT8, DType.FP32, scaled_activations=True).pack(W_q, torch.rand(N, 1), 7)
    assert (l.W_group_mode, l.channel_scale_mode) == (1, 3)
    # fp8 x fp8, no scales / both scaled (reference: tests/test_int.py:226-271)
    W8 = W.float().to(torch.float8_e4m3fn)
    l = _layer(8, None, K, N, DType.FP8, DType.BF16, scaled_activations=True).pack(W8, None, None)
    assert (l.W_group_mode, l.channel_scale_mode) == (0, 2) and l.W_q.stride() == (1, K)
    l = _layer(8, K, K, N, DType.FP8, DType.BF16, scaled_activations=True).pack(W8, torch.rand(N, 1), None)
    assert (l.W_group_mode, l.channel_scale_mode) == (0, 3)
    # float inputs never get dynamic activation quantisation
    assert _layer(4, 128, K, N, DType.FP16, DType.FP16, scaled_activations=True).scaled_activations is False


def test_pack_mxfp4_layout():
    N, K = 64, 256
    codes = torch.randint(0, 16, (N, K)).to(torch.uint8)
    e8 = torch.randint(110, 130, (N, K // 32)).to(torch.uint8).view(torch.float8_e8m0fnu)
    l = gemlite_amd.helper.A4W4_MXFP_dynamic(device="cpu", dtype=torch.bfloat16).from_weights(codes, scales=e8)
    # bytes [N, K/2] (low nibble = even k) handed over as the [K/2, N] view; e8m0 scales as the [N, K/32] view
    assert l.W_q.shape == (K // 2, N) and l.W_q.stride() == (1, K // 2) and l.W_q.dtype == torch.uint8
    assert int(l.W_q[3, 5]) == int(codes[5, 6]) | (int(codes[5, 7]) << 4)
    assert l.scales.shape == (N, K // 32) and l.scales.dtype == torch.uint8 and l.scales.stride() == (K // 32, 1)
    assert (l.W_group_mode, l.channel_scale_mode, l.elements_per_sample) == (0, 4, 2)
    assert l.W_q.numel() == N * K // 2  # packed byte count (reference: tests/test_mxfp.py:96)


def test_packing_widths_and_dtypes():
    # W_q storage dtype per packing width (reference: tests/test_serialization.py:334-356)
    N, K = 32, 128
    W_q = torch.randint(0, 16, (N, K)).to(torch.uint8)
    s, z = torch.rand(N * K // 64, 1).half(), torch.rand(N * K // 64, 1).half()
    for width, dt in ((8, torch.uint8), (16, torch.int16), (32, torch.int32)):
        l = _layer(4, 64, K, N).pack(W_q, s, z, packing_bitwidth=width)
        assert l.W_q.dtype == dt and l.W_q.shape == (K * 4 // width, N)


def test_constructor_errors():
    with pytest.raises(NotImplementedError):
        GemLiteLinear(3, 64, 128, 128)
    with pytest.raises(NotImplementedError):
        GemLiteLinear(4, 64, 100, 128)  # K % 32
    with pytest.raises(NotImplementedError):
        GemLiteLinear(4, 96, 128, 128)  # K % group_size
    with pytest.raises(NotImplementedError):
        GemLiteLinear(4, 8, 128, 128)   # group_size < 16
    with pytest.raises(NotImplementedError):
        GemLiteLinear(4, 64, 128, 128, input_dtype=DType.INT32)
    with pytest.raises(Exception, match="floating-point zeros"):
        _layer(4, 128, 256, 64, DType.INT8, DType.FP32).pack(
            torch.zeros(64, 256, dtype=torch.uint8), torch.rand(64, 1), torch.rand(128, 1) + 0.3)
    with pytest.raises(Exception, match="not packed"):
        _layer().pack(torch.zeros(64, 256, dtype=torch.int32), None, None)


def test_state_dict_roundtrip():
    N, K, gs = 64, 256, 64
    W_q = torch.randint(0, 16, (N, K)).to(torch.uint8)
    s, z = torch.rand(N * K // gs, 1).half(), torch.rand(N * K // gs, 1).half()
    fresh = _layer(4, gs, K, N)
    assert set(fresh.state_dict().keys()) == {"W_q", "scales", "zeros", "metadata", "orig_shape", "meta_scale"}
    a = _layer(4, gs, K, N).pack(W_q, s, z, bias=torch.rand(N).half())
    sd = a.state_dict()
    assert set(sd.keys()) == {"W_q", "scales", "zeros", "metadata", "orig_shape", "meta_scale", "bias"}
    b = GemLiteLinear()
    b.load_state_dict(dict(sd))
    assert b.get_meta_args() == a.get_meta_args() and (b.in_features, b.out_features) == (K, N)
    for ta, tb in zip(a.get_tensor_args(), b.get_tensor_args()):
        assert torch.equal(ta, tb)
    # through a parent module, strict
    seq_a = torch.nn.Sequential(a)
    seq_b = torch.nn.Sequential(GemLiteLinear())
    seq_b.load_state_dict(seq_a.state_dict(), strict=True)
    assert seq_b[0].get_meta_args() == a.get_meta_args() and torch.equal(seq_b[0].bias, a.bias)
    # overridden modes are what gets saved
    a.W_group_mode, a.channel_scale_mode = 3, 0
    assert a.state_dict()["metadata"].tolist()[9:11] == [0, 3]
    with pytest.raises(RuntimeError, match="missing required keys"):
        GemLiteLinear().load_state_dict({"scales": s})


def test_dispatcher_host_and_library_agree():
    for nbits in (1, 2, 4, 8, 16):
        for mx in (False, True):
            for M in (1, 2, 3, 4, 5, 8, 16, 32, 63, 64, 65, 512, 4096, 8192):
                name = gemlite_amd.get_matmul_type(M, nbits, mx)
                assert name == orc.get_matmul_type(M, nbits, mx)
                assert gemlite_amd.GEMLITE_MATMUL_TYPES[_ext.get_matmul_type_id(M, nbits, mx)] == name
    for M in list(range(0, 300)) + [1000, 3000, 4096, 4097, 100000]:
        assert gemlite_amd.get_closest_m(M) == orc.get_closest_m(M) == _ext.get_closest_m(M)
    assert gemlite_amd.get_type_id(DType.BF16.value, 4) == 104 and gemlite_amd.get_type_id(DType.MXFP4.value, 4) == 1704
    assert gemlite_amd.config_key(3, 4096, 4096, 128, 8, 104) == "(4, 4096, 4096, 128, 8, 104)"


def test_config_cache_roundtrip(tmp_path):
    gemlite_amd.reset_config()
    gemlite_amd.GEMLITE_CONFIG_CACHE.setdefault("GEMV_REVSPLITK", {})["(1, 4096, 4096, 128, 8, 104)"] = {"tile_config": 2}
    f = str(tmp_path / "cfg.json")
    gemlite_amd.cache_config(f)
    gemlite_amd.reset_config()
    assert gemlite_amd.GEMLITE_CONFIG_CACHE == {}
    assert gemlite_amd.load_config(f) is True
    assert gemlite_amd.GEMLITE_CONFIG_CACHE["GEMV_REVSPLITK"]["(1, 4096, 4096, 128, 8, 104)"] == {"tile_config": 2}
    assert gemlite_amd.load_config(str(tmp_path / "missing.json"), print_error=False) is False
    gemlite_amd.reset_config()


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "gemlite_amd.h")).read()
    declared = set(re.findall(r"\b(gla_[a-z0-9_]+)\s*\(", header))
    assert declared and declared == set(_ext.SYMBOLS)
    lib = ctypes.CDLL(_ext.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert _ext.load_library().gla_abi_version() == 1


def test_abi_struct_matches_header():
    header = open(os.path.join(ROOT, "include", "gemlite_amd.h")).read()
    body = header[header.index("typedef struct gla_matmul_args {"): header.index("} gla_matmul_args;")]
    names = []
    for line in body.splitlines()[1:]:
        line = line.split("/*")[0].strip()
        if not line.endswith(";"):
            continue
        decl = line[:-1]
        for part in decl.split(",") if "*" not in decl else [decl]:
            names.append(part.strip().split()[-1].lstrip("*"))
    assert names == [f[0] for f in _ext.MatmulArgs._fields_]


def test_abi_rejects_bad_arguments_without_a_gpu():
    lib = _ext.load_library()
    a = _ext.MatmulArgs()
    assert lib.gla_matmul(None, None) == -1 and b"NULL" in lib.gla_last_error()
    a.struct_size = 4
    assert lib.gla_matmul(ctypes.byref(a), None) == -1 and b"struct_size" in lib.gla_last_error()
    a.struct_size = ctypes.sizeof(_ext.MatmulArgs)
    a.M, a.N, a.K = 1, 0, 64
    assert lib.gla_matmul(ctypes.byref(a), None) == -1
    a.N = 64
    assert lib.gla_matmul(ctypes.byref(a), None) == -1  # NULL operands
    a.x = a.w = a.out = 4096  # never dereferenced: validation fails first
    a.elements_per_sample, a.W_nbits = 8, 4
    a.input_dtype = DType.NVFP4.value
    assert lib.gla_matmul(ctypes.byref(a), None) == -2
    a.input_dtype, a.output_dtype, a.acc_dtype = DType.FP16.value, DType.FP16.value, DType.FP32.value
    a.W_group_mode = 7
    assert lib.gla_matmul(ctypes.byref(a), None) == -3
    a.W_group_mode, a.group_size = 4, 48
    a.scales = a.zeros = 4096
    assert lib.gla_matmul(ctypes.byref(a), None) == -4  # K % group_size
    a.group_size, a.scales = 64, None
    assert lib.gla_matmul(ctypes.byref(a), None) == -1  # mode needs scales
    a.matmul_type = 9
    assert lib.gla_matmul(ctypes.byref(a), None) == -3
    # activation-quant and packing entry points validate before launching
    assert lib.gla_scale_activations_per_token(None, 1, 64, 1, 64, None, 4, None, None) == -1
    assert lib.gla_scale_activations_per_token(4096, 1, 60, 1, 60, 4096, 4, 4096, None) == -4
    assert lib.gla_scale_activations_per_token(4096, 1, 64, 1, 64, 4096, 2, 4096, None) == -2
    assert lib.gla_scale_activations_mxfp4(4096, 1, 48, 1, 48, 4096, 4096, None) == -4
    assert lib.gla_pack_over_cols(4096, 4096, 4, 30, 4, 32, None) == -4
    assert lib.gla_pack_over_cols(4096, 4096, 4, 32, 3, 32, None) == -3


def test_forward_requires_gpu_and_library():
    l = _layer().pack(torch.zeros(64, 256, dtype=torch.uint8), torch.ones(128, 1).half(), torch.ones(128, 1).half())
    with pytest.raises(RuntimeError, match="GPU only"):
        l(torch.zeros(1, 256).half())
    with pytest.raises(RuntimeError, match="not found"):
        _ext.load_library(os.path.join(ROOT, "no_such_dir", "libgemlite_amd.so"))


def test_operand_bounds_are_checked_on_the_host():
    # strides that would walk outside a tensor are refused before any launch
    N, K, M = 64, 256, 2
    x = torch.zeros(M, K, dtype=torch.float16)
    W = torch.zeros(K // 8, N, dtype=torch.int32)
    s = torch.zeros(K // 128, N, dtype=torch.float16)
    out = torch.zeros(M, N, dtype=torch.float16)
    kw = dict(W_nbits=4, group_size=128, unpack_mask=15, elements_per_sample=8, input_dtype=1, output_dtype=1,
              acc_dtype=0, meta_dtype=1, channel_scale_mode=0, W_group_mode=4, data_contiguous=1)
    _ext.build_matmul_args(x, W, s, s, None, out, **kw)  # consistent: accepted
    with pytest.raises(ValueError, match="scales"):
        _ext.build_matmul_args(x, W, s.t(), s, None, out, **kw)   # [N, G] view read as [G, N]
    with pytest.raises(ValueError, match="x:"):
        _ext.build_matmul_args(x[:, : K // 2].contiguous(), W, s, s, None, out, **kw)  # x shorter than K
    with pytest.raises(ValueError, match="out"):
        _ext.build_matmul_args(x, W, s, s, None, out[:1].clone(), **kw)
    # micro-scaled layers hand their scales over as a row-major [N, K/32] array
    codes = torch.randint(0, 16, (N, K)).to(torch.uint8)
    e8 = torch.randint(110, 130, (N, K // 32)).to(torch.uint8)
    l = gemlite_amd.helper.A4W4_MXFP_dynamic(device="cpu", dtype=torch.bfloat16).from_weights(codes, scales=e8)
    m = l.get_meta_args()
    a = _ext.build_matmul_args(
        torch.zeros(M, K // 2, dtype=torch.uint8), l.W_q, l.scales, l.zeros, torch.zeros(32, K // 32, dtype=torch.uint8),
        torch.zeros(M, N, dtype=torch.bfloat16), W_nbits=m[1], group_size=m[2], unpack_mask=m[3],
        elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6], acc_dtype=m[7], meta_dtype=m[8],
        channel_scale_mode=m[9], W_group_mode=m[10], data_contiguous=m[11])
    assert (a.meta_stride_g, a.meta_stride_n) == (1, K // 32) and (a.w_stride_k, a.w_stride_n) == (1, K // 2)


def test_custom_op_is_registered_with_a_fake():
    # the functional forward is also a torch custom op, traceable without running a kernel
    # (reference: gemlite/core.py:193-200, :276-285)
    import gemlite_amd
    from torch._subclasses.fake_tensor import FakeTensorMode
    op = gemlite_amd.forward_functional_op
    assert op is not None and hasattr(torch.ops.gemlite, "forward_functional")
    N, K, M = 64, 128, 3
    l = GemLiteLinear(4, 64, K, N, DType.FP16, DType.BF16)
    l.pack(torch.randint(0, 16, (N, K)).to(torch.uint8), torch.ones(N * K // 64, 1).half(), torch.ones(N * K // 64, 1).half())
    with FakeTensorMode():
        x = torch.empty((2, M, K), dtype=torch.float16, device="cuda")
        tensors = [torch.empty(t.shape, dtype=t.dtype, device="cuda") for t in l.get_tensor_args()]
        y = torch.ops.gemlite.forward_functional(x, None, tensors, l.get_meta_args(), -1)
        assert y.shape == (2, M, N) and y.dtype == torch.bfloat16 and y.device.type == "cuda"


def _family(layer, M, x_dtype, scales_x=None, x=None):
    m = layer.get_meta_args()
    K = layer.in_features
    if x is None:
        x = torch.zeros(M, K, dtype=x_dtype)
    out = torch.zeros(M, layer.out_features, dtype=gemlite_amd.DTYPE_TO_TORCH[m[6]])
    a = _ext.build_matmul_args(
        x, layer.W_q, layer.scales, layer.zeros, scales_x, out, W_nbits=m[1], group_size=m[2], unpack_mask=m[3],
        elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6], acc_dtype=m[7], meta_dtype=m[8],
        channel_scale_mode=m[9], W_group_mode=m[10], data_contiguous=m[11])
    return _ext.matmul_family(a)


def test_packed_layers_without_a_tiled_gemm_take_the_mid_batch_kernel():
    # host logic only.  Groups of 32 and 1-bit codes have no tiled GEMM (and 2-bit gs 32 / 1-bit gs 32, 64 no streaming
    # kernel either): which family takes them at each row count, and that the preferences only switch between kernels
    # that accept the call.
    g = torch.Generator().manual_seed(0)
    N, K = 512, 1024
    Ms = (1, 4, 16, 17, 64, 65, 300)

    def layer(nbits, gs, dt=DType.BF16, tdt=torch.bfloat16):
        W_q = torch.randint(0, 2 ** nbits, (N, K), generator=g).to(torch.uint8)
        return GemLiteLinear(nbits, gs, K, N, dt, dt).pack(W_q, torch.rand(N * K // gs, 1).to(tdt), torch.rand(N * K // gs, 1).to(tdt))

    assert [_family(layer(2, 32), M, torch.bfloat16) for M in Ms] == ["WN_MID"] * 7
    assert [_family(layer(1, 64), M, torch.bfloat16) for M in Ms] == ["GENERIC"] + ["WN_MID"] * 6   # one row: the K-split vector kernel
    assert [_family(layer(1, 32), M, torch.bfloat16) for M in Ms] == ["GENERIC"] + ["WN_MID"] * 6
    # 4- and 8-bit codes in groups of 32, 1-bit codes in groups of 128: the GEMV (row chunks) up to 64 rows on a small layer
    for l in (layer(4, 32), layer(8, 32), layer(1, 128)):
        assert [_family(l, M, torch.bfloat16) for M in Ms] == ["GEMV_PACKED"] * 5 + ["WN_MID"] * 2
    # (at prefill size such layers unpack their weights first and run the 16-bit GEMM: from 512 rows, 1- and 2-bit codes from 1024)
    assert [_family(layer(4, 32), M, torch.bfloat16) for M in (511, 512)] == ["WN_MID", "GEMM_16BIT"]
    assert [_family(layer(2, 32), M, torch.bfloat16) for M in (1023, 1024)] == ["WN_MID", "GEMM_16BIT"]
    assert [_family(layer(1, 64), M, torch.bfloat16) for M in (1023, 1024)] == ["WN_MID", "GEMM_16BIT"]
    # groups of 16: the mid-batch kernel at any row count (2-, 4-, 8-bit codes); 1-bit codes stay with the generic kernels
    for l in (layer(2, 16), layer(4, 16), layer(8, 16)):
        assert [_family(l, M, torch.bfloat16) for M in Ms] == ["WN_MID"] * 7
    assert [_family(layer(1, 16), M, torch.bfloat16) for M in (1, 64)] == ["GENERIC"] * 2
    # a preference for the mid-batch kernel is honoured where it is eligible (any row count) and ignored elsewhere
    l4 = layer(4, 128, DType.FP16, torch.float16)
    m = l4.get_meta_args()
    for M, tile, fam in ((1, -4, "WN_MID"), (16, -4, "WN_MID"), (300, -4, "WN_MID"), (16, 2008, "WN_MID"), (16, -1, "GEMV_PACKED"),
                         (300, -1, "GEMM_WN")):
        a = _ext.build_matmul_args(torch.zeros(M, K, dtype=torch.float16), l4.W_q, l4.scales, l4.zeros, None,
                                   torch.zeros(M, N, dtype=torch.float16), W_nbits=m[1], group_size=m[2], unpack_mask=m[3],
                                   elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6], acc_dtype=m[7], meta_dtype=m[8],
                                   channel_scale_mode=m[9], W_group_mode=m[10], data_contiguous=m[11], tile_config=tile)
        assert _ext.matmul_family(a) == fam, (M, tile, _ext.matmul_family(a))
    lg = layer(1, 16)
    mg = lg.get_meta_args()
    a = _ext.build_matmul_args(torch.zeros(8, K, dtype=torch.bfloat16), lg.W_q, lg.scales, lg.zeros, None,
                               torch.zeros(8, N, dtype=torch.bfloat16), W_nbits=mg[1], group_size=mg[2], unpack_mask=mg[3],
                               elements_per_sample=mg[4], input_dtype=mg[5], output_dtype=mg[6], acc_dtype=mg[7], meta_dtype=mg[8],
                               channel_scale_mode=mg[9], W_group_mode=mg[10], data_contiguous=mg[11], tile_config=-4)
    assert _ext.matmul_family(a) == "GENERIC"
    # unquantised layers: vector kernels for decode, the MFMA GEMM from 9 rows
    W = torch.randn(N, K).to(torch.float16)
    l16 = GemLiteLinear(16, None, K, N, DType.FP16, DType.FP16).pack(W, None, None)
    assert [_family(l16, M, torch.float16) for M in (1, 8, 9, 64, 4096)] == ["GENERIC"] * 2 + ["GEMM_16BIT"] * 3


def test_benchmark_configurations_take_a_tuned_kernel_family():
    # host logic only: which family gla_matmul would launch (the layout-agnostic kernel is correct but slow,
    # so none of the benchmark configurations may fall to it)
    g = torch.Generator().manual_seed(0)
    N, K = 512, 1024
    # A16W4 gs128 fp16 (decode and prefill)
    W_q = torch.randint(0, 16, (N, K), generator=g).to(torch.uint8)
    s, z = torch.rand(N * K // 128, 1).half(), torch.rand(N * K // 128, 1).half()
    l = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q, s, z)
    # (up to 64 rows a layer this small stays with the streaming kernel, as row chunks of 16: see the next test)
    # (from 4096 rows of fp16 the weights are unpacked first and the 16-bit GEMM runs)
    assert [_family(l, M, torch.float16) for M in (1, 2, 4, 8, 16, 64, 65, 1000, 4096)] == ["GEMV_PACKED"] * 6 + ["GEMM_WN"] * 2 + ["GEMM_16BIT"]
    # A16W8 channel-wise and A16W2 gs64, bf16
    W8 = torch.randint(0, 256, (N, K), generator=g).to(torch.uint8)
    l8 = GemLiteLinear(8, K, K, N, DType.BF16, DType.BF16).pack(W8, torch.rand(N, 1).bfloat16(), torch.rand(N, 1).bfloat16())
    assert (l8.W_group_mode, l8.channel_scale_mode) == (1, 1)
    assert [_family(l8, M, torch.bfloat16) for M in (1, 16, 64, 65, 512)] == ["GEMV_PACKED"] * 3 + ["GEMM_WN"] * 2
    l8h = GemLiteLinear(8, K, K, N, DType.FP16, DType.FP16).pack(W8, torch.rand(N, 1).half(), torch.rand(N, 1).half())
    assert [_family(l8h, M, torch.float16) for M in (1, 16, 64, 100)] == ["GEMV_PACKED"] * 3 + ["GEMM_WN"]
    K2 = 4096
    W2 = torch.randint(0, 4, (N, K2), generator=g).to(torch.uint8)
    l2 = GemLiteLinear(2, 64, K2, N, DType.BF16, DType.BF16).pack(
        W2, torch.rand(N * K2 // 64, 1).bfloat16(), torch.rand(N * K2 // 64, 1).bfloat16())
    assert [_family(l2, M, torch.bfloat16) for M in (1, 16, 64, 65, 512)] == ["GEMV_PACKED"] * 3 + ["GEMM_WN"] * 2
    # A8W8 fp8 / int8 dynamic and INT8 x INT8 -> INT32
    Wb = torch.randn(N, K, generator=g).bfloat16() * 0.02
    for proc, dt in ((gemlite_amd.helper.A8W8_FP8_dynamic, torch.float8_e4m3fn), (gemlite_amd.helper.A8W8_INT8_dynamic, torch.int8)):
        la = proc(device="cpu").from_weights(Wb)
        # streaming up to 2 rows, operands as they are into the MFMA in one launch up to 32 (K = 1024 is a multiple of 128), the tiled GEMM above
        for M, fam in ((1, "GEMV_KMAJOR"), (2, "GEMV_KMAJOR"), (3, "K_SKINNY"), (32, "K_SKINNY"), (33, "GEMM_8BIT"), (4096, "GEMM_8BIT")):
            xq = torch.zeros(M, K, dtype=dt)
            assert _family(la, M, None, scales_x=torch.ones(M, 1), x=xq) == fam
    # MXFP4
    codes = torch.randint(0, 16, (N, K), generator=g).to(torch.uint8)
    e8 = torch.randint(110, 130, (N, K // 32), generator=g).to(torch.uint8)
    lm = gemlite_amd.helper.A4W4_MXFP_dynamic(device="cpu", dtype=torch.bfloat16).from_weights(codes, scales=e8)
    for M in (1, 32, 1024):
        xq = torch.zeros(M, K // 2, dtype=torch.uint8)
        sx = torch.full(((M + 31) // 32 * 32, K // 32), 127, dtype=torch.uint8)
        assert _family(lm, M, None, scales_x=sx, x=xq) == {1: "MX_STREAM", 32: "K_SKINNY", 1024: "GEMM_MXFP4"}[M]


def test_tile_config_can_state_a_preference_between_streaming_and_matrix_kernels():
    """GLA_TILE_PREFER_STREAMING (-2) / GLA_TILE_PREFER_MATRIX (-3): where both kinds of kernel take a call, the
    preference decides; where only one does, it runs; -1 keeps the library's own hand-off."""
    g = torch.Generator().manual_seed(0)
    N, K = 512, 1024
    W_q = torch.randint(0, 16, (N, K), generator=g).to(torch.uint8)
    s, z = torch.rand(N * K // 128, 1).half(), torch.rand(N * K // 128, 1).half()
    l = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q, s, z)
    m = l.get_meta_args()

    def fam(M, tile):
        x = torch.zeros(M, K, dtype=torch.float16)
        out = torch.zeros(M, N, dtype=torch.float16)
        a = _ext.build_matmul_args(x, l.W_q, l.scales, l.zeros, None, out, W_nbits=m[1], group_size=m[2], unpack_mask=m[3],
                                   elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6], acc_dtype=m[7],
                                   meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10], data_contiguous=m[11],
                                   tile_config=tile)
        return _ext.matmul_family(a)
    assert [fam(M, -1) for M in (8, 32, 100)] == ["GEMV_PACKED", "GEMV_PACKED", "GEMM_WN"]
    assert [fam(M, -3) for M in (8, 32, 100)] == ["GEMM_WN"] * 3
    assert [fam(M, -2) for M in (8, 32, 100)] == ["GEMV_PACKED"] * 3
    # 1-bit codes have no matrix-core kernel: the streaming one runs whatever the preference
    W1 = torch.randint(0, 2, (N, K), generator=g).to(torch.uint8)
    l1 = GemLiteLinear(1, 128, K, N, DType.FP16, DType.FP16).pack(W1, torch.rand(N * K // 128, 1).half(), torch.rand(N * K // 128, 1).half())
    m1 = l1.get_meta_args()
    x = torch.zeros(40, K, dtype=torch.float16)
    a = _ext.build_matmul_args(x, l1.W_q, l1.scales, l1.zeros, None, torch.zeros(40, N, dtype=torch.float16), W_nbits=m1[1],
                               group_size=m1[2], unpack_mask=m1[3], elements_per_sample=m1[4], input_dtype=m1[5],
                               output_dtype=m1[6], acc_dtype=m1[7], meta_dtype=m1[8], channel_scale_mode=m1[9],
                               W_group_mode=m1[10], data_contiguous=m1[11], tile_config=-3)
    assert _ext.matmul_family(a) == "GEMV_PACKED"


def test_tuner_candidates_and_cache_file_round_trip(tmp_path):
    from gemlite_amd import tune
    assert tune.candidate_configs("GEMV_PACKED", 1, 4096)[0] == -1
    c = tune.candidate_configs("GEMM_WN", 64, 8192)
    assert c[0] == -1 and 64 + 1000 * 8 in c and all(v == -1 or v % 1000 in (32, 64, 128, 256) for v in c)
    assert tune.candidate_configs("GENERIC", 1, 64) == [-1]
    # entries the tuner writes survive cache_config / load_config in the reference's file layout
    GemLiteLinear.reset_config()
    key = gemlite_amd.core.config_key(64, 4096, 4096, 128, 8, gemlite_amd.core.get_type_id(1, 4))
    gemlite_amd.GEMLITE_CONFIG_CACHE.setdefault("GEMM", {})[key] = {"tile_config": 8064, "us": 12.5}
    f = str(tmp_path / "cfg.json")
    GemLiteLinear.cache_config(f)
    GemLiteLinear.reset_config()
    GemLiteLinear.load_config(f)
    assert gemlite_amd.core._cached_tile_config("GEMM", key) == 8064
    GemLiteLinear.reset_config()


def test_kernel_plugin_registry_has_the_reference_interface():
    """One class per matmul type with `kernel`, `matmul_type` and a static `forward` taking the
    reference's argument list (reference: gemlite/core.py:57-67, triton_kernels/gemm_kernels.py:741-746)."""
    import inspect
    m = gemlite_amd.GEMLITE_TRITON_MAPPING
    assert list(m) == gemlite_amd.GEMLITE_MATMUL_TYPES
    want = ["x", "W_q", "scales", "zeros", "scales_x", "W_nbits", "group_size", "unpack_mask", "elements_per_sample",
            "input_dtype", "output_dtype", "acc_dtype", "meta_dtype", "channel_scale_mode", "W_group_mode",
            "data_contiguous", "type_id", "meta_scale"]
    for name, cls in m.items():
        assert cls.matmul_type == name and isinstance(cls.kernel, list)
        assert list(inspect.signature(cls.forward).parameters) == want


def test_mxfp8_processor_packs_like_the_reference():
    """A8W8_MXFP_dynamic: fp8 codes kept as the [K, N] view, e8m0 scales [N, K/32] K-contiguous,
    W_group_mode 0 and channel_scale_mode 2 (post_scale) / 4 (reference: gemlite/helper.py:876-923);
    the module's weight quantiser agrees with the oracle's."""
    from oracle import oracle as orc
    g = torch.Generator().manual_seed(2)
    W = (torch.randn((64, 256), generator=g) * 0.03).to(torch.bfloat16)
    q = gemlite_amd.quant_utils.WeightQuantizerMXFP(compute_dtype=torch.bfloat16, device="cpu")
    codes, e8 = q.quantize_mxfp8(W, index=True)
    want_codes, want_e8 = orc.quantize_mxfp8_weights(W.float().numpy())
    assert np.array_equal(codes.view(torch.uint8).reshape(64, 256).numpy(), want_codes)
    assert np.array_equal(e8.view(torch.uint8).reshape(64, 8).numpy(), want_e8)
    for post_scale, csm in ((True, 2), (False, 4)):
        proc = gemlite_amd.helper.A8W8_MXFP_dynamic(device="cpu", dtype=torch.bfloat16, post_scale=post_scale)
        l = proc.from_weights(codes.view(64, 256), scales=e8.view(64, 8))
        assert (l.W_group_mode, l.channel_scale_mode) == (0, csm)
        assert l.input_dtype == gemlite_amd.DType.MXFP8 and l.scaled_activations and l.elements_per_sample == 1
        assert l.W_q.shape == (256, 64) and l.W_q.stride() == (1, 256) and l.W_q.dtype == torch.float8_e4m3fn
        assert l.scales.shape == (64, 8) and l.scales.stride() == (8, 1) and l.scales.dtype == torch.uint8


def test_weight_only_and_mixed_mx_processors():
    """A16W8_MXFP / A16W4_MXFP keep fp16 / bf16 activations (input and output type MXFP16 / MXBF16,
    W_group_mode 2, channel_scale_mode 0; reference: gemlite/helper.py:199-237, 384-420);
    A8W4_MXFP_dynamic is MXFP8 activations x MXFP4 weights (reference: gemlite/helper.py:950-1040).
    They run the streaming MX kernel; weight-only layers take the matrix cores above 2 rows."""
    g = torch.Generator().manual_seed(5)
    N, K = 64, 256
    W = (torch.randn((N, K), generator=g) * 0.03).to(torch.bfloat16)
    lin = torch.nn.Linear(K, N, bias=True, dtype=torch.bfloat16)
    lin.weight.data = W.clone()
    for cls, nbits, e, wdt in ((gemlite_amd.helper.A16W8_MXFP, 8, 1, torch.float8_e4m3fn),
                               (gemlite_amd.helper.A16W4_MXFP, 4, 2, torch.uint8)):
        for dtype, dt in ((torch.float16, DType.MXFP16), (torch.bfloat16, DType.MXBF16)):
            l = cls(device="cpu", dtype=dtype).from_linear(lin, del_orig=False)
            assert l.input_dtype == dt and l.output_dtype == dt and not l.scaled_activations
            assert (l.W_nbits, l.group_size, l.elements_per_sample) == (nbits, 32, e)
            assert (l.W_group_mode, l.channel_scale_mode) == (2, 0)
            assert l.W_q.shape == (K // e, N) and l.W_q.stride() == (1, K // e) and l.W_q.dtype == wdt
            assert l.scales.shape == (N, K // 32) and l.scales.dtype == torch.uint8 and l.scales.stride() == (K // 32, 1)
            assert l.bias.dtype == dtype
            assert gemlite_amd.DTYPE_TO_TORCH[l.get_meta_args()[6]] == dtype
            # streaming kernel up to 2 rows, weights straight to the matrix cores up to 16, the tiled GEMM above (K = 256 is a multiple of 128)
            for M, fam in ((1, "MX_STREAM"), (2, "MX_STREAM"), (3, "MX_SKINNY"), (16, "MX_SKINNY"), (17, "GEMM_KBYTES_MX"), (100, "GEMM_KBYTES_MX")):
                m = l.get_meta_args()
                x = torch.zeros(M, K, dtype=dtype)
                out = torch.zeros(M, N, dtype=dtype)
                a = _ext.build_matmul_args(
                    x, l.W_q, l.scales, l.zeros, None, out, W_nbits=m[1], group_size=m[2], unpack_mask=m[3],
                    elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6], acc_dtype=m[7], meta_dtype=m[8],
                    channel_scale_mode=m[9], W_group_mode=m[10], data_contiguous=m[11])
                assert _ext.matmul_family(a) == fam
    # from_weights of pre-quantised codes gives the same layer as from_linear
    q = gemlite_amd.quant_utils.WeightQuantizerMXFP(compute_dtype=torch.bfloat16, device="cpu")
    codes, e8 = q.quantize_mxfp4(W, index=True)
    l4 = gemlite_amd.helper.A16W4_MXFP(device="cpu", dtype=torch.float16).from_weights(codes.view(N, K), e8.view(N, K // 32))
    l4b = gemlite_amd.helper.A16W4_MXFP(device="cpu", dtype=torch.float16).from_linear(lin, del_orig=False)
    assert torch.equal(l4.W_q, l4b.W_q) and torch.equal(l4.scales, l4b.scales)
    # MXFP8 activations x MXFP4 weights
    for post_scale, csm in ((True, 2), (False, 4)):
        l = gemlite_amd.helper.A8W4_MXFP_dynamic(device="cpu", dtype=torch.bfloat16, post_scale=post_scale).from_linear(
            lin, del_orig=False)
        assert l.input_dtype == DType.MXFP8 and l.scaled_activations and (l.W_nbits, l.elements_per_sample) == (4, 2)
        assert (l.W_group_mode, l.channel_scale_mode) == (0, csm)
        # streaming up to 2 rows; 3..32 rows (K = 256 is one turn of the skinny kernel) in one launch on the mixed
        # fp8 x fp4 form of the scaled MFMA; the tiled GEMM above
        for M, fam in ((1, "MX_STREAM"), (2, "MX_STREAM"), (4, "K_SKINNY"), (5, "K_SKINNY"), (32, "K_SKINNY"),
                       (33, "GEMM_MXFP8"), (64, "GEMM_MXFP8")):
            xq = torch.zeros(M, K, dtype=torch.float8_e4m3fn)
            sx = torch.ones(M, 1) if post_scale else torch.full(((M + 31) // 32 * 32, K // 32), 127, dtype=torch.uint8)
            assert _family(l, M, None, scales_x=sx, x=xq) == fam
    # MXFP4 x MXFP4 whose K is a multiple of 32 but not of 128 streams too (the matrix-core kernel wants 128)
    K2 = 96
    codes = torch.randint(0, 16, (N, K2), generator=g).to(torch.uint8)
    e8 = torch.randint(110, 130, (N, K2 // 32), generator=g).to(torch.uint8)
    lm = gemlite_amd.helper.A4W4_MXFP_dynamic(device="cpu", dtype=torch.bfloat16).from_weights(codes, scales=e8)
    assert _family(lm, 3, None, scales_x=torch.full((32, K2 // 32), 127, dtype=torch.uint8),
                   x=torch.zeros(3, K2 // 2, dtype=torch.uint8)) == "MX_STREAM"


def test_block_quant_processor_packs_like_the_reference():
    """A8W8 with block_quant=True: W_group_mode 0, channel_scale_mode 5, fp32 block scales stored
    [K/128, N/128], accumulator type fp32, codes and scales equal to the oracle's per-block quantiser
    (reference: gemlite/helper.py:517-617); pre-quantised weights are taken as they are."""
    from oracle import oracle as orc
    g = torch.Generator().manual_seed(9)
    N, K = 200, 384
    W = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    for proc, to_int8, wdt, in_dt in ((gemlite_amd.helper.A8W8_INT8_dynamic, True, torch.int8, DType.INT8),
                                      (gemlite_amd.helper.A8W8_FP8_dynamic, False, torch.float8_e4m3fn, DType.FP8)):
        l = proc(device="cpu", block_quant=True).from_weights(W)
        assert (l.W_group_mode, l.channel_scale_mode) == (0, 5) and l.scaled_activations
        assert l.input_dtype == in_dt and l.acc_dtype == DType.FP32 and l.meta_dtype == DType.FP32
        assert l.W_q.shape == (K, N) and l.W_q.stride() == (1, K) and l.W_q.dtype == wdt
        assert l.scales.shape == (3, 2) and l.scales.dtype == torch.float32 and l.scales.is_contiguous()
        assert [int(v) for v in l.metadata.tolist()] == l.get_meta_args()
        codes, s = orc.quantize_block_weights(W.float().numpy(), to_int8)
        assert np.array_equal(l.scales.numpy(), s.T)
        got = l.W_q.t().contiguous()
        assert np.array_equal(got.numpy() if to_int8 else got.view(torch.uint8).numpy(), codes)
        l2 = proc(device="cpu", dtype=torch.bfloat16, block_quant=True).from_weights(
            l.W_q.t().contiguous(), scales=l.scales.t().contiguous())
        assert torch.equal(l2.W_q.view(torch.uint8), l.W_q.view(torch.uint8)) and torch.equal(l2.scales, l.scales)
        # (a layer this small streams its first 3 rows)
        for M, fam in ((1, "BLOCKQ_STREAM"), (3, "BLOCKQ_STREAM"), (4, "GEMM_BLOCKQ"), (5, "GEMM_BLOCKQ"), (300, "GEMM_BLOCKQ")):
            xq = torch.zeros(M, K, dtype=wdt)
            assert _family(l, M, None, scales_x=torch.ones(M, K // 128), x=xq) == fam


def test_ternary_processors_pack_like_the_reference():
    """(reference: gemlite/helper.py:1208-1321) 2-bit codes w + 1, scalar zero 1, fp32 channel scales."""
    g = torch.Generator().manual_seed(0)
    N, K = 256, 1024
    W = torch.randint(-1, 2, (N, K), generator=g).to(torch.float16)
    l = gemlite_amd.helper.A16W158_INT(device="cpu").from_weights(W, torch.tensor(0.037))
    assert (l.W_nbits, l.group_size, l.W_group_mode, l.channel_scale_mode) == (2, K, 1, 1)
    assert l.zeros.numel() == 1 and int(l.zeros) == 1 and l.scales.dtype == torch.float32 and not l.scaled_activations
    assert torch.equal(gemlite_amd.unpack_over_cols(l.W_q.t().contiguous(), 2, K, torch.uint8), (W + 1).to(torch.uint8))
    assert [_family(l, M, torch.float16) for M in (1, 16, 64, 65)] == ["GEMV_PACKED"] * 3 + ["GEMM_WN"]
    d = gemlite_amd.helper.A8W158_INT_dynamic(device="cpu").from_weights(W, torch.tensor(0.037))
    assert (d.W_group_mode, d.channel_scale_mode, d.input_dtype, d.acc_dtype) == (1, 3, DType.INT8, DType.INT32)
    assert d.scaled_activations and d.output_dtype == DType.FP16
    # int8 activations on packed codes have no kernel of their own: the library widens them to fp16 in the workspace
    # and runs the packed-code kernels, so the call reports those families, asks for the room, and refuses to run
    # without it before anything is launched
    import ctypes
    lib = _ext.load_library()
    for M, fam in ((1, "GEMV_PACKED"), (40, "GEMV_PACKED"), (300, "GEMM_WN")):
        xq = torch.zeros(M, K, dtype=torch.int8)
        m = d.get_meta_args()
        out = torch.zeros(M, N, dtype=torch.float16)
        a = _ext.build_matmul_args(xq, d.W_q, d.scales, d.zeros, torch.ones(M, 1), out, W_nbits=m[1], group_size=m[2],
                                   unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
                                   acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
                                   data_contiguous=m[11])
        assert _ext.matmul_family(a) == fam
        need = lib.gla_matmul_workspace_bytes(ctypes.byref(a))
        assert need >= (4 << 20) + M * K * 2
        assert lib.gla_matmul(ctypes.byref(a), None) == -5   # GLA_ERR_WORKSPACE_TOO_SMALL: no workspace given
        assert b"widened" in lib.gla_last_error()


# ------------------------------------------------------------------ workspace keyed by (device, stream)
def test_workspace_is_per_stream(monkeypatch):
    """Two streams never share scratch; one stream keeps its buffer across calls, grows by replacement and
    never frees the outgrown one (a captured graph may still point at it)."""
    monkeypatch.setattr(_ext, "_new_workspace", lambda size, device: torch.zeros(size, dtype=torch.uint8))
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: False)
    monkeypatch.setattr(_ext, "_workspaces", {})
    monkeypatch.setattr(_ext, "_retired_workspaces", [])
    monkeypatch.setattr(_ext, "_last_eager_key", {})
    dev = torch.device("cuda", 0)
    a = _ext.get_workspace(dev, 1024, stream=0x1000)
    b = _ext.get_workspace(dev, 1024, stream=0x2000)
    assert a.data_ptr() != b.data_ptr()
    assert _ext.get_workspace(dev, 4096, stream=0x1000) is a          # within the 8 MiB floor: same buffer
    big = _ext.get_workspace(dev, 20 << 20, stream=0x1000)
    assert big is not a and big.numel() >= 20 << 20 and a in _ext._retired_workspaces
    assert _ext.get_workspace(dev, 1024, stream=0x2000) is b
    assert _ext.get_workspace(torch.device("cuda", 1), 1024, stream=0x1000) is not big
    # under capture nothing is allocated: a stream with a buffer keeps it, a stream without one takes the
    # buffer of the stream this thread last launched on eagerly, and a request no buffer can serve is refused
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    assert _ext.get_workspace(dev, 1024, stream=0x1000) is big
    assert _ext.get_workspace(dev, 1024, stream=0x3000) is b           # last eager launch went to stream 0x2000
    with pytest.raises(RuntimeError, match="captured"):
        _ext.get_workspace(dev, 9 << 20, stream=0x3000)                # b holds 8 MiB
    assert 0x3000 not in [k[2] for k in _ext._workspaces]


def test_static_scratch_entry_point_refuses_oversize_without_a_gpu():
    lib = _ext.load_library()
    assert lib.gla_static_scratch_bytes() == 72 << 20
    a = _ext.MatmulArgs()
    a.struct_size = ctypes.sizeof(a)
    a.matmul_type = 3
    a.M, a.N, a.K = 512, 16384, 16384
    for f in ("x", "w", "scales", "zeros", "out"):
        setattr(a, f, 1 << 20)  # never dereferenced: the size check comes first
    a.x_stride_m, a.x_stride_k, a.w_stride_k, a.w_stride_n = 16384, 1, 16384, 1
    a.out_stride_m, a.out_stride_n, a.meta_stride_g, a.meta_stride_n = 16384, 1, 16384, 1
    a.W_nbits, a.group_size, a.unpack_mask, a.elements_per_sample = 2, 64, 3, 16
    a.input_dtype = a.output_dtype = a.meta_dtype = a.zeros_dtype = DType.BF16.value
    a.acc_dtype, a.channel_scale_mode, a.W_group_mode, a.data_contiguous = DType.FP32.value, 0, 4, 1
    a.w_dtype, a.tile_config = DType.INT32.value, 4256
    need = lib.gla_matmul_workspace_bytes(ctypes.byref(a))
    assert need > 72 << 20
    assert lib.gla_matmul_static(ctypes.byref(a), None) == -5
    assert b"gla_matmul_static" in lib.gla_last_error() and str(need).encode() in lib.gla_last_error()


# ------------------------------------------------------------------ torch custom op
def test_custom_op_fake_shape_and_dtype():
    """The registered op's fake implementation (what torch.compile sees) returns [..., N] in the layer's
    output type, on the input's device, without touching any kernel."""
    from torch._subclasses.fake_tensor import FakeTensorMode
    from gemlite_amd import core

    assert core.forward_functional_op is not None
    meta = [0, 4, 128, 15, 8, DType.BF16.value, DType.BF16.value, DType.FP32.value, DType.BF16.value, 0, 4, 1]
    with FakeTensorMode():
        x = torch.empty((3, 5, 256), dtype=torch.bfloat16)
        W_q = torch.empty((32, 96), dtype=torch.int32)
        s = torch.empty((2, 96), dtype=torch.bfloat16)
        out = core.forward_functional_op(x, None, [W_q, s, s, torch.empty((), dtype=torch.float32)], meta, -1)
        assert tuple(out.shape) == (3, 5, 96) and out.dtype == torch.bfloat16 and out.device == x.device
        meta[6] = DType.FP32.value
        out = torch.ops.gemlite.forward_functional(x, None, [W_q, s, s, torch.empty((), dtype=torch.float32)], meta, 4)
        assert out.dtype == torch.float32
    # eager calls take the plain function; the op is only used while a graph is being traced
    assert not torch.compiler.is_compiling()


# ------------------------------------------------------------------ patch_model
class _CountingProcessor:
    def __init__(self):
        self.seen = []

    def from_linear(self, layer):
        self.seen.append(layer.name)
        return torch.nn.Identity()


def test_patch_model_replaces_linears_and_skips_named_modules():
    from gemlite_amd import helper

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.q_proj = torch.nn.Linear(32, 32)
            self.norm = torch.nn.LayerNorm(32)
            self.mlp = torch.nn.Sequential(torch.nn.Linear(32, 64), torch.nn.ReLU(), torch.nn.Linear(64, 32))

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = torch.nn.ModuleList([Block(), Block()])
            self.lm_head = torch.nn.Linear(32, 100)
            self.visual = torch.nn.Sequential(torch.nn.Linear(32, 32))

    proc = _CountingProcessor()
    model = helper.patch_model(Model(), device="cpu", processor=proc)
    assert sorted(proc.seen) == sorted(
        [f"layers.{i}.{n}" for i in (0, 1) for n in ("q_proj", "mlp.0", "mlp.2")])
    assert isinstance(model.layers[0].q_proj, torch.nn.Identity) and isinstance(model.layers[1].mlp[2], torch.nn.Identity)
    assert isinstance(model.lm_head, torch.nn.Linear) and isinstance(model.visual[0], torch.nn.Linear)
    assert isinstance(model.layers[0].norm, torch.nn.LayerNorm)

    class HqqOnly:
        def from_hqqlinear(self, layer):
            return layer

    with pytest.raises(ImportError):
        helper.patch_model(Model(), device="cpu", processor=HqqOnly())


def test_weight_only_mx_batches_go_as_e4m3_terms_on_large_layers():
    """Host logic only: 3..16 rows of fp16 / bf16 on MXFP4 / MXFP8 weights.  The skinny kernel of the narrow formats takes
    them, as sums of e4m3 terms, where that measured faster: while the terms fit one 16-row tile (bf16 8 rows, fp16 5) on
    MXFP4 layers of 50 M weights or more and on MXFP8 layers with K >= 8192 and N <= 8192, with two tiles (bf16 up to 16
    rows) on long-K layers; GLA_TILE_PREFER_MID asks for it anywhere; the call then needs a workspace for the terms."""
    def layer(cls, dtype, N, K):
        e = 2 if cls is gemlite_amd.helper.A16W4_MXFP else 1
        W_q = torch.zeros((N, K // e), dtype=torch.uint8)
        if e == 1:
            W_q = W_q.view(torch.float8_e4m3fn)
        return cls(device="cpu", dtype=dtype).from_packed_weights(W_q, torch.full((N, K // 32), 127, dtype=torch.uint8))

    def args(l, M, dtype, tile=-1):
        m = l.get_meta_args()
        return _ext.build_matmul_args(
            torch.zeros(M, l.in_features, dtype=dtype), l.W_q, l.scales, l.zeros, None, torch.zeros(M, l.out_features, dtype=dtype),
            W_nbits=m[1], group_size=m[2], unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6],
            acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10], data_contiguous=m[11], tile_config=tile)

    W4, W8 = gemlite_amd.helper.A16W4_MXFP, gemlite_amd.helper.A16W8_MXFP
    bf, fp = torch.bfloat16, torch.float16
    fams = lambda l, dtype, Ms: [_ext.matmul_family(args(l, M, dtype)) for M in Ms]
    Ms = (2, 3, 5, 6, 8, 9, 16, 17)
    long_k = layer(W4, bf, 4096, 14336)
    assert fams(long_k, bf, Ms) == ["MX_STREAM"] + ["K_SKINNY"] * 6 + ["GEMM_KBYTES_MX"]
    assert fams(layer(W4, fp, 4096, 14336), fp, Ms) == ["MX_STREAM", "K_SKINNY", "K_SKINNY"] + ["MX_SKINNY"] * 4 + ["GEMM_KBYTES_MX"]
    assert fams(layer(W4, bf, 14336, 4096), bf, Ms) == ["MX_STREAM"] + ["K_SKINNY"] * 4 + ["MX_SKINNY"] * 2 + ["GEMM_KBYTES_MX"]
    small = layer(W4, bf, 4096, 4096)
    assert fams(small, bf, Ms) == ["MX_STREAM"] + ["MX_SKINNY"] * 6 + ["GEMM_KBYTES_MX"]
    assert fams(layer(W8, bf, 4096, 14336), bf, Ms) == ["MX_STREAM"] + ["K_SKINNY"] * 6 + ["GEMM_KBYTES_MX"]
    assert fams(layer(W8, bf, 14336, 4096), bf, Ms) == ["MX_STREAM"] + ["MX_SKINNY"] * 6 + ["GEMM_KBYTES_MX"]
    # the preference: honoured up to 16 (fp16: 10) rows, ignored outside; the terms and their scale bytes go to the workspace
    assert [_ext.matmul_family(args(small, M, bf, -4)) for M in (2, 3, 16, 17)] == ["MX_STREAM", "K_SKINNY", "K_SKINNY", "GEMM_KBYTES_MX"]
    small_fp = layer(W4, fp, 4096, 4096)
    assert [_ext.matmul_family(args(small_fp, M, fp, -4)) for M in (10, 11)] == ["K_SKINNY", "MX_SKINNY"]
    private = 4 << 20
    assert _ext.matmul_workspace_need(args(small, 8, bf, -4)) == private + 16 * 4096 + 16 * 128
    assert _ext.matmul_workspace_need(args(small, 9, bf, -4)) == private + 32 * 4096 + 32 * 128
    assert _ext.matmul_workspace_need(args(small_fp, 5, fp, -4)) == private + 16 * 4096 + 16 * 128
    assert _ext.matmul_workspace_need(args(small, 8, bf)) == 0


def test_packed_layers_unpack_their_weights_first_at_prefill_size():
    """Host logic only: from 4096 rows of fp16, 2048 of bf16 (or with GLA_TILE_PREFER_UNPACKED above 16) a call of the fused packed-weight GEMM
    becomes weight unpacking + the 16-bit GEMM, reported as that family, with N * K * 2 bytes more workspace; an explicit
    tile keeps the fused kernel."""
    g = torch.Generator().manual_seed(0)
    N, K = 512, 1024
    W_q = torch.randint(0, 16, (N, K), generator=g).to(torch.uint8)
    l = GemLiteLinear(4, 128, K, N, DType.FP16, DType.FP16).pack(W_q, torch.rand(N * K // 128, 1).half(), torch.rand(N * K // 128, 1).half())
    m = l.get_meta_args()

    def args(M, tile=-1):
        return _ext.build_matmul_args(torch.zeros(M, K, dtype=torch.float16), l.W_q, l.scales, l.zeros, None,
                                      torch.zeros(M, N, dtype=torch.float16), W_nbits=m[1], group_size=m[2], unpack_mask=m[3],
                                      elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6], acc_dtype=m[7], meta_dtype=m[8],
                                      channel_scale_mode=m[9], W_group_mode=m[10], data_contiguous=m[11], tile_config=tile)

    assert [_ext.matmul_family(args(M)) for M in (65, 4095, 4096, 9000)] == ["GEMM_WN", "GEMM_WN", "GEMM_16BIT", "GEMM_16BIT"]
    assert _ext.matmul_family(args(4096, -3)) == "GEMM_WN"   # the preference for the tiled GEMM keeps the fused kernel
    assert [_ext.matmul_family(args(M, -5)) for M in (16, 17, 300)] == ["GEMV_PACKED", "GEMM_16BIT", "GEMM_16BIT"]
    assert _ext.matmul_family(args(2048, 2128)) == "GEMM_WN"
    need = _ext.matmul_workspace_need(args(4096))
    assert need >= (4 << 20) + N * K * 2 and need % 256 == 0
    assert _ext.matmul_workspace_need(args(300, -5)) >= (4 << 20) + N * K * 2


def test_byte_weight_layers_convert_their_weights_first_from_2048_rows():
    """Host logic only: unpacked int8 weight bytes under 16-bit activations.  From 2048 rows (or with
    GLA_TILE_PREFER_UNPACKED above 16) the bytes are converted into the workspace and the 16-bit GEMM runs; the preference
    for the tiled GEMM keeps the byte-weight kernel."""
    N, K = 512, 1024
    W = (torch.randn(N, K) * 0.02).to(torch.bfloat16)
    for post_scale in (True, False):
        proc = gemlite_amd.helper.A16W8_INT8(device="cpu", post_scale=post_scale)
        W_q, s = gemlite_amd.quantize_weights_per_channel(W, torch.int8)
        proc.dtype = torch.bfloat16
        l = proc.from_weights(W_q, scales=s)
        m = l.get_meta_args()

        def args(M, tile=-1):
            return _ext.build_matmul_args(torch.zeros(M, K, dtype=torch.bfloat16), l.W_q, l.scales, l.zeros, None,
                                          torch.zeros(M, N, dtype=torch.bfloat16), W_nbits=m[1], group_size=m[2], unpack_mask=m[3],
                                          elements_per_sample=m[4], input_dtype=m[5], output_dtype=m[6], acc_dtype=m[7],
                                          meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10], data_contiguous=m[11],
                                          tile_config=tile)

        assert [_ext.matmul_family(args(M)) for M in (16, 17, 2047, 2048)] == ["GEMV_KMAJOR", "GEMM_KBYTES", "GEMM_KBYTES", "GEMM_16BIT"]
        assert [_ext.matmul_family(args(M, -5)) for M in (16, 17)] == ["GEMV_KMAJOR", "GEMM_16BIT"]
        assert _ext.matmul_family(args(4096, -3)) == "GEMM_KBYTES"
        assert _ext.matmul_workspace_need(args(2048)) >= (4 << 20) + N * K * 2
