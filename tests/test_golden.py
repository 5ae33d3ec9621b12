"""Golden vectors (tests/golden/*.npz, written by tests/golden/make_fixtures.py): the oracle must
reproduce them (CPU), and the HIP path must match them through the C ABI (GPU): codes and integer
accumulators bit for bit, float outputs within 1e-2 relative Frobenius error (and a tighter bound)."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FROB_TOL = 1e-2


def load(name):
    return np.load(os.path.join(GOLDEN, name))  # allow_pickle stays False


def rel_frob(y, ref):
    y, ref = np.asarray(y, np.float64), np.asarray(ref, np.float64)
    return float(np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-30))


def grouped_cases(z):
    tags = sorted({k.split(".")[0] for k in z.files})
    for t in tags:
        yield t, {k.split(".", 1)[1]: z[k] for k in z.files if k.startswith(t + ".")}


# ------------------------------------------------------------------ CPU: the oracle against the fixtures
def test_oracle_reproduces_bitpack():
    z = load("bitpack.npz")
    for nbits in (1, 2, 4, 8):
        for width in (8, 16, 32, 64):
            W, P = z[f"w_{nbits}_{width}"], z[f"p_{nbits}_{width}"]
            assert np.array_equal(orc.pack_over_cols(W, nbits, width), P)
            assert np.array_equal(orc.unpack_over_cols(P, nbits, W.shape[1]), W)
            # independent of the oracle: rebuild every word from its codes
            e = width // nbits
            words = P.astype(np.uint64) & np.uint64(2 ** width - 1)
            for j in range(e):
                assert np.array_equal((words >> np.uint64(nbits * j)) & np.uint64(2 ** nbits - 1), W[:, j::e])


def test_oracle_reproduces_grouped_int():
    z = load("grouped_int.npz")
    for tag, c in grouped_cases(z):
        nbits, gs, mode = (int(v) for v in c["meta"])
        W_q, x = c["W_q"], c["x"].astype(np.float32)
        s, zr = c["scales"].astype(np.float32), c["zeros"].astype(np.float32)
        y = orc.matmul_int(x, W_q.T.astype(np.float32), s if mode >= 2 else None, zr if mode in (1, 3, 4) else None,
                           None, mode, 0, gs)
        assert np.array_equal(y, c["y"]), tag
        assert np.array_equal(orc.pack_over_cols(W_q, nbits, 32), c["packed"]), tag
        # independent of the oracle's dequantize: the closed form per mode, in float64
        S = np.repeat(s.astype(np.float64), gs, axis=0)
        Z = np.repeat(zr.astype(np.float64), gs, axis=0)
        q = W_q.T.astype(np.float64)
        W = {1: q - Z, 2: q * S, 3: (q - Z) * S, 4: q * S + Z}[mode]
        # the oracle rounds dequantised weights like the reference (to the meta dtype); allow that much
        assert rel_frob(c["y"], x.astype(np.float64) @ W) < 2e-3, tag


def test_oracle_reproduces_act_quant_int8_mxfp4():
    z = load("act_quant.npz")
    x = z["x"]
    q8, s8 = orc.scale_activations_per_token(x, True)
    assert np.array_equal(q8, z["int8_codes"]) and np.array_equal(s8, z["int8_scales"])
    qf, sf = orc.scale_activations_per_token(x, False)
    assert np.array_equal(qf, z["fp8_codes"]) and np.array_equal(sf, z["fp8_scales"])
    q4, s4 = orc.scale_activations_mxfp4(x)
    assert np.array_equal(q4, z["mxfp4_codes"]) and np.array_equal(s4, z["mxfp4_scales"])
    # properties the numbers must have whatever produced them
    assert np.all(np.abs(x - z["int8_codes"].astype(np.float32) * z["int8_scales"]) <= z["int8_scales"] * 0.5 + 1e-12)
    assert z["int8_scales"][2, 0] == np.float32(1e-6) and not z["int8_codes"][2].any()
    assert z["mxfp4_scales"].shape == (32, 8) and np.all(z["mxfp4_scales"][7:] == 127)
    sc = np.repeat(orc.e8m0_decode(z["mxfp4_scales"][:7]), 32, axis=1)
    deq = orc.e2m1_decode(orc.unpack_fp4_bytes(z["mxfp4_codes"])) * sc
    assert np.all(np.abs(deq - x) <= sc)  # half the widest e2m1 step (4 -> 6) times the block scale
    amax = np.abs(x.reshape(7, 8, 32)).max(axis=2)
    nz = amax > 2.0 ** -20
    assert np.all(6.0 * orc.e8m0_decode(z["mxfp4_scales"][:7])[nz] >= amax[nz])  # no block overflows the format


def test_oracle_reproduces_int8_and_mxfp4_products():
    z = load("int8.npz")
    acc = z["A"].astype(np.int64) @ z["B"].astype(np.int64).T
    assert np.array_equal(acc, z["acc"])
    y = orc.matmul_int(z["A"], z["B"].T, None, None, z["scales_x"], 0, 3, 256, int_acc=True, scales_n=z["scales_w"])
    assert np.array_equal(y, z["y"])
    m = load("mxfp4.npz")
    codes, e8 = orc.quantize_mxfp4_weights(m["W"])
    assert np.array_equal(codes, m["w_codes"]) and np.array_equal(e8, m["w_scales"])
    a_p, a_s = orc.scale_activations_mxfp4(m["x"])
    assert np.array_equal(a_p, m["x_packed"]) and np.array_equal(a_s, m["x_scales"])
    assert np.array_equal(orc.matmul_mx(orc.unpack_fp4_bytes(a_p), a_s[:5], codes, e8), m["y"])
    assert rel_frob(m["y"], m["x"].astype(np.float64) @ m["W"].astype(np.float64).T) < 0.2  # format error only


# ------------------------------------------------------------------ GPU: the HIP path against the fixtures
@pytest.mark.gpu
def test_hip_bitpack_matches_golden(device):
    from gemlite_amd.bitpack import pack_weights_over_cols_hip, unpack_over_cols_hip
    z = load("bitpack.npz")
    for nbits in (1, 2, 4, 8):
        for width in (8, 16, 32, 64):
            W, P = z[f"w_{nbits}_{width}"], z[f"p_{nbits}_{width}"]
            packed, _ = pack_weights_over_cols_hip(torch.from_numpy(W).to(device), nbits, width, transpose=False)
            assert np.array_equal(packed.cpu().numpy(), P)
            assert np.array_equal(unpack_over_cols_hip(packed, nbits, W.shape[1]).cpu().numpy(), W)


@pytest.mark.gpu
@pytest.mark.parametrize("matmul_type", ["GEMV_REVSPLITK", "GEMM_SPLITK", "GEMM"])
def test_hip_grouped_int_matches_golden(device, matmul_type):
    import gemlite_amd
    from gemlite_amd import _ext
    z = load("grouped_int.npz")
    for tag, c in grouped_cases(z):
        nbits, gs, mode = (int(v) for v in c["meta"])
        W = torch.from_numpy(np.ascontiguousarray(c["packed"].T)).to(device)        # [K/e, N] int32
        s = torch.from_numpy(c["scales"]).to(device)
        zr = torch.from_numpy(c["zeros"]).to(device)
        x = torch.from_numpy(c["x"]).to(device)
        M, N = x.shape[0], W.shape[1]
        out = torch.empty((M, N), dtype=torch.float16, device=device)
        args = _ext.build_matmul_args(
            x, W, s if mode >= 2 else None, zr if mode in (1, 3, 4) else None, None, out,
            W_nbits=nbits, group_size=gs, unpack_mask=2 ** nbits - 1, elements_per_sample=32 // nbits,
            input_dtype=1, output_dtype=1, acc_dtype=0, meta_dtype=1, channel_scale_mode=0, W_group_mode=mode,
            data_contiguous=1, matmul_type=gemlite_amd.GEMLITE_MATMUL_TYPES_MAPPING[matmul_type])
        _ext.matmul(args, device)
        torch.cuda.synchronize()
        err = rel_frob(out.float().cpu().numpy(), c["y"])
        assert err <= FROB_TOL and err <= 1.5e-3, (tag, matmul_type, err)


@pytest.mark.gpu
def test_hip_act_quant_matches_golden(device):
    import gemlite_amd
    z = load("act_quant.npz")
    x = torch.from_numpy(z["x"]).to(torch.bfloat16).to(device)
    q8, s8 = gemlite_amd.scale_activations_per_token(x, torch.int8)
    assert np.array_equal(q8.cpu().numpy(), z["int8_codes"]) and np.array_equal(s8.cpu().numpy(), z["int8_scales"])
    qf, sf = gemlite_amd.scale_activations_per_token(x, torch.float8_e4m3fn)
    assert np.array_equal(qf.view(torch.uint8).cpu().numpy(), z["fp8_codes"])
    assert np.array_equal(sf.cpu().numpy(), z["fp8_scales"])
    q4, s4 = gemlite_amd.scale_activations_mxfp4(x)
    assert np.array_equal(q4.cpu().numpy(), z["mxfp4_codes"]) and np.array_equal(s4.cpu().numpy(), z["mxfp4_scales"])


@pytest.mark.gpu
def test_hip_int8_and_mxfp4_products_match_golden(device):
    from gemlite_amd import DType, GemLiteLinear, helper
    z = load("int8.npz")
    W = torch.from_numpy(z["B"]).to(device)
    layer = GemLiteLinear(8, None, W.shape[1], W.shape[0], DType.INT8, DType.INT32).pack(W, None, None)
    for mt in ("GEMV", "GEMM_SPLITK", "GEMM"):
        y = layer.forward_manual(torch.from_numpy(z["A"]).to(device), matmul_type=mt)
        assert y.dtype == torch.int32 and np.array_equal(y.cpu().numpy(), z["acc"]), mt
    m = load("mxfp4.npz")
    layer = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_weights(
        torch.from_numpy(m["w_codes"]).to(device), scales=torch.from_numpy(m["w_scales"]).to(device))
    y = layer(torch.from_numpy(m["x"]).to(torch.bfloat16).to(device))
    assert rel_frob(y.float().cpu().numpy(), m["y"]) <= 6e-3


def test_oracle_reproduces_mx_and_block_quant():
    z = load("mx_blockq.npz")
    W, x = z["W"], z["x"]
    M = x.shape[0]
    c4, e4 = orc.quantize_mxfp4_weights(W)
    c8, e8 = orc.quantize_mxfp8_weights(W)
    assert np.array_equal(c4, z["w4_codes"]) and np.array_equal(e4, z["w4_scales"])
    assert np.array_equal(c8, z["w8_codes"]) and np.array_equal(e8, z["w8_scales"])
    xq8, xs8 = orc.scale_activations_mxfp8(x)
    assert np.array_equal(xq8, z["x_mxfp8_codes"]) and np.array_equal(xs8, z["x_mxfp8_scales"])
    assert np.array_equal(orc.matmul_mx_mixed(x, "float", None, c4, "e2m1", e4), z["y_a16w4"])
    assert np.array_equal(orc.matmul_mx_mixed(x, "float", None, c8, "e4m3", e8), z["y_a16w8"])
    assert np.array_equal(orc.matmul_mx_mixed(z["x_token_codes"], "e4m3", None, c4, "e2m1", e4, scales_x=z["x_token_scales"]),
                          z["y_a8w4_token"])
    assert np.array_equal(orc.matmul_mx_mixed(xq8, "e4m3", xs8[:M], c4, "e2m1", e4), z["y_a8w4_mx"])
    # whatever produced the numbers: each result is the float matmul up to the formats' quantisation error,
    # and the dequantised weights are within half a code step of the originals
    ref = x.astype(np.float64) @ W.astype(np.float64).T
    for key, tol in (("y_a16w4", 0.2), ("y_a16w8", 0.05), ("y_a8w4_token", 0.2), ("y_a8w4_mx", 0.2)):
        assert rel_frob(z[key], ref) < tol, key
    deq8 = orc.e4m3fn_decode(z["w8_codes"]) * np.repeat(orc.e8m0_decode(z["w8_scales"]), 32, axis=1)
    assert np.all(np.abs(deq8 - W) <= np.abs(W) * 2.0 ** -4 + 1e-9)
    for name, to_int8, tol in (("int8", True, 0.02), ("fp8", False, 0.06)):
        wq, ws = orc.quantize_block_weights(W, to_int8)
        aq, asx = orc.scale_activations_per_block(x, to_int8)
        assert np.array_equal(wq, z[f"bq_{name}_w_codes"]) and np.array_equal(ws, z[f"bq_{name}_w_scales"])
        assert np.array_equal(aq, z[f"bq_{name}_x_codes"]) and np.array_equal(asx, z[f"bq_{name}_x_scales"])
        assert ws.shape == (1, 2) and asx.shape == (M, 2)
        assert rel_frob(z[f"bq_{name}_y"], ref) < tol, name


@pytest.mark.gpu
def test_hip_mx_and_block_quant_match_golden(device):
    import gemlite_amd
    from gemlite_amd import helper
    z = load("mx_blockq.npz")
    x = torch.from_numpy(z["x"]).to(torch.bfloat16).to(device)
    M = x.shape[0]
    # quantisers: bit for bit
    q, s = gemlite_amd.scale_activations_mxfp8(x)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), z["x_mxfp8_codes"]) and np.array_equal(s.cpu().numpy(), z["x_mxfp8_scales"])
    for name, dt in (("int8", torch.int8), ("fp8", torch.float8_e4m3fn)):
        q, s = gemlite_amd.scale_activations_per_block(x, dt)
        got = q.cpu().numpy() if dt == torch.int8 else q.view(torch.uint8).cpu().numpy()
        assert np.array_equal(got, z[f"bq_{name}_x_codes"]) and np.array_equal(s.cpu().numpy(), z[f"bq_{name}_x_scales"])
    w4, e4 = torch.from_numpy(z["w4_codes"]), torch.from_numpy(z["w4_scales"])
    w8 = torch.from_numpy(z["w8_codes"]).view(torch.float8_e4m3fn)
    cases = [
        ("y_a16w4", helper.A16W4_MXFP(device=device, dtype=torch.bfloat16).from_weights(w4, e4)),
        ("y_a16w8", helper.A16W8_MXFP(device=device, dtype=torch.bfloat16).from_weights(w8, torch.from_numpy(z["w8_scales"]))),
        ("y_a8w4_token", helper.A8W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_weights(w4, scales=e4)),
        ("y_a8w4_mx", helper.A8W4_MXFP_dynamic(device=device, dtype=torch.bfloat16, post_scale=False).from_weights(w4, scales=e4)),
        ("bq_int8_y", helper.A8W8_INT8_dynamic(device=device, dtype=torch.bfloat16, block_quant=True).from_weights(
            torch.from_numpy(z["bq_int8_w_codes"]), scales=torch.from_numpy(z["bq_int8_w_scales"]))),
        ("bq_fp8_y", helper.A8W8_FP8_dynamic(device=device, dtype=torch.bfloat16, block_quant=True).from_weights(
            torch.from_numpy(z["bq_fp8_w_codes"]).view(torch.float8_e4m3fn), scales=torch.from_numpy(z["bq_fp8_w_scales"]))),
    ]
    for key, layer in cases:
        for rows in (M, 2):   # 6 rows: matrix-core kernels; 2 rows: the streaming kernels
            y = layer(x[:rows])
            torch.cuda.synchronize()
            assert rel_frob(y.float().cpu().numpy(), z[key][:rows]) <= 6e-3, (key, rows)
