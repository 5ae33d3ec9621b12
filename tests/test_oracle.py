"""Pins the CPU oracle (oracle/oracle.py, oracle/oracle_c.c) without the reference:
hand-computed answers, brute force, closed forms, library routines (torch's own
low-precision casts), and the assertions the reference's tests make."""
import ctypes
import os

import numpy as np
import pytest
import torch

from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------ bit packing
def test_pack_known_words():
    row = np.arange(8, dtype=np.uint8).reshape(1, 8)
    assert orc.pack_over_cols(row, 4, 32)[0, 0] == 0x76543210
    # a code >= 8 in the top nibble sets the sign bit of the int32 word
    row = np.array([[0, 0, 0, 0, 0, 0, 0, 15]], dtype=np.uint8)
    w = orc.pack_over_cols(row, 4, 32)
    assert w.dtype == np.int32 and w[0, 0] == -268435456  # 0xF0000000
    # 2-bit codes, 8-bit words: 3,2,1,0 -> 0b00_01_10_11
    assert orc.pack_over_cols(np.array([[3, 2, 1, 0]], dtype=np.uint8), 2, 8)[0, 0] == 0b00011011
    # 8-bit codes, 32-bit words: little-endian bytes
    assert orc.pack_over_cols(np.array([[0x11, 0x22, 0x33, 0x84]], dtype=np.uint8), 8, 32)[0, 0] == 0x84332211 - (1 << 32)


@pytest.mark.parametrize("nbits", [1, 2, 4, 8])
@pytest.mark.parametrize("width", [8, 16, 32, 64])
def test_pack_bruteforce_and_roundtrip(nbits, width):
    rng = np.random.default_rng(nbits * 100 + width)
    e = width // nbits
    W = rng.integers(0, 2 ** nbits, size=(5, 3 * e), dtype=np.uint8)
    packed = orc.pack_over_cols(W, nbits, width)
    assert packed.shape == (5, 3) and packed.dtype == orc._WORD_DTYPES[width]
    # brute force with python ints
    for r in range(5):
        for c in range(3):
            word = 0
            for i in range(e):
                word |= int(W[r, c * e + i]) << (nbits * i)
            assert int(packed[r, c]) & ((1 << width) - 1) == word
    assert np.array_equal(orc.unpack_over_cols(packed, nbits, 3 * e), W)


def test_c_pack_matches_numpy():
    lib = ctypes.CDLL(os.path.join(ROOT, "oracle", "liboracle_c.so"))
    rng = np.random.default_rng(0)
    for nbits in (1, 2, 4, 8):
        W = rng.integers(0, 2 ** nbits, size=(7, 64), dtype=np.uint8)
        out = np.zeros((7, 64 * nbits // 32), dtype=np.int32)
        lib.orc_pack_over_cols_32(
            W.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(7), ctypes.c_int64(64), ctypes.c_int(nbits),
            out.ctypes.data_as(ctypes.c_void_p),
        )
        assert np.array_equal(out, orc.pack_over_cols(W, nbits, 32))


# ------------------------------------------------------------------ codecs
def test_e2m1_table():
    assert list(orc.e2m1_decode(np.arange(8))) == [0, 0.5, 1, 1.5, 2, 3, 4, 6]
    assert list(orc.e2m1_decode(np.arange(8, 16))[1:]) == [-0.5, -1, -1.5, -2, -3, -4, -6]
    assert np.signbit(orc.e2m1_decode(8))


def test_e2m1_against_torch_fp4_dtype():
    # torch's packed fp4 dtype decodes the same nibbles (low nibble first), where this torch build converts it
    if hasattr(torch, "float4_e2m1fn_x2"):
        b = torch.arange(256, dtype=torch.uint8)
        try:
            vals = b.view(torch.float4_e2m1fn_x2).to(torch.float32)
        except Exception:
            pytest.skip("torch cannot convert float4_e2m1fn_x2 on this build")
        vals = vals.numpy().reshape(256, -1)
        if vals.shape[1] == 2:
            assert np.array_equal(vals[:, 0], orc.e2m1_decode(np.arange(256) & 15))
            assert np.array_equal(vals[:, 1], orc.e2m1_decode(np.arange(256) >> 4))


def test_e8m0_against_torch():
    b = torch.arange(255, dtype=torch.uint8)
    ref = b.view(torch.float8_e8m0fnu).to(torch.float32).numpy().astype(np.float64)
    mine = orc.e8m0_decode(np.arange(255))
    # torch returns fp32: 2^-127 is subnormal there but exact
    assert np.array_equal(mine.astype(np.float32), ref.astype(np.float32))
    assert np.isnan(orc.e8m0_decode(255))
    assert orc.e8m0_decode(127) == 1.0 and orc.e8m0_decode(128) == 2.0


def test_e4m3_codec_against_torch():
    b = torch.arange(256, dtype=torch.uint8)
    ref = b.view(torch.float8_e4m3fn).to(torch.float32).numpy()
    mine = orc.e4m3fn_decode(np.arange(256))
    ok = ~np.isnan(ref)
    assert np.array_equal(mine[ok], ref[ok]) and np.all(np.isnan(mine[~ok]))
    assert mine[0x7E] == 448.0
    # encode: random values, exact midpoints and the range ends, against torch's RNE cast
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.normal(0, 50, 20000), rng.uniform(-448, 448, 20000), rng.normal(0, 0.01, 5000),
        [0.0, -0.0, 448.0, -448.0, 2 ** -9, 2 ** -10, 3 * 2 ** -10],
        (ref[ok][:-1].astype(np.float64) + ref[ok][1:].astype(np.float64))[np.abs(ref[ok][:-1]) < 400] / 2,
    ]).astype(np.float32)
    x = np.clip(x, -448, 448)
    t = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    mine = orc.e4m3fn_encode(x)
    # +-0 may differ in sign bit handling only when x == -0.0
    assert np.array_equal(mine, t)


def test_round_to_bf16_against_torch():
    rng = np.random.default_rng(2)
    x = rng.normal(0, 3, 10000).astype(np.float32)
    assert np.array_equal(orc.round_to_bf16(x), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


# ------------------------------------------------------------------ dequant / matmul
def test_dequantize_closed_forms():
    q = np.array([[0, 5, 15]], dtype=np.uint8)
    s = np.array([[0.5]], dtype=np.float32)
    z = np.array([[7.0]], dtype=np.float32)
    assert np.array_equal(orc.dequantize(q, None, None, 0), [[0, 5, 15]])
    assert np.array_equal(orc.dequantize(q, None, z, 1), [[-7, -2, 8]])
    assert np.array_equal(orc.dequantize(q, None, 7, 1), [[-7, -2, 8]])
    assert np.array_equal(orc.dequantize(q, s, None, 2), [[0, 2.5, 7.5]])
    assert np.array_equal(orc.dequantize(q, s, z, 3), [[-3.5, -1, 4]])
    assert np.array_equal(orc.dequantize(q, s, -z * s, 4), [[-3.5, -1, 4]])  # fma form, z' = -z*s


def test_mode4_is_single_rounding():
    # q*s + z' where the double-rounded fp32 result differs from the fused one
    q = np.array([[3.0]], dtype=np.float32)
    s = np.array([[1.0 + 2 ** -23]], dtype=np.float32)
    z = np.array([[-3.0]], dtype=np.float32)
    fused = orc.dequantize(q, s, z, 4)[0, 0]
    assert fused == np.float32(3 * 2.0 ** -23)  # exact: 3*(1+2^-23) - 3
    assert np.float32(np.float32(q * s) + z)[0, 0] != fused  # q*s rounds to 3+2^-21 first


def test_matmul_reduces_to_library_matmul():
    rng = np.random.default_rng(3)
    M, K, N, gs = 3, 64, 8, 32
    x = rng.normal(size=(M, K)).astype(np.float32)
    q = rng.integers(0, 16, size=(K, N), dtype=np.uint8)
    ones = np.ones((K // gs, N), dtype=np.float32)
    zeros = np.zeros((K // gs, N), dtype=np.float32)
    ref = x.astype(np.float64) @ q.astype(np.float64)
    # scales = 1, zeros = 0 in every mode is the plain integer matmul
    for mode, s, z in [(0, None, None), (1, None, zeros), (2, ones, None), (3, ones, zeros), (4, ones, zeros)]:
        out = orc.matmul_int(x, q, s, z, None, mode, 0, gs)
        assert np.allclose(out, ref, rtol=1e-6), mode
    # a one-hot activation picks out one dequantised row
    s = rng.uniform(0.5, 2, size=(K // gs, N)).astype(np.float32)
    z = rng.uniform(0, 15, size=(K // gs, N)).astype(np.float32)
    onehot = np.zeros((1, K), dtype=np.float32)
    onehot[0, 37] = 1.0
    out = orc.matmul_int(onehot, q, s, z, None, 3, 0, gs)
    assert np.allclose(out[0], (q[37].astype(np.float32) - z[37 // gs]) * s[37 // gs], rtol=1e-6)
    # channel scaling is linear in each scale
    sx = rng.uniform(0.5, 2, size=(M, 1)).astype(np.float32)
    sn = rng.uniform(0.5, 2, size=(N,)).astype(np.float32)
    base = orc.matmul_int(x, q, None, None, None, 0, 0, gs).astype(np.float64)
    assert np.allclose(orc.matmul_int(x, q, None, None, sx, 0, 3, gs, scales_n=sn), base * sx * sn, rtol=1e-6)
    assert np.allclose(orc.matmul_int(x, q, None, None, sx, 0, 2, gs), base * sx, rtol=1e-6)
    assert np.allclose(orc.matmul_int(x, q, None, None, None, 0, 1, gs, scales_n=sn), base * sn, rtol=1e-6)


def test_int_acc_is_exact():
    rng = np.random.default_rng(4)
    x = rng.integers(-128, 128, size=(5, 256), dtype=np.int8)
    w = rng.integers(-128, 128, size=(256, 7), dtype=np.int8)
    out = orc.matmul_int(x, w, None, None, None, 0, 0, 256, int_acc=True)
    assert np.array_equal(out, (torch.from_numpy(x).long() @ torch.from_numpy(w).long()).numpy())
    out = orc.matmul_int(x, w.view(np.uint8) & 15, None, 7, None, 1, 0, 256, int_acc=True)
    assert np.array_equal(out, x.astype(np.int64) @ ((w.view(np.uint8) & 15).astype(np.int64) - 7))


def test_hqq_path_matches_grouped_matmul_and_c_port():
    rng = np.random.default_rng(5)
    M, N, K, gs = 2, 24, 256, 128
    x = rng.normal(size=(M, K)).astype(np.float32)
    Wq = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    scales = np.abs(rng.normal(0, 0.02, size=(N * K // gs, 1))).astype(np.float32)
    zeros = rng.uniform(6, 9, size=(N * K // gs, 1)).astype(np.float32)
    y = orc.hqq_dequant_matmul(x, Wq, scales, zeros, gs)
    # same thing through the kernel-side layout: [K, N] codes, [K/gs, N] metadata, mode 3
    y2 = orc.matmul_int(x, Wq.T, scales.reshape(N, -1).T, zeros.reshape(N, -1).T, None, 3, 0, gs)
    assert np.allclose(y, y2, rtol=1e-4, atol=1e-5)
    # C port
    lib = ctypes.CDLL(os.path.join(ROOT, "oracle", "liboracle_c.so"))
    W = np.zeros((N, K), dtype=np.float32)
    yc = np.zeros((M, N), dtype=np.float32)
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    lib.orc_hqq_dequantize(p(Wq), p(scales), p(zeros), ctypes.c_int64(N), ctypes.c_int64(K), ctypes.c_int64(gs), p(W), 2)
    lib.orc_matmul_nt_f32(p(x), p(W), ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_int64(K), p(yc), 2)
    assert np.allclose(yc, y, rtol=1e-4, atol=1e-5)


def test_matmul_mx_special_cases():
    rng = np.random.default_rng(6)
    M, N, K = 3, 5, 64
    a = rng.integers(0, 16, size=(M, K), dtype=np.uint8)
    b = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    unit = np.full((M, K // 32), 127, dtype=np.uint8)
    unit_b = np.full((N, K // 32), 127, dtype=np.uint8)
    ref = orc.e2m1_decode(a).astype(np.float64) @ orc.e2m1_decode(b).astype(np.float64).T
    assert np.array_equal(orc.matmul_mx(a, unit, b, unit_b), ref.astype(np.float32))
    # raising one block scale by one doubles that block's contribution only
    sa = unit.copy()
    sa[:, 1] = 128
    ref2 = ref + orc.e2m1_decode(a[:, 32:]).astype(np.float64) @ orc.e2m1_decode(b[:, 32:]).astype(np.float64).T
    assert np.array_equal(orc.matmul_mx(a, sa, b, unit_b), ref2.astype(np.float32))
    assert np.array_equal(orc.unpack_fp4_bytes(np.array([[0x21, 0xF8]], dtype=np.uint8)), [[1, 2, 8, 15]])


# ------------------------------------------------------------------ activation quant
def test_per_token_int8_properties():
    rng = np.random.default_rng(7)
    x = rng.normal(size=(6, 128)).astype(np.float32)
    q, s = orc.scale_activations_per_token(x, True)
    assert s.shape == (6, 1) and s.dtype == np.float32
    assert np.allclose(s[:, 0], np.abs(x).max(axis=1) / 127, rtol=1e-6)
    assert np.abs(q).max() <= 127 and np.all(np.abs(q).max(axis=1) == 127)
    assert np.all(np.abs(x - q.astype(np.float32) * s) <= s / 2 * (1 + 1e-5))
    # floor(y + 0.5): halves go up, also for negatives (-0.5 -> 0, -1.5 -> -1)
    x2 = np.array([[127.0, 0.5, 1.5, -0.5, -1.5, 2.5, -2.5, 0.0]], dtype=np.float32)
    q2, s2 = orc.scale_activations_per_token(x2, True)
    assert s2[0, 0] == 1.0 and list(q2[0]) == [127, 1, 2, 0, -1, 3, -2, 0]
    # all-zero row: scale floor 1e-6
    q3, s3 = orc.scale_activations_per_token(np.zeros((1, 8), dtype=np.float32), True)
    assert s3[0, 0] == np.float32(1e-6) and not q3.any()


def test_per_token_fp8_against_torch_formula():
    rng = np.random.default_rng(8)
    x = (rng.normal(size=(5, 256)) * rng.uniform(0.01, 10, size=(5, 1))).astype(np.float32)
    q, s = orc.scale_activations_per_token(x, False)
    t = torch.from_numpy(x)
    ts = (t.abs().amax(dim=1, keepdim=True) / 448.0).clamp_(min=1e-6)
    tq = (t / ts).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn)
    assert np.array_equal(s, ts.numpy())
    assert np.array_equal(q, tq.view(torch.uint8).numpy())


def test_mxfp4_exponent_rule():
    # exponent = ceil(log2(v)) + 127 for normal v, clamped to [97, 254]
    v = np.array([1.0, 1.0000001, 2.0, 3.0, 0.75, 0.5, 2.0 ** -40, 0.0, 2.0 ** 127, 3e38], dtype=np.float32)
    assert list(orc.next_power_of_2_exponent(v)) == [127, 128, 128, 129, 127, 126, 97, 97, 254, 254]


def test_mxfp4_exhaustive_binade():
    # every bf16 value in [1, 2) and [4, 8) (both signs), scaled so that the group maximum fixes
    # the scale at 1: codes must follow the strict-threshold rule
    mant = np.arange(128, dtype=np.uint32)
    vals = []
    for e in (127, 128, 129):
        bits = (e << 23) | (mant << 16)
        vals.append(bits.astype(np.uint32).view(np.float32))
    vals = np.concatenate(vals)
    vals = np.concatenate([vals, -vals, [0.0, -0.0, 0.25, -0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 0.1, -0.1]]).astype(np.float32)
    vals = vals[np.abs(vals) <= 6.0]
    pad = (-len(vals)) % 31
    vals = np.concatenate([vals, np.zeros(pad, dtype=np.float32)])
    groups = vals.reshape(-1, 31)
    x = np.concatenate([np.full((groups.shape[0], 1), 6.0, dtype=np.float32), groups], axis=1).reshape(1, -1)
    packed, scales = orc.scale_activations_mxfp4(x)
    assert np.all(scales[0] == 127) and np.all(scales[1:] == 127) and scales.shape[0] == 32
    codes = orc.unpack_fp4_bytes(packed)[0]
    flat = x[0]
    for v, c in zip(flat, codes):
        a = abs(float(v))
        mag = sum(a > t for t in (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0))
        assert c == (mag if v >= 0 else mag + 8), (v, c)
    # ties go toward zero; a negative value that rounds to zero keeps the sign bit; -0.0 does not
    look = {float(v): int(c) for v, c in zip(flat, codes)}
    assert look[0.25] == 0 and look[0.75] == 1 and look[2.5] == 4 and look[5.0] == 6
    assert look[-0.25] == 8 and look[float(np.float32(-0.1))] == 8
    neg_zero = [int(c) for v, c in zip(flat, codes) if v == 0 and np.signbit(v)]
    assert neg_zero and all(c == 0 for c in neg_zero)


def test_mxfp4_scale_and_error_bound():
    rng = np.random.default_rng(9)
    x = (rng.normal(size=(40, 256)) * rng.uniform(1e-3, 1e3, size=(40, 1))).astype(np.float32)
    packed, scales = orc.scale_activations_mxfp4(x)
    assert packed.shape == (40, 128) and scales.shape == (64, 8)
    assert np.all(scales[40:] == 127)
    amax = np.abs(x.reshape(40, 8, 32)).max(axis=2)
    s = orc.e8m0_decode(scales[:40])
    assert np.all(s >= amax / 6 * (1 - 1e-6)) and np.all(s / 2 < amax / 6)  # smallest power of two >= amax/6
    deq = orc.e2m1_decode(orc.unpack_fp4_bytes(packed)).reshape(40, 8, 32) * s[:, :, None]
    # e2m1 grid spacing is at most 2 (between 4 and 6): error <= 1 * s
    assert np.all(np.abs(deq - x.reshape(40, 8, 32)) <= s[:, :, None] * (1 + 1e-6))


# ------------------------------------------------------------------ weight quantisers
def test_quantize_mxfp4_weights():
    rng = np.random.default_rng(10)
    W = rng.normal(0, 0.02, size=(16, 128)).astype(np.float32)
    codes, e = orc.quantize_mxfp4_weights(W)
    assert codes.shape == (16, 128) and e.shape == (16, 4) and codes.max() <= 15
    s = orc.e8m0_decode(e)
    amax = np.abs(W.reshape(16, 4, 32)).max(axis=2)
    assert np.all(s >= amax / 6 * (1 - 1e-6)) and np.all(s / 2 < amax / 6)
    deq = orc.e2m1_decode(codes).reshape(16, 4, 32) * s[:, :, None]
    assert np.all(np.abs(deq - W.reshape(16, 4, 32)) <= s[:, :, None] * (1 + 1e-6))
    assert not np.any(codes == 8)  # -0 is never produced on the weight side
    # the torch-side quantiser of the product makes the same codes
    from gemlite_amd.quant_utils import WeightQuantizerMXFP

    q, sc = WeightQuantizerMXFP().quantize_mxfp4(torch.from_numpy(W), index=True)
    assert np.array_equal(q.view(16, 128).numpy(), codes)
    assert np.array_equal(sc.view(torch.uint8).view(16, 4).numpy(), e)


def test_quantize_per_channel():
    rng = np.random.default_rng(11)
    W = rng.normal(0, 0.02, size=(8, 64)).astype(np.float32)
    q, s = orc.quantize_per_channel(W, True)
    assert np.all(np.abs(q).max(axis=1) == 127)
    assert np.all(np.abs(W - q.astype(np.float32) * s) <= s / 2 * (1 + 1e-5))
    from gemlite_amd.quant_utils import quantize_weights_per_channel

    tq, ts = quantize_weights_per_channel(torch.from_numpy(W), torch.int8)
    assert np.array_equal(tq.numpy(), q) and np.array_equal(ts.numpy(), s)
    q8, s8 = orc.quantize_per_channel(W, False)
    tq8, ts8 = quantize_weights_per_channel(torch.from_numpy(W), torch.float8_e4m3fn)
    assert np.array_equal(tq8.view(torch.uint8).numpy(), q8) and np.array_equal(ts8.numpy(), s8)


def test_weight_quantizer_ties_by_hand():
    """Known answers written out by hand, independent of any quantiser code.

    MXFP4 weights (reference: gemlite/quant_utils.py:80-88): `searchsorted` without `right=True`
    returns the first threshold >= |v|, so a value exactly on a threshold takes the LOWER e2m1
    value.  A block whose amax is 6 has scale 2^0, so the values below are their own quotients.
    Negative values that round to zero lose their sign (index of the first match of -0.0 == 0.0).
    INT8 per channel (reference: gemlite/helper.py:651-657): `round_()` is round-half-to-even;
    a row whose amax is 127 has scale 1."""
    block = np.zeros(32, dtype=np.float32)
    vals = [6.0, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5.0, -6.0,
            0.26, 0.76, 2.51, 5.01, -0.0, 0.0]
    want = [7, 0, 1, 2, 3, 4, 5, 6, 0, 9, 10, 11, 12, 13, 14, 15,
            1, 2, 5, 7, 0, 0]
    block[:len(vals)] = vals
    for scale_exp in (0, -7, 5):   # the same quotients under other block scales (powers of two: exact)
        codes, e = orc.quantize_mxfp4_weights((block * np.float32(2.0 ** scale_exp)).reshape(1, 32))
        assert e.tolist() == [[127 + scale_exp]]
        assert codes[0, :len(vals)].tolist() == want, scale_exp
        assert not np.any(codes[0, len(vals):])

    row = np.zeros(16, dtype=np.float32)
    v8 = [127.0, 0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, -3.5, 2.49, 2.51, -126.5, 126.5]
    w8 = [127, 0, 2, 2, 4, 0, -2, -2, -4, 2, 3, -126, 126]
    row[:len(v8)] = v8
    q, s = orc.quantize_per_channel(row.reshape(1, 16), True)
    assert s.tolist() == [[1.0]] and q[0, :len(v8)].tolist() == w8
    # the same row scaled by a power of two: same codes, scaled scale
    q, s = orc.quantize_per_channel((row * np.float32(0.125)).reshape(1, 16), True)
    assert s.tolist() == [[0.125]] and q[0, :len(v8)].tolist() == w8
    # fp8: amax 448 -> scale 1; 17, 19 lie halfway between e4m3 neighbours (16, 18, 20) -> nearest even mantissa
    row8 = np.zeros(16, dtype=np.float32)
    row8[:5] = [448.0, 17.0, 19.0, -17.0, 1.0]
    q8, s8 = orc.quantize_per_channel(row8.reshape(1, 16), False)
    assert s8.tolist() == [[1.0]]
    assert orc.e4m3fn_decode(q8)[0, :5].tolist() == [448.0, 16.0, 20.0, -16.0, 1.0]


# ------------------------------------------------------------------ host logic
def test_matmul_type_table():
    # the decision table in the reference's source, including every batch size of the benchmark configs
    t = orc.get_matmul_type
    assert [t(m, 4) for m in (1, 2, 4, 5, 8, 16, 63, 64, 4096)] == [
        "GEMV_REVSPLITK", "GEMV_REVSPLITK", "GEMV_REVSPLITK", "GEMM_SPLITK", "GEMM_SPLITK", "GEMM_SPLITK",
        "GEMM_SPLITK", "GEMM", "GEMM"]
    assert [t(m, 8) for m in (1, 2, 3, 16, 64, 512)] == [
        "GEMV_SPLITK", "GEMV_SPLITK", "GEMM_SPLITK", "GEMM_SPLITK", "GEMM", "GEMM"]
    assert [t(m, 2) for m in (1, 16, 64, 512)] == ["GEMV_REVSPLITK", "GEMM_SPLITK", "GEMM", "GEMM"]
    assert [t(m, 4, True) for m in (1, 32, 1024, 8192)] == ["GEMM_SPLITK", "GEMM_SPLITK", "GEMM", "GEMM"]


def test_closest_m_table():
    g = orc.get_closest_m
    assert [g(m) for m in (0, 1, 2, 3, 5, 9, 17, 24, 25, 33, 48, 49, 65, 97, 129, 250, 1000, 3000, 4096, 5000)] == [
        1, 1, 2, 4, 8, 16, 24, 24, 32, 48, 48, 64, 96, 128, 192, 256, 1024, 3072, 4096, 4096]


def test_select_modes_like_reference_tests():
    s = orc.select_modes
    N = 2032
    assert s(False, 0, None, N, False) == (0, 0)                       # fp16 x fp16  (tests/test_int.py:111-113)
    assert s(True, N * 31, "tensor", N, False) == (4, 0)               # A16W4 grouped, fma (tests/test_int.py:136-139)
    assert s(True, N * 31, "tensor", N, False, fma_mode=False) == (3, 0)
    assert s(True, N, "int", N, False) == (1, 1)                       # int8 x Wn channelwise (tests/test_int.py:161-163)
    assert s(False, 0, "int", N, True) == (1, 2)                       # dynamic activations only (tests/test_int.py:188-190)
    assert s(True, N, "int", N, True) == (1, 3)                        # both scaled (tests/test_int.py:216-218)
    assert s(False, 0, None, N, True) == (0, 2)                        # fp8 x fp8 dynamic (tests/test_int.py:241-243)
    assert s(True, N, None, N, True) == (0, 3)                         # fp8 both scaled (tests/test_int.py:269-271)
    assert s(True, N, None, N, False) == (0, 1)                        # weight-only channelwise
    assert s(True, N * 132, None, N, True, mx=True) == (2, 0)          # micro-scaled formats


# ------------------------------------------------------------------ MXFP8 weights
def test_mxfp8_weight_quantizer_matches_torch_codecs_and_bounds():
    """oracle.quantize_mxfp8_weights against torch's own e4m3fn / e8m0 casts of the same closed form,
    plus what the format fixes: power-of-two scales, |w/s| <= 448, reconstruction within half an
    e4m3 step of the block's top binade."""
    g = torch.Generator().manual_seed(11)
    W = (torch.randn((24, 256), generator=g) * 0.05).float()
    W[3, 32:64] = 0.0                       # an all-zero block: scale clamps to 2^-30, codes 0
    W[5, 0] = 3.0                           # an outlier sets its block's scale
    codes, e8 = orc.quantize_mxfp8_weights(W.numpy())
    flat = W.reshape(-1, 32)
    ideal = flat.abs().amax(dim=1, keepdim=True) / 448.0
    s = (2 ** torch.ceil(torch.log2(ideal))).clamp_(min=2.0 ** -30)
    want_codes = (flat / s).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).reshape(24, 256).numpy()
    want_e8 = s.to(torch.float8_e8m0fnu).view(torch.uint8).reshape(24, 8).numpy()
    assert np.array_equal(codes, want_codes) and np.array_equal(e8, want_e8)
    assert e8[3, 1] == 127 - 30 and not codes[3, 32:64].any()
    sc = orc.e8m0_decode(e8)
    deq = orc.e4m3fn_decode(codes) * np.repeat(sc, 32, axis=1)
    # every block's largest value lands in the top binade [256, 448] * s or below; the e4m3 step there is 32 s
    assert np.all(np.abs(deq - W.numpy()) <= 16.0 * np.repeat(sc, 32, axis=1) + 1e-12)
    amax = np.abs(W.numpy()).reshape(24, 8, 32).max(axis=2)
    nz = amax > 0
    assert np.all(amax[nz] / sc[nz] <= 448.0) and np.all(amax[nz] / sc[nz] > 224.0)


def test_matmul_mxfp8_weights_closed_forms():
    """Unit scales reduce it to a plain matmul of the decoded values; raising one block's scale byte by
    one doubles exactly that block's contribution; the row scale multiplies the row."""
    rng = np.random.default_rng(5)
    M, N, K = 3, 4, 64
    a = rng.standard_normal((M, K)).astype(np.float32)
    b_codes = rng.integers(0, 0x77, size=(N, K), dtype=np.uint8)          # finite e4m3 codes
    ones = np.full((N, K // 32), 127, dtype=np.uint8)
    sx = np.ones((M, 1), dtype=np.float32)
    base = orc.matmul_mxfp8_weights(a, sx, b_codes, ones)
    B = orc.e4m3fn_decode(b_codes).astype(np.float64)
    assert np.allclose(base, a.astype(np.float64) @ B.T, rtol=1e-6)
    bumped = ones.copy(); bumped[2, 1] = 128
    want = base.astype(np.float64).copy()
    want[:, 2] += a[:, 32:].astype(np.float64) @ B[2, 32:]
    assert np.allclose(orc.matmul_mxfp8_weights(a, sx, b_codes, bumped), want, rtol=1e-6)
    sx2 = np.array([[1.0], [0.5], [3.0]], dtype=np.float32)
    assert np.allclose(orc.matmul_mxfp8_weights(a, sx2, b_codes, ones), base * sx2, rtol=1e-6)


def test_mxfp8_activation_quantizer_closed_forms():
    """oracle.scale_activations_mxfp8 against torch's e4m3fn cast of the same scaled values, the
    exponent rule on hand-picked maxima, padding rows, and the reconstruction bound of the format."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn((5, 128), generator=g).to(torch.bfloat16).float()
    x[1, 32:64] = 0.0
    x[2, 0] = 448.0; x[2, 1:32] = 0.25          # amax / 448 == 1 exactly: exponent 127, no round-up
    x[3, 0] = 449.0                             # just above: mantissa != 0 -> exponent 128
    codes, e8 = orc.scale_activations_mxfp8(x.numpy())
    assert codes.shape == (5, 128) and e8.shape == (32, 4) and np.all(e8[5:] == 127)
    assert e8[1, 1] == 97 and not codes[1, 32:64].any()
    assert e8[2, 0] == 127 and e8[3, 0] == 128
    s = torch.from_numpy(orc.e8m0_decode(e8[:5])).repeat_interleave(32, dim=1)
    want = (x / s).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(codes, want)
    deq = orc.e4m3fn_decode(codes) * s.numpy()
    # a value of magnitude v s with v <= 448 is off by at most half an e4m3 step at v: 2^(floor(log2 v) - 4)
    assert np.all(np.abs(deq - x.numpy()) <= np.maximum(np.abs(x.numpy()) / 16.0, s.numpy() * 2.0 ** -10) + 1e-30)


def test_matmul_mxfp8_block_scaled_closed_form():
    rng = np.random.default_rng(8)
    a = rng.integers(0, 0x77, size=(2, 64), dtype=np.uint8)
    b = rng.integers(0, 0x77, size=(3, 64), dtype=np.uint8)
    sa = np.array([[127, 130], [125, 127]], dtype=np.uint8)
    sb = np.array([[127, 127], [126, 129], [127, 120]], dtype=np.uint8)
    A, B = orc.e4m3fn_decode(a).astype(np.float64), orc.e4m3fn_decode(b).astype(np.float64)
    want = np.zeros((2, 3))
    for m in range(2):
        for n in range(3):
            for blk in range(2):
                sl = slice(32 * blk, 32 * blk + 32)
                want[m, n] += 2.0 ** (int(sa[m, blk]) - 127) * 2.0 ** (int(sb[n, blk]) - 127) * (A[m, sl] @ B[n, sl])
    assert np.allclose(orc.matmul_mxfp8(a, sa, b, sb), want, rtol=1e-6)


def test_matmul_mx_mixed_reduces_to_the_pinned_forms():
    """The general micro-scaled matmul agrees with the e2m1 x e2m1 and e4m3 x e4m3 forms pinned above,
    is a plain matmul for float activations and unit weight scales, scales one block's contribution
    by two when that block's weight scale goes up by one, and its per-row scale is a row scaling."""
    rng = np.random.default_rng(16)
    M, N, K = 3, 5, 96
    a4 = rng.integers(0, 16, size=(M, K), dtype=np.uint8)
    b4 = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    sa = rng.integers(120, 131, size=(M, K // 32), dtype=np.uint8)
    sb = rng.integers(120, 131, size=(N, K // 32), dtype=np.uint8)
    assert np.array_equal(orc.matmul_mx_mixed(a4, "e2m1", sa, b4, "e2m1", sb), orc.matmul_mx(a4, sa, b4, sb))
    a8 = rng.integers(0, 0x7F, size=(M, K), dtype=np.uint8)   # below the NaN code
    b8 = rng.integers(0, 0x7F, size=(N, K), dtype=np.uint8)
    assert np.array_equal(orc.matmul_mx_mixed(a8, "e4m3", sa, b8, "e4m3", sb), orc.matmul_mxfp8(a8, sa, b8, sb))
    rows = rng.uniform(0.5, 2.0, size=(M, 1)).astype(np.float32)
    assert np.array_equal(orc.matmul_mx_mixed(a8, "e4m3", None, b8, "e4m3", sb, scales_x=rows),
                          orc.matmul_mxfp8_weights(orc.e4m3fn_decode(a8), rows, b8, sb))
    # float activations, unit scales: a plain matmul against the decoded codes (small integers / halves: exact)
    x = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
    unit = np.full((N, K // 32), 127, dtype=np.uint8)
    assert np.array_equal(orc.matmul_mx_mixed(x, "float", None, b4, "e2m1", unit),
                          (x.astype(np.float64) @ orc.e2m1_decode(b4).astype(np.float64).T).astype(np.float32))
    # mixed kinds: fp8 activations x fp4 weights; bumping block 1 of the weight scales doubles that block
    base = orc.matmul_mx_mixed(a8, "e4m3", None, b4, "e2m1", unit).astype(np.float64)
    up = unit.copy()
    up[:, 1] = 128
    blk = orc.e4m3fn_decode(a8[:, 32:64]).astype(np.float64) @ orc.e2m1_decode(b4[:, 32:64]).astype(np.float64).T
    assert np.array_equal(orc.matmul_mx_mixed(a8, "e4m3", None, b4, "e2m1", up), (base + blk).astype(np.float32))


def test_block_quant_closed_forms():
    """Per-block activation quantiser, 128 x 128 weight quantiser and the block-scaled matmul."""
    rng = np.random.default_rng(21)
    M, N, K = 5, 200, 384
    x = rng.normal(size=(M, K)).astype(np.float32)
    x[1, 128:256] = 0.0          # an all-zero block takes the floor scale
    for to_int8, qmax in ((True, 127.0), (False, 448.0)):
        codes, s = orc.scale_activations_per_block(x, to_int8)
        assert codes.shape == (M, K) and s.shape == (M, 3) and s.dtype == np.float32
        amax = np.abs(x.reshape(M, 3, 128)).max(axis=2)
        assert np.array_equal(s, np.maximum(amax / np.float32(qmax), np.float32(1e-6)).astype(np.float32))
        assert s[1, 1] == np.float32(1e-6)
        vals = codes.astype(np.float32) if to_int8 else orc.e4m3fn_decode(codes)
        back = vals.reshape(M, 3, 128) * s[:, :, None]
        step = s[:, :, None] * (0.5 + 1e-3 if to_int8 else 1.0)  # int8: half a step; fp8: within 2^-4 relative
        bound = step if to_int8 else np.maximum(np.abs(x.reshape(M, 3, 128)) * 2.0 ** -4, s[:, :, None] * 2.0 ** -9) * 1.01
        assert np.all(np.abs(back - x.reshape(M, 3, 128)) <= bound)
        # each block is the per-token quantiser applied to that block alone, up to x*(1/s) vs x/s
        c_tok, s_tok = orc.scale_activations_per_token(x[:, :128], to_int8)
        assert np.array_equal(s_tok[:, 0], s[:, 0])
        assert np.mean(c_tok != codes[:, :128]) < 0.01
    # the extreme value of a block maps to the end of the range
    c8, s8 = orc.scale_activations_per_block(x, True)
    i = np.abs(x[0, :128]).argmax()
    assert abs(int(c8[0, i])) == 127
    # weights: N = 200 is padded to 256; scales [2, 3]; per-block amax; a block of zeros -> 1e-6
    W = (rng.normal(size=(N, K)) * 0.02).astype(np.float32)
    W[:128, 256:] = 0.0
    for to_int8, qmax in ((True, 127.0), (False, 448.0)):
        codes, s = orc.quantize_block_weights(W, to_int8)
        assert codes.shape == (N, K) and s.shape == (2, 3) and s[0, 2] == np.float32(1e-6)
        assert np.isclose(s[1, 0], np.abs(W[128:, :128]).max() / qmax, rtol=1e-6)
        vals = codes.astype(np.float32) if to_int8 else orc.e4m3fn_decode(codes)
        deq = vals * np.repeat(np.repeat(s, 128, axis=0)[:N], 128, axis=1)
        assert np.linalg.norm(deq - W) / np.linalg.norm(W) < (0.01 if to_int8 else 0.04)
    # int8 rounds half to even on the weight side: 2.5 steps -> 2
    Wt = np.zeros((128, 128), dtype=np.float32)
    Wt[0, 0], Wt[0, 1], Wt[0, 2] = 127.0, 2.5, 3.5
    ct, st = orc.quantize_block_weights(Wt, True)
    assert st[0, 0] == 1.0 and list(ct[0, :3]) == [127, 2, 4]
    # matmul: unit scales = plain integer matmul; doubling one activation block scale adds that block once more
    a = rng.integers(-128, 128, size=(M, K)).astype(np.float32)
    b = rng.integers(-128, 128, size=(N, K)).astype(np.float32)
    ones_a, ones_b = np.ones((M, 3), np.float32), np.ones((2, 3), np.float32)
    ref = a.astype(np.float64) @ b.astype(np.float64).T
    assert np.array_equal(orc.matmul_block_quant(a, ones_a, b, ones_b), ref.astype(np.float32))
    sa = ones_a.copy()
    sa[:, 1] = 2.0
    extra = a[:, 128:256].astype(np.float64) @ b[:, 128:256].astype(np.float64).T
    assert np.array_equal(orc.matmul_block_quant(a, sa, b, ones_b), (ref + extra).astype(np.float32))
    sb = ones_b.copy()
    sb[1, :] = 0.5   # rows 128.. of the weight
    want = ref.copy()
    want[:, 128:] *= 0.5
    assert np.array_equal(orc.matmul_block_quant(a, ones_a, b, sb), want.astype(np.float32))
