"""CPU restatement of the reference's quantized-matmul path (numpy).

TEST INFRASTRUCTURE ONLY.  Nothing in the product (`gemlite_amd/`) imports this
module; it is the checker used by `tests/`, `__graft_entry__.smoke()` and the
`cpu_baseline` leg of `bench.py`.

Every function restates one piece of the reference and cites it.  How each is
pinned (tests/test_oracle.py):

  pack_over_cols / unpack_over_cols   hand-computed words, brute force on all
                                      (nbits, width) pairs, round trips
  dequantize                          closed forms per mode on hand values
  select_modes                        the mode assertions of the reference's
                                      own tests (tests/test_int.py)
  matmul_int / matmul_mx              special cases that reduce to plain
                                      integer / float matmul, one-hot probes
  e2m1 / e8m0 / e4m3 codecs           all code points against torch's decoders
  scale_activations_per_token         |x - y*s| <= s/2, torch fp8 cast,
                                      floor(y+.5) ties
  scale_activations_mxfp4             exhaustive sweep of one binade of bf16
                                      values against the threshold rule,
                                      tie and -0 cases, scale = 2^ceil(log2)
  quantize_mxfp4_weights              dequantised error bound, e8m0 range
  get_matmul_type / get_closest_m     the table in the reference's source

No function needed an import of the reference to be pinned.
"""
import numpy as np

# ---------------------------------------------------------------------------
# bit packing
# ---------------------------------------------------------------------------
_WORD_DTYPES = {8: np.uint8, 16: np.int16, 32: np.int32, 64: np.int64}
_UWORD_DTYPES = {8: np.uint8, 16: np.uint16, 32: np.uint32, 64: np.uint64}


def pack_over_cols(W_q, W_nbits, packing_bitwidth):
    """word[r, j // e] |= W_q[r, j] << (W_nbits * (j % e)); signed storage types
    (reference: gemlite/bitpack.py:36-60, gemlite/dtypes.py:95-100).
    Returns the [rows, cols // e] matrix *before* the transpose."""
    e = packing_bitwidth // W_nbits
    rows, cols = W_q.shape
    assert cols % e == 0
    out = np.zeros((rows, cols // e), dtype=_UWORD_DTYPES[packing_bitwidth])
    for j in range(cols):
        shift = (j % e) * W_nbits
        out[:, j // e] |= W_q[:, j].astype(_UWORD_DTYPES[packing_bitwidth]) << np.array(
            shift, dtype=_UWORD_DTYPES[packing_bitwidth]
        )
    return out.view(_WORD_DTYPES[packing_bitwidth])


def unpack_over_cols(W_packed, W_nbits, num_output_cols):
    """(word >> (i * W_nbits)) & mask for i in range(e), arithmetic shift on the
    signed word (reference: gemlite/bitpack.py:146-162)."""
    rows, cols = W_packed.shape
    e = num_output_cols // cols
    mask = (1 << W_nbits) - 1
    words = W_packed.astype(np.int64)
    out = np.zeros((rows, cols, e), dtype=np.uint8)
    for i in range(e):
        out[:, :, i] = ((words >> (i * W_nbits)) & mask).astype(np.uint8)
    return out.reshape(rows, num_output_cols)


# ---------------------------------------------------------------------------
# low-precision float codecs
# ---------------------------------------------------------------------------
E2M1_VALUES = np.array(
    [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], dtype=np.float32
)  # reference: gemlite/quant_utils.py:36-41; gemlite/triton_kernels/gemv_kernels.py:17-25 (LUT/2)
E2M1_THRESHOLDS = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)
# reference: gemlite/quant_utils.py:53-59


def e2m1_decode(codes):
    return E2M1_VALUES[np.asarray(codes, dtype=np.int64) & 15]


def e8m0_decode(b):
    """2^(b - 127); 255 is NaN (OCP MX)."""
    b = np.asarray(b, dtype=np.int64)
    out = np.ldexp(np.float64(1.0), b - 127)
    out = np.where(b == 255, np.nan, out)
    return out


def e4m3fn_decode(b):
    """OCP e4m3fn: bias 7, no infinities, S.1111.111 is NaN."""
    b = np.asarray(b, dtype=np.int64)
    sign = np.where(b & 0x80, -1.0, 1.0)
    exp = (b >> 3) & 0xF
    man = b & 7
    normal = np.ldexp(1.0 + man / 8.0, exp - 7)
    sub = np.ldexp(man / 8.0, -6)
    val = np.where(exp == 0, sub, normal)
    val = np.where((exp == 15) & (man == 7), np.nan, val)
    return (sign * val).astype(np.float32)


_E4M3_POS = None


def e4m3fn_encode(x):
    """float32 -> e4m3fn byte, round to nearest even, |x| <= 448 expected
    (the cast the reference applies after clamping, gemlite/quant_utils.py:501-506)."""
    global _E4M3_POS
    if _E4M3_POS is None:
        _E4M3_POS = e4m3fn_decode(np.arange(0, 127)).astype(np.float64)  # 0 .. 448 ascending
    x = np.asarray(x, dtype=np.float32)
    a = np.abs(x).astype(np.float64)
    idx = np.searchsorted(_E4M3_POS, a, side="left")  # first code >= a
    idx = np.clip(idx, 0, 126)
    lo = np.clip(idx - 1, 0, 126)
    d_hi = _E4M3_POS[idx] - a
    d_lo = a - _E4M3_POS[lo]
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & (lo % 2 == 0))
    code = np.where(pick_lo, lo, idx)
    code = np.where(a >= _E4M3_POS[126], 126, code)
    return (code | np.where(np.signbit(x), 0x80, 0)).astype(np.uint8)


def round_to_bf16(x):
    """float32 -> nearest-even bf16, returned as float32."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


# ---------------------------------------------------------------------------
# dequantisation and matmul
# ---------------------------------------------------------------------------
def dequantize(q, scales, zeros, W_group_mode):
    """Modes 0..4 (reference: gemlite/triton_kernels/utils.py:73-105), in fp32."""
    q = q.astype(np.float32)
    if W_group_mode == 0:
        return q
    if W_group_mode == 1:
        return q - np.float32(zeros) if np.isscalar(zeros) else q - zeros.astype(np.float32)
    if W_group_mode == 2:
        return q * scales.astype(np.float32)
    if W_group_mode == 3:
        z = np.float32(zeros) if np.isscalar(zeros) else zeros.astype(np.float32)
        return (q - z) * scales.astype(np.float32)
    if W_group_mode == 4:
        # fma(q, s, z'): single rounding of q*s + z'
        return (q.astype(np.float64) * scales.astype(np.float64) + zeros.astype(np.float64)).astype(np.float32)
    raise ValueError(W_group_mode)


def dequantize_weights(q_kn, scales_gn, zeros_gn, W_group_mode, group_size):
    """Dequantise a [K, N] code matrix with [K/group_size, N] metadata."""
    K, N = q_kn.shape
    if W_group_mode == 0:
        return q_kn.astype(np.float32)
    if np.isscalar(zeros_gn) or (zeros_gn is not None and np.size(zeros_gn) == 1):
        z = np.float32(np.asarray(zeros_gn).reshape(-1)[0])
    elif zeros_gn is not None:
        z = np.repeat(zeros_gn.astype(np.float32), group_size, axis=0)[:K]
    else:
        z = None
    s = None if scales_gn is None else np.repeat(scales_gn.astype(np.float32), group_size, axis=0)[:K]
    return dequantize(q_kn, s, z, W_group_mode)


def matmul_int(x, w_kn, scales_gn, zeros_gn, scales_x, W_group_mode, channel_scale_mode, group_size,
               int_acc=False, scales_n=None):
    """out[M, N] of the grouped-integer kernels: dequantise, sum over K, channel scaling
    (reference: gemlite/triton_kernels/gemm_kernels.py:405-496).  Accumulation is in
    float64 (int64 when ``int_acc``), so this is the exact value every fp32 / int32
    accumulation order approximates."""
    if int_acc:
        w = w_kn.astype(np.int64)
        if W_group_mode == 1:
            w = w - int(np.asarray(zeros_gn).reshape(-1)[0])
        acc = x.astype(np.int64) @ w
        if channel_scale_mode == 0:
            return acc
        acc = acc.astype(np.float64)
    else:
        w = dequantize_weights(w_kn, scales_gn, zeros_gn, W_group_mode, group_size)
        acc = x.astype(np.float64) @ w.astype(np.float64)
    if channel_scale_mode == 1:
        acc = acc * scales_n.astype(np.float64).reshape(1, -1)
    elif channel_scale_mode == 2:
        acc = acc * scales_x.astype(np.float64).reshape(-1, 1)
    elif channel_scale_mode == 3:
        acc = acc * (scales_x.astype(np.float64).reshape(-1, 1) * scales_n.astype(np.float64).reshape(1, -1))
    return acc.astype(np.float32)


def hqq_dequant_matmul(x, W_q, scales, zeros, group_size):
    """The CPU path named as baseline: W = (W_q - zeros) * scales per group of
    `group_size` consecutive K, then y = x @ W.T, all fp32
    (reference: README.md:84, tests/test_int.py:54)."""
    N, K = W_q.shape
    W = ((W_q.astype(np.float32).reshape(-1, group_size) - zeros.astype(np.float32).reshape(-1, 1))
         * scales.astype(np.float32).reshape(-1, 1)).reshape(N, K)
    return x.astype(np.float32) @ W.T


def matmul_mx(a_codes, a_scales, b_codes, b_scales):
    """Block-scaled e2m1 x e2m1: sum over 32-blocks of 2^(sa-127) 2^(sb-127) sum_k a_k b_k
    (reference: gemlite/triton_kernels/gemm_kernels.py:696-726, tl.dot_scaled).
    a_codes [M, K] nibble codes, a_scales [M, K/32] bytes, b_codes [N, K], b_scales [N, K/32]."""
    A = e2m1_decode(a_codes).astype(np.float64) * np.repeat(e8m0_decode(a_scales), 32, axis=1)
    B = e2m1_decode(b_codes).astype(np.float64) * np.repeat(e8m0_decode(b_scales), 32, axis=1)
    return (A @ B.T).astype(np.float32)


def unpack_fp4_bytes(packed):
    """[R, K/2] bytes -> [R, K] nibble codes, even k in the low nibble
    (reference: gemlite/core.py:592-594 with gemlite/bitpack.py:36-60 at 4 bits / 8-bit words)."""
    p = np.asarray(packed, dtype=np.uint8)
    out = np.empty((p.shape[0], p.shape[1] * 2), dtype=np.uint8)
    out[:, 0::2] = p & 15
    out[:, 1::2] = p >> 4
    return out


# ---------------------------------------------------------------------------
# activation quantisation
# ---------------------------------------------------------------------------
def scale_activations_per_token(x, to_int8):
    """s = max(amax|row| / qmax, 1e-6) in fp32; y = clamp(x / s); int8: floor(y + 0.5)
    (the rounding the reference uses on AMD GPUs); fp8: e4m3fn cast
    (reference: gemlite/quant_utils.py:467-508, :289-296, :19-24).
    Returns (codes as int8 / e4m3fn bytes, scales [M, 1] fp32)."""
    x = np.asarray(x, dtype=np.float32)
    qmax = np.float32(127.0 if to_int8 else 448.0)
    qmin = np.float32(-128.0 if to_int8 else -448.0)
    s = np.abs(x).max(axis=1, keepdims=True).astype(np.float32) / qmax
    s = np.maximum(s, np.float32(1e-6)).astype(np.float32)
    y = np.clip((x / s).astype(np.float32), qmin, qmax)
    if to_int8:
        codes = np.floor(y + np.float32(0.5)).astype(np.int8)
    else:
        codes = e4m3fn_encode(y)
    return codes, s


def next_power_of_2_exponent(val):
    """Biased exponent of the smallest power of two >= val, clamped to [97, 254]
    (reference: gemlite/quant_utils.py:697-705 with eps_exp = -30)."""
    bits = np.asarray(val, dtype=np.float32).view(np.uint32)
    exp = ((bits >> 23) & 0xFF).astype(np.int64)
    exp = exp + ((bits & 0x7FFFFF) != 0)
    return np.clip(exp, 127 - 30, 254)


def scale_activations_mxfp4(x):
    """Per 32 values: e8m0 exponent from amax / 6, codes by 7 strict threshold compares,
    +8 when x / s < 0, two codes per byte (even k low); scales padded to a multiple of 32
    rows with 127 (reference: gemlite/quant_utils.py:2005-2135).
    Returns ([M, K/2] uint8, [M_pad, K/32] uint8)."""
    x = np.asarray(x, dtype=np.float32)
    M, K = x.shape
    g = x.reshape(M, K // 32, 32)
    amax = np.abs(g).max(axis=2)
    exp = next_power_of_2_exponent((amax / np.float32(6.0)).astype(np.float32))
    s = (exp.astype(np.uint32) << 23).view(np.float32)
    wq = (g / s[:, :, None]).astype(np.float32)
    idx = (np.abs(wq)[..., None] > E2M1_THRESHOLDS).sum(axis=-1)
    codes = np.where(wq >= 0, idx, idx + 8).astype(np.uint8).reshape(M, K)
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    M_pad = (M + 31) // 32 * 32
    scales = np.full((M_pad, K // 32), 127, dtype=np.uint8)
    scales[:M] = exp.astype(np.uint8)
    return packed, scales


def scale_activations_mxfp8(x):
    """Per 32 values: e8m0 exponent from amax / 448, codes = e4m3fn(clamp(x * (1 / s), -448, 448)),
    round to nearest even; scales padded to a multiple of 32 rows with 127
    (reference: gemlite/quant_utils.py:1025-1127; 1 / s is an exact power of two).
    Returns ([M, K] e4m3fn bytes, [M_pad, K/32] uint8)."""
    x = np.asarray(x, dtype=np.float32)
    M, K = x.shape
    g = x.reshape(M, K // 32, 32)
    amax = np.abs(g).max(axis=2)
    exp = next_power_of_2_exponent((amax / np.float32(448.0)).astype(np.float32))
    s = (exp.astype(np.uint32) << 23).view(np.float32)
    y = np.clip((g * (np.float32(1.0) / s)[:, :, None]).astype(np.float32), np.float32(-448.0), np.float32(448.0))
    codes = e4m3fn_encode(y.reshape(M, K))
    M_pad = (M + 31) // 32 * 32
    scales = np.full((M_pad, K // 32), 127, dtype=np.uint8)
    scales[:M] = exp.astype(np.uint8)
    return codes, scales


# ---------------------------------------------------------------------------
# weight quantisers
# ---------------------------------------------------------------------------
def quantize_mxfp4_weights(W):
    """s = clamp(2^ceil(log2(amax/6)), 2^-30); value = nearest e2m1 of |w/s| with ties
    down (searchsorted, left) times sign; code = position in E2M1_VALUES, +-0 -> 0
    (reference: gemlite/quant_utils.py:130-168, :80-99).
    Returns ([N, K] codes, [N, K/32] e8m0 bytes)."""
    W = np.asarray(W, dtype=np.float32)
    N, K = W.shape
    flat = W.reshape(-1, 32)
    ideal = np.abs(flat).max(axis=1, keepdims=True) / np.float32(6.0)
    with np.errstate(divide="ignore"):
        s = np.exp2(np.ceil(np.log2(ideal))).astype(np.float32)
    s = np.maximum(s, np.float32(2.0 ** -30))
    r = (flat / s).astype(np.float32)
    idx = np.searchsorted(E2M1_THRESHOLDS, np.abs(r), side="left")
    val = E2M1_VALUES[idx] * np.sign(r)
    codes = idx + np.where(val < 0, 8, 0)
    # e8m0 byte of a power of two is its biased exponent
    e = (s.view(np.uint32) >> 23).astype(np.uint8)
    return codes.astype(np.uint8).reshape(N, K), e.reshape(N, K // 32)


def quantize_mxfp8_weights(W):
    """Blocks of 32: s = clamp(2^ceil(log2(amax/448)), 2^-30); codes = e4m3fn(clamp(w/s, -448, 448))
    (reference: gemlite/quant_utils.py:102-128).  Returns ([N, K] e4m3fn bytes, [N, K/32] e8m0 bytes)."""
    W = np.asarray(W, dtype=np.float32)
    N, K = W.shape
    flat = W.reshape(-1, 32)
    ideal = np.abs(flat).max(axis=1, keepdims=True) / np.float32(448.0)
    with np.errstate(divide="ignore"):
        s = np.exp2(np.ceil(np.log2(ideal))).astype(np.float32)
    s = np.maximum(s, np.float32(2.0 ** -30))
    y = np.clip((flat / s).astype(np.float32), np.float32(-448.0), np.float32(448.0))
    e = (s.view(np.uint32) >> 23).astype(np.uint8)
    return e4m3fn_encode(y).reshape(N, K), e.reshape(N, K // 32)


def matmul_mxfp8_weights(a, scales_x, b_codes, b_scales):
    """fp8 activations a [M, K] (decoded values) with one fp32 scale per row applied after the K sum x
    MXFP8 weights: out[m, n] = scales_x[m] * sum_k a[m, k] * e4m3(b[n, k]) * 2^(sb[n, k/32] - 127)
    (reference: gemlite/triton_kernels/gemm_kernels.py:659-726 with channel_scale_mode 2; the block
    products are exact in fp32, only the accumulation order is free)."""
    A = np.asarray(a, dtype=np.float64)
    B = e4m3fn_decode(b_codes).astype(np.float64) * np.repeat(e8m0_decode(b_scales), 32, axis=1)
    return ((A @ B.T) * np.asarray(scales_x, dtype=np.float64).reshape(-1, 1)).astype(np.float32)


def matmul_mxfp8(a_codes, a_scales, b_codes, b_scales):
    """Block-scaled e4m3 x e4m3: sum over 32-blocks of 2^(sa-127) 2^(sb-127) sum_k a_k b_k
    (reference: gemlite/triton_kernels/gemm_kernels.py:659-726, tl.dot_scaled)."""
    A = e4m3fn_decode(a_codes).astype(np.float64) * np.repeat(e8m0_decode(a_scales), 32, axis=1)
    B = e4m3fn_decode(b_codes).astype(np.float64) * np.repeat(e8m0_decode(b_scales), 32, axis=1)
    return (A @ B.T).astype(np.float32)


def matmul_mx_mixed(a, a_kind, a_scales, b_codes, b_kind, b_scales, scales_x=None):
    """The general form of the reference's micro-scaled matmul: activations of kind `a_kind` in
    {"float" (fp16/bf16/fp32 values as they are), "e4m3" (bytes), "e2m1" (nibble codes)} with
    optional e8m0 block scales `a_scales` [M, K/32] (None = unit scales, what the reference passes
    for weight-only layers and for channel_scale_mode 2), weights of kind `b_kind` in {"e4m3",
    "e2m1"} [N, K] with e8m0 block scales [N, K/32], and an optional fp32 scale per activation row
    applied after the K sum (channel_scale_mode 2)
    (reference: gemlite/triton_kernels/gemm_kernels.py:563-581 operand kinds, :659-664 unit
    activation scales, :696 tl.dot_scaled, :714-717 per-row scale)."""
    def decode(v, kind):
        if kind == "e4m3":
            return e4m3fn_decode(v).astype(np.float64)
        if kind == "e2m1":
            return e2m1_decode(v).astype(np.float64)
        return np.asarray(v, dtype=np.float64)
    A = decode(a, a_kind)
    if a_scales is not None:
        A = A * np.repeat(e8m0_decode(a_scales), 32, axis=1)
    B = decode(b_codes, b_kind) * np.repeat(e8m0_decode(b_scales), 32, axis=1)
    out = A @ B.T
    if scales_x is not None:
        out = out * np.asarray(scales_x, dtype=np.float64).reshape(-1, 1)
    return out.astype(np.float32)


def scale_activations_per_block(x, to_int8, block=128):
    """One fp32 scale per (row, `block` values): s = max(amax / qmax, 1e-6); y = clamp(x * (1 / s));
    int8: floor(y + 0.5) (the rounding the reference uses on AMD GPUs), fp8: e4m3fn cast
    (reference: gemlite/quant_utils.py:2614-2676, :289-296).  Returns (codes [M, K], scales [M, K/block])."""
    x = np.asarray(x, dtype=np.float32)
    M, K = x.shape
    qmax = np.float32(127.0 if to_int8 else 448.0)
    qmin = np.float32(-128.0 if to_int8 else -448.0)
    t = x.reshape(M, K // block, block)
    s = np.maximum(np.abs(t).max(axis=2).astype(np.float32) / qmax, np.float32(1e-6)).astype(np.float32)
    r = (np.float32(1.0) / s).astype(np.float32)
    y = np.clip((t * r[:, :, None]).astype(np.float32), qmin, qmax)
    if to_int8:
        codes = np.floor(y + np.float32(0.5)).astype(np.int8)
    else:
        codes = e4m3fn_encode(y)
    return codes.reshape(M, K), s


def quantize_block_weights(W, to_int8, block=128):
    """One fp32 scale per block x block tile of the [N, K] weight (edges padded with zeros):
    s = max(amax / qmax, 1e-6); codes = clamp(W / s), int8 rounded half to even (torch.round), fp8
    e4m3fn cast (reference: gemlite/helper.py:556-580).  Returns (codes [N, K], scales [ceil(N/b), ceil(K/b)])."""
    W = np.asarray(W, dtype=np.float32)
    N, K = W.shape
    Np, Kp = -(-N // block) * block, -(-K // block) * block
    Wp = np.zeros((Np, Kp), dtype=np.float32)
    Wp[:N, :K] = W
    t = Wp.reshape(Np // block, block, Kp // block, block)
    qmax = np.float32(127.0 if to_int8 else 448.0)
    qmin = np.float32(-128.0 if to_int8 else -448.0)
    s = np.maximum(np.abs(t).max(axis=(1, 3)).astype(np.float32) / qmax, np.float32(1e-6)).astype(np.float32)
    y = np.clip((t / s[:, None, :, None]).astype(np.float32), qmin, qmax)
    if to_int8:
        codes = np.rint(y).astype(np.int8)
    else:
        codes = e4m3fn_encode(y)
    return codes.reshape(Np, Kp)[:N, :K].copy(), s


def matmul_block_quant(a, scales_a, b, scales_b, block=128):
    """out[m, n] = sum_kb (sum_{k in kb} a[m, k] b[n, k]) * scales_a[m, kb] * scales_b[n // block, kb]
    with a, b the decoded code values (reference: gemlite/triton_kernels/gemm_kernels.py:441-450)."""
    A = np.asarray(a, dtype=np.float64)
    B = np.asarray(b, dtype=np.float64)
    M, K = A.shape
    N = B.shape[0]
    sa = np.repeat(np.asarray(scales_a, dtype=np.float64), block, axis=1)[:, :K]
    sb = np.repeat(np.repeat(np.asarray(scales_b, dtype=np.float64), block, axis=0)[:N], block, axis=1)[:, :K]
    return ((A * sa) @ (B * sb).T).astype(np.float32)


def quantize_per_channel(W, to_int8):
    """s = max(amax_row / qmax, 1e-6); W_q = clamp(W / s); int8 rounds half to even
    (torch.round_), fp8 casts (reference: gemlite/helper.py:635-657)."""
    W = np.asarray(W, dtype=np.float32)
    qmax = np.float32(127.0 if to_int8 else 448.0)
    qmin = np.float32(-128.0 if to_int8 else -448.0)
    s = np.maximum(np.abs(W).max(axis=1, keepdims=True) / qmax, np.float32(1e-6)).astype(np.float32)
    y = np.clip((W / s).astype(np.float32), qmin, qmax)
    if to_int8:
        return np.rint(y).astype(np.int8), s
    return e4m3fn_encode(y), s


# ---------------------------------------------------------------------------
# host logic
# ---------------------------------------------------------------------------
def get_matmul_type(M, W_nbits, mx=False):
    """(reference: gemlite/core.py:163-179)"""
    if M >= 64:
        return "GEMM"
    limit = 4 if (W_nbits < 8 and not mx) else 2
    if M > limit:
        return "GEMM_SPLITK"
    if mx:
        return "GEMM_SPLITK"
    return "GEMV_REVSPLITK" if W_nbits < 8 else "GEMV_SPLITK"


def get_closest_m(M, max_m=4096):
    """Next value in {2^i} U {(2^i + 2^(i+1)) / 2, / 4 : 2^i >= 32, 2^(i+1) <= max_m}
    (reference: gemlite/triton_kernels/utils.py:185-220, mode 'next')."""
    vals = set()
    i = 0
    while 2 ** i <= max_m:
        v, nxt = 2 ** i, 2 ** (i + 1)
        vals.add(v)
        if v >= 32 and nxt <= max_m:
            vals.add((v + nxt) // 2)
            vals.add((v + nxt) // 4)
        i += 1
    if M > max_m:
        return max_m
    return min(v for v in vals if v >= M)


def select_modes(has_scales, scales_numel, zeros_kind, out_features, scaled_activations, fma_mode=True, mx=False):
    """(W_group_mode, channel_scale_mode) chosen by pack()
    (reference: gemlite/core.py:647-703, :733-735).
    zeros_kind: None | 'tensor' | 'int'."""
    wgm, csm = -1, 0
    if not has_scales and zeros_kind is None:
        wgm = 0
        csm = 2 if scaled_activations else 0
    channelwise = has_scales and scales_numel == out_features
    if zeros_kind is None:
        wgm = 2 if has_scales else 0
    elif zeros_kind == "tensor":
        wgm = 4 if (fma_mode and not channelwise) else 3
    else:
        wgm = 3 if has_scales else 1
    if not scaled_activations and channelwise:
        csm = 1
        wgm = 1 if zeros_kind is not None else 0
    if scaled_activations and not channelwise:
        csm = 2
    if scaled_activations and channelwise:
        csm = 3
        wgm = 1 if zeros_kind is not None else 0
    if mx:
        wgm, csm = 2, 0
    return wgm, csm
