#!/usr/bin/env python3
"""Write the golden vectors under tests/golden/ from the CPU oracle.

The reference ships no data files or known-answer vectors for this path (its tests draw random
inputs on the GPU), so these fixtures are produced by `oracle/oracle.py`, whose functions are
pinned one by one in tests/test_oracle.py.  They freeze inputs and expected outputs of every
stage of the path at small sizes, so that neither the oracle nor the HIP kernels can drift
unnoticed:

    python3 tests/golden/make_fixtures.py        # rewrites tests/golden/*.npz

Each .npz holds plain arrays only (loaded with numpy's default allow_pickle=False).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as orc  # noqa: E402


def f16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16)


def grouped_int_case(rng, nbits, N, K, gs, M, mode):
    """One packed-integer layer + activations + expected output for W_group_mode `mode`."""
    W_q = rng.integers(0, 2 ** nbits, size=(N, K), dtype=np.uint8)
    scales = f16(np.abs(rng.normal(0, 0.02, size=(K // gs, N))) + 1e-3)       # [K/gs, N]
    zeros = f16(rng.uniform(2 ** nbits * 3 / 8, 2 ** nbits * 9 / 16, size=(K // gs, N)))
    if mode == 4:  # stored zero is -z * s rounded once to fp16 (reference: gemlite/core.py:655-662)
        zeros_stored = f16(-zeros.astype(np.float32) * scales.astype(np.float32))
    else:
        zeros_stored = zeros
    x = f16(rng.normal(0, 1, size=(M, K)))
    packed = orc.pack_over_cols(W_q, nbits, 32)                                 # [N, K/e]
    y = orc.matmul_int(x.astype(np.float32), W_q.T.astype(np.float32),
                       scales.astype(np.float32) if mode >= 2 else None,
                       zeros_stored.astype(np.float32) if mode in (1, 3, 4) else None,
                       None, mode, 0, gs)
    return dict(W_q=W_q, packed=packed, scales=scales, zeros=zeros_stored, x=x, y=y,
                meta=np.array([nbits, gs, mode], dtype=np.int32))


def main():
    rng = np.random.default_rng(20240607)
    # ---- bit packing: every (bits, word width)
    out = {}
    for nbits in (1, 2, 4, 8):
        for width in (8, 16, 32, 64):
            e = width // nbits
            W = rng.integers(0, 2 ** nbits, size=(5, 3 * e), dtype=np.uint8)
            out[f"w_{nbits}_{width}"] = W
            out[f"p_{nbits}_{width}"] = orc.pack_over_cols(W, nbits, width)
    np.savez_compressed(os.path.join(HERE, "bitpack.npz"), **out)

    # ---- grouped integer weights x fp16 activations, every dequant mode that takes tensors
    out = {}
    for nbits, N, K, gs, M, mode in ((4, 64, 256, 128, 3, 4), (4, 64, 256, 64, 5, 3), (8, 32, 256, 128, 2, 3),
                                     (2, 64, 256, 64, 1, 4), (4, 64, 256, 128, 40, 4), (1, 32, 256, 128, 2, 3),
                                     (4, 64, 256, 128, 3, 2), (4, 64, 256, 128, 3, 1)):
        c = grouped_int_case(rng, nbits, N, K, gs, M, mode)
        tag = f"b{nbits}_g{gs}_m{M}_mode{mode}"
        for k, v in c.items():
            out[f"{tag}.{k}"] = v
    np.savez_compressed(os.path.join(HERE, "grouped_int.npz"), **out)

    # ---- activation quantisers (bit-exact outputs)
    x = rng.normal(0, 1.5, size=(7, 256)).astype(np.float32)
    x[2, :] = 0.0                       # all-zero row: scale clamps to 1e-6
    x[3, 5] = 300.0                     # outlier
    xb = orc.round_to_bf16(x)
    q8, s8 = orc.scale_activations_per_token(xb, True)
    qf, sf = orc.scale_activations_per_token(xb, False)
    q4, s4 = orc.scale_activations_mxfp4(xb)
    np.savez_compressed(os.path.join(HERE, "act_quant.npz"), x=xb, int8_codes=q8, int8_scales=s8,
                        fp8_codes=qf, fp8_scales=sf, mxfp4_codes=q4, mxfp4_scales=s4)

    # ---- INT8 x INT8 -> INT32 (exact) and the dynamic A8W8 epilogue
    A = rng.integers(-128, 128, size=(9, 256), dtype=np.int8)
    B = rng.integers(-128, 128, size=(40, 256), dtype=np.int8)
    acc = A.astype(np.int64) @ B.astype(np.int64).T
    sa = np.abs(rng.normal(0, 0.01, size=(9, 1))).astype(np.float32) + 1e-4
    sb = np.abs(rng.normal(0, 0.01, size=(1, 40))).astype(np.float32) + 1e-4
    np.savez_compressed(os.path.join(HERE, "int8.npz"), A=A, B=B, acc=acc.astype(np.int32), scales_x=sa, scales_w=sb,
                        y=(acc.astype(np.float64) * (sa.astype(np.float64) * sb.astype(np.float64))).astype(np.float32))

    # ---- MXFP4: weight quantiser, activation quantiser and the block-scaled product
    W = rng.normal(0, 0.02, size=(48, 256)).astype(np.float32)
    W = orc.round_to_bf16(W)
    codes, e8 = orc.quantize_mxfp4_weights(W)
    xa = orc.round_to_bf16(rng.normal(0, 1, size=(5, 256)).astype(np.float32))
    a_packed, a_scales = orc.scale_activations_mxfp4(xa)
    y = orc.matmul_mx(orc.unpack_fp4_bytes(a_packed), a_scales[:5], codes, e8)
    np.savez_compressed(os.path.join(HERE, "mxfp4.npz"), W=W, w_codes=codes, w_scales=e8, x=xa,
                        x_packed=a_packed, x_scales=a_scales, y=y)
    mx_and_block_quant()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))


def mx_and_block_quant():
    """Weight-only MX layers, MXFP8 activations x MXFP4 weights, MXFP8 quantisers, and 128 x 128 block
    quantisation (own generator, so that the files above do not depend on this section)."""
    rng = np.random.default_rng(20240608)
    N, K, M = 40, 256, 6
    W = orc.round_to_bf16(rng.normal(0, 0.02, size=(N, K)).astype(np.float32))
    W[:, 32:64] *= 8.0
    x = orc.round_to_bf16(rng.normal(0, 1, size=(M, K)).astype(np.float32))
    c4, e4 = orc.quantize_mxfp4_weights(W)
    c8, e8 = orc.quantize_mxfp8_weights(W)
    xq8, xs8 = orc.scale_activations_mxfp8(x)
    xqt, xst = orc.scale_activations_per_token(x, False)
    out = dict(W=W, x=x, w4_codes=c4, w4_scales=e4, w8_codes=c8, w8_scales=e8,
               x_mxfp8_codes=xq8, x_mxfp8_scales=xs8, x_token_codes=xqt, x_token_scales=xst,
               y_a16w4=orc.matmul_mx_mixed(x, "float", None, c4, "e2m1", e4),
               y_a16w8=orc.matmul_mx_mixed(x, "float", None, c8, "e4m3", e8),
               y_a8w4_token=orc.matmul_mx_mixed(xqt, "e4m3", None, c4, "e2m1", e4, scales_x=xst),
               y_a8w4_mx=orc.matmul_mx_mixed(xq8, "e4m3", xs8[:M], c4, "e2m1", e4))
    for name, to_int8 in (("int8", True), ("fp8", False)):
        wq, ws = orc.quantize_block_weights(W, to_int8)
        aq, asx = orc.scale_activations_per_block(x, to_int8)
        a = aq if to_int8 else orc.e4m3fn_decode(aq)
        b = wq if to_int8 else orc.e4m3fn_decode(wq)
        out.update({f"bq_{name}_w_codes": wq, f"bq_{name}_w_scales": ws, f"bq_{name}_x_codes": aq,
                    f"bq_{name}_x_scales": asx, f"bq_{name}_y": orc.matmul_block_quant(a, asx, b, ws)})
    np.savez_compressed(os.path.join(HERE, "mx_blockq.npz"), **out)


if __name__ == "__main__":
    main()
