#!/usr/bin/env python3
"""Headline benchmark: A16W4 group-128 decode GEMV (M = 1) on the Llama-3-8B MLP shapes.

A "step" is one decode token through the two MLP linears of the benchmark configuration:
x[1,4096] -> W_up[14336,4096] -> h[1,14336] -> W_down[4096,14336] -> y[1,4096], both
A16W4 (HQQ asymmetric, group 128, 32-bit packing, fp16), launched through the C ABI
(`gla_matmul`).  Consecutive steps use different weight copies (several GB in total) so that no
cache level holds the weights between steps.  The metric is algorithmic bytes per step (every
operand read once, the output written once) divided by the time per step.

`extra` carries the other points of the benchmark table, each measured in the same run: the
4096^2 decode GEMV, the 16384^2 8-bit channel-wise and 2-bit group-64 layers at M = 1/16/64/512,
fp8 / int8 / MXFP4 GEMMs, MXFP4 at M = 1/32/1024/8192, the activation quantisers, and the rate at
which a plain read kernel streams the same footprints on this box.  Every bandwidth-bound point
rotates over distinct copies of its operands that add up to more than 512 MB, twice the 256 MB
Infinity Cache, and is timed as a HIP-graph replay with one launch per copy.

Prints ONE JSON line (see the `out` dict at the end).
"""
import argparse
import ctypes
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import gemlite_amd  # noqa: E402
from gemlite_amd import DType, GemLiteLinear, _ext  # noqa: E402

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
ROTATE_BYTES = 600e6   # distinct operand bytes a bandwidth-bound point cycles through (> 2 x 256 MB)

SHAPES = [(14336, 4096), (4096, 14336)]  # (N, K): up / down projection
GROUP = 128


def algorithmic_bytes(N, K, M=1, nbits=4, gs=GROUP, elt=2):
    """W_q + scales + zeros + x + out, each touched once (16-bit metadata and activations)."""
    return N * K * nbits // 8 + 2 * (N * K // gs) * elt + M * K * elt + M * N * elt


def make_layer(N, K, seed, device):
    g = torch.Generator(device="cpu").manual_seed(seed)
    W_q = torch.randint(0, 16, (N, K), generator=g, dtype=torch.int32).to(torch.uint8)
    scales = (torch.randn((N * K // GROUP, 1), generator=g) * 0.02).abs().to(torch.float16)
    zeros = (torch.rand((N * K // GROUP, 1), generator=g) * 3 + 6).to(torch.float16)
    layer = GemLiteLinear(4, GROUP, K, N, DType.FP16, DType.FP16)
    layer.pack(W_q.to(device), scales.to(device), zeros.to(device))
    return layer, (W_q, scales, zeros)


def clone_layer(layer):
    c = GemLiteLinear()
    c.load_state_dict({k: v.clone() for k, v in layer.state_dict().items()})
    return c


class Launch:
    """A prepared `gla_matmul` call: argument struct built once, launched on the current stream."""

    def __init__(self, lib, layer, x, out, device, scales_x=None, quantise_inside=False):
        """quantise_inside: x holds fp16 / bf16 rows and the kernel quantises them to the layer's input type itself."""
        m = layer.get_meta_args()
        self.lib = lib
        in_dt = m[5]
        if quantise_inside:
            pass
        elif scales_x is None and not gemlite_amd.dtypes.is_mx_dtype(in_dt):
            in_dt = gemlite_amd.TORCH_TO_DTYPE[x.dtype].value  # the kernels read x as the type it has
        elif scales_x is None:  # weight-only MX layer
            in_dt = DType.MXFP16.value if x.dtype == torch.float16 else DType.MXBF16.value
        self.args = _ext.build_matmul_args(
            x, layer.W_q, layer.scales, layer.zeros, scales_x, out,
            W_nbits=m[1], group_size=m[2], unpack_mask=m[3], elements_per_sample=m[4], input_dtype=in_dt,
            output_dtype=m[6], acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
            data_contiguous=m[11],  # matmul type left to the dispatcher
            x_quant_from=gemlite_amd.TORCH_TO_DTYPE[x.dtype].value if quantise_inside else 0,
        )
        need = lib.gla_matmul_workspace_bytes(ctypes.byref(self.args))
        if need < 0:
            raise RuntimeError(lib.gla_last_error().decode())
        if need > 0:
            ws = _ext.get_workspace(device, need, stream=0)   # one buffer for everything this script launches:
            self.args.workspace = ws.data_ptr()               # all of it runs in order on one stream
            self.args.workspace_bytes = ws.numel()
        self.keep = (layer, x, out, scales_x)

    def __call__(self):
        rc = self.lib.gla_matmul(ctypes.byref(self.args), torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError(self.lib.gla_last_error().decode())


class Timer:
    """Event timing on the stream the work is launched on (a side stream, also used for capture)."""

    def __init__(self):
        self.side = torch.cuda.Stream()

    def graph_us(self, fns, reps):
        """Average microseconds per call: one graph holding every callable of `fns` once, replayed `reps` times."""
        with torch.cuda.stream(self.side):
            for f in fns[:2]:
                f()
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=self.side):
                for f in fns:
                    f()
            gr.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(self.side)
            for _ in range(reps):
                gr.replay()
            e1.record(self.side)
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (reps * len(fns))

    def eager_us(self, fn, reps, warm=3):
        with torch.cuda.stream(self.side):
            for _ in range(warm):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(self.side)
            for _ in range(reps):
                fn()
            e1.record(self.side)
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps


def copies_for(nbytes):
    return max(2, int(ROTATE_BYTES // nbytes) + 1)


def bw_point(us, nbytes, **more):
    gbs = nbytes / us / 1e3
    return {"us": round(us, 2), "GB/s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
            "bytes": int(nbytes), **more}


def extra_points(lib, device, T, quick):
    """The other points of the benchmark table (synthetic data, same C ABI)."""
    from gemlite_amd import helper
    out = {}
    g = torch.Generator(device="cpu").manual_seed(7)
    stream = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731

    # ---- what a plain read kernel streams on this box (launch ramp and tail included), rotated buffers
    sink = torch.zeros(1, dtype=torch.float32, device=device)
    ceil = {}
    for label, nbytes in (("9MB", 8929280), ("31MB", 31232000), ("268MB", 268435456)):
        n = copies_for(nbytes)
        bufs = [torch.full((nbytes // 4,), 0x01010101, dtype=torch.int32, device=device) for _ in range(n)]

        def reader(b, shape):
            def run():
                rc = (lib.gla_probe_read(b.data_ptr(), b.numel() * 4, sink.data_ptr(), stream()) if shape is None else
                      lib.gla_probe_read_cfg(b.data_ptr(), b.numel() * 4, sink.data_ptr(), *shape, stream()))
                if rc != 0:
                    raise RuntimeError(lib.gla_last_error().decode())
            return run
        # a few launch shapes (workgroups, threads, 128-bit loads in flight per lane); the best one is the ceiling
        best = None
        for shape in (None, (256, 1024, 8), (224, 1024, 8), (256, 1024, 16), (512, 512, 8), (512, 1024, 4), (1024, 256, 16),
                      (2048, 256, 8), (256, 512, 16)):
            us = T.graph_us([reader(b, shape) for b in bufs], 4 if nbytes > 1e8 else 10)
            if best is None or us < best[0]:
                best = (us, shape)
        ceil[label] = bw_point(best[0], nbytes, copies=n,
                               launch_shape="default" if best[1] is None else
                               f"{best[1][0]} workgroups x {best[1][1]} threads x {best[1][2]} loads in flight")
        del bufs
    out["read_ceiling"] = {"kernel": "gla_probe_read / gla_probe_read_cfg (contiguous chunks, 128-bit non-temporal loads, nothing "
                                     "stored), best of nine launch shapes", **ceil}
    torch.cuda.empty_cache()

    # ---- C1: A16W4 gs128 fp16, K = N = 4096, M = 1 (and the same layer at M = 4096 below)
    N = K = 4096
    base, _ = make_layer(N, K, seed=11, device=device)
    nbytes = algorithmic_bytes(N, K)
    layers = [base] + [clone_layer(base) for _ in range(copies_for(nbytes) - 1)]
    x1 = torch.randn((1, K), generator=g).to(torch.float16).to(device)
    y1 = torch.empty((1, N), dtype=torch.float16, device=device)
    us = T.graph_us([Launch(lib, l, x1, y1, device) for l in layers], 10)
    out["gemv_a16w4_gs128_4096sq_M1"] = bw_point(
        us, nbytes, copies=len(layers), frac_of_read_ceiling=round(nbytes / us / 1e3 / ceil["9MB"]["GB/s"], 4))
    del layers

    # ---- the generic family's vector kernels at M = 1: 1-bit codes in groups of 64 (shorter than a step of the
    # streaming kernel) and 16-bit weights, both 4096 -> 14336
    Ng, Kg = 14336, 4096
    W1 = torch.randint(0, 2, (Ng, Kg), generator=g, dtype=torch.int32).to(torch.uint8)
    s1 = (torch.randn((Ng * Kg // 64, 1), generator=g) * 0.02).abs().to(torch.float16)
    z1 = torch.rand((Ng * Kg // 64, 1), generator=g).to(torch.float16)
    base1 = GemLiteLinear(1, 64, Kg, Ng, DType.FP16, DType.FP16).pack(W1.to(device), s1.to(device), z1.to(device))
    nbytes = algorithmic_bytes(Ng, Kg, nbits=1, gs=64)
    layers = [base1] + [clone_layer(base1) for _ in range(copies_for(nbytes) - 1)]
    yg = torch.empty((1, Ng), dtype=torch.float16, device=device)
    us = T.graph_us([Launch(lib, l, x1, yg, device) for l in layers], 10)
    out["gemv_a16w1_gs64_M1"] = bw_point(us, nbytes, copies=len(layers), N=Ng, K=Kg)
    del layers, base1, W1, s1, z1
    W16 = (torch.randn((Ng, Kg), generator=g) * 0.02).to(torch.float16)
    nbytes = Ng * Kg * 2 + Kg * 2 + Ng * 2
    layers = [GemLiteLinear(16, None, Kg, Ng, DType.FP16, DType.FP16).pack(W16.to(device), None, None)
              for _ in range(copies_for(nbytes))]
    us = T.graph_us([Launch(lib, l, x1, yg, device) for l in layers], 10)
    out["gemv_a16w16_fp16_M1"] = bw_point(us, nbytes, copies=len(layers), N=Ng, K=Kg)
    del layers, W16
    torch.cuda.empty_cache()

    # Sustained matrix rate of this board: a register-only MFMA loop (no memory traffic) with zero and
    # with random operand bits.  With random bits the power limit lowers the clock; that rate, not the
    # datasheet one, is what a GEMM on real data can at most reach here.
    probe = {}
    for name, dt in (("fp16", 1), ("bf16", 2), ("fp8", 3), ("int8", 4), ("mxfp4", 17)):
        rates = {}
        for label, rnd in (("zero_operands", 0), ("random_operands", 1)):
            flops = ctypes.c_double(0.0)

            def run():
                if lib.gla_probe_mfma(dt, rnd, 60000, sink.data_ptr(), ctypes.byref(flops), stream()) != 0:
                    raise RuntimeError(lib.gla_last_error().decode())
            us = T.eager_us(run, 3, warm=1)
            rates[label + "_TFLOP/s"] = round(flops.value / us / 1e6, 1)
        probe[name] = rates
    out["mfma_probe"] = probe

    def gemm_point(name, M, N, K, us, peak_tf, kind, us_zero=None, us_e2e=None):
        tf = 2.0 * M * N * K / us / 1e6
        sustained = probe[kind]["random_operands_TFLOP/s"]
        out[name] = {"M": M, "N": N, "K": K, "us": round(us, 1), "TFLOP/s": round(tf, 1),
                     "frac_of_peak": round(tf / peak_tf, 4), "peak_TFLOP/s": peak_tf,
                     "frac_of_sustained_mfma": round(tf / sustained, 4)}
        if us_zero is not None:
            # the same launch on all-zero operands: same instructions and memory traffic, but far less
            # switching power, so the clock stays up; the gap to `us` is the board's power limit
            out[name]["us_zero_operands"] = round(us_zero, 1)
            out[name]["frac_of_peak_zero_operands"] = round(2.0 * M * N * K / us_zero / 1e6 / peak_tf, 4)
        if us_e2e is not None:
            out[name]["us_with_activation_quantiser"] = round(us_e2e, 1)

    def zeroed(run, *tensors):
        """Time `run` again with the given operand tensors zero-filled (they are scratch copies)."""
        for t in tensors:
            t.view(torch.uint8).zero_()
        return T.eager_us(run, 20)

    # A16W4 gs128 fp16, M = 4096: as the library runs it (weights unpacked into the workspace, then the 16-bit MFMA
    # GEMM), and beside it the fused-dequant MFMA GEMM it hands over from (the preference for the tiled GEMM keeps it)
    M = 4096
    x = torch.randn((M, K), generator=g).to(torch.float16).to(device)
    y = torch.empty((M, N), dtype=torch.float16, device=device)
    fused = Launch(lib, base, x, y, device)
    fused.args.tile_config = -3  # GLA_TILE_PREFER_MATRIX
    us_fused = T.eager_us(fused, 40)
    run = Launch(lib, base, x, y, device)
    us = T.eager_us(run, 40)
    family = _ext.matmul_family(run.args)
    gemm_point("gemm_a16w4_gs128_fp16", M, N, K, us, 2500.0, "fp16", zeroed(run, x, base.W_q.data))
    out["gemm_a16w4_gs128_fp16"]["family"] = family
    out["gemm_a16w4_gs128_fp16"]["us_fused_dequant_kernel"] = round(us_fused, 1)
    del base, run, fused
    # an unquantised layer of the same shape (W_nbits = 16): fp16 x fp16 on the K-contiguous MFMA GEMM, and the vendor's
    # plain GEMM on the same operands in the same run
    W16 = (torch.randn((N, K), generator=g) * 0.02).to(torch.float16).to(device)
    l16 = GemLiteLinear(16, None, K, N, DType.FP16, DType.FP16).pack(W16, None, None)
    run = Launch(lib, l16, x, y, device)
    us = T.eager_us(run, 40)
    us_vendor = T.eager_us(lambda: torch.matmul(x, l16.W_q, out=y), 20)
    gemm_point("gemm_a16w16_fp16", M, N, K, us, 2500.0, "fp16", zeroed(run, x, W16))
    out["gemm_a16w16_fp16"]["vendor_library_same_operands"] = {"us": round(us_vendor, 1), "entry": "torch.matmul"}
    del l16, W16, x, y, run

    # ---- C3: bf16 activations, K = N = 16384: 8-bit channel-wise and 2-bit group-64 weights, M = 1 / 16 / 64 / 512
    N = K = 16384
    for tag, nbits, gs in (("a16w8_channelwise", 8, K), ("a16w2_gs64", 2, 64)):
        W_q = torch.randint(0, 2 ** nbits, (N, K), dtype=torch.uint8, device=device)
        groups = N * K // gs
        sc = (torch.randn((groups, 1), device=device) * 0.01).abs().clamp_(min=1e-4).to(torch.bfloat16)
        zr = (torch.rand((groups, 1), device=device) * (2 ** nbits) / 4 + (2 ** nbits) * 3 / 8).to(torch.bfloat16)
        layer = helper.A16Wn(device=device, post_scale=True).from_weights(W_q, sc, zr, nbits, gs)
        del W_q
        wbytes = N * K * nbits // 8 + 2 * groups * 2   # codes + scales + zeros
        layers = [layer] + [clone_layer(layer) for _ in range(copies_for(wbytes) - 1)]
        for M in (1, 16, 64, 512):
            if quick and M in (16, 64):
                continue
            xm = torch.randn((M, K), device=device).to(torch.bfloat16)
            ym = torch.empty((M, N), dtype=torch.bfloat16, device=device)
            us = T.graph_us([Launch(lib, l, xm, ym, device) for l in layers], 4)
            nbytes = wbytes + M * K * 2 + M * N * 2
            if M <= 16:
                out[f"gemv_{tag}_16384sq_M{M}"] = bw_point(us, nbytes, copies=len(layers))
            else:
                gemm_point(f"gemm_{tag}_16384sq_M{M}", M, N, K, us, 2500.0, "bf16")
                out[f"gemm_{tag}_16384sq_M{M}"].update({"GB/s": round(nbytes / us / 1e3, 1),
                                                        "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)})
        del layers, layer
        torch.cuda.empty_cache()

    # ---- C4: A8W8 fp8 / int8 dynamic, M = 4096, N = K = 8192: activation quantiser + GEMM
    M, N, K = 4096, 8192, 8192
    W = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16).to(device)
    xs = [torch.randn((M, K), device=device).to(torch.bfloat16) for _ in range(copies_for(M * K * 3))]
    x = xs[0]
    y = torch.empty((M, N), dtype=torch.bfloat16, device=device)
    for name, proc, wdt in (("fp8", helper.A8W8_FP8_dynamic, torch.float8_e4m3fn), ("int8", helper.A8W8_INT8_dynamic, torch.int8)):
        layer = proc(device=device).from_weights(W)
        xq, sx = gemlite_amd.scale_activations_per_token(x, wdt)
        run = Launch(lib, layer, xq, y, device, scales_x=sx)
        us = T.eager_us(run, 40)
        us_e2e = T.eager_us(lambda: layer(x), 20)
        # the vendor library on the same operands in the same run, for what this box's power limit lets a tuned
        # GEMM reach (not part of the product path): torch._scaled_mm (hipBLASLt, row-wise fp32 scales -> bf16) and
        # torch._int_mm (int32 output, no scales).  Absent or failing entry points are skipped.
        vendor = {}
        try:
            if name == "fp8":
                sb = layer.scales.float().reshape(1, N).contiguous()
                vfn = lambda: torch._scaled_mm(xq, layer.W_q, scale_a=sx.float().reshape(M, 1), scale_b=sb, out_dtype=torch.bfloat16)  # noqa: E731
            else:
                vfn = lambda: torch._int_mm(xq, layer.W_q)  # noqa: E731
            vendor["us"] = round(T.eager_us(vfn, 20), 1)
        except Exception as e:  # noqa: BLE001
            vendor = {"skipped": str(e)[:120]}
        us_zero = zeroed(run, xq, layer.W_q.data)
        if "us" in vendor:
            vendor["us_zero_operands"] = round(T.eager_us(vfn, 20), 1)
        gemm_point(f"gemm_a8w8_{name}", M, N, K, us, 5000.0, name, us_zero, us_e2e)
        out[f"gemm_a8w8_{name}"]["vendor_library_same_operands"] = dict(
            vendor, entry="torch._scaled_mm (row-wise scales)" if name == "fp8" else "torch._int_mm")
        # the quantiser alone, reading a different activation matrix every launch
        xq_o, sx_o = torch.empty_like(xq), torch.empty_like(sx)
        fns = [(lambda xi=xi: _ext.scale_activations_per_token(xi, xq_o, sx_o)) for xi in xs]
        us = T.graph_us(fns, 6)
        out[f"actquant_per_token_{name}"] = bw_point(us, M * K * 3 + M * 4, M=M, K=K, copies=len(xs))
        if name == "fp8":
            # what a plain streaming kernel with the same traffic (2 bytes read, 1 written per element, no row reduction)
            # reaches on this box: torch's elementwise cast bf16 -> uint8 of the same matrices
            u8 = torch.empty((M, K), dtype=torch.uint8, device=device)
            us_cast = T.graph_us([(lambda xi=xi: u8.copy_(xi)) for xi in xs], 6)
            out[f"actquant_per_token_{name}"]["elementwise_cast_same_traffic_us"] = round(us_cast, 2)
            out[f"actquant_per_token_{name}"]["speed_vs_that_cast"] = round(us_cast / us, 3)
        # decode: one row through the K-major streaming kernel (8-bit activations), weights rotated
        wbytes = N * K + N * 4
        layers = [layer] + [clone_layer(layer) for _ in range(copies_for(wbytes) - 1)]
        xq1, sx1 = gemlite_amd.scale_activations_per_token(x[:1].contiguous(), wdt)
        y1 = torch.empty((1, N), dtype=torch.bfloat16, device=device)
        us = T.graph_us([Launch(lib, l, xq1, y1, device, scales_x=sx1) for l in layers], 6)
        out[f"gemv_a8w8_{name}_M1"] = bw_point(us, wbytes + K + 4 + N * 2, N=N, K=K, copies=len(layers))
        # ... and end to end: the per-token quantiser of the bf16 row and the GEMV on its codes, both in the graph
        x1b = x[:1].contiguous()
        fns = []
        for l in layers:
            fns.append(lambda: _ext.scale_activations_per_token(x1b, xq1, sx1))
            fns.append(Launch(lib, l, xq1, y1, device, scales_x=sx1))
        us_pair = T.graph_us(fns, 6) * 2
        out[f"gemv_a8w8_{name}_M1"]["us_with_activation_quantiser"] = round(us_pair, 2)
        # ... and with the row quantised inside the GEMV (one launch; what forward() runs at decode sizes)
        us_in = T.graph_us([Launch(lib, l, x1b, y1, device, quantise_inside=True) for l in layers], 6)
        out[f"gemv_a8w8_{name}_M1"]["us_quantised_inside_the_matmul"] = round(us_in, 2)
        # a decode batch of 8 rows: both operands as they are into the MFMA, one launch
        xq8, sx8 = gemlite_amd.scale_activations_per_token(x[:8].contiguous(), wdt)
        y8 = torch.empty((8, N), dtype=torch.bfloat16, device=device)
        ls8 = [Launch(lib, l, xq8, y8, device, scales_x=sx8) for l in layers]
        out[f"gemv_a8w8_{name}_M8"] = bw_point(T.graph_us(ls8, 6), wbytes + 8 * (K + 4) + 8 * N * 2, N=N, K=K, copies=len(layers),
                                               family=_ext.matmul_family(ls8[0].args))
        del layer, layers, xq, sx, run, xq1, sx1, fns, ls8, xq8, sx8
    # MXFP8 weights, fp8 activations quantised per token (the reference processor's default)
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.bfloat16)
    lin.weight.data = W
    layer = helper.A8W8_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_linear(lin.to(device), del_orig=False)
    xq, sx = gemlite_amd.scale_activations_per_token(x, torch.float8_e4m3fn)
    run = Launch(lib, layer, xq, y, device, scales_x=sx)
    us = T.eager_us(run, 40)
    gemm_point("gemm_a8w8_mxfp8", M, N, K, us, 5000.0, "fp8", zeroed(run, xq, layer.W_q.data))
    del layer, lin, xq, sx, run
    # 128 x 128 block-quantised fp8 / int8 (channel_scale_mode 5)
    if not quick:
        for name, proc, wdt in (("fp8", helper.A8W8_FP8_dynamic, torch.float8_e4m3fn), ("int8", helper.A8W8_INT8_dynamic, torch.int8)):
            layer = proc(device=device, block_quant=True).from_weights(W)
            xq, sx = gemlite_amd.scale_activations_per_block(x, wdt)
            us = T.eager_us(Launch(lib, layer, xq, y, device, scales_x=sx), 30)
            gemm_point(f"gemm_a8w8_{name}_block_quant", M, N, K, us, 5000.0, name)
            xq_o, sx_o = torch.empty_like(xq), torch.empty_like(sx)
            us = T.graph_us([(lambda xi=xi: _ext.scale_activations_per_block(xi, xq_o, sx_o)) for xi in xs], 6)
            out[f"actquant_per_block_{name}"] = bw_point(us, M * K * 3 + M * K // 128 * 4, M=M, K=K, copies=len(xs))
            del layer, xq, sx
        # A16W8 weight-only int8 bytes (unpacked), bf16: M = 4096 (MFMA GEMM) and M = 1 (streaming, rotated)
        layer = helper.A16W8_INT8(device=device, post_scale=True).from_weights(W)
        us = T.eager_us(Launch(lib, layer, x, y, device), 20)
        gemm_point("gemm_a16w8_int8_bytes_bf16", M, N, K, us, 2500.0, "bf16")
        wbytes = N * K + N * 4
        layers = [layer] + [clone_layer(layer) for _ in range(copies_for(wbytes) - 1)]
        x1 = x[:1].contiguous()
        y1 = torch.empty((1, N), dtype=torch.bfloat16, device=device)
        us = T.graph_us([Launch(lib, l, x1, y1, device) for l in layers], 6)
        out["gemv_a16w8_int8_bytes_M1"] = bw_point(us, wbytes + K * 2 + N * 2, N=N, K=K, copies=len(layers))
        del layers, layer
    del W, xs, x, y
    torch.cuda.empty_cache()

    # ---- C5: MXFP4 x MXFP4, K = N = 16384, M = 1 / 32 / 1024 / 4096 / 8192
    N = K = 16384
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.bfloat16)
    lin.weight.data = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    layer = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_linear(lin.to(device))
    del lin
    wbytes = N * K // 2 + N * K // 32
    layers = [layer] + [clone_layer(layer) for _ in range(copies_for(wbytes) - 1)]
    for M in (1, 32):
        xm = torch.randn((M, K), device=device).to(torch.bfloat16)
        xq, sx = gemlite_amd.scale_activations_mxfp4(xm)
        ym = torch.empty((M, N), dtype=torch.bfloat16, device=device)
        ls = [Launch(lib, l, xq, ym, device, scales_x=sx) for l in layers]
        us = T.graph_us(ls, 6)
        out[f"gemv_a4w4_mxfp4_16384sq_M{M}"] = bw_point(us, wbytes + M * K // 2 + M * K // 32 + M * N * 2, copies=len(layers),
                                                        family=_ext.matmul_family(ls[0].args))
        del ls
        fns = []
        for l in layers:   # end to end: MXFP4 quantiser of the bf16 rows + GEMV, both in the graph
            fns.append(lambda: _ext.scale_activations_mxfp4(xm, xq, sx))
            fns.append(Launch(lib, l, xq, ym, device, scales_x=sx))
        out[f"gemv_a4w4_mxfp4_16384sq_M{M}"]["us_with_activation_quantiser"] = round(T.graph_us(fns, 6) * 2, 2)
        if M == 1:  # the rows the streaming kernel takes: quantised inside it (one launch; what forward() runs)
            us_in = T.graph_us([Launch(lib, l, xm, ym, device, quantise_inside=True) for l in layers], 6)
            out[f"gemv_a4w4_mxfp4_16384sq_M{M}"]["us_quantised_inside_the_matmul"] = round(us_in, 2)
        del fns
    # the same format on an 8192^2 layer at decode batches: weights straight from registers into the scaled MFMA
    N8 = K8 = 8192
    lin = torch.nn.Linear(K8, N8, bias=False, dtype=torch.bfloat16)
    lin.weight.data = (torch.randn((N8, K8), generator=g) * 0.02).to(torch.bfloat16)
    layer8 = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_linear(lin.to(device))
    del lin
    wbytes8 = N8 * K8 // 2 + N8 * K8 // 32
    layers8 = [layer8] + [clone_layer(layer8) for _ in range(copies_for(wbytes8) - 1)]
    for M in (8, 32):
        xm = torch.randn((M, K8), device=device).to(torch.bfloat16)
        xq, sx = gemlite_amd.scale_activations_mxfp4(xm)
        ym = torch.empty((M, N8), dtype=torch.bfloat16, device=device)
        ls = [Launch(lib, l, xq, ym, device, scales_x=sx) for l in layers8]
        us = T.graph_us(ls, 6)
        out[f"gemv_a4w4_mxfp4_8192sq_M{M}"] = bw_point(us, wbytes8 + M * K8 // 2 + M * K8 // 32 + M * N8 * 2, copies=len(layers8),
                                                       family=_ext.matmul_family(ls[0].args))
        del ls
    del layers8, layer8
    w_saved = layer.W_q.data.clone()
    for M in (1024, 4096, 8192):
        if quick and M == 1024:
            continue
        xm = torch.randn((M, K), device=device).to(torch.bfloat16)
        xq, sx = gemlite_amd.scale_activations_mxfp4(xm)
        ym = torch.empty((M, N), dtype=torch.bfloat16, device=device)
        run = Launch(lib, layer, xq, ym, device, scales_x=sx)
        us = T.eager_us(run, 12)
        us_e2e = T.eager_us(lambda: layer(xm), 8)
        us_zero = None
        vendor = None
        if M == 4096:
            # the vendor library on the same codes and block scales (torch._scaled_mm with e2m1 pairs and e8m0
            # scales; timing only, its scale layout conventions are not checked), as for fp8 above
            try:
                a4, b4 = xq.view(torch.float4_e2m1fn_x2), layer.W_q.data.view(torch.float4_e2m1fn_x2)
                sa8 = sx[:M].contiguous().view(torch.float8_e8m0fnu)
                sb8 = layer.scales.data.contiguous().view(torch.float8_e8m0fnu)
                vfn = lambda: torch._scaled_mm(a4, b4, scale_a=sa8, scale_b=sb8, out_dtype=torch.bfloat16)  # noqa: E731
                vendor = {"us": round(T.eager_us(vfn, 8), 1), "entry": "torch._scaled_mm (e2m1 x e2m1, e8m0 block scales)"}
            except Exception as e:  # noqa: BLE001
                vendor = {"skipped": str(e)[:120]}
            us_zero = zeroed(run, xq, layer.W_q.data)
            if "us" in vendor:
                vendor["us_zero_operands"] = round(T.eager_us(vfn, 8), 1)
            layer.W_q.data.copy_(w_saved)
        name = f"gemm_a4w4_mxfp4_M{M}" if M != 4096 else "gemm_a4w4_mxfp4"
        gemm_point(name, M, N, K, us, 10100.0, "mxfp4", us_zero, us_e2e)
        if vendor is not None:
            out[name]["vendor_library_same_operands"] = vendor
        if M == 4096:
            xs = [xm] + [torch.randn((M, K), device=device).to(torch.bfloat16) for _ in range(copies_for(M * K * 2.5) - 1)]
            xq_o, sx_o = torch.empty_like(xq), torch.empty_like(sx)
            us = T.graph_us([(lambda xi=xi: _ext.scale_activations_mxfp4(xi, xq_o, sx_o)) for xi in xs], 4)
            out["actquant_mxfp4"] = bw_point(us, M * K * 2 + M * K // 2 + M * K // 32, M=M, K=K, copies=len(xs))
            del xs
        del xm, xq, sx, ym, run
    del w_saved
    w_codes, w_scales = layer.W_q.data, layer.scales.data
    del layers

    if not quick:
        # Weight-only MXFP4 (bf16 activations as they are) on the same codes, rotated: M = 1, 2, 4, 8
        wo = helper.A16W4_MXFP(device=device, dtype=torch.bfloat16).from_packed_weights(
            w_codes.t(), w_scales.view(torch.float8_e8m0fnu))
        wos = [wo] + [clone_layer(wo) for _ in range(copies_for(wbytes) - 1)]
        for M in (1, 2, 4, 8):
            xm = torch.randn((M, K), device=device).to(torch.bfloat16)
            ym = torch.empty((M, N), dtype=torch.bfloat16, device=device)
            us = T.graph_us([Launch(lib, l, xm, ym, device) for l in wos], 4)
            out[f"gemv_a16w4_mxfp_M{M}"] = bw_point(us, wbytes + M * K * 2 + M * N * 2, copies=len(wos))
        del wos
        # ... at M = 4096 on the matrix cores (weights converted to bf16 fragments in registers)
        xm = torch.randn((4096, K), device=device).to(torch.bfloat16)
        ym = torch.empty((4096, N), dtype=torch.bfloat16, device=device)
        us = T.eager_us(Launch(lib, wo, xm, ym, device), 10)
        gemm_point("gemm_a16w4_mxfp_bf16", 4096, N, K, us, 2500.0, "bf16")
        # ... and under fp8 activations quantised per token (A8W4_MXFP_dynamic): the mixed fp8 x fp4 scaled MFMA
        a84 = helper.A8W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_packed_weights(
            w_codes.t(), scales=w_scales.view(torch.float8_e8m0fnu))
        xq, sx = gemlite_amd.scale_activations_per_token(xm, torch.float8_e4m3fn)
        us = T.eager_us(Launch(lib, a84, xq, ym, device, scales_x=sx), 10)
        gemm_point("gemm_a8w4_mxfp", 4096, N, K, us, 5000.0, "fp8")
    return out


def prefetch_experiment(lib, sets, launches, side, n_steps):
    """Microseconds per decode step when every launch runs beside a gla_prefetch of the next launch's weights,
    captured as a forked and re-joined branch of the same graph."""
    seq = []
    for i in range(n_steps):
        s, (up, down) = sets[i % len(sets)], launches[i % len(launches)]
        seq += [(up, s[0]), (down, s[1])]
    other = torch.cuda.Stream()
    with torch.cuda.stream(side):
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr, stream=side):
            for i, (launch, _) in enumerate(seq):
                nxt = seq[i + 1][1] if i + 1 < len(seq) else None
                if nxt is not None:
                    fork = torch.cuda.Event()
                    fork.record(side)
                    other.wait_event(fork)
                    for t in (nxt.W_q, nxt.scales, nxt.zeros):
                        if lib.gla_prefetch(t.data_ptr(), t.numel() * t.element_size(), 0, other.cuda_stream) != 0:
                            raise RuntimeError(lib.gla_last_error().decode())
                launch()
                if nxt is not None:
                    join = torch.cuda.Event()
                    join.record(other)
                    side.wait_event(join)
        gr.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(side)
        for _ in range(4):
            gr.replay()
        e1.record(side)
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (4 * n_steps)


def run_point(name, lib, device, T):
    """One GEMM point alone, a few launches: the workload of the per-kernel counter profiles under profiles/."""
    from gemlite_amd import helper
    g = torch.Generator(device="cpu").manual_seed(7)
    if name in ("gemm_a8w8_fp8", "gemm_a8w8_int8", "gemm_a8w8_fp8_block_quant", "gemm_a8w8_int8_block_quant"):
        M, N, K = 4096, 8192, 8192
        W = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16).to(device)
        x = torch.randn((M, K), generator=g).to(torch.bfloat16).to(device)
        fp8, blockq = "fp8" in name, name.endswith("block_quant")
        layer = (helper.A8W8_FP8_dynamic if fp8 else helper.A8W8_INT8_dynamic)(device=device, block_quant=blockq).from_weights(W)
        quant = gemlite_amd.scale_activations_per_block if blockq else gemlite_amd.scale_activations_per_token
        xq, sx = quant(x, torch.float8_e4m3fn if fp8 else torch.int8)
        peak = 5000.0
    elif name in ("gemm_a4w4_mxfp4", "gemm_a4w4_mxfp4_M8192"):
        M, N, K = (8192 if name.endswith("8192") else 4096), 16384, 16384
        lin = torch.nn.Linear(K, N, bias=False, dtype=torch.bfloat16)
        lin.weight.data = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
        layer = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_linear(lin.to(device))
        x = torch.randn((M, K), generator=g).to(torch.bfloat16).to(device)
        xq, sx = gemlite_amd.scale_activations_mxfp4(x)
        peak = 10100.0
    elif name in ("gemm_a16w4_gs128_fp16", "gemm_a16w4_gs128_fp16_fused"):
        # as the library runs it (from 4096 rows of fp16: weights unpacked into the workspace, then the 16-bit GEMM), or
        # kept on the fused-dequant kernel with the preference for the tiled GEMM
        M = N = K = 4096
        layer, _ = make_layer(N, K, seed=11, device=device)
        xq, sx = torch.randn((M, K), generator=g).to(torch.float16).to(device), None
        peak = 2500.0
    elif name in ("gemv_a16w8_channelwise_16384sq_M16", "gemm_a16w8_channelwise_16384sq_M64"):
        # 8-bit channel-wise codes under bf16 at 16 / 64 rows: the mid-batch kernel (one layer, a few launches)
        M, N, K = (16 if name.endswith("M16") else 64), 16384, 16384
        W_q = torch.randint(0, 256, (N, K), dtype=torch.uint8, device=device)
        sc = (torch.randn((N, 1), device=device) * 0.01).abs().clamp_(min=1e-4).to(torch.bfloat16)
        zr = (torch.rand((N, 1), device=device) * 64 + 96).to(torch.bfloat16)
        layer = helper.A16Wn(device=device, post_scale=True).from_weights(W_q, sc, zr, 8, K)
        del W_q
        xq, sx = torch.randn((M, K), device=device).to(torch.bfloat16), None
        peak = 2500.0
    else:
        sys.exit(f"bench.py: unknown --point {name}")
    y = torch.empty((M, N), dtype=torch.float16 if name.startswith("gemm_a16w4_gs128_fp16") else torch.bfloat16, device=device)
    launch = Launch(lib, layer, xq, y, device, scales_x=sx)
    if name.endswith("_fused"):
        launch.args.tile_config = -3  # GLA_TILE_PREFER_MATRIX
        need = lib.gla_matmul_workspace_bytes(ctypes.byref(launch.args))
        ws = _ext.get_workspace(device, max(need, 1), stream=0)
        launch.args.workspace, launch.args.workspace_bytes = ws.data_ptr(), ws.numel()
    us = T.eager_us(launch, 10)
    tf = 2.0 * M * N * K / us / 1e6
    print(json.dumps({"point": name, "M": M, "N": N, "K": K, "us": round(us, 1), "TFLOP/s": round(tf, 1),
                      "frac_of_peak": round(tf / peak, 4)}))


def cpu_baseline(host_tensors, x_host, y_gpu, threads):
    """The reference's CPU path (HQQ dequantize + fp32 matmul) on this box's host cores, on whole steps of the
    same workload: the C restatement (oracle/oracle_c.c, OpenMP), which also gives the parity check, and
    the same two operations written with torch (`W = (W_q - z) * s`; `x @ W.T`), as a user of the reference
    without a GPU would run them."""
    import numpy as np

    lib = ctypes.CDLL(os.path.join(ROOT, "oracle", "liboracle_c.so"))
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    i64 = ctypes.c_int64
    arrs = []
    for (W_q, scales, zeros) in host_tensors:
        arrs.append((np.ascontiguousarray(W_q.numpy()), scales.float().numpy().reshape(-1).copy(),
                     zeros.float().numpy().reshape(-1).copy()))
    Wbuf = [np.empty(a[0].shape, dtype=np.float32) for a in arrs]

    def step(x):
        v = x
        for (W_q, s, z), W in zip(arrs, Wbuf):
            N, K = W_q.shape
            lib.orc_hqq_dequantize(p(W_q), p(s), p(z), i64(N), i64(K), i64(GROUP), p(W), threads)
            y = np.empty((1, N), dtype=np.float32)
            lib.orc_matmul_nt_f32(p(v), p(W), i64(1), i64(N), i64(K), p(y), threads)
            v = np.ascontiguousarray(y.astype(np.float16).astype(np.float32))  # fp16 hand-over like the GPU chain
        return v

    def timed(fn, budget_s, max_reps):
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            dt = time.perf_counter() - t0
            if dt > budget_s or reps >= max_reps:
                return dt / reps, reps

    x32 = np.ascontiguousarray(x_host.float().numpy())
    y_ref = step(x32)
    sec, reps = timed(lambda: step(x32), 10.0, 2000)  # about 10 s of CPU work
    err = float(np.linalg.norm(y_gpu.astype(np.float64) - y_ref) / np.linalg.norm(y_ref))

    torch.set_num_threads(threads)
    tl = [(W_q.view(W_q.shape[0], -1, GROUP), s.float().view(W_q.shape[0], -1, 1), z.float().view(W_q.shape[0], -1, 1))
          for (W_q, s, z) in host_tensors]

    def torch_step():
        v = x_host.float()
        for (q, s, z) in tl:
            W = ((q.float() - z) * s).view(q.shape[0], -1)
            v = (v @ W.t()).to(torch.float16).float()
        return v

    sec_torch, reps_torch = timed(torch_step, 6.0, 200)
    return sec, reps, err, sec_torch, reps_torch


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--rotate-gb", type=float, default=3.0, help="total bytes of distinct weight copies")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary benchmark points")
    ap.add_argument("--quick-extra", action="store_true", help="a subset of the secondary points")
    ap.add_argument("--point", default=None,
                    help="run one GEMM point alone (gemm_a8w8_fp8, gemm_a8w8_int8, gemm_a4w4_mxfp4, gemm_a4w4_mxfp4_M8192, "
                         "gemm_a16w4_gs128_fp16, gemm_a8w8_fp8_block_quant, gemm_a8w8_int8_block_quant) for a profiler, print its line and exit")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a 256 MiB device copy (a kernel of known traffic, to scale profiler byte counters)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (the hot path has no cross-GPU work); use --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    lib = _ext.load_library()
    T = Timer()
    if a.point:
        run_point(a.point, lib, device, T)
        return

    step_bytes = sum(algorithmic_bytes(N, K) for N, K in SHAPES)
    copies = max(2, int(a.rotate_gb * 1e9 // step_bytes) + 1)

    # weights: one seeded set per shape, cloned `copies` times on the device
    base, host = [], []
    for i, (N, K) in enumerate(SHAPES):
        layer, host_t = make_layer(N, K, seed=i, device=device)
        base.append(layer)
        host.append(host_t)
    sets = [base] + [[clone_layer(l) for l in base] for _ in range(copies - 1)]

    g = torch.Generator(device="cpu").manual_seed(1234)
    x_host = torch.randn((1, SHAPES[0][1]), generator=g).to(torch.float16)
    x = x_host.to(device)
    h = torch.empty((1, SHAPES[0][0]), dtype=torch.float16, device=device)
    y = torch.empty((1, SHAPES[1][0]), dtype=torch.float16, device=device)
    launches = [(Launch(lib, s[0], x, h, device), Launch(lib, s[1], h, y, device)) for s in sets]

    def run_steps(first, count):
        for i in range(first, first + count):
            up, down = launches[i % copies]
            up()
            down()

    # ---- warm-up (eager), then graphs of the timed steps
    side = T.side
    with torch.cuda.stream(side):
        run_steps(0, a.warmup)
        torch.cuda.synchronize()
        chunk = min(a.steps, 256)
        full, rem = divmod(a.steps, chunk)
        graphs = []
        for n_steps in ([chunk] if full else []) + ([rem] if rem else []):
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=side):
                run_steps(0, n_steps)
            graphs.append(gr)
        torch.cuda.synchronize()
        for gr in graphs:  # one untimed replay each
            gr.replay()
        torch.cuda.synchronize()

        # ---- timed region: exactly a.steps steps, bracketed by synchronisations; the device time between two events
        # on the launch stream is what `value` is computed from, the host clock around the same region is reported
        # beside it (at a few hundred microseconds of work it mostly measures the host's launch and wake-up latency)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record(side)
        if full:
            for _ in range(full):
                graphs[0].replay()
        if rem:
            graphs[-1].replay()
        e1.record(side)
        torch.cuda.synchronize()
        elapsed_host = time.perf_counter() - t0
        elapsed = e0.elapsed_time(e1) * 1e-3
    ms_per_step = elapsed * 1e3 / a.steps
    value = step_bytes / (elapsed / a.steps) / 1e9
    y_gpu = y.float().cpu().numpy()

    # ---- the same steps with the next launch's weights pulled into the 256 MB memory-side cache by gla_prefetch on
    # a forked branch of the graph while the current launch runs (an experiment, not the metric: reported as it is)
    prefetch_us = None
    if not a.no_extra:
        prefetch_us = prefetch_experiment(lib, sets, launches, side, min(a.steps, 64))

    # ---- launch duration of each of the two kernels of a step: HIP events on the launch stream around a
    # graph that holds only that kernel, one launch per weight copy
    up_avg = T.graph_us([l[0] for l in launches], 8)
    down_avg = T.graph_us([l[1] for l in launches], 8)

    # the other batch sizes of the decode configuration (same weights, same rotation, graph replay)
    batch_points = {}
    if not a.no_extra:
        for M in (2, 4, 8, 16):
            for which, name in ((0, "up"), (1, "down")):
                N, K = SHAPES[which]
                xm = torch.randn((M, K), generator=g).to(torch.float16).to(device)
                om = torch.empty((M, N), dtype=torch.float16, device=device)
                us = T.graph_us([Launch(lib, s[which], xm, om, device) for s in sets], 4)
                batch_points[f"gemv_mlp_{name}_M{M}"] = bw_point(us, algorithmic_bytes(N, K, M=M))

    if a.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # the roofline object describes the heavier of the two launches of a step (same bytes, more time)
    kbytes = [algorithmic_bytes(*s) for s in SHAPES]
    heavy = 1 if down_avg >= up_avg else 0
    heavy_us = max(up_avg, down_avg)
    achieved = kbytes[heavy] / (heavy_us * 1e-6) / 1e9
    names = ["4096->14336 (up projection, 224 workgroups, K in one slab)",
             "14336->4096 (down projection, 64 column tiles x 4 K slabs)"]
    out = {
        "metric": "A16W4 gs128 GEMV GB/s (%HBM peak) @M=1",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp16",
        "data": "synthetic",
        "config": {
            "workload": "A16W4 HQQ gs=128 fp16 Llama-3-8B MLP decode, M=1: 4096->14336 then 14336->4096 per step",
            "bytes_per_step": step_bytes,
            "weight_copies": copies,
            "launch": "HIP graph replay of prepared gla_matmul calls",
            "timer": "HIP events on the launch stream around the replays, device synchronised before and after",
            "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "gemv_direct_kernel<4-bit, fp16, M=1> on " + names[heavy],
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "bytes_per_launch": kbytes[heavy],
            "avg_launch_us": round(heavy_us, 3),
            "traffic": None,
        },
        "extra": {
            "host_clock_GBps": round(step_bytes / (elapsed_host / a.steps) / 1e9, 1),
            "host_clock_ms_per_step": round(elapsed_host * 1e3 / a.steps, 6),
            "up_proj_avg_launch_us": round(up_avg, 3),
            "up_proj_GBps": round(kbytes[0] / (up_avg * 1e-6) / 1e9, 1),
            "down_proj_avg_launch_us": round(down_avg, 3),
            "down_proj_GBps": round(kbytes[1] / (down_avg * 1e-6) / 1e9, 1),
            **batch_points,
        },
    }

    # traffic per launch of that kernel as read from the HBM byte counters, when a profile holds it (counters are
    # collected by separate rocprofv3 --pmc runs of this script, not in this run)
    traffic_file = os.path.join(ROOT, "profiles", "gemv_direct_a16w4_traffic.json")
    if os.path.exists(traffic_file):
        with open(traffic_file) as f:
            prof = json.load(f)
        out["roofline"]["traffic"] = prof.get("hbm_bytes_per_launch_down" if heavy else "hbm_bytes_per_launch")
        out["roofline"]["traffic_source"] = (f"profiles/gemv_direct_a16w4_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, "
                                             f"taken at commit {prof.get('commit', 'unrecorded')})")
    if prefetch_us is not None:
        out["extra"]["decode_step_with_prefetch_on_forked_graph_branch"] = {
            "us_per_step": round(prefetch_us, 2), "GB/s": round(step_bytes / prefetch_us / 1e3, 1),
            "us_per_step_without": round(ms_per_step * 1e3, 2),
            "note": "gla_prefetch of launch i+1's W_q, scales and zeros on a second captured stream, forked before and joined "
                    "after launch i; the fork and join cost more than the cache-fed launch saves"}

    if not a.no_extra:
        del launches, sets, base
        torch.cuda.empty_cache()
        out["extra"].update(extra_points(lib, device, T, a.quick_extra))
        rc = out["extra"]["read_ceiling"]["31MB"]["GB/s"]
        out["roofline"]["frac_of_read_ceiling_on_this_box"] = round(achieved / rc, 4)

    if not a.no_cpu:
        cores = os.cpu_count() or 1
        threads = min(cores, 16)   # the box's CPU share for one GPU
        sec, reps, err, sec_torch, reps_torch = cpu_baseline(host, x_host, y_gpu, threads)
        out["cpu_baseline"] = {
            "value": round(step_bytes / sec / 1e9, 3),
            "unit": "GB/s",
            "cores": cores,
            "threads": threads,
            "kind": "port",
            "sample": f"{reps} whole steps (HQQ dequantize of both weight matrices + fp32 matmul, C/OpenMP restatement), "
                      f"{sec * 1e3:.1f} ms per step",
            "torch_fp32_dequant_matmul": {
                "value": round(step_bytes / sec_torch / 1e9, 3), "unit": "GB/s", "threads": threads,
                "sample": f"{reps_torch} whole steps of ((W_q - z) * s) then x @ W.T in torch fp32, {sec_torch * 1e3:.1f} ms per step"},
        }
        out["extra"]["gpu_vs_cpu_rel_frobenius_err"] = round(err, 6)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
