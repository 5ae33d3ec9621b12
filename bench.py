#!/usr/bin/env python3
"""Headline benchmark: A16W4 group-128 decode GEMV (M = 1) on the Llama-3-8B MLP shapes.

A "step" is one decode token through the two MLP linears of the benchmark configuration:
x[1,4096] -> W_up[14336,4096] -> h[1,14336] -> W_down[4096,14336] -> y[1,4096], both
A16W4 (HQQ asymmetric, group 128, 32-bit packing, fp16), launched through the C ABI
(`gla_matmul`).  Consecutive steps use different weight copies (several GB in total) so that no
cache level holds the weights between steps.  The metric is algorithmic bytes per step (every
operand read once, the output written once) divided by the time per step.

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

SHAPES = [(14336, 4096), (4096, 14336)]  # (N, K): up / down projection
GROUP = 128


def algorithmic_bytes(N, K, M=1, nbits=4, gs=GROUP):
    """W_q + scales + zeros + x + out, each touched once (fp16 metadata and activations)."""
    return N * K * nbits // 8 + 2 * (N * K // gs) * 2 + M * K * 2 + M * N * 2


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

    def __init__(self, lib, layer, x, out, device):
        m = layer.get_meta_args()
        self.lib = lib
        self.args = _ext.build_matmul_args(
            x, layer.W_q, layer.scales, layer.zeros, None, out,
            W_nbits=m[1], group_size=m[2], unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5],
            output_dtype=m[6], acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
            data_contiguous=m[11],  # matmul type left to the dispatcher (RevSplit-K up to 4 rows, Split-K GEMM above)
        )
        need = lib.gla_matmul_workspace_bytes(ctypes.byref(self.args))
        if need < 0:
            raise RuntimeError(lib.gla_last_error().decode())
        if need > 0:
            ws = _ext.get_workspace(device, need)
            self.args.workspace = ws.data_ptr()
            self.args.workspace_bytes = ws.numel()
        self.keep = (layer, x, out)

    def __call__(self):
        rc = self.lib.gla_matmul(ctypes.byref(self.args), torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError(self.lib.gla_last_error().decode())


def time_us(fn, reps, warm=25):
    """Average microseconds per call of `fn` on the current stream (events on that stream)."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps


def extra_points(lib, device):
    """The other points of the benchmark table, measured briefly (synthetic data, same C ABI):
    GEMM TFLOP/s at M=4096 for each operand format, activation quantisers, the 4096^2 decode GEMV."""
    from gemlite_amd import helper
    out = {}
    g = torch.Generator(device="cpu").manual_seed(7)

    def prepared(layer, x, scales_x, y):
        m = layer.get_meta_args()
        args = _ext.build_matmul_args(
            x, layer.W_q, layer.scales, layer.zeros, scales_x, y,
            W_nbits=m[1], group_size=m[2], unpack_mask=m[3], elements_per_sample=m[4], input_dtype=m[5],
            output_dtype=m[6], acc_dtype=m[7], meta_dtype=m[8], channel_scale_mode=m[9], W_group_mode=m[10],
            data_contiguous=m[11])
        need = lib.gla_matmul_workspace_bytes(ctypes.byref(args))
        if need > 0:
            ws = _ext.get_workspace(device, need)
            args.workspace, args.workspace_bytes = ws.data_ptr(), ws.numel()

        def run():
            if lib.gla_matmul(ctypes.byref(args), torch.cuda.current_stream().cuda_stream) != 0:
                raise RuntimeError(lib.gla_last_error().decode())
        return run

    # Sustained matrix rate of this board: a register-only MFMA loop (no memory traffic) with zero and
    # with random operand bits.  With random bits the power limit lowers the clock; that rate, not the
    # datasheet one, is what a GEMM on real data can at most reach here.
    sink = torch.zeros(1, dtype=torch.float32, device=device)
    probe = {}
    for name, dt in (("fp16", 1), ("bf16", 2), ("fp8", 3), ("int8", 4), ("mxfp4", 17)):
        rates = {}
        for label, rnd in (("zero_operands", 0), ("random_operands", 1)):
            flops = ctypes.c_double(0.0)

            def run():
                if lib.gla_probe_mfma(dt, rnd, 60000, sink.data_ptr(), ctypes.byref(flops),
                                      torch.cuda.current_stream().cuda_stream) != 0:
                    raise RuntimeError(lib.gla_last_error().decode())
            us = time_us(run, 3, warm=1)
            rates[label + "_TFLOP/s"] = round(flops.value / us / 1e6, 1)
        probe[name] = rates
    out["mfma_probe"] = probe

    def point(name, M, N, K, us, peak_tf, kind, us_zero=None):
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

    def zeroed(run, *tensors):
        """Time `run` again with the given operand tensors zero-filled (they are scratch copies)."""
        for t in tensors:
            t.view(torch.uint8).zero_()
        return time_us(run, 30)

    # A16W4 gs128 fp16, M = 4096 (fused-dequant MFMA GEMM)
    M, N, K = 4096, 4096, 4096
    layer, _ = make_layer(N, K, seed=11, device=device)
    x = torch.randn((M, K), generator=g).to(torch.float16).to(device)
    y = torch.empty((M, N), dtype=torch.float16, device=device)
    run = prepared(layer, x, None, y)
    us = time_us(run, 50)
    point("gemm_a16w4_gs128_fp16", M, N, K, us, 2500.0, "fp16", zeroed(run, x, layer.W_q.data))
    del layer, x, y

    # A8W8 fp8 / int8 dynamic, M = 4096, N = K = 8192: activation quantiser + GEMM
    M, N, K = 4096, 8192, 8192
    W = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16).to(device)
    x = torch.randn((M, K), generator=g).to(torch.bfloat16).to(device)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=device)
    for name, proc, wdt in (("fp8", helper.A8W8_FP8_dynamic, torch.float8_e4m3fn), ("int8", helper.A8W8_INT8_dynamic, torch.int8)):
        layer = proc(device=device).from_weights(W)
        xq, sx = gemlite_amd.scale_activations_per_token(x, wdt)
        run = prepared(layer, xq, sx, y)
        us = time_us(run, 50)
        point(f"gemm_a8w8_{name}", M, N, K, us, 5000.0, name, zeroed(run, xq, layer.W_q.data))
        us = time_us(lambda: gemlite_amd.scale_activations_per_token(x, wdt), 20)
        out[f"actquant_per_token_{name}"] = {"M": M, "K": K, "us": round(us, 1),
                                            "GB/s": round((M * K * 3 + M * 4) / us / 1e3, 1)}
        del layer, xq, sx
    del W, x, y

    # A8W8 MXFP8 weights, fp8 activations quantised per token (the reference processor's default), M = 4096, N = K = 8192
    M, N, K = 4096, 8192, 8192
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.bfloat16)
    lin.weight.data = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    layer = helper.A8W8_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_linear(lin.to(device))
    del lin
    x = torch.randn((M, K), generator=g).to(torch.bfloat16).to(device)
    xq, sx = gemlite_amd.scale_activations_per_token(x, torch.float8_e4m3fn)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=device)
    run = prepared(layer, xq, sx, y)
    us = time_us(run, 50)
    point("gemm_a8w8_mxfp8", M, N, K, us, 5000.0, "fp8", zeroed(run, xq, layer.W_q.data))
    del layer, x, xq, sx, y

    # A16W8 weight-only int8 bytes (unpacked), bf16, N = K = 8192: M = 4096 (MFMA GEMM) and M = 1 (streaming)
    M, N, K = 4096, 8192, 8192
    W = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16).to(device)
    layer = helper.A16W8_INT8(device=device, post_scale=True).from_weights(W)
    del W
    x = torch.randn((M, K), generator=g).to(torch.bfloat16).to(device)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=device)
    run = prepared(layer, x, None, y)
    us = time_us(run, 30)
    point("gemm_a16w8_int8_bytes_bf16", M, N, K, us, 2500.0, "bf16")
    x1 = x[:1].contiguous()
    y1 = torch.empty((1, N), dtype=torch.bfloat16, device=device)
    us = time_us(prepared(layer, x1, None, y1), 50)
    out["gemv_a16w8_int8_bytes_M1"] = {"N": N, "K": K, "us": round(us, 1), "GB/s": round((N * K + N * 4 + K * 2 + N * 2) / us / 1e3, 1),
                                       "note": "64 MB of weights, same buffer every call: served partly by the 256 MB Infinity Cache"}
    del layer, x, y, x1, y1

    # A4W4 MXFP4 dynamic, M = 4096, N = K = 16384
    M, N, K = 4096, 16384, 16384
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.bfloat16)
    lin.weight.data = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    layer = helper.A4W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_linear(lin.to(device))
    del lin
    x = torch.randn((M, K), generator=g).to(torch.bfloat16).to(device)
    xq, sx = gemlite_amd.scale_activations_mxfp4(x)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=device)
    run = prepared(layer, xq, sx, y)
    us = time_us(run, 30)
    w_saved = layer.W_q.data.clone()
    point("gemm_a4w4_mxfp4", M, N, K, us, 10100.0, "mxfp4", zeroed(run, xq, layer.W_q.data))
    layer.W_q.data.copy_(w_saved)
    del w_saved
    us = time_us(lambda: gemlite_amd.scale_activations_mxfp4(x), 20)
    out["actquant_mxfp4"] = {"M": M, "K": K, "us": round(us, 1),
                             "GB/s": round((M * K * 2 + M * K // 2 + M * K // 32) / us / 1e3, 1)}
    # the same layer at M = 1: weight-streaming, HBM-bound
    x1 = torch.randn((1, K), generator=g).to(torch.bfloat16).to(device)
    xq1, sx1 = gemlite_amd.scale_activations_mxfp4(x1)
    y1 = torch.empty((1, N), dtype=torch.bfloat16, device=device)
    us = time_us(prepared(layer, xq1, sx1, y1), 50)
    out["gemv_a4w4_mxfp4_M1"] = {"N": N, "K": K, "us": round(us, 1),
                                 "GB/s": round((N * K // 2 + N * K // 32 + K // 2 + N * 2) / us / 1e3, 1)}
    w_codes, w_scales = layer.W_q.data, layer.scales.data
    del layer, x, xq, sx, y, xq1, sx1, y1

    # Weight-only MXFP4 (bf16 activations as they are) on the same codes: the streaming MX kernel, M = 1, 2, 4
    wo = helper.A16W4_MXFP(device=device, dtype=torch.bfloat16).from_packed_weights(
        w_codes.t(), w_scales.view(torch.float8_e8m0fnu))
    for M in (1, 2, 4):
        xm = torch.randn((M, K), generator=g).to(torch.bfloat16).to(device)
        ym = torch.empty((M, N), dtype=torch.bfloat16, device=device)
        us = time_us(prepared(wo, xm, None, ym), 50)
        out[f"gemv_a16w4_mxfp_M{M}"] = {"N": N, "K": K, "us": round(us, 1),
                                        "GB/s": round((N * K // 2 + N * K // 32 + M * K * 2 + M * N * 2) / us / 1e3, 1)}
    out["gemv_a16w4_mxfp_M1"]["note"] = "134 MB of weights, same buffer every call: served partly by the 256 MB Infinity Cache"
    # ... and at M = 4096 on the matrix cores (weights converted to bf16 fragments in registers)
    xm = torch.randn((4096, K), generator=g).to(torch.bfloat16).to(device)
    ym = torch.empty((4096, N), dtype=torch.bfloat16, device=device)
    us = time_us(prepared(wo, xm, None, ym), 20)
    point("gemm_a16w4_mxfp_bf16", 4096, N, K, us, 2500.0, "bf16")
    # ... and under fp8 activations quantised per token (A8W4_MXFP_dynamic): the mixed fp8 x fp4 scaled MFMA
    a84 = helper.A8W4_MXFP_dynamic(device=device, dtype=torch.bfloat16).from_packed_weights(
        w_codes.t(), scales=w_scales.view(torch.float8_e8m0fnu))
    xq, sx = gemlite_amd.scale_activations_per_token(xm, torch.float8_e4m3fn)
    us = time_us(prepared(a84, xq, sx, ym), 20)
    point("gemm_a8w4_mxfp", 4096, N, K, us, 5000.0, "fp8")
    del wo, a84, xq, sx, w_codes, w_scales, xm, ym

    # 128 x 128 block-quantised fp8 / int8 (channel_scale_mode 5), N = K = 8192: per-block activation quantiser,
    # the MFMA GEMM at M = 4096 and the streaming kernel at M = 1
    M, N, K = 4096, 8192, 8192
    W = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16).to(device)
    x = torch.randn((M, K), generator=g).to(torch.bfloat16).to(device)
    y = torch.empty((M, N), dtype=torch.bfloat16, device=device)
    y1 = torch.empty((1, N), dtype=torch.bfloat16, device=device)
    for name, proc, wdt in (("fp8", helper.A8W8_FP8_dynamic, torch.float8_e4m3fn), ("int8", helper.A8W8_INT8_dynamic, torch.int8)):
        layer = proc(device=device, block_quant=True).from_weights(W)
        xq, sx = gemlite_amd.scale_activations_per_block(x, wdt)
        us = time_us(prepared(layer, xq, sx, y), 30)
        point(f"gemm_a8w8_{name}_block_quant", M, N, K, us, 5000.0, name)
        us = time_us(lambda: gemlite_amd.scale_activations_per_block(x, wdt), 20)
        out[f"actquant_per_block_{name}"] = {"M": M, "K": K, "us": round(us, 1),
                                            "GB/s": round((M * K * 3 + M * K // 128 * 4) / us / 1e3, 1)}
        xq1, sx1 = gemlite_amd.scale_activations_per_block(x[:1].contiguous(), wdt)
        us = time_us(prepared(layer, xq1, sx1, y1), 50)
        out[f"gemv_a8w8_{name}_block_quant_M1"] = {
            "N": N, "K": K, "us": round(us, 1), "GB/s": round((N * K + N * K // 16384 * 4 + K + N * 2) / us / 1e3, 1),
            "note": "64 MB of weights, same buffer every call: served partly by the 256 MB Infinity Cache"}
        del layer, xq, sx, xq1, sx1
    return out


def cpu_baseline(host_tensors, x_host, y_gpu, threads):
    """The reference's CPU path (HQQ dequantize + fp32 matmul) as restated in oracle/oracle_c.c,
    timed on this box's host cores on whole steps of the same workload; also the parity check."""
    import numpy as np

    lib = ctypes.CDLL(os.path.join(ROOT, "oracle", "liboracle_c.so"))
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
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

    x32 = np.ascontiguousarray(x_host.float().numpy())
    y_ref = step(x32)  # warm-up + reference output
    reps, t0 = 0, time.perf_counter()
    while True:
        step(x32)
        reps += 1
        dt = time.perf_counter() - t0
        if dt > 10.0 or reps >= 20:
            break
    sec = dt / reps
    err = float(np.linalg.norm(y_gpu.astype(np.float64) - y_ref) / np.linalg.norm(y_ref))
    return sec, reps, err


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--rotate-gb", type=float, default=3.0, help="total bytes of distinct weight copies")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary benchmark points")
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
    run_steps(0, a.warmup)
    torch.cuda.synchronize()

    chunk = min(a.steps, 256)
    full, rem = divmod(a.steps, chunk)
    side = torch.cuda.Stream()
    graphs = []
    with torch.cuda.stream(side):
        run_steps(0, 2)
        torch.cuda.synchronize()
        for n_steps in ([chunk] if full else []) + ([rem] if rem else []):
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=side):
                run_steps(0, n_steps)
            graphs.append(gr)
    torch.cuda.synchronize()
    for gr in graphs:  # one untimed replay each
        gr.replay()
    torch.cuda.synchronize()

    # ---- timed region: exactly a.steps steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if full:
        for _ in range(full):
            graphs[0].replay()
    if rem:
        graphs[-1].replay()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / a.steps
    value = step_bytes / (elapsed / a.steps) / 1e9

    # ---- launch duration of the dominant kernel (the 4096 -> 14336 GEMV): HIP events on the
    # launch stream around a timed region that holds only that kernel, one launch per weight copy
    def kernel_avg_us(which, reps=8):
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(gr, stream=side):
                for i in range(copies):
                    launches[i][which]()
            gr.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(side)
            for _ in range(reps):
                gr.replay()
            e1.record(side)
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (reps * copies)

    up_avg = kernel_avg_us(0)
    down_avg = kernel_avg_us(1)

    # the other batch sizes of the decode configuration (same weights, same rotation, graph replay)
    def batch_avg_us(M, which, reps=4):
        N, K = SHAPES[which]
        xm = torch.randn((M, K), generator=g).to(torch.float16).to(device)
        om = torch.empty((M, N), dtype=torch.float16, device=device)
        ls = [Launch(lib, s[which], xm, om, device) for s in sets]
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            for l in ls[:2]:
                l()
            torch.cuda.synchronize()
            with torch.cuda.graph(gr, stream=side):
                for l in ls:
                    l()
            gr.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(side)
            for _ in range(reps):
                gr.replay()
            e1.record(side)
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (reps * copies)

    batch_points = {}
    if not a.no_extra:
        for M in (2, 4, 8, 16):
            for which, name in ((0, "up"), (1, "down")):
                us = batch_avg_us(M, which)
                batch_points[f"gemv_mlp_{name}_M{M}"] = {
                    "us": round(us, 2), "GB/s": round(algorithmic_bytes(*SHAPES[which], M=M) / us / 1e3, 1)}
    kbytes = algorithmic_bytes(*SHAPES[0])
    achieved = kbytes / (up_avg * 1e-6) / 1e9

    y_gpu = y.float().cpu().numpy()

    if a.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

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
            "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "gemv_direct_kernel<4-bit, fp16, M=1> on 4096->14336",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "bytes_per_launch": kbytes,
            "avg_launch_us": round(up_avg, 3),
            "traffic": None,
        },
        "extra": {
            "down_proj_avg_launch_us": round(down_avg, 3),
            "down_proj_GBps": round(algorithmic_bytes(*SHAPES[1]) / (down_avg * 1e-6) / 1e9, 1),
            **batch_points,
        },
    }

    # traffic per launch of the dominant kernel as read from the HBM byte counters, when a profile holds it
    traffic_file = os.path.join(ROOT, "profiles", "gemv_direct_a16w4_traffic.json")
    if os.path.exists(traffic_file):
        with open(traffic_file) as f:
            out["roofline"]["traffic"] = json.load(f).get("hbm_bytes_per_launch")

    if not a.no_extra:
        del launches, sets, base
        torch.cuda.empty_cache()
        out["extra"].update(extra_points(lib, device))

    if not a.no_cpu:
        threads = min(os.cpu_count() or 1, 16)
        sec, reps, err = cpu_baseline(host, x_host, y_gpu, threads)
        out["cpu_baseline"] = {
            "value": round(step_bytes / sec / 1e9, 3),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": f"{reps} whole steps (HQQ dequantize of both weight matrices + fp32 matmul), "
                      f"{sec * 1e3:.1f} ms per step",
        }
        out["extra"]["gpu_vs_cpu_rel_frobenius_err"] = round(err, 6)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
