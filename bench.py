#!/usr/bin/env python3
"""Benchmark of the W4A32 quantized-Linear hot path on one MI355X.

A "step" is one decode token's worth of W4A32 Linears at M=1 on Qwen2-1.5B shapes: 28 layers
x {q, k, v, o, gate, up, down} + lm_head, every layer with its own weights (868 MB of
nibbles+scales per step, more than the 256 MB Infinity Cache, so weights come from HBM as
they do in real decoding). Each Linear is the whole op (per-row int8 quantisation of the
activations + the product), exactly what the operator boundary runs per call.

Prints ONE JSON line. `value` = algorithmic bytes of the step / time per step (GB/s), inputs
resident in HBM. `roofline` = the decode product kernel alone over the same launches (HIP
events on the launch stream), against 8 TB/s. `extra` carries the M=512 prefill TFLOP/s per
shape and the per-shape decode figures. `cpu_baseline` = the scalar CPU restatement of the
reference path on this host, on a bounded sample.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
LAYERS = 28
# name, K, N, bias, count per layer
LAYER_LINEARS = [
    ("q_proj", 1536, 1536, True),
    ("k_proj", 1536, 256, True),
    ("v_proj", 1536, 256, True),
    ("o_proj", 1536, 1536, False),
    ("gate_proj", 1536, 8960, False),
    ("up_proj", 1536, 8960, False),
    ("down_proj", 8960, 1536, False),
]
LM_HEAD = ("lm_head", 1536, 151936, False)


def algorithmic_bytes(M, K, N, bias):
    """nibbles + bf16 block scales (+ bias) + activations in + outputs out."""
    return N * K // 2 + N * (K // 32) * 2 + (N * 4 if bias else 0) + M * K * 4 + M * N * 4


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-gemm", action="store_true", help="skip the prefill (M=512) leg")
    ap.add_argument("--eager", action="store_true", help="launch from Python instead of a HIP graph")
    ap.add_argument("--roofline-only", action="store_true",
                    help="only the product-kernel passes (the run profiled under rocprofv3)")
    return ap.parse_args()


class Linear:
    def __init__(self, pkg, torch, name, K, N, bias, gen):
        w = torch.randn((N, K), generator=gen, device="cuda", dtype=torch.float32) * 0.02
        b = (torch.randn((N,), generator=gen, device="cuda", dtype=torch.float32) * 0.02) if bias else None
        self.name, self.K, self.N, self.has_bias = name, K, N, bias
        self.packed = pkg.quant_pack_rhs(w, b)
        self.bytes = {m: algorithmic_bytes(m, K, N, bias) for m in (1, 512)}
        torch.cuda.synchronize()
        del w


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (--gpus 1); nothing here shards across "
              "devices, so no multi-GPU figure is produced.", file=sys.stderr)
        sys.exit(2)

    import torch

    pkg = importlib.import_module("mllm-advanced_amd")
    L = pkg.lib()                       # raises if the HIP library is missing: no fallback
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    torch.cuda.set_device(0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)

    # ---- synthetic model: random-init weights of the named shapes, quantised by the library
    layers = [[Linear(pkg, torch, n, K, N, b, gen) for (n, K, N, b) in LAYER_LINEARS]
              for _ in range(LAYERS)]
    lm_head = Linear(pkg, torch, *LM_HEAD, gen)
    step_linears = [lin for layer in layers for lin in layer] + [lm_head]
    step_bytes = sum(l.bytes[1] for l in step_linears)

    xgen = torch.Generator(device="cuda")
    xgen.manual_seed(1)
    x_by_k = {K: torch.randn((1, K), generator=xgen, device="cuda") for K in (1536, 8960)}
    ws_by_k = {K: torch.empty(pkg.workspace_bytes(1, K), dtype=torch.uint8, device="cuda")
               for K in (1536, 8960)}
    y_by_n = {N: torch.empty((1, N), device="cuda") for N in (256, 1536, 8960, 151936)}
    stream = torch.cuda.Stream()
    sptr = stream.cuda_stream

    def whole_op_pass():
        for l in step_linears:
            rc = L.w4a32_matmul(y_by_n[l.N].data_ptr(), x_by_k[l.K].data_ptr(), l.packed.data_ptr(),
                                ws_by_k[l.K].data_ptr(), 1, l.K, l.N, sptr)
            if rc:
                raise pkg.W4A32Error(f"w4a32_matmul({l.name}) -> {rc}")

    def product_only_pass():
        for l in step_linears:
            rc = L.w4a32_matmul_quantized(y_by_n[l.N].data_ptr(), ws_by_k[l.K].data_ptr(),
                                          l.packed.data_ptr(), 1, l.K, l.N, sptr)
            if rc:
                raise pkg.W4A32Error(f"w4a32_matmul_quantized({l.name}) -> {rc}")

    def timed(fn, steps, warmup, use_graph):
        """warmup, then exactly `steps` passes between two events on the launch stream."""
        with torch.cuda.stream(stream):
            for _ in range(max(warmup, 1)):
                fn()
            stream.synchronize()
            run = fn
            if use_graph:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=stream):
                    fn()
                run = graph.replay
                run()
                stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            e0.record(stream)
            for _ in range(steps):
                run()
            e1.record(stream)
            torch.cuda.synchronize()
            wall = time.perf_counter() - t0
        return e0.elapsed_time(e1) / steps, wall * 1e3 / steps

    use_graph = not args.eager
    # quantise the activations once so the product-only pass has valid inputs
    with torch.cuda.stream(stream):
        whole_op_pass()
    stream.synchronize()

    ms_prod, _ = timed(product_only_pass, args.steps, args.warmup, use_graph)
    n_launch = len(step_linears)
    roof_avg_us = ms_prod * 1e3 / n_launch
    roof_bytes = step_bytes / n_launch
    achieved = roof_bytes / (roof_avg_us * 1e-6) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                "kernel": "gemv_dot4_kernel<1>", "launches_per_step": n_launch,
                "avg_launch_us": round(roof_avg_us, 3), "algorithmic_bytes_per_launch": int(roof_bytes)}
    if args.roofline_only:
        print(json.dumps({"roofline": roofline}))
        return

    ms_step, wall_ms = timed(whole_op_pass, args.steps, args.warmup, use_graph)
    value = step_bytes / (ms_step * 1e-3) / 1e9

    extra = {"decode_linears_tokens_per_s": round(1e3 / ms_step, 1),
             "wall_ms_per_step": round(wall_ms, 4), "graph": use_graph,
             "product_only_ms_per_step": round(ms_prod, 4)}

    # ---- per-shape decode figures (product kernel, weights rotated over the 28 layers)
    per_shape = {}
    reps = 20
    with torch.cuda.stream(stream):
        for idx, (name, K, N, b) in enumerate(LAYER_LINEARS + [LM_HEAD]):
            lins = [lm_head] if name == "lm_head" else [layer[idx] for layer in layers]
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            for l in lins:
                L.w4a32_matmul_quantized(y_by_n[N].data_ptr(), ws_by_k[K].data_ptr(),
                                         l.packed.data_ptr(), 1, K, N, sptr)
            e0.record(stream)
            for _ in range(reps):
                for l in lins:
                    L.w4a32_matmul_quantized(y_by_n[N].data_ptr(), ws_by_k[K].data_ptr(),
                                             l.packed.data_ptr(), 1, K, N, sptr)
            e1.record(stream)
            stream.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / (reps * len(lins))
            per_shape[name] = {"us": round(us, 2),
                               "GBps": round(lins[0].bytes[1] / (us * 1e-6) / 1e9, 1),
                               "note": "cache-resident" if name == "lm_head" else "rotating 28 buffers"}
    extra["decode_per_shape"] = per_shape

    # ---- prefill leg: M=512 whole op per shape
    if not args.no_gemm:
        M = 512
        gemm = {}
        total_flop, total_ms = 0.0, 0.0
        with torch.cuda.stream(stream):
            for idx, (name, K, N, b) in enumerate(LAYER_LINEARS):
                lin = layers[0][idx]
                x = torch.randn((M, K), generator=xgen, device="cuda")
                ws = torch.empty(pkg.workspace_bytes(M, K), dtype=torch.uint8, device="cuda")
                y = torch.empty((M, N), device="cuda")

                def call():
                    rc = L.w4a32_matmul(y.data_ptr(), x.data_ptr(), lin.packed.data_ptr(),
                                        ws.data_ptr(), M, K, N, sptr)
                    if rc:
                        raise pkg.W4A32Error(f"w4a32_matmul M=512 ({name}) -> {rc}")
                for _ in range(3):
                    call()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(10):
                    call()
                e1.record(stream)
                stream.synchronize()
                ms = e0.elapsed_time(e1) / 10
                flop = 2.0 * M * N * K
                gemm[name] = {"ms": round(ms, 4), "TFLOPs": round(flop / (ms * 1e-3) / 1e12, 2)}
                total_flop += flop
                total_ms += ms
        extra["prefill_M512_per_shape"] = gemm
        extra["prefill_M512_layer_TFLOPs"] = round(total_flop / (total_ms * 1e-3) / 1e12, 2)

    # ---- CPU baseline: scalar restatement of the reference path, bounded sample
    cpu = None
    if not args.no_cpu:
        sys.path.insert(0, os.path.join(ROOT, "oracle"))
        import w4a32_oracle as orc
        sample = layers[0]
        host = []
        for l in sample:
            u4, sc, bias = pkg.unpack_native(l.packed, l.N, l.K, want_bias=True)
            torch.cuda.synchronize()
            host.append((l, u4.cpu().numpy(), sc.cpu().numpy().view("uint16"),
                         bias.cpu().numpy() if l.has_bias else None))
        xs = {K: x_by_k[K].cpu().numpy() for K in x_by_k}
        for (l, u4, sc, bias) in host:      # page in
            orc.linear(xs[l.K], u4, sc, bias=bias, threads=1)
        reps_cpu, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 10.0:
            for (l, u4, sc, bias) in host:
                orc.linear(xs[l.K], u4, sc, bias=bias, threads=1)
            reps_cpu += 1
        dt = time.perf_counter() - t0
        layer_bytes = sum(l.bytes[1] for l in sample)
        cpu = {"value": round(layer_bytes * reps_cpu / dt / 1e9, 3), "unit": "GB/s", "cores": 1,
               "kind": "port",
               "sample": f"{reps_cpu} passes over one decoder layer's 7 W4A32 Linears at M=1 "
                         f"({layer_bytes} algorithmic bytes per pass), scalar C restatement of the "
                         f"reference path; the reference runs decode (M=1) as a single task",
               "host_cpus": os.cpu_count()}

    out = {
        "metric": "W4 GEMV HBM GB/s (M=1)", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic (torch cuda generator seed 0, N(0,0.02^2) f32 weights quantised to 4-bit "
                "block-32 by the library; activations N(0,1) seed 1)",
        "config": {"workload": "config 2 at M=1: Qwen2-1.5B decode Linears, 28 layers x "
                               "{q,k,v,o,gate,up,down} + lm_head, distinct weights per layer, "
                               "whole op per Linear (row quant + product)",
                   "M": 1, "launched_linears": n_launch, "algorithmic_bytes_per_step": step_bytes},
        "roofline": roofline, "cpu_baseline": cpu, "extra": extra,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
