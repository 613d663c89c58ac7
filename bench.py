#!/usr/bin/env python3
"""Benchmark of the FP8 hot path on one MI355X.

One step = one pass of the Llama-style MLP hot path over one batch (benchmark config 2):
    X bf16 [8192,4096] --per-token amax/scale/E4M3 quantize--> Xq
    H = SiLU(Xq.Wg^T) * (Xq.Wu^T)      fused gate/up FP8 GEMM, N=14336, bf16 out
    H --per-token quantize--> Hq
    Y = Hq.Wd^T                        down-proj FP8 GEMM, K=14336, N=4096, bf16 out
Weights are quantized once before the timed region (they change per optimizer step, not per batch).
All inputs are resident in HBM when the timed region starts.

Prints ONE JSON line.  `value` is the step's GEMM work (2*M*N*K for gate, up and down) divided by the
whole step time, quantize passes included.  `roofline` describes the dominant kernel (the fused
gate/up GEMM) from HIP events recorded around that launch inside the timed region; `cpu_baseline`
is the reference's CPU linear-forward idiom on config 1, timed on this host.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

FP8_PEAK_TFLOPS = 5000.0      # MI355X dense FP8 MFMA peak (published)
HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E peak (published)
# HBM bytes per launch of the fused gate/up GEMM from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# script, scaled by what the same counters read for a 1 GiB device copy (fetch x2.000, write x1.000):
# 1,384,194 KiB read + 229,423 KiB written.  Not measurable from inside the process; re-measure when the kernel changes.
GATEUP_HBM_TRAFFIC_BYTES = (1384194 + 229423) * 1024


def cpu_baseline(sample_rows=3072):
    """A bounded sample of config 2's gate projection on the host cores: the first `sample_rows` token rows
    against the full gate weight [14336,4096].  Per-token / per-channel amax -> E4M3 quantize (oracle
    rounding), dequantize, then Y = dequant(X).dequant(W)^T as one scalar fp32 dot per output with the rows
    split over threads (the loop idiom of src/cpu_trainer.cpp:306-324), bf16 output."""
    import numpy as np
    sys.path.insert(0, str(ROOT / "tests"))
    import oracle_lib as orc      # checker code, used here only as the reported CPU baseline

    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    cores = max(1, min(cores, 16))
    rng = np.random.default_rng(1)
    T, K, N = sample_rows, 4096, 14336
    x = rng.standard_normal((T, K), dtype=np.float32)
    u = rng.random((T, K), dtype=np.float32)
    x[u < 0.0005] = 40.0
    x[u > 0.9995] = -40.0
    del u
    w = rng.standard_normal((N, K), dtype=np.float32)
    w *= np.float32(0.02)
    xb, wb = orc.bf16_from_f32(x), orc.bf16_from_f32(w)
    del x, w
    t0 = time.perf_counter()
    xq, _, xd = orc.quantize_rows(xb)
    wq, _, wd = orc.quantize_rows(wb)
    xf = orc.e4m3_unpack(xq) * xd[:, None]
    wf = orc.e4m3_unpack(wq) * wd[:, None]
    t1 = time.perf_counter()
    orc.linear_forward_f32(xf, wf, threads=cores)
    t2 = time.perf_counter()
    flop = 2.0 * T * K * N
    return {
        "value": round(flop / (t2 - t0) / 1e12, 6), "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"config 2 gate projection, first {T} of 8192 token rows x full W[14336x4096]: per-row amax + E4M3 "
                  f"quantize + dequantize ({t1 - t0:.1f} s) and scalar fp32 linear forward on {cores} threads "
                  f"({t2 - t1:.1f} s), one pass",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy, so a rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this "
                         "command carries a kernel of known traffic to scale the counters by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus must be 1 (no multi-GPU path is built)")

    import torch
    import __graft_entry__ as entry

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    cf = entry.load_package().lib()      # raises if libcf_fp8.so is missing: there is no fallback
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    st = torch.cuda.current_stream().cuda_stream

    M, K, N = 8192, 4096, 14336
    g = torch.Generator(device=dev).manual_seed(2)
    x = torch.randn((M, K), generator=g, device=dev)
    u = torch.rand((M, K), generator=g, device=dev)
    x = torch.where(u < 0.0005, torch.full_like(x, 40.0), x)
    x = torch.where(u > 0.9995, torch.full_like(x, -40.0), x).to(torch.bfloat16)
    del u
    wg = (torch.randn((N, K), generator=g, device=dev) * 0.02).to(torch.bfloat16)
    wu = (torch.randn((N, K), generator=g, device=dev) * 0.02).to(torch.bfloat16)
    wd = (torch.randn((K, N), generator=g, device=dev) * 0.02).to(torch.bfloat16)

    def qrows(t):
        r, c = t.shape
        q = torch.empty((r, c), dtype=torch.uint8, device=dev)
        s = torch.empty(r, device=dev)
        d = torch.empty(r, device=dev)
        cf.cf_fp8_quantize_rows(t, r, c, 0, q, s, d, st)
        return q, s, d

    wgq, _, wgd = qrows(wg)
    wuq, _, wud = qrows(wu)
    wdq, _, wdd = qrows(wd)
    del wg, wu, wd

    xq = torch.empty((M, K), dtype=torch.uint8, device=dev)
    xs = torch.empty(M, device=dev); xd = torch.empty(M, device=dev)
    h = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    hq = torch.empty((M, N), dtype=torch.uint8, device=dev)
    hs = torch.empty(M, device=dev); hd = torch.empty(M, device=dev)
    y = torch.empty((M, K), dtype=torch.bfloat16, device=dev)

    ev = lambda: torch.cuda.Event(enable_timing=True)
    marks = []        # timed steps: one bracket, around the dominant kernel
    detail = []       # breakdown steps (after the timed region): a bracket around every kernel

    def step(mode):
        """mode 0: no events; 1: events around the gate/up GEMM only; 2: events around every kernel."""
        e = [ev() for _ in range(5)] if mode else None
        if mode == 2: e[0].record()
        cf.cf_fp8_quantize_rows(x, M, K, 0, xq, xs, xd, st)
        if mode: e[1].record()
        cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wgq, K, wgd, 1, 2, None, wuq, wud, h, N, 0, st)
        if mode: e[2].record()
        cf.cf_fp8_quantize_rows(h, M, N, 0, hq, hs, hd, st)
        if mode == 2: e[3].record()
        cf.cf_fp8_gemm_nt_bf16_ex(M, K, N, hq, N, 0, hd, wdq, N, wdd, 1, 0, None, None, None, y, K, 0, st)
        if mode == 2:
            e[4].record()
            detail.append(e)
        elif mode == 1:
            marks.append(e)

    if args.traffic_calibration:
        src = torch.full((1 << 30,), 7, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)          # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step(0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(1)
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    ms_per_step = (t1 - t0) * 1e3 / args.steps
    # per-kernel breakdown: the same steps again with a bracket around every kernel, outside the timed region
    # (each bracket costs a launch gap, which the timed steps should not pay four times over)
    for _ in range(min(args.steps, 20)):
        step(2)
    torch.cuda.synchronize()

    def back_to_back(fn, launches=20, batches=3):
        """ms per launch of `fn` launched back to back (no other kernel, no event between the launches)."""
        ts = []
        for _ in range(batches):
            a, b = ev(), ev()
            a.record()
            for _ in range(launches):
                fn()
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b) / launches)
        return sorted(ts)[len(ts) // 2]

    # outside the timed steps: the two quantize kernels on their own (the brackets inside a step include a launch gap
    # that is a quarter of a 20 us kernel)
    qx_alone_ms = back_to_back(lambda: cf.cf_fp8_quantize_rows(x, M, K, 0, xq, xs, xd, st))
    qh_alone_ms = back_to_back(lambda: cf.cf_fp8_quantize_rows(h, M, N, 0, hq, hs, hd, st))
    seg = [sum(e[i].elapsed_time(e[i + 1]) for e in detail) / len(detail) for i in range(4)]   # ms
    seg[1] = sum(e[1].elapsed_time(e[2]) for e in marks) / len(marks)       # the dominant kernel: from the timed steps
    flop_gateup = 2.0 * 2.0 * M * N * K
    flop_down = 2.0 * M * K * N
    total_flop = flop_gateup + flop_down
    value = total_flop / (ms_per_step * 1e-3) / 1e12
    gateup_tflops = flop_gateup / (seg[1] * 1e-3) / 1e12
    down_tflops = flop_down / (seg[3] * 1e-3) / 1e12
    qx_bytes = 3.0 * M * K + 8.0 * M          # 2 B read + 1 B written per element, scale + descale per row
    qh_bytes = 3.0 * M * N + 8.0 * M
    qx_gbps = qx_bytes / (seg[0] * 1e-3) / 1e9
    qh_gbps = qh_bytes / (seg[2] * 1e-3) / 1e9

    props = torch.cuda.get_device_properties(dev)
    out = {
        "metric": "fp8_gemm_tflops_mlp_m8192_n14336_k4096_with_quantize",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3",
        "data": "synthetic",
        "config": {
            "workload": "config 2: Llama MLP, M=8192 K=4096 N=14336; per-token quantize -> fused gate/up E4M3 GEMM "
                        "with SiLU epilogue -> per-token quantize -> down-proj GEMM; per-token x per-channel scales",
            "device": props.name, "compute_units": props.multi_processor_count,
        },
        "gemm_gateup_tflops": round(gateup_tflops, 1),
        "gemm_gateup_pct_fp8_peak": round(100.0 * gateup_tflops / FP8_PEAK_TFLOPS, 2),
        "gemm_down_tflops": round(down_tflops, 1),
        "gemm_down_pct_fp8_peak": round(100.0 * down_tflops / FP8_PEAK_TFLOPS, 2),
        "quantize_x_gbps": round(qx_gbps, 1),
        "quantize_x_pct_hbm_peak": round(100.0 * qx_gbps / HBM_PEAK_GBPS, 2),
        "quantize_h_gbps": round(qh_gbps, 1),
        "quantize_h_pct_hbm_peak": round(100.0 * qh_gbps / HBM_PEAK_GBPS, 2),
        "kernel_ms": {"quantize_x": round(seg[0], 4), "gemm_gateup_silu": round(seg[1], 4),
                      "quantize_h": round(seg[2], 4), "gemm_down": round(seg[3], 4)},
        "quantize_back_to_back": {
            "note": "the same two kernels launched 20 times back to back outside the timed steps (no launch gap in the "
                    "bracket; part of the input stays in the 256 MB memory-side cache between launches)",
            "quantize_x_ms": round(qx_alone_ms, 4), "quantize_x_gbps": round(qx_bytes / (qx_alone_ms * 1e-3) / 1e9, 1),
            "quantize_x_pct_hbm_peak": round(100.0 * qx_bytes / (qx_alone_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
            "quantize_h_ms": round(qh_alone_ms, 4), "quantize_h_gbps": round(qh_bytes / (qh_alone_ms * 1e-3) / 1e9, 1),
            "quantize_h_pct_hbm_peak": round(100.0 * qh_bytes / (qh_alone_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
        },
        "roofline": {
            "kernel": "k_gemm_nt_ring<e4m3,silu_gate,row_col> M=8192 N=2x14336 K=4096",
            "bound": "mfma", "achieved": round(gateup_tflops, 1), "peak": FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(gateup_tflops / FP8_PEAK_TFLOPS, 4), "traffic": GATEUP_HBM_TRAFFIC_BYTES,
        },
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
