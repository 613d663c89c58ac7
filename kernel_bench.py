#!/usr/bin/env python3
"""Per-kernel timing of the FP8 hot path at the benchmark shapes, against each kernel's roofline.

    python kernel_bench.py [--iters 20]

Every kernel is timed with events on the launch stream (median of three batches of `--iters` launches) and
reported with its algorithmic bytes or FLOPs: HBM-bound kernels as GB/s and a fraction of 8 TB/s, GEMMs as
TFLOP/s and a fraction of the 5.0 PFLOP/s dense FP8 MFMA peak.  Inputs are synthetic and resident in HBM.
bench.py measures the headline step; this script covers the other entry points and shapes.
"""
from __future__ import annotations

import argparse
import ctypes
import importlib.util
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent
HBM_PEAK = 8000.0      # GB/s
FP8_PEAK = 5000.0      # TFLOP/s


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--only", default="", help="time only the rows whose name contains this text (for profiler runs)")
    ap.add_argument("--sustain", type=float, default=0.0,
                    help="after timing a GEMM row, hold it back to back for this many seconds and print the rate, the socket "
                         "power and the shader clock over the second half of that time (sysfs, as bench.py samples them)")
    args = ap.parse_args()
    import torch
    sys.path.insert(0, str(ROOT))
    import __graft_entry__ as entry

    cf = entry.load_package().lib()
    dev = torch.device("cuda:0")
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device=dev).manual_seed(5)

    def bf16(*shape, sigma=1.0):
        return (torch.randn(*shape, device=dev, generator=g) * sigma).to(torch.bfloat16)

    def fp8(*shape, e5m2=False):
        x = torch.randn(*shape, device=dev, generator=g)
        if e5m2:
            return (x * (57344.0 / x.abs().max())).to(torch.float8_e5m2).view(torch.uint8)
        return (x * (448.0 / x.abs().max())).to(torch.float8_e4m3fn).view(torch.uint8)

    def u8(*shape):
        return torch.empty(*shape, dtype=torch.uint8, device=dev)

    def f32(*shape):
        return torch.rand(*shape, device=dev) + 0.5

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        ts = []
        for _ in range(3):
            a = torch.cuda.Event(enable_timing=True)
            b = torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(args.iters):
                fn()
            b.record()
            torch.cuda.synchronize()
            ts.append(a.elapsed_time(b) / args.iters)
        return sorted(ts)[1] * 1e-3      # seconds

    print(f"{'kernel':<64} {'shape':<26} {'us':>9} {'rate':>14} {'of peak':>8}")

    def hbm(name, shape, nbytes, fn):
        if args.only not in name:
            fn()                         # later rows use what this one leaves behind
            return
        t = timed(fn)
        gbps = nbytes / t / 1e9
        print(f"{name:<64} {shape:<26} {t * 1e6:9.1f} {gbps:9.0f} GB/s {100 * gbps / HBM_PEAK:7.1f}%", flush=True)

    BF16_PEAK = 2500.0          # dense bf16 matrix peak, TFLOP/s

    def sustained(fn, flop):
        import time
        from bench import PowerSampler
        with PowerSampler(period_s=0.01) as ps:
            t0 = time.perf_counter()
            n = 0
            while time.perf_counter() - t0 < args.sustain:
                for _ in range(50):
                    fn()
                torch.cuda.synchronize()
                n += 50
            dt = time.perf_counter() - t0
        r = ps.report(skip_fraction=0.5)
        print(f"    held {dt:.1f} s: {dt / n * 1e6:9.1f} us per launch = {flop * n / dt / 1e12:6.0f} TFLOP/s, "
              f"{r.get('socket_power_w_avg')} W of {ps.cap_watts()} W, shader clock {r.get('sclk_mhz_avg')} MHz", flush=True)

    def mfma16(name, shape, flop, fn):
        if args.only not in name:
            return
        t = timed(fn)
        tf = flop / t / 1e12
        print(f"{name:<64} {shape:<26} {t * 1e6:9.1f} {tf:7.0f} TFLOP/s {100 * tf / BF16_PEAK:7.1f}% (of bf16 peak)", flush=True)
        if args.sustain > 0:
            sustained(fn, flop)

    def mfma(name, shape, flop, fn):
        if args.only not in name:
            fn()                         # later rows use what this one leaves behind
            return
        t = timed(fn)
        tf = flop / t / 1e12
        print(f"{name:<64} {shape:<26} {t * 1e6:9.1f} {tf:7.0f} TFLOP/s {100 * tf / FP8_PEAK:7.1f}%", flush=True)
        if args.sustain > 0:
            sustained(fn, flop)

    # ---- config 2 activations / weights: quantize family -------------------------------------------
    M, K, N = 8192, 4096, 14336
    x = bf16(M, K)
    n = x.numel()
    q = u8(M, K)
    amax = torch.zeros(1, device=dev); sc = torch.ones(1, device=dev); de = torch.ones(1, device=dev)
    hbm("amax_bf16", f"{M}x{K}", 2.0 * n, lambda: cf.cf_fp8_amax_bf16(x, n, amax, st))
    hbm("quantize_e4m3 (known scale)", f"{M}x{K}", 3.0 * n, lambda: cf.cf_fp8_quantize_e4m3(x, q, sc, n, st))
    hbm("quantize_e4m3_record (previous scale + amax)", f"{M}x{K}", 3.0 * n,
        lambda: cf.cf_fp8_quantize_e4m3_record(x, q, sc, amax, n, st))
    # delayed scaling, steady state: the reference's sequence as separate launches against the one-launch step
    hist = torch.zeros(16, device=dev); cur = torch.zeros(1, dtype=torch.int32, device=dev); cnt = torch.zeros(1, dtype=torch.int32, device=dev)
    ssnap = torch.ones(1, device=dev); dsnap = torch.ones(1, device=dev)
    running = torch.zeros(1, device=dev); arrived = torch.zeros(1, dtype=torch.int32, device=dev)

    def delayed_separate():
        ssnap.copy_(sc); dsnap.copy_(de); amax.zero_()
        cf.cf_fp8_quantize_e4m3_record(x, q, sc, amax, n, st)
        cf.cf_fp8_update_delayed_scale(amax, 448.0, sc, de, hist, 16, cur, cnt, st)
    hbm("delayed-scaling step: 2 copies + memset + record + update", f"{M}x{K}", 3.0 * n, delayed_separate)
    hbm("delayed-scaling step: cf_fp8_quantize_delayed_step (1 launch)", f"{M}x{K}", 3.0 * n,
        lambda: cf.cf_fp8_quantize_delayed_step(x, q, n, 0, amax, sc, de, ssnap, dsnap, hist, 16, cur, cnt, running, arrived, st))
    sc.fill_(1.0); de.fill_(1.0)
    hbm("quantize_e5m2 (known scale)", f"{M}x{K}", 3.0 * n, lambda: cf.cf_fp8_quantize_e5m2(x, q, sc, n, st))
    rs = torch.empty(M, device=dev); rd = torch.empty(M, device=dev)
    hbm("quantize_rows (per-token, one pass)", f"{M}x{K}", 3.0 * n + 8 * M, lambda: cf.cf_fp8_quantize_rows(x, M, K, 0, q, rs, rd, st))
    # producers fused with the quantize (FFN input: rmsnorm -> row clip -> per-token quantize)
    gamma = (1.0 + 0.1 * torch.randn(K, device=dev, generator=g)).to(torch.bfloat16)
    normed = torch.empty_like(x)
    ceiling = 65.0            # about the median row norm after normalisation: half the rows are clipped
    hbm("rmsnorm_forward", f"{M}x{K}", 4.0 * n, lambda: cf.cf_rmsnorm_forward(x, gamma, normed, None, M, K, 1e-6, st))
    hbm("act_row_clip_abs (in place, half the rows clipped)", f"{M}x{K}", 3.0 * n,
        lambda: cf.cf_act_row_clip_abs(normed, M, K, ceiling, None, st))

    def unfused():
        cf.cf_rmsnorm_forward(x, gamma, normed, None, M, K, 1e-6, st)
        cf.cf_act_row_clip_abs(normed, M, K, ceiling, None, st)
        cf.cf_fp8_quantize_rows(normed, M, K, 0, q, rs, rd, st)
    hbm("rmsnorm + clip + quantize_rows, three launches", f"{M}x{K}", 5.0 * n + 8 * M, unfused)
    hbm("rmsnorm_clip_quantize_rows (fused, keeps the bf16 row)", f"{M}x{K}", 5.0 * n + 8 * M,
        lambda: cf.cf_rmsnorm_clip_quantize_rows(x, gamma, M, K, 1e-6, ceiling, 0, normed, None, q, rs, rd, st))
    hbm("rmsnorm_clip_quantize_rows (fused, fp8 only)", f"{M}x{K}", 3.0 * n + 8 * M,
        lambda: cf.cf_rmsnorm_clip_quantize_rows(x, gamma, M, K, 1e-6, ceiling, 0, None, None, q, rs, rd, st))
    hbm("rmsnorm_clip_quantize_record (fused, per-tensor)", f"{M}x{K}", 5.0 * n,
        lambda: cf.cf_rmsnorm_clip_quantize_record(x, gamma, M, K, 1e-6, ceiling, 0, normed, None, q, sc, amax, st))
    h = bf16(M, N)
    hq = u8(M, N)
    hbm("quantize_rows (per-token, one pass)", f"{M}x{N}", 3.0 * h.numel() + 8 * M,
        lambda: cf.cf_fp8_quantize_rows(h, M, N, 0, hq, rs, rd, st))
    w = bf16(K, N, sigma=0.02)       # [in, out]
    wt = u8(N, K)
    w8 = u8(K, N)
    hbm("quantize_transpose_e4m3 (weight refresh)", f"{K}x{N}", 3.0 * w.numel(),
        lambda: cf.cf_fp8_quantize_transpose_e4m3(w, wt, sc, K, N, st))
    # refresh_fp8_weights for one weight: amax, scale, and the two layouts (one read for both)
    hbm("refresh_weight: amax + scale + fwd8 and bwd8 layouts", f"{K}x{N}", 6.0 * w.numel(),
        lambda: cf.cf_fp8_refresh_weight(w, wt, w8, amax, sc, de, K, N, 0, 1, st))
    hbm("  the reference's sequence: amax, scale, quantize, quantize-transpose", f"{K}x{N}", 6.0 * w.numel(),
        lambda: (cf.cf_fp8_amax_bf16(w, w.numel(), amax, st), cf.cf_fp8_scale_from_amax(amax, 448.0, sc, de, st),
                 cf.cf_fp8_quantize_e4m3(w, w8, sc, w.numel(), st), cf.cf_fp8_quantize_transpose_e4m3(w, wt, sc, K, N, st)))
    hq2 = u8(N, M)
    hbm("quant_and_transpose_e4m3 (dual, for wgrad)", f"{M}x{N}", 4.0 * h.numel(),
        lambda: cf.cf_fp8_quant_and_transpose_e4m3(h, hq, hq2, sc, M, N, st))
    dy8 = fp8(M, K, e5m2=True)
    dyt = u8(K, M)
    hbm("transpose_u8 (dY for wgrad)", f"{M}x{K}", 2.0 * dy8.numel(), lambda: cf.cf_transpose_u8(dy8, dyt, M, K, st))
    gate = bf16(M, N); up = bf16(M, N); out = torch.empty_like(gate)
    hbm("swiglu_forward (stand-alone)", f"{M}x{N}", 6.0 * gate.numel(),
        lambda: cf.cf_swiglu_forward(gate, up, out, gate.numel(), st))
    dout = bf16(M, N, sigma=0.01); dgate = torch.empty_like(gate); dup = torch.empty_like(gate)
    hbm("swiglu_backward (stand-alone)", f"{M}x{N}", 10.0 * gate.numel(),
        lambda: cf.cf_swiglu_backward(dout, gate, up, dgate, dup, gate.numel(), st))
    acc32 = torch.zeros(N, device=dev)
    hbm("col_sum_strided_bf16 (bias gradient, sequential rows)", f"{M}x{N}", 2.0 * gate.numel(),
        lambda: cf.cf_col_sum_strided_bf16(gate, acc32, M, N, N, 0, st))
    del gate, up, out, h, hq, hq2, w, wt, w8, dout, dgate, dup

    # ---- config 3: block-scaled ---------------------------------------------------------------------
    M3, N3, K3 = 4096, 7168, 7168
    a3 = bf16(M3, K3); a3q = u8(M3, K3)
    s3 = torch.empty(M3, K3 // 128, device=dev); d3 = torch.empty_like(s3)
    hbm("quantize_block_1x128", f"{M3}x{K3}", 3.0 * a3.numel() + 8.0 * s3.numel(),
        lambda: cf.cf_fp8_quantize_block_1x128(a3, M3, K3, a3q, s3, d3, st))
    w3 = bf16(N3, K3, sigma=0.02); w3q = u8(N3, K3)
    sw3 = torch.empty(N3 // 128, K3 // 128, device=dev); dw3 = torch.empty_like(sw3)
    hbm("quantize_block_128x128", f"{N3}x{K3}", 3.0 * w3.numel(), lambda: cf.cf_fp8_quantize_block_128x128(w3, N3, K3, w3q, sw3, dw3, st))
    c3 = torch.empty((M3, N3), dtype=torch.bfloat16, device=dev)
    mfma("gemm block-scaled 1x128 / 128x128 (config 3)", f"{M3}x{N3}x{K3}", 2.0 * M3 * N3 * K3,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(M3, N3, K3, a3q, K3, 0, d3, w3q, K3, dw3, 2, 0, None, None, None, c3, N3, 0, st))
    del a3, a3q, w3, w3q, c3

    # ---- config 2 and 4 GEMMs -----------------------------------------------------------------------
    xq = fp8(M, K); wg = fp8(N, K); wu = fp8(N, K); wd = fp8(K, N); hq = fp8(M, N)
    xd = f32(M); wgd = f32(N); wud = f32(N); wdd = f32(K)
    c = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    y = torch.empty((M, K), dtype=torch.bfloat16, device=dev)
    mfma("gemm per-tensor, bf16 out (lt_gemm_fp8_nt form)", f"{M}x{N}x{K}", 2.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_nt_bf16(M, N, K, xq, K, 0, sc, wg, de, c, N, st))
    mfma("gemm per-token x per-channel, bf16 out", f"{M}x{N}x{K}", 2.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wg, K, wgd, 1, 0, None, None, None, c, N, 0, st))
    mfma("gemm gate+up fused SiLU-gate (config 2)", f"{M}x2x{N}x{K}", 4.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wg, K, wgd, 1, 2, None, wu, wud, c, N, 0, st))
    mfma("gemm down projection (config 2)", f"{M}x{K}x{N}", 2.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(M, K, N, hq, N, 0, xd, wd, N, wdd, 1, 0, None, None, None, y, K, 0, st))
    # the same two launches on the persistent kernel's 32 x 32 x 64 MFMA form (CF_GEMM_FLAG_MFMA32 = 16; the default for
    # these epilogues is the 16 x 16 x 128 form, which does more at the same socket power)
    mfma("32x32x64 MFMA: gemm gate+up fused SiLU-gate (config 2)", f"{M}x2x{N}x{K}", 4.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wg, K, wgd, 1, 2, None, wu, wud, c, N, 16, st))
    mfma("32x32x64 MFMA: gemm down projection (config 2)", f"{M}x{K}x{N}", 2.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(M, K, N, hq, N, 0, xd, wd, N, wdd, 1, 0, None, None, None, y, K, 16, st))
    # The same launch on operands without entropy (every byte 0x38 = 1.0): the matrix cores' power follows how much
    # their inputs toggle, and on such data the part stays below its power cap at full clock.  What separates this
    # row from the one on quantized data is the power cap, not the kernel (use --sustain to see power and clock).
    if args.only in "gemm gate+up fused SiLU-gate (config 2), constant operands":
        x1 = torch.full_like(xq, 0x38); g1 = torch.full_like(wg, 0x38); u1 = torch.full_like(wu, 0x38)
        mfma("gemm gate+up fused SiLU-gate (config 2), constant operands", f"{M}x2x{N}x{K}", 4.0 * M * N * K,
             lambda: cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, x1, K, 0, xd, g1, K, wgd, 1, 2, None, u1, wud, c, N, 0, st))
        del x1, g1, u1
    # the same two launches on the 128 x 128-tile kernel that runs two workgroups per CU (CF_GEMM_FLAG_DUO = 4;
    # 12 = without starting the second workgroup of a CU half a tile late)
    mfma("duo: gemm gate+up fused SiLU-gate (config 2), 2 workgroups per CU", f"{M}x2x{N}x{K}", 4.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wg, K, wgd, 1, 2, None, wu, wud, c, N, 4, st))
    mfma("duo in step: gemm gate+up fused SiLU-gate (config 2)", f"{M}x2x{N}x{K}", 4.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(M, N, K, xq, K, 0, xd, wg, K, wgd, 1, 2, None, wu, wud, c, N, 12, st))
    mfma("duo: gemm down projection (config 2), 2 workgroups per CU", f"{M}x{K}x{N}", 2.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(M, K, N, hq, N, 0, xd, wd, N, wdd, 1, 0, None, None, None, y, K, 4, st))
    dy = fp8(M, N, e5m2=True)
    mfma("gemm dgrad, E5M2 dY (config 4)", f"{M}x{K}x{N}", 2.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_nt_bf16(M, K, N, dy, N, 1, sc, wd, de, y, K, st))
    xt = fp8(N, M); dyt = fp8(K, M, e5m2=True)
    dw = torch.zeros((N, K), dtype=torch.float32, device=dev)
    mfma("gemm wgrad, fp32 accumulate into dW (config 4)", f"{N}x{K}x{M}", 2.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_tn_accum_f32(N, K, M, xt, sc, dyt, de, dw, K, st))
    dwb = torch.zeros((N, K), dtype=torch.bfloat16, device=dev)
    mfma("gemm wgrad, bf16 accumulate into dW (config 4 shape)", f"{N}x{K}x{M}", 2.0 * M * N * K,
         lambda: cf.cf_fp8_gemm_tn_accum_bf16(N, K, M, xt, sc, dyt, de, dwb, K, st))
    del xq, wg, wu, wd, hq, c, y, dy, xt, dyt, dw, dwb

    # ---- loss head: one chunk of the fused classifier (2048 rows x 32000 logits) ----------------------------
    CR, V = 2048, 32000
    logits = bf16(CR, V, sigma=3.0)
    labels = torch.randint(0, V, (CR,), device=dev, generator=g, dtype=torch.int32)
    nvalid = torch.full((1,), CR, dtype=torch.int32, device=dev)
    cgrad = torch.empty_like(logits); cg8 = u8(CR, V); closs = torch.zeros(1, device=dev)
    hbm("cross_entropy_fwd_bwd_chunk (bf16 gradient)", f"{CR}x{V}", 4.0 * CR * V,
        lambda: cf.cf_cross_entropy_fwd_bwd_chunk(logits, labels, closs, cgrad, CR, V, nvalid, st))

    def ce_then_quant():
        cf.cf_cross_entropy_fwd_bwd_chunk(logits, labels, closs, cgrad, CR, V, nvalid, st)
        cf.cf_fp8_quantize_e5m2_record(cgrad, cg8, sc, amax, CR * V, st)
    hbm("cross entropy, then E5M2 recording quantize (2 launches)", f"{CR}x{V}", 5.0 * CR * V, ce_then_quant)
    hbm("cross_entropy_fwd_bwd_chunk_quant_e5m2 (fused)", f"{CR}x{V}", 5.0 * CR * V,
        lambda: cf.cf_cross_entropy_fwd_bwd_chunk_quant_e5m2(logits, labels, closs, cgrad, cg8, sc, amax, CR, V, nvalid, st))
    del logits, cgrad, cg8
    CR2, V2 = 512, 128256
    logits = bf16(CR2, V2, sigma=3.0)
    labels2 = torch.randint(0, V2, (CR2,), device=dev, generator=g, dtype=torch.int32)
    cgrad = torch.empty_like(logits); cg8 = u8(CR2, V2)
    hbm("cross_entropy_fwd_bwd_chunk_quant_e5m2 (fused, 1024 lanes per row)", f"{CR2}x{V2}", 5.0 * CR2 * V2,
        lambda: cf.cf_cross_entropy_fwd_bwd_chunk_quant_e5m2(logits, labels2, closs, cgrad, cg8, sc, amax, CR2, V2, nvalid, st))
    del logits, cgrad, cg8

    # ---- config 5: MoE ------------------------------------------------------------------------------
    T, H, E, k, Ie = 16384, 2048, 64, 6, 1408
    logits = torch.randn(T, E, device=dev, generator=g)
    rw = logits.clone()
    hbm("softmax + top-k route (in place)", f"{T}x{E} k={k}", 8.0 * T * E,
        lambda: (rw.copy_(logits), cf.cf_moe_topk_route_f32(rw, T, E, k, st, None, None, 1)))
    counts = torch.zeros(E, dtype=torch.int32, device=dev)
    idx = torch.zeros(E * T, dtype=torch.int32, device=dev)
    offs = torch.zeros(E, dtype=torch.int32, device=dev)
    hbm("build_expert_row_lists", f"{T}x{E}", 4.0 * T * E + 4.0 * T * k,
        lambda: cf.cf_moe_build_expert_row_lists(rw, counts, idx, T, E, st))
    cf.cf_moe_expert_offsets_from_counts(counts, offs, E, st)
    total = T * k
    hq = fp8(T, H); hd = f32(T)
    wg = fp8(E * Ie, H); wu = fp8(E * Ie, H); wd = fp8(E * H, Ie)
    wgd = f32(E * Ie); wud = f32(E * Ie); wdd = f32(E * H)
    cidx = torch.zeros(total, dtype=torch.int32, device=dev)
    cf.cf_moe_compact_row_index(counts, offs, idx, T, E, cidx, st)
    gathered = u8(total, H)
    hbm("gather_rows_u8 (token permute, stand-alone)", f"{total}x{H}", 2.0 * total * H,
        lambda: cf.cf_moe_gather_rows_u8(hq, gathered, cidx, total, H, st))
    sz = ctypes.c_size_t(0)
    cf.raw_cf_fp8_grouped_gemm_workspace_bytes(total, E, ctypes.byref(sz))
    ws = u8(sz.value)
    act = torch.empty((total, Ie), dtype=torch.bfloat16, device=dev)
    mfma("grouped gate+up SiLU-gate, fused permute (config 5)", f"{total}x2x{Ie}x{H}", 4.0 * total * Ie * H,
         lambda: cf.cf_fp8_grouped_gemm_nt_bf16_ex(total, Ie, H, E, counts, offs, hq, T, H, cidx, hd, wg, wgd, 1, 2, wu, wud,
                                                   act, Ie, ws, sz.value, st))
    actq = fp8(total, Ie); ad = f32(total)
    actq_x = fp8(total, H)
    yy = torch.empty((total, H), dtype=torch.bfloat16, device=dev)
    mfma("grouped down projection (config 5)", f"{total}x{H}x{Ie}", 2.0 * total * Ie * H,
         lambda: cf.cf_fp8_grouped_gemm_nt_bf16_ex(total, H, Ie, E, counts, offs, actq, total, Ie, None, ad, wd, wdd, 1, 0, None, None,
                                                   yy, H, ws, sz.value, st))
    # the config 5 shapes as dense GEMMs (one expert's weights for all rows): what the short K costs without the
    # grouping, on the 256 x 256-tile kernel and on the two-workgroups-per-CU kernel
    mfma("dense at the config 5 shape: gate+up SiLU-gate", f"{total}x2x{Ie}x{H}", 4.0 * total * Ie * H,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(total, Ie, H, actq_x, H, 0, ad, wg, H, wgd, 1, 2, None, wu, wud, act, Ie, 0, st))
    mfma("duo: dense at the config 5 shape: gate+up SiLU-gate", f"{total}x2x{Ie}x{H}", 4.0 * total * Ie * H,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(total, Ie, H, actq_x, H, 0, ad, wg, H, wgd, 1, 2, None, wu, wud, act, Ie, 4, st))
    mfma("dense at the config 5 shape: down projection", f"{total}x{H}x{Ie}", 2.0 * total * Ie * H,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(total, H, Ie, actq, Ie, 0, ad, wd, Ie, wdd, 1, 0, None, None, None, yy, H, 0, st))
    mfma("duo: dense at the config 5 shape: down projection", f"{total}x{H}x{Ie}", 2.0 * total * Ie * H,
         lambda: cf.cf_fp8_gemm_nt_bf16_ex(total, H, Ie, actq, Ie, 0, ad, wd, Ie, wdd, 1, 0, None, None, None, yy, H, 4, st))
    mixed = torch.zeros((T, H), dtype=torch.bfloat16, device=dev)
    hbm("unpermute_weighted_bf16", f"{total}x{H}", 2.0 * total * H + 4.0 * T * H,
        lambda: cf.cf_moe_unpermute_weighted_bf16(mixed, yy, rw, counts, offs, idx, T, E, H, st))
    slot = torch.empty((T, E), dtype=torch.int32, device=dev)
    hbm("build_slot_index", f"{T}x{E}", 8.0 * total, lambda: cf.cf_moe_build_slot_index(counts, offs, idx, T, E, slot, st))
    hbm("unpermute_indexed_bf16 (slot table instead of the search)", f"{total}x{H}", 2.0 * total * H + 4.0 * T * H,
        lambda: cf.cf_moe_unpermute_indexed_bf16(mixed, yy, rw, slot, T, E, H, 0, st))
    sz2 = ctypes.c_size_t(0)
    cf.raw_cf_moe_grouped_swiglu_workspace_bytes(total, E, H, Ie, ctypes.byref(sz2))
    ws2 = u8(sz2.value)
    mfma("grouped SwiGLU expert bank, whole pipeline (config 5)", f"T={T} E={E} k={k}", 6.0 * total * Ie * H,
         lambda: cf.cf_moe_grouped_swiglu_forward_fp8(hq, hd, rw, counts, offs, idx, wg, wgd, wu, wud, wd, wdd, mixed, T, H, Ie, E,
                                                      total, ws2, sz2.value, st))

    # the GELU expert loop (per-tensor descales): the one-call bank that re-quantizes the activations, and
    # moe_grouped_expert_forward_fp8's contract (GELU output kept beyond bf16, 16-row tiles) on the same operands
    one = torch.full((1,), 0.01, device=dev)
    sz3 = ctypes.c_size_t(0)
    cf.raw_cf_moe_grouped_gelu_workspace_bytes(T, total, E, H, Ie, ctypes.byref(sz3))
    ws3 = u8(sz3.value)
    gq = u8(total, Ie); gs = f32(total); gd = f32(total)
    hbm("gelu_quantize_rows_e4m3 (gelu_forward + per-token quantize)", f"{total}x{Ie}", 3.0 * total * Ie,
        lambda: cf.cf_gelu_quantize_rows_e4m3(act, total, Ie, gq, gs, gd, st))
    mfma("grouped GELU expert bank, whole pipeline (re-quantizing)", f"T={T} E={E} k={k}", 4.0 * total * Ie * H,
         lambda: cf.cf_moe_grouped_gelu_forward_fp8(hq, one, 0, rw, counts, offs, idx, wg, one, wd, one, mixed, T, H, Ie, E, total,
                                                    ws3, sz3.value, st))
    # the same loop with the reference's activation scale: one delayed-scaling slot per expert (state blocks of
    # cf_act_slot_state_words(8) words, scale 1 after the first call's history update)
    words = cf.raw_cf_act_slot_state_words(8)
    bank = torch.zeros((E, words), dtype=torch.float32, device=dev)
    bank[:, 1] = 64.0; bank[:, 2] = 1.0 / 64.0; bank[:, 3] = 64.0; bank[:, 4] = 1.0 / 64.0
    bank_i = bank.view(torch.int32); bank_i[:, 8:12] = 0
    rowd = f32(total)
    hbm("grouped per-expert delayed-scale quantize with GELU (1 launch, 64 slots)", f"{total}x{Ie}", 3.0 * total * Ie,
        lambda: cf.cf_moe_grouped_quantize_delayed(act, gq, Ie, E, counts, offs, total, bank, words, 8, 0, 1, 0, rowd, st))
    mfma("grouped GELU expert bank with per-expert activation slots", f"T={T} E={E} k={k}", 4.0 * total * Ie * H,
         lambda: cf.cf_moe_grouped_gelu_forward_fp8_slots(hq, one, 0, rw, counts, offs, idx, wg, one, wd, one, mixed, T, H, Ie, E, total,
                                                          bank, words, 8, 0, 0, ws3, sz3.value, st))
    sz4 = ctypes.c_size_t(0)
    cf.raw_cf_moe_grouped_expert_forward_fp8_workspace(T, total, E, H, Ie, None, ctypes.byref(sz4))
    ws4 = u8(sz4.value)
    mfma("moe_grouped_expert_forward_fp8 with a workspace (fp32 fc_in, 3-term E4M3 GELU, FP8 fc_out)", f"T={T} E={E} k={k}",
         4.0 * total * Ie * H,
         lambda: cf.cf_moe_grouped_expert_forward_fp8_ws(hq, one, 0, rw, counts, None, idx, wg, one, wd, one, mixed, T, H, Ie, E, total,
                                                         ws4, sz4.value, st))
    del ws4
    iters, args.iters = args.iters, 5
    mfma("moe_grouped_expert_forward_fp8 form (fp32 GELU kept, MFMA)", f"T={T} E={E} k={k}", 4.0 * total * Ie * H,
         lambda: cf.cf_moe_grouped_expert_forward_fp8(hq, one, 0, rw, counts, offs, idx, wg, one, wd, one, mixed, T, H, Ie, E, total, st))
    hb16 = bf16(T, H); wi16 = bf16(E * Ie, H, sigma=0.02); wo16 = bf16(E * H, Ie, sigma=0.02)
    sz5 = ctypes.c_size_t(0)
    cf.raw_cf_moe_grouped_expert_forward_bf16_workspace(T, total, E, H, Ie, None, ctypes.byref(sz5))
    ws5 = u8(sz5.value)
    mfma16("moe_grouped_expert_forward_bf16 with a workspace (grouped bf16 GEMMs, GELU rounded to bf16)", f"T={T} E={E} k={k}",
           4.0 * total * Ie * H,
           lambda: cf.cf_moe_grouped_expert_forward_bf16_ws(hb16, rw, counts, None, idx, wi16, wo16, mixed, T, H, Ie, E, total,
                                                            ws5, sz5.value, st))
    del ws5
    mfma("moe_grouped_expert_forward_bf16 (the bf16 sibling, MFMA)", f"T={T} E={E} k={k}", 4.0 * total * Ie * H,
         lambda: cf.cf_moe_grouped_expert_forward_bf16(hb16, rw, counts, offs, idx, wi16, wo16, mixed, T, H, Ie, E, total, st))
    args.iters = iters
    del ws3, gq, hb16, wi16, wo16

    # ---- the selected-expert backward's custom kernels at the same size --------------------------------
    dmixed = bf16(T, H)
    eout = bf16(total, H)
    dlog = torch.empty((T, E), dtype=torch.float32, device=dev)
    # per slot: reads a row of expert_out, writes the gradient row over it and 4 bytes; the rows of d_mixed are
    # counted once (each is used by k slots and the repeats come from cache)
    hbm("grouped route grad (row dot + weighted gather, all experts)", f"{total}x{H}", 4.0 * total * H + 2.0 * T * H + 4.0 * T * E,
        lambda: cf.cf_moe_grouped_route_grad_bf16(dmixed, eout, dlog, rw, counts, offs, idx, T, E, H, st))
    hcounts = counts.cpu().tolist(); hoffs = offs.cpu().tolist(); idx2 = idx.view(E, T)

    def per_expert():
        # the reference's sequence: two launches per expert (src/trainer.cu:7722-7725)
        for e in range(E):
            n_e = hcounts[e]
            if n_e == 0:
                continue
            slot = eout[hoffs[e]:hoffs[e] + n_e]
            cf.cf_moe_row_dot_selected_bf16(dmixed, slot, dlog, idx2[e], n_e, H, E, e, st)
            cf.cf_moe_gather_scale_rows_bf16(dmixed, slot, rw, idx2[e], n_e, e, E, H, st)
    hbm("  the same as two launches per expert", f"{total}x{H}", 4.0 * total * H + 2.0 * T * H + 4.0 * T * E, per_expert)
    dhid = torch.zeros((T, H), dtype=torch.bfloat16, device=dev)
    hbm("unpermute_add_bf16 (scatter-add, all experts)", f"{total}x{H}", 2.0 * total * H + 4.0 * T * H,
        lambda: cf.cf_moe_unpermute_add_bf16(dhid, yy, rw, counts, offs, idx, T, E, H, st))
    pre = bf16(total, Ie); gpost = bf16(total, Ie, sigma=0.01); gpre = torch.empty_like(pre)
    hbm("gelu_forward_bf16", f"{total}x{Ie}", 4.0 * total * Ie, lambda: cf.cf_gelu_forward_bf16(pre, gpre, total * Ie, st))
    hbm("gelu_backward_bf16", f"{total}x{Ie}", 6.0 * total * Ie, lambda: cf.cf_gelu_backward_bf16(pre, gpost, gpre, total * Ie, st))

    # the four bf16 GEMMs of the same backward, every expert in one launch (bf16 matrix peak 2.5 PFLOP/s)
    wo16 = bf16(E * H, Ie, sigma=0.02); wi16 = bf16(E * Ie, H, sigma=0.02)
    d_out = bf16(total, H, sigma=0.01); xg = bf16(total, H)
    d_act = torch.empty((total, Ie), dtype=torch.bfloat16, device=dev); d_x = torch.empty((total, H), dtype=torch.bfloat16, device=dev)
    g_out = torch.zeros((E * H, Ie), dtype=torch.bfloat16, device=dev); g_in = torch.zeros((E * Ie, H), dtype=torch.bfloat16, device=dev)
    fl = 2.0 * total * Ie * H
    mfma16("grouped bf16 dgrad: d_act = d_out . fc_out_w (nn)", f"{total}x{Ie}x{H}", fl,
           lambda: cf.cf_moe_grouped_gemm_bf16_nn(total, Ie, H, E, counts, offs, d_out, H, wo16, d_act, Ie, ws, sz.value, st))
    mfma16("grouped bf16 wgrad: g_out += d_out^T . act (tn, bf16 C)", f"{H}x{Ie}x~{total // E} x{E}", fl,
           lambda: cf.cf_moe_grouped_gemm_bf16_tn_accum_bf16(H, Ie, total, E, counts, offs, d_out, H, pre, Ie, g_out, st))
    mfma16("grouped bf16 dgrad: d_x = d_pre . fc_in_w (nn)", f"{total}x{H}x{Ie}", fl,
           lambda: cf.cf_moe_grouped_gemm_bf16_nn(total, H, Ie, E, counts, offs, gpost, Ie, wi16, d_x, H, ws, sz.value, st))
    mfma16("grouped bf16 wgrad: g_in += d_pre^T . x (tn, bf16 C)", f"{Ie}x{H}x~{total // E} x{E}", fl,
           lambda: cf.cf_moe_grouped_gemm_bf16_tn_accum_bf16(Ie, H, total, E, counts, offs, gpost, Ie, xg, H, g_in, st))

    # the same kernel, dense, on constant operands (no data toggling: full clock, below the power cap) with ten output
    # tiles per workgroup at two K: the difference is the K loop's time, the rest the per-tile cost
    if args.only is None or "bf16 dense" in args.only or args.only in "bf16 dense":
        Md, Nd = 16384, 10240
        for Kd in (2048, 8192):
            ad = torch.ones((Md, Kd), dtype=torch.bfloat16, device=dev); bd = torch.ones((Kd, Nd), dtype=torch.bfloat16, device=dev)
            cd = torch.empty((Md, Nd), dtype=torch.bfloat16, device=dev)
            mfma16(f"bf16 dense nn, constant operands, K = {Kd}", f"{Md}x{Nd}x{Kd}", 2.0 * Md * Nd * Kd,
                   lambda: cf.cf_gemm_bf16_nn(Md, Nd, Kd, ad, Kd, bd, Nd, cd, Nd, st))
            del ad, bd, cd

    # the whole selected-expert backward of the GELU bank in one call: FP8 recompute, route gradient, four bf16 GEMMs,
    # gelu_backward, scatter-add (16 launches per expert in the reference's host loop)
    szb = ctypes.c_size_t(0)
    cf.raw_cf_moe_grouped_gelu_backward_workspace(T, total, E, H, Ie, None, ctypes.byref(szb))
    wsb = u8(szb.value + 256)
    wsb_ptr = wsb.data_ptr() + (-wsb.data_ptr()) % 256
    hid16 = bf16(T, H); d_rw = torch.empty((T, E), dtype=torch.float32, device=dev)
    if args.only in "grouped GELU expert bank backward, whole pipeline":
        t = timed(lambda: cf.cf_moe_grouped_gelu_backward_fp8(dmixed, hq, one, 0, hid16, rw, counts, offs, idx, wg, one, wd, one, wi16, wo16,
                                                                d_rw, g_in, g_out, dhid, T, H, Ie, E, total, wsb_ptr, szb.value, st))
        fl8, fl16 = 4.0 * total * Ie * H, 8.0 * total * Ie * H
        print(f"{'grouped GELU expert bank backward, whole pipeline':<64} {f'T={T} E={E} k={k}':<26} {t * 1e6:9.1f} "
              f"{(fl8 + fl16) / t / 1e12:7.0f} TFLOP/s (FP8 recompute {fl8 / 1e12:.2f} + bf16 {fl16 / 1e12:.2f} TFLOP)", flush=True)


if __name__ == "__main__":
    main()
