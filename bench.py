#!/usr/bin/env python3
"""Benchmark of the Metis NVFP4 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

Headline: Metis NVFP4 linear TFLOP/s at 8192x4096x14336, rank 64 (config 3).
One step = one pass of the forward hot path over one batch that is already resident in HBM:
    NVFP4-quantize X (RNE)  ->  T = (X V^T) * s in bf16  ->  fused GEMM
    out = deq(Q(X)) deq(Q(W - U S V^T))^T + T U^T      (fp32 accumulate, bf16 store)
The residual weight is quantized once outside the timed region (it changes only at an
optimizer step).  The same JSON line also carries the quantizer (config 1) and the fused
RMSNorm->quant (config 2) throughput with their own rooflines, and a CPU baseline: the oracle's
restatement of the reference arithmetic timed on this host's cores on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "fp4-post_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2516.6      # dense bf16/fp16 MFMA: 256 CU x 4096 flop/clk x 2.4 GHz
QUANT_BYTES_PER_ELT = 2.5625   # 2 B read + 0.5 B codes + 1/16 B scale
NORMQ_BYTES_PER_ELT = 4.5625   # + 2 B normed
# HBM bytes per launch.  NOT measured in this run: constants from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# fp4-post_amd/metis_hip/tools/profile_workload.py on the same shapes, scaled by what the same counters read for a
# 64 MiB copy (x2.0 KiB per FETCH_SIZE unit, x1.0 KiB per WRITE_SIZE unit); summary in profiles/hbm_traffic_pmc.md
TRAFFIC_SOURCE = ("profiles/hbm_traffic_pmc.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE on profile_workload.py, "
                  "calibrated by a 64 MiB copy); a constant, not measured in this run")
TRAFFIC_GEMM_C3 = 1666.5e6      # gemm_xt_kernel: 1431.6 MB fetched (tiled f16 operands re-read below L2) + 234.9 MB written
TRAFFIC_QUANT_C1 = 94.6e6       # quant_codes_contig_kernel 88.2 MB + quant_scales_kernel 6.4 MB
TRAFFIC_NORMQ_C2 = 323.5e6      # rmsnorm_quant_rows_kernel 310.8 MB + quant_scales_kernel 12.7 MB
TRAFFIC_DECODE_C5 = 160.8e6     # the five launches of the decode layer: 150.7 MB fetched + 10.0 MB written


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.lower().startswith("model name"):
                    return ln.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or "unknown"


def outlier_activation(torch, seed, rows, cols, device):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g)
    idx = torch.randperm(cols, generator=g)[: max(1, round(cols * 0.001))]
    x[:, idx] *= 20.0
    return x.bfloat16().to(device)


def config3_inputs(torch, device, M=8192, K=4096, N=14336, r=64):
    """X ~ N(0,1); W ~ N(0, 0.02^2) + planted rank-16 spike of spectral norm 5; rank-64 truncated
    SVD of W in fp32 (eigendecomposition of W^T W, exact for the leading subspace)."""
    g = torch.Generator().manual_seed(1003)
    x = torch.randn(M, K, generator=g).bfloat16().to(device)
    w = (torch.randn(N, K, generator=g) * 0.02).to(device)
    a = torch.linalg.qr(torch.randn(N, 16, generator=g).to(device))[0]
    b = torch.linalg.qr(torch.randn(K, 16, generator=g).to(device))[0]
    sig = 5.0 * 0.9 ** torch.arange(16, device=device, dtype=torch.float32)
    w = w + (a * sig) @ b.T
    evals, evecs = torch.linalg.eigh(w.T @ w)
    v = evecs[:, -r:].flip(1)                       # [K, r]
    s = evals[-r:].flip(0).clamp_min(0).sqrt()      # [r]
    u = (w @ v) / s                                 # [N, r]
    res = (w - (u * s) @ v.T).bfloat16()
    return x, v.T.contiguous().bfloat16(), s.bfloat16(), u.contiguous().bfloat16(), res


def time_region(torch, fn, steps, warmup):
    """(wall seconds for `steps` calls, per-call kernel ms from events on the launch stream)."""
    for _ in range(warmup):
        fn(None)
    torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(pairs[i])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ev_ms = sum(a.elapsed_time(b) for a, b in pairs) / steps
    return t1 - t0, ev_ms


def region_us(torch, fn, steps, warmup):
    """Average duration of one call in microseconds: ONE pair of events around `steps` back-to-back calls on the launch
    stream (what a kernel trace of the same region adds up to, launch gaps included)."""
    for _ in range(warmup):
        fn(None)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn(None)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps * 1e3


def flushed_us(torch, fn, flush, n=15):
    """Median duration of one call (events on the launch stream) when a read of `flush` (larger than the caches and the
    256 MB memory-side cache together) runs before every call: inputs come from HBM itself, not from what the previous
    iteration of a timing loop left in a cache.  A read, not a fill: dirty lines would have to be written back while the
    timed call runs."""
    ts = []
    words = flush.view(torch.int32)
    for _ in range(n):
        words.sum()
        pair = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
        fn(pair)
        torch.cuda.synchronize()
        ts.append(pair[0].elapsed_time(pair[1]) * 1e3)
    ts.sort()
    return ts[len(ts) // 2]


def settle(torch, fn, seconds=1.0):
    """Untimed launches of the headline step until `seconds` have passed: the part's clock needs about a second under
    load to settle, whatever --warmup says.  Returns the seconds spent."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while True:
        for _ in range(10):
            fn(None)
        torch.cuda.synchronize()
        if time.perf_counter() - t0 >= seconds:
            return time.perf_counter() - t0


def ceilings_leg(torch, dev, st):
    """Byte-only and MFMA-only kernels (fp4-post_amd/csrc/ceilings.hip, built beside the library) on this device, now."""
    import ctypes
    path = os.path.join(ROOT, "fp4-post_amd", "metis_hip", "libmetis_ceilings.so")
    C = ctypes.CDLL(path)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    C.metis_ceiling_stream.restype, C.metis_ceiling_stream.argtypes = i32, [vp, vp, vp, vp, i64, i32, i32, vp]
    C.metis_ceiling_mfma.restype, C.metis_ceiling_mfma.argtypes = i32, [vp, vp, i32, i32, vp]
    out = {"source": "fp4-post_amd/csrc/ceilings.hip: kernels that only move the hot kernels' bytes, or only issue their MFMAs, "
                     "in this process on this device (events around 50 back-to-back launches)"}
    n2 = 16384 * 4096
    xb = torch.randn(n2, device=dev).bfloat16()
    nb = torch.empty(n2, dtype=torch.bfloat16, device=dev)
    cb = torch.empty(n2 // 2, dtype=torch.uint8, device=dev)
    ab = torch.empty(n2 // 16, dtype=torch.int16, device=dev)

    def us_of(fn, n=50, w=10):
        for _ in range(w):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e3
    for name, elems, mix, bpe in (("quantizer_bytes_config1", n2 // 2, 0, QUANT_BYTES_PER_ELT), ("fused_norm_bytes_config2", n2, 1, NORMQ_BYTES_PER_ELT)):
        best = None
        for grid in (768, 1024, 2048):
            def run():
                assert C.metis_ceiling_stream(xb.data_ptr(), nb.data_ptr(), cb.data_ptr(), ab.data_ptr(), elems, mix, grid, st) == 0
            us = us_of(run)
            if best is None or us < best[0]:
                best = (us, grid)
        out[name] = {"us": round(best[0], 2), "GBps_on_algorithmic_bytes": round(elems * bpe / best[0] / 1e3, 1),
                     "frac_of_hbm_peak": round(elems * bpe / best[0] / 1e3 / HBM_PEAK_GBS, 4), "grid": best[1]}
    del xb, nb, cb, ab
    res_ = torch.empty(512 * 256, dtype=torch.float32, device=dev)
    iters = 4000
    for name, src in (("mfma_f16_loop_constant_operands", torch.ones(32768, dtype=torch.float16, device=dev)),
                      ("mfma_f16_loop_normal_operands", torch.randn(32768, generator=torch.Generator().manual_seed(1)).to(torch.float16).to(dev))):
        best = 0.0
        for per_cu in (1, 2):
            grid = 256 * per_cu

            def run():
                assert C.metis_ceiling_mfma(src.data_ptr(), res_.data_ptr(), iters, grid, st) == 0
            us = us_of(run, n=5, w=2)
            best = max(best, grid * 4 * iters * 16 * 32768.0 / us / 1e6)
        out[name] = {"tflops": round(best, 1), "frac_of_mfma_peak": round(best / MFMA_PEAK_TFLOPS, 4)}
    return out


def cpu_baseline_linear(torch, x, v, s, u, res, budget_rows=2048):
    """Oracle (port of the reference arithmetic, PyTorch CPU eager) on the first rows of config 3."""
    from oracle import metis_oracle as O
    xs = x[:budget_rows].cpu()
    vc, sc, uc, rc = v.cpu(), s.cpu(), u.cpu(), res.cpu()
    reps, dt = 0, 0.0
    while dt < 12.0 and reps < 64:                      # about 10-30 s of CPU work
        t0 = time.perf_counter()
        O.metis_forward(xs, vc, sc, uc, rc, None, p32=True)
        dt += time.perf_counter() - t0
        reps += 1
    M, K, N, r = budget_rows, x.shape[1], res.shape[0], v.shape[0]
    flops = (2.0 * M * N * K + 2.0 * M * K * r + 2.0 * M * r * N) * reps
    return flops / dt / 1e12, dt, reps


def cpu_baseline_quant(torch, x, rows=8192):
    from oracle import c_oracle as C
    from oracle import metis_oracle as O
    xs = x[:rows].cpu().contiguous()
    t0 = time.perf_counter()
    O.nvfp4_pack(xs.float())
    t_torch = time.perf_counter() - t0
    C.nvfp4_pack(xs, 0)
    t0 = time.perf_counter()
    C.nvfp4_pack(xs, 0)
    t_c = time.perf_counter() - t0
    nbytes = xs.numel() * QUANT_BYTES_PER_ELT
    return nbytes / t_torch / 1e9, nbytes / t_c / 1e9, C.threads()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true", help="skip the config-5 decode-layer leg")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the one-GPU hot path only: this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    from metis_hip import ops

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    M, K, N, r = 8192, 4096, 14336, 64

    # ------------------------------------------------------------------ headline: config 3
    x, v, s, u, res = config3_inputs(torch, dev, M, K, N, r)
    pw = ops.quantize(res)                                     # cached packed residual weight
    pw.persistent = True                                       # as LinearLowbit marks a cached weight: its tiled expansion is kept
    vt = v.T.contiguous()

    # parity gate before any timing (bf16 vs bf16, P32): a 256-row slice against the CPU oracle
    from oracle import metis_oracle as O
    t_chk = torch.matmul(x[:256], vt) * s
    y_chk = ops.linear_fwd(ops.quantize(x[:256]), pw, t=t_chk, u=u)
    want = O.metis_forward(x[:256].cpu(), v.cpu(), s.cpu(), u.cpu(), res.cpu(), None, p32=True)
    err = float((y_chk.cpu().double() - want.double()).norm() / want.double().norm())
    if not err <= 2e-3:
        print(f"parity gate failed: relative Frobenius error {err:.3e} > 2e-3", file=sys.stderr)
        sys.exit(1)

    def step(ev):
        # what BitLinear.forward does for a cached weight of this size, spelled out so that the events bracket the GEMM
        # launch alone: one pass over X that quantizes it (codes and parked block maxima: the expansion forms unit and
        # scale bytes itself) and forms (X V^T) * s in bf16; the expansion into the tiled binary16 layout; the pipelined GEMM
        px, _, t = ops.quantize_project(x, v, s)
        ax = ops.expand_tiled(px, cache=False)
        if ev is not None:
            ev[0].record()
        y = ops.linear_fwd_tiled(px, pw, t=t, u=u, a_tiled=ax)
        if ev is not None:
            ev[1].record()
        return y

    settle_s = settle(torch, step, 1.0)
    wall, gemm_ms = time_region(torch, step, args.steps, args.warmup)
    flops_step = 2.0 * M * N * K + 2.0 * M * K * r + 2.0 * M * r * N
    gemm_flops = 2.0 * M * N * K + 2.0 * M * r * N             # what the fused GEMM launch computes
    value = flops_step * args.steps / wall / 1e12
    gemm_tflops = gemm_flops / (gemm_ms * 1e-3) / 1e12

    # ------------------------------------------------------------------ config 1: quantizer
    x1 = outlier_activation(torch, 1001, 8192, 4096, dev)

    from metis_hip import _lib
    L = _lib.load()
    st = torch.cuda.current_stream().cuda_stream

    def buffers(rows, cols):
        return (torch.empty(rows, cols // 2, dtype=torch.uint8, device=dev),
                torch.empty(rows, cols // 16, dtype=torch.uint8, device=dev),
                torch.empty(1, dtype=torch.float32, device=dev),
                torch.zeros(L.metis_nvfp4_workspace_bytes(rows, cols), dtype=torch.uint8, device=dev))

    # outputs and workspace are allocated once, as a C caller of the library would hold them
    qc, qs, qu, qws = buffers(8192, 4096)

    def qstep(ev):
        if ev is not None:
            ev[0].record()
        rc = L.metis_nvfp4_quant_row(x1.data_ptr(), 8192, 4096, 4096, 0, qc.data_ptr(), qs.data_ptr(), qu.data_ptr(),
                                     qws.data_ptr(), qws.numel(), st)
        if ev is not None:
            ev[1].record()
        assert rc == 0

    qsteps = max(args.steps, 100)
    _, q_pair_ms = time_region(torch, qstep, qsteps, args.warmup)
    q_ms = region_us(torch, qstep, qsteps, args.warmup) * 1e-3
    q_bytes = x1.numel() * QUANT_BYTES_PER_ELT
    q_gbs = q_bytes / (q_ms * 1e-3) / 1e9
    flush_buf = torch.zeros(512 << 20, dtype=torch.uint8, device=dev)
    q_cold_us = flushed_us(torch, qstep, flush_buf)

    # deferred scale bytes: the first launch alone (codes + parked block maxima); the consumer forms unit and bytes
    qdef = torch.empty(L.metis_nvfp4_deferred_bytes(8192, 4096), dtype=torch.uint8, device=dev)

    def qdstep(ev):
        if ev is not None:
            ev[0].record()
        rc = L.metis_nvfp4_quant_row_deferred(x1.data_ptr(), 8192, 4096, 0, None, qc.data_ptr(), qdef.data_ptr(), qdef.numel(), st)
        if ev is not None:
            ev[1].record()
        assert rc == 0

    qd_ms = region_us(torch, qdstep, qsteps, args.warmup) * 1e-3
    qd_gbs = q_bytes / (qd_ms * 1e-3) / 1e9

    # the opt-in single-launch variant (needs the device to itself: every workgroup must be resident)
    def q1step(ev):
        if ev is not None:
            ev[0].record()
        rc = L.metis_nvfp4_quant_row_resident(x1.data_ptr(), 8192, 4096, 0, qc.data_ptr(), qs.data_ptr(), qu.data_ptr(),
                                              qws.data_ptr(), qws.numel(), 0, st)
        if ev is not None:
            ev[1].record()
        assert rc == 0

    q1_ms = region_us(torch, q1step, qsteps, args.warmup) * 1e-3
    q1_gbs = q_bytes / (q1_ms * 1e-3) / 1e9

    # the round trip as config 1 states it: codes, scale bytes AND the dequantized bf16 tensor from one call
    qdq = torch.empty(8192, 4096, dtype=torch.bfloat16, device=dev)

    def qrstep(ev):
        rc = L.metis_nvfp4_quant_dequant_row(x1.data_ptr(), 8192, 4096, 0, qc.data_ptr(), qs.data_ptr(), qu.data_ptr(), qdq.data_ptr(),
                                             qws.data_ptr(), qws.numel(), st)
        assert rc == 0

    qr_ms = region_us(torch, qrstep, qsteps, args.warmup) * 1e-3
    qr_bytes = x1.numel() * NORMQ_BYTES_PER_ELT                 # 2 B read + 0.5625 B packed + 2 B dequantized
    qr_gbs = qr_bytes / (qr_ms * 1e-3) / 1e9
    del qdq

    # ------------------------------------------------------------------ config 2: fused RMSNorm -> quant
    h = outlier_activation(torch, 1002, 16384, 4096, dev)
    gamma = (1 + 0.1 * torch.randn(4096, generator=torch.Generator().manual_seed(1002))).bfloat16().to(dev)

    nc, ns, nu, nws = buffers(16384, 4096)
    normed = torch.empty(16384, 4096, dtype=torch.bfloat16, device=dev)

    def nstep(ev):
        if ev is not None:
            ev[0].record()
        rc = L.metis_rmsnorm_nvfp4_quant(h.data_ptr(), gamma.data_ptr(), 1e-6, 16384, 4096, 0, normed.data_ptr(),
                                         nc.data_ptr(), ns.data_ptr(), nu.data_ptr(), nws.data_ptr(), nws.numel(), st)
        if ev is not None:
            ev[1].record()
        assert rc == 0

    _, n_pair_ms = time_region(torch, nstep, qsteps, args.warmup)
    n_ms = region_us(torch, nstep, qsteps, args.warmup) * 1e-3
    n_bytes = h.numel() * NORMQ_BYTES_PER_ELT
    n_gbs = n_bytes / (n_ms * 1e-3) / 1e9
    n_cold_us = flushed_us(torch, nstep, flush_buf)
    del flush_buf

    ndef = torch.empty(L.metis_nvfp4_deferred_bytes(16384, 4096), dtype=torch.uint8, device=dev)

    def ndstep(ev):
        if ev is not None:
            ev[0].record()
        rc = L.metis_rmsnorm_nvfp4_quant_deferred(h.data_ptr(), gamma.data_ptr(), 1e-6, 16384, 4096, 0, normed.data_ptr(),
                                                  nc.data_ptr(), ndef.data_ptr(), ndef.numel(), st)
        if ev is not None:
            ev[1].record()
        assert rc == 0

    nd_ms = region_us(torch, ndstep, qsteps, args.warmup) * 1e-3
    nd_gbs = n_bytes / (nd_ms * 1e-3) / 1e9

    # the same under the reference's default arguments (mean mode): RMSNorm that leaves the column mean of its output, then
    # the centred quantizer on the normed tensor (mean + QDQ(x - mean), bitlinear.py:311-336)
    nm_ms = None
    try:
        nmean = torch.empty(4096, dtype=torch.float32, device=dev)
        nmws = torch.empty(max(L.metis_rmsnorm_colmean_workspace_bytes(16384, 4096), 16), dtype=torch.uint8, device=dev)

        def nmstep(ev):
            rc = L.metis_rmsnorm_colmean(h.data_ptr(), gamma.data_ptr(), 1e-6, 16384, 4096, normed.data_ptr(), nmean.data_ptr(), 1, None, 0,
                                         None, nmws.data_ptr(), nmws.numel(), st)
            assert rc == 0
            rc = L.metis_nvfp4_quant_centered(normed.data_ptr(), 16384, 4096, 4096, 0, nmean.data_ptr(), 0, 0, None, 0, 0, nc.data_ptr(),
                                              ns.data_ptr(), nu.data_ptr(), nws.data_ptr(), nws.numel(), st)
            assert rc == 0
        nm_ms = region_us(torch, nmstep, qsteps, args.warmup) * 1e-3
    except Exception as exc:  # an optional leg must not cost the headline line
        nm_err = f"{type(exc).__name__}: {exc}"[:300]

    # ------------------------------------------------------------------ the kernels that serve two consumers from one pass
    # (config-3 activation: quantizer + rank-r projection; config-4 output gradient: row- and column-blocked packing),
    # each beside the two calls it replaces
    one_pass = None
    try:
        def us_of(fn, n=40, w=10):
            for _ in range(w):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return round(e0.elapsed_time(e1) / n * 1e3, 1)
        dy4 = (torch.randn(4096, 8960, generator=torch.Generator().manual_seed(2004)) * 1e-3).bfloat16().to(dev)
        one_pass = {
            "quantize_and_project": {
                "workload": "config-3 activation bf16 [8192,4096], r = 64: NVFP4 codes + parked block maxima and (x V^T) * s",
                "two_calls_us": us_of(lambda: (ops.quantize(x, deferred=True), ops.lowrank_project(x, v, s))),
                "one_pass_us": us_of(lambda: ops.quantize_project(x, v, s))},
            "both_packings_of_dY": {
                "workload": "config-4 output gradient bf16 [4096,8960]: stochastic row-blocked and column-blocked NVFP4 packing incl. scale bytes",
                "two_calls_us": us_of(lambda: (ops.quantize(dy4, sr=True, seed=1), ops.quantize(dy4, col=True, sr=True, seed=1, offset=1 << 24))),
                "one_pass_us": us_of(lambda: ops.quantize_both_sr(dy4, seed=1, offset_row=0, offset_col=1 << 24))}}
        del dy4
    except Exception as exc:  # an optional leg must not cost the headline line
        one_pass = {"error": f"{type(exc).__name__}: {exc}"[:300]}

    # ------------------------------------------------------------------ config 5, decode step: the seven
    # projections of one Qwen2.5-7B decoder layer at M = 64 rows (rank 64), packed weights streamed once
    dec = None
    if not args.no_decode:
        try:
            shapes = [(3584, 3584), (512, 3584), (512, 3584), (3584, 3584), (18944, 3584), (18944, 3584), (3584, 18944)]
            gd = torch.Generator().manual_seed(1005)
            ws_, acts, lows = [], {}, []
            for (n_, k_) in shapes:
                ws_.append(ops.quantize((torch.randn(n_, k_, generator=gd) * 0.02).bfloat16().to(dev)))
                if k_ not in acts:
                    acts[k_] = ops.quantize(torch.randn(64, k_, generator=gd).bfloat16().to(dev))
                lows.append((torch.randn(64, 64, generator=gd).bfloat16().to(dev), torch.randn(n_, 64, generator=gd).bfloat16().to(dev)))
            outs = [torch.empty(64, n_, dtype=torch.bfloat16, device=dev) for (n_, _) in shapes]

            import ctypes
            from metis_hip import _lib as _ml

            def member_array(idx):
                arr = (_ml.LinearMember * len(idx))()
                for j, i_ in enumerate(idx):
                    # cached weights: packed, plus the same bytes in the decode layout that the decode-sized kernel streams as whole lines
                    arr[j] = _ml.LinearMember(ws_[i_].codes.data_ptr(), ws_[i_].scales.data_ptr(), ws_[i_].unit.data_ptr(),
                                              lows[i_][0].data_ptr(), lows[i_][1].data_ptr(), 64, None, outs[i_].data_ptr(),
                                              shapes[i_][0], 0, 0, ops.decode_weight(ws_[i_]).data_ptr())
                return arr
            # projection groups share their activation: q/k/v in one call, o, gate/up in one call, down
            calls = [(3584, member_array([0, 1, 2])), (3584, member_array([3])), (3584, member_array([4, 5])),
                     (18944, member_array([6]))]
            # split-K scratch of the calls that use one (the down projection); calls run in order on one stream
            need_ = max(L.metis_linear_grouped_workspace_bytes(64, k_, ctypes.cast(arr, ctypes.c_void_p), len(arr)) for k_, arr in calls)
            gws = torch.empty(max(need_, 16), dtype=torch.uint8, device=dev)

            # mean mode (the reference's default arguments): the packed activation is a centred residual and the
            # binary32 centre enters inside the same launches
            centres = {k_: (torch.randn(k_, generator=gd) * 0.1).to(dev) for k_ in acts}

            # bf16 arithmetic (the reference's all-bf16 forward): the same kernel with bf16 operands and roundings, on the
            # packed activation or on ready operands built once per activation
            aops = {k_: torch.empty(L.metis_nvfp4_decode_operand_bytes(64, k_), dtype=torch.uint8, device=dev) for k_ in acts}

            def layer(centred=False, bf16=0, row_major=False):
                s_ = torch.cuda.current_stream().cuda_stream
                for k_, arr in calls:
                    a_ = acts[k_]
                    # the activation as its quantizer leaves it for a decode-sized call: in the decode layout (no scale pointer)
                    ac_, as_ = (a_.codes.data_ptr(), a_.scales.data_ptr()) if row_major else (a_.decode_layout.data_ptr(), None)
                    if bf16 == 1:
                        rc = L.metis_linear_fwd_grouped_bf16(ac_, as_, a_.unit.data_ptr(), 64, k_,
                                                             ctypes.cast(arr, ctypes.c_void_p), len(arr), 0, gws.data_ptr(), gws.numel(), s_)
                    elif bf16 == 2:
                        rc = L.metis_nvfp4_decode_operand(a_.codes.data_ptr(), a_.scales.data_ptr(), a_.unit.data_ptr(), 64, k_, 1, None,
                                                          aops[k_].data_ptr(), s_)
                        assert rc == 0
                        rc = L.metis_linear_fwd_grouped_operand(aops[k_].data_ptr(), a_.unit.data_ptr(), 64, k_,
                                                                ctypes.cast(arr, ctypes.c_void_p), len(arr), 0, 1, gws.data_ptr(), gws.numel(), s_)
                    elif centred:
                        rc = L.metis_linear_fwd_grouped_centered(ac_, as_, a_.unit.data_ptr(), 64, k_,
                                                                 ctypes.cast(arr, ctypes.c_void_p), len(arr), 0, centres[k_].data_ptr(),
                                                                 gws.data_ptr(), gws.numel(), s_)
                    else:
                        rc = L.metis_linear_fwd_grouped(ac_, as_, a_.unit.data_ptr(), 64, k_,
                                                        ctypes.cast(arr, ctypes.c_void_p), len(arr), 0, gws.data_ptr(), gws.numel(), s_)
                    assert rc == 0

            def replay_us(fn):
                side = torch.cuda.Stream()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.stream(side):
                    fn()
                    torch.cuda.synchronize()
                    with torch.cuda.graph(graph, stream=side):
                        for _ in range(10):
                            fn()
                graph.replay()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(10):
                    graph.replay()
                e1.record()
                torch.cuda.synchronize()
                return e0.elapsed_time(e1) / 100 * 1e3
            d_us = replay_us(layer)
            d_rm_us = replay_us(lambda: layer(row_major=True))
            d_mean_us = replay_us(lambda: layer(True))
            d_bf16_us = replay_us(lambda: layer(bf16=1))
            d_bf16_op_us = replay_us(lambda: layer(bf16=2))
            d_bytes = sum(n_ * k_ for n_, k_ in shapes) * (0.5 + 1.0 / 16)
            d_flops = sum(2.0 * 64 * n_ * k_ for n_, k_ in shapes)
            dec = {"workload": "config 5 decode: 7 projections of a Qwen2.5-7B layer, M=64, r=64, packed weights cached in the decode layout, "
                               "activations in the decode layout as their quantizer's second launch leaves them; q/k/v and gate/up as grouped calls (graph replay)",
                   "us_per_layer": round(d_us, 1), "tflops": round(d_flops / d_us / 1e6, 1),
                   "us_per_layer_row_major_activation": round(d_rm_us, 1),
                   "roofline": {"bound": "hbm", "kernel": "gemm_nvfp4_skinny_grouped_kernel", "achieved": round(d_bytes / d_us / 1e3, 1),
                                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(d_bytes / d_us / 1e3 / HBM_PEAK_GBS, 4),
                                "traffic": TRAFFIC_DECODE_C5, "traffic_source": TRAFFIC_SOURCE},
                   "mean_mode_us_per_layer": round(d_mean_us, 1),
                   "bf16_arithmetic_us_per_layer": {"packed_activation": round(d_bf16_us, 1),
                                                    "ready_operands_incl_4_builds": round(d_bf16_op_us, 1)}}
        except Exception as exc:  # an optional leg must not cost the headline line
            dec = {"workload": "config 5 decode", "error": f"{type(exc).__name__}: {exc}"[:300]}

    # ------------------------------------------------------------------ config 4: one QAT projection, forward +
    # dgrad + wgrad through the module path (L = 4096 tokens, gate/up shape 1536 -> 8960, bf16 tensors)
    qat = None
    if not args.no_decode:
        try:
            from metis_hip import LinearLowbit, LinearLowbitFunction, MetisArgs
            LinearLowbitFunction.compute_dtype = torch.float32
            margs = MetisArgs.direct_fp4()
            margs.cache_quantized_weight = True
            lin = LinearLowbit(1536, 8960, bias=False, args=margs, device=dev, storage_dtype=torch.bfloat16,
                               compute_dtype=torch.float32)
            xq_ = torch.randn(1, 4096, 1536, generator=torch.Generator().manual_seed(1004)).bfloat16().to(dev).requires_grad_(True)
            dy_ = (torch.randn(1, 4096, 8960, generator=torch.Generator().manual_seed(2004)) * 1e-3).bfloat16().to(dev)
            dy_ = dy_.float()        # the layer's output is binary32 in this arithmetic: the upstream gradient arrives in that dtype

            def qat_step(ev):
                if ev is not None:
                    ev[0].record()
                y_ = lin(xq_)
                y_.backward(dy_)
                if ev is not None:
                    ev[1].record()
                lin.weight.grad = None
                xq_.grad = None
            _, qat_ms = time_region(torch, qat_step, 10, 3)
            qat = {"workload": "config 4: LinearLowbit 1536->8960, L=4096, forward + dgrad + wgrad incl. RNE/SR quantization "
                               "of X, dY (row and column blocked) through the Python module path (P32 arithmetic)",
                   "us_per_step": round(qat_ms * 1e3, 1), "tflops": round(3 * 2.0 * 4096 * 1536 * 8960 / (qat_ms * 1e-3) / 1e12, 1)}
        except Exception as exc:  # an optional leg must not cost the headline line
            qat = {"workload": "config 4 projection", "error": f"{type(exc).__name__}: {exc}"[:300]}
        # the same projection under the reference's default arguments: mean mode for activations and gradients
        try:
            from metis_hip import BitLinear
            mean_args = MetisArgs(cache_quantized_weight=True)
            mean_args.enable_forward_svd = False
            mlin = BitLinear(1536, 8960, args=mean_args, bias=False, dtype=torch.bfloat16, compute_dtype=torch.float32).to(dev).warmup_linear

            def mean_step(ev):
                if ev is not None:
                    ev[0].record()
                y_ = mlin(xq_)
                y_.backward(dy_)
                if ev is not None:
                    ev[1].record()
                mlin.weight.grad = None
                xq_.grad = None
            _, mean_ms = time_region(torch, mean_step, 10, 3)
            qat["mean_mode"] = {"workload": "same projection, metis_mode=mean for activations and output gradients (column "
                                            "mean + centred NVFP4 residual, rank-one terms inside the GEMMs)",
                                "us_per_step": round(mean_ms * 1e3, 1)}
            LinearLowbitFunction.enable_activation_svd = False     # class-level switches: back to the direct mode
            LinearLowbitFunction.enable_backward_svd = False
        except Exception as exc:
            if isinstance(qat, dict):
                qat["mean_mode"] = {"error": f"{type(exc).__name__}: {exc}"[:300]}

    # the same projection under the NV recipe (tiled random Hadamard rotation around the weight QDQ and the two
    # weight-gradient operands): on the packed kernels, and on the module's generic path (rotation kernel, three-call
    # QDQ, dequantized tensors, torch matmuls) that hadamard_backend = "torch_gemm" selects
    if not args.no_decode and isinstance(qat, dict):
        try:
            nv_args = MetisArgs.direct_fp4()
            nv_args.cache_quantized_weight = True
            nlin = LinearLowbit(1536, 8960, bias=False, args=nv_args, device=dev, storage_dtype=torch.bfloat16, compute_dtype=torch.float32)
            LinearLowbitFunction.enable_nv_recipe = True

            def nv_step(ev):
                if ev is not None:
                    ev[0].record()
                y_ = nlin(xq_)
                y_.backward(dy_)
                if ev is not None:
                    ev[1].record()
                nlin.weight.grad = None
                xq_.grad = None
            nv = {"workload": "same projection, enable_nv_recipe (rotation fused into the row quantizer, tiled GEMM operands rotated back "
                              "block by block, quantization blocks along the last dimension as in the reference)"}
            for backend, key in (("auto", "us_per_step"), ("torch_gemm", "us_per_step_generic_path")):
                LinearLowbitFunction.hadamard_backend = backend
                nlin._quantized_weight_cache = None
                _, nv_ms = time_region(torch, nv_step, 10, 3)
                nv[key] = round(nv_ms * 1e3, 1)
            qat["nv_recipe"] = nv
        except Exception as exc:
            qat["nv_recipe"] = {"error": f"{type(exc).__name__}: {exc}"[:300]}
        finally:
            LinearLowbitFunction.enable_nv_recipe = False
            LinearLowbitFunction.hadamard_backend = "auto"

    # config 4 as named: gate, up and down projections of the 1.5B-class MLP, each a rank-32 BitLinear, forward + backward
    if not args.no_decode and isinstance(qat, dict):
        try:
            from metis_hip import BitLinear
            a4 = MetisArgs.direct_fp4(forward_svd_rank=32)
            g4 = torch.Generator().manual_seed(1004)
            projs = []
            for (k_, n_) in ((1536, 8960), (1536, 8960), (8960, 1536)):
                bl = BitLinear(k_, n_, args=a4, bias=False, dtype=torch.bfloat16, compute_dtype=torch.bfloat16).to(dev)
                with torch.no_grad():
                    bl.warmup_linear.weight.copy_((torch.randn(n_, k_, generator=g4) * 0.02).bfloat16())
                bl.split()
                projs.append(bl)
            x_h = torch.randn(1, 4096, 1536, generator=g4).bfloat16().to(dev).requires_grad_(True)
            x_i = torch.randn(1, 4096, 8960, generator=g4).bfloat16().to(dev).requires_grad_(True)
            dy_i = (torch.randn(1, 4096, 8960, generator=g4) * 1e-3).bfloat16().to(dev)
            dy_h = (torch.randn(1, 4096, 1536, generator=g4) * 1e-3).bfloat16().to(dev)

            def mlp_step(ev):
                if ev is not None:
                    ev[0].record()
                for bl, xx, dd in ((projs[0], x_h, dy_i), (projs[1], x_h, dy_i), (projs[2], x_i, dy_h)):
                    bl(xx).backward(dd)
                if ev is not None:
                    ev[1].record()
                for bl in projs:
                    for p_ in bl.parameters():
                        p_.grad = None
                x_h.grad = None
                x_i.grad = None
            _, mlp_ms = time_region(torch, mlp_step, 10, 3)
            qat["three_projections"] = {"workload": "gate, up, down as BitLinear r=32 (bf16 arithmetic, direct NVFP4 mode), L=4096: forward + "
                                                    "dgrad + wgrad + rank-r gradients of each, through the modules",
                                        "us_per_step": round(mlp_ms * 1e3, 1),
                                        "tflops": round(3 * 3 * 2.0 * 4096 * 1536 * 8960 / (mlp_ms * 1e-3) / 1e12, 1)}
            LinearLowbitFunction.compute_dtype = torch.float32
            del projs
        except Exception as exc:
            qat["three_projections"] = {"error": f"{type(exc).__name__}: {exc}"[:300]}

    # ------------------------------------------------------------------ the "svd" mode of the activation decomposition:
    # ker = U diag(s) V formed in registers, x - ker encoded, packed residual (and the dense sum) written
    svd_leg = None
    if not args.no_decode:
        try:
            gs = torch.Generator().manual_seed(1007)
            Ls, Ds, rs = 4096, 3584, 64
            xs_ = outlier_activation(torch, 1008, Ls, Ds, dev)
            us32 = (torch.randn(Ls, rs, generator=gs) * 0.3).to(dev)
            vt32 = (torch.randn(rs, Ds, generator=gs) / Ds ** 0.5).to(dev)
            flops_s = 2.0 * Ls * Ds * rs
            svd_leg = {"workload": f"metis_nvfp4_quant_lowrank_residual on bf16 [{Ls},{Ds}], rank {rs}: binary32 fused multiply-adds on the "
                                   "vector units in a fixed order (bit parity with the CPU restatement), 2 r flops and 2.5625 B per element",
                       "bound": "valu_f32", "peak": 157.3, "unit": "TFLOP/s"}
            for tag, mode_, u_, v_ in (("binary32", ops.MODE_P32, us32, vt32), ("bf16", ops.MODE_PB16, us32.bfloat16(), vt32.bfloat16())):
                for dense_ in (False, True):
                    us_t = region_us(torch, lambda ev: ops.quantize_lowrank_residual(xs_, u_, v_, mode_, dense=dense_), 20, 5)
                    svd_leg[f"{tag}_{'dense' if dense_ else 'packed'}_us"] = round(us_t, 2)
                    if not dense_:
                        svd_leg[f"{tag}_frac"] = round(flops_s / (us_t * 1e-6) / 1e12 / 157.3, 4)
            from metis_hip.quant import Cast2NVFp4e2m1BlockNOSR as Qn

            def op_by_op(ev=None):
                ker = us32 @ vt32
                return ker + Qn.quantize_dequantize(xs_.float() - ker)
            svd_leg["binary32_op_by_op_us"] = round(region_us(torch, op_by_op, 10, 3), 2)
        except Exception as exc:  # an optional leg must not cost the headline line
            svd_leg = {"error": f"{type(exc).__name__}: {exc}"[:300]}

    # ------------------------------------------------------------------ a tile-starved shape: 1024-token prefill
    # through the Qwen2.5-7B down projection (56 output tiles on 256 CUs; K split through a workspace)
    prefill = None
    if not args.no_decode:
        try:
            gp = torch.Generator().manual_seed(1005)
            xp = ops.quantize(outlier_activation(torch, 1006, 1024, 18944, dev))
            wp = ops.quantize((torch.randn(3584, 18944, generator=gp) * 0.02).bfloat16().to(dev))
            tp_ = torch.randn(1024, 64, generator=gp).bfloat16().to(dev)
            up_ = torch.randn(3584, 64, generator=gp).bfloat16().to(dev)

            def prefill_step(ev):
                if ev is not None:
                    ev[0].record()
                ops.linear_fwd(xp, wp, t=tp_, u=up_)
                if ev is not None:
                    ev[1].record()
            _, pf_ms = time_region(torch, prefill_step, 20, 5)
            prefill = {"workload": "1024-token prefill, Qwen2.5-7B down projection 18944->3584, r=64, packed operands "
                                   "(split-K GEMM + reduce)",
                       "us_per_call": round(pf_ms * 1e3, 1),
                       "tflops": round(2.0 * 1024 * 3584 * (18944 + 64) / (pf_ms * 1e-3) / 1e12, 1)}
        except Exception as exc:  # an optional leg must not cost the headline line
            prefill = {"workload": "short prefill projection", "error": f"{type(exc).__name__}: {exc}"[:300]}

    # ------------------------------------------------------------------ config 5 through the modules: one
    # Qwen2.5-7B-shaped decoder layer, every projection a rank-64 BitLinear, fused RMSNorm->quant in front of
    # q/k/v and gate/up; prefill of 8 x 2048 tokens, then a decode step of 64 sequences against a 2048-token KV cache
    layer_leg = None
    if not args.no_decode:
        try:
            from transformers.models.qwen2.modeling_qwen2 import Qwen2Config, Qwen2DecoderLayer, Qwen2RotaryEmbedding
            from metis_hip import MetisArgs, replace_model_with_metis
            cfg = Qwen2Config(hidden_size=3584, intermediate_size=18944, num_attention_heads=28, num_key_value_heads=4,
                              head_dim=128, num_hidden_layers=1, vocab_size=128, max_position_embeddings=4096)
            cfg._attn_implementation = "sdpa"
            lyr = Qwen2DecoderLayer(cfg, layer_idx=0).to(torch.bfloat16)
            gl = torch.Generator().manual_seed(1005)
            with torch.no_grad():
                for name_, p_ in lyr.named_parameters():
                    if p_.dim() == 2 or name_.endswith("bias"):
                        p_.copy_((torch.randn(p_.shape, generator=gl) * 0.02).to(p_.dtype))
            holder = torch.nn.ModuleDict({"layer": lyr.to(dev)})
            replace_model_with_metis(holder, MetisArgs.direct_fp4(forward_svd_rank=64), fuse_norms=True)
            rope = Qwen2RotaryEmbedding(cfg).to(dev)
            xp_ = torch.randn(8, 2048, 3584, generator=gl).bfloat16().to(dev)
            pos_p = torch.arange(2048, device=dev).unsqueeze(0).expand(8, -1)
            pe_p = rope(xp_, pos_p)
            xd_ = torch.randn(64, 1, 3584, generator=gl).bfloat16().to(dev)
            pos_d = torch.full((64, 1), 2048, dtype=torch.long, device=dev)
            pe_d = rope(xd_, pos_d)

            def prefill_layer(ev):
                if ev is not None:
                    ev[0].record()
                with torch.no_grad():
                    holder["layer"](xp_, position_embeddings=pe_p, attention_mask=None, position_ids=pos_p)
                if ev is not None:
                    ev[1].record()
            _, pl_ms = time_region(torch, prefill_layer, 10, 3)
            lin_flops = 2.0 * 16384 * 233.05e6                       # 233.05 M linear parameters per layer
            # the projections and norms alone (what this library provides): the layer minus attention
            def decode_layer(ev=None):
                if ev is not None:
                    ev[0].record()
                with torch.no_grad():
                    holder["layer"](xd_, position_embeddings=pe_d, attention_mask=None, position_ids=pos_d)
                if ev is not None:
                    ev[1].record()
            _, dl_ms = time_region(torch, decode_layer, 50, 10)
            try:
                dl_graph_us = replay_us(decode_layer)
            except Exception as exc_:
                dl_graph_us = None
            dec_bytes = 233.05e6 * (0.5 + 1.0 / 16)
            layer_leg = {"workload": "config 5: Qwen2.5-7B-shaped decoder layer through the patched modules (BitLinear r=64, fused "
                                     "RMSNorm->NVFP4, bf16 arithmetic), no autograd: prefill 8x2048 tokens, then a 64x1 decode step "
                                     "(attention by torch SDPA, causal, no KV history in the decode step)",
                         "prefill_ms": round(pl_ms, 3), "prefill_linear_tflops": round(lin_flops / (pl_ms * 1e-3) / 1e12, 1),
                         "decode_us_eager": round(dl_ms * 1e3, 1),
                         "decode_us_graph_replay": None if dl_graph_us is None else round(dl_graph_us, 1),
                         "decode_packed_weight_GBps": None if dl_graph_us is None else round(dec_bytes / dl_graph_us / 1e3, 1)}
            del holder, lyr
            # the same decode step under the NV recipe (weights packed in the rotated domain; the activation's operand
            # carries the rotation, so the decode-sized kernel still streams the packed weights)
            try:
                from metis_hip import LinearLowbitFunction as F_
                lyr = Qwen2DecoderLayer(cfg, layer_idx=0).to(torch.bfloat16)
                gl = torch.Generator().manual_seed(1005)
                with torch.no_grad():
                    for name_, p_ in lyr.named_parameters():
                        if p_.dim() == 2 or name_.endswith("bias"):
                            p_.copy_((torch.randn(p_.shape, generator=gl) * 0.02).to(p_.dtype))
                holder = torch.nn.ModuleDict({"layer": lyr.to(dev)})
                nv_args = MetisArgs.direct_fp4(forward_svd_rank=64)
                nv_args.enable_nv_recipe = True
                replace_model_with_metis(holder, nv_args, fuse_norms=True)
                layer_leg["decode_us_graph_replay_nv_recipe"] = round(replay_us(decode_layer), 1)
                del holder, lyr
            except Exception as exc_:
                layer_leg["decode_us_graph_replay_nv_recipe"] = f"{type(exc_).__name__}: {exc_}"[:200]
            finally:
                F_.enable_nv_recipe = False
        except Exception as exc:  # an optional leg must not cost the headline line
            layer_leg = {"workload": "config 5 decoder layer", "error": f"{type(exc).__name__}: {exc}"[:300]}

    line = {
        "metric": "Metis NVFP4 linear TFLOP/s at 8192x4096x14336 (rank 64)",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "nvfp4 (e2m1 x e4m3) expanded exactly to f16, f32 accumulate; low-rank bf16",
        "data": "synthetic",
        "settle_s": round(settle_s, 2),
        "config": {"workload": "config 3: Metis low-rank-residual linear forward, X[8192,4096] W[14336,4096] r=64; "
                               "step = one pass over X (NVFP4 codes + block maxima, and X.V^T*s) + expand X to tiled f16 (forms unit and scale bytes) + fused pipelined GEMM (packed W and its tiled f16 expansion cached)",
                   "parity_mode": "P32", "parity_rel_fro_256_rows": err},
        "roofline": {"bound": "mfma", "kernel": "gemm_xt_kernel", "achieved": round(gemm_tflops, 2),
                     "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(gemm_tflops / MFMA_PEAK_TFLOPS, 4),
                     "traffic": TRAFFIC_GEMM_C3, "traffic_source": TRAFFIC_SOURCE, "kernel_ms": round(gemm_ms, 4)},
        "quant": {"workload": "config 1: NVFP4 RNE quantize bf16 [8192,4096] (P32), codes+scales+unit",
                  "value": round(q_gbs, 1), "unit": "GB/s", "us_per_call": round(q_ms * 1e3, 2),
                  "timing": "events around the region of back-to-back calls on the launch stream; us_per_call_event_pairs brackets every call with its own pair",
                  "us_per_call_event_pairs": round(q_pair_ms * 1e3, 2),
                  "us_per_call_caches_flushed": round(q_cold_us, 2),
                  "caches_flushed": "a read of 512 MiB before every call (own event pair, median of 15): nothing is served from the 256 MB "
                                    "memory-side cache, which in the back-to-back loop still holds the 67 MB input of the previous call",
                  "round_trip": {"workload": "the same tensor through metis_nvfp4_quant_dequant_row: codes + scale bytes + unit + the dequantized bf16 "
                                             "tensor (config 1's three outputs) from one call of two launches; 4.5625 B/element = 153.09 MB",
                                 "value": round(qr_gbs, 1), "unit": "GB/s", "us_per_call": round(qr_ms * 1e3, 2),
                                 "frac": round(qr_gbs / HBM_PEAK_GBS, 4)},
                  "roofline": {"bound": "hbm", "kernel": "quant_codes_contig_kernel+quant_scales_kernel",
                               "achieved": round(q_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                               "frac": round(q_gbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_QUANT_C1, "traffic_source": TRAFFIC_SOURCE},
                  "single_launch": {"value": round(q1_gbs, 1), "unit": "GB/s", "us_per_call": round(q1_ms * 1e3, 2),
                                           "frac": round(q1_gbs / HBM_PEAK_GBS, 4)},
                  "deferred_scale_bytes": {"workload": "the same tensor through metis_nvfp4_quant_row_deferred: codes + parked bf16 block "
                                                       "maxima (2 B/block instead of the 1 B/block of scale bytes); unit and E4M3 bytes are "
                                                       "formed by the consumer (the tiled expansion ahead of the GEMM, as in the headline "
                                                       "step); priced on the same 2.5625 B/element",
                                           "value": round(qd_gbs, 1), "unit": "GB/s", "us_per_call": round(qd_ms * 1e3, 2),
                                           "frac": round(qd_gbs / HBM_PEAK_GBS, 4)}},
        "rmsnorm_quant": {"workload": "config 2: fused RMSNorm->NVFP4 bf16 [16384,4096] (P32), normed+codes+scales",
                          "value": round(n_gbs, 1), "unit": "GB/s", "us_per_call": round(n_ms * 1e3, 2),
                          "us_per_call_event_pairs": round(n_pair_ms * 1e3, 2),
                          "us_per_call_caches_flushed": round(n_cold_us, 2),
                          "roofline": {"bound": "hbm", "kernel": "rmsnorm_quant_rows_kernel+quant_scales_kernel",
                                       "achieved": round(n_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                       "frac": round(n_gbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_NORMQ_C2,
                                       "traffic_source": TRAFFIC_SOURCE},
                          "mean_mode": ({"workload": "the reference's default arguments: metis_rmsnorm_colmean (normed + column mean over tokens "
                                                     "from one pass) + metis_nvfp4_quant_centered on the normed tensor (binary32 centre); four "
                                                     "launches, priced on the same 4.5625 B/element (the quantizer's re-read of the normed "
                                                     "tensor is not algorithmic)",
                                         "value": round(n_bytes / (nm_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "us_per_call": round(nm_ms * 1e3, 2),
                                         "frac": round(n_bytes / (nm_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)} if nm_ms is not None else {"error": nm_err}),
                          "deferred_scale_bytes": {"workload": "the same through metis_rmsnorm_nvfp4_quant_deferred (normed + codes + parked "
                                                               "block maxima; unit and E4M3 bytes formed by the consumer); priced on the "
                                                               "same 4.5625 B/element",
                                                   "value": round(nd_gbs, 1), "unit": "GB/s", "us_per_call": round(nd_ms * 1e3, 2),
                                                   "frac": round(nd_gbs / HBM_PEAK_GBS, 4)}},
    }
    try:
        line["ceilings"] = ceilings_leg(torch, dev, st)
    except Exception as exc:  # an optional leg must not cost the headline line
        line["ceilings"] = {"error": f"{type(exc).__name__}: {exc}"[:300]}
    if one_pass is not None:
        line["one_pass_kernels"] = one_pass
    if dec is not None:
        line["decode_layer"] = dec
    if layer_leg is not None:
        line["decoder_layer_modules"] = layer_leg
    if qat is not None:
        line["qat_projection"] = qat
    if prefill is not None:
        line["short_prefill_projection"] = prefill
    if svd_leg is not None:
        line["svd_mode_residual_quant"] = svd_leg
    if not args.no_cpu_baseline:
        torch_threads = torch.get_num_threads()
        cpu_tflops, cpu_dt, cpu_reps = cpu_baseline_linear(torch, x, v, s, u, res)
        q_torch, q_c, c_threads = cpu_baseline_quant(torch, x1)
        line["cpu_baseline"] = {
            "value": round(cpu_tflops, 4), "unit": "TFLOP/s", "cores": torch_threads, "kind": "port", "cpu_model": cpu_model(),
            "sample": f"oracle metis_forward (PyTorch CPU eager restatement of the reference) on the first 2048 of "
                      f"8192 rows incl. QDQ of the full residual weight each pass, {cpu_reps} passes, {cpu_dt:.1f} s",
            "quant_GBps_torch_eager": round(q_torch, 2), "quant_GBps_c_port": round(q_c, 2),
            "quant_c_port_threads": c_threads, "quant_sample": "all 8192 rows of config 1, one pass each",
        }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
