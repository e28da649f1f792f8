"""Profiling workload: a few launches of each hot kernel at the benchmark shapes, plus a plain
device-to-device copy of known size that calibrates the FETCH_SIZE / WRITE_SIZE counters.

    rocprofv3 --kernel-trace --stats -- python3 fp4-post_amd/metis_hip/tools/profile_workload.py
    rocprofv3 --pmc FETCH_SIZE       -- python3 fp4-post_amd/metis_hip/tools/profile_workload.py
    rocprofv3 --pmc WRITE_SIZE       -- python3 fp4-post_amd/metis_hip/tools/profile_workload.py

`--extra` adds the other kernels of the library at representative shapes: bf16-arithmetic, stochastic-rounding,
column-blocked, binary32-input and two-packings-in-one-pass quantizers, the K-sliced rank-r projection, the skinny (decode) GEMM, the split-K GEMM with its reduction and
the kernels of the mean mode.

    rocprofv3 --kernel-trace --stats -- python3 fp4-post_amd/metis_hip/tools/profile_workload.py --extra

`--decode` runs the four grouped GEMM calls of one 7B-class decoder layer at 64 tokens (q/k/v, o, gate/up, down) next to
the same calibration copy: the decode leg of the benchmark.

    rocprofv3 --pmc FETCH_SIZE       -- python3 fp4-post_amd/metis_hip/tools/profile_workload.py --decode
"""
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from metis_hip import ops  # noqa: E402


def main(reps: int = 5):
    g = torch.Generator().manual_seed(1001)
    x = torch.randn(8192, 4096, generator=g).bfloat16().cuda()          # config 1 / config 3 activations
    h = torch.randn(16384, 4096, generator=g).bfloat16().cuda()         # config 2 hidden states
    gamma = (1 + 0.1 * torch.randn(4096, generator=g)).bfloat16().cuda()
    w = (torch.randn(14336, 4096, generator=g) * 0.02).bfloat16().cuda()
    t = torch.randn(8192, 64, generator=g).bfloat16().cuda()
    u = torch.randn(14336, 64, generator=g).bfloat16().cuda()
    v = (torch.randn(64, 4096, generator=g) / 64).bfloat16().cuda()
    s = torch.rand(64, generator=g).bfloat16().cuda()
    dy = (torch.randn(8192, 14336, generator=g) * 1e-3).bfloat16().cuda()
    y = torch.empty_like(x)
    xs = x[:4096, :3584].contiguous()                                   # svd mode: [4096, 3584], rank 64
    us = (torch.randn(4096, 64, generator=g) * 0.3).cuda()
    vt = (torch.randn(64, 3584, generator=g) / 60).cuda()
    pw = ops.quantize(w)
    pw.persistent = True                                                # a cached weight: the pipelined GEMM on tiled expansions
    for _ in range(reps):
        y.copy_(x)                                                      # calibration: 64 MiB read, 64 MiB written
        px = ops.quantize(x)
        ops.rmsnorm_quantize(h, gamma, 1e-6)
        # deferred scale bytes: the quantizers' first launch alone, the expansion forms unit and bytes (expand_xt_kernel<0, 0, 1, 0>)
        ops.expand_tiled(ops.quantize(x, deferred=True), cache=False)
        ops.rmsnorm_quantize(h, gamma, 1e-6, deferred=True)
        ops.quantize_dequantize(x)                                      # round trip: quant_codes_contig_kernel + quant_scales_dequant_kernel
        normed, me, _ = ops.rmsnorm_colmean(h, gamma, 1e-6, torch.float32)   # mean mode: rmsnorm_colsum_rows_kernel + finish
        ops.quantize(normed, 0, center=me)                              # ... and the centred quantizer on the normed tensor
        ops.quantize_lowrank_residual(xs, us, vt, 0)                    # svd mode: quant_lowrank_residual_kernel + scales
        ops.quantize_lowrank_residual(xs, us, vt, 0, dense=True)        # ... + lowrank_add_dequant_kernel
        ops.linear_fwd(px, pw, t=t, u=u)                                # expand_xt_kernel + gemm_xt_kernel
        ops.linear_fwd(px, pw, t=t, u=u, tiled=False, split_k=False)    # gemm_nvfp4_large_kernel (expansion inside the K loop)
        _, t_ = ops.lowrank_project(x, v, s)                            # lowrank_nt_kernel<2, -1>: x V^T and (x V^T) * s
        ops.quantize_project(x, v, s)                                   # lowrank_nt_kernel<2, 0>: the same pass also quantizes x
        ops.lowrank_contract_tokens(dy, t_)                             # lowrank_tn_kernel + finish: dY^T t
    torch.cuda.synchronize()
    del px, pw, y
    torch.cuda.synchronize()


def extra(reps: int = 5):
    g = torch.Generator().manual_seed(1002)
    xf = torch.randn(8192, 4096, generator=g).cuda()                    # binary32, not bf16-valued
    x = xf.bfloat16()
    dec = torch.randn(64, 18944, generator=g).bfloat16().cuda()         # decode step: 64 tokens
    pre = torch.randn(1024, 18944, generator=g).bfloat16().cuda()       # short prefill
    w_up = ops.quantize((torch.randn(18944, 3584, generator=g) * 0.02).bfloat16().cuda())
    w_down = ops.quantize((torch.randn(3584, 18944, generator=g) * 0.02).bfloat16().cuda())
    p_dec_up, p_dec_down, p_pre = ops.quantize(dec[:, :3584].contiguous()), ops.quantize(dec), ops.quantize(pre)
    me_cache = torch.zeros(3584, dtype=torch.bfloat16, device="cuda")
    me_down = torch.full((18944,), 0.01, device="cuda")
    v_up = (torch.randn(128, 3584, generator=g) / 60).bfloat16().cuda()   # the stacked V of gate and up, r = 64 each
    s_up = torch.rand(128, generator=g).bfloat16().cuda()
    u_up = (torch.randn(18944, 64, generator=g) * 0.1).bfloat16().cuda()
    # bf16 arithmetic at decode size: operands packed in that arithmetic, the reference's roundings in the GEMM
    w_up16 = ops.quantize((torch.randn(18944, 3584, generator=g) * 0.02).bfloat16().cuda(), 1)
    p_dec16 = ops.quantize(dec[:, :3584].contiguous(), 1)
    me16 = torch.full((3584,), 0.01, dtype=torch.bfloat16, device="cuda")
    v_pre = (torch.randn(64, 18944, generator=g) / 130).bfloat16().cuda()
    s_pre = torch.rand(64, generator=g).bfloat16().cuda()
    for i in range(reps):
        ops.linear_fwd_grouped(p_dec16, [(w_up16, None, None, None), (w_up16, None, None, None)], reference_rounding=True)
        ops.linear_fwd_grouped(p_dec16, [(w_up16, None, None, None), (w_up16, None, None, None)], reference_rounding=True, center=me16)
        ops.quantize(x, 1)                                              # bf16 arithmetic, round to nearest
        ops.quantize(x, 0, col=True)                                    # column-blocked
        ops.quantize(x, 0, sr=True, seed=i)                             # stochastic rounding, own stream
        ops.quantize(x, 0, sr=True, col=True, seed=i)
        ops.quantize(xf, 0)                                             # binary32 input
        ops.quantize(xf, 0, sr=True, col=True, seed=i)
        ops.quantize_both_sr(x, 0, seed=i, offset_row=0, offset_col=1 << 24)     # row and column packings of one tensor in one pass
        ops.quantize_both_sr(xf, 0, seed=i, offset_row=0, offset_col=1 << 24)
        ops.lowrank_project(pre, v_pre, s_pre)                          # 1024 x 18944, r 64: 16 K slices + finish
        ops.linear_fwd(p_dec_up, w_up)                                  # skinny: 64 x 18944 x 3584
        ops.linear_fwd(p_dec_down, w_down)                              # skinny: 64 x 3584 x 18944
        ops.linear_fwd(p_pre, w_down)                                   # split-K: 1024 x 3584 x 18944
        # mean mode: column mean, centred quantizers, packed weight x mean, rank-one operands
        me = ops.column_mean(x, torch.float32)
        ops.column_mean(xf, torch.float32)
        ops.quantize(x, 0, center=me)                                   # binary32 arithmetic: literal element rule
        ops.quantize(x, 1, center=me.bfloat16())                        # bf16 arithmetic: hardware converter
        ops.quantize(xf, 0, sr=True, col=True, seed=i, center=me)
        wm = ops.matvec(w_up, me[:3584])
        ops.rank_one_operands(18944, 3584, (wm, me[:3584]), (wm, me[:3584]))
        # mean mode at decode size: running mean, centred quantizer, rank-r projection, centre inside the grouped GEMM
        xd = dec[:, :3584].contiguous()
        me_d, me_d32 = ops.column_mean_running(xd, me_cache, 4096, torch.bfloat16)
        p_res = ops.quantize(xd, 1, center=me_d)
        _, t_d = ops.lowrank_project(xd, v_up, s_up)
        ops.linear_fwd_grouped(p_res, [(w_up, t_d[:, :64], u_up, None), (w_up, t_d[:, 64:], u_up, None)], center=me_d32)
        ops.linear_fwd_grouped(p_dec_down, [(w_down, None, None, None)], center=me_down)     # K in slices, centre inside
        # decode-sized layer call in bf16 arithmetic, small steps merged: quantizer || projection's partial sums, then
        # finishing step || operand build (gate/up's stacked V on a quantized activation; down's own V)
        p_up16 = ops.quantize(xd, 1, deferred=True)
        ops.project_and_operand(xd, v_up, s_up, p_up16, 1)
        p_dn16, pending = ops.quantize_project_decode(dec, v_pre, 1)
        ops.project_and_operand(dec, v_pre, s_pre, p_dn16, 1, pending=pending)
        # NV recipe at decode size: the activation's operand rotated for a weight packed in the rotated domain
        ops.decode_operand(ops.quantize(dec, 1, deferred=True), 1, rotate=0x5a3c)
    torch.cuda.synchronize()


def decode(reps: int = 5):
    g = torch.Generator().manual_seed(1005)
    x = torch.randn(8192, 4096, generator=g).bfloat16().cuda()
    y = torch.empty_like(x)
    groups = []
    for k, ns in ((3584, (3584, 512, 512)), (3584, (3584,)), (3584, (18944, 18944)), (18944, (3584,))):
        a = ops.quantize(torch.randn(64, k, generator=g).bfloat16().cuda())
        members = [(ops.quantize((torch.randn(n, k, generator=g) * 0.02).bfloat16().cuda()), torch.randn(64, 64, generator=g).bfloat16().cuda(),
                    torch.randn(n, 64, generator=g).bfloat16().cuda(), None) for n in ns]
        for m in members:
            m[0].persistent = True                                      # cached weights: streamed from the decode layout
        groups.append((a, members))
    for _ in range(reps):
        y.copy_(x)                                                      # calibration: 64 MiB read, 64 MiB written
        for a, members in groups:
            ops.linear_fwd_grouped(a, members)
    torch.cuda.synchronize()
    del groups, y
    torch.cuda.synchronize()


if __name__ == "__main__":
    if "--extra" in sys.argv[1:]:
        extra()
    elif "--decode" in sys.argv[1:]:
        decode()
    else:
        main()
