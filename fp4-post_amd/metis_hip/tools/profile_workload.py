"""Profiling workload: a few launches of each hot kernel at the benchmark shapes, plus a plain
device-to-device copy of known size that calibrates the FETCH_SIZE / WRITE_SIZE counters.

    rocprofv3 --kernel-trace --stats -- python3 fp4-post_amd/metis_hip/tools/profile_workload.py
    rocprofv3 --pmc FETCH_SIZE       -- python3 fp4-post_amd/metis_hip/tools/profile_workload.py
    rocprofv3 --pmc WRITE_SIZE       -- python3 fp4-post_amd/metis_hip/tools/profile_workload.py
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
    y = torch.empty_like(x)
    pw = ops.quantize(w)
    for _ in range(reps):
        y.copy_(x)                                                      # calibration: 64 MiB read, 64 MiB written
        px = ops.quantize(x)
        ops.rmsnorm_quantize(h, gamma, 1e-6)
        ops.linear_fwd(px, pw, t=t, u=u)
    torch.cuda.synchronize()


if __name__ == "__main__":
    main()
