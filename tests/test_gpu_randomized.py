"""Randomized parity sweeps (fixed seeds): many small shapes through every quantizer variant and every GEMM
kernel, against the torch restatement of the reference (bit-exact) and double precision respectively."""
import random

import pytest
import torch

from helpers import rel_fro

pytestmark = pytest.mark.gpu


def _values(rng, rows, cols, kind):
    g = torch.Generator().manual_seed(rng.randrange(1 << 30))
    x = torch.randn(rows, cols, generator=g) * torch.exp(torch.randn(rows, 1, generator=g) * rng.choice([0.1, 1.0, 3.0]))
    if kind == "ties":                                            # multiples of a quarter: quotients land on thresholds
        x = torch.randint(-12, 13, (rows, cols), generator=g).float() * 0.25
    elif kind == "tiny":
        x = x * 1e-20
    elif kind == "huge":
        x = x * 1e20
    if rng.random() < 0.5:
        x.view(-1)[::rng.choice([3, 17, 97])] = 0
    if rng.random() < 0.3:
        x[:, :16] = 0                                             # all-zero blocks
    if rng.random() < 0.3:
        x.view(-1)[::211] *= 50
    return x, g


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_quantizer_variants_bit_exact_on_random_cases(seed):
    """Arithmetic (binary32 on bf16 data, bf16, binary32 on binary32 data) x blocking (rows, columns) x rounding
    (nearest, stochastic with shared draws) x centre (none, column mean) on 150 random shapes per seed."""
    from metis_hip import ops
    from oracle import metis_oracle as O
    rng = random.Random(seed)
    for case in range(150):
        col = rng.random() < 0.4
        rows = rng.choice([1, 2, 5, 16, 31, 33, 64, 100, 255, 256, 300])
        cols = 16 * rng.choice([1, 2, 3, 4, 5, 8, 16, 17, 32, 64])
        if col:
            rows = 16 * rng.choice([1, 2, 3, 4, 5, 8, 16, 17])
        mode = rng.choice([0, 1, 2])                              # 2: binary32 tensor, binary32 arithmetic
        x, g = _values(rng, rows, cols, rng.choice(["n", "n", "ties", "tiny", "huge"]))
        xin = x if mode == 2 else x.bfloat16()
        arith = xin if mode == 1 else xin.float()
        me = arith.mean(dim=0) if rng.random() < 0.3 else None
        res = arith if me is None else arith - me
        noise = None
        if rng.random() < 0.4:
            noise = torch.rand(rows, cols, generator=g)
            noise = noise.bfloat16() if mode == 1 else noise
        p = ops.quantize(xin.cuda(), 1 if mode == 1 else 0, col=col, sr=noise is not None,
                         noise=None if noise is None else noise.cuda(), center=None if me is None else me.cuda())
        codes, scales, unit, _ = (O.nvfp4_pack_col if col else O.nvfp4_pack)(res, noise)
        torch.cuda.synchronize()
        what = f"seed {seed} case {case}: rows={rows} cols={cols} col={col} mode={mode} sr={noise is not None} centre={me is not None}"
        assert torch.equal(p.codes.cpu(), codes), what
        assert torch.equal(p.scales.cpu(), scales), what
        assert float(p.unit.cpu()) == float(unit), what


@pytest.mark.parametrize("seed", [11, 12])
def test_gemm_kernels_on_random_shapes(seed):
    """Skinny, 256-tile, split-K and 128-tile kernels, with and without low-rank term, bf16 / binary32 bias, both
    output dtypes, on 120 random shapes per seed: binary32 output within 1e-5 of double precision."""
    from metis_hip import ops
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for case in range(120):
        M = rng.choice([1, 7, 32, 33, 64, 65, 128, 200, 255, 256, 257, 300, 512, 1024])
        N = 4 * rng.choice([1, 8, 9, 16, 24, 64, 65, 96, 128, 192, 256, 300, 512, 1000])
        K = 32 * rng.choice([1, 2, 3, 4, 6, 8, 16, 17, 32, 64, 100, 128])
        r = rng.choice([0, 0, 32, 64, 96])
        x = torch.randn(M, K, generator=g).bfloat16().cuda()
        w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().cuda()
        t = u = bias = None
        if r:
            t, u = torch.randn(M, r, generator=g).bfloat16().cuda(), torch.randn(N, r, generator=g).bfloat16().cuda()
        kind = rng.choice(["none", "bf16", "f32"])
        if kind != "none":
            bias = torch.randn(N, generator=g).cuda() if kind == "f32" else torch.randn(N, generator=g).bfloat16().cuda()
        px, pw = ops.quantize(x), ops.quantize(w)
        want = ops.dequantize(px, torch.float32).double() @ ops.dequantize(pw, torch.float32).double().T
        if r:
            want = want + t.double() @ u.double().T
        if bias is not None:
            want = want + bias.double()
        what = f"seed {seed} case {case}: M={M} N={N} K={K} r={r} bias={kind}"
        y32 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32)
        assert rel_fro(y32.cpu(), want.cpu()) <= 1e-5, what
        y16 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias)
        assert rel_fro(y16.cpu().float(), y32.cpu().bfloat16().float()) <= 2e-4, what     # the same sums, one bf16 rounding
