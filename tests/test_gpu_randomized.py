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


@pytest.mark.parametrize("seed", [21, 22])
def test_pipelined_gemm_on_random_shapes(seed):
    """The pipelined GEMM on tiled expansions against the packed-operand kernels on the same packed tensors (the same
    products, binary32 sums in another order): any row and column count (partial tiles, fewer rows than a tile), any
    contraction that 32 divides, with and without low-rank term, bias kinds, both output dtypes, split and unsplit;
    and in bf16 arithmetic against the reference's rounding sequence evaluated in torch."""
    from metis_hip import ops
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for case in range(60):
        M = rng.choice([1, 16, 33, 255, 256, 257, 300, 512, 700, 1024])
        N = 4 * rng.choice([1, 9, 64, 65, 96, 128, 200, 256, 300])
        K = 32 * rng.choice([1, 2, 3, 4, 8, 17, 32, 64, 100])
        r = rng.choice([0, 0, 32, 64])
        x = torch.randn(M, K, generator=g).bfloat16().cuda()
        w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().cuda()
        t = u = bias = None
        if r:
            t, u = torch.randn(M, r, generator=g).bfloat16().cuda(), torch.randn(N, r, generator=g).bfloat16().cuda()
        kind = rng.choice(["none", "bf16", "f32"])
        if kind != "none":
            bias = torch.randn(N, generator=g).cuda() if kind == "f32" else torch.randn(N, generator=g).bfloat16().cuda()
        split = rng.random() < 0.5
        what = f"seed {seed} case {case}: M={M} N={N} K={K} r={r} bias={kind} split={split}"
        px, pw = ops.quantize(x), ops.quantize(w)
        want = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32, tiled=False, split_k=False)
        got = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, out_dtype=torch.float32, tiled=True, split_k=split)
        assert rel_fro(got.cpu(), want.cpu()) <= 1e-6, what
        got16 = ops.linear_fwd(px, pw, t=t, u=u, bias=bias, tiled=True, split_k=split)
        assert rel_fro(got16.cpu().float(), want.cpu().bfloat16().float()) <= 2e-4, what
        if kind != "f32":
            # bf16 arithmetic: bf16 dequantized operands, product rounded to bf16, bias added in bf16, low-rank term, rounding
            qx, qw = ops.quantize(x, 1), ops.quantize(w, 1)
            ref = (qx.dequantize(torch.bfloat16).double() @ qw.dequantize(torch.bfloat16).double().T).float().bfloat16()
            if bias is not None:
                ref = ref + bias
            if r:
                ref = (ref.float() + (t.double() @ u.double().T).float()).bfloat16()
            faithful = ops.linear_fwd(qx, qw, t=t, u=u, bias=bias, tiled=True, split_k=split, reference_rounding=True)
            assert rel_fro(faithful.cpu().float(), ref.cpu().float()) <= 3e-4, what      # single bf16 roundings of sums taken in another order


@pytest.mark.parametrize("seed", [31])
def test_rotated_and_transposed_tiled_operands_on_random_shapes(seed):
    """NV-recipe operands: rotation + quantizer in one pass equals the two steps bit for bit, and GEMMs on the tiled
    operands (plain, rotated back, transposed, transposed and rotated back) equal the products of the dequantized
    tensors, over random shapes incl. ragged row tiles."""
    from metis_hip import LinearLowbitFunction as F, ops
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    mask = F._hadamard_mask()
    for case in range(30):
        L = 32 * rng.choice([1, 2, 5, 8, 9, 16])
        N = 16 * rng.choice([2, 3, 4, 6, 8, 13, 16])
        K = 32 * rng.choice([1, 2, 3, 5, 8, 12])
        mode = rng.choice([0, 1])
        what = f"seed {seed} case {case}: L={L} N={N} K={K} mode={mode}"
        a = torch.randn(L, K, generator=g).bfloat16().cuda()
        dy = (torch.randn(L, N, generator=g) * 1e-2).bfloat16().cuda()
        pa = ops.quantize_rht(a, mode, mask)
        two = ops.quantize(ops.hadamard16(a.float() if mode == 0 else a, mask), mode)
        assert torch.equal(pa.codes, two.codes) and torch.equal(pa.scales, two.scales) and torch.equal(pa.unit, two.unit), what
        pdy = ops.quantize_rht(dy, mode, mask) if rng.random() < 0.7 else ops.quantize(dy, mode)
        dt = torch.float32 if mode == 0 else torch.bfloat16
        da, ddy = pa.dequantize(dt).double(), pdy.dequantize(dt).double()
        tol = 2e-4 if mode == 0 else 3e-3
        # contraction over tokens: dY~^T [N, L] . X~^T [K, L]^T
        gw = ops.gemm_tiled(ops.expand_tiled_transposed(pdy, mode=mode), pdy.unit, ops.expand_tiled_transposed(pa, mode=mode), pa.unit,
                            N, K, L, mode=mode, out_dtype=torch.float32)
        assert rel_fro(gw.double().cpu(), (ddy.T @ da).cpu()) <= tol, what
        if N % 32 == 0:
            # contraction over N: dY~ [L, N] . W~^T [K, N]^T with W~ a rotated weight [N, K]
            w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().cuda()
            pw = ops.quantize_rht(w, mode, mask)
            gx = ops.gemm_tiled(ops.expand_tiled(pdy, cache=False, mode=mode), pdy.unit, ops.expand_tiled_transposed(pw, mode=mode), pw.unit,
                                L, K, N, mode=mode, out_dtype=torch.float32)
            assert rel_fro(gx.double().cpu(), (ddy @ pw.dequantize(dt).double()).cpu()) <= tol, what


@pytest.mark.parametrize("seed", [41])
def test_rank_r_kernels_and_dense_operands_on_random_shapes(seed):
    """Row projection x V^T (* s), token contractions a^T b, and a dense tensor as a tiled operand, on random shapes
    with ragged row counts and column counts that are not multiples of the tile."""
    from metis_hip import ops
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for case in range(40):
        M = rng.choice([256, 257, 300, 511, 1000, 2048])
        K = 64 * rng.choice([1, 2, 3, 4, 7, 16, 33])
        R = rng.choice([32, 64, 128])
        what = f"seed {seed} case {case}: M={M} K={K} R={R}"
        x = torch.randn(M, K, generator=g).bfloat16().cuda()
        v = (torch.randn(R, K, generator=g) / K ** 0.5).bfloat16().cuda()
        s = (torch.rand(R, generator=g) + 0.5).bfloat16().cuda()
        xv, t = ops.lowrank_project(x, v, s)
        want = x.double() @ v.double().T
        d = (xv.double() - want).abs()
        assert bool((d <= want.abs() * 2.0 ** -8 + 1e-6 * float(want.abs().max())).all()), what
        assert torch.equal(t, xv * s), what
        C = 8 * rng.choice([4, 8, 9, 31, 64, 100])
        a = torch.randn(M, C, generator=g).bfloat16().cuda()
        transpose = rng.random() < 0.5
        got = ops.lowrank_contract_tokens(a, t, out_dtype=torch.float32, transpose=transpose)
        want2 = a.double().T @ t.double()
        want2 = want2.T if transpose else want2
        assert rel_fro(got.double().cpu(), want2.cpu()) <= 1e-5, what
        # a dense bf16 tensor as one operand of the tiled GEMM (bf16 arithmetic): x as activations against dense v
        if K % 32 == 0:
            qx = ops.quantize(x, 1)
            y = ops.gemm_tiled(ops.expand_tiled(qx, cache=False, mode=1), qx.unit, ops.dense_expand_tiled(v, 1), qx.unit, M, R, K, mode=1,
                               out_dtype=torch.bfloat16)
            ref = (qx.dequantize(torch.bfloat16).double() @ v.double().T).float().bfloat16()
            assert rel_fro(y.float().cpu(), ref.float().cpu()) <= 3e-4, what


@pytest.mark.parametrize("seed", [51, 52])
def test_one_pass_kernels_on_random_cases(seed):
    """The two kernels that serve two consumers from one pass, on 40 random shapes and value ranges per seed (zeros,
    all-zero blocks, outliers, tiny and huge magnitudes, exact ties): both stochastic packings of a tensor against the row
    and the column call (same seed and offsets: same bytes), and the quantizer inside the rank-r projection's pass against
    the quantizer's own kernels (same bytes) and double precision (the projection)."""
    from metis_hip import ops
    rng = random.Random(seed)
    for case in range(40):
        kind = rng.choice(["plain", "plain", "ties", "tiny", "huge"])
        mode = rng.choice([0, 1])
        # both packings: every shape with both dimensions multiples of 16
        rows, cols = 16 * rng.randint(1, 40), 16 * rng.randint(1, 40)
        x, _ = _values(rng, rows, cols, kind)
        wide = mode == 0 and rng.random() < 0.3
        xin = (x if wide else x.bfloat16()).cuda()
        sd, o1, o2 = rng.randrange(1 << 62), rng.randrange(1 << 40), rng.randrange(1 << 40)
        pr, pc = ops.quantize_both_sr(xin, mode, seed=sd, offset_row=o1, offset_col=o2)
        wr = ops.quantize(xin, mode, sr=True, seed=sd, offset=o1)
        wc = ops.quantize(xin, mode, col=True, sr=True, seed=sd, offset=o2)
        torch.cuda.synchronize()
        what = f"seed {seed} case {case}: {rows}x{cols} {kind} mode {mode} wide {wide}"
        assert torch.equal(pr.codes, wr.codes) and torch.equal(pr.scales, wr.scales) and torch.equal(pr.unit, wr.unit), what
        assert torch.equal(pc.codes, wc.codes) and torch.equal(pc.scales, wc.scales) and torch.equal(pc.unit, wc.unit), what
        # quantizer + projection: 256 rows and more, K a multiple of 64, rank 32 or 64
        M, K, R = rng.randint(256, 700), 64 * rng.randint(1, 24), rng.choice([32, 64])
        a, g = _values(rng, M, K, kind)
        a = a.bfloat16().cuda()
        v = (torch.randn(R, K, generator=g) / K ** 0.5).bfloat16().cuda()
        s = (torch.rand(R, generator=g) + 0.5).bfloat16().cuda()
        p, xv, t = ops.quantize_project(a, v, s, mode)
        want = ops.quantize(a, mode)
        torch.cuda.synchronize()
        what = f"seed {seed} case {case}: {M}x{K} r{R} {kind} mode {mode}"
        assert torch.equal(p.codes, want.codes) and torch.equal(p.scales, want.scales) and torch.equal(p.unit, want.unit), what
        ref = a.double() @ v.double().T
        if kind != "huge":                                        # bf16 sums of 1e20-sized terms overflow nothing, but the bound is relative anyway
            assert rel_fro(xv.float().cpu(), ref.cpu()) <= 4e-3, what
        assert torch.equal(t, (xv.float() * s.float()).bfloat16()), what
