"""Pins on the oracle that do not come from the reference: closed forms, library routines,
brute force and invariants.  A plausible slip (dropped term, wrong tie rule, wrong nibble
order, transposed block axis) fails at least one of these.

What pins what
  e4m3 encode/decode (C)      : torch.float8_e4m3fn cast over every byte, every midpoint and its
                                neighbours, and random values (library routine)
  magnitude codes, P32        : nearest point of the E2M1 grid with ties to the even code, exact
                                away from a 2^-20-relative neighbourhood of the ties (closed form)
  magnitude codes, both modes : all 65 536 bf16 patterns x several block scalars, torch
                                restatement vs C restatement (two independent implementations)
  scales / unit               : closed form from the block maxima; invariants listed below
  column packing              : equals row packing of the transpose
  RMSNorm                     : torch.nn.functional.rms_norm and an fp64 evaluation
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import metis_oracle as O
from helpers import rel_fro, synthetic_activation

GRID = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=torch.float64)


def test_e4m3_decode_all_bytes_against_torch():
    b = torch.arange(256, dtype=torch.uint8)
    want = b.view(torch.float8_e4m3fn).float()
    got = torch.tensor([C.e4m3_decode(int(i)) for i in b])
    assert torch.equal(torch.nan_to_num(got, nan=-7.0), torch.nan_to_num(want, nan=-7.0))


def test_e4m3_encode_against_torch_cast():
    vals = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    vals = vals[torch.isfinite(vals) & (vals >= 0)].sort().values
    mids = (vals[:-1] + vals[1:]) / 2
    pts = torch.cat([vals, mids, torch.tensor([448.0, 456.0, 463.9, 464.0, 464.1, 479.9, 480.0, 1e6,
                                               2.0 ** -10, 2.0 ** -10 * 1.0001, 2.0 ** -11, 1e-30, 0.0])])
    near = torch.cat([pts, torch.nextafter(pts, torch.tensor(1e9)), torch.nextafter(pts, torch.tensor(-1.0))])
    g = torch.Generator().manual_seed(5)
    rnd = torch.cat([torch.rand(20000, generator=g) * 500, torch.rand(20000, generator=g) * 0.05,
                     torch.exp(torch.rand(20000, generator=g) * 30 - 25)])
    allv = torch.cat([near, rnd, -near, -rnd]).float()
    want = allv.to(torch.float8_e4m3fn).view(torch.uint8)
    got = torch.tensor([C.e4m3_encode(float(v)) for v in allv], dtype=torch.uint8)
    bad = (got != want).nonzero()
    assert bad.numel() == 0, (allv[bad[:5, 0]], got[bad[:5, 0]], want[bad[:5, 0]])


def test_p32_codes_are_nearest_e2m1_point_ties_to_even():
    """Closed form: code = argmin |x/s - grid| with ties to the even code (P32)."""
    x = synthetic_activation(77, 256, 512).float()
    codes, scales, unit, _ = O.nvfp4_pack(x)
    nib = torch.stack((codes & 0xF, codes >> 4), -1).reshape(x.shape)
    s = O.block_scalars(x).double().repeat_interleave(16, dim=1)
    y = x.double().abs() / s                                   # exact quotient in grid units
    d = (y.unsqueeze(-1) - GRID).abs()
    best = d.argmin(-1)
    dmin = d.min(-1).values
    tie = (d == dmin.unsqueeze(-1)).sum(-1) > 1
    # on a tie the even code wins
    lo = (d == dmin.unsqueeze(-1)).float().argmax(-1)
    even = torch.where(lo % 2 == 0, lo, lo + 1)
    want = torch.where(tie, even, best)
    # the op sequence may deviate only within 2^-20 (relative) of a midpoint
    mid = (GRID[:-1] + GRID[1:]) / 2
    near_mid = ((y.unsqueeze(-1) - mid).abs() <= mid * 2.0 ** -20).any(-1) & ~tie
    ok = ((nib & 7).long() == want) | near_mid
    assert bool(ok.all())
    assert int(tie.sum()) > 0                                  # the data does exercise ties
    assert torch.equal((nib >> 3).bool(), x < 0)               # sign nibble


@pytest.mark.parametrize("mode", [0, 1])
def test_all_bf16_patterns_times_block_scalars_torch_vs_c(mode):
    """Brute force over every bf16 magnitude: two independent restatements must agree."""
    pat = torch.arange(0, 0x7F80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)   # finite, >= 0
    n = (pat.numel() // 15) * 15
    for amax in (6.0, 1.0, 0.75, 0.0283203125, 448.0, 3.0e-5, 2.984375):
        am = torch.tensor(amax).bfloat16()
        body = pat[:n].reshape(-1, 15)
        body = torch.where(body.float() <= am.float(), body, torch.zeros_like(body))
        x = torch.cat([am.expand(body.shape[0], 1), body], dim=1)
        x[1::2] = -x[1::2]
        x = x.reshape(-1, 256).contiguous() if x.numel() % 256 == 0 else x.contiguous()
        xin = x.float() if mode == 0 else x
        codes, scales, unit, _ = O.nvfp4_pack(xin)
        cc, cs, cu, _ = C.nvfp4_pack(x, mode)
        assert torch.equal(codes, cc) and torch.equal(scales, cs) and float(unit) == cu


@pytest.mark.parametrize("mode", [0, 1])
def test_invariants(mode):
    x = synthetic_activation(78, 128, 256)
    x[5, 32:48] = 0
    xin = x.float() if mode == 0 else x
    codes, scales, unit, _ = O.nvfp4_pack(xin)
    nib = torch.stack((codes & 0xF, codes >> 4), -1).reshape(x.shape)
    # unit closed form
    amax = x.float().abs().max()
    if mode == 0:
        assert float(unit) == float((amax / 6 + 1e-9) / 448)
    # the block holding the tensor maximum has scale byte 0x7E (= 448)
    r, c = divmod(int(x.float().abs().argmax()), x.shape[1])
    assert int(scales[r, c // 16]) == 0x7E
    # each block's largest element gets magnitude code 7
    blk = x.float().abs().view(128, -1, 16)
    arg = blk.argmax(-1)
    top = (nib & 7).view(128, -1, 16).gather(-1, arg.unsqueeze(-1)).squeeze(-1)
    nonzero = blk.amax(-1) > 0
    assert bool((top[nonzero] == 7).all())
    # all-zero block: codes 0, scale byte 0, dequant 0
    assert int(codes[5, 16:24].sum()) == 0 and int(scales[5, 2]) == 0
    # odd symmetry
    c2, s2, u2, _ = O.nvfp4_pack(-xin)
    assert torch.equal(s2, scales) and float(u2) == float(unit)
    flip = torch.where(x.view(128, -1) != 0, torch.tensor(0x8, dtype=torch.uint8), torch.tensor(0, dtype=torch.uint8))
    nib2 = torch.stack((c2 & 0xF, c2 >> 4), -1).reshape(x.shape)
    assert torch.equal(nib2, nib ^ flip)
    # nibble order: element 2j low, 2j+1 high
    one = torch.zeros(1, 16).bfloat16()
    one[0, 0], one[0, 1] = 6.0, -3.0
    c1, _, _, _ = O.nvfp4_pack(one.float() if mode == 0 else one)
    assert int(c1[0, 0]) == (0x7 | ((0x8 | 0x5) << 4))


def test_col_pack_is_row_pack_of_transpose():
    x = synthetic_activation(79, 64, 96).float()
    cc, cs, cu, _ = O.nvfp4_pack_col(x)
    rc, rs, ru, _ = O.nvfp4_pack(x.t().contiguous())
    assert cc.shape == (96, 32) and cs.shape == (96, 4)
    assert torch.equal(cc, rc) and torch.equal(cs, rs) and float(cu) == float(ru)
    # tensor scale does not depend on the block axis
    assert float(cu) == float(O.nvfp4_pack(x)[2])


def test_rmsnorm_against_library_and_fp64():
    g = torch.Generator().manual_seed(80)
    x = synthetic_activation(80, 64, 512)
    gamma = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16()
    got = O.rmsnorm(x, gamma, 1e-6)
    lib = torch.nn.functional.rms_norm(x.float(), (512,), gamma.float(), 1e-6)
    xd = x.double()
    f64 = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-6) * gamma.double()
    assert rel_fro(got, f64) < 4e-3 and rel_fro(got, lib) < 4e-3     # two bf16 roundings
    cn, cc, cs, cu = C.rmsnorm_nvfp4(x, gamma, 1e-6, 0)
    assert rel_fro(cn, got) < 2e-3
    # codes of the C pipeline are exactly the oracle's codes of the C pipeline's own normed tensor
    oc, os_, ou, _ = O.nvfp4_pack(cn.float())
    assert torch.equal(oc, cc) and torch.equal(os_, cs) and float(ou) == cu


def test_value_error_on_non_divisible_last_dim():
    with pytest.raises(ValueError):
        O.nvfp4_qdq(torch.zeros(4, 24))


def test_rotation_of_the_nv_recipe_is_summed_in_the_order_of_the_reference_matrix_product():
    """The NV recipe rotates a tile of 16 with a binary32 matrix product (src/Metis/Metis/bitlinear.py:195-202, torch.mm on
    the CPU).  For the weight gradient's second operand -- the already quantized input, rotated and quantized AGAIN
    (495-501) -- the summation order of those 16-term sums decides codes: rotated values of quantized data sit on FP4
    rounding boundaries far more often than ordinary data.  On the reference's own vectors: adding the terms in the order
    k = 0 .. 15 (what the kernels do) reproduces the reference's operand bit for bit, while a butterfly network and a
    double-precision sum rounded once each leave about 5 % of its elements different, 2e-2 in the Frobenius norm."""
    import os
    import numpy as np
    from helpers import rel_fro, t
    from oracle import metis_oracle as O
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    g = dict(np.load(os.path.join(here, "metis_reference_hadamard_wide.npz")))
    sign = t(dict(np.load(os.path.join(here, "metis_reference_hadamard.npz")))["had_sign16"]).float()
    H = torch.tensor([[1.0]])
    while H.shape[0] < 16:
        H = torch.cat([torch.cat([H, H], 1), torch.cat([H, -H], 1)], 0)
    xq = t(g["hw_p32_xq"]).float().reshape(-1, 16)
    want = t(g["hw_p32_wgrad_x"]).float().reshape(-1, 16)

    def sequential(v):
        acc = torch.zeros_like(v)
        for k in range(16):
            acc = acc + v[:, k:k + 1] * H[k:k + 1, :]
        return acc

    def butterfly(v):
        w = v.clone()
        h = 1
        while h < 16:
            for j in range(16):
                if (j & h) == 0:
                    a, b = w[:, j].clone(), w[:, j + h].clone()
                    w[:, j], w[:, j + h] = a + b, a - b
            h <<= 1
        return w

    def operand(product):
        rotated = product(xq * sign).reshape(-1, 96)
        q = O.nvfp4_qdq(rotated).reshape(-1, 16)
        return sequential(q) * (1.0 / 16) * sign

    assert torch.equal(operand(sequential), want)
    for other in (butterfly, lambda v: (v.double() @ H.double()).float()):
        got = operand(other)
        assert 5e-3 < rel_fro(got, want) < 5e-2 and 0.9 < float((got == want).float().mean()) < 0.99
