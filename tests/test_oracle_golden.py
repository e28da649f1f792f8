"""The oracle (torch restatement and C restatement) against vectors the reference itself produced.

Fixtures: tests/golden/metis_reference_golden.npz, written by tests/golden/make_golden.py.
Everything here is bit-exact (atol = rtol = 0).
"""
import pytest
import torch

from oracle import c_oracle as C
from oracle import metis_oracle as O
from helpers import same_bits, t

MODES = [("p32", 0), ("pb16", 1)]


def _inp(x_bf16, tag):
    return x_bf16.float() if tag == "p32" else x_bf16


@pytest.mark.parametrize("tag,mode", MODES)
@pytest.mark.parametrize("case", ["rne", "rne3d", "rnew"])
def test_fused_qdq_matches_reference(golden, case, tag, mode):
    x = t(golden[f"{case}_x"])
    want = t(golden[f"{case}_qdq_{tag}"])
    got = O.nvfp4_qdq(_inp(x, tag))
    assert same_bits(got, want)
    # packed integers -> dequant reproduces the reference output too
    codes, scales, unit, ncl = O.nvfp4_pack(_inp(x, tag))
    assert ncl == 0
    assert same_bits(O.nvfp4_unpack_dequant(codes, scales, unit, want.dtype).reshape(want.shape), want)
    # C restatement: same integers, same dequantized values
    c_codes, c_scales, c_unit, _ = C.nvfp4_pack(x.reshape(-1, x.shape[-1]).contiguous(), mode)
    assert torch.equal(c_codes, codes) and torch.equal(c_scales, scales) and c_unit == float(unit)
    ob, of = C.nvfp4_dequant(c_codes, c_scales, c_unit, mode)
    assert same_bits((of if mode == 0 else ob).reshape(want.shape), want)


@pytest.mark.parametrize("tag,mode", MODES)
def test_three_call_form_matches_reference(golden, tag, mode):
    x = _inp(t(golden["rne_x"]), tag)
    s = O.get_scalar(x)
    assert same_bits(s, t(golden[f"rne_scalar_{tag}"]))
    xq = O.quant(x, s)
    assert same_bits(xq, t(golden[f"rne_quant_{tag}"]))
    s_arg = s.clone()
    out = O.rquant(xq, s_arg)
    assert same_bits(out, t(golden[f"rne_rquant_{tag}"]))
    assert same_bits(s_arg, t(golden[f"rne_scalar_after_rquant_{tag}"]))   # in-place side effect
    assert same_bits(out, t(golden[f"rne_qdq_{tag}"]))                     # reference test 17-26


@pytest.mark.parametrize("tag,mode", MODES)
def test_stochastic_rounding_with_shared_noise_matches_reference(golden, tag, mode):
    x_b = t(golden["sr_x"])
    x = _inp(x_b, tag)
    u = t(golden[f"sr_noise_{tag}"])
    s = O.get_scalar(x)
    xq = O.quant(x, s, noise=u)
    assert same_bits(xq, t(golden[f"sr_quant_{tag}"]))
    want = t(golden[f"sr_rquant_{tag}"])
    assert same_bits(O.rquant(xq, s.clone()), want)
    assert same_bits(O.nvfp4_qdq(x, noise=u), want)
    # packed form: identical wherever the reference stayed on the E2M1 grid (r <= 7)
    codes, scales, unit, ncl = O.nvfp4_pack(x, noise=u)
    deq = O.nvfp4_unpack_dequant(codes, scales, unit, want.dtype)
    off_grid = (t(golden[f"sr_quant_{tag}"]).abs() > 6)
    assert int(off_grid.sum()) == ncl
    assert torch.equal(deq[~off_grid], want[~off_grid])
    c_codes, c_scales, c_unit, c_ncl = C.nvfp4_pack(x_b.contiguous(), mode, u.contiguous())
    assert torch.equal(c_codes, codes) and torch.equal(c_scales, scales) and c_ncl == ncl


def test_linear_forward_backward_matches_reference(golden):
    """bitlinear.py:407-513 in fp32: RNE on x and w forward, SR on dY backward (shared noise)."""
    x, w, b, dy = (t(golden[k]) for k in ("lin_x", "lin_w", "lin_b", "lin_dy"))
    xq, wq = O.nvfp4_qdq(x), O.nvfp4_qdq(w)
    y = O.linear_forward(xq, wq, b)
    assert same_bits(y, t(golden["lin_y"]))
    dyq = O.nvfp4_qdq(dy, noise=t(golden["lin_noise_dy"]))
    gx, gw = O.linear_backward(dyq, xq, wq)
    assert same_bits(gx, t(golden["lin_gx"]))
    assert same_bits(gw, t(golden["lin_gw"]))
    assert same_bits(dy.sum(dim=(0, 1)), t(golden["lin_gb"]))


def test_bitlinear_forward_matches_reference(golden):
    """bitlinear.py:736-769 with quantized X and V in the rank-r branch (current reference file)."""
    x, b = t(golden["lin_x"]), t(golden["lin_b"])
    v, u, s, res = (t(golden[k]) for k in ("bl_v", "bl_u", "bl_s", "bl_res"))
    xq = O.nvfp4_qdq(x)
    y = torch.matmul(xq, O.nvfp4_qdq(v).T)
    y = torch.mul(s, y)
    y = torch.matmul(y, u.T)
    y = y + O.linear_forward(xq, O.nvfp4_qdq(res), b)
    assert same_bits(y, t(golden["bl_y"]))
    # and the oracle's own composite, the function the GPU tests compare against: the same sum, rounded to bf16 once
    got = O.metis_forward(x, v, s, u, res, b, p32=True, quantized_lowrank=True)
    assert got.dtype == torch.bfloat16 and same_bits(got, t(golden["bl_y"]).bfloat16())


def test_c_oracle_binary32_input_mode_matches_torch_restatement():
    """Mode 2 of the C oracle (binary32 arithmetic on values that are not bf16 values) against the torch
    restatement, which the reference's golden vectors pin; on bf16-valued data it equals mode 0."""
    import torch
    from oracle import c_oracle as C, metis_oracle as O
    g = torch.Generator().manual_seed(5)
    x = torch.randn(64, 256, generator=g) * torch.exp(torch.randn(64, 1, generator=g))
    x.view(-1)[::53] = 0
    u = torch.rand(64, 256, generator=g)
    for noise in (None, u):
        codes, scales, unit, _ = O.nvfp4_pack(x, noise)
        cc, cs, cu, _ = C.nvfp4_pack(x, 2, noise)
        assert torch.equal(cc, codes) and torch.equal(cs, scales) and cu == float(unit)
    xb = x.bfloat16()
    a, b = C.nvfp4_pack(xb, 0), C.nvfp4_pack(xb.float(), 2)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) and a[2] == b[2]


@pytest.mark.parametrize("tag,dt", [("p32", "float32"), ("pb16", "bfloat16")])
def test_mean_mode_formula_matches_reference(tag, dt):
    """mean + QDQ(x - mean) with the oracle's QDQ reproduces the reference's svd_quant(metis_mode="mean") output bit
    for bit, for a prefill call and for the single-token decode call that updates the weighted running mean."""
    import os
    import numpy as np
    import torch
    from helpers import same_bits, t
    from oracle import metis_oracle as O
    g = dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "metis_reference_mean_mode.npz")))
    D = getattr(torch, dt)
    x = t(g["mean_x"]).to(D).reshape(-1, 64)
    me = x.mean(dim=0, keepdim=True)
    assert same_bits(me, t(g[f"mean_cache_{tag}"]))
    assert same_bits((me + O.nvfp4_qdq(x - me)).reshape(2, 24, 64), t(g[f"mean_out_{tag}"]))
    step = t(g["mean_step"]).to(D).reshape(-1, 64)
    count = x.shape[0]
    me2 = (me * count + step.mean(dim=0, keepdim=True) * step.shape[0]) / (count + step.shape[0])
    assert int(g[f"mean_step_count_{tag}"][0]) == count + step.shape[0]
    assert same_bits(me2, t(g[f"mean_step_cache_{tag}"]))
    assert same_bits((me2 + O.nvfp4_qdq(step - me2)).reshape(4, 1, 64), t(g[f"mean_step_out_{tag}"]))


@pytest.mark.parametrize("tag,dt", [("f32", "float32"), ("bf16", "bfloat16")])
def test_svd_mode_recomposition_matches_reference(tag, dt):
    """svd_quant(metis_mode="svd") of the reference (bitlinear.py:243-309), restated from the point where the factors of
    its torch.svd_lowrank call exist (they are recorded in the fixture).  The restatement fixes the order in which ker's
    rank products are added (k ascending, one fused multiply-add each); on the reference's vectors that order
    reproduces its library product bit for bit -- ker and the final tensor -- and with the reference's own ker handed
    in, everything behind it (residual, QDQ, sum) is bit-exact by construction of the same op sequence.  A transposed
    factor, a dropped diag(s) or a quantizer applied to the wrong operand changes every element."""
    import os
    import numpy as np
    g = dict(np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "metis_reference_svd_mode.npz")))
    D = getattr(torch, dt)
    x = t(g[f"svd_{tag}_x"]).to(D).reshape(-1, 256)
    u, s, v = (t(g[f"svd_{tag}_{n}"]) for n in "usv")
    ug, sg, vg = u.to(D), s.to(D), v.to(D).T.contiguous()
    ker, res, y = O.svd_mode_recompose(x, ug.clone(), sg, vg.clone())
    assert same_bits(ker, t(g[f"svd_{tag}_ker"]))
    assert same_bits(y.reshape(2, 64, 256), t(g[f"svd_{tag}_y"]))
    _, _, y2 = O.svd_mode_recompose(x, ug.clone(), sg, vg.clone(), ker=t(g[f"svd_{tag}_ker"]))
    assert same_bits(y2.reshape(2, 64, 256), t(g[f"svd_{tag}_y"]))
    # the fixed order is one valid evaluation of the product: against torch's own matmul it agrees to rounding
    uq, vq = t(g[f"svd_{tag}_uq"]), t(g[f"svd_{tag}_vq"])
    lib = (uq @ torch.diag(sg) @ vq).float()
    assert float((ker.float() - lib).abs().max()) <= (1e-5 if dt == "float32" else 2 ** -7) * float(lib.abs().max())
    # and a wrong order of factors is nowhere near
    assert not same_bits(C.lowrank_product((uq.float() * sg.float()).contiguous(), vq.float().flip(0).contiguous()).to(D), ker)
