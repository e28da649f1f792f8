"""The "svd" mode of the activation decomposition on the kernels (reference src/Metis/Metis/bitlinear.py:243-309).

With the factors of the rank-r approximation given, the reference computes ker = U diag(s) V, QDQ(x - ker) and their sum.
`metis_nvfp4_quant_lowrank_residual` forms ker in registers, encodes the residual there and writes the packed residual
and (optionally) the dense sum.  Bar: bit for bit -- against the reference's own vectors (tests/golden, factors recorded
from its torch.svd_lowrank call) and against the op-for-op oracle on shapes the fixture does not hold (ragged tiles,
ranks 16..80, binary32 tensors that are not bf16 values).
"""
import os

import numpy as np
import pytest
import torch

from helpers import synthetic_activation

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "metis_reference_svd_mode.npz")


def _bf(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def _quantized_factors(ug, sg, vg):
    """U and V through the three calls (reference 283-293), then U diag(s) as the elementwise product it is."""
    from metis_hip.quant import Cast2NVFp4e2m1BlockNOSR as Q
    s_u, s_v = Q.get_scalar(ug), Q.get_scalar(vg)
    ugq = Q.rquant(Q.quant(ug, s_u), s_u)
    vgq = Q.rquant(Q.quant(vg, s_v), s_v)
    return ugq * sg, vgq


@pytest.mark.parametrize("tag,dt", [("f32", torch.float32), ("bf16", torch.bfloat16)])
def test_reference_vectors_bit_for_bit(tag, dt):
    from metis_hip import ops
    z = np.load(GOLD)
    D = 256
    x = _bf(z[f"svd_{tag}_x"]).reshape(-1, D)
    u, s, v = (torch.from_numpy(z[f"svd_{tag}_{n}"]) for n in "usv")
    want = (torch.from_numpy(z[f"svd_{tag}_y"]) if dt == torch.float32 else _bf(z[f"svd_{tag}_y"])).reshape(-1, D)
    us, vt = _quantized_factors(u.to(dt).cuda(), s.to(dt).cuda(), v.to(dt).T.contiguous().cuda())
    mode = ops.MODE_P32 if dt == torch.float32 else ops.MODE_PB16
    inputs = [x.cuda()] + ([x.float().cuda()] if dt == torch.float32 else [])      # a bf16 tensor widened in registers, or binary32
    for xin in inputs:
        packed, dense = ops.quantize_lowrank_residual(xin, us, vt, mode, dense=True)
        torch.cuda.synchronize()
        assert dense.dtype == dt and torch.equal(dense.cpu(), want)
        # the packed residual alone: ker + dequantized residual is the same tensor
        ker = torch.from_numpy(z[f"svd_{tag}_ker"]) if dt == torch.float32 else _bf(z[f"svd_{tag}_ker"])
        assert torch.equal(ker + ops.dequantize(packed, dt).cpu(), want)
        only, none = ops.quantize_lowrank_residual(xin, us, vt, mode)
        assert none is None and torch.equal(only.codes, packed.codes) and torch.equal(only.scales, packed.scales)


@pytest.mark.parametrize("rows,cols,r", [(64, 256, 16), (100, 272, 32), (1, 16, 16), (257, 3584, 64), (130, 528, 80), (63, 4096, 48)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_against_the_oracle_on_ragged_shapes(rows, cols, r, dt):
    from metis_hip import ops
    from oracle import metis_oracle as O
    g = torch.Generator().manual_seed(rows * 7 + cols + r)
    x = synthetic_activation(500 + rows, rows, cols)
    x_dev = x.cuda()                                                       # bf16 tensor: widened in registers under binary32 arithmetic
    if dt == torch.float32 and rows % 2:
        x = x.float() + 1e-3 * torch.randn(rows, cols, generator=g)       # binary32 values that are not bf16 values
        x_dev = x.cuda()
    else:
        x = x.to(dt)
    ug = (torch.randn(rows, r, generator=g) / r ** 0.5).to(dt)
    sg = (torch.rand(r, generator=g) * 30 + 0.5).sort(descending=True).values.to(dt)
    vg = (torch.randn(r, cols, generator=g) / cols ** 0.5).to(dt)
    ker, res, want = O.svd_mode_recompose(x.clone(), ug.clone(), sg, vg.clone())
    us, vt = _quantized_factors(ug.cuda(), sg.cuda(), vg.cuda())
    mode = ops.MODE_P32 if dt == torch.float32 else ops.MODE_PB16
    packed, dense = ops.quantize_lowrank_residual(x_dev, us, vt, mode, dense=True)
    torch.cuda.synchronize()
    assert torch.equal(ops.dequantize(packed, dt).cpu(), res)
    assert torch.equal(dense.cpu(), want)
    codes, scales, unit, _ = O.nvfp4_pack(x - ker)
    assert torch.equal(packed.codes.cpu(), codes) and torch.equal(packed.scales.cpu(), scales)
    assert float(packed.unit.cpu()) == float(unit)


def test_shapes_the_kernel_does_not_take_are_refused():
    from metis_hip import ops
    x = torch.zeros(32, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        ops.quantize_lowrank_residual(x, torch.zeros(32, 8, device="cuda"), torch.zeros(8, 64, device="cuda"))
    with pytest.raises(ValueError):
        ops.quantize_lowrank_residual(x, torch.zeros(32, 16, device="cuda"), torch.zeros(16, 48, device="cuda"))
    with pytest.raises(ValueError):
        ops.quantize_lowrank_residual(x, torch.zeros(32, 16, dtype=torch.bfloat16, device="cuda"),
                                      torch.zeros(16, 64, dtype=torch.bfloat16, device="cuda"), ops.MODE_P32)
    empty, _ = ops.quantize_lowrank_residual(x[:0], torch.zeros(0, 16, device="cuda"), torch.zeros(16, 64, device="cuda"))
    assert empty.codes.numel() == 0


@pytest.fixture
def svd_mode():
    from metis_hip import LinearLowbitFunction as F, quant_func
    keep = {k: getattr(F, k) for k in ("q_forward_input", "q_forward_weight", "q_backward_input", "q_backward_weight",
                                       "q_backward_outputgrad", "enable_activation_svd", "enable_backward_svd", "enable_nv_recipe",
                                       "compute_dtype", "metis_mode", "activation_lowrank_svd", "activation_lowrank_niter",
                                       "activation_broadcast_dim", "tp_simulate")}
    F.q_forward_input = F.q_forward_weight = quant_func["nvfp4e2m1bnosr"]
    F.q_backward_input = F.q_backward_weight = F.q_backward_outputgrad = quant_func["nvfp4e2m1b"]
    F.enable_activation_svd, F.enable_backward_svd, F.enable_nv_recipe = True, False, False
    F.metis_mode, F.activation_lowrank_svd, F.activation_lowrank_niter = "svd", 32, 2
    F.activation_broadcast_dim, F.tp_simulate, F.compute_dtype = -1, False, torch.float32
    yield F
    for k, v in keep.items():
        setattr(F, k, v)


def _lowrank_plus_noise(seed, rows, cols, rank=8):
    g = torch.Generator().manual_seed(seed)
    a = torch.linalg.qr(torch.randn(rows, rank, generator=g))[0]
    b = torch.linalg.qr(torch.randn(cols, rank, generator=g))[0]
    return ((a * (30.0 * 0.8 ** torch.arange(rank))) @ b.T + 0.05 * torch.randn(rows, cols, generator=g)).bfloat16()


@pytest.mark.parametrize("compute", [torch.float32, torch.bfloat16])
def test_svd_quant_runs_on_the_fused_kernel_and_agrees_with_the_op_by_op_evaluation(svd_mode, compute, monkeypatch):
    """LinearLowbitFunction.svd_quant (reference 213-369) on a device tensor: one fused launch for ker, the residual's
    codes and the sum.  The same call with the kernel switched off evaluates the reference's expressions with torch
    operators from the same factors (same random stream); the two differ only through the order in which ker's rank
    products are added (a library product there): last-bit differences of ker, and a different code in the few
    elements whose residual sat on a rounding boundary."""
    from metis_hip import ops
    F = svd_mode
    q = F.q_forward_input
    x = _lowrank_plus_noise(3, 384, 512).to(compute).reshape(2, 192, 512).cuda()
    calls = []
    real = ops.quantize_lowrank_residual
    monkeypatch.setattr(ops, "quantize_lowrank_residual", lambda *a, **k: calls.append(a[0].shape) or real(*a, **k))
    torch.manual_seed(77)
    got = F.svd_quant(x, q, rank=32, niter=2, metis_mode="svd")
    assert calls == [(384, 512)] and got.shape == x.shape and got.dtype == compute
    monkeypatch.setattr(F, "_svd_mode_on_kernels", staticmethod(lambda *a: False))
    torch.manual_seed(77)
    want = F.svd_quant(x, q, rank=32, niter=2, metis_mode="svd")
    assert len(calls) == 1
    # last-bit differences of ker are everywhere (binary32) or rare (bf16); a different code is a visible step
    step = (got.float() - want.float()).abs() > (1e-4 if compute == torch.float32 else 2e-2) * want.float().abs().max()
    assert float(step.float().mean()) < 0.02, float(step.float().mean())
    assert float((got.float() - want.float()).norm() / want.float().norm()) < 2e-3
    # the simulated tensor-parallel split treats every chunk of columns on its own: four launches
    monkeypatch.undo()
    monkeypatch.setattr(ops, "quantize_lowrank_residual", lambda *a, **k: calls.append(a[0].shape) or real(*a, **k))
    torch.manual_seed(78)
    out = F.svd_quant(x, q, rank=16, niter=1, tp_simulate=True, tp_parts=4, metis_mode="svd")
    assert calls[1:] == [(384, 128)] * 4 and out.shape == x.shape


@pytest.mark.parametrize("compute", [torch.float32, torch.bfloat16])
def test_linear_lowbit_in_svd_mode(svd_mode, compute, monkeypatch):
    """A LinearLowbit layer under metis_mode="svd": the forward multiplies the packed residual and the packed V with the
    packed weight and adds the rank-r correction; the result agrees with the reference's formula
    (ker + QDQ(x - ker)) QDQ(W)^T evaluated with torch operators from the same factors.  With autograd the dense
    activation is kept and the backward pass multiplies with it, as the reference's does (443-513)."""
    from types import SimpleNamespace
    from metis_hip import LinearLowbit, ops
    from metis_hip.quant import _NVFP4Base
    F = svd_mode
    F.compute_dtype = compute
    K, N, L = 512, 192, 320
    layer = LinearLowbit(K, N, bias=True, args=SimpleNamespace(device="cuda", cache_quantized_weight=True),
                         storage_dtype=torch.bfloat16, compute_dtype=compute)
    x = _lowrank_plus_noise(5, L, K).cuda()
    seen = []
    real = ops.quantize_lowrank_residual
    monkeypatch.setattr(ops, "quantize_lowrank_residual", lambda *a, **k: seen.append(k.get("dense")) or real(*a, **k))
    with torch.no_grad():
        torch.manual_seed(5)
        y = layer(x)
    assert seen == [False] and y.dtype == compute and y.shape == (L, N)

    def generic(xin):
        torch.manual_seed(5)
        xq = F.svd_quant(xin.to(compute), F.q_forward_input, rank=32, niter=2, metis_mode="svd")
        wq = F.q_forward_weight.quantize_dequantize(layer.weight.detach().to(compute))
        return xq, wq

    monkeypatch.setattr(F, "_svd_mode_on_kernels", staticmethod(lambda *a: False))
    xq, wq = generic(x)
    want = (xq.double() @ wq.double().T + layer.bias.detach().double())
    monkeypatch.undo()
    assert float((y.double() - want).norm() / want.norm()) < (2e-3 if compute == torch.float32 else 6e-3)
    # training: dense activation kept, gradients of the reference's formula
    seen.clear()
    monkeypatch.setattr(ops, "quantize_lowrank_residual", lambda *a, **k: seen.append(k.get("dense")) or real(*a, **k))
    xr = x.clone().requires_grad_(True)
    torch.manual_seed(5)
    _NVFP4Base.sr_offset = 0
    y2 = layer(xr)
    dy = torch.randn(L, N, generator=torch.Generator().manual_seed(6)).to(compute).cuda() * 1e-2
    y2.backward(dy)
    assert seen == [True]
    _NVFP4Base.sr_offset = 0
    dyq = F._quantize_wgrad_operand(dy, F.q_backward_outputgrad).reshape(L, N)
    gw = dyq.double().T @ xq.double()
    gx = dyq.double() @ wq.double()
    assert float((layer.weight.grad.double() - gw).norm() / gw.norm()) < 1e-2
    assert float((xr.grad.double() - gx).norm() / gx.norm()) < 1e-2
    assert float((layer.bias.grad.double() - dy.double().sum(0)).norm() / dy.double().sum(0).norm()) < 1e-2
