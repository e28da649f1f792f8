"""GPU parity of the fused RMSNorm -> NVFP4 kernel (C ABI) against the CPU oracle.

Bar: normed output within 2e-3 relative Frobenius error of the oracle (the row mean is summed in
a different order, so single bf16 roundings may flip); codes, scale bytes and unit bit-exact
against the oracle's packing of the kernel's own bf16 normed tensor.
"""
import pytest
import torch

from helpers import rel_fro, synthetic_activation

pytestmark = pytest.mark.gpu

TOL = 2e-3


def _gamma(seed, cols):
    g = torch.Generator().manual_seed(seed)
    return (1 + 0.1 * torch.randn(cols, generator=g)).bfloat16()


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("rows,cols", [(64, 512), (33, 1536), (16, 4096), (5, 8192), (7, 48), (3, 12288), (256, 512), (300, 3584), (257, 4096)])
def test_fused_rmsnorm_quant(rows, cols, mode):
    from metis_hip import ops
    from oracle import metis_oracle as O
    x = synthetic_activation(1002 + rows, rows, cols)
    gamma = _gamma(7, cols)
    normed, p = ops.rmsnorm_quantize(x.cuda(), gamma.cuda(), 1e-6, mode)
    torch.cuda.synchronize()
    want = O.rmsnorm(x, gamma, 1e-6)
    assert rel_fro(normed.cpu(), want) <= TOL
    # elementwise: the row sum is taken in a different order, so rstd may differ in its last bit; a flip of the first
    # bf16 rounding (x * rstd) can carry through the multiplication by gamma and its rounding: at most two bf16 ulps
    d = (normed.cpu().float() - want.float()).abs()
    assert bool((d <= want.float().abs() * 2.0 ** -6 + 1e-30).all())
    assert float((d > 0).float().mean()) < 0.01                  # and that is rare
    mine = normed.cpu()
    codes, scales, unit, _ = O.nvfp4_pack(mine.float() if mode == 0 else mine)
    assert torch.equal(p.codes.cpu(), codes) and torch.equal(p.scales.cpu(), scales)
    assert float(p.unit.cpu()) == float(unit)
    # packed-only variant produces the same integers
    none, p2 = ops.rmsnorm_quantize(x.cuda(), gamma.cuda(), 1e-6, mode, want_normed=False)
    assert none is None and torch.equal(p2.codes, p.codes) and torch.equal(p2.scales, p.scales)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("rows,cols", [(64, 512), (300, 3584), (16384, 4096), (7, 96)])
def test_fused_rmsnorm_quant_with_deferred_scale_bytes(rows, cols, mode):
    """deferred=True: the main kernel only.  Same normed tensor and codes; scale bytes and unit appear on first access
    with the bytes of the two-launch call, and the tiled expansion forms them itself, bit-equal to the eager tensor's."""
    from metis_hip import ops
    x = synthetic_activation(1100 + rows, rows, cols).cuda()
    gamma = _gamma(8, cols).cuda()
    normed, ref = ops.rmsnorm_quantize(x, gamma, 1e-6, mode)
    normed2, lazy = ops.rmsnorm_quantize(x, gamma, 1e-6, mode, deferred=True)
    assert torch.equal(normed, normed2) and torch.equal(lazy.codes, ref.codes)
    assert lazy.__dict__.get("_scales") is None
    assert torch.equal(ops.expand_tiled(lazy, cache=False, mode=mode), ops.expand_tiled(ref, cache=False, mode=mode))
    assert lazy.__dict__.get("_scales") is None and float(lazy.unit.cpu()) == float(ref.unit.cpu())
    _, lazy2 = ops.rmsnorm_quantize(x, gamma, 1e-6, mode, want_normed=False, deferred=True)
    assert torch.equal(lazy2.scales, ref.scales) and float(lazy2.unit.cpu()) == float(ref.unit.cpu())


def test_fused_rmsnorm_quant_config2_full_size():
    """bf16 [16384, 4096], gamma = 1 + N(0, 0.1^2), eps = 1e-6 (P32)."""
    from metis_hip import ops
    from oracle import c_oracle as C
    x = synthetic_activation(1002, 16384, 4096)
    gamma = _gamma(1002, 4096)
    normed, p = ops.rmsnorm_quantize(x.cuda(), gamma.cuda(), 1e-6, 0)
    torch.cuda.synchronize()
    cn, _, _, _ = C.rmsnorm_nvfp4(x, gamma, 1e-6, 0)
    assert rel_fro(normed.cpu(), cn) <= TOL
    cc, cs, cu, _ = C.nvfp4_pack(normed.cpu().contiguous(), 0)
    assert torch.equal(p.codes.cpu(), cc) and torch.equal(p.scales.cpu(), cs) and float(p.unit.cpu()) == cu


def test_value_error_and_limits():
    from metis_hip import ops
    with pytest.raises(ValueError):
        ops.rmsnorm_quantize(torch.zeros(4, 40, dtype=torch.bfloat16, device="cuda"),
                             torch.ones(40, dtype=torch.bfloat16, device="cuda"), 1e-6)
