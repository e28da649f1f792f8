"""GPU parity of the pieces of the mean mode (column mean kept in high precision, centred residual in
NVFP4): centred quantizers bit-exact against the oracle on x - me, the packed matrix-vector product and
the binary32 bias of the GEMM against double precision."""
import pytest
import torch

from helpers import rel_fro, synthetic_activation

pytestmark = pytest.mark.gpu


def _check(p, codes, scales, unit, what):
    torch.cuda.synchronize()
    assert torch.equal(p.codes.cpu(), codes), f"codes differ ({what}): {(p.codes.cpu() != codes).sum().item()}"
    assert torch.equal(p.scales.cpu(), scales), f"scales differ ({what})"
    assert float(p.unit.cpu()) == float(unit), f"unit differs ({what})"


def _offset_activation(seed, rows, cols):
    x = synthetic_activation(seed, rows, cols).float()
    g = torch.Generator().manual_seed(seed + 1)
    return (x + 3.0 * torch.randn(1, cols, generator=g)).bfloat16()        # a per-column offset worth removing


@pytest.mark.parametrize("col", [False, True])
@pytest.mark.parametrize("src", ["bf16", "f32"])
def test_centered_quant_binary32_arithmetic(col, src):
    """x - me in binary32 (one rounding, as the reference's `input_flat - me`), then the quantizer."""
    from metis_hip import ops
    from oracle import metis_oracle as O
    x = _offset_activation(500, 256, 192)
    xin = x.float() if src == "bf16" else x.float() + 1e-3 * torch.randn(256, 192, generator=torch.Generator().manual_seed(3))
    me = xin.mean(dim=0)
    res = xin - me
    p = ops.quantize((x if src == "bf16" else xin).cuda(), 0, col=col, center=me.cuda())
    codes, scales, unit, _ = (O.nvfp4_pack_col if col else O.nvfp4_pack)(res)
    _check(p, codes, scales, unit, f"rne col={col} {src}")
    u = torch.rand(256, 192, generator=torch.Generator().manual_seed(4))
    p = ops.quantize((x if src == "bf16" else xin).cuda(), 0, col=col, sr=True, noise=u.cuda(), center=me.cuda())
    codes, scales, unit, _ = (O.nvfp4_pack_col if col else O.nvfp4_pack)(res, u)
    _check(p, codes, scales, unit, f"sr col={col} {src}")


@pytest.mark.parametrize("col", [False, True])
def test_centered_quant_bf16_arithmetic(col):
    from metis_hip import ops
    from oracle import metis_oracle as O
    x = _offset_activation(510, 128, 256)
    me = x.mean(dim=0)                                             # bf16, as torch gives it for a bf16 tensor
    res = x - me                                                   # bf16 subtraction: one rounding
    p = ops.quantize(x.cuda(), 1, col=col, center=me.cuda())
    codes, scales, unit, _ = (O.nvfp4_pack_col if col else O.nvfp4_pack)(res)
    _check(p, codes, scales, unit, f"pb16 col={col}")
    u = torch.rand(128, 256, generator=torch.Generator().manual_seed(5)).bfloat16()
    p = ops.quantize(x.cuda(), 1, col=col, sr=True, noise=u.cuda(), center=me.cuda())
    codes, scales, unit, _ = (O.nvfp4_pack_col if col else O.nvfp4_pack)(res, u)
    _check(p, codes, scales, unit, f"pb16 sr col={col}")


def test_centered_quant_own_stream_and_errors():
    from metis_hip import _lib, ops
    x = _offset_activation(520, 64, 128).cuda()
    me = x.float().mean(dim=0)
    a = ops.quantize(x, 0, sr=True, seed=7, offset=3, center=me)
    b = ops.quantize(x, 0, sr=True, seed=7, offset=3, center=me)
    rne = ops.quantize(x, 0, center=me)
    assert torch.equal(a.codes, b.codes) and torch.equal(a.scales, rne.scales) and float(a.unit) == float(rne.unit)
    with pytest.raises(ValueError):
        ops.quantize(x, 0, center=me[:-1])


@pytest.mark.parametrize("rows,cols", [(192, 256), (1000, 48), (3584, 18944), (5, 16)])
def test_packed_matvec(rows, cols):
    from metis_hip import ops
    g = torch.Generator().manual_seed(rows + cols)
    w = (torch.randn(rows, cols, generator=g) * 0.05).bfloat16().cuda()
    p = ops.quantize(w)
    v = torch.randn(cols, generator=g).cuda()
    deq = ops.dequantize(p, torch.float32).double()
    y = ops.matvec(p, v, alpha=0.5)
    want = 0.5 * (deq @ v.double())
    assert rel_fro(y.cpu().double(), want.cpu()) <= 1e-5
    ones = ops.matvec(p)
    assert rel_fro(ones.cpu().double(), deq.sum(dim=1).cpu()) <= 1e-5
    split = torch.zeros(rows, 32, dtype=torch.bfloat16, device="cuda")
    out = torch.empty(rows, dtype=torch.float32, device="cuda")
    ops.matvec(p, v, out=out, split=split, split_col=4)
    torch.cuda.synchronize()
    back = split[:, 4].float() + split[:, 5].float() + split[:, 6].float()
    assert torch.equal(back, out) or float((back - out).abs().max()) <= 1e-7 * float(out.abs().max())
    assert int((split[:, :4] != 0).sum()) == 0 and int((split[:, 7:] != 0).sum()) == 0


@pytest.mark.parametrize("M,N,K", [(64, 512, 1024), (300, 260, 512), (512, 512, 2048), (128, 136, 96)])
def test_gemm_binary32_bias(M, N, K):
    """Every GEMM kernel (skinny, 256-tiles, split-K, 128-tiles) adds a binary32 bias at full precision."""
    from metis_hip import ops
    g = torch.Generator().manual_seed(M + N)
    x = synthetic_activation(530 + M, M, K).cuda()
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16().cuda()
    bias = (torch.randn(N, generator=g) * 3.0).cuda()             # binary32, not bf16-valued
    px, pw = ops.quantize(x), ops.quantize(w)
    got = ops.linear_fwd(px, pw, bias=bias, out_dtype=torch.float32)
    want = ops.dequantize(px, torch.float32).double() @ ops.dequantize(pw, torch.float32).double().T + bias.double()
    torch.cuda.synchronize()
    assert rel_fro(got.cpu(), want.cpu()) <= 1e-6
