"""CPU oracle for the Metis NVFP4 hot path (TEST INFRASTRUCTURE, not product code).

This file restates, op for op and with the same PyTorch CPU operators, the arithmetic
of the reference implementation so that the HIP kernels can be checked for bit parity.
Only tests, the smoke check and the benchmark's CPU-baseline leg may import it; the
shipped package never does.

Every tensor op below rounds to the dtype ``D`` of its input exactly as eager PyTorch
does, so the two parity modes are obtained by choosing the input dtype:

* P32  : call with ``x_bf16.float()``  -> fp32 arithmetic on bf16-valued inputs
* PB16 : call with the bf16 tensor     -> every eager op rounds to bf16

Reference files followed (paths relative to the reference checkout):
  src/Metis/Metis/quant.py:6-36      fused NVFP4 round-to-nearest QDQ
  src/Metis/Metis/quant.py:118-128   E2M1 element rule (compress / round / expand)
  src/Metis/Metis/quant.py:137-147   stochastic-rounding element rule
  src/Metis/Metis/quant.py:183-195   block reshape
  src/Metis/Metis/quant.py:435-477, 545-548  get_scalar / quant / rquant
  src/Metis/models/llama.py:23-31    RMSNorm
  src/Metis/Metis/bitlinear.py:407-441   LinearLowbitFunction.forward
  src/Metis/Metis/bitlinear.py:443-513   LinearLowbitFunction.backward
  src/Metis/Metis/bitlinear.py:736-769   BitLinear.forward
  src/Metis/Metis/bitlinear.py:243-309   svd_quant, metis_mode="svd" (factors given)

Pinning status (which independent evidence fixes each function) is listed in
``tests/test_oracle_pins.py`` and in the design notes; nothing here is "parity
unpinned".

The reference never materialises FP4 codes or E4M3 bytes (it returns dequantized
tensors); ``nvfp4_pack`` exposes the integers that its arithmetic passes through:
  code nibble  = (x < 0) << 3 | r      r = the rounded compressed magnitude, 0..7
  scale byte   = bits of (scalar / unit) cast to float8_e4m3fn
  unit         = max(scalar) / 448
and ``nvfp4_unpack_dequant`` rebuilds the reference's output from them with the
reference's own last three multiplications, so pack -> unpack == fused QDQ bit for bit.
"""
from __future__ import annotations

import torch

BLOCK = 16
# value (in units of scalar/2) of each magnitude code: quant.py:32-34 expand step
E2M1_TWICE = (0.0, 1.0, 2.0, 3.0, 4.0, 6.0, 8.0, 12.0)


def _blocks(x: torch.Tensor):
    """[..., C] -> [R, C/16, 16]; ValueError when 16 does not divide C (quant.py:400-403)."""
    cols = x.shape[-1]
    if cols % BLOCK != 0:
        raise ValueError(
            f"NVFP4 block shape (1, {BLOCK}) does not divide tensor shape {tuple(x.shape)}"
        )
    flat = x.reshape(-1, cols)
    return flat.view(flat.shape[0], cols // BLOCK, BLOCK)


def block_scalars(x: torch.Tensor) -> torch.Tensor:
    """Raw per-block scalar, quant.py:19 and 449-455: amax|x| / 6 + 1e-9  -> [R, C/16]."""
    b = _blocks(x)
    return b.abs().amax(dim=2) / 6 + 1e-9


def tensor_unit(scalar: torch.Tensor) -> torch.Tensor:
    """quant.py:21-22: unit = max|scalar| / 448 (0-dim tensor of dtype D)."""
    return scalar.abs().amax() / 448


def e4m3_scale(scalar: torch.Tensor, unit: torch.Tensor) -> torch.Tensor:
    """quant.py:23: (scalar / unit) cast to float8_e4m3fn (the stored block-scale byte)."""
    return (scalar / unit).to(torch.float8_e4m3fn)


def _compress(q: torch.Tensor) -> torch.Tensor:
    """quant.py:28-30 / 125: fold [4,8] by 1/2 and [8,12] by 1/4 so codes are integers."""
    return q - (torch.relu(q - 4) / 2 + torch.relu(q - 8) / 4)


def _expand(r: torch.Tensor) -> torch.Tensor:
    """quant.py:32-34 / 127: inverse of the fold on the integer grid."""
    return r + (torch.relu(r - 4) + torch.relu(r - 6) * 2)


def magnitude_codes(x: torch.Tensor, scalar: torch.Tensor, noise: torch.Tensor | None = None):
    """Rounded compressed magnitude r (same dtype as x) for every element, [R, C/16, 16].

    RNE (quant.py:27-31): r = round(compress(|x| / (scalar/2))).
    SR  (quant.py:139-145): compress, then += (noise - 0.5), then round; ``noise`` stands in
    for torch.rand_like so the draw can be shared with the kernel under test.
    """
    b = _blocks(x)
    q = b.abs() / (scalar.unsqueeze(-1) / 2)
    q = _compress(q)
    if noise is not None:
        q = q + (noise.reshape(b.shape).to(q.dtype) - 0.5)
    return torch.round(q)


def nvfp4_qdq(x: torch.Tensor, noise: torch.Tensor | None = None) -> torch.Tensor:
    """Fused QDQ, quant.py:6-36 (noise=None) or the SR three-call result (quant.py:273-388)."""
    b = _blocks(x)
    scalar = block_scalars(x)
    unit = tensor_unit(scalar)
    dq = e4m3_scale(scalar, unit).to(scalar.dtype) * unit
    r = magnitude_codes(x, scalar, noise)
    v = _expand(r)
    out = v * b.sign() / 2 * dq.unsqueeze(-1)
    return out.reshape(x.shape)


# ----------------------------------------------------------------------------- 3-call form
def get_scalar(x: torch.Tensor) -> torch.Tensor:
    """quant.py:435-455 -> [R, C/16]."""
    return block_scalars(x)


def quant(x: torch.Tensor, s: torch.Tensor, noise: torch.Tensor | None = None) -> torch.Tensor:
    """quant.py:459-466 (+118-128 or 137-147): values in {0, +-.5, ..., +-6} as dtype D."""
    b = _blocks(x)
    r = magnitude_codes(x, s.reshape(b.shape[0], b.shape[1]), noise)
    return (_expand(r) * b.sign() / 2).reshape(x.shape)


def rquant(xq: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    """quant.py:470-548: E4M3 round trip of s / (max s / 448), then xq * s.

    The reference divides ``s`` IN PLACE (line 473); this restatement keeps that side
    effect because callers can observe it.
    """
    b = _blocks(xq)
    smax = s.abs().max()
    s /= smax / 448
    s2 = s.to(torch.float8_e4m3fn).to(s.dtype)
    s2 *= smax / 448
    return (b * s2.reshape(b.shape[0], b.shape[1], 1)).reshape(xq.shape)


# ----------------------------------------------------------------------------- "svd" mode, factors given
def svd_mode_recompose(x: torch.Tensor, ug: torch.Tensor, sg: torch.Tensor, vg: torch.Tensor, ker: torch.Tensor | None = None):
    """bitlinear.py:276-303 from the point where the factors exist: x [L, D], ug [L, r], sg [r], vg [r, D] (already
    `vg.T`), all in the dtype D of the arithmetic.  U and V go through the three calls, ker = ug @ diag(sg) @ vg, the
    residual through the fused QDQ.  Returns (ker, residual QDQ, ker + residual QDQ).

    ker: the reference's matrix product leaves the order of its additions to the BLAS; this restatement takes
    `ug @ diag(sg)` as the elementwise product it is (one nonzero term per sum) and sums the second product in the
    order k = 0 .. r-1 with fused multiply-adds in binary32 (oracle/metis_oracle.c), rounding to bf16 once in bf16
    arithmetic.  A caller may pass another ker (the reference's own) to check everything behind it bit for bit."""
    from . import c_oracle
    s_u, s_v = get_scalar(ug), get_scalar(vg)
    ugq = rquant(quant(ug, s_u), s_u)
    vgq = rquant(quant(vg, s_v), s_v)
    if ker is None:
        us = ugq * sg                                  # == ugq @ diag(sg): every other term of the sums is an exact zero
        ker = c_oracle.lowrank_product(us.float(), vgq.float()).to(x.dtype)
    res = nvfp4_qdq(x - ker)
    return ker, res, ker + res


# ----------------------------------------------------------------------------- packed view
def nvfp4_pack(x: torch.Tensor, noise: torch.Tensor | None = None):
    """Integers the reference arithmetic passes through.

    Returns (codes u8 [R, C/2], scales u8 [R, C/16], unit 0-dim tensor of dtype D, n_clamped).
    Element 2j sits in the low nibble of byte j.  Under SR the reference can round the block
    maximum up to r = 8 (an off-grid value 8*scalar that no FP4 code represents); such elements
    are clamped to r = 7 and counted in n_clamped.  RNE never produces them.
    """
    b = _blocks(x)
    scalar = block_scalars(x)
    unit = tensor_unit(scalar)
    sbytes = e4m3_scale(scalar, unit).view(torch.uint8)
    r = magnitude_codes(x, scalar, noise)
    n_clamped = int((r > 7).sum())
    r = r.clamp(0, 7).to(torch.uint8)
    nib = r | ((b < 0).to(torch.uint8) << 3)
    nib = nib.reshape(b.shape[0], -1)
    codes = nib[:, 0::2] | (nib[:, 1::2] << 4)
    return codes.contiguous(), sbytes.contiguous(), unit, n_clamped


def nvfp4_unpack_dequant(codes: torch.Tensor, scales: torch.Tensor, unit: torch.Tensor,
                         dtype: torch.dtype) -> torch.Tensor:
    """quant.py:23-24,32-35 applied to stored integers: ((v*sign)/2) * (e4m3 * unit) in ``dtype``."""
    rows = codes.shape[0]
    nib = torch.stack((codes & 0xF, codes >> 4), dim=-1).reshape(rows, -1)
    mag = torch.tensor(E2M1_TWICE, dtype=dtype)[(nib & 7).long()]
    sign = torch.where((nib & 8) != 0, -1.0, 1.0).to(dtype)
    dq = scales.view(torch.float8_e4m3fn).to(dtype) * unit.to(dtype)
    vals = (mag * sign / 2).view(rows, -1, BLOCK) * dq.unsqueeze(-1)
    return vals.reshape(rows, -1)


def nvfp4_pack_col(x: torch.Tensor, noise: torch.Tensor | None = None):
    """Blocks of 16 along dim 0 (the transposed operand of a token-contracting GEMM).

    Equals row packing of x.T; output shapes [C, R/2], [C, R/16].
    """
    xt = x.reshape(-1, x.shape[-1]).t().contiguous()
    nt = None if noise is None else noise.reshape(-1, noise.shape[-1]).t().contiguous()
    return nvfp4_pack(xt, nt)


# ----------------------------------------------------------------------------- RMSNorm
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """llama.py:23-31: fp32 normalisation, cast to the input dtype, then * weight."""
    xf = x.float()
    normed = xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
    return normed.type_as(x) * weight


def rmsnorm_nvfp4(x: torch.Tensor, weight: torch.Tensor, eps: float, p32: bool = True):
    """RMSNorm then NVFP4 packing of the normed tensor (the contract of the fused kernel).

    There is no fused op in the reference; its contract is llama.py:23-31 followed by
    quant.py:6-36 on the result (bitlinear.py:371-393 is the call site of the latter).
    """
    y = rmsnorm(x, weight, eps)
    codes, scales, unit, _ = nvfp4_pack(y.float() if p32 else y)
    return y, codes, scales, unit


# ----------------------------------------------------------------------------- linear
def linear_forward(xq: torch.Tensor, wq: torch.Tensor, bias: torch.Tensor | None):
    """bitlinear.py:435-438: out = X^ @ W^.T (+ bias) on already-dequantized operands."""
    out = torch.matmul(xq, wq.T)
    if bias is not None:
        out = out + bias
    return out


def metis_forward(x: torch.Tensor, v: torch.Tensor, s: torch.Tensor, u: torch.Tensor,
                  w_res: torch.Tensor, bias: torch.Tensor | None, p32: bool = True,
                  quantized_lowrank: bool = False, mean_mode: bool = False) -> torch.Tensor:
    """Low-rank-residual linear, bitlinear.py:736-769 with the sub-module layout of 863-879.

    y = ulinear(s * vlinear(x)) + warmup_linear(x)
      = ((x . v^T) * s) . u^T  +  QDQ(x) . QDQ(w_res)^T + bias
    x [M,K] bf16, v [r,K], s [r], u [N,r], w_res [N,K] (all bf16).
    Default (north-star) variant: the low-rank operands are bf16 -- t = bf16(bf16(x . v^T) * s) is
    the stored rank-r activation -- and both branches are ACCUMULATED IN FP32 and summed before
    the single rounding of the output to bf16.  With ``quantized_lowrank`` the rank-r branch
    consumes QDQ(x) and QDQ(v) in dtype D as the current reference file does
    (bitlinear.py:752, 863-871).  The residual branch is computed in fp32 (p32) or bf16.
    ``mean_mode`` (bitlinear.py:311-336, metis_mode="mean", a first call without cached mean): the residual branch
    sees X^ = me + QDQ(x - me) with me the column mean over tokens, every op in dtype D (the expression
    tests/test_oracle_golden.py pins against the reference's own svd_quant outputs).
    Returns bf16 [M,N].
    """
    D = torch.float32 if p32 else torch.bfloat16
    if mean_mode:
        xd = x.to(D)
        me = xd.mean(dim=0, keepdim=True)
        xq = me + nvfp4_qdq(xd - me)
    else:
        xq = nvfp4_qdq(x.to(D))
    wq = nvfp4_qdq(w_res.to(D))
    res = linear_forward(xq, wq, None if bias is None else bias.to(D))
    if quantized_lowrank:
        t = torch.matmul(xq, nvfp4_qdq(v.to(D)).T)
        t = s.to(D) * t
        low = torch.matmul(t, u.to(D).T)
    else:
        t = torch.matmul(x, v.T)
        t = s * t
        low = torch.matmul(t.float(), u.float().T)
    return (low.float() + res.float()).to(torch.bfloat16)


def linear_backward(dyq: torch.Tensor, xq: torch.Tensor, wq: torch.Tensor):
    """bitlinear.py:502-510 on dequantized operands: (grad_input, grad_weight fp32)."""
    gw = torch.matmul(dyq.reshape(-1, dyq.shape[-1]).T, xq.reshape(-1, xq.shape[-1]))
    gx = torch.matmul(dyq, wq)
    return gx, gw.to(torch.float32)
