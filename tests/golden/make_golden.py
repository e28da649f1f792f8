"""Writes tests/golden/*.npz by running the reference's own quantizer / autograd code on CPU.

Run once, in the build container only (the reference checkout does not exist on GPU boxes):

    python tests/golden/make_golden.py [/root/reference]
    python tests/golden/make_golden.py /root/reference hadamard_wide     (only metis_reference_hadamard_wide.npz)
    python tests/golden/make_golden.py /root/reference rollout_bf16      (only metis_reference_rollout_bf16.npz)
    python tests/golden/make_golden.py /root/reference svd_mode          (only metis_reference_svd_mode.npz)

Why an import and not only closed forms: the results recorded here depend on the exact
sequence of per-op roundings of eager PyTorch (bf16-per-op mode differs from an ideal
round-to-nearest E2M1 conversion in ~1 % of elements), on torch's CPU random stream for the
stochastic-rounding quantizer, and on the wiring of the autograd function -- none of which a
closed form fixes bit for bit.  The fixtures are data only: inputs, the uniform draws that the
reference consumed, and its outputs.  bf16 tensors are stored as their uint16 bit patterns.
"""
from __future__ import annotations

import os
import sys
from types import SimpleNamespace

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
sys.dont_write_bytecode = True
sys.path.insert(0, os.path.join(REF, "src", "Metis"))

from Metis import quant as rq  # noqa: E402
from Metis import bitlinear as rb  # noqa: E402


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 -> uint16 patterns; fp32 stays fp32."""
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()
    return t.contiguous().numpy().copy()


def planted_input(seed: int, rows: int, cols: int) -> torch.Tensor:
    """bf16 test tensor with outlier channels, exact ties, a zero block, tiny and huge blocks."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g)
    x[:, 5] *= 20.0                                   # outlier channel
    x[:, cols - 3] *= 20.0
    x = x.bfloat16()
    x[1, 0:16] = 0.0                                  # all-zero block
    x[2, 16:32] = torch.tensor([6.0, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0,
                                -0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5.0, -6.0]).bfloat16()  # scalar=1: every midpoint
    x[3, 32:48] = (torch.randn(16, generator=g) * 1e-12).bfloat16()   # scalar dominated by 1e-9
    x[4, 48:64] = (torch.randn(16, generator=g) * 1e-4).bfloat16()    # small block -> subnormal E4M3 scale
    x[5, 0:16] = (torch.randn(16, generator=g) * 3e4).bfloat16()      # huge block sets the tensor scale
    x[6, 64:80] = torch.tensor([3.0, 0.125, 0.375, 0.625, 0.875, 1.25, 1.75, 2.5,
                                -3.0, -0.125, -0.375, -0.625, -0.875, -1.25, -1.75, -2.5]).bfloat16()  # scalar=.5 midpoints
    x[7, 80:96] = -0.0
    return x


def golden_rne(out: dict):
    x = planted_input(11, 64, 256)
    out["rne_x"] = bits(x)
    for tag, xin in (("p32", x.float()), ("pb16", x)):
        q = rq.Cast2NVFp4e2m1BlockNOSR
        out[f"rne_qdq_{tag}"] = bits(q.quantize_dequantize(xin.clone()))
        s = q.get_scalar(xin.clone())
        out[f"rne_scalar_{tag}"] = bits(s)
        xq = q.quant(xin.clone(), s)
        out[f"rne_quant_{tag}"] = bits(xq)
        s_arg = s.clone()
        out[f"rne_rquant_{tag}"] = bits(q.rquant(xq, s_arg))
        out[f"rne_scalar_after_rquant_{tag}"] = bits(s_arg)      # reference mutates its argument
    # a 3-D activation-shaped case (batch, tokens, hidden)
    g = torch.Generator().manual_seed(12)
    x3 = (torch.randn(2, 24, 128, generator=g) * 0.7).bfloat16()
    out["rne3d_x"] = bits(x3)
    out["rne3d_qdq_p32"] = bits(rq.Cast2NVFp4e2m1BlockNOSR.quantize_dequantize(x3.float()))
    out["rne3d_qdq_pb16"] = bits(rq.Cast2NVFp4e2m1BlockNOSR.quantize_dequantize(x3))
    # weight-like magnitudes (N(0, 0.02^2)): the 1e-9 term perturbs every scalar
    g = torch.Generator().manual_seed(13)
    w = (torch.randn(48, 192, generator=g) * 0.02).bfloat16()
    out["rnew_x"] = bits(w)
    out["rnew_qdq_p32"] = bits(rq.Cast2NVFp4e2m1BlockNOSR.quantize_dequantize(w.float()))
    out["rnew_qdq_pb16"] = bits(rq.Cast2NVFp4e2m1BlockNOSR.quantize_dequantize(w))


def golden_sr(out: dict):
    x = planted_input(21, 32, 128)
    out["sr_x"] = bits(x)
    for tag, xin in (("p32", x.float()), ("pb16", x)):
        q = rq.Cast2NVFp4e2m1Block
        s = q.get_scalar(xin.clone())
        blocks_shape = (xin.shape[0], 1, xin.shape[1] // 16, 16)
        torch.manual_seed(2004)
        u = torch.rand(blocks_shape, dtype=xin.dtype)            # the draw rand_like will make
        torch.manual_seed(2004)
        xq = q.quant(xin.clone(), s)
        out[f"sr_noise_{tag}"] = bits(u.reshape(xin.shape))
        out[f"sr_quant_{tag}"] = bits(xq)
        out[f"sr_rquant_{tag}"] = bits(q.rquant(xq, s.clone()))


def _configure(fwd_in, fwd_w, bwd_g, dtype):
    F = rb.LinearLowbitFunction
    F.q_forward_input = rq.quant_func[fwd_in]
    F.q_forward_weight = rq.quant_func[fwd_w]
    F.q_backward_input = rq.quant_func[bwd_g]
    F.q_backward_weight = rq.quant_func[bwd_g]
    F.q_backward_outputgrad = rq.quant_func[bwd_g]
    F.enable_activation_svd = False
    F.enable_backward_svd = False
    F.enable_nv_recipe = False
    F.compute_dtype = dtype
    F.metis_mode = "mean"


def golden_linear(out: dict):
    """LinearLowbit forward + backward (direct FP4 path) and a hand-assembled BitLinear forward."""
    g = torch.Generator().manual_seed(31)
    B, T, K, N, r = 2, 16, 64, 48, 8
    x = torch.randn(B, T, K, generator=g).bfloat16().float()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().float()
    b = (torch.randn(N, generator=g) * 0.1).bfloat16().float()
    dy = (torch.randn(B, T, N, generator=g) * 1e-3).bfloat16().float()
    args = SimpleNamespace(device="cpu", cache_quantized_weight=False, forward_svd_rank=r)
    _configure("nvfp4e2m1bnosr", "nvfp4e2m1bnosr", "nvfp4e2m1b", torch.float32)

    layer = rb.LinearLowbit(K, N, bias=True, args=args)
    with torch.no_grad():
        layer.weight.copy_(w)
        layer.bias.copy_(b)
    xr = x.clone().requires_grad_(True)
    y = layer(xr)
    torch.manual_seed(2005)
    u = torch.rand((B * T, 1, N // 16, 16), dtype=torch.float32)
    torch.manual_seed(2005)
    y.backward(dy)
    out["lin_x"], out["lin_w"], out["lin_b"], out["lin_dy"] = bits(x), bits(w), bits(b), bits(dy)
    out["lin_y"] = bits(y.detach())
    out["lin_noise_dy"] = bits(u.reshape(B, T, N))
    out["lin_gx"] = bits(xr.grad)
    out["lin_gw"] = bits(layer.weight.grad)
    out["lin_gb"] = bits(layer.bias.grad)

    # BitLinear assembled by hand (split() needs a GPU): low-rank branch + residual branch
    bl = rb.BitLinear.__new__(rb.BitLinear)
    torch.nn.Module.__init__(bl)
    bl.args = args
    bl.is_svd_quant = True
    bl.mean_cache = {}
    bl.activation_group = None
    bl._merged_rollout_weight_cache = None
    bl.layer_name = "golden.layer"
    bl.vlinear = rb.LinearLowbit(K, r, bias=False, args=args)
    bl.ulinear = torch.nn.Linear(r, N, bias=False)
    bl.warmup_linear = rb.LinearLowbit(K, N, bias=True, args=args)
    U, S, Vh = torch.linalg.svd(w, full_matrices=False)
    with torch.no_grad():
        bl.vlinear.weight.copy_(Vh[:r])
        bl.ulinear.weight.copy_(U[:, :r])
        bl.s = torch.nn.Parameter(S[:r].clone())
        bl.warmup_linear.weight.copy_(w - (U[:, :r] * S[:r]) @ Vh[:r])
        bl.warmup_linear.bias.copy_(b)
    _configure("nvfp4e2m1bnosr", "nvfp4e2m1bnosr", "nvfp4e2m1b", torch.float32)
    with torch.no_grad():
        yb = bl(x)
    out["bl_v"] = bits(bl.vlinear.weight.detach())
    out["bl_u"] = bits(bl.ulinear.weight.detach())
    out["bl_s"] = bits(bl.s.detach())
    out["bl_res"] = bits(bl.warmup_linear.weight.detach())
    out["bl_y"] = bits(yb)


def golden_hadamard(out: dict):
    """Tiled random Hadamard rotation of the NV recipe (bitlinear.py:75-211, 395-405, 495-501, 577-585):
    the rotation itself, a rotated wgrad operand through the NVFP4 quantizer, and LinearLowbit forward +
    backward with round-to-nearest quantizers everywhere (no random draws involved)."""
    F = rb.LinearLowbitFunction
    g = torch.Generator().manual_seed(41)
    x = torch.randn(6, 48, generator=g).bfloat16().float()
    F.hadamard_tile_size, F.hadamard_backend, F.hadamard_workspace_mb = 16, "torch_gemm", 128
    out["had_x"] = bits(x)
    out["had_sign16"] = bits(F._get_hadamard_sign(16, torch.device("cpu"), torch.float32))
    out["had_fwd"] = bits(F._apply_hadamard_blocks(x, inverse=False))
    out["had_inv"] = bits(F._apply_hadamard_blocks(x, inverse=True))
    out["had_fwd_bf16"] = bits(F._apply_hadamard_blocks(x.bfloat16(), inverse=False))
    _configure("nvfp4e2m1bnosr", "nvfp4e2m1bnosr", "nvfp4e2m1bnosr", torch.float32)
    F.enable_nv_recipe = True
    try:
        out["had_wgrad_operand_p32"] = bits(F._quantize_wgrad_operand(x.clone(), rq.Cast2NVFp4e2m1BlockNOSR))
        B, T, K, N = 2, 16, 64, 48
        xl = torch.randn(B, T, K, generator=g).bfloat16().float()
        w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().float()
        dy = (torch.randn(B, T, N, generator=g) * 1e-3).bfloat16().float()
        layer = rb.LinearLowbit(K, N, bias=False, args=SimpleNamespace(device="cpu", cache_quantized_weight=False))
        with torch.no_grad():
            layer.weight.copy_(w)
        xr = xl.clone().requires_grad_(True)
        y = layer(xr)
        y.backward(dy)
        out["had_lin_x"], out["had_lin_w"], out["had_lin_dy"] = bits(xl), bits(w), bits(dy)
        out["had_lin_y"], out["had_lin_gx"], out["had_lin_gw"] = bits(y.detach()), bits(xr.grad), bits(layer.weight.grad)
    finally:
        F.enable_nv_recipe = False


def golden_hadamard_wide(out: dict):
    """NV recipe through LinearLowbit at a shape whose backward contractions are multiples of 32 (64 tokens,
    96 -> 64 features), round-to-nearest quantizers everywhere: once in binary32 arithmetic, once with bf16 tensors
    and bf16 arithmetic (the GRPO / QAT configuration)."""
    F = rb.LinearLowbitFunction
    g = torch.Generator().manual_seed(43)
    B, T, K, N = 2, 32, 96, 64
    xl = torch.randn(B, T, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    dy = (torch.randn(B, T, N, generator=g) * 1e-3).bfloat16()
    out["hw_x"], out["hw_w"], out["hw_dy"] = bits(xl), bits(w), bits(dy)
    F.hadamard_tile_size, F.hadamard_backend, F.hadamard_workspace_mb = 16, "torch_gemm", 128
    for tag, dtype in (("p32", torch.float32), ("pb16", torch.bfloat16)):
        _configure("nvfp4e2m1bnosr", "nvfp4e2m1bnosr", "nvfp4e2m1bnosr", dtype)
        F.enable_nv_recipe = True
        try:
            layer = rb.LinearLowbit(K, N, bias=False, args=SimpleNamespace(device="cpu", cache_quantized_weight=False))
            layer.weight.data = w.to(dtype).clone()
            layer.compute_dtype = dtype
            xr = xl.to(dtype).clone().requires_grad_(True)
            y = layer(xr)
            y.backward(dy.to(dtype))
            out[f"hw_{tag}_wq"] = bits(layer._get_quantized_weight(layer.weight.detach().to(dtype)))
            # the two weight-gradient operands as the backward pass forms them (495-501): rotated, quantized, rotated back
            xq = F.quantize_input(xl.to(dtype).clone())
            out[f"hw_{tag}_xq"] = bits(xq)
            out[f"hw_{tag}_wgrad_x"] = bits(F._quantize_wgrad_operand(xq.clone(), F.q_backward_input))
            out[f"hw_{tag}_wgrad_dy"] = bits(F._quantize_wgrad_operand(dy.to(dtype).clone(), F.q_backward_outputgrad))
            out[f"hw_{tag}_y"], out[f"hw_{tag}_gx"] = bits(y.detach()), bits(xr.grad)
            out[f"hw_{tag}_gw"] = bits(layer.weight.grad)
        finally:
            F.enable_nv_recipe = False
            F.compute_dtype = torch.float32


def golden_mean_mode(out: dict):
    """Mean mode (bitlinear.py:311-336): column mean over tokens kept, centred residual through the fused QDQ; a
    prefill call, then a single-token decode call on the same cache (weighted running mean), in binary32 and in
    bf16; and LinearLowbit forward + backward with the mode on for activations and output gradients
    (round-to-nearest quantizers everywhere, so no random draws are involved)."""
    F = rb.LinearLowbitFunction
    g = torch.Generator().manual_seed(51)
    q = rq.Cast2NVFp4e2m1BlockNOSR
    x = (torch.randn(2, 24, 64, generator=g) + 2.0 * torch.randn(1, 1, 64, generator=g)).bfloat16()
    step = (torch.randn(4, 1, 64, generator=g) + 1.0).bfloat16()
    out["mean_x"], out["mean_step"] = bits(x), bits(step)
    for tag, cast in (("p32", torch.float32), ("pb16", torch.bfloat16)):
        cache = {}
        out[f"mean_out_{tag}"] = bits(F.svd_quant(x.to(cast), quant_func=q, metis_mode="mean", mean_cache=cache, cache_key="k"))
        out[f"mean_cache_{tag}"] = bits(cache["k"][0])
        out[f"mean_step_out_{tag}"] = bits(F.svd_quant(step.to(cast), quant_func=q, metis_mode="mean", mean_cache=cache, cache_key="k"))
        out[f"mean_step_cache_{tag}"] = bits(cache["k"][0])
        out[f"mean_step_count_{tag}"] = np.array([cache["k"][1]], dtype=np.int64)
    _configure("nvfp4e2m1bnosr", "nvfp4e2m1bnosr", "nvfp4e2m1bnosr", torch.float32)
    F.enable_activation_svd, F.enable_backward_svd = True, True
    F.activation_lowrank_svd = F.backward_lowrank_svd = 8
    F.activation_lowrank_niter, F.backward_lowrank_niter = 0, 0
    F.activation_broadcast_dim, F.backward_broadcast_dim = 0, -1
    F.tp_simulate = False
    try:
        B, T, K, N = 2, 16, 64, 48
        xl = (torch.randn(B, T, K, generator=g) + 1.5 * torch.randn(1, 1, K, generator=g)).bfloat16().float()
        w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().float()
        b = (torch.randn(N, generator=g) * 0.1).bfloat16().float()
        dy = ((torch.randn(B, T, N, generator=g) + 0.5 * torch.randn(1, 1, N, generator=g)) * 1e-3).bfloat16().float()
        layer = rb.LinearLowbit(K, N, bias=True, args=SimpleNamespace(device="cpu", cache_quantized_weight=False))
        with torch.no_grad():
            layer.weight.copy_(w)
            layer.bias.copy_(b)
        xr = xl.clone().requires_grad_(True)
        y = layer(xr)
        y.backward(dy)
        out["mean_lin_x"], out["mean_lin_w"], out["mean_lin_b"], out["mean_lin_dy"] = bits(xl), bits(w), bits(b), bits(dy)
        out["mean_lin_y"], out["mean_lin_gx"] = bits(y.detach()), bits(xr.grad)
        out["mean_lin_gw"], out["mean_lin_gb"] = bits(layer.weight.grad), bits(layer.bias.grad)
    finally:
        F.enable_activation_svd, F.enable_backward_svd = False, False


def golden_rollout(out: dict):
    """Rollout shortcut of BitLinear.forward (rollout_merge_active, no autograd): one matmul of the quantized
    activation against the cached merged weight (U diag s) Q(V) + Q(W_res), next to the three-GEMM forward of the
    same layer.  binary32 arithmetic; the layer is assembled by hand as in golden_linear."""
    g = torch.Generator().manual_seed(47)
    B, T, K, N, r = 2, 24, 96, 64, 8
    x = torch.randn(B, T, K, generator=g).bfloat16().float()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().float()
    b = (torch.randn(N, generator=g) * 0.1).bfloat16().float()
    args = SimpleNamespace(device="cpu", cache_quantized_weight=True, forward_svd_rank=r)
    _configure("nvfp4e2m1bnosr", "nvfp4e2m1bnosr", "nvfp4e2m1b", torch.float32)
    bl = rb.BitLinear.__new__(rb.BitLinear)
    torch.nn.Module.__init__(bl)
    bl.args = args
    bl.is_svd_quant = True
    bl.mean_cache = {}
    bl.activation_group = None
    bl._merged_rollout_weight_cache = None
    bl.layer_name = "golden.rollout"
    bl.vlinear = rb.LinearLowbit(K, r, bias=False, args=args)
    bl.ulinear = torch.nn.Linear(r, N, bias=False)
    bl.warmup_linear = rb.LinearLowbit(K, N, bias=True, args=args)
    U, S, Vh = torch.linalg.svd(w, full_matrices=False)
    with torch.no_grad():
        bl.vlinear.weight.copy_(Vh[:r].bfloat16().float())
        bl.ulinear.weight.copy_(U[:, :r].bfloat16().float())
        bl.s = torch.nn.Parameter(S[:r].bfloat16().float().clone())
        bl.warmup_linear.weight.copy_((w - (U[:, :r] * S[:r]) @ Vh[:r]).bfloat16().float())
        bl.warmup_linear.bias.copy_(b)
    with torch.no_grad():
        y_three = bl(x)
        rb.BitLinear.rollout_merge_active = True
        try:
            y_merged = bl(x)
            merged_w = bl._get_merged_rollout_weight(torch.float32)
            again = bl._get_merged_rollout_weight(torch.float32)
            assert again is merged_w                                  # cached on the parameter versions
            bl.s.add_(0.0)                                            # bumps the version: the cache is dropped
            assert bl._get_merged_rollout_weight(torch.float32) is not merged_w
        finally:
            rb.BitLinear.rollout_merge_active = False
    out["ro_x"], out["ro_b"] = bits(x), bits(b)
    out["ro_v"], out["ro_u"] = bits(bl.vlinear.weight.detach()), bits(bl.ulinear.weight.detach())
    out["ro_s"], out["ro_res"] = bits(bl.s.detach()), bits(bl.warmup_linear.weight.detach())
    out["ro_merged_weight"] = bits(merged_w)
    out["ro_y_merged"] = bits(y_merged)
    out["ro_y_three_gemm"] = bits(y_three)


def golden_rollout_bf16(out: dict):
    """The rollout shortcut with bf16 tensors and bf16 arithmetic (the GRPO configuration), rank 32, 256 tokens: merged
    weight and the one-matmul forward, assembled by hand as in golden_rollout."""
    g = torch.Generator().manual_seed(53)
    B, T, K, N, r = 2, 128, 128, 96, 32
    dt = torch.bfloat16
    x = torch.randn(B, T, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16().float()
    b = (torch.randn(N, generator=g) * 0.1).bfloat16()
    args = SimpleNamespace(device="cpu", cache_quantized_weight=True, forward_svd_rank=r)
    _configure("nvfp4e2m1bnosr", "nvfp4e2m1bnosr", "nvfp4e2m1b", dt)
    try:
        bl = rb.BitLinear.__new__(rb.BitLinear)
        torch.nn.Module.__init__(bl)
        bl.args = args
        bl.is_svd_quant = True
        bl.mean_cache = {}
        bl.activation_group = None
        bl._merged_rollout_weight_cache = None
        bl.layer_name = "golden.rollout16"
        bl.vlinear = rb.LinearLowbit(K, r, bias=False, args=args, storage_dtype=dt, compute_dtype=dt)
        bl.ulinear = torch.nn.Linear(r, N, bias=False, dtype=dt)
        bl.warmup_linear = rb.LinearLowbit(K, N, bias=True, args=args, storage_dtype=dt, compute_dtype=dt)
        U, S, Vh = torch.linalg.svd(w, full_matrices=False)
        with torch.no_grad():
            bl.vlinear.weight.copy_(Vh[:r].bfloat16())
            bl.ulinear.weight.copy_(U[:, :r].bfloat16())
            bl.s = torch.nn.Parameter(S[:r].bfloat16().clone())
            bl.warmup_linear.weight.copy_((w - (U[:, :r] * S[:r]) @ Vh[:r]).bfloat16())
            bl.warmup_linear.bias.copy_(b)
        with torch.no_grad():
            rb.BitLinear.rollout_merge_active = True
            try:
                y_merged = bl(x)
                merged_w = bl._get_merged_rollout_weight(dt)
            finally:
                rb.BitLinear.rollout_merge_active = False
        assert y_merged.dtype == dt and merged_w.dtype == dt
        out["ro16_x"], out["ro16_b"] = bits(x), bits(b)
        out["ro16_v"], out["ro16_u"] = bits(bl.vlinear.weight.detach()), bits(bl.ulinear.weight.detach())
        out["ro16_s"], out["ro16_res"] = bits(bl.s.detach()), bits(bl.warmup_linear.weight.detach())
        out["ro16_merged_weight"] = bits(merged_w)
        out["ro16_y_merged"] = bits(y_merged)
    finally:
        rb.LinearLowbitFunction.compute_dtype = torch.float32


def golden_svd_mode(out: dict):
    """LinearLowbitFunction.svd_quant with metis_mode="svd" (bitlinear.py:243-309) on a [2, 64, 256] activation, rank 32,
    in binary32 and in bf16 arithmetic.  The factors come from torch.svd_lowrank, which draws from torch's random
    stream: a recording wrapper around it keeps what it returned, so that a consumer of this file starts from the same
    factors.  ker is not returned by the reference; it is recomputed here by the reference's own expressions
    (:276-296) on the reference's quantizer, for the comparison of summation orders."""
    q = rq.Cast2NVFp4e2m1BlockNOSR
    g = torch.Generator().manual_seed(71)
    B, T, D, r = 2, 64, 256, 32
    low = torch.randn(B * T, 6, generator=g) @ torch.randn(6, D, generator=g)
    x = (low + 0.3 * torch.randn(B * T, D, generator=g)).reshape(B, T, D)
    x[..., 7] *= 12.0
    for tag, dt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        xin = x.bfloat16().to(dt)                     # bf16 values in both cases
        kept = {}
        real = torch.svd_lowrank

        def recording(a, q=6, niter=2, M=None):
            u, s, v = real(a, q=q, niter=niter, M=M)
            kept["u"], kept["s"], kept["v"] = u.clone(), s.clone(), v.clone()
            return u, s, v

        torch.manual_seed(1000 + len(tag))
        torch.svd_lowrank = recording
        try:
            y = rb.LinearLowbitFunction.svd_quant(xin.clone(), quant_func=q, rank=r, niter=2, broadcast_dim=-1, metis_mode="svd")
        finally:
            torch.svd_lowrank = real
        ug, sg, vg = kept["u"].to(dt), kept["s"].to(dt), kept["v"].to(dt).T
        us_, vs_ = q.get_scalar(ug), q.get_scalar(vg)
        ugq = q.rquant(q.quant(ug, us_), us_)
        vgq = q.rquant(q.quant(vg, vs_), vs_)
        ker = ugq @ torch.diag(sg) @ vgq
        again = ker + q.quantize_dequantize(xin.reshape(-1, D) - ker)
        assert torch.equal(again.view(B, T, D), y)    # the recomputation follows the reference's path
        out[f"svd_{tag}_x"] = bits(xin.bfloat16())    # bf16 values in both cases
        out[f"svd_{tag}_u"], out[f"svd_{tag}_s"], out[f"svd_{tag}_v"] = bits(kept["u"]), bits(kept["s"]), bits(kept["v"])
        out[f"svd_{tag}_uq"], out[f"svd_{tag}_vq"] = bits(ugq), bits(vgq)
        out[f"svd_{tag}_ker"] = bits(ker)
        out[f"svd_{tag}_y"] = bits(y)


def main():
    torch.set_num_threads(1)
    if len(sys.argv) > 2 and sys.argv[2] == "svd_mode":         # only this file (the others are not touched)
        sv: dict = {}
        golden_svd_mode(sv)
        path = os.path.join(HERE, "metis_reference_svd_mode.npz")
        np.savez_compressed(path, **sv)
        print(f"wrote {path}: {len(sv)} arrays, {os.path.getsize(path)} bytes")
        return
    if len(sys.argv) > 2 and sys.argv[2] == "rollout_bf16":     # only this file (the others are not touched)
        ro16: dict = {}
        golden_rollout_bf16(ro16)
        path = os.path.join(HERE, "metis_reference_rollout_bf16.npz")
        np.savez_compressed(path, **ro16)
        print(f"wrote {path}: {len(ro16)} arrays, {os.path.getsize(path)} bytes")
        return
    if len(sys.argv) > 2 and sys.argv[2] == "hadamard_wide":    # only this file (the others are not touched)
        hw: dict = {}
        golden_hadamard_wide(hw)
        path = os.path.join(HERE, "metis_reference_hadamard_wide.npz")
        np.savez_compressed(path, **hw)
        print(f"wrote {path}: {len(hw)} arrays, {os.path.getsize(path)} bytes")
        return
    out: dict = {}
    golden_rne(out)
    golden_sr(out)
    golden_linear(out)
    path = os.path.join(HERE, "metis_reference_golden.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes; torch {torch.__version__}")
    had: dict = {}
    golden_hadamard(had)
    path = os.path.join(HERE, "metis_reference_hadamard.npz")
    np.savez_compressed(path, **had)
    print(f"wrote {path}: {len(had)} arrays, {os.path.getsize(path)} bytes")
    ro: dict = {}
    golden_rollout(ro)
    path = os.path.join(HERE, "metis_reference_rollout.npz")
    np.savez_compressed(path, **ro)
    print(f"wrote {path}: {len(ro)} arrays, {os.path.getsize(path)} bytes")
    mm: dict = {}
    golden_mean_mode(mm)
    path = os.path.join(HERE, "metis_reference_mean_mode.npz")
    np.savez_compressed(path, **mm)
    print(f"wrote {path}: {len(mm)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
