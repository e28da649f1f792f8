"""RMSNorm fused with the NVFP4 quantization of its output, wired into a projection group.

The reference has no fused norm: it runs the model's RMSNorm (src/Metis/models/llama.py:23-31; the
Hugging Face Qwen2/Llama classes compute the same thing) and then the first projection of a
{q,k,v} or {gate,up} group quantizes the normed tensor once for the whole group
(src/Metis/Metis/bitlinear.py:676-702).  `FusedRMSNormQuant` replaces the norm module in front of
such a group: one kernel reads the hidden states once and writes the normed bf16 tensor and its
packed NVFP4 form, and the packed tensor is left in the group's cache under the identity of the
normed tensor, which is exactly what the group's first projection would have put there.
"""
from __future__ import annotations

import weakref

import torch
from torch import nn

from . import ops
from ._lib import MODE_P32, MODE_PB16
from .ops import CenteredNVFP4
from .bitlinear import BitLinear, LinearLowbitFunction
from .quant import is_hip_nvfp4


class _NormedWithGrad(torch.autograd.Function):
    """Carries the kernel's normed output into autograd: forward hands the precomputed tensor through,
    backward is the RMSNorm gradient in binary32."""

    @staticmethod
    def forward(ctx, x, weight, normed, eps):
        ctx.save_for_backward(x, weight)
        ctx.eps = eps
        return normed.view_as(normed)

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        xf, gf = x.float(), g.float()
        rstd = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + ctx.eps)
        xhat = xf * rstd
        prod = (gf * xhat.to(x.dtype).float()).reshape(-1, x.shape[-1])
        if prod.is_cuda and prod.shape[1] % 4 == 0:
            g_weight = ops.column_sum(prod, torch.float32).to(weight.dtype)     # torch's reduction over dim 0 is ~8x slower
        else:
            g_weight = prod.sum(dim=0).to(weight.dtype)
        gh = gf * weight.float()
        g_x = (rstd * (gh - xhat * (gh * xhat).mean(dim=-1, keepdim=True))).to(x.dtype)
        return g_x, g_weight, None, None


class FusedRMSNormQuant(nn.Module):
    """Drop-in for an RMSNorm module (`weight`, `variance_epsilon`) whose output feeds a projection group."""

    def __init__(self, weight: nn.Parameter, eps: float, group: dict):
        super().__init__()
        self.weight = weight
        self.variance_epsilon = eps
        self.group = group

    @classmethod
    def from_norm(cls, norm: nn.Module, group: dict) -> "FusedRMSNormQuant":
        eps = getattr(norm, "variance_epsilon", None)
        if eps is None:
            eps = getattr(norm, "eps", 1e-6)
        return cls(norm.weight, float(eps), group)

    def extra_repr(self):
        return f"{tuple(self.weight.shape)}, eps={self.variance_epsilon}, group={self.group['name']}"

    def _plain(self, x):
        dtype = x.dtype
        h = x.to(torch.float32)
        h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.variance_epsilon)
        return self.weight * h.to(dtype)

    def _mean_mode(self, x: torch.Tensor):
        """The reference's default arguments (mean mode, src/grpo/grpo.py:66-69): the group's activation is
        mean + QDQ(normed - mean) with the column mean over tokens (src/Metis/Metis/bitlinear.py:311-336).  One pass
        over x writes the normed tensor and leaves its column sums; the centred quantizer then reads the normed tensor.
        The running mean of single-token decode calls is kept in the group's cache exactly as the first projection of
        the group would keep it."""
        F = LinearLowbitFunction
        cd = F.compute_dtype
        cols = x.shape[-1]
        rows = x.numel() // cols
        group = self.group
        cache, key = group["mean_cache"], f"{group['name']}.shared"
        seq_len = x.shape[1] if x.dim() == 3 else x.shape[0]
        running = seq_len == 1 and key in cache
        cached_mean, cached_count = cache[key] if running else (None, 0)
        if cached_count + rows > 2 ** 24:
            return None
        normed, me, me32 = ops.rmsnorm_colmean(x, self.weight, self.variance_epsilon, cd, cached_mean, cached_count)
        cache[key] = (me.detach().unsqueeze(0), cached_count + rows)
        more = {"deferred": True} if (F._bf16_rounding() and me.dtype == torch.bfloat16) else {}
        packed = CenteredNVFP4(F.q_forward_input.pack(normed, arith=cd, center=me, **more), me, me32)
        return normed, packed

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        F = LinearLowbitFunction
        cols = x.shape[-1]
        fused = (x.is_cuda and x.dtype == torch.bfloat16 and self.weight.dtype == torch.bfloat16 and cols % 32 == 0
                 and cols <= 16384 and is_hip_nvfp4(F.q_forward_input) and (not F.enable_nv_recipe or F._nv_on_kernels())
                 and x.numel() > 0)     # (NV recipe: the forward quantizes its activation unrotated, like any other)
        mean_mode = fused and F.enable_activation_svd
        if mean_mode:
            fused = (F._mean_mode_packable() and cols <= 4096 and F.compute_dtype in (torch.float32, torch.bfloat16)
                     and self.group.get("mean_cache") is not None)
        if not fused:
            return self._plain(x)
        mode = MODE_P32 if F.compute_dtype == torch.float32 else MODE_PB16
        with torch.no_grad():
            if mean_mode:
                got = self._mean_mode(x)
                if got is None:
                    return self._plain(x)
                normed, packed = got
                packed.residual.shared = True
            else:
                cached = all(m._weights_cached() for m in self.group.get("members", ()))
                normed, packed = ops.rmsnorm_quantize(x, self.weight, self.variance_epsilon, mode,
                                                      deferred=F._scales_formed_by_consumer(x.numel() // cols, cached))
        normed = normed.reshape(x.shape)
        out = _NormedWithGrad.apply(x, self.weight, normed, self.variance_epsilon) if torch.is_grad_enabled() and (
            x.requires_grad or self.weight.requires_grad) else normed
        group = self.group

        def clear(ref):
            if group.get("input_ref") is ref:
                group["input_ref"] = None
                group["quantized_input"] = None

        if not mean_mode:
            packed.shared = True                 # read by every member of the group: its tiled expansion is kept while it lives
        group["input_ref"] = weakref.ref(out, clear)
        group["quantized_input"] = packed
        return out


def fuse_rmsnorm_into_groups(model: nn.Module) -> int:
    """Replace `input_layernorm` / `post_attention_layernorm` of every decoder layer whose q/k/v or
    gate/up projections are BitLinear layers sharing an activation group.  Returns the number of norms
    replaced.  Layers with other layouts are left alone."""
    replaced = 0
    for layer in model.modules():
        for norm_name, path in (("input_layernorm", ("self_attn", "q_proj")), ("post_attention_layernorm", ("mlp", "gate_proj"))):
            norm = getattr(layer, norm_name, None)
            owner = getattr(layer, path[0], None)
            proj = getattr(owner, path[1], None) if owner is not None else None
            if norm is None or isinstance(norm, FusedRMSNormQuant) or not isinstance(proj, BitLinear):
                continue
            group = getattr(proj, "activation_group", None)
            if group is None or not hasattr(norm, "weight") or norm.weight.dim() != 1:
                continue
            setattr(layer, norm_name, FusedRMSNormQuant.from_norm(norm, group))
            replaced += 1
    return replaced
