"""Model patching with the reference's interface (src/grpo/grpo.py:62-215).

``MetisArgs`` carries the same fields with the same defaults; ``replace_linear_with_metis`` swaps every
targeted nn.Linear for a BitLinear, copies its weights, wires q/k/v and gate/up projections to one
shared activation-quantization group each, and factorises the weight when forward SVD is enabled.
"""
from __future__ import annotations

import torch

from .bitlinear import BitLinear

DEFAULT_TARGETS = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]


class MetisArgs:
    """Metis configuration (reference grpo.py:62-117; same attribute names and defaults)."""

    def __init__(self, metis_mode: str = "mean", enable_forward_svd: bool = True, enable_activation_svd: bool = True,
                 enable_backward_svd: bool = True, forward_svd_rank: int = 64, activation_lowrank_svd: int = 64,
                 backward_lowrank_svd: int = 64, cache_quantized_weight: bool = False, compile_qdq: bool = False,
                 enable_nv_recipe: bool = False, hadamard_workspace_mb: int = 128, hadamard_tile_size: int = 16,
                 hadamard_backend: str = "auto"):
        self.device = "cuda"
        self.enable_forward_svd = enable_forward_svd
        self.enable_lowbit = True
        self.enable_te = False
        self.q_forward_input = "nvfp4e2m1bnosr"
        self.q_forward_weight = "nvfp4e2m1bnosr"
        self.q_backward_input = "nvfp4e2m1b"
        self.q_backward_weight = "nvfp4e2m1b"
        self.q_backward_outputgrad = "nvfp4e2m1b"
        self.enable_backward_svd = enable_backward_svd
        self.backward_lowrank_svd = backward_lowrank_svd
        self.backward_lowrank_niter = 2
        self.enable_activation_svd = enable_activation_svd
        self.activation_lowrank_svd = activation_lowrank_svd
        self.activation_lowrank_niter = 0
        self.activation_broadcast_dim = 0
        self.backward_broadcast_dim = -1
        self.enable_nv_recipe = enable_nv_recipe
        self.hadamard_workspace_mb = hadamard_workspace_mb
        self.hadamard_tile_size = hadamard_tile_size
        self.hadamard_backend = hadamard_backend
        self.gradacc_broadcast = False
        self.gradacc_broadcast_steps = 1
        self.forward_svd_warmup_steps = 50      # split() is called by the patcher, not the constructor
        self.forward_svd_rank = forward_svd_rank
        self.tp_simulation = False
        self.tp_parts = 4
        self.metis_mode = metis_mode
        self.cache_quantized_weight = cache_quantized_weight
        self.compile_qdq = compile_qdq

    @classmethod
    def direct_fp4(cls, forward_svd_rank: int = 64, cache_quantized_weight: bool = True) -> "MetisArgs":
        """Low-rank-residual weights with direct NVFP4 activations and gradients -- the configuration
        the fused kernels accelerate (the reference's `qat_fp4` preset, scripts/grpo/run_experiment.sh)."""
        return cls(enable_forward_svd=True, enable_activation_svd=False, enable_backward_svd=False,
                   forward_svd_rank=forward_svd_rank, cache_quantized_weight=cache_quantized_weight)


def replace_linear_with_metis(model, dtype, metis_args, target_modules=None, compute_dtype=None):
    """Replace targeted nn.Linear modules by BitLinear in place (reference grpo.py:119-196)."""
    if target_modules is None:
        target_modules = list(DEFAULT_TARGETS)
    if compute_dtype is None:
        compute_dtype = torch.float32
    activation_groups = {}
    for name, module in list(model.named_modules()):
        leaf = name.split(".")[-1]
        if leaf not in target_modules or not isinstance(module, torch.nn.Linear):
            continue
        if "." in name:
            parent = model.get_submodule(".".join(name.split(".")[:-1]))
        else:
            parent = model
        if module.weight.numel() == 0:
            raise NotImplementedError("ZeRO-3 partitioned parameters must be gathered before patching")
        args = metis_args
        new_layer = BitLinear(in_features=module.in_features, out_features=module.out_features, args=args,
                              bias=module.bias is not None, dtype=dtype, compute_dtype=compute_dtype)
        new_layer.to(module.weight.device)
        with torch.no_grad():
            new_layer.warmup_linear.weight.copy_(module.weight)
            if module.bias is not None:
                new_layer.warmup_linear.bias.copy_(module.bias)
        new_layer.layer_name = name
        prefix = name.rsplit(".", 1)[0] if "." in name else ""
        if leaf in {"q_proj", "k_proj", "v_proj"}:
            group_name = f"{prefix}.qkv"
        elif leaf in {"gate_proj", "up_proj"}:
            group_name = f"{prefix}.gate_up"
        else:
            group_name = None
        if group_name is not None:
            new_layer.activation_group = activation_groups.setdefault(
                group_name, {"name": group_name, "mean_cache": {}, "input_ref": None, "quantized_input": None, "members": []})
            new_layer.activation_group["members"].append(new_layer)
        if metis_args.enable_forward_svd:
            new_layer.split()
        setattr(parent, leaf, new_layer)
    return model


def replace_model_with_metis(model, metis_args=None, fuse_norms: bool = False):
    """bf16 storage and compute, default targets (reference grpo.py:199-215).  fuse_norms additionally
    replaces the RMSNorm in front of every q/k/v and gate/up group by the fused norm+quant module."""
    if metis_args is None:
        metis_args = MetisArgs()
    model = replace_linear_with_metis(model=model, dtype=torch.bfloat16, metis_args=metis_args,
                                      target_modules=list(DEFAULT_TARGETS), compute_dtype=torch.bfloat16)
    if fuse_norms:
        from .norm import fuse_rmsnorm_into_groups
        fuse_rmsnorm_into_groups(model)
    return model
