"""metis_hip: the Metis NVFP4 hot path on MI355X (gfx950) behind the reference's Python interface.

    from metis_hip import quant_func, LinearLowbitFunction, LinearLowbit, BitLinear
    from metis_hip import MetisArgs, replace_linear_with_metis, replace_model_with_metis

Compute goes through libmetis_hip.so (hand-written HIP kernels, C ABI in include/metis_hip.h).
"""
from . import ops
from ._lib import MODE_P32, MODE_PB16, MetisHipError
from .bitlinear import BitLinear, LinearLowbit, LinearLowbitFunction
from .norm import FusedRMSNormQuant, fuse_rmsnorm_into_groups
from .ops import CenteredNVFP4, PackedNVFP4
from .patch import MetisArgs, replace_linear_with_metis, replace_model_with_metis
from .quant import (BlockQuantFunc, Cast2Fp32, Cast2NVFp4e2m1Block, Cast2NVFp4e2m1BlockNOSR, QuantFunc,
                    nvfp4_nosr_qdq_compile_status, quant_func)

__all__ = ["FusedRMSNormQuant", "fuse_rmsnorm_into_groups", "nvfp4_nosr_qdq_compile_status", "ops", "PackedNVFP4", "CenteredNVFP4", "MODE_P32", "MODE_PB16", "MetisHipError", "quant_func", "QuantFunc", "BlockQuantFunc",
           "Cast2Fp32", "Cast2NVFp4e2m1Block", "Cast2NVFp4e2m1BlockNOSR", "LinearLowbitFunction", "LinearLowbit",
           "BitLinear", "MetisArgs", "replace_linear_with_metis", "replace_model_with_metis"]
