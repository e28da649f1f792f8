"""ctypes binding of libmetis_hip.so (the C ABI declared in include/metis_hip.h).

The product path has no CPU or PyTorch fallback: if the shared library is missing or a call
returns an error code, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmetis_hip.so")

OK, E_ARG, E_SHAPE, E_WORKSPACE, E_LAUNCH, E_DEVICE, E_TOO_LARGE = 0, -1, -2, -3, -4, -5, -6
class LinearMember(ctypes.Structure):
    """metis_linear_member of include/metis_hip.h: one weight matrix of a grouped GEMM."""
    _fields_ = [("b_codes", ctypes.c_void_p), ("b_scales", ctypes.c_void_p), ("b_unit", ctypes.c_void_p),
                ("t", ctypes.c_void_p), ("u", ctypes.c_void_p), ("r", ctypes.c_int64), ("bias", ctypes.c_void_p),
                ("out", ctypes.c_void_p), ("N", ctypes.c_int64), ("bias_is_f32", ctypes.c_int64), ("ldt", ctypes.c_int64),
                ("b_decode", ctypes.c_void_p)]


MODE_P32, MODE_PB16 = 0, 1
MODE_P32_F32 = 2      # quantizer entry points only: binary32 arithmetic on a binary32 tensor
DTYPE_BF16, DTYPE_F32 = 0, 1

_vp, _i64, _i32, _u64, _f32, _sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_uint64,
                                    ctypes.c_float, ctypes.c_size_t)

# name -> (restype, argtypes); must list every symbol include/metis_hip.h declares
SIGNATURES = {
    "metis_version": (_i32, []),
    "metis_error_string": (ctypes.c_char_p, [_i32]),
    "metis_nvfp4_workspace_bytes": (_sz, [_i64, _i64]),
    "metis_nvfp4_quant_row": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_quant_dequant_row": (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_quant_row_static": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _vp, _vp, _vp]),
    "metis_nvfp4_quant_row_resident": (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _sz, ctypes.c_uint32, _vp]),
    "metis_nvfp4_quant_col": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_quant_sr_row": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _u64, _u64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_quant_sr_col": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _u64, _u64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_get_scalar": (_i32, [_vp, _i64, _i64, _i32, _vp, _vp]),
    "metis_nvfp4_quant_values": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _vp, _u64, _u64, _vp, _vp]),
    "metis_nvfp4_rquant": (_i32, [_vp, _vp, _i64, _i64, _i32, _vp, _vp, _vp]),
    "metis_nvfp4_dequant": (_i32, [_vp, _vp, _vp, _i64, _i64, _i32, _vp, _i32, _vp]),
    "metis_rmsnorm_nvfp4_quant": (_i32, [_vp, _vp, _f32, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_linear_member_size": (_sz, []),
    "metis_nvfp4_decode_weight_bytes": (_sz, [_i64, _i64]),
    "metis_nvfp4_decode_weight": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp]),
    "metis_rmsnorm_colmean_workspace_bytes": (_sz, [_i64, _i64]),
    "metis_rmsnorm_colmean": (_i32, [_vp, _vp, _f32, _i64, _i64, _vp, _vp, _i32, _vp, _i64, _vp, _vp, _sz, _vp]),
    "metis_linear_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _i32, _vp]),
    "metis_nvfp4_expand_f16": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp]),
    "metis_linear_fwd_expanded": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _i32, _vp]),
    "metis_nvfp4_expand_tiled_bytes": (_sz, [_i64, _i64]),
    "metis_nvfp4_expand_tiled": (_i32, [_vp, _vp, _vp, _i64, _i64, _i32, _vp, _vp]),
    "metis_linear_tiled_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32]),
    "metis_dense_expand_tiled": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _i32, _vp, _vp]),
    "metis_hadamard16": (_i32, [_vp, _i64, _i64, _i64, _i32, _i32, ctypes.c_uint32, _vp, _i64, _vp]),
    "metis_nvfp4_quant_row_rht": (_i32, [_vp, _i64, _i64, _i64, _i32, ctypes.c_uint32, _i32, _u64, _u64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_expand_tiled_rht": (_i32, [_vp, _vp, _vp, _i64, _i64, _i32, ctypes.c_uint32, _i32, _i32, _vp, _vp]),
    "metis_nvfp4_quant_sr_both": (_i32, [_vp, _i64, _i64, _i64, _i32, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64, _vp, _vp, _vp, _vp, _vp,
                                  _vp, _vp, _sz, _vp]),
    "metis_nvfp4_deferred_bytes": (_sz, [_i64, _i64]),
    "metis_nvfp4_quant_row_deferred": (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _vp, _sz, _vp]),
    "metis_rmsnorm_nvfp4_quant_deferred": (_i32, [_vp, _vp, _f32, _i64, _i64, _i32, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_deferred_scales": (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _vp]),
    "metis_nvfp4_expand_tiled_deferred": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _vp, _vp, _vp, _vp]),
    "metis_nvfp4_expand_tiled_centered": (_i32, [_vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp]),
    "metis_linear_fwd_tiled": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _i32, _vp, _i32, _i32, _vp, _sz, _vp]),
    "metis_linear_dgrad": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i32, _vp]),
    "metis_linear_wgrad": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i32, _vp]),
    "metis_nvfp4_quant_centered": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _i32, _i32, _vp, _u64, _u64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_quant_row_decode": (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_rmsnorm_nvfp4_quant_decode": (_i32, [_vp, _vp, _f32, _i64, _i64, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_quant_lowrank_residual": (_i32, [_vp, _i32, _vp, _vp, _i64, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_matvec_affine": (_i32, [_vp, _vp, _vp, _i64, _i64, _vp, _f32, _vp, _f32, _vp, _vp]),
    "metis_rank_one_operands": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp]),
    "metis_column_mean_workspace_bytes": (_sz, [_i64]),
    "metis_column_mean": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _i32, _vp, _sz, _vp]),
    "metis_column_mean_running": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _i64, _vp, _vp, _i32, _vp, _sz, _vp]),
    "metis_column_sum": (_i32, [_vp, _i64, _i64, _i64, _i32, _vp, _i32, _vp, _sz, _vp]),
    "metis_nvfp4_matvec": (_i32, [_vp, _vp, _vp, _i64, _i64, _vp, _f32, _vp, _vp, _i64, _i32, _vp]),
    "metis_linear_fwd_f32bias": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _i32, _vp, _sz, _vp]),
    "metis_lowrank_project_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "metis_lowrank_project": (_i32, [_vp, _i64, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_lowrank_project_rows": (_i32, [_vp, _i64, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    "metis_lowrank_scale_grad": (_i32, [_vp, _vp, _i64, _i64, _vp, _i32, _vp]),
    "metis_lowrank_project_rows_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "metis_lowrank_project_rows_ws": (_i32, [_vp, _i64, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "metis_nvfp4_quant_project_deferred": (_i32, [_vp, _i64, _i64, _i32, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _sz, _vp, _sz, _vp]),
    "metis_lowrank_tokens_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "metis_lowrank_contract_tokens": (_i32, [_vp, _i64, _vp, _i64, _i64, _i64, _vp, _i32, _i32, _vp, _sz, _vp]),
    "metis_linear_fwd_grouped": (_i32, [_vp, _vp, _vp, _i64, _i64, _vp, _i32, _i32, _vp, _sz, _vp]),
    "metis_linear_fwd_grouped_bf16": (_i32, [_vp, _vp, _vp, _i64, _i64, _vp, _i32, _i32, _vp, _sz, _vp]),
    "metis_nvfp4_decode_operand_bytes": (_sz, [_i64, _i64]),
    "metis_nvfp4_decode_operand": (_i32, [_vp, _vp, _vp, _i64, _i64, _i32, _vp, _vp, _vp]),
    "metis_nvfp4_decode_operand_deferred": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _vp, _vp, _vp, _vp]),
    "metis_nvfp4_decode_operand_rht": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, ctypes.c_uint32, _vp, _vp]),
    "metis_decode_quant_project_deferred": (_i32, [_vp, _i64, _i64, _i32, _vp, _vp, _sz, _vp, _i64, _vp, _sz, _vp]),
    "metis_decode_prepare_deferred": (_i32, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _sz, _vp, _vp, _i64, _i64, _i32, _i32, _vp, _vp, _vp, _i32,
                                             ctypes.c_uint32, _vp]),
    "metis_linear_fwd_grouped_operand": (_i32, [_vp, _vp, _i64, _i64, _vp, _i32, _i32, _i32, _vp, _sz, _vp]),
    "metis_linear_grouped_workspace_bytes": (_sz, [_i64, _i64, _vp, _i32]),
    "metis_linear_fwd_grouped_centered": (_i32, [_vp, _vp, _vp, _i64, _i64, _vp, _i32, _i32, _vp, _vp, _sz, _vp]),
    "metis_linear_grouped_centered_supported": (_i32, [_i64, _i64, _vp, _i32, _i32]),
    "metis_linear_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "metis_linear_fwd_ws": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _i32, _vp, _sz, _vp]),
    "metis_linear_dgrad_ws": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i32, _vp, _sz, _vp]),
    "metis_linear_wgrad_ws": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i32, _vp, _sz, _vp]),
}

_lib = None


class MetisHipError(RuntimeError):
    pass


def load():
    """Load the library once; raises MetisHipError if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MetisHipError(
                f"{LIB_PATH} not found: build it with `make -C fp4-post_amd/csrc` "
                "(or __graft_entry__.build()); there is no fallback path"
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        if lib.metis_linear_member_size() != ctypes.sizeof(LinearMember):
            raise MetisHipError(f"{LIB_PATH} was built from another revision of include/metis_hip.h: metis_linear_member is "
                                f"{lib.metis_linear_member_size()} bytes there, {ctypes.sizeof(LinearMember)} here; rebuild it")
        _lib = lib
    return _lib


def check(rc: int, what: str, shape=None):
    """Map a return code to the exception the reference raises for the same condition."""
    if rc == OK:
        return
    msg = load().metis_error_string(rc).decode()
    if rc == E_SHAPE:
        # quant.py:400-403 raises ValueError for a last dim that 16 does not divide
        raise ValueError(f"NVFP4 block shape (1, 16) does not divide tensor shape {tuple(shape) if shape is not None else '?'}")
    raise MetisHipError(f"{what}: {msg} (code {rc})")
