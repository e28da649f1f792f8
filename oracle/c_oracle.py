"""ctypes access to the C restatement in metis_oracle.c (TEST INFRASTRUCTURE).

Inputs and outputs are torch CPU tensors; bf16 tensors are passed as their 16-bit patterns.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmetis_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libmetis_oracle.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
        L.metis_oracle_nvfp4_pack.argtypes = [vp, i64, i64, i64, i32, vp, vp, vp, vp, vp]
        L.metis_oracle_nvfp4_pack.restype = i32
        L.metis_oracle_nvfp4_dequant.argtypes = [vp, vp, f32, i64, i64, i32, vp, vp]
        L.metis_oracle_nvfp4_dequant.restype = i32
        L.metis_oracle_rmsnorm.argtypes = [vp, vp, f32, i64, i64, vp]
        L.metis_oracle_rmsnorm.restype = i32
        L.metis_oracle_rmsnorm_nvfp4.argtypes = [vp, vp, f32, i64, i64, i32, vp, vp, vp, vp]
        L.metis_oracle_rmsnorm_nvfp4.restype = i32
        L.metis_oracle_e4m3_encode.argtypes = [f32]
        L.metis_oracle_e4m3_encode.restype = ctypes.c_uint8
        L.metis_oracle_e4m3_decode.argtypes = [ctypes.c_uint8]
        L.metis_oracle_e4m3_decode.restype = f32
        L.metis_oracle_f32_to_bf16.argtypes = [f32]
        L.metis_oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.metis_oracle_threads.restype = i32
        L.metis_oracle_lowrank_product.argtypes = [vp, vp, i64, i64, i64, vp]
        L.metis_oracle_lowrank_product.restype = i32
        _lib = L
    return _lib


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def nvfp4_pack(x_bf16: torch.Tensor, mode: int, noise: torch.Tensor | None = None):
    """-> (codes u8 [R,C/2], scales u8 [R,C/16], unit float, n_clamped).  mode 2: binary32 arithmetic on a
    float32 tensor whose values need not be bf16 values."""
    assert x_bf16.is_contiguous() and x_bf16.dtype == (torch.float32 if mode == 2 else torch.bfloat16)
    x2 = x_bf16.reshape(-1, x_bf16.shape[-1])
    rows, cols = x2.shape
    if cols % 16:
        raise ValueError(f"NVFP4 block shape (1, 16) does not divide tensor shape {tuple(x_bf16.shape)}")
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8)
    scales = torch.empty(rows, cols // 16, dtype=torch.uint8)
    unit = torch.zeros(1, dtype=torch.float32)
    ncl = torch.zeros(1, dtype=torch.int64)
    if noise is not None:
        want = torch.bfloat16 if mode == 1 else torch.float32
        assert noise.dtype == want and noise.is_contiguous() and noise.numel() == x2.numel()
    rc = lib().metis_oracle_nvfp4_pack(_p(x2), rows, cols, cols, mode, _p(noise), _p(codes),
                                       _p(scales), _p(unit), _p(ncl))
    assert rc == 0
    return codes, scales, float(unit), int(ncl)


def nvfp4_dequant(codes, scales, unit: float, mode: int):
    """-> (bf16 tensor, f32 tensor) of shape [R, C]."""
    rows, half = codes.shape
    cols = half * 2
    ob = torch.empty(rows, cols, dtype=torch.bfloat16)
    of = torch.empty(rows, cols, dtype=torch.float32)
    rc = lib().metis_oracle_nvfp4_dequant(_p(codes), _p(scales), unit, rows, cols, mode, _p(ob), _p(of))
    assert rc == 0
    return ob, of


def rmsnorm_nvfp4(x_bf16, gamma_bf16, eps: float, mode: int):
    rows, cols = x_bf16.reshape(-1, x_bf16.shape[-1]).shape
    normed = torch.empty(rows, cols, dtype=torch.bfloat16)
    codes = torch.empty(rows, cols // 2, dtype=torch.uint8)
    scales = torch.empty(rows, cols // 16, dtype=torch.uint8)
    unit = torch.zeros(1, dtype=torch.float32)
    rc = lib().metis_oracle_rmsnorm_nvfp4(_p(x_bf16.contiguous()), _p(gamma_bf16.contiguous()), eps, rows,
                                          cols, mode, _p(normed), _p(codes), _p(scales), _p(unit))
    assert rc == 0
    return normed, codes, scales, float(unit)


def e4m3_encode(v: float) -> int:
    return int(lib().metis_oracle_e4m3_encode(v))


def e4m3_decode(b: int) -> float:
    return float(lib().metis_oracle_e4m3_decode(b))


def threads() -> int:
    return int(lib().metis_oracle_threads())


def lowrank_product(us: torch.Tensor, vt: torch.Tensor) -> torch.Tensor:
    """us [rows, r] @ vt [r, cols] in binary32 with the additions in the order k = 0 .. r-1, one fused multiply-add each."""
    assert us.dtype == torch.float32 and vt.dtype == torch.float32 and us.shape[1] == vt.shape[0]
    us, vt = us.contiguous(), vt.contiguous()
    ker = torch.empty(us.shape[0], vt.shape[1], dtype=torch.float32)
    rc = lib().metis_oracle_lowrank_product(_p(us), _p(vt), us.shape[0], vt.shape[1], us.shape[1], _p(ker))
    assert rc == 0
    return ker
