"""Shared helpers for the parity tests."""
import numpy as np
import torch


def bf16_from_bits(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def t(a: np.ndarray) -> torch.Tensor:
    """Golden array -> tensor (uint16 arrays are bf16 bit patterns)."""
    if a.dtype == np.uint16:
        return bf16_from_bits(a)
    return torch.from_numpy(a.copy())


def same_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Bit equality except that +0 and -0 compare equal (torch.equal semantics)."""
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a, b)


def rel_fro(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


def synthetic_activation(seed: int, rows: int, cols: int, outliers: int | None = None) -> torch.Tensor:
    """N(0,1) bf16 with 0.1 % of columns scaled x20 (outlier channels)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g)
    n_out = max(1, round(cols * 0.001)) if outliers is None else outliers
    idx = torch.randperm(cols, generator=g)[:n_out]
    x[:, idx] *= 20.0
    return x.bfloat16()
