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


def untile(buf, rows, cols, dtype):
    """Row-major [rows, cols] view of a tiled GEMM operand (tiles of 16 rows x 32 k, 1 KiB each, tile (rb, kb) at
    byte ((rb * cols / 32) + kb) * 1024, row q's 8-element chunk c in slot q * 4 + (c ^ swz(q)))."""
    import torch
    tiles = buf.view(dtype).reshape(-1, cols // 32, 16, 4, 8)
    q = torch.arange(16, device=buf.device)
    swz = ((q >> 2) & 1) | ((((q >> 1) ^ (q >> 3)) & 1) << 1)
    slot = torch.arange(4, device=buf.device)[None, :] ^ swz[:, None]
    unswz = torch.gather(tiles, 3, slot[None, None, :, :, None].expand(tiles.shape[0], tiles.shape[1], 16, 4, 8))
    return unswz.permute(0, 2, 1, 3, 4).reshape(-1, cols)[:rows]


def from_decode_operand(buf, rows, cols, dtype):
    """Row-major [rows, cols] view of a decode-sized activation operand: piece ((row tile, iteration, m), lane) of 8
    elements holds k = 256 it + 128 (lane / 32) + 8 m .. of row 32 tile + lane % 32."""
    v = buf.view(dtype).reshape(-1, cols // 256, 16, 2, 32, 8)          # [tile, it, m, half, row, 8]
    return v.permute(0, 4, 1, 3, 2, 5).reshape(-1, cols)[:rows]
