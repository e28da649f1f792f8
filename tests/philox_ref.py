"""Philox4x32-10 in numpy (Salmon, Moraes, Dror, Shaw, SC'11) for checking the device stream."""
import numpy as np

M0, M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
W0, W1 = 0x9E3779B9, 0xBB67AE85
MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10(ctr: np.ndarray, key: np.ndarray) -> np.ndarray:
    """ctr [n,4] uint32, key [n,2] or [2] uint32 -> [n,4] uint32."""
    c = ctr.astype(np.uint64)
    k = np.broadcast_to(key.astype(np.uint64), (c.shape[0], 2)).copy()
    for _ in range(10):
        p0 = M0 * c[:, 0]
        p1 = M1 * c[:, 2]
        hi0, lo0 = p0 >> np.uint64(32), p0 & MASK
        hi1, lo1 = p1 >> np.uint64(32), p1 & MASK
        c = np.stack([hi1 ^ c[:, 1] ^ k[:, 0], lo1, hi0 ^ c[:, 3] ^ k[:, 1], lo0], axis=1)
        k[:, 0] = (k[:, 0] + np.uint64(W0)) & MASK
        k[:, 1] = (k[:, 1] + np.uint64(W1)) & MASK
    return c.astype(np.uint32)


def uniform_for_elements(n_elems: int, seed: int, offset: int, bf16: bool) -> np.ndarray:
    """Uniform draws the kernels assign to packed-orientation element indices 0..n-1.

    Element e uses word e % 4 of the draw with 64-bit counter offset + e // 4 and 64-bit key seed.
    float32: (word >> 8) * 2^-24; bf16: (word >> 24) * 2^-8.
    """
    n4 = (n_elems + 3) // 4
    cnt = np.uint64(offset) + np.arange(n4, dtype=np.uint64)
    ctr = np.zeros((n4, 4), dtype=np.uint32)
    ctr[:, 0] = (cnt & MASK).astype(np.uint32)
    ctr[:, 1] = (cnt >> np.uint64(32)).astype(np.uint32)
    key = np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint32)
    words = philox4x32_10(ctr, key).reshape(-1)[:n_elems]
    if bf16:
        return (words >> np.uint32(24)).astype(np.float32) * np.float32(2.0 ** -8)
    return (words >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24)
