"""4-bit code packing helpers with the reference's signatures (pq_hsa/index/packing.py:6-60).

The device index stores one little-endian 32-bit word per key, nibble ``m`` = code of subspace
``m``; its byte view is exactly the reference's ``[N, ceil(M/2)]`` uint8 layout (low nibble =
even subspace, high nibble = odd, an odd M padded with a zero nibble).  These helpers convert
between ``[N, M]`` code matrices and that byte layout for inspection, checkpoints and tests;
the kernels never unpack through them.
"""

from __future__ import annotations

import torch

_NIBBLE = 0x0F


def _need_matrix(t: torch.Tensor, what: str) -> None:
    if t.ndim != 2:
        raise ValueError(f"{what}, got {tuple(t.shape)}")


def pack_4bit_codes(codes: torch.Tensor) -> torch.Tensor:
    """``[N, M]`` codes in 0..15 -> ``[N, ceil(M/2)]`` bytes."""
    _need_matrix(codes, "codes must be [N, M]")
    if codes.numel() and not bool(((codes >= 0) & (codes <= _NIBBLE)).all()):
        raise ValueError("4-bit packing requires codes in [0, 15]")
    rows, m = codes.shape
    pairs = torch.zeros(rows, (m + 1) // 2, 2, dtype=torch.uint8, device=codes.device)
    pairs.view(rows, -1)[:, :m] = codes.to(torch.uint8)          # (even, odd) side by side
    return pairs[..., 0] | (pairs[..., 1] << 4)


def unpack_4bit_codes(packed: torch.Tensor, num_subspaces: int) -> torch.Tensor:
    """``[N, ceil(M/2)]`` bytes -> ``[N, M]`` codes (int64, the reference's dtype)."""
    _need_matrix(packed, "packed codes must be [N, ceil(M/2)]")
    if num_subspaces <= 0:
        raise ValueError("num_subspaces must be positive")
    width = (num_subspaces + 1) // 2
    if packed.shape[1] != width:
        raise ValueError(f"packed width must be {width} for {num_subspaces} subspaces, got {packed.shape[1]}")
    both = torch.stack((packed & _NIBBLE, packed >> 4), dim=2)    # [N, width, (low, high)]
    return both.reshape(packed.shape[0], 2 * width)[:, :num_subspaces].long()
