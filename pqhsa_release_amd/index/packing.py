"""4-bit code packing helpers with the reference's signatures (pq_hsa/index/packing.py:6-60).

The device index stores one little-endian 32-bit word per key, nibble ``m`` = code of subspace
``m``; its byte view is exactly the reference's ``[N, 4]`` uint8 layout (low nibble = even
subspace, high nibble = odd).  These helpers convert between ``[N, M]`` code matrices and that
byte layout for inspection, checkpoints and tests; the kernels never unpack through them.
"""

from __future__ import annotations

import torch


def pack_4bit_codes(codes: torch.Tensor) -> torch.Tensor:
    if codes.ndim != 2:
        raise ValueError(f"codes must be [N, M], got {tuple(codes.shape)}")
    if codes.numel() > 0 and (codes.min() < 0 or codes.max() > 15):
        raise ValueError("4-bit packing requires codes in [0, 15]")
    c = codes.to(torch.uint8)
    if c.shape[1] % 2 == 1:
        c = torch.cat([c, torch.zeros(c.shape[0], 1, dtype=torch.uint8, device=c.device)], dim=1)
    return (c[:, 0::2] & 0x0F) | (c[:, 1::2] << 4)


def unpack_4bit_codes(packed: torch.Tensor, num_subspaces: int) -> torch.Tensor:
    if packed.ndim != 2:
        raise ValueError(f"packed codes must be [N, ceil(M/2)], got {tuple(packed.shape)}")
    if num_subspaces <= 0:
        raise ValueError("num_subspaces must be positive")
    width = (num_subspaces + 1) // 2
    if packed.shape[1] != width:
        raise ValueError(f"packed width must be {width} for {num_subspaces} subspaces, got {packed.shape[1]}")
    out = torch.empty(packed.shape[0], num_subspaces, dtype=torch.long, device=packed.device)
    out[:, 0::2] = (packed[:, :width] & 0x0F).long()
    if num_subspaces > 1:
        out[:, 1::2] = (packed[:, : num_subspaces // 2] >> 4).long()
    return out
