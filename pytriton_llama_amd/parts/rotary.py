"""Rotary position encoding: the frequencies, and their application to q and k."""
from __future__ import annotations

import math
from typing import Optional

import torch

from .. import ops
from .base import Part, register_part


def default_inv_freq(theta: float, dim: int) -> torch.Tensor:
    """inv_freq_j = theta^(-2j/dim), float32
    (lite_llama/models/RotaryEmbedding.py:51)."""
    return 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.int64).float() / dim))


def llama3_inv_freq(theta: float, dim: int, factor: float, low_freq_factor: float,
                    high_freq_factor: float, original_max_position_embeddings: int) -> torch.Tensor:
    """The llama3 rescale of the frequencies by wavelength band
    (lite_llama/models/RotaryEmbedding.py:77-100): long waves divided by
    ``factor``, short waves kept, a linear blend between the two bands."""
    inv_freq = default_inv_freq(theta, dim)
    low_wavelen = original_max_position_embeddings / low_freq_factor
    high_wavelen = original_max_position_embeddings / high_freq_factor
    wavelen = 2 * math.pi / inv_freq
    scaled = torch.where(wavelen > low_wavelen, inv_freq / factor, inv_freq)
    smooth = (original_max_position_embeddings / wavelen - low_freq_factor) / (
        high_freq_factor - low_freq_factor)
    blended = (1 - smooth) * scaled / factor + smooth * scaled
    medium = ~(wavelen < high_wavelen) & ~(wavelen > low_wavelen)
    return torch.where(medium, blended, scaled)


@register_part("position", "rotary")
class RotaryEncoding(Part):
    """Rotate-half RoPE. ``rope_type`` "default" or "llama3" with its four numbers
    (lite_llama/models/RotaryEmbedding.py:103-106,133-136). The angle
    position * inv_freq and its sine and cosine are float32, as in
    RotaryEmbedding.py:200-220 (attention_scaling is 1.0 there, :48)."""
    kernel_libraries = ("rope",)

    def __init__(self, head_dim: int, theta: float, rope_type: str = "default",
                 factor: float = 1.0, low_freq_factor: float = 1.0, high_freq_factor: float = 1.0,
                 original_max_position_embeddings: int = 0):
        if head_dim % 2:
            raise ValueError(f"rotary pairs need an even head size, got {head_dim}")
        self.head_dim = int(head_dim)
        if rope_type == "default":
            inv = default_inv_freq(theta, head_dim)
        elif rope_type == "llama3":
            inv = llama3_inv_freq(theta, head_dim, factor, low_freq_factor, high_freq_factor,
                                  original_max_position_embeddings)
        else:
            raise ValueError(f"unknown rope_type {rope_type!r}")
        self.inv_freq_host = inv.float().contiguous()
        self.inv_freq: Optional[torch.Tensor] = None

    def load(self, tensors, dtype, device) -> None:
        self.inv_freq = self.inv_freq_host.to(device)

    def rotary_inv_freq(self) -> Optional[torch.Tensor]:
        return self.inv_freq

    def apply(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor) -> None:
        """Rotate q and k ([T, heads, D] views of one buffer) in place."""
        ops.rope_store(q, k, k, positions, self.inv_freq, None, None, None, 1, k_in_place=True)
