"""Rotary position encoding with optional llama3 frequency scaling
(tinyserve_llm/model/llama.py:107-128,139-161).

The table [max_position, head_dim] = [cos | sin] is computed once, on the CPU, in 32-bit, with the
operations and operand order of the reference, and uploaded; mixers rotate with it inside their
own kernels (pairing i with i + head_dim/2, llama.py:131-136).
"""

from __future__ import annotations

import math

import torch

from tinyserve_llm_amd.parts.base import PositionEncoding, register


def inverse_frequencies(head_dim: int, theta: float, scaling: dict | None, max_position: int) -> torch.Tensor:
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float) / head_dim))
    if scaling is None:
        return inv_freq
    factor, lo, hi = scaling["factor"], scaling["low_freq_factor"], scaling["high_freq_factor"]
    old_len = scaling.get("original_max_position_embeddings", max_position)
    wavelen = 2 * math.pi / inv_freq
    slowed = torch.where(wavelen > old_len / lo, inv_freq / factor, inv_freq)
    smooth = (old_len / wavelen - lo) / (hi - lo)
    blended = (1 - smooth) * slowed / factor + smooth * slowed
    medium = ~(wavelen < old_len / hi) * ~(wavelen > old_len / lo)
    return torch.where(medium, blended, slowed)


@register("position_encoding", "rope")
class Rope(PositionEncoding):
    graph_safe = True

    def __init__(self, head_dim: int, max_position: int, theta: float, scaling: dict | None = None,
                 rotary_dim: int | None = None) -> None:
        """`rotary_dim` (even, up to head_dim; default: all of it): the leading dimensions of a head
        that turn, dimension j with j + rotary_dim / 2; the table is that wide and the rest of a head
        passes unchanged (the Llama models turn whole heads)."""
        rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if rotary_dim % 2 or not 2 <= rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {rotary_dim}: an even number from 2 to head_dim {head_dim}")
        self.head_dim = head_dim
        self.rotary_dim = rotary_dim
        self.max_position = max_position
        self.theta = theta
        self.scaling = scaling
        self.inv_freq = inverse_frequencies(rotary_dim, theta, scaling, max_position)
        self.cos_sin: torch.Tensor | None = None

    def host_table(self) -> torch.Tensor:
        t = torch.arange(self.max_position, dtype=torch.float)
        freqs = torch.einsum("i,j -> ij", t, self.inv_freq)
        return torch.cat((freqs.cos(), freqs.sin()), dim=-1).contiguous()

    def prepare(self, device: torch.device) -> None:
        self.cos_sin = self.host_table().to(device)

    def rotary_table(self) -> torch.Tensor | None:
        return self.cos_sin
