"""Rotary position encoding: float tables of cos and sin per position.

inv_freq[i] = 1 / theta^(2i/r) over the r rotated elements of a head; optional "llama3" rescale of the
low frequencies; angle[p, i] = p * inv_freq[i] in float (pagedllm/model/llama.py:86-128).  The tables
hold r/2 columns (the reference's cat[freqs, freqs] repeats them).  The rotation itself is done by the
mixer's kernel, fused with the cache write; this part says how: ``rotary_dim`` = r (default: the whole
head, as in the reference) and ``interleaved`` (pairs (2i, 2i+1) instead of the reference's (i, i + r/2)).
"""

from __future__ import annotations

import math

import torch

from .base import PositionEncoding
from .registry import BuildEnv, register_position_encoding


def llama3_rescale(inv_freq: torch.Tensor, factor: float, low_freq_factor: float, high_freq_factor: float,
                   original_max_position_embeddings: int) -> torch.Tensor:
    """Waves longer than orig/low are slowed by `factor`, shorter than orig/high stay, those in
    between are blended.  The formula is taken from pagedllm/model/llama.py:86-97 as it stands there
    (it is the published llama3 rule; there is one way to write it)."""
    wavelen = 2 * math.pi / inv_freq
    low_wl = original_max_position_embeddings / low_freq_factor
    high_wl = original_max_position_embeddings / high_freq_factor
    smooth = (original_max_position_embeddings / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
    blended = (1 - smooth) * inv_freq / factor + smooth * inv_freq
    out = torch.where(wavelen > low_wl, inv_freq / factor, inv_freq)
    middle = (wavelen <= low_wl) & (wavelen >= high_wl)
    return torch.where(middle, blended, out)


class RotaryEncoding(PositionEncoding):
    def __init__(self, params: dict, env: BuildEnv):
        self.head_dim = int(params["head_dim"])
        self.theta = float(params["theta"])
        self.scaling = params.get("scaling")
        self.rotary_dim = int(params.get("rotary_dim") or self.head_dim)
        self.interleaved = bool(params.get("interleaved", False))
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary encoding turns pairs of elements: the rotated width must be even and at most the head "
                             f"size {self.head_dim}, got {self.rotary_dim}")
        if self.scaling:
            kind = self.scaling.get("rope_type", self.scaling.get("type"))
            if kind != "llama3":
                raise NotImplementedError(f"rope_type={kind!r} not supported (default and llama3 only)")
        self.device = env.device
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None
        self.num_positions = 0

    def inverse_frequencies(self) -> torch.Tensor:
        d = self.rotary_dim
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        if self.scaling:
            s = self.scaling
            inv_freq = llama3_rescale(inv_freq, float(s["factor"]), float(s.get("low_freq_factor", 1.0)),
                                      float(s.get("high_freq_factor", 4.0)),
                                      int(s.get("original_max_position_embeddings", 8192)))
        return inv_freq

    def prepare(self, max_positions: int) -> None:
        if max_positions <= self.num_positions:
            return
        t = torch.arange(max_positions, dtype=torch.float32)
        angles = torch.outer(t, self.inverse_frequencies())          # [P, rotary_dim/2], float
        self.cos = angles.cos().to(self.device).contiguous()
        self.sin = angles.sin().to(self.device).contiguous()
        self.num_positions = max_positions


register_position_encoding("rotary", RotaryEncoding)
