"""Rotary position embedding backed by the HIP kernel (interface of nanovllmx/layers/rotary_embedding.py:27-102)."""
from __future__ import annotations

import torch
from torch import nn

from .. import ops


def build_cos_sin_cache(rotary_dim: int, max_position_embeddings: int, base: float) -> torch.Tensor:
    """fp32 (max_pos, rotary_dim) = [cos(t * f_j) | sin(t * f_j)], f_j = base^(-2j/rotary_dim)
    (rotary_embedding.py:52-71; built on the CPU in fp32 so that every rank holds identical bits)."""
    exponents = torch.arange(0, rotary_dim, 2, dtype=torch.float) / rotary_dim
    inv_freq = 1.0 / (base ** exponents)
    t = torch.arange(max_position_embeddings, dtype=torch.float)
    angles = torch.einsum("i,j -> ij", t, inv_freq)
    return torch.cat((angles.cos(), angles.sin()), dim=-1)


class RotaryEmbedding(nn.Module):
    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: float,
                 dtype: torch.dtype | None = None) -> None:
        super().__init__()
        if head_size != 128 or rotary_dim != head_size:
            raise NotImplementedError("the HIP rotary kernel is built for rotary_dim == head_size == 128")
        self.head_size, self.rotary_dim = head_size, rotary_dim
        self.max_position_embeddings, self.base, self.dtype = max_position_embeddings, base, dtype
        cache = build_cos_sin_cache(rotary_dim, max_position_embeddings, base)
        if dtype is not None:   # the kernel reads fp32; a narrower table is widened again, rounding kept
            cache = cache.to(dtype).to(torch.float32)
        self.register_buffer("cos_sin_cache", cache, persistent=False)

    def forward(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                offsets: torch.Tensor | None = None):
        """Pairs element j with j + D/2 of every head and writes the rotated pair to (2j, 2j+1)
        (rotary_embedding.py:19-24); q.k is unchanged by the common permutation."""
        if offsets is not None:
            positions = positions + offsets
        if self.cos_sin_cache.dtype != torch.float32:   # model.to(bf16) casts buffers too
            self.cos_sin_cache = self.cos_sin_cache.float()
        return ops.rope(positions, query, key, self.cos_sin_cache, self.head_size)


def rotary_frequencies(dims: int, base: float, scaling: dict | None = None):
    """(frequencies, magnitude) of a rotation of `dims` dimensions in dims / 2 pairs: f_i = base^(-2i / dims), float64 (dims / 2).
    `scaling` stretches the slow pairs, in one of two ways that its keys tell apart.
    {factor, original, fast, slow} (YaRN: B. Peng, J. Quesnelle, H. Fan, E. Shippole, "YaRN: Efficient Context Window Extension of
    Large Language Models"): a pair that completes `turns` turns over `original` positions has index d(turns) = dims ln(original /
    (2 pi turns)) / (2 ln base); between lo = floor(d(fast)) and hi = ceil(d(slow)) (clipped to the table) a ramp goes from 0 to 1,
    a frequency becomes f / factor where the ramp is 1 and stays f where it is 0, and cos and sin are multiplied by
    0.1 ln(factor) + 1.
    {factor, original, low, high} (bands of wavelength, as the Llama 3.1 models scale theirs): with wavelength L = 2 pi / f, f stays
    where L < original / high, becomes f / factor where L > original / low, and between the two is the blend (1 - s) f / factor + s f
    with s = (original / L - low) / (high - low); the magnitude stays 1."""
    import math

    idx = torch.arange(dims // 2, dtype=torch.float64)
    freq = float(base) ** (-2.0 * idx / dims)
    if not scaling:
        return freq, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])
    if "low" in scaling or "high" in scaling:
        low, high = float(scaling["low"]), float(scaling["high"])
        wave = 2.0 * math.pi / freq
        s = ((original / wave - low) / (high - low)) if high != low else torch.zeros_like(freq)
        blend = (1.0 - s) * freq / factor + s * freq
        out = torch.where(wave < original / high, freq, torch.where(wave > original / low, freq / factor, blend))
        return out, 1.0

    def index_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

    lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
    ramp = ((idx - lo) / max(hi - lo, 0.001)).clamp_(0.0, 1.0)
    return freq / factor * ramp + freq * (1.0 - ramp), 0.1 * math.log(factor) + 1.0
