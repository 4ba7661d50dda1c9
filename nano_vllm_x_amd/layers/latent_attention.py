"""Latent attention: keys and values of every head are linear maps of one cached vector per token."""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from .rotary_embedding import rotary_frequencies


class LatentAttention(nn.Module):
    """q = W_uq RMSnorm(W_dq h), c = RMSnorm(W_dkv h) (both norms with a plain weight); per head k = W_uk c, v = W_uv c,
    softmax(scale * q . k) over the causal prefix, the head's output times sigmoid(W_g h)_head, then W_o.  No positions.

    The cache holds c alone (kv_rank values per token).  The kernel attends over the cached latents directly: the key map is
    folded into the query (q~ = W_uk^T q, per head) and the value map is applied to the weighted sum of latents, which is
    the same function and reads kv_rank instead of heads * (dim + vdim) values per key.  The three projections of h (query
    latent, key/value latent, gates) are one matrix product."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, q_rank: int, kv_rank: int, scale: float, eps: float, layer_id: int):
        super().__init__()
        self.heads, self.dim, self.vdim, self.q_rank, self.kv_rank = heads, dim, vdim, q_rank, kv_rank
        self.scale, self.eps, self.layer_id = scale, eps, layer_id
        self.down_proj = nn.Linear(width, q_rank + kv_rank + heads, bias=False)     # rows: dq | dkv | g
        self.q_norm = nn.Parameter(torch.ones(q_rank, dtype=torch.float32))
        self.kv_norm = nn.Parameter(torch.ones(kv_rank, dtype=torch.float32))
        self.uq_proj = nn.Linear(q_rank, heads * dim, bias=False)
        self.uk = nn.Parameter(torch.empty(heads, dim, kv_rank))       # W_uk, head by head
        self.uv = nn.Parameter(torch.empty(heads, vdim, kv_rank))      # W_uv, head by head
        self.o_proj = nn.Linear(heads * vdim, width, bias=False)

    def forward(self, h: torch.Tensor, md) -> torch.Tensor:
        t = h.shape[0]
        cache = md.cache.latent(self.layer_id)
        cq, gate = ops.latent_prep(self.down_proj(h), self.q_norm, self.kv_norm, self.eps, md.out_slots, cache, self.heads)
        q = self.uq_proj(cq).view(t, self.heads, self.dim).transpose(0, 1)              # (heads, T, dim)
        q_folded = torch.bmm(q, self.uk)                                                 # (heads, T, kv_rank)
        o = ops.latent_attn(q_folded, cache, md.kv_indices, md.kv_start, md.kv_len, md.layout, self.scale, gate=gate)
        v = torch.bmm(o, self.uv.transpose(1, 2))                                        # (heads, T, vdim)
        return self.o_proj(v.transpose(0, 1).reshape(t, self.heads * self.vdim))


class RotaryLatentAttention(nn.Module):
    """Latent attention with positions: q = W_q h, head by head [dim plain | rot rotated]; W_dkv h = [latent (kv_rank) | one key part
    (rot) that all heads share]; c = RMSnorm(latent) with a plain weight; per head k = [W_uk c | rotated key part], v = W_uv c;
    softmax(scale * q . k) over the causal prefix, the head's output times sigmoid(W_g h)_head, then W_o.  The rotated parts turn in
    neighbouring pairs by position * f_i (`rot` = {base, scaling}: rotary_frequencies over rot dimensions, cos and sin times its
    magnitude).

    The cache holds [c | rotated key part] per token and nothing per head.  The attention runs over those rows directly
    (ops.latent_attn): the key map is folded into the query, q~ = [W_uk^T q_plain | q_rotated], the value map applied to the weighted
    sum of rows -- both as ONE batched product each, with an identity block (zero block) for the rotated columns.  Rows are padded
    with zeros to a length the matrix-core kernel is built for.  The projections q | dkv | g are one matrix product."""

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, scale: float, eps: float, rot: dict, cache_name):
        super().__init__()
        if rot_dim % 2:
            raise ValueError("the rotated part of a head must be even")
        self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank = heads, dim, rot_dim, vdim, kv_rank
        self.scale, self.eps, self.cache_name = float(scale), eps, cache_name
        if rot_dim:
            freq, self.mag = rotary_frequencies(rot_dim, rot["base"], rot.get("scaling"))
            self.register_buffer("freq", freq.to(torch.float64), persistent=False)
        else:
            self.freq, self.mag = None, 1.0
        self.row = self.padded_row(kv_rank + rot_dim)
        hd = dim + rot_dim
        self.q_cols, self.kv_cols = heads * hd, kv_rank + rot_dim
        self.in_proj = nn.Linear(width, self.q_cols + self.kv_cols + heads, bias=False)      # rows: q | dkv | g
        self.kv_norm = nn.Parameter(torch.ones(kv_rank, dtype=torch.float32))
        # W_uk and W_uv head by head, widened to the cache row: the rotated columns pass through the key fold and drop out of the values
        self.uk = nn.Parameter(torch.zeros(heads, hd, self.row))
        self.uv = nn.Parameter(torch.zeros(heads, self.row, vdim))
        self.o_proj = nn.Linear(heads * vdim, width, bias=False)

    @staticmethod
    def padded_row(n: int) -> int:
        """The row length at or above n for which the matrix-core attention over latents is built (multiples of 32 up to 256, then
        of 64 up to 512); n itself beyond that."""
        for r in list(range(32, 257, 32)) + [320, 384, 448, 512]:
            if r >= n:
                return r
        return n

    def cache_rows(self) -> dict:
        return {self.cache_name: self.row}

    @torch.no_grad()
    def load_maps(self, uk: torch.Tensor | None = None, uv: torch.Tensor | None = None):
        """W_uk (heads * dim, kv_rank) / W_uv (heads * vdim, kv_rank) of a checkpoint into the widened parameters."""
        if uk is not None:
            self.uk[:, :self.dim, :self.kv_rank].copy_(uk.view(self.heads, self.dim, self.kv_rank))
            eye = torch.eye(self.rot_dim, dtype=self.uk.dtype, device=self.uk.device)
            self.uk[:, self.dim:, self.kv_rank:self.kv_rank + self.rot_dim].copy_(eye.expand(self.heads, -1, -1))
        if uv is not None:
            self.uv[:, :self.kv_rank, :].copy_(uv.view(self.heads, self.vdim, self.kv_rank).transpose(1, 2))

    def forward(self, h: torch.Tensor, positions: torch.Tensor, md) -> torch.Tensor:
        t = h.shape[0]
        cache = md.cache.latent(self.cache_name)
        q, gate = ops.latent_rope_prep(self.in_proj(h), (0, self.q_cols, self.q_cols + self.kv_cols), positions, self.freq, self.mag, self.kv_norm,
                                       self.eps, md.out_slots, cache, self.heads, self.dim, self.rot_dim)
        q_folded = torch.bmm(q.view(t, self.heads, self.dim + self.rot_dim).transpose(0, 1), self.uk)      # (heads, T, row)
        o = ops.latent_attn(q_folded, cache, md.kv_indices, md.kv_start, md.kv_len, md.layout, self.scale, gate=gate)
        v = torch.bmm(o, self.uv)                                                                           # (heads, T, vdim)
        return self.o_proj(v.transpose(0, 1).reshape(t, self.heads * self.vdim))
