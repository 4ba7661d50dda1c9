"""Causal attention with grouped key/value heads and separate key and value sizes over per-token key and value rows in the
token cache: SoftcapAttention (rotary positions on a leading part of each head, unit-mean-square values, capped scores) and
NormedAttention (query/key RMS norms, optional rotation of keys AND values, window, distance penalty, output gate, borrowed
keys and values)."""
from __future__ import annotations

import torch
from torch import nn

from .. import ops
from .rotary_embedding import rotary_frequencies


class SoftcapAttention(nn.Module):
    """q = W_q h, k = W_k h (rotated by position), v = W_v h (each head divided by its root mean square, cached so);
    score = scale * q . k, then cap * tanh(score / cap) (cap None or 0: none), softmax over the causal prefix, W_o on the
    concatenated heads.  Query head j reads key/value head j // (heads / kv_heads).  `rot` = {dims, base, scaling | None}.
    The three projections are one matrix product; the cache holds two rows per token under `cache_names`."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, rot: dict, scale: float, softcap, eps: float, cache_names):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("query heads must be a multiple of key/value heads")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.softcap, self.eps = float(scale), float(softcap or 0.0), eps
        self.k_name, self.v_name = cache_names
        self.rot_dims = int(rot["dims"]) if rot else 0
        if self.rot_dims % 2 or self.rot_dims > dim:
            raise ValueError("the rotated part of a head must be even and within the head")
        if self.rot_dims:
            freq, self.mag = rotary_frequencies(self.rot_dims, rot["base"], rot.get("scaling"))
            self.register_buffer("freq", freq.to(torch.float64), persistent=False)
        else:
            self.freq, self.mag = None, 1.0
        self.qkv_proj = nn.Linear(width, heads * dim + kv_heads * (dim + vdim), bias=False)     # rows: q | k | v
        self.o_proj = nn.Linear(heads * vdim, width, bias=False)

    def cache_rows(self) -> dict:
        return {self.k_name: self.kv_heads * self.dim, self.v_name: self.kv_heads * self.vdim}

    def forward(self, h: torch.Tensor, positions: torch.Tensor, md) -> torch.Tensor:
        k_cache, v_cache = md.cache.latent(self.k_name), md.cache.latent(self.v_name)
        q = ops.rope_vnorm_store(self.qkv_proj(h), positions, self.freq, self.mag, self.rot_dims, self.eps, md.out_slots, k_cache, v_cache,
                                 self.heads, self.kv_heads, self.dim, self.vdim)
        o = ops.softcap_attn(q, k_cache, v_cache, md.kv_indices, md.kv_start, md.kv_len, md.layout, self.scale, self.softcap, self.heads,
                             self.kv_heads, self.dim, self.vdim)
        return self.o_proj(o)


class NormedAttention(nn.Module):
    """Softmax attention whose queries and keys pass an RMS norm, with these parts, each optional:
      qk_norm   "head": every q and k head by its own root mean square, weight (dim) shared by the heads; "row": all heads of a
                token's q (and of its k) at once, weights of heads * dim and kv_heads * dim entries; "none"
      rot       {dims, base, interleaved, scaling}: the first `dims` of every q and k head turned by position * f_m, f_m = base^(-2m/dims)
                (stretched by `scaling`, see rotary_frequencies; one that changes the magnitude is refused), pair m being (m, m + dims/2),
                or (2m, 2m + 1) if interleaved
      rotate_values   the value of position j is cached turned by j * base^(-2m/vdim) over all of vdim (same pair layout) and a
                head's read-out at position i is turned back by i, so every value enters in the frame of its distance to i
      softcap   scores through cap tanh(. / cap);   window   a token sees itself and the window - 1 before it
      distance_penalty   r1_h ln(1 + r2_h (i - j)) taken off the score (r1, r2: one number per head)
      sink_score   the softmax's sum has one more term exp(sink_score) without a value (0.0: one is added to the denominator)
      out_gate  the concatenated heads times sigmoid(W_g h): True, one gate per element; "head", one per head
      bias      q, k, v projections with biases;   o_bias   the output projection too
      kv_source (k_name, v_name) of another layer's cache rows: no key/value projections here, that layer's rows are read.
    The projections q | k | v | g are rows of ONE matrix product: the module's own (`forward`), or a wider one that the caller
    shares between several mechanisms (`attend`, with the first column of this module's block)."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, eps: float, cache_names, qk_norm: str = "head",
                 rot: dict | None = None, rotate_values: bool = False, softcap=None, window=None, distance_penalty: bool = False,
                 out_gate=False, bias: bool = False, kv_source=None, own_proj: bool = True, sink_score=None, o_bias: bool = False):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("query heads must be a multiple of key/value heads")
        if qk_norm not in ("head", "row", "none"):
            raise ValueError(f"unknown query/key norm {qk_norm!r}")
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.softcap, self.eps, self.window = float(scale), float(softcap or 0.0), eps, int(window or 0)
        if out_gate not in (False, True, "head"):
            raise ValueError(f"unknown output gate {out_gate!r}")
        self.qk_norm, self.out_gate, self.borrows = qk_norm, out_gate, kv_source is not None
        self.sink_score = None if sink_score is None else float(sink_score)
        self.k_name, self.v_name = kv_source if self.borrows else cache_names
        self.rot_dims = int(rot["dims"]) if rot else 0
        self.interleaved = bool(rot and rot.get("interleaved"))
        if self.rot_dims % 2 or self.rot_dims > dim:
            raise ValueError("the rotated part of a head must be even and within the head")
        if rotate_values and (not rot or vdim % 2):
            raise ValueError("rotated values need a rotation base and an even value size")
        freq = None
        if self.rot_dims:
            freq, mag = rotary_frequencies(self.rot_dims, rot["base"], rot.get("scaling"))
            if mag != 1.0:
                raise NotImplementedError("a frequency scaling that changes the rotation's magnitude is not built for this attention")
        self.register_buffer("freq", freq.to(torch.float64) if self.rot_dims else None, persistent=False)
        self.register_buffer("vfreq", rotary_frequencies(vdim, rot["base"])[0].to(torch.float64) if rotate_values else None, persistent=False)
        n_w = {"head": (dim, dim), "row": (heads * dim, kv_heads * dim), "none": (0, 0)}[qk_norm]
        if n_w[0]:
            self.q_norm = nn.Parameter(torch.zeros(n_w[0], dtype=torch.float32))
            if not self.borrows:
                self.k_norm = nn.Parameter(torch.zeros(n_w[1], dtype=torch.float32))
        if distance_penalty:
            self.r1 = nn.Parameter(torch.zeros(heads, dtype=torch.float32))
            self.r2 = nn.Parameter(torch.zeros(heads, dtype=torch.float32))
        else:
            self.r1 = self.r2 = None
        # columns of this module's block of a projection: q | k | v | g
        self.q_cols = heads * dim
        self.k_cols = 0 if self.borrows else kv_heads * dim
        self.v_cols = 0 if self.borrows else kv_heads * vdim
        self.g_cols = heads if out_gate == "head" else heads * vdim if out_gate else 0
        self.proj_rows = self.q_cols + self.k_cols + self.v_cols + self.g_cols
        self.has_bias = bias
        if own_proj:
            self.in_proj = nn.Linear(width, self.proj_rows, bias=bias)
            if bias:
                nn.init.zeros_(self.in_proj.bias)      # the gate's rows have no bias: theirs stays zero
        self.o_proj = nn.Linear(heads * vdim, width, bias=o_bias)

    def cache_rows(self) -> dict:
        return {} if self.borrows else {self.k_name: self.kv_heads * self.dim, self.v_name: self.kv_heads * self.vdim}

    def attend(self, x: torch.Tensor, col0: int, positions: torch.Tensor, md) -> torch.Tensor:
        k_cache, v_cache = md.cache.latent(self.k_name), md.cache.latent(self.v_name)
        k0 = col0 + self.q_cols
        v0 = k0 + self.k_cols
        g0 = v0 + self.v_cols
        own = not self.borrows
        q, v_turn = ops.attn_prep_store(x, (col0, k0, v0), positions, getattr(self, "q_norm", None), getattr(self, "k_norm", None), self.qk_norm, self.eps,
                                self.freq, self.rot_dims, self.interleaved, self.vfreq, md.out_slots if own else None,
                                k_cache if own else None, v_cache if own else None, self.heads, self.kv_heads if own else 0, self.dim, self.vdim)
        o = ops.softcap_attn(q, k_cache, v_cache, md.kv_indices, md.kv_start, md.kv_len, md.layout, self.scale, self.softcap, self.heads,
                             self.kv_heads, self.dim, self.vdim, window=self.window, r1=self.r1, r2=self.r2, v_turn=v_turn,
                             v_interleaved=self.interleaved, gate=x[:, g0:g0 + self.g_cols] if self.out_gate else None,
                             sink_score=self.sink_score)
        return self.o_proj(o)

    def forward(self, h: torch.Tensor, positions: torch.Tensor, md) -> torch.Tensor:
        return self.attend(self.in_proj(h), 0, positions, md)
