"""Recurrent token mixers backed by the HIP scan kernels."""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops


class MinGRU(nn.Module):
    """Gated recurrence with gates that are functions of the current token alone (no dependence on the state): with z = sigmoid(W_z h + b_z), u = W_x h + b_x and
    cand = u + 1/2 (u >= 0) or sigmoid(u) (u < 0), the state moves as S <- (1 - z) S + z cand and the layer returns
    W_o (S * silu(W_g h)).  The three input projections are one matrix product; gates, candidate and state are float32
    inside the scan kernel, and the state (`inner` floats per sequence) lives in the state pool under `state_name`."""

    def __init__(self, width: int, inner: int, state_name):
        super().__init__()
        self.width, self.inner, self.state_name = width, inner, state_name
        self.zxg_proj = nn.Linear(width, 3 * inner, bias=True)     # rows: z | x | g (the gate g has no bias: zeros)
        self.o_proj = nn.Linear(inner, width, bias=False)

    def state_shapes(self) -> dict:
        return {self.state_name: (self.inner,)}

    def forward(self, h: torch.Tensor, md) -> torch.Tensor:
        zxg = self.zxg_proj(h)
        y = ops.mingru_scan(zxg, md.cache.state(self.state_name), md.layout)
        return self.o_proj(y)


def _f32(*shape):
    return nn.Parameter(torch.zeros(*shape, dtype=torch.float32))


class MLSTM(nn.Module):
    """Matrix memory per head with an exponential input gate and a sigmoid forget gate, both capped, kept finite by a
    running maximum m (which starts at 0):  i = cap tanh((W_i h + b_i) / cap), f = logsigmoid(cap tanh((W_f h + b_f) / cap)),
    m' = max(f + m, i), S <- e^(f + m - m') S + e^(i - m') k v^T, n likewise with k alone,
    o = S^T q / (max(|n . q|, e^(-m')) + 1e-6) with q = W_q h / sqrt(dim).  Each head's o is divided by its root mean square,
    the heads times `norm` times sigmoid(W_g h), then W_o.  q, k, v and the output gate are one matrix product; the two
    gate projections are float32 and so are S, n and m, which live in the state pool under (state_name, "S" | "n" | "m")."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float, state_name):
        super().__init__()
        self.heads, self.dim, self.vdim, self.gate_cap, self.eps, self.state_name = heads, dim, vdim, float(gate_cap), eps, state_name
        self.qkvg_proj = nn.Linear(width, 2 * heads * dim + 2 * heads * vdim, bias=False)     # rows: q | k | v | g
        self.gate_w, self.gate_b = _f32(2 * heads, width), _f32(2 * heads)                   # rows: input | forget
        self.norm = _f32(heads * vdim)
        self.o_proj = nn.Linear(heads * vdim, width, bias=False)

    def state_shapes(self) -> dict:
        n = self.state_name
        return {(n, "S"): (self.heads, self.dim, self.vdim), (n, "n"): (self.heads, self.dim), (n, "m"): (self.heads,)}

    def forward(self, h: torch.Tensor, md) -> torch.Tensor:
        hd, he, n = self.heads * self.dim, self.heads * self.vdim, self.state_name
        x = self.qkvg_proj(h)
        gates = ops.skinny_proj(h, self.gate_w)
        o = ops.mlstm_scan(x, (0, hd, 2 * hd), gates, self.gate_b, self.gate_cap, md.cache.state((n, "S")), md.cache.state((n, "n")),
                           md.cache.state((n, "m")), md.layout, self.heads, self.dim, self.vdim)
        y = ops.head_norm_gate(o, self.norm, self.eps, gate=x[:, 2 * hd + he:], kind="sigmoid")
        return self.o_proj(y)


class GatedDelta(nn.Module):
    """Delta rule with a per-head decay.  q, k (kv_heads x dim) and v (heads x vdim) pass a short causal convolution per channel
    and silu; q and k are scaled to unit length per head (q also by 1 / sqrt(dim)); beta = sigmoid(W_b h),
    g = exp(-exp(A_log) softplus(W_a h + dt_bias)); per head S <- g S, u = beta (v - S^T k), S <- S + k u^T, o = S^T q (the
    read sees the token's own write).  Each head's o is divided by its root mean square, times `norm` (vdim, shared by the
    heads), times silu(W_g h), then W_o.  State: S (float32) and the last taps - 1 inputs of the convolution."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, eps: float, state_name):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.heads, self.kv_heads, self.dim, self.vdim, self.taps, self.eps, self.state_name = heads, kv_heads, dim, vdim, taps, eps, state_name
        self.conv_ch = 2 * kv_heads * dim + heads * vdim
        self.qkvg_proj = nn.Linear(width, self.conv_ch + heads * vdim, bias=False)            # rows: q | k | v | g
        self.conv_w = _f32(taps, self.conv_ch)                                                # row j: the tap taps - 1 - j tokens back
        self.ab_w = _f32(2 * heads, width)                                                    # rows: decay | write strength
        self.a_log, self.dt_bias = _f32(heads), _f32(heads)
        self.norm = _f32(vdim)
        self.o_proj = nn.Linear(heads * vdim, width, bias=False)

    def state_shapes(self) -> dict:
        shapes = {(self.state_name, "S"): (self.heads, self.dim, self.vdim)}
        if self.taps > 1:
            shapes[(self.state_name, "conv")] = (self.taps - 1, self.conv_ch)
        return shapes

    def forward(self, h: torch.Tensor, md) -> torch.Tensor:
        gd, n = self.kv_heads * self.dim, self.state_name
        x = self.qkvg_proj(h)
        xc = ops.short_conv_silu(x[:, :self.conv_ch], self.conv_w, md.cache.state((n, "conv")) if self.taps > 1 else None, md.layout)
        ab = ops.skinny_proj(h, self.ab_w)
        o = ops.delta_scan(xc, (0, gd, 2 * gd), ab, self.a_log, self.dt_bias, md.cache.state((n, "S")), md.layout, self.heads, self.kv_heads,
                           self.dim, self.vdim)
        y = ops.head_norm_gate(o, self.norm, self.eps, gate=x[:, self.conv_ch:], kind="silu")
        return self.o_proj(y)


class TimeMix(nn.Module):
    """RWKV-style time mixing.  Each of r, k, v, g, w reads its own blend of the token's input and its predecessor's,
    h + (h_prev - h) * mu_s; r, k, v = W_r, W_k, W_v of their blends (heads x dim), gate = silu(W_g blend_g), decay
    w = exp(-exp(W_w2 tanh(W_w1 blend_w) + w0)) per head and key channel.  Per head o = (S + diag(bonus) k v^T)^T r, then
    S <- diag(w) S + k v^T.  Each head's o is divided by its root mean square, times `norm`, times the gate, then W_o.
    State: S (float32) and the predecessor's input row.  The four wide projections are one batched matrix product; the
    decay's two small ones are float32 (ops.skinny_proj, the tanh applied as the second one reads its input)."""

    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, width: int, heads: int, dim: int, decay_rank: int, eps: float, state_name):
        super().__init__()
        self.width, self.heads, self.dim, self.eps, self.state_name = width, heads, dim, eps, state_name
        hd = heads * dim
        self.mu = _f32(len(self.MIXES), width)
        self.rkvg = nn.Parameter(torch.empty(4, hd, width))
        self.w1, self.w2, self.w0 = _f32(decay_rank, width), _f32(hd, decay_rank), _f32(hd)
        self.bonus = _f32(heads, dim)
        self.norm = _f32(hd)
        self.o_proj = nn.Linear(hd, width, bias=False)

    def state_shapes(self) -> dict:
        return {(self.state_name, "S"): (self.heads, self.dim, self.dim), (self.state_name, "prev"): (self.width,)}

    def forward(self, h: torch.Tensor, md) -> torch.Tensor:
        n = self.state_name
        blends = ops.token_shift_mix(h, self.mu, md.cache.state((n, "prev")), md.layout)          # (5, T, width)
        proj = torch.bmm(blends[:4], self.rkvg.transpose(1, 2))                                    # (4, T, heads * dim)
        wlog = ops.skinny_proj(ops.skinny_proj(blends[4], self.w1), self.w2, in_act="tanh")
        o = ops.rwkv_scan(proj[0], proj[1], proj[2], wlog, self.w0, self.bonus, md.cache.state((n, "S")), md.layout, self.heads, self.dim)
        y = ops.head_norm_gate(o, self.norm, self.eps, gate=proj[3], kind="silu")
        return self.o_proj(y)


class DecayLinearAttention(nn.Module):
    """Linear attention with one constant decay per head: q = silu(W_q h), k = silu(W_k h) (heads x dim), v = silu(W_v h) (heads x
    vdim); per head S <- decay_h S + k v^T, o = S^T q (the read sees the token's own write, no other scale).  The concatenated heads
    are divided by their common root mean square, times `norm`, times sigmoid(W_g h), then W_o.  State: S (float32), zero at a
    sequence's start.  The projections q | k | v | g are rows of one matrix product: the module's own (`forward`), or a wider one
    the caller shares between several mechanisms (`mix`, with the first column of this module's block)."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay, eps: float, state_name, own_proj: bool = True):
        super().__init__()
        decay = [float(d) for d in decay]
        if len(decay) != heads:
            raise ValueError(f"{heads} heads need {heads} decays, got {len(decay)}")
        self.heads, self.dim, self.vdim, self.eps, self.state_name = heads, dim, vdim, eps, state_name
        self.register_buffer("decay", torch.tensor(decay, dtype=torch.float32), persistent=False)
        self.proj_rows = 2 * heads * dim + 2 * heads * vdim
        if own_proj:
            self.in_proj = nn.Linear(width, self.proj_rows, bias=False)
        self.norm = _f32(heads * vdim)
        self.o_proj = nn.Linear(heads * vdim, width, bias=False)

    def state_shapes(self) -> dict:
        return {(self.state_name, "S"): (self.heads, self.dim, self.vdim)}

    def mix(self, x: torch.Tensor, col0: int, md) -> torch.Tensor:
        hd, he = self.heads * self.dim, self.heads * self.vdim
        o = ops.decay_scan(x, (col0, col0 + hd, col0 + 2 * hd), self.decay, md.cache.state((self.state_name, "S")), md.layout, self.heads,
                           self.dim, self.vdim, act="silu")
        g0 = col0 + 2 * hd + he
        y = ops.head_norm_gate(o.view(-1, 1, he), self.norm, self.eps, gate=x[:, g0:g0 + he], kind="sigmoid")
        return self.o_proj(y)

    def forward(self, h: torch.Tensor, md) -> torch.Tensor:
        return self.mix(self.in_proj(h), 0, md)


class RGLRU(nn.Module):
    """Recurrent block around a real-gated linear recurrent unit (S. De, S. L. Smith et al., "Griffin: Mixing Gated Linear
    Recurrences with Local Attention for Efficient Language Models").  Two branches of `inner` channels: y = gelu_tanh(W_y h + b_y),
    and u = causal convolution per channel (taps, with a bias, no activation) of W_x h + b_x.  The channels form `blocks` equal
    blocks; within block b the gates are r = sigmoid(A_b u_b + a_b), i = sigmoid(B_b u_b + b_b) with square matrices A_b, B_b.  Then
    a = exp(-decay_scale * r * softplus(lam)), S <- a S + sqrt(1 - a^2) * i * u (from S = 0, the first token like every other), and
    the layer returns W_o (S * y).  State: S (float32) and the convolution's last taps - 1 inputs.
    The two branch projections are one matrix product, the two gate maps of all blocks one batched product; gates, decay and state are
    float32 inside the scan kernel; the channel's constant decay_scale * softplus(lam) is formed once, when the weights are in place."""

    def __init__(self, width: int, inner: int, blocks: int, taps: int, decay_scale: float, state_name):
        super().__init__()
        if inner % blocks:
            raise ValueError("the channels must divide into the blocks")
        self.width, self.inner, self.blocks, self.taps, self.decay_scale, self.state_name = width, inner, blocks, taps, float(decay_scale), state_name
        bw = inner // blocks
        self.in_proj = nn.Linear(width, 2 * inner, bias=True)              # rows: y | x
        self.conv_w = _f32(taps, inner)                                    # row j: the tap taps - 1 - j tokens back
        self.conv_b = _f32(inner)
        self.gate_w = nn.Parameter(torch.empty(blocks, bw, 2 * bw))        # per block: input channel -> recurrence gate | input gate
        self.gate_b = _f32(2, inner)                                       # rows: recurrence gate | input gate
        self.lam = _f32(inner)
        self.register_buffer("rate", torch.zeros(inner, dtype=torch.float32), persistent=False)
        self.o_proj = nn.Linear(inner, width, bias=False)

    def finalize(self):
        """After the weights are loaded: the constant factor of every channel's decay exponent."""
        self.rate.copy_(self.decay_scale * F.softplus(self.lam.detach().double()).float())

    def state_shapes(self) -> dict:
        shapes = {(self.state_name, "S"): (self.inner,)}
        if self.taps > 1:
            shapes[(self.state_name, "conv")] = (self.taps - 1, self.inner)
        return shapes

    def forward(self, h: torch.Tensor, md) -> torch.Tensor:
        n, t = self.state_name, h.shape[0]
        yx = self.in_proj(h)
        u = ops.short_conv(yx[:, self.inner:], self.conv_w, md.cache.state((n, "conv")) if self.taps > 1 else None, md.layout, bias=self.conv_b)
        gates = torch.bmm(u.view(t, self.blocks, -1).transpose(0, 1), self.gate_w)      # (blocks, T, 2 * block width)
        s = ops.rglru_scan(yx[:, :self.inner], u, gates, self.gate_b, self.rate, md.cache.state((n, "S")), md.layout)
        return self.o_proj(s)
