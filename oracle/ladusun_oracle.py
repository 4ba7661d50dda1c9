"""Ladusun, restated plainly: float64, one function per mechanism, whole sequences at once (no cache, no state, no batching), so
that nothing here shares code or structure with the package.  `cfg` is the parsed config.json, `w` maps checkpoint names to tensors.

    streams   x_1..x_S all start as embed[token] * scale.  A sublayer q of a layer reads u = sum_s in_q[s] x_s, computes
              y = ls_q * f(rmsnorm(u) * norm_q) and every stream moves at once: x_t' = sum_s mix_q[s, t] x_s + out_q[t] y.
              The model's stream is sum_s x_s; logits = embed @ (rmsnorm(sum) * final.norm).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def plain_frequencies(dims, base):
    return torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)


def banded_frequencies(dims, base, sc):
    """Wavelength bands: short waves (below original / high) keep their frequency, long ones (above original / low) are divided
    by `factor`, the band between is blended linearly in original / wavelength."""
    out = []
    for f in plain_frequencies(dims, base).tolist():
        wave = 2.0 * math.pi / f
        if wave < sc["original"] / sc["high"]:
            out.append(f)
        elif wave > sc["original"] / sc["low"]:
            out.append(f / sc["factor"])
        else:
            s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
            out.append((1.0 - s) * f / sc["factor"] + s * f)
    return torch.tensor(out, dtype=F64), 1.0


def ramped_frequencies(dims, base, sc):
    """A ramp over the pair index between the pairs that make `fast` and `slow` turns over `original` positions; cos and sin grow
    by 0.1 ln(factor) + 1."""
    def index_of(turns):
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(index_of(sc["fast"])), 0)
    hi = min(math.ceil(index_of(sc["slow"])), dims - 1)
    out = []
    for i, f in enumerate(plain_frequencies(dims, base).tolist()):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / sc["factor"] * r + f * (1.0 - r))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(sc["factor"]) + 1.0


def turn_pairs(x, pos, freq, mag=1.0):
    """x (..., T, n): neighbours (2i, 2i + 1) of the first 2 * len(freq) entries turned by pos * freq[i]; the rest unchanged."""
    n = 2 * freq.numel()
    ang = pos.to(F64)[:, None] * freq[None, :]
    c, s = torch.cos(ang) * mag, torch.sin(ang) * mag
    a, b = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = a * c - b * s
    out[..., 1:n:2] = b * c + a * s
    return out


def attention_keys_values(h, w, p, m, pos):
    """The rows an attention layer caches: rotated keys (T, G, dim) and values (T, G, vdim)."""
    t = h.shape[0]
    g = m["kv_heads"]
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(t, g, m["dim"])
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(t, g, m["vdim"])
    return turn_pairs(k.transpose(0, 1), pos, *attention_frequencies(m)).transpose(0, 1), v


def attention_frequencies(m):
    rot = m["rot"]
    if rot.get("scaling"):
        return banded_frequencies(rot["dims"], rot["base"], rot["scaling"])
    return plain_frequencies(rot["dims"], rot["base"]), 1.0


def sink_softmax_readout(q, k, v, pos_q, pos_k, scale, cap=None, sink=0.0):
    """One head: q (T, dim) at positions pos_q over keys k (S, dim), values v (S, vdim) at positions pos_k.  Scores scale * q . k
    pass cap * tanh(. / cap); key j counts for query i when pos_k[j] <= pos_q[i]; the weights are exp(score) over
    exp(sink) + the sum of the visible ones (sink None: over the sum alone), so they add up to less than one."""
    s = (q @ k.T) * scale
    if cap:
        s = cap * torch.tanh(s / cap)
    seen = pos_q[:, None] >= pos_k[None, :]
    e = torch.where(seen, torch.exp(s), torch.zeros_like(s))
    extra = 0.0 if sink is None else math.exp(sink)
    return (e / (extra + e.sum(-1, keepdim=True))) @ v


def sink_attention(h, w, p, m, pos, kv):
    """Grouped-head attention with capped scores, a silent extra term of score 0 in the softmax's denominator, and one sigmoid
    gate per head.  `kv` = (keys, values) as attention_keys_values makes them (this layer's, or a lender's)."""
    t = h.shape[0]
    hq, g = m["heads"], m["kv_heads"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(t, hq, m["dim"]).transpose(0, 1)
    q = turn_pairs(q, pos, *attention_frequencies(m))
    keys, values = kv
    gate = torch.sigmoid(h @ w[p + "g"].T)                                   # (T, heads)
    heads = [sink_softmax_readout(q[j], keys[:, j // (hq // g)], values[:, j // (hq // g)], pos, pos, m["scale"], m.get("softcap")) * gate[:, j:j + 1]
             for j in range(hq)]
    return torch.cat(heads, -1) @ w[p + "o"].T + w[p + "o.b"]


def latent_attention(h, w, p, m, pos, eps):
    """Keys and values of all heads from one normed latent per token, plus one rotated key part that the heads share."""
    t = h.shape[0]
    hq, d, r, vd, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m["rot"]
    freq, mag = ramped_frequencies(rot["dims"], rot["base"], rot["scaling"]) if rot.get("scaling") else (plain_frequencies(rot["dims"], rot["base"]), 1.0)
    q = (h @ w[p + "q"].T).view(t, hq, d + r).transpose(0, 1)
    down = h @ w[p + "dkv"].T
    c = rms(down[:, :rank], eps) * w[p + "dkv.norm"]
    k_rot = turn_pairs(down[:, rank:], pos, freq, mag)
    q_rot = turn_pairs(q[..., d:], pos, freq, mag)
    k_plain = (c @ w[p + "uk"].T).view(t, hq, d)
    v = (c @ w[p + "uv"].T).view(t, hq, vd)
    gate = torch.sigmoid(h @ w[p + "g"].T)
    causal = pos[:, None] >= pos[None, :]
    heads = []
    for j in range(hq):
        s = (q[j, :, :d] @ k_plain[:, j].T + q_rot[j] @ k_rot.T) * m["scale"]
        s = torch.where(causal, s, torch.full_like(s, -math.inf))
        heads.append(torch.softmax(s, -1) @ v[:, j] * gate[:, j:j + 1])
    return torch.cat(heads, -1) @ w[p + "o"].T


def causal_conv(x, taps, bias):
    """x (T, channels); taps (channels, n) whose last column multiplies the current token; zeros stand before the first token."""
    t, n = x.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros(n - 1, x.shape[1], dtype=x.dtype), x])
    return bias + sum(padded[j:j + t] * taps[:, j] for j in range(n))


def gated_recurrence(u, r_pre, i_pre, lam, start=None):
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) sigmoid(i_pre_t) u_t with a_t = exp(-8 sigmoid(r_pre_t) softplus(lam)), every channel on
    its own, from `start` (zeros if None).  Returns all S_t (T, channels)."""
    a = torch.exp(-8.0 * torch.sigmoid(r_pre) * torch.nn.functional.softplus(lam))
    b = torch.sqrt(1.0 - a * a) * torch.sigmoid(i_pre) * u
    state = torch.zeros_like(u[0]) if start is None else start
    out = []
    for n in range(u.shape[0]):
        state = a[n] * state + b[n]
        out.append(state)
    return torch.stack(out)


def rglru(h, w, p, m):
    """Two branches: a gelu gate, and a per-channel causal convolution followed by a diagonal recurrence whose decay and input gate
    are sigmoids of block-diagonal maps of the convolved branch."""
    t = h.shape[0]
    width, blocks, taps = m["width"], m["blocks"], m["conv"]
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    x = h @ w[p + "x"].T + w[p + "x.b"]
    u = causal_conv(x, w[p + "conv"], w[p + "conv.b"])
    bw = width // blocks
    ub = u.view(t, blocks, bw)
    r = (torch.einsum("tbi,boi->tbo", ub, w[p + "ra"]) + w[p + "ra.b"]).reshape(t, width)
    i = (torch.einsum("tbi,boi->tbo", ub, w[p + "ri"]) + w[p + "ri.b"]).reshape(t, width)
    return (gated_recurrence(u, r, i, w[p + "lam"]) * y) @ w[p + "o"].T


def dense_ff(h, w, p):
    return torch.relu(h @ w[p + "up"].T + w[p + "up.b"]) ** 2 @ w[p + "down"].T + w[p + "down.b"]


def route(h, w, p, router):
    """(ids, weights) per token: softmax over all experts, experts outside the best groups struck out, the `top` largest kept and
    their scores divided by their sum."""
    return route_logits(h @ w[p + "router"].T, router)


def route_logits(z, router):
    n, top = router["experts"], router["top"]
    s = torch.softmax(z, -1)
    groups = router.get("groups")
    allowed = torch.ones_like(s, dtype=torch.bool)
    if groups:
        per = n // groups["count"]
        best = s.view(-1, groups["count"], per).max(-1).values
        keep = best.topk(groups["keep"], -1).indices
        ok = torch.zeros_like(best, dtype=torch.bool).scatter_(1, keep, True)
        allowed = ok[:, :, None].expand(-1, -1, per).reshape(-1, n)
    ids = torch.where(allowed, s, torch.full_like(s, -1.0)).topk(top, -1).indices
    chosen = s.gather(1, ids)
    return ids, chosen / (chosen.sum(-1, keepdim=True) + 1e-20)


def limited_glu(g, u, limit):
    """The gate capped from above, the other branch clamped on both sides and shifted by one."""
    g = torch.clamp(g, max=limit)
    u = torch.clamp(u, -limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def expert(h, w, p, limit):
    return limited_glu(h @ w[p + "gate"].T, h @ w[p + "up"].T, limit) @ w[p + "down"].T


def moe_ff(h, w, p, mlp):
    ids, wts = route(h, w, p, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(ids[t].tolist(), wts[t]):
            out[t] += a * expert(h[t:t + 1], w, f"{p}e{e}.", mlp["expert"]["limit"])[0]
    return out


def read_streams(xs, a_in):
    """What a sublayer reads of the streams xs (a list of (T, width)): sum_s a_in[s] xs[s]."""
    return sum(a_in[s] * xs[s] for s in range(len(xs)))


def move_streams(xs, y, mix, a_out):
    """All streams at once from the old ones: stream t becomes sum_s mix[s, t] xs[s] + a_out[t] y."""
    n = len(xs)
    return [sum(mix[s, t] * xs[s] for s in range(n)) + a_out[t] * y for t in range(n)]


def forward(cfg: dict, weights: dict, tokens, layer_sums: list | None = None):
    """Logits (T, vocab) of one sequence computed whole.  `layer_sums`, a list, receives the sum of the streams after every layer."""
    w = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    n_streams = int(cfg.get("streams") or 1)
    pos = torch.arange(len(tokens))
    x0 = w["embed"][torch.as_tensor(tokens)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    xs = [x0.clone() for _ in range(n_streams)]
    kept = {}

    def sublayer(q, p, fn):
        nonlocal xs
        hyper = (p + f"hc{q}.in") in w
        u = read_streams(xs, w[p + f"hc{q}.in"]) if hyper else xs[0]
        y = fn(rms(u, eps) * w[p + f"norm{q}"])
        if (p + f"ls{q}") in w:
            y = y * w[p + f"ls{q}"]
        if hyper:
            xs = move_streams(xs, y, w[p + f"hc{q}.mix"], w[p + f"hc{q}.out"])
        else:
            xs = [xs[0] + y]

    for i, layer in enumerate(cfg["layers"]):
        p, m, kind = f"l{i}.", layer["mixer"], layer["type"]
        if kind == "attention":
            def mixer(h, m=m, p=p, i=i):
                src = m.get("kv_from")
                if src is None:
                    kept[i] = attention_keys_values(h, w, p + "mix.", m, pos)
                    src = i
                return sink_attention(h, w, p + "mix.", m, pos, kept[src])
        elif kind == "latent_attention":
            def mixer(h, m=m, p=p):
                return latent_attention(h, w, p + "mix.", m, pos, eps)
        elif kind == "rglru":
            def mixer(h, m=m, p=p):
                return rglru(h, w, p + "mix.", m)
        else:
            raise ValueError(kind)
        sublayer(1, p, mixer)
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                sublayer(2, p, lambda h, p=p: dense_ff(h, w, p + "mlp."))
            else:
                sublayer(2, p, lambda h, p=p, mlp=mlp: moe_ff(h, w, p + "mlp.", mlp))
        if layer_sums is not None:
            layer_sums.append(sum(xs))
    return (rms(sum(xs), eps) * w["final.norm"]) @ w["embed"].T
