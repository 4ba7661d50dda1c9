"""Plain restatement of the Gibavik design: one slow function per mechanism, whole sequences, token by token where the
design has a recurrence.  CPU tensors, float64 by default.  Nothing here is shared with the product path
(nano_vllm_x_amd/gibavik.py and the kernels it launches); the tests compare the two.

Notation: T tokens, W model width, H query heads, G key/value heads, D key size, E value size.  A weight dictionary `p`
maps the checkpoint's tensor names to tensors; `spec` is an entry of config.json's "layers".
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64
GLU_SLOPE = 1.702


def _lin(w, x, b=None):
    y = x @ w.to(x.dtype).T
    return y if b is None else y + b.to(x.dtype)


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """Rows of x scaled to unit mean square, times ONE number g."""
    return unit_rms(x, eps) * g.to(x.dtype).reshape(())


# ---- rotations ------------------------------------------------------------------------------------------------------
def turn(x, pos, base: float, dims: int, interleaved: bool = False, sign: float = 1.0):
    """x (T, heads, size): the first `dims` entries of every head are turned in pairs by sign * pos * base^(-2m/dims), pair m
    being (m, m + dims/2), or (2m, 2m + 1) if `interleaved`; the rest pass unchanged."""
    out = x.clone()
    half = dims // 2
    m = torch.arange(half, dtype=x.dtype)
    ang = sign * pos.to(x.dtype)[:, None] * (float(base) ** (-2.0 * m / dims))[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    if interleaved:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2], out[..., 1:dims:2] = a * c - b * s, b * c + a * s
    else:
        a, b = x[..., :half], x[..., half:dims]
        out[..., :half], out[..., half:dims] = a * c - b * s, b * c + a * s
    return out


# ---- softmax attention ------------------------------------------------------------------------------------------------
def attend(q, k, v, scale: float, cap=None, window=None, r1=None, r2=None):
    """q (T, H, D), k (T, G, D), v (T, G, E) of one sequence from its first token.  Token i sees j <= i (and i - j < window if
    there is one).  score = scale q.k, capped by cap tanh(./cap) if there is a cap, minus r1_h ln(1 + r2_h (i - j)) if the
    heads have distance numbers.  Returns (T, H, E)."""
    t, h, _ = q.shape
    g = k.shape[1]
    out = torch.zeros(t, h, v.shape[2], dtype=q.dtype)
    for hd in range(h):
        kv = hd // (h // g)
        for i in range(t):
            lo = 0 if not window else max(0, i - window + 1)
            s = (k[lo:i + 1, kv] @ q[i, hd]) * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            if r1 is not None:
                dist = torch.arange(i - lo, -1, -1, dtype=q.dtype)
                s = s - r1[hd].to(q.dtype) * torch.log(1.0 + r2[hd].to(q.dtype) * dist)
            w = torch.softmax(s, dim=0)
            out[i, hd] = w @ v[lo:i + 1, kv]
    return out


def biased_attention_keys(p, pre, m, h, eps):
    """Keys (after their norm over the whole projection) and values of a distance-biased attention layer: (T, G, D), (T, G, E)."""
    g, d, e = m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    t = h.shape[0]
    k = _lin(p[pre + "k"], h, p[pre + "k.b"])
    k = unit_rms(k, eps) * p[pre + "k.norm"].to(h.dtype)
    v = _lin(p[pre + "v"], h, p[pre + "v.b"])
    return k.view(t, g, d), v.view(t, g, e)


def biased_attention(p, pre, m, h, eps, kv=None):
    """The 'attention' mixer.  `kv`: the (keys, values) of the layer this one borrows them from, or None for its own.
    Returns (output (T, W), (keys, values))."""
    t = h.shape[0]
    hq, d = m["heads"], m["dim"]
    q = _lin(p[pre + "q"], h, p[pre + "q.b"])
    q = (unit_rms(q, eps) * p[pre + "q.norm"].to(h.dtype)).view(t, hq, d)
    if kv is None:
        kv = biased_attention_keys(p, pre, m, h, eps)
    o = attend(q, kv[0], kv[1], m["scale"], cap=m.get("softcap"), window=(m.get("mask") or {}).get("size"), r1=p[pre + "r1"], r2=p[pre + "r2"])
    return _lin(p[pre + "o"], o.reshape(t, -1)), kv


def windowed_attention(p, pre, m, h, pos, eps):
    """Left branch of the parallel mixer: per-head query/key norm, rotary positions on a leading part of q and k, values
    turned by their position and the read-out turned back, capped scores, sliding window, sigmoid output gate."""
    t = h.shape[0]
    hq, g, d, e = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = _lin(p[pre + "q"], h, p[pre + "q.b"]).view(t, hq, d)
    k = _lin(p[pre + "k"], h, p[pre + "k.b"]).view(t, g, d)
    v = _lin(p[pre + "v"], h, p[pre + "v.b"]).view(t, g, e)
    q = unit_rms(q, eps) * p[pre + "q.norm"].to(h.dtype)
    k = unit_rms(k, eps) * p[pre + "k.norm"].to(h.dtype)
    rot = m.get("rot")
    inter = bool(rot) and rot.get("layout") == "interleaved"
    if rot:
        q = turn(q, pos, rot["base"], rot["dims"], inter)
        k = turn(k, pos, rot["base"], rot["dims"], inter)
        v = turn(v, pos, rot["base"], e, inter)
    o = attend(q, k, v, m["scale"], cap=m.get("softcap"), window=(m.get("mask") or {}).get("size"))
    if rot:
        o = turn(o, pos, rot["base"], e, inter, sign=-1.0)
    o = o.reshape(t, hq * e) * torch.sigmoid(_lin(p[pre + "g"], h))
    return _lin(p[pre + "o"], o)


# ---- decayed outer-product memory ---------------------------------------------------------------------------------------
def decayed_memory(q, k, v, decay, state=None):
    """q, k (T, H, D), v (T, H, E); per head S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  Returns (o (T, H, E), S)."""
    t, h, d = q.shape
    e = v.shape[2]
    s = torch.zeros(h, d, e, dtype=q.dtype) if state is None else state.clone()
    out = torch.zeros(t, h, e, dtype=q.dtype)
    dec = torch.as_tensor(decay, dtype=q.dtype).view(h, 1, 1)
    for i in range(t):
        s = dec * s + k[i][:, :, None] * v[i][:, None, :]
        out[i] = torch.einsum("hde,hd->he", s, q[i])
    return out, s


def lightning(p, pre, m, h, eps):
    """Right branch of the parallel mixer."""
    t = h.shape[0]
    hh, d, e = m["heads"], m["dim"], m["vdim"]
    silu = torch.nn.functional.silu
    q = silu(_lin(p[pre + "q"], h)).view(t, hh, d)
    k = silu(_lin(p[pre + "k"], h)).view(t, hh, d)
    v = silu(_lin(p[pre + "v"], h)).view(t, hh, e)
    o, _ = decayed_memory(q, k, v, m["decay"])
    o = unit_rms(o.reshape(t, hh * e), eps) * p[pre + "norm"].to(h.dtype)
    return _lin(p[pre + "o"], o * torch.sigmoid(_lin(p[pre + "g"], h)))


def parallel_mixer(p, pre, m, h, pos, eps):
    return m["left_scale"] * windowed_attention(p, pre + "left.", m["left"], h, pos, eps) + \
        m["right_scale"] * lightning(p, pre + "right.", m["right"], h, eps)


# ---- feed-forward ---------------------------------------------------------------------------------------------------------
def dense_ff(p, pre, mlp, h):
    lim = float(mlp["limit"])
    g = torch.clamp(_lin(p[pre + "gate"], h), max=lim)
    u = torch.clamp(_lin(p[pre + "up"], h), -lim, lim)
    return _lin(p[pre + "down"], g * torch.sigmoid(GLU_SLOPE * g) * (u + 1.0))


def table_experts(p, pre, mlp, h, tokens):
    """Each token id has its experts in a table; every chosen expert weighs 1 / top."""
    top = int(mlp["router"]["top"])
    table = p[pre + "table"]
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e in table[int(tokens[i])].tolist()[:top]:
            q = f"{pre}e{int(e)}."
            x = h[i:i + 1]
            y = torch.nn.functional.silu(_lin(p[q + "gate"], x)) * _lin(p[q + "up"], x)
            out[i] += _lin(p[q + "down"], y)[0] / top
    return out


# ---- the model --------------------------------------------------------------------------------------------------------------
def forward(cfg: dict, p: dict, tokens, dtype=F64, streams=None):
    """Logits (T, vocab) of one sequence from its first token.  `streams`: a list that receives the residual stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.int64)
    pos = torch.arange(len(tokens))
    x = p["embed"].to(dtype)[tokens] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    kept = {}
    for i, spec in enumerate(cfg["layers"]):
        pre, m = f"l{i}.mix.", spec["mixer"]
        if spec["type"] == "parallel":
            y = parallel_mixer(p, pre, m, x, pos, eps)
        elif spec["type"] == "attention":
            src = m.get("kv_from")
            y, kept[i] = biased_attention(p, pre, m, x, eps, kv=None if src is None else kept[int(src)])
        else:
            raise ValueError(spec["type"])
        x = x + scalar_norm(y, p[f"l{i}.norm1"], eps)
        mlp = spec.get("mlp")
        if mlp is not None:
            y = dense_ff(p, f"l{i}.mlp.", mlp, x) if mlp["kind"] == "dense" else table_experts(p, f"l{i}.mlp.", mlp, x, tokens)
            x = x + scalar_norm(y, p[f"l{i}.norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    z = _lin(p["head"], scalar_norm(x, p["final.norm"], eps))
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z
