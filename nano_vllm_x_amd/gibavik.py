"""Gibavik: a decoder stack whose sublayers read the float32 residual stream as it is and whose RESULTS are normed before
they are added:
    x <- x + g1 * mixer(x) / rms(mixer(x));   x <- x + g2 * ff(x) / rms(ff(x))          (g1, g2: one number each per layer)
with x = embed[token] * embedding.scale at the start and logits = cap * tanh(head(gf * x / rms(x)) / cap) at the end.

A layer's mixer is one of
  attention  softmax attention over all earlier tokens: grouped heads, biased projections, query and key normed over the whole
             projection, no rotation; the score loses r1_h ln(1 + r2_h * distance).  A layer may borrow the cached keys and values
             of an earlier attention layer (`kv_from`) and then has only queries of its own.
  parallel   two mixers on the same input, their results weighted and summed: LEFT a sliding-window softmax attention (per-head
             query/key norm, rotary positions on a leading part of each head, values rotated by their position and the read-out
             rotated back, capped scores, sigmoid output gate), RIGHT linear attention with a constant decay per head (silu on q,
             k, v; matrix state per head; joint RMS norm of the heads; sigmoid output gate).
and its feed-forward is dense (clamped gate and up, g sigmoid(1.702 g)(u + 1)), a mixture of silu-gated experts chosen by a table
of token ids (weight 1 / top each), or absent.

config.json gives every size, the order of the layers and the constants; the mechanisms live in layers/ (cap_attention.py,
recurrent.py, moe.py) with their constants as arguments.  Between the matrix products (library GEMMs; all input projections of a
mixer are ONE product) every step is a HIP kernel of this package, one launch per sublayer boundary (ops.postnorm_residual).
The stream, norms, attention scores, positions and angles, and the recurrent state are float32 in every activation format.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Iterable

import torch
import torch.nn.functional as F
from torch import nn

from . import distributed as tpd
from . import ops
from .layers.cap_attention import NormedAttention
from .layers.moe import TableMoE
from .layers.recurrent import DecayLinearAttention

MIXERS = ("attention", "parallel")
GLU_SLOPE = 1.702      # dense feed-forward: y = g * sigmoid(1.702 g) * (u + 1)


def _rot_spec(m: dict):
    rot = m.get("rot")
    if not rot:
        return None
    return {"dims": int(rot["dims"]), "base": float(rot["base"]), "interleaved": rot.get("layout") == "interleaved"}


def _softmax_spec(m: dict) -> dict:
    """Sizes and constants of a softmax-attention mixer (the 'attention' mixer or the left branch of 'parallel')."""
    mask = m.get("mask") or {}
    out = {"heads": int(m["heads"]), "kv_heads": int(m.get("kv_heads", m["heads"])), "dim": int(m["dim"]), "vdim": int(m.get("vdim", m["dim"])),
           "scale": float(m["scale"]), "softcap": float(m["softcap"]) if m.get("softcap") else None,
           "window": int(mask["size"]) if mask.get("size") else None, "rot": _rot_spec(m)}
    if m.get("kv_from") is not None:
        out["kv_from"] = int(m["kv_from"])
    return out


@dataclass
class GibavikConfig:
    vocab_size: int
    width: int
    eps: float
    embedding_scale: float
    logit_softcap: float
    layers: list = field(default_factory=list)     # per layer: {"type", "mixer": {...}, "mlp": {...} | None}
    torch_dtype: str = "bfloat16"
    architecture: str = "Gibavik"

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict) -> "GibavikConfig":
        layers = []
        for i, layer in enumerate(d["layers"]):
            kind, m, mlp = layer["type"], layer["mixer"], layer.get("mlp")
            if kind == "attention":
                m = _softmax_spec(m)
                src = m.get("kv_from")
                if src is not None:
                    if not (0 <= src < i and layers[src]["type"] == "attention" and "kv_from" not in layers[src]["mixer"]):
                        raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with keys and values of its own")
                    theirs = layers[src]["mixer"]
                    if any(theirs[k] != m[k] for k in ("kv_heads", "dim", "vdim")):
                        raise ValueError(f"layer {i}: its key/value heads and sizes must equal those of layer {src}")
            elif kind == "parallel":
                r = m["right"]
                decay = [float(v) for v in r["decay"]]
                if len(decay) != int(r["heads"]):
                    raise ValueError(f"layer {i}: one decay per head")
                m = {"left": _softmax_spec(m["left"]), "left_scale": float(m.get("left_scale", 1.0)), "right_scale": float(m.get("right_scale", 1.0)),
                     "right": {"heads": int(r["heads"]), "dim": int(r["dim"]), "vdim": int(r.get("vdim", r["dim"])), "decay": decay}}
            else:
                raise ValueError(f"layer {i}: unknown mixer {kind!r} (known: {MIXERS})")
            if mlp is not None:
                if mlp.get("kind") == "dense":
                    mlp = {"kind": "dense", "ff": int(mlp["ff"]), "limit": float(mlp["limit"])}
                elif mlp.get("kind") == "moe":
                    mlp = {"kind": "moe", "expert": {"ff": int(mlp["expert"]["ff"])},
                           "router": {"experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"])}}
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append({"type": kind, "mixer": m, "mlp": mlp})
        return cls(vocab_size=int(d["vocab"]), width=int(d["width"]), eps=float(d["norm"]["eps"]),
                   embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)), logit_softcap=float(d.get("logit_softcap") or 0.0),
                   layers=layers, torch_dtype=d.get("torch_dtype", d.get("dtype", "bfloat16")))

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            def soft(m):
                out = {k: m[k] for k in ("heads", "kv_heads", "dim", "vdim", "scale")}
                if m["softcap"]:
                    out["softcap"] = m["softcap"]
                if m["window"]:
                    out["mask"] = {"size": m["window"]}
                if m["rot"]:
                    out["rot"] = {"dims": m["rot"]["dims"], "base": m["rot"]["base"]}
                    if m["rot"]["interleaved"]:
                        out["rot"]["layout"] = "interleaved"
                if "kv_from" in m:
                    out["kv_from"] = m["kv_from"]
                return out
            m = layer["mixer"]
            mixer = soft(m) if layer["type"] == "attention" else {"left": soft(m["left"]), "right": dict(m["right"]), "left_scale": m["left_scale"],
                                                                 "right_scale": m["right_scale"]}
            layers.append({"type": layer["type"], "mixer": mixer, "mlp": layer["mlp"]})
        return {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.eps},
                "embedding": {"scale": self.embedding_scale}, "logit_softcap": self.logit_softcap, "layers": layers}


def _f32(*shape):
    return nn.Parameter(torch.zeros(*shape, dtype=torch.float32))


class ParallelMixer(nn.Module):
    """Windowed attention (left) and decayed linear attention (right) on the same input: one matrix product gives both their
    projections (rows: left q | k | v | g, right q | k | v | g); the boundary kernel forms left_scale * left + right_scale * right."""

    def __init__(self, width: int, m: dict, eps: float, i: int):
        super().__init__()
        a, r = m["left"], m["right"]
        self.left = NormedAttention(width, a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["scale"], eps, cache_names=((i, "k"), (i, "v")),
                                    qk_norm="head", rot=a["rot"], rotate_values=a["rot"] is not None, softcap=a["softcap"], window=a["window"],
                                    out_gate=True, bias=True, own_proj=False)
        self.right = DecayLinearAttention(width, r["heads"], r["dim"], r["vdim"], r["decay"], eps, state_name=(i, "mix"), own_proj=False)
        self.in_proj = nn.Linear(width, self.left.proj_rows + self.right.proj_rows, bias=True)
        nn.init.zeros_(self.in_proj.bias)      # it stays zero where the design has no bias (the gates, the right branch)
        self.left_scale, self.right_scale = m["left_scale"], m["right_scale"]


class DenseGLU(nn.Module):
    """W_down (g sigmoid(alpha g) (u + 1)) with g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); gate and up are one product."""

    def __init__(self, width: int, ff: int, limit: float, alpha: float):
        super().__init__()
        self.ff, self.limit, self.alpha = ff, float(limit), float(alpha)
        self.gu_proj = nn.Linear(width, 2 * ff, bias=False)      # rows: gate | up
        self.down = nn.Linear(ff, width, bias=False)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(ops.moe_glu(self.gu_proj(h), self.limit, self.alpha, 1.0))


class GibavikLayer(nn.Module):
    def __init__(self, cfg: GibavikConfig, i: int):
        super().__init__()
        spec = cfg.layers[i]
        w, m = cfg.width, spec["mixer"]
        self.kind = spec["type"]
        if self.kind == "attention":
            src = m.get("kv_from")
            self.mixer = NormedAttention(w, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], cfg.eps, cache_names=((i, "k"), (i, "v")),
                                         qk_norm="row", rot=m["rot"], softcap=m["softcap"], window=m["window"], distance_penalty=True, bias=True,
                                         kv_source=None if src is None else ((src, "k"), (src, "v")))
        else:
            self.mixer = ParallelMixer(w, m, cfg.eps, i)
        self.norm1 = _f32(1)
        mlp = spec["mlp"]
        self.mlp_kind = mlp["kind"] if mlp is not None else None
        self.mlp = None
        if mlp is not None:
            if mlp["kind"] == "dense":
                self.mlp = DenseGLU(w, mlp["ff"], mlp["limit"], GLU_SLOPE)
            else:
                self.mlp = TableMoE(w, mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"], cfg.vocab_size)
            self.norm2 = _f32(1)


class GibavikForCausalLM(nn.Module):
    family = "seq_state"       # per-token cache rows + per-sequence state slots; ragged steps

    def __init__(self, cfg: GibavikConfig):
        super().__init__()
        if tpd.tp_size() * tpd.pp_size() != 1:
            raise NotImplementedError("Gibavik runs on one rank: its recurrent state and token cache are not sharded")
        self.config = cfg
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
        self.layers = nn.ModuleList(GibavikLayer(cfg, i) for i in range(len(cfg.layers)))
        self.final_norm = _f32(1)
        self.head = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
        self.metadata = None
        self.layer_streams = None      # a list: forward() appends a copy of the residual stream after every layer (diagnostics)
        self.start_layer, self.end_layer = 0, len(cfg.layers)

    # -- what the runner asks -------------------------------------------------------------------------
    def finalize(self):
        pass

    def pack_decode_weights(self):
        pass

    def set_attention_metadata(self, metadata):
        self.metadata = metadata

    def latent_ranks(self) -> dict:
        """Rows of the per-token cache: name -> elements per token (keys and values of every attention that has its own)."""
        rows = {}
        for l in self.layers:
            rows.update((l.mixer.left if l.kind == "parallel" else l.mixer).cache_rows())
        return rows

    def state_shapes(self) -> dict:
        shapes = {}
        for l in self.layers:
            if l.kind == "parallel":
                shapes.update(l.mixer.right.state_shapes())
        return shapes

    # -- forward ----------------------------------------------------------------------------------------
    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Final-normed hidden states (tokens, width) in the activations' format."""
        md, cfg = self.metadata, self.config
        assert md is not None
        eps = cfg.eps
        decode_step = md.layout.qo_indptr is None
        x, h = ops.embed_scale(input_ids, self.embed, cfg.embedding_scale)
        n_layers = len(self.layers)
        if n_layers == 0:
            return ops.postnorm_residual(x, w_next=self.final_norm, eps=eps, out_dtype=self.embed.dtype)
        # the experts of a token hang on its id alone: every layer's choices and expert order are made now, with one host read
        plans = TableMoE.plan_step([l.mlp if l.mlp_kind == "moe" else None for l in self.layers], input_ids, decode_step)
        for i, layer in enumerate(self.layers):
            last = i + 1 == n_layers
            closing = self.final_norm if last and layer.mlp is None else None
            if layer.kind == "parallel":
                mx = layer.mixer
                p = mx.in_proj(h)
                h = ops.postnorm_residual(x, y=mx.left.attend(p, 0, positions, md), y2=mx.right.mix(p, mx.left.proj_rows, md), a=mx.left_scale,
                                          b=mx.right_scale, w_post=layer.norm1, eps=eps, w_next=closing)
            else:
                h = ops.postnorm_residual(x, y=layer.mixer(h, positions, md), w_post=layer.norm1, eps=eps, w_next=closing)
            if layer.mlp is not None:
                y = layer.mlp(h) if layer.mlp_kind == "dense" else layer.mlp(h, input_ids, decode_step, plan=plans[i])
                h = ops.postnorm_residual(x, y=y, w_post=layer.norm2, eps=eps, w_next=self.final_norm if last else None)
            if self.layer_streams is not None:
                self.layer_streams.append(x.clone())
        return h

    def compute_logits(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """float32 logits, through cap * tanh(. / cap) where the model has a cap."""
        return ops.tanh_cap(F.linear(hidden_states, self.head), self.config.logit_softcap)

    # -- weights ----------------------------------------------------------------------------------------
    @torch.no_grad()
    def load_weights(self, weights: Iterable):
        """Checkpoint tensors under the design's names ('embed', 'l<i>.mix.left.q', 'l<i>.mlp.e<j>.up', ...) -> the fused parameters."""
        got = set()
        for name, w in weights:
            self._load_one(name, w)
            got.add(name)
        missing = [n for n in checkpoint_names(self.config) if n not in got]
        if missing:
            raise KeyError(f"checkpoint lacks {len(missing)} tensors, e.g. {missing[:4]}")

    def _load_one(self, name: str, w: torch.Tensor):
        def put(p, rows=None):
            dst = p if rows is None else p[rows[0]:rows[1]]
            src = w.reshape(dst.shape) if w.numel() == dst.numel() == 1 else w      # a norm's one number is stored without a shape
            if dst.shape != src.shape:
                raise ValueError(f"{name}: checkpoint shape {tuple(w.shape)}, model wants {tuple(dst.shape)}")
            dst.copy_(src)

        top = {"embed": self.embed, "final.norm": self.final_norm, "head": self.head}
        if name in top:
            return put(top[name])
        head, _, rest = name.partition(".")
        if not (head[:1] == "l" and head[1:].isdigit() and int(head[1:]) < len(self.layers)):
            raise KeyError(f"unexpected tensor {name!r}")
        layer = self.layers[int(head[1:])]
        if rest in ("norm1", "norm2") and hasattr(layer, rest):
            return put(getattr(layer, rest))
        if rest.startswith("mlp.") and layer.mlp is not None:
            what = rest[4:]
            if layer.mlp_kind == "dense":
                ff = layer.mlp.ff
                where = {"gate": (layer.mlp.gu_proj.weight, (0, ff)), "up": (layer.mlp.gu_proj.weight, (ff, 2 * ff)), "down": (layer.mlp.down.weight, None)}
                if what in where:
                    return put(*where[what])
            else:
                moe = layer.mlp
                if what == "table":
                    if w.dtype not in (torch.int32, torch.int64) or w.shape != moe.table.shape:
                        raise ValueError(f"{name}: the experts' table must be integers of shape {tuple(moe.table.shape)}")
                    if int(w.min()) < 0 or int(w.max()) >= moe.experts:
                        raise ValueError(f"{name}: expert ids outside 0..{moe.experts - 1}")
                    return moe.table.copy_(w)
                e, _, part = what.partition(".")
                if e[:1] == "e" and e[1:].isdigit() and int(e[1:]) < moe.experts:
                    j, ff = int(e[1:]), moe.ff
                    where = {"gate": (moe.w_gu[j], (0, ff)), "up": (moe.w_gu[j], (ff, 2 * ff)), "down": (moe.w_d[j], None)}
                    if part in where:
                        return put(*where[part])
        if rest.startswith("mix."):
            where = self._mixer_targets(layer).get(rest[4:])
            if where is not None:
                return put(*where)
        raise KeyError(f"unexpected tensor {name!r}")

    @staticmethod
    def _attention_targets(a: NormedAttention, proj: nn.Linear, col0: int, prefix: str) -> dict:
        """Checkpoint names of one softmax attention -> (parameter, row range or None); its projections are rows of `proj` from col0."""
        out = {}
        at = col0
        for s, n in (("q", a.q_cols), ("k", a.k_cols), ("v", a.v_cols), ("g", a.g_cols)):
            if n:
                out[prefix + s] = (proj.weight, (at, at + n))
                if a.has_bias and s != "g":
                    out[prefix + s + ".b"] = (proj.bias, (at, at + n))
            at += n
        if a.qk_norm != "none":
            out[prefix + "q.norm"] = (a.q_norm, None)
            if not a.borrows:
                out[prefix + "k.norm"] = (a.k_norm, None)
        if a.r1 is not None:
            out[prefix + "r1"], out[prefix + "r2"] = (a.r1, None), (a.r2, None)
        out[prefix + "o"] = (a.o_proj.weight, None)
        return out

    @classmethod
    def _mixer_targets(cls, layer) -> dict:
        m = layer.mixer
        if layer.kind == "attention":
            return cls._attention_targets(m, m.in_proj, 0, "")
        out = cls._attention_targets(m.left, m.in_proj, 0, "left.")
        r, p, at = m.right, m.in_proj.weight, m.left.proj_rows
        hd, he = r.heads * r.dim, r.heads * r.vdim
        for s, n in (("q", hd), ("k", hd), ("v", he), ("g", he)):
            out["right." + s] = (p, (at, at + n))
            at += n
        out["right.norm"], out["right.o"] = (r.norm, None), (r.o_proj.weight, None)
        return out

    @torch.no_grad()
    def init_random(self, seed: int = 0):
        self.load_weights(random_checkpoint(self.config, seed))


def checkpoint_shapes(cfg: GibavikConfig) -> dict:
    """name -> shape of every tensor of a checkpoint of this configuration."""
    w, shapes = cfg.width, {"embed": (cfg.vocab_size, cfg.width)}

    def soft(p, a, per_head_norm, gate, penalty):
        qd, kd, vd = a["heads"] * a["dim"], a["kv_heads"] * a["dim"], a["kv_heads"] * a["vdim"]
        shapes.update({p + "q": (qd, w), p + "q.b": (qd,), p + "q.norm": (a["dim"] if per_head_norm else qd,)})
        if "kv_from" not in a:
            shapes.update({p + "k": (kd, w), p + "k.b": (kd,), p + "v": (vd, w), p + "v.b": (vd,), p + "k.norm": (a["dim"] if per_head_norm else kd,)})
        if gate:
            shapes[p + "g"] = (a["heads"] * a["vdim"], w)
        if penalty:
            shapes[p + "r1"], shapes[p + "r2"] = (a["heads"],), (a["heads"],)
        shapes[p + "o"] = (w, a["heads"] * a["vdim"])

    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer["mixer"]
        shapes[p + "norm1"] = ()
        if layer["type"] == "attention":
            soft(p + "mix.", m, False, False, True)
        else:
            soft(p + "mix.left.", m["left"], True, True, False)
            r = m["right"]
            hd, he = r["heads"] * r["dim"], r["heads"] * r["vdim"]
            shapes.update({p + "mix.right.q": (hd, w), p + "mix.right.k": (hd, w), p + "mix.right.v": (he, w), p + "mix.right.g": (he, w),
                           p + "mix.right.o": (w, he), p + "mix.right.norm": (he,)})
        mlp = layer["mlp"]
        if mlp is not None:
            shapes[p + "norm2"] = ()
            if mlp["kind"] == "dense":
                shapes.update({p + "mlp.gate": (mlp["ff"], w), p + "mlp.up": (mlp["ff"], w), p + "mlp.down": (w, mlp["ff"])})
            else:
                ff, n = mlp["expert"]["ff"], mlp["router"]["experts"]
                for j in range(n):
                    shapes.update({f"{p}mlp.e{j}.gate": (ff, w), f"{p}mlp.e{j}.up": (ff, w), f"{p}mlp.e{j}.down": (w, ff)})
                shapes[p + "mlp.table"] = (cfg.vocab_size, mlp["router"]["top"])
    shapes["final.norm"] = ()
    shapes["head"] = (cfg.vocab_size, w)
    return shapes


def checkpoint_names(cfg: GibavikConfig) -> list:
    return list(checkpoint_shapes(cfg))


def random_checkpoint(cfg: GibavikConfig, seed: int = 0):
    """(name, tensor) pairs of a seeded random checkpoint, rounded to bfloat16 values (as a stored checkpoint is), one tensor at a
    time.  Matrices are scaled by 1/sqrt(fan-in); norm weights are near one; biases and distance numbers are small; every row of
    an experts' table holds different experts."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    experts = {f"l{i}.mlp.table": l["mlp"]["router"]["experts"] for i, l in enumerate(cfg.layers) if l["mlp"] is not None and l["mlp"]["kind"] == "moe"}
    for name, shape in checkpoint_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if name in experts:
            yield name, torch.stack([torch.randperm(experts[name], generator=gen)[:shape[1]] for _ in range(shape[0])]).to(torch.int32)
            continue
        rnd = torch.randn(shape, generator=gen)
        if leaf in ("norm", "norm1", "norm2"):
            w = 1.0 + 0.1 * rnd
        elif leaf == "b":
            w = 0.2 * rnd
        elif leaf == "r1":
            w = 0.5 + 0.25 * torch.rand(shape, generator=gen)
        elif leaf == "r2":
            w = 0.05 + 0.2 * torch.rand(shape, generator=gen)
        elif name == "embed":
            w = rnd
        else:
            w = rnd * shape[-1] ** -0.5
        yield name, w.to(torch.bfloat16).float()
