"""Ladusun: a pre-normed decoder stack over SEVERAL residual streams (hyper-connections), float32 throughout:
    all streams start as embed[token] * embedding.scale;  a sublayer reads u = sum_s in[s] x_s, computes y = ls * f(rmsnorm(u) * w)
    (ls: a weight per channel), and every stream moves at once: x_j <- sum_s mix[s, j] x_s + out[j] y;
    logits = embed @ (rmsnorm(sum_s x_s) * w_final)  (the table itself, without its scale).
A configuration without `streams` has one stream and the plain sum x <- x + y.

A layer's mixer is one of
  attention         grouped heads, biased projections, rotary positions on a leading part of each head in neighbouring pairs
                    (frequencies stretched by wavelength bands), capped scores, a softmax whose denominator has one more term of
                    score 0, one sigmoid output gate per head; a layer may read the cached keys and values of an earlier attention
                    layer (`kv_from`) and then has queries, gates and an output projection only;
  latent_attention  one normed latent per token from which every head's keys and values are linear maps, plus one rotated key part
                    shared by the heads (YaRN-stretched frequencies); plain softmax; one sigmoid output gate per head;
  rglru             a gelu branch times a real-gated linear recurrence behind a short causal convolution;
and its feed-forward is dense (W_down relu(W_up h + b)^2 + b), a mixture of experts behind a softmax router with groups, or absent.

config.json gives every size, the order of the layers and the constants; the mechanisms live in layers/ (cap_attention.py,
latent_attention.py, recurrent.py, moe.py) with their constants as arguments.  Between the matrix products (library GEMMs; all
input projections of a mixer are ONE product) every step is a HIP kernel of this package, one launch per sublayer boundary
(ops.hyper_mix: layer scale, the streams' mixing, the next sublayer's read weights and its norm).  The streams, norms, attention
scores, positions and angles, routers, gates of the recurrence and its state are float32 in every activation format.
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
from .layers.latent_attention import RotaryLatentAttention
from .layers.moe import GroupedSoftmaxMoE
from .layers.recurrent import RGLRU

MIXERS = ("attention", "latent_attention", "rglru")
SINK_SCORE = 0.0          # the extra term of the attention's softmax sum is exp(0)
RGLRU_DECAY_SCALE = 8.0   # log a = -8 r softplus(lam)
GLU_SLOPE = 1.702         # expert: y = g sigmoid(1.702 g) (u + 1)
ROUTER_NORM_EPS = 1e-20   # chosen scores / (their sum + 1e-20)


def _rot(m: dict, dims=None):
    rot = m.get("rot") or {}
    out = {"dims": int(rot.get("dims", 0) if dims is None else dims), "base": float(rot.get("base", 10000.0)), "interleaved": True}
    if rot.get("scaling"):
        out["scaling"] = {k: float(v) for k, v in rot["scaling"].items()}
    return out


@dataclass
class LadusunConfig:
    vocab_size: int
    width: int
    eps: float
    embedding_scale: float
    streams: int | None                      # None: one stream, plain residual sum (no hyper-connection tensors)
    layers: list = field(default_factory=list)     # per layer: {"type", "mixer": {...}, "mlp": {...} | None}
    torch_dtype: str = "bfloat16"
    architecture: str = "Ladusun"

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def n_streams(self) -> int:
        return self.streams or 1

    @classmethod
    def from_dict(cls, d: dict) -> "LadusunConfig":
        layers = []
        for i, layer in enumerate(d["layers"]):
            kind, m, mlp = layer["type"], layer["mixer"], layer.get("mlp")
            if kind == "attention":
                heads = int(m["heads"])
                m2 = {"heads": heads, "kv_heads": int(m.get("kv_heads", heads)), "dim": int(m["dim"]), "vdim": int(m.get("vdim", m["dim"])),
                      "scale": float(m["scale"]), "softcap": float(m["softcap"]) if m.get("softcap") else None, "rot": _rot(m)}
                src = m.get("kv_from")
                if src is not None:
                    src = int(src)
                    if not (0 <= src < i and layers[src]["type"] == "attention" and "kv_from" not in layers[src]["mixer"]):
                        raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with keys and values of its own")
                    theirs = layers[src]["mixer"]
                    if any(theirs[k] != m2[k] for k in ("kv_heads", "dim", "vdim")):
                        raise ValueError(f"layer {i}: its key/value heads and sizes must equal those of layer {src}")
                    m2["kv_from"] = src
                m = m2
            elif kind == "latent_attention":
                rot_dim = int(m.get("rot_dim", 0))
                m = {"heads": int(m["heads"]), "dim": int(m["dim"]), "rot_dim": rot_dim, "vdim": int(m.get("vdim", m["dim"])),
                     "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]), "rot": _rot(m, rot_dim)}
            elif kind == "rglru":
                m = {"width": int(m["width"]), "blocks": int(m.get("blocks", 1)), "conv": int(m.get("conv", 1))}
            else:
                raise ValueError(f"layer {i}: unknown mixer {kind!r} (known: {MIXERS})")
            if mlp is not None:
                if mlp.get("kind") == "dense":
                    mlp = {"kind": "dense", "ff": int(mlp["ff"])}
                elif mlp.get("kind") == "moe":
                    r, groups = mlp["router"], mlp["router"].get("groups")
                    mlp = {"kind": "moe", "expert": {"ff": int(mlp["expert"]["ff"]), "limit": float(mlp["expert"]["limit"])},
                           "router": {"experts": int(r["experts"]), "top": int(r["top"]),
                                      "groups": {"count": int(groups["count"]), "keep": int(groups["keep"])} if groups else None}}
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append({"type": kind, "mixer": m, "mlp": mlp})
        streams = d.get("streams")
        return cls(vocab_size=int(d["vocab"]), width=int(d["width"]), eps=float(d["norm"]["eps"]),
                   embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)), streams=int(streams) if streams is not None else None,
                   layers=layers, torch_dtype=d.get("torch_dtype", d.get("dtype", "bfloat16")))

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            m = dict(layer["mixer"])
            if "rot" in m:
                rot = {k: v for k, v in m["rot"].items() if k != "interleaved"}
                if layer["type"] == "latent_attention":
                    rot.pop("dims")
                m["rot"] = rot
            if m.get("softcap", 0) is None:
                m.pop("softcap")
            mlp = layer["mlp"]
            if mlp is not None and mlp["kind"] == "moe" and mlp["router"]["groups"] is None:
                mlp = {**mlp, "router": {k: v for k, v in mlp["router"].items() if k != "groups"}}
            layers.append({"type": layer["type"], "mixer": m, "mlp": mlp})
        out = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.width, "norm": {"eps": self.eps},
               "embedding": {"scale": self.embedding_scale}, "layers": layers}
        if self.streams is not None:
            out["streams"] = self.streams
        return out


def _f32(*shape):
    return nn.Parameter(torch.zeros(*shape, dtype=torch.float32))


class DenseRelu2(nn.Module):
    """W_down relu(W_up h + b_up)^2 + b_down."""

    def __init__(self, width: int, ff: int):
        super().__init__()
        self.ff = ff
        self.up = nn.Linear(width, ff, bias=True)
        self.down = nn.Linear(ff, width, bias=True)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(ops.relu2(self.up(h)))


class HyperConnection(nn.Module):
    """What one sublayer needs at its two ends: the weights it reads the streams with and its norm (in front), its layer scale, the
    streams' mixing matrix ([from, to]) and the weights its result enters them with (behind).  With `learned` False the streams'
    numbers are constants of a single plain residual stream."""

    def __init__(self, width: int, streams: int, learned: bool):
        super().__init__()
        self.norm, self.ls = _f32(width), _f32(width)
        if learned:
            self.w_in, self.w_out, self.mix = _f32(streams), _f32(streams), _f32(streams, streams)
        else:
            assert streams == 1
            for name in ("w_in", "w_out", "mix"):
                self.register_buffer(name, torch.ones(1, dtype=torch.float32), persistent=False)


class LadusunLayer(nn.Module):
    def __init__(self, cfg: LadusunConfig, i: int):
        super().__init__()
        spec = cfg.layers[i]
        w, m = cfg.width, spec["mixer"]
        self.kind = spec["type"]
        if self.kind == "attention":
            src = m.get("kv_from")
            self.mixer = NormedAttention(w, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], cfg.eps, cache_names=((i, "k"), (i, "v")),
                                         qk_norm="none", rot=m["rot"] if m["rot"]["dims"] else None, softcap=m["softcap"], out_gate="head", bias=True,
                                         o_bias=True, sink_score=SINK_SCORE, kv_source=None if src is None else ((src, "k"), (src, "v")))
        elif self.kind == "latent_attention":
            self.mixer = RotaryLatentAttention(w, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"], cfg.eps, m["rot"], cache_name=i)
        else:
            self.mixer = RGLRU(w, m["width"], m["blocks"], m["conv"], RGLRU_DECAY_SCALE, state_name=(i, "mix"))
        learned = cfg.streams is not None
        self.hc1 = HyperConnection(w, cfg.n_streams, learned)
        mlp = spec["mlp"]
        self.mlp_kind = mlp["kind"] if mlp is not None else None
        self.mlp = None
        if mlp is not None:
            if mlp["kind"] == "dense":
                self.mlp = DenseRelu2(w, mlp["ff"])
            else:
                r, g = mlp["router"], mlp["router"]["groups"]
                self.mlp = GroupedSoftmaxMoE(w, r["experts"], r["top"], mlp["expert"]["ff"], mlp["expert"]["limit"], GLU_SLOPE, 1.0,
                                             groups=g["count"] if g else None, keep=g["keep"] if g else None, norm_eps=ROUTER_NORM_EPS)
            self.hc2 = HyperConnection(w, cfg.n_streams, learned)


class LadusunForCausalLM(nn.Module):
    family = "seq_state"       # per-token cache rows + per-sequence state slots; ragged steps

    def __init__(self, cfg: LadusunConfig):
        super().__init__()
        if tpd.tp_size() * tpd.pp_size() != 1:
            raise NotImplementedError("Ladusun runs on one rank: its recurrent state and token cache are not sharded")
        self.config = cfg
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.width))
        self.layers = nn.ModuleList(LadusunLayer(cfg, i) for i in range(len(cfg.layers)))
        self.final_norm = _f32(cfg.width)
        self.metadata = None
        self._subs = None
        self.layer_streams = None      # a list: forward() appends the sum of the streams after every layer (diagnostics)
        self.start_layer, self.end_layer = 0, len(cfg.layers)

    # -- what the runner asks -------------------------------------------------------------------------
    def finalize(self):
        pass

    def pack_decode_weights(self):
        """Called when the weights are in place: constants that are functions of them."""
        for l in self.layers:
            if l.kind == "rglru":
                l.mixer.finalize()

    def set_attention_metadata(self, metadata):
        self.metadata = metadata

    def latent_ranks(self) -> dict:
        """Rows of the per-token cache: name -> elements per token (keys and values of every attention that has its own, the
        latent row of every latent attention)."""
        rows = {}
        for l in self.layers:
            if l.kind != "rglru":
                rows.update(l.mixer.cache_rows())
        return rows

    def state_shapes(self) -> dict:
        shapes = {}
        for l in self.layers:
            if l.kind == "rglru":
                shapes.update(l.mixer.state_shapes())
        return shapes

    # -- forward ----------------------------------------------------------------------------------------
    def sublayers(self) -> list:
        """(hyper-connection, function of (h, positions, metadata, decode step), whether a layer ends here) of every sublayer, in order."""
        if self._subs is None:
            out = []
            for l in self.layers:
                if l.kind == "rglru":
                    out.append((l.hc1, lambda h, pos, md, dec, m=l.mixer: m(h, md), l.mlp is None))
                else:
                    out.append((l.hc1, lambda h, pos, md, dec, m=l.mixer: m(h, pos, md), l.mlp is None))
                if l.mlp_kind == "dense":
                    out.append((l.hc2, lambda h, pos, md, dec, f=l.mlp: f(h), True))
                elif l.mlp_kind == "moe":
                    out.append((l.hc2, lambda h, pos, md, dec, f=l.mlp: f(h, dec), True))
            self._subs = out
        return self._subs

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        """Final-normed hidden states (tokens, width) in the activations' format."""
        md, cfg = self.metadata, self.config
        assert md is not None
        eps, dtype = cfg.eps, self.embed.dtype
        decode_step = md.layout.qo_indptr is None
        x0, _ = ops.embed_scale(input_ids, self.embed, cfg.embedding_scale)
        subs = self.sublayers()
        first = subs[0][0] if subs else None
        x, h = ops.hyper_mix(x0, w_in=first.w_in if first else None, w_norm=first.norm if first else self.final_norm, eps=eps,
                             n_streams=cfg.n_streams, out_dtype=dtype)
        for i, (hc, fn, layer_ends) in enumerate(subs):
            y = fn(h, positions, md, decode_step)
            nxt = subs[i + 1][0] if i + 1 < len(subs) else None
            x, h = ops.hyper_mix(x, y, scale=hc.ls, mix=hc.mix, w_out=hc.w_out, w_in=nxt.w_in if nxt else None,
                                 w_norm=nxt.norm if nxt else self.final_norm, eps=eps)
            if layer_ends and self.layer_streams is not None:
                self.layer_streams.append(x.sum(1))
        return h

    def compute_logits(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """float32 logits against the embedding table itself."""
        return F.linear(hidden_states, self.embed).float()

    # -- weights ----------------------------------------------------------------------------------------
    @torch.no_grad()
    def load_weights(self, weights: Iterable):
        """Checkpoint tensors under the design's names ('embed', 'l<i>.mix.q', 'l<i>.hc1.mix', 'l<i>.mlp.e<j>.up', ...) -> the fused
        parameters.  Every tensor the configuration calls for must be there, in its shape; a tensor it does not call for is left
        out with a warning (nothing of the model reads it)."""
        wanted, got, surplus = checkpoint_shapes(self.config), set(), []
        for name, w in weights:
            if name not in wanted:
                surplus.append(name)
                continue
            self._load_one(name, w)
            got.add(name)
        missing = [n for n in wanted if n not in got]
        if missing:
            raise KeyError(f"checkpoint lacks {len(missing)} tensors, e.g. {missing[:4]}")
        if surplus:
            import warnings
            warnings.warn(f"checkpoint holds {len(surplus)} tensors that this configuration does not use, e.g. {surplus[:4]}")
        self.pack_decode_weights()

    def _load_one(self, name: str, w: torch.Tensor):
        def put(p, rows=None, transpose=False):
            dst = p if rows is None else p[rows[0]:rows[1]]
            src = w.t() if transpose else w
            if dst.shape != src.shape:
                raise ValueError(f"{name}: checkpoint shape {tuple(w.shape)}, model wants {tuple(dst.shape)}")
            dst.copy_(src)

        top = {"embed": self.embed, "final.norm": self.final_norm}
        if name in top:
            return put(top[name])
        head, _, rest = name.partition(".")
        if not (head[:1] == "l" and head[1:].isdigit() and int(head[1:]) < len(self.layers)):
            raise KeyError(f"unexpected tensor {name!r}")
        layer = self.layers[int(head[1:])]
        for q in ("1", "2"):
            hc = getattr(layer, "hc" + q, None)
            if hc is None:
                continue
            simple = {"norm" + q: hc.norm, "ls" + q: hc.ls}
            if self.config.streams is not None:
                simple.update({f"hc{q}.in": hc.w_in, f"hc{q}.out": hc.w_out, f"hc{q}.mix": hc.mix})
            if rest in simple:
                return put(simple[rest])
        if rest.startswith("mlp.") and layer.mlp is not None:
            what = rest[4:]
            if layer.mlp_kind == "dense":
                f = layer.mlp
                where = {"up": f.up.weight, "up.b": f.up.bias, "down": f.down.weight, "down.b": f.down.bias}
                if what in where:
                    return put(where[what])
            else:
                moe = layer.mlp
                if what == "router":
                    return put(moe.router)
                e, _, part = what.partition(".")
                if e[:1] == "e" and e[1:].isdigit() and int(e[1:]) < moe.experts:
                    j, ff = int(e[1:]), moe.ff
                    where = {"gate": (moe.w_gu[j], (0, ff)), "up": (moe.w_gu[j], (ff, 2 * ff)), "down": (moe.w_d[j], None)}
                    if part in where:
                        return put(*where[part])
        if rest.startswith("mix."):
            what, m = rest[4:], layer.mixer
            if layer.kind == "attention":
                at = 0
                for s, n in (("q", m.q_cols), ("k", m.k_cols), ("v", m.v_cols), ("g", m.g_cols)):
                    if n and what == s:
                        return put(m.in_proj.weight, (at, at + n))
                    if n and s != "g" and what == s + ".b":
                        return put(m.in_proj.bias, (at, at + n))
                    at += n
                if what == "o":
                    return put(m.o_proj.weight)
                if what == "o.b":
                    return put(m.o_proj.bias)
            elif layer.kind == "latent_attention":
                q, kv = m.q_cols, m.kv_cols
                where = {"q": (m.in_proj.weight, (0, q)), "dkv": (m.in_proj.weight, (q, q + kv)), "g": (m.in_proj.weight, (q + kv, q + kv + m.heads)),
                         "dkv.norm": (m.kv_norm, None), "o": (m.o_proj.weight, None)}
                if what in where:
                    return put(*where[what])
                if what in ("uk", "uv"):
                    want = (m.heads * (m.dim if what == "uk" else m.vdim), m.kv_rank)
                    if tuple(w.shape) != want:
                        raise ValueError(f"{name}: checkpoint shape {tuple(w.shape)}, model wants {want}")
                    return m.load_maps(**{what: w.to(m.uk.dtype)})
            else:
                n, bw = m.inner, m.inner // m.blocks
                where = {"y": (m.in_proj.weight, (0, n)), "y.b": (m.in_proj.bias, (0, n)), "x": (m.in_proj.weight, (n, 2 * n)),
                         "x.b": (m.in_proj.bias, (n, 2 * n)), "conv.b": (m.conv_b, None), "lam": (m.lam, None), "o": (m.o_proj.weight, None)}
                if what in where:
                    return put(*where[what])
                if what == "conv":                      # stored (channels, taps), kept (taps, channels)
                    return put(m.conv_w, transpose=True)
                if what in ("ra", "ri"):                # stored per block [out, in]; kept per block [in, out] with both gates side by side
                    if tuple(w.shape) != (m.blocks, bw, bw):
                        raise ValueError(f"{name}: checkpoint shape {tuple(w.shape)}, model wants {(m.blocks, bw, bw)}")
                    c0 = 0 if what == "ra" else bw
                    return m.gate_w[:, :, c0:c0 + bw].copy_(w.transpose(1, 2))
                if what in ("ra.b", "ri.b"):
                    if tuple(w.shape) != (m.blocks, bw):
                        raise ValueError(f"{name}: checkpoint shape {tuple(w.shape)}, model wants {(m.blocks, bw)}")
                    return m.gate_b[0 if what == "ra.b" else 1].copy_(w.reshape(-1))
        raise KeyError(f"unexpected tensor {name!r}")

    @torch.no_grad()
    def init_random(self, seed: int = 0):
        self.load_weights(random_checkpoint(self.config, seed))


def checkpoint_shapes(cfg: LadusunConfig) -> dict:
    """name -> shape of every tensor of a checkpoint of this configuration."""
    w, s, shapes = cfg.width, cfg.n_streams, {"embed": (cfg.vocab_size, cfg.width)}
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer["mixer"]
        shapes.update({p + "norm1": (w,), p + "ls1": (w,)})
        if layer["type"] == "attention":
            qd, kd, vd = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            shapes.update({p + "mix.q": (qd, w), p + "mix.q.b": (qd,)})
            if "kv_from" not in m:
                shapes.update({p + "mix.k": (kd, w), p + "mix.k.b": (kd,), p + "mix.v": (vd, w), p + "mix.v.b": (vd,)})
            shapes.update({p + "mix.g": (m["heads"], w), p + "mix.o": (w, m["heads"] * m["vdim"]), p + "mix.o.b": (w,)})
        elif layer["type"] == "latent_attention":
            h, r = m["heads"], m["kv_rank"]
            shapes.update({p + "mix.q": (h * (m["dim"] + m["rot_dim"]), w), p + "mix.dkv": (r + m["rot_dim"], w), p + "mix.dkv.norm": (r,),
                           p + "mix.uk": (h * m["dim"], r), p + "mix.uv": (h * m["vdim"], r), p + "mix.g": (h, w), p + "mix.o": (w, h * m["vdim"])})
        else:
            n, b, bw = m["width"], m["blocks"], m["width"] // m["blocks"]
            shapes.update({p + "mix.y": (n, w), p + "mix.y.b": (n,), p + "mix.x": (n, w), p + "mix.x.b": (n,), p + "mix.conv": (n, m["conv"]),
                           p + "mix.conv.b": (n,), p + "mix.ra": (b, bw, bw), p + "mix.ra.b": (b, bw), p + "mix.ri": (b, bw, bw),
                           p + "mix.ri.b": (b, bw), p + "mix.lam": (n,), p + "mix.o": (w, n)})
        mlp = layer["mlp"]
        if mlp is not None:
            shapes.update({p + "norm2": (w,), p + "ls2": (w,)})
            if mlp["kind"] == "dense":
                shapes.update({p + "mlp.up": (mlp["ff"], w), p + "mlp.up.b": (mlp["ff"],), p + "mlp.down": (w, mlp["ff"]), p + "mlp.down.b": (w,)})
            else:
                ff, n = mlp["expert"]["ff"], mlp["router"]["experts"]
                for j in range(n):
                    shapes.update({f"{p}mlp.e{j}.gate": (ff, w), f"{p}mlp.e{j}.up": (ff, w), f"{p}mlp.e{j}.down": (w, ff)})
                shapes[p + "mlp.router"] = (n, w)
        if cfg.streams is not None:
            for q in ("1", "2") if mlp is not None else ("1",):
                shapes.update({f"{p}hc{q}.in": (s,), f"{p}hc{q}.out": (s,), f"{p}hc{q}.mix": (s, s)})
    shapes["final.norm"] = (w,)
    return shapes


def checkpoint_names(cfg: LadusunConfig) -> list:
    return list(checkpoint_shapes(cfg))


def random_checkpoint(cfg: LadusunConfig, seed: int = 0):
    """(name, tensor) pairs of a seeded random checkpoint, rounded to bfloat16 values (as a stored checkpoint is), one tensor at a
    time.  Matrices are scaled by 1/sqrt(fan-in); norm weights and layer scales are near one; biases are small; the streams' mixing
    matrices are near the identity and their read and write weights near 1/streams and 1."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    s = cfg.n_streams
    for name, shape in checkpoint_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        rnd = torch.randn(shape, generator=gen)
        if leaf in ("norm", "norm1", "norm2"):
            w = 1.0 + 0.1 * rnd
        elif leaf in ("ls1", "ls2"):
            w = 0.5 + 0.1 * rnd
        elif leaf == "b":
            w = 0.2 * rnd
        elif leaf == "lam":
            w = 0.5 * rnd - 1.0
        elif leaf == "conv":
            w = rnd * 0.5
        elif leaf == "in":
            w = 1.0 / s + 0.1 * rnd
        elif leaf == "out":
            w = 1.0 + 0.1 * rnd
        elif leaf == "mix" and len(shape) == 2 and shape == (s, s) and ".hc" in name:
            w = torch.eye(s) + 0.1 * rnd
        elif name == "embed":
            w = rnd
        else:
            w = rnd * shape[-1] ** -0.5
        yield name, w.to(torch.bfloat16).float()
