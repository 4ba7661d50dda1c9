"""Host side of the Gibavik family, without a device: configuration, registry, checkpoint names and where their tensors land in
the fused parameters, and properties of the restatement that the GPU tests lean on."""
import json

import pytest
import torch

from oracle import gibavik_oracle as go

LEFT = {"heads": 6, "kv_heads": 3, "dim": 12, "vdim": 20, "mask": {"size": 5}, "rot": {"dims": 8, "base": 3000.0}, "scale": 0.25, "softcap": 30.0}
LAYERS = [{"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 10, "vdim": 6, "scale": 0.3}, "mlp": None},
          {"type": "parallel", "mixer": {"left": LEFT, "right": {"heads": 2, "dim": 14, "vdim": 8, "decay": [0.7, 0.99]}, "left_scale": 0.5, "right_scale": 2.0},
           "mlp": {"kind": "moe", "expert": {"ff": 18}, "router": {"experts": 3, "top": 2}}},
          {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 10, "vdim": 6, "scale": 0.1, "kv_from": 0}, "mlp": {"kind": "dense", "ff": 22, "limit": 1.0}}]
CFG = {"architecture": "Gibavik", "vocab": 53, "width": 36, "norm": {"eps": 1e-6}, "embedding": {"scale": 4.0}, "logit_softcap": 12.0, "layers": LAYERS}


def test_registry_reads_the_configuration_from_a_directory(tmp_path):
    from nano_vllm_x_amd.gibavik import GibavikConfig, GibavikForCausalLM
    from nano_vllm_x_amd.registry import load_config, model_class_of
    (tmp_path / "config.json").write_text(json.dumps(CFG))
    cfg = load_config(str(tmp_path))
    assert isinstance(cfg, GibavikConfig) and model_class_of(cfg) is GibavikForCausalLM and GibavikForCausalLM.family == "seq_state"
    assert (cfg.vocab_size, cfg.width, cfg.hidden_size, cfg.eps, cfg.embedding_scale, cfg.logit_softcap) == (53, 36, 36, 1e-6, 4.0, 12.0)
    assert [l["type"] for l in cfg.layers] == ["attention", "parallel", "attention"] and cfg.layers[0]["mlp"] is None
    left = cfg.layers[1]["mixer"]["left"]
    assert left["window"] == 5 and left["softcap"] == 30.0 and left["rot"] == {"dims": 8, "base": 3000.0, "interleaved": False}
    assert cfg.layers[0]["mixer"]["window"] is None and cfg.layers[0]["mixer"]["rot"] is None and cfg.layers[2]["mixer"]["kv_from"] == 0
    again = GibavikConfig.from_dict(json.loads(json.dumps(cfg.to_dict())))
    assert again.layers == cfg.layers and again.eps == cfg.eps and again.logit_softcap == cfg.logit_softcap
    with pytest.raises(ValueError):
        GibavikConfig.from_dict({**CFG, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]})
    with pytest.raises(ValueError):      # keys borrowed from a later layer, or from one that borrows
        GibavikConfig.from_dict({**CFG, "layers": [LAYERS[2], LAYERS[0]]})
    with pytest.raises(ValueError):
        GibavikConfig.from_dict({**CFG, "layers": LAYERS + [{**LAYERS[2], "mixer": {**LAYERS[2]["mixer"], "kv_from": 2}}]})
    with pytest.raises(ValueError):      # other key/value sizes than the lender's
        GibavikConfig.from_dict({**CFG, "layers": LAYERS[:2] + [{**LAYERS[2], "mixer": {**LAYERS[2]["mixer"], "vdim": 8}}]})
    with pytest.raises(ValueError):
        GibavikConfig.from_dict({**CFG, "layers": [{**LAYERS[1], "mixer": {**LAYERS[1]["mixer"], "right": {"heads": 2, "dim": 4, "decay": [0.5]}}}]})


def test_checkpoint_tensors_land_in_the_fused_parameters():
    from nano_vllm_x_amd.gibavik import GibavikConfig, GibavikForCausalLM, checkpoint_shapes, random_checkpoint
    cfg = GibavikConfig.from_dict(CFG)
    w = dict(random_checkpoint(cfg, 3))
    assert {k: tuple(v.shape) for k, v in w.items()} == checkpoint_shapes(cfg)
    assert "l0.norm2" not in w and "l2.mix.k" not in w and "l2.mix.k.norm" not in w and "l2.mix.q.norm" in w and "l1.mlp.e2.down" in w
    assert w["l1.mlp.table"].dtype == torch.int32 and all(len(set(r)) == 2 for r in w["l1.mlp.table"].tolist())
    model = GibavikForCausalLM(cfg).float()
    model.load_weights(w.items())
    a, p, b = model.layers[0].mixer, model.layers[1].mixer, model.layers[2].mixer
    assert torch.equal(a.in_proj.weight[40:60], w["l0.mix.k"]) and torch.equal(a.in_proj.bias[60:72], w["l0.mix.v.b"]) and a.in_proj.weight.shape[0] == 72
    assert torch.equal(a.q_norm, w["l0.mix.q.norm"]) and a.q_norm.numel() == 40 and torch.equal(a.r2, w["l0.mix.r2"])
    rows = p.in_proj.weight
    assert torch.equal(rows[72:108], w["l1.mix.left.k"]) and torch.equal(rows[108:168], w["l1.mix.left.v"]) and torch.equal(rows[168:288], w["l1.mix.left.g"])
    assert torch.equal(rows[288:316], w["l1.mix.right.q"]) and torch.equal(rows[344:360], w["l1.mix.right.v"]) and torch.equal(rows[360:], w["l1.mix.right.g"])
    assert torch.equal(p.in_proj.bias[:72], w["l1.mix.left.q.b"]) and not p.in_proj.bias[168:].any()        # gates and the right branch: no bias
    assert p.left.q_norm.numel() == 12 and torch.equal(p.right.norm, w["l1.mix.right.norm"]) and p.right.decay.tolist() == pytest.approx([0.7, 0.99])
    assert b.in_proj.weight.shape[0] == 20 and torch.equal(b.in_proj.weight, w["l2.mix.q"]) and not hasattr(b, "k_norm")
    moe, dense = model.layers[1].mlp, model.layers[2].mlp
    assert torch.equal(moe.w_gu[2, 18:], w["l1.mlp.e2.up"]) and torch.equal(moe.w_d[0], w["l1.mlp.e0.down"]) and torch.equal(moe.table, w["l1.mlp.table"])
    assert torch.equal(dense.gu_proj.weight[22:], w["l2.mlp.up"]) and model.layers[1].norm2.item() == w["l1.norm2"].item()
    assert set(model.latent_ranks()) == {(0, "k"), (0, "v"), (1, "k"), (1, "v")} and model.latent_ranks()[(1, "v")] == 60
    assert model.state_shapes() == {((1, "mix"), "S"): (2, 14, 8)}
    with pytest.raises(KeyError):
        model.load_weights([(k, v) for k, v in w.items() if k != "l1.mix.left.k.b"])
    with pytest.raises(KeyError):
        model.load_weights(list(w.items()) + [("l2.mix.k", torch.zeros(20, 36))])


def test_restatement_is_causal_and_its_window_has_the_stated_edge():
    from nano_vllm_x_amd.gibavik import GibavikConfig, random_checkpoint
    cfg = GibavikConfig.from_dict(CFG)
    w = dict(random_checkpoint(cfg, 1))
    toks = torch.randint(0, 53, (12,), generator=torch.Generator().manual_seed(0)).tolist()
    full = go.forward(CFG, w, toks)
    assert torch.allclose(go.forward(CFG, w, toks[:7]), full[:7], atol=1e-12)
    assert (go.forward(CFG, w, [(toks[0] + 1) % 53] + toks[1:])[-1] - full[-1]).abs().max() > 1e-6
    # a window of w keys: the token itself and the w - 1 before it
    g = torch.Generator().manual_seed(2)
    q, k, v = torch.randn(9, 1, 4, generator=g).double(), torch.randn(9, 1, 4, generator=g).double(), torch.randn(9, 1, 3, generator=g).double()
    o = go.attend(q, k, v, 0.5, window=3)
    moved = v.clone()
    moved[5] += 1.0
    o2 = go.attend(q, k, moved, 0.5, window=3)
    changed = [(o2[i] - o[i]).abs().max().item() > 1e-12 for i in range(9)]
    assert changed == [False] * 5 + [True, True, True, False]
    # values turned by their positions and the read-out turned back: what is summed depends on distances only
    pos = torch.arange(9)
    a = go.turn(go.attend(q, k, go.turn(v.repeat(1, 1, 2), pos, 50.0, 6), 0.5), pos, 50.0, 6, sign=-1.0)
    b = go.turn(go.attend(q, k, go.turn(v.repeat(1, 1, 2), pos + 100, 50.0, 6), 0.5), pos + 100, 50.0, 6, sign=-1.0)
    assert torch.allclose(a, b, atol=1e-9)
