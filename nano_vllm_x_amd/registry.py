"""Model registry: config.json names an architecture, the registry gives its configuration reader and model class.

An entry is (read configuration from the parsed config.json, model class).  The model class tells the runner what kind of
cache it needs through its `family` attribute: "paged_kv" (K and V rows per token: paged attention) or "seq_state" (rows
per token for the layers that attend -- a latent, or keys and values -- plus per-sequence state slots)."""
from __future__ import annotations

import json
import os


def _qwen3():
    from .qwen3 import Qwen3Config, Qwen3ForCausalLM
    return Qwen3Config.from_dict, Qwen3ForCausalLM


def _kabidra():
    from .kabidra import KabidraConfig, KabidraForCausalLM
    return KabidraConfig.from_dict, KabidraForCausalLM


def _meronex():
    from .meronex import MeronexConfig, MeronexForCausalLM
    return MeronexConfig.from_dict, MeronexForCausalLM


def _gibavik():
    from .gibavik import GibavikConfig, GibavikForCausalLM
    return GibavikConfig.from_dict, GibavikForCausalLM


def _ladusun():
    from .ladusun import LadusunConfig, LadusunForCausalLM
    return LadusunConfig.from_dict, LadusunForCausalLM


# architecture name (config.json "architectures"[0] or "architecture") -> loader of (config reader, model class)
ARCHITECTURES = {"Qwen3ForCausalLM": _qwen3, "Kabidra": _kabidra, "Meronex": _meronex, "Gibavik": _gibavik, "Ladusun": _ladusun}


def architecture_of(config: dict) -> str:
    names = config.get("architectures") or [config.get("architecture")]
    for name in names:
        if name in ARCHITECTURES:
            return name
    if names == [None] and "hidden_size" in config:      # a bare Qwen3 geometry (presets, test configurations)
        return "Qwen3ForCausalLM"
    raise ValueError(f"no model registered for architecture {names}; known: {sorted(ARCHITECTURES)}")


def load_config(model: str):
    """Configuration object of the model directory `model` (or of a Qwen3 preset name, as qwen3.load_config takes it)."""
    cfg_file = os.path.join(model, "config.json")
    if os.path.isfile(cfg_file):
        with open(cfg_file) as f:
            d = json.load(f)
        return ARCHITECTURES[architecture_of(d)]()[0](d)
    from .qwen3 import load_config as qwen3_preset
    return qwen3_preset(model)


def model_class_of(cfg):
    """Model class for a configuration object made by load_config (or built by hand)."""
    name = getattr(cfg, "architecture", None) or "Qwen3ForCausalLM"
    return ARCHITECTURES[name]()[1]
