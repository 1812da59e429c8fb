"""Model registry: which model class serves a checkpoint directory or a ready configuration object.

A model's config.json names its architecture either the HuggingFace way (`architectures: [...]`) or,
for the framework's own formats, with a single `architecture` string; the latter kind brings its own
configuration class (`config_class.from_pretrained(dir)`), the former is read with transformers'
AutoConfig. New model families are added here and nowhere else in the engine.
"""
from __future__ import annotations

import json
import os


def _qwen3():
    from .qwen3 import Qwen3ForCausalLM
    return Qwen3ForCausalLM


def _kagalorn():
    from .kagalorn import KagalornForCausalLM
    return KagalornForCausalLM


def _bokulorn():
    from .bokulorn import BokulornForCausalLM
    return BokulornForCausalLM


def _givozen():
    from .givozen import GivozenForCausalLM
    return GivozenForCausalLM


def _bisuzen():
    from .bisuzen import BisuzenForCausalLM
    return BisuzenForCausalLM


MODELS = {
    "Qwen3ForCausalLM": _qwen3,
    "Kagalorn": _kagalorn,
    "Bokulorn": _bokulorn,
    "Givozen": _givozen,
    "Bisuzen": _bisuzen,
}
DEFAULT = "Qwen3ForCausalLM"


def architecture_of(hf_config) -> str:
    names = getattr(hf_config, "architectures", None) or ()
    for name in names:
        if name in MODELS:
            return name
    return DEFAULT       # ready-made namespaces with the Qwen3 fields carry no name


def model_class(hf_config):
    return MODELS[architecture_of(hf_config)]()


def load_config(path: str):
    """The configuration object of the checkpoint directory `path`."""
    with open(os.path.join(path, "config.json")) as f:
        raw = json.load(f)
    name = raw.get("architecture")
    if isinstance(name, str):
        if name not in MODELS:
            raise ValueError(f"unknown architecture '{name}' (known: {sorted(MODELS)})")
        return MODELS[name]().config_class.from_pretrained(path)
    from transformers import AutoConfig
    return AutoConfig.from_pretrained(path)
