"""Model families the engine serves, chosen by ``config.json``: the ``architecture`` key (or the first entry of Hugging Face's
``architectures``) names an entry of ``MODEL_REGISTRY``; a file with neither is a Qwen2 description, as before.

A family is *padded* (rows of equal length over the static per-request cache: the Jacobi decoders' forward) or *ragged*
(one flat batch of prompt portions and decoded tokens over a paged pool and state slots)."""
from __future__ import annotations

import importlib
import json
from pathlib import Path

# architecture -> (module, config class, family)
MODEL_REGISTRY = {
    "Qwen2ForCausalLM": ("jacobiforcing_amd.modeling.qwen2", "Qwen2Config", "padded"),
    "Lokizen": ("jacobiforcing_amd.modeling.lokizen", "LokizenConfig", "ragged"),
    "Vumalix": ("jacobiforcing_amd.modeling.vumalix", "VumalixConfig", "ragged"),
    "Bamanex": ("jacobiforcing_amd.modeling.bamanex", "BamanexConfig", "ragged"),
    "Mikipel": ("jacobiforcing_amd.modeling.mikipel", "MikipelConfig", "ragged"),
}


def architecture_of(model_dir) -> str:
    d = json.loads((Path(model_dir) / "config.json").read_text())
    return d.get("architecture") or (d.get("architectures") or ["Qwen2ForCausalLM"])[0]


def read_model_config(model_dir):
    """The model description object of ``model_dir`` (its class depends on the architecture)."""
    arch = architecture_of(model_dir)
    if arch not in MODEL_REGISTRY:
        raise ValueError(f"{model_dir}: architecture {arch!r} is not served (known: {sorted(MODEL_REGISTRY)})")
    mod, cls, _ = MODEL_REGISTRY[arch]
    return getattr(importlib.import_module(mod), cls).from_json(Path(model_dir) / "config.json")


def family_of(hf_config) -> str:
    return getattr(hf_config, "family", "padded")
