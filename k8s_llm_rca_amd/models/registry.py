"""Model registry: which class serves which architecture, by preset name or by a
checkpoint folder's config.json.

* ``llama`` / ``mixtral`` -- :class:`~.llama.LlamaModel` (Hugging Face config.json: ``hidden_size`` ...)
* ``opt``                 -- :class:`~.opt.OPTModel` (the CPU plumbing backend)
* ``zasapel``             -- :class:`~.zasapel.ZasapelModel` (config.json with ``"architecture": "Zasapel"``)
* ``ligipel``             -- :class:`~.ligipel.LigipelModel` (config.json with ``"architecture": "Ligipel"``)
* ``lizesun``             -- :class:`~.lizesun.LizesunModel` (config.json with ``"architecture": "Lizesun"``)
* ``pumozen``             -- :class:`~.pumozen.PumozenModel` (config.json with ``"architecture": "Pumozen"``)

The last four describe their layers one by one in config.json (``OWN_CONFIG``): their
configuration objects are built from it, not from a preset with overrides.
"""
from __future__ import annotations

import json
import os
from dataclasses import replace

from . import config as C


# architectures whose config.json lists the layers (``"architecture": <name>``): module, model class
OWN_CONFIG = {"zasapel": ("zasapel", "ZasapelModel"), "ligipel": ("ligipel", "LigipelModel"),
              "lizesun": ("lizesun", "LizesunModel"), "pumozen": ("pumozen", "PumozenModel")}


def _module(arch: str):
    import importlib
    return importlib.import_module(f"{__package__}.{OWN_CONFIG[arch][0]}")


def get_any_config(name: str, **overrides):
    """A preset of any architecture."""
    for arch in OWN_CONFIG:
        presets = _module(arch).PRESETS
        if name in presets:
            return replace(presets[name], **overrides) if overrides else presets[name]
    return C.get_config(name, **overrides)


def build_model(mc, device, dtype, pc=None, seed: int = 0):
    """A randomly initialised model of the configuration's architecture."""
    if mc.arch == "opt":
        from .opt import OPTModel
        return OPTModel(mc, device, dtype, seed=seed)
    if mc.arch in OWN_CONFIG:
        return getattr(_module(mc.arch), OWN_CONFIG[mc.arch][1])(mc, device, dtype, pc, seed=seed)
    from .llama import LlamaModel
    return LlamaModel(mc, device, dtype, pc, seed=seed)


def checkpoint_arch(path: str) -> str:
    with open(os.path.join(path, "config.json") if os.path.isdir(path) else path) as f:
        d = json.load(f)
    if str(d.get("architecture", "")).lower() in OWN_CONFIG:
        return str(d["architecture"]).lower()
    return "mixtral" if d.get("num_local_experts") else "llama"


def load_model(path: str, device, dtype, pc=None):
    """The model a checkpoint folder holds, chosen by its config.json."""
    arch = checkpoint_arch(path)
    if arch in OWN_CONFIG:
        return _module(arch).load_checkpoint(path, device, dtype, pc)
    from .llama import LlamaModel
    from .weights import config_from_hf, load_safetensors
    mc = config_from_hf(path)
    model = LlamaModel(mc, device, dtype, pc, init=False)
    load_safetensors(model, path)
    return model
