"""Model registry: which class serves which architecture, by preset name or by a
checkpoint folder's config.json.

* ``llama`` / ``mixtral`` -- :class:`~.llama.LlamaModel` (Hugging Face config.json: ``hidden_size`` ...)
* ``opt``                 -- :class:`~.opt.OPTModel` (the CPU plumbing backend)
* ``zasapel``             -- :class:`~.zasapel.ZasapelModel` (config.json with ``"architecture": "Zasapel"``)
"""
from __future__ import annotations

import json
import os
from dataclasses import replace

from . import config as C


def get_any_config(name: str, **overrides):
    """A preset of any architecture."""
    from .zasapel import PRESETS as ZP
    if name in ZP:
        return replace(ZP[name], **overrides) if overrides else ZP[name]
    return C.get_config(name, **overrides)


def build_model(mc, device, dtype, pc=None, seed: int = 0):
    """A randomly initialised model of the configuration's architecture."""
    if mc.arch == "opt":
        from .opt import OPTModel
        return OPTModel(mc, device, dtype, seed=seed)
    if mc.arch == "zasapel":
        from .zasapel import ZasapelModel
        return ZasapelModel(mc, device, dtype, pc, seed=seed)
    from .llama import LlamaModel
    return LlamaModel(mc, device, dtype, pc, seed=seed)


def checkpoint_arch(path: str) -> str:
    with open(os.path.join(path, "config.json") if os.path.isdir(path) else path) as f:
        d = json.load(f)
    if str(d.get("architecture", "")).lower() == "zasapel":
        return "zasapel"
    return "mixtral" if d.get("num_local_experts") else "llama"


def load_model(path: str, device, dtype, pc=None):
    """The model a checkpoint folder holds, chosen by its config.json."""
    if checkpoint_arch(path) == "zasapel":
        from .zasapel import load_checkpoint
        return load_checkpoint(path, device, dtype, pc)
    from .llama import LlamaModel
    from .weights import config_from_hf, load_safetensors
    mc = config_from_hf(path)
    model = LlamaModel(mc, device, dtype, pc, init=False)
    load_safetensors(model, path)
    return model
