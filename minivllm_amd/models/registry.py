"""Which model class serves which checkpoint.

A model family registers (a) the ``architecture`` / ``model_type`` strings of ``config.json``
it answers to, (b) how that file becomes its configuration object and (c) its module class.
``ModelRunner`` builds whatever the engine configuration's ``model`` object names; the command
line and the loaders go through ``config_from_path``.

What the engine asks of a configuration object: ``vocab_size``, ``name``, ``max_position`` and
``architecture``; of a model object: ``forward(input_ids, positions)`` returning the rows of
the final hidden state, ``lm_head`` and, for families whose cache is not the plain
``[layers, blocks, kv heads, block, head_dim]`` pair, the ``CacheSpec`` protocol of
``engine.cache_spec``.
"""
from __future__ import annotations

import json
import os
from typing import Callable, Dict, Tuple

_FAMILIES: Dict[str, Tuple[Callable, Callable]] = {}


def register(names, config_from_dict: Callable, model_class: Callable) -> None:
    """``model_class`` may be a zero-argument callable returning the class (lazy import)."""
    for n in names:
        _FAMILIES[n.lower()] = (config_from_dict, model_class)


def _family_of(cfg_json: dict) -> str:
    name = cfg_json.get("architecture") or cfg_json.get("model_type")
    if name is None and cfg_json.get("architectures"):
        name = cfg_json["architectures"][0]
    if name is None:
        raise ValueError("config.json names no architecture / model_type")
    return str(name).lower()


def config_from_path(path: str):
    """The model configuration object for the checkpoint folder ``path``."""
    _ensure_builtin()
    with open(os.path.join(path, "config.json")) as f:
        c = json.load(f)
    fam = _family_of(c)
    if fam not in _FAMILIES:
        raise ValueError(f"unsupported architecture {fam!r} (have: {sorted(_FAMILIES)})")
    return _FAMILIES[fam][0](c, os.path.basename(os.path.normpath(path)))


def model_class_for(model_config):
    _ensure_builtin()
    fam = getattr(model_config, "architecture", "qwen3").lower()
    if fam not in _FAMILIES:
        raise ValueError(f"unsupported architecture {fam!r} (have: {sorted(_FAMILIES)})")
    cls = _FAMILIES[fam][1]
    return cls() if not isinstance(cls, type) else cls


_BUILTIN = False


def _ensure_builtin() -> None:
    global _BUILTIN
    if _BUILTIN:
        return
    _BUILTIN = True

    def dense(c, name):
        from minivllm_amd.utils.loader import model_config_from_dict
        return model_config_from_dict(c, name)

    def qwen3_class():
        from minivllm_amd.models.qwen3 import Qwen3ForCausalLM
        return Qwen3ForCausalLM

    register(["qwen3", "qwen2", "llama", "mistral", "qwen3forcausallm", "qwen2forcausallm",
              "llamaforcausallm", "mistralforcausallm"], dense, qwen3_class)

    def natilix_cfg(c, name):
        from minivllm_amd.models.natilix import NatilixConfig
        return NatilixConfig.from_dict(c, name)

    def natilix_class():
        from minivllm_amd.models.natilix import NatilixForCausalLM
        return NatilixForCausalLM

    register(["natilix"], natilix_cfg, natilix_class)

    def pelenex_cfg(c, name):
        from minivllm_amd.models.pelenex import PelenexConfig
        return PelenexConfig.from_dict(c, name)

    def pelenex_class():
        from minivllm_amd.models.pelenex import PelenexForCausalLM
        return PelenexForCausalLM

    register(["pelenex"], pelenex_cfg, pelenex_class)

    def kidupel_cfg(c, name):
        from minivllm_amd.models.kidupel import KidupelConfig
        return KidupelConfig.from_dict(c, name)

    def kidupel_class():
        from minivllm_amd.models.kidupel import KidupelForCausalLM
        return KidupelForCausalLM

    register(["kidupel"], kidupel_cfg, kidupel_class)

    def zegelix_cfg(c, name):
        from minivllm_amd.models.zegelix import ZegelixConfig
        return ZegelixConfig.from_dict(c, name)

    def zegelix_class():
        from minivllm_amd.models.zegelix import ZegelixForCausalLM
        return ZegelixForCausalLM

    register(["zegelix"], zegelix_cfg, zegelix_class)
