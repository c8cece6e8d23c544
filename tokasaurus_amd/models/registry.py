"""The one registry from an architecture's name to its model: the ``model_type``
of config.json picks a configuration class and a function that turns that
configuration into a ``ModelSpec`` (the counterpart of the ``models`` dict at
tokasaurus/model/utils.py:321-340)."""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable

from tokasaurus_amd.config.model_config import ConfigError, LlamaConfig, read_config_json
from tokasaurus_amd.models.causal_lm import CausalLM
from tokasaurus_amd.models.llama import llama_spec
from tokasaurus_amd.models.spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[dict[str, Any]], Any]
    spec_from_config: Callable[[Any], ModelSpec]
    # class names a config.json may give under "architectures" for this architecture: they
    # choose it when the file has no model_type
    class_names: tuple[str, ...] = ()


ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(arch: Architecture, replace: bool = False) -> None:
    if arch.name in ARCHITECTURES and not replace:
        raise KeyError(f"architecture {arch.name!r} is already registered")
    ARCHITECTURES[arch.name] = arch


register_architecture(Architecture("llama", LlamaConfig.from_dict, llama_spec, class_names=("LlamaForCausalLM",)))


def architecture_of(config_dict: dict[str, Any]) -> Architecture:
    """By ``model_type`` (the reference's only key, tokasaurus/model/utils.py:338-340); a file
    without one is taken by the first name under ``architectures`` that a registered
    architecture claims."""
    name = config_dict.get("model_type")
    if name is None:
        classes = config_dict.get("architectures") or []
        by_class = {c: a for a in ARCHITECTURES.values() for c in a.class_names}
        for c in classes:
            if c in by_class:
                return by_class[c]
        raise ConfigError(
            f"config.json has no model_type and its architectures {list(classes)} name no registered model class; "
            f"registered: model_type {sorted(ARCHITECTURES)}, architectures {sorted(by_class)}")
    if name not in ARCHITECTURES:
        raise ConfigError(f"unknown model_type {name!r}; registered architectures: {sorted(ARCHITECTURES)}")
    return ARCHITECTURES[name]


def config_from_folder(model_dir: str | Path, rope_scaling_override: tuple[bool, dict | None] = (False, None)):
    d = read_config_json(model_dir)
    arch = architecture_of(d)
    cfg = arch.config_from_dict(d)
    if rope_scaling_override[0]:
        cfg = cfg.with_rope_scaling(rope_scaling_override[1])
    return arch, cfg


def build_model(arch: Architecture, cfg: Any) -> CausalLM:
    return CausalLM(arch.spec_from_config(cfg))
