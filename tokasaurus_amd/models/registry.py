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
from tokasaurus_amd.config.kupuzen_config import KupuzenConfig
from tokasaurus_amd.models.kupuzen import kupuzen_spec
from tokasaurus_amd.models.llama import llama_spec
from tokasaurus_amd.config.taborax_config import TaboraxConfig
from tokasaurus_amd.models.taborax import taborax_spec
from tokasaurus_amd.config.sakevik_config import SakevikConfig
from tokasaurus_amd.models.sakevik import sakevik_spec
from tokasaurus_amd.config.sazilorn_config import SazilornConfig
from tokasaurus_amd.models.sazilorn import sazilorn_spec
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
register_architecture(Architecture("kupuzen", KupuzenConfig.from_dict, kupuzen_spec, class_names=("Kupuzen",)))
register_architecture(Architecture("taborax", TaboraxConfig.from_dict, taborax_spec, class_names=("Taborax",)))
register_architecture(Architecture("sakevik", SakevikConfig.from_dict, sakevik_spec, class_names=("Sakevik",)))
register_architecture(Architecture("sazilorn", SazilornConfig.from_dict, sazilorn_spec, class_names=("Sazilorn",)))


def architecture_of(config_dict: dict[str, Any]) -> Architecture:
    """By ``model_type`` (the reference's only key, tokasaurus/model/utils.py:338-340); a file
    without one is taken by the first name under ``architectures`` that a registered
    architecture claims."""
    name = config_dict.get("model_type")
    if name is None:
        # a file may name its one class under "architecture" instead of listing classes
        one = config_dict.get("architecture")
        classes = list(config_dict.get("architectures") or []) + ([one] if isinstance(one, str) else [])
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
    if hasattr(cfg, "with_tensor_shapes"):
        # sizes that only the checkpoint knows (config.json does not repeat them)
        from tokasaurus_amd.weights.loader import tensor_shapes

        cfg = cfg.with_tensor_shapes(tensor_shapes(model_dir))
    return arch, cfg


def build_model(arch: Architecture, cfg: Any) -> CausalLM:
    return CausalLM(arch.spec_from_config(cfg))
