"""One registry from an architecture's name (``architectures[0]`` of config.json) to its typed
configuration and the function that turns the configuration into a ModelSpec.  The reference
keeps the same table in its converter (tools/convert.py:29, :56-58)."""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable, Dict, Mapping, Optional

from .config import kikarax as kikarax_config
from .config import kuponex as kuponex_config
from .config import sepedra as sepedra_config
from .config import vupolix as vupolix_config
from .config.llama import ConfigError, LlamaConfig
from .models.kikarax import TINY_KIKARAX, kikarax_spec
from .models.kuponex import TINY_KUPONEX, kuponex_spec
from .models.llama import TINY_LLAMA, llama_spec
from .models.sepedra import TINY_SEPEDRA, sepedra_spec
from .models.vupolix import TINY_VUPOLIX, vupolix_spec
from .parts.base import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[Mapping[str, Any]], Any]
    spec_from_config: Callable[[Any], ModelSpec]
    tiny_config: Optional[Mapping[str, Any]] = None     # a small config.json of this architecture for simulations and smoke runs
    # (config, {tensor name: shape}) -> config with the sizes filled in that only the checkpoint's tensor shapes give
    sizes_from_tensors: Optional[Callable[[Mapping[str, Any], Mapping[str, tuple]], Dict[str, Any]]] = None


ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_from_dict, spec_from_config, tiny_config=None, sizes_from_tensors=None) -> None:
    if name in ARCHITECTURES:
        raise ValueError(f"architecture '{name}' is already registered")
    ARCHITECTURES[name] = Architecture(name, config_from_dict, spec_from_config, tiny_config, sizes_from_tensors)


def architecture_of(config: Mapping[str, Any]) -> Architecture:
    """By ``architectures[0]`` (the exporters' list) or, where a config.json names just one, ``architecture``."""
    archs = config.get("architectures")
    if isinstance(archs, (list, tuple)) and archs:
        name = archs[0]
    elif isinstance(config.get("architecture"), str):
        name = config["architecture"]
    else:
        raise ConfigError("config.json lacks 'architectures': [name]")
    arch = ARCHITECTURES.get(name)
    if arch is None:
        raise ConfigError(f"unsupported architecture {name}; registered: {sorted(ARCHITECTURES)}")
    return arch


def read_model_config(folder: str | Path) -> Dict[str, Any]:
    """config.json of a model folder, completed from the shapes in its safetensors headers where the architecture
    takes sizes from there."""
    from .weights import safetensors_io
    raw = read_config(folder)
    arch = architecture_of(raw)
    if arch.sizes_from_tensors is not None:
        shapes: Dict[str, tuple] = {}
        for shard in sorted(Path(folder).glob("*.safetensors")):
            header, _ = safetensors_io.read_header(shard)
            shapes.update({name: tuple(int(s) for s in info["shape"]) for name, info in header.items()})
        raw = arch.sizes_from_tensors(raw, shapes)
    return raw


def read_config(folder: str | Path) -> Dict[str, Any]:
    path = Path(folder) / "config.json"
    if not path.exists():
        raise ConfigError(f"cannot open {path}")
    return json.loads(path.read_text())


register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, llama_spec, TINY_LLAMA)
register_architecture(kuponex_config.ARCHITECTURE, kuponex_config.KuponexConfig.from_dict, kuponex_spec, TINY_KUPONEX,
                      kuponex_config.sizes_from_tensors)
register_architecture(sepedra_config.ARCHITECTURE, sepedra_config.SepedraConfig.from_dict, sepedra_spec, TINY_SEPEDRA)
register_architecture(kikarax_config.ARCHITECTURE, kikarax_config.KikaraxConfig.from_dict, kikarax_spec, TINY_KIKARAX)
register_architecture(vupolix_config.ARCHITECTURE, vupolix_config.VupolixConfig.from_dict, vupolix_spec, TINY_VUPOLIX,
                      vupolix_config.sizes_from_tensors)
