"""One registry from the architecture's name (config.json `architectures[0]`)
to its typed configuration, as `arch_name` + the `match` of the reference do
(src/arch/mod.rs:33-37, src/main.rs:33-45)."""
from __future__ import annotations

import json
import os
from typing import Any, Callable, Dict

from .llama import ConfigError, LlamaConfig
from .gokosun import GokosunConfig
from .lilatar import LilatarConfig
from .tuvodra import TuvodraConfig
from .vivisun import VivisunConfig

# name -> function(config dict) -> typed config with .model_spec() and .to_dict()
_ARCHITECTURES: Dict[str, Callable[[Dict[str, Any]], Any]] = {}


def register_architecture(name: str, from_dict: Callable[[Dict[str, Any]], Any]) -> None:
    _ARCHITECTURES[name] = from_dict


def architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(d: Dict[str, Any]):
    archs = d.get("architectures")
    if not archs and isinstance(d.get("architecture"), str):     # files that name one architecture, in the singular
        archs = [d["architecture"]]
    if not archs:
        raise ConfigError("missing config key: architectures")
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unsupported architecture: {name} (known: {', '.join(architectures())})")
    return _ARCHITECTURES[name](d)


def load_config(path: str):
    """`path` is a model folder or its config.json.  An architecture some of whose sizes only the tensors' shapes
    give (`sizes_from_tensors`) is shown the shapes of the folder's tensors, read from the files' headers."""
    folder = path if os.path.isdir(path) else os.path.dirname(path)
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path) as f:
            d = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"no config.json at {path}") from None
    config = config_from_dict(d)
    if hasattr(config, "sizes_from_tensors"):
        from ..weights.loader import open_model_files
        from ..weights.safetensors_io import SafetensorsError
        try:
            config.sizes_from_tensors({name: tuple(f.entries[name][1]) for name, f in open_model_files(folder).items()})
        except (SafetensorsError, OSError):
            pass            # no tensors beside the configuration: the sizes must be in the file
    return config


register_architecture("LlamaForCausalLM", LlamaConfig.from_dict)
register_architecture("Tuvodra", TuvodraConfig.from_dict)
register_architecture("Lilatar", LilatarConfig.from_dict)
register_architecture("Vivisun", VivisunConfig.from_dict)
register_architecture("Gokosun", GokosunConfig.from_dict)
