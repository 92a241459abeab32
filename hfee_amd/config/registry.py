"""One registry from an architecture's name to its configuration class and model.

The reference keeps a map from the architecture string to what differs between
architectures and answers an unknown name with `unsupported model architecture %q`
(/root/reference/internal/llm/model.go:50-56, 77-81).  Here an entry holds the
class that parses config.json and the function that turns the parsed
configuration into a `ModelSpec` (the list of parts and their order).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from .base import ConfigError, read_config_json
from .specs import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type                       # has from_dict(dict, where) and to_dict()
    model_spec: Callable[[object], ModelSpec]


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_class: type, model_spec: Callable) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_class, model_spec)


def architecture_names() -> list[str]:
    return sorted(_ARCHITECTURES)


def lookup_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(f'unsupported model architecture "{name}" '
                          f"(known: {', '.join(architecture_names()) or 'none'})") from None


def architecture_of(config_json: dict, where: str = "config.json") -> Architecture:
    archs = config_json.get("architectures")
    if archs is None and isinstance(config_json.get("architecture"), str):     # a single name under the singular key
        return lookup_architecture(config_json["architecture"])
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError(f"{where}: key 'architectures' must be a list naming the model class "
                          f"(or 'architecture' its name)")
    return lookup_architecture(archs[0])


def config_from_dict(config_json: dict, where: str = "config.json"):
    arch = architecture_of(config_json, where)
    return arch.config_class.from_dict(config_json, where)


def config_from_folder(model_dir: str):
    """A configuration class with `reads_tensor_shapes = True` also gets the shapes of the folder's
    tensors (from the checkpoint's header; no data is read): sizes that config.json leaves to them."""
    data = read_config_json(model_dir)
    where = f"{model_dir}/config.json"
    arch = architecture_of(data, where)
    if getattr(arch.config_class, "reads_tensor_shapes", False):
        from ..weights.safetensors_io import Checkpoint, SafetensorsError
        try:
            ckpt = Checkpoint(model_dir)
            shapes = {n: tuple(ckpt.entry(n).shape) for n in ckpt.names()}
        except (SafetensorsError, OSError):
            shapes = None          # (a folder with a configuration only: random weights)
        return arch.config_class.from_dict(data, where, tensor_shapes=shapes)
    return arch.config_class.from_dict(data, where)


def model_spec_of(config) -> ModelSpec:
    return lookup_architecture(config.architecture).model_spec(config)
