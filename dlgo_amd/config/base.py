"""Typed model configurations and the one registry from architecture name to model.

A configuration class reads the keys of its architecture's own config.json,
checks them, and derives sizes once.  Nothing here knows a model size: every
number comes from the file.  computerex/dlgo fills a flat ModelConfig from GGUF
metadata with four hard errors (models/llm/config.go:43-123) and looks an
architecture up with a silent default (models/llm/arch.go:33-43); here an
unknown name is an error that lists the known ones.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Mapping, Optional, Tuple, Type


class ConfigError(ValueError):
    """A config.json that cannot be used; the message names the key and the rule."""


_MISSING = object()


class KeyReader:
    """Reads typed keys of a config.json mapping and collects every complaint."""

    def __init__(self, raw: Mapping[str, Any], where: str = "config.json"):
        self.raw = raw
        self.where = where
        self.problems: list[str] = []

    def _get(self, key: str, default: Any):
        if key in self.raw and self.raw[key] is not None:
            return self.raw[key]
        if default is _MISSING:
            self.problems.append(f"{key}: required key is missing")
            return None
        return default

    def integer(self, key: str, default: Any = _MISSING, minimum: int | None = None):
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v.is_integer():
                v = int(v)
            else:
                self.problems.append(f"{key}: expected an integer, found {v!r}")
                return None
        if minimum is not None and v < minimum:
            self.problems.append(f"{key}: must be >= {minimum}, found {v}")
            return None
        return v

    def number(self, key: str, default: Any = _MISSING, positive: bool = False):
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            self.problems.append(f"{key}: expected a number, found {v!r}")
            return None
        v = float(v)
        if positive and not v > 0:
            self.problems.append(f"{key}: must be > 0, found {v}")
            return None
        return v

    def boolean(self, key: str, default: Any = _MISSING):
        v = self._get(key, default)
        if v is None:
            return None
        if not isinstance(v, bool):
            self.problems.append(f"{key}: expected true or false, found {v!r}")
            return None
        return v

    def string(self, key: str, default: Any = _MISSING):
        v = self._get(key, default)
        if v is None:
            return None
        if not isinstance(v, str):
            self.problems.append(f"{key}: expected a string, found {v!r}")
            return None
        return v

    def complain(self, text: str) -> None:
        self.problems.append(text)

    def finish(self) -> None:
        if self.problems:
            raise ConfigError(f"{self.where}: " + "; ".join(self.problems))


@dataclass(frozen=True)
class ModelConfig:
    """What every architecture's configuration offers to the rest of the library.  Engine, entry point, loop and
    random weights ask these methods and read no key of their own: which keys a config.json has is the
    architecture's business alone (computerex/dlgo keeps one descriptor per architecture the same way,
    models/llm/arch.go:17-43)."""

    architecture: str

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError

    def context_length(self) -> Optional[int]:
        """The longest sequence the model's positions are defined for; None if nothing in the model bounds it."""
        return None

    def stop_tokens(self) -> Tuple[int, ...]:
        """Token ids that end a sequence unless a request says otherwise."""
        return ()

    def describe(self) -> List[str]:
        """The sizes worth printing, as short phrases ("16 layers", "2048 dim", ...)."""
        return []

    def storage_dtype(self) -> str:
        """The element type a checkpoint of this model is stored in ("bfloat16", "float16" or "float32")."""
        return "bfloat16"

    def init_std(self) -> Optional[float]:
        """The standard deviation random matrices are drawn with, if the configuration names one."""
        return None

    def stored_as(self, dtype_name: str) -> "ModelConfig":
        """The configuration of the same model whose checkpoint is stored in another element type (an architecture
        whose config.json does not record the type returns itself)."""
        return self


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Type[ModelConfig]
    build: Callable[[ModelConfig], Any]   # config -> parts.model.DecoderModel (weights not yet loaded)


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_class: Type[ModelConfig], build: Callable[[ModelConfig], Any]) -> None:
    """Make `name` (the string in config.json's "architectures") known.  Registering a
    name again replaces it, as models/llm/arch.go:61-63 does."""
    _ARCHITECTURES[name] = Architecture(name, config_class, build)


def _builtin() -> None:
    """The architectures that ship with the library register themselves when their package is imported."""
    import importlib
    importlib.import_module("dlgo_amd.models")


def known_architectures() -> list[str]:
    _builtin()
    return sorted(_ARCHITECTURES)


def architecture_of(raw: Mapping[str, Any]) -> Architecture:
    names = raw.get("architectures")
    if isinstance(names, str):
        names = [names]
    if not names or not isinstance(names, (list, tuple)) or not isinstance(names[0], str):
        raise ConfigError('config.json: "architectures" must name the model class, e.g. ["LlamaForCausalLM"]')
    name = names[0]
    _builtin()
    if name not in _ARCHITECTURES:
        raise ConfigError(f"config.json: unknown architecture {name!r}; known: {', '.join(known_architectures()) or '(none)'}")
    return _ARCHITECTURES[name]


def config_from_dict(raw: Mapping[str, Any]) -> ModelConfig:
    return architecture_of(raw).config_class.from_dict(raw)


def read_config_json(folder_or_file: str) -> Dict[str, Any]:
    path = folder_or_file
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path) as f:
            raw = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"{path}: no such file") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not JSON ({e})") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return raw


def load_config(folder_or_file: str) -> ModelConfig:
    return config_from_dict(read_config_json(folder_or_file))


def build_model(config: ModelConfig):
    """The registry's second half: configuration -> model made of parts."""
    _builtin()
    if config.architecture not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture {config.architecture!r}; known: {', '.join(known_architectures())}")
    return _ARCHITECTURES[config.architecture].build(config)
