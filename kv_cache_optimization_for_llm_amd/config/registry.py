"""Registries: architecture name -> model description, part kind -> part class.

A model is never named in engine code.  ``config.json``'s ``architectures[0]`` picks an
:class:`Architecture` here; the architecture turns the configuration into a
:class:`~kv_cache_optimization_for_llm_amd.models.spec.ModelSpec`, which names, layer by layer, the
kind of mixer, feed-forward, norm and position encoding and their constants.  The part
registries turn those kinds into objects.  Anything - a test included - may register another
architecture or another part without touching this package.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Mapping


class RegistryError(KeyError):
    def __str__(self) -> str:  # KeyError would show the repr of the message
        return self.args[0] if self.args else ""


class Registry:
    def __init__(self, what: str):
        self.what = what
        self._items: Dict[str, Any] = {}

    def register(self, name: str, item: Any = None, *, replace: bool = False):
        def put(obj):
            if name in self._items and not replace:
                raise RegistryError(f"{self.what} {name!r} is already registered")
            self._items[name] = obj
            return obj
        return put if item is None else put(item)

    def unregister(self, name: str) -> None:
        self._items.pop(name, None)

    def get(self, name: str) -> Any:
        try:
            return self._items[name]
        except KeyError:
            raise RegistryError(
                f"unknown {self.what} {name!r}; registered: {sorted(self._items)}") from None

    def names(self):
        return sorted(self._items)

    def __contains__(self, name: str) -> bool:
        return name in self._items


@dataclass(frozen=True)
class Architecture:
    """How one ``architectures[0]`` name becomes a model.

    ``parse_config`` turns the raw ``config.json`` dictionary into the architecture's typed
    configuration (and rejects what it cannot run); ``build_spec`` turns that into a ModelSpec.
    """

    name: str
    parse_config: Callable[[Mapping[str, Any]], Any]
    build_spec: Callable[[Any], Any]


ARCHITECTURES = Registry("architecture")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block arrangement")
ROTARY_FREQUENCIES = Registry("rotary frequency rule")     # name -> f(rot_dim, theta, **params) -> fp32 [rot_dim / 2]


def register_architecture(name: str, parse_config, build_spec, *, replace: bool = False) -> Architecture:
    arch = Architecture(name, parse_config, build_spec)
    ARCHITECTURES.register(name, arch, replace=replace)
    return arch


def architecture_for(config_dict: Mapping[str, Any]) -> Architecture:
    archs = config_dict.get("architectures")
    if not archs or not isinstance(archs, (list, tuple)):
        raise RegistryError(
            "config.json has no 'architectures' list; registered: " f"{ARCHITECTURES.names()}")
    return ARCHITECTURES.get(archs[0])
