"""One registry from an architecture's name to everything that builds and loads it.

A family is registered under the names that config.json may carry: the entries of
``architectures`` (``GPT2LMHeadModel``) and the ``model_type`` (``gpt2``); both resolve to the
same entry.  The reference keys its registry on ``model_type`` (src/models/auto.rs:299-697);
looking at ``architectures`` first is this library's own addition.

A family supplies four things and nothing else in the library knows its name:
  config_class   typed configuration with ``from_dict`` (validating) and ``to_dict``
  plan           config -> ModelPlan: the layers, their parts and the order they run in, as data
  contract       config -> list of TensorSpec: the checkpoint's tensor names, shapes and layouts
  init           (config, generator) -> dict of tensors under checkpoint names (random weights)
"""

from dataclasses import dataclass
from typing import Callable, Tuple

from .base import UnsupportedArchitecture, unwrap_text_config


@dataclass(frozen=True)
class Family:
    name: str
    architectures: Tuple[str, ...]
    model_types: Tuple[str, ...]
    config_class: type
    plan: Callable
    contract: Callable
    init: Callable


_FAMILIES = {}


def register_family(family, replace=False):
    """Adds a family under all its names; a name already taken is an error unless ``replace``."""
    for key in family.architectures + family.model_types:
        if key in _FAMILIES and _FAMILIES[key].name != family.name and not replace:
            raise ValueError(f"architecture name {key!r} is already registered for {_FAMILIES[key].name}")
    for key in family.architectures + family.model_types:
        _FAMILIES[key] = family
    return family


def unregister_family(name):
    for key in [k for k, f in _FAMILIES.items() if f.name == name]:
        del _FAMILIES[key]


def supported_names():
    return sorted(_FAMILIES)


def resolve_family(config_json):
    """The family a parsed config.json asks for: ``architectures[0]`` first, then ``model_type``."""
    data = unwrap_text_config(config_json)
    candidates = []
    architectures = data.get("architectures")
    if isinstance(architectures, (list, tuple)):
        candidates += [a for a in architectures if isinstance(a, str)]
    if isinstance(data.get("model_type"), str):
        candidates.append(data["model_type"])
    for name in candidates:
        if name in _FAMILIES:
            return _FAMILIES[name]
    asked = ", ".join(f"`{c}`" for c in candidates) or "nothing"
    raise UnsupportedArchitecture(
        f"config.json names {asked}, which is not executable; supported values: "
        + ", ".join(supported_names()))
