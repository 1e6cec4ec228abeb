"""One registry from an architecture's name to the code that builds its model.

config.json names the architecture in ``architectures[0]``.  An entry holds two
functions: ``parse_config`` turns the json dictionary into the architecture's
typed configuration, and ``build_plan`` turns that configuration into a
``ModelPlan`` (the list of layers, their parts, their weights' names, their
cache needs and the order in which they run).  Everything below the plan is
generic, so adding an architecture means registering one more entry.

The reference has no registry: its entry points hardcode one preset
(``generate.py:273``, ``model/llama.py:335``).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Mapping


@dataclass(frozen=True)
class Architecture:
    name: str
    parse_config: Callable[[Mapping[str, Any]], Any]
    build_plan: Callable[[Any], Any]


_ARCHITECTURES: Dict[str, Architecture] = {}


class UnknownArchitecture(KeyError):
    def __str__(self) -> str:  # KeyError would print the repr of the message
        return self.args[0]


def register_architecture(name: str, parse_config, build_plan, *, replace: bool = False) -> Architecture:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    entry = Architecture(name=name, parse_config=parse_config, build_plan=build_plan)
    _ARCHITECTURES[name] = entry
    return entry


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def known_architectures() -> list:
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise UnknownArchitecture(
            f"architecture {name!r} is not registered; known: {', '.join(known_architectures()) or '(none)'}"
        ) from None


def architecture_of(config_dict: Mapping[str, Any]) -> Architecture:
    """The entry that ``config.json``'s ``architectures[0]`` names."""
    archs = config_dict.get("architectures")
    if not archs:
        raise UnknownArchitecture(
            "config.json has no 'architectures' entry; known: " + ", ".join(known_architectures())
        )
    return get_architecture(archs[0])
