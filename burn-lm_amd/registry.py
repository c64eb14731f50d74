"""One registry from names to what they build.

* architectures: the name in ``config.json`` (``architectures[0]`` or ``model_type``) -> an
  ``Architecture`` (how to read its configuration and how to lay out its parts).  The reference
  fills a map from model name to server at compile time (crates/burn-lm-registry/src/lib.rs:5-43,
  crates/burn-lm-macros/src/lib.rs:343-439); here it is a table filled at import and open to
  additions at run time.
* part kinds: mixers, feed-forwards, norms, position encodings and blocks by kind name, so a
  layer plan can pick them layer by layer.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict


class RegistryError(KeyError):
    def __str__(self):
        return self.args[0] if self.args else ""


@dataclass(frozen=True)
class Architecture:
    name: str
    read_config: Callable  # dict (config.json) -> typed configuration
    plan: Callable         # (configuration, tensor names in the checkpoint or None) -> ModelPlan
    checkpoint_tensors: Callable = None  # configuration -> {name: (shape, initialiser or role)} of a fresh checkpoint
    display_name: str = ""
    created_by: str = ""
    # text side (used by the server and the command line, never by the engine):
    chat_template: Callable = None       # list of {"role", "content"} messages -> prompt text; None: contents joined by newlines
    special_tokens: dict = None          # names in tokenizer.json: {"bos": str, "eos": str, "stops": (str, ...)}


_ARCHITECTURES: Dict[str, Architecture] = {}
_PARTS: Dict[str, Dict[str, type]] = {"mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {},
                                      "embedding": {}, "head": {}}


def register_architecture(arch: Architecture, *aliases: str) -> None:
    for name in (arch.name, *aliases):
        _ARCHITECTURES[name] = arch


def architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise RegistryError(f"no architecture named {name!r} is registered; known: "
                            f"{', '.join(sorted(_ARCHITECTURES)) or 'none'}") from None


def architectures() -> Dict[str, Architecture]:
    return dict(_ARCHITECTURES)


def register_part(family: str, kind: str, cls: type) -> None:
    if family not in _PARTS:
        raise RegistryError(f"no part family {family!r}; families: {', '.join(_PARTS)}")
    _PARTS[family][kind] = cls


def part(family: str, kind: str) -> type:
    try:
        return _PARTS[family][kind]
    except KeyError:
        raise RegistryError(f"no {family} of kind {kind!r} is registered; known: "
                            f"{', '.join(sorted(_PARTS.get(family, {}))) or 'none'}") from None


def parts(family: str) -> Dict[str, type]:
    return dict(_PARTS[family])


def architecture_of(config_dict: dict) -> Architecture:
    """The architecture a config.json names, by ``architectures[0]`` and then ``model_type``."""
    names = []
    a = config_dict.get("architectures")
    if isinstance(a, list):
        names += [x for x in a if isinstance(x, str)]
    if isinstance(config_dict.get("model_type"), str):
        names.append(config_dict["model_type"])
    if not names:
        raise RegistryError("config.json names no architecture (keys 'architectures' or 'model_type'); known: "
                            + ", ".join(sorted(_ARCHITECTURES)))
    for n in names:
        if n in _ARCHITECTURES:
            return _ARCHITECTURES[n]
    return architecture(names[0])
