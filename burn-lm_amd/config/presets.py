"""Named shapes for the random-weights mode, read from ``presets.json`` beside this file."""
import json
import os


def presets() -> dict:
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "presets.json")) as f:
        d = json.load(f)
    return {k: v for k, v in d.items() if not k.startswith("_")}


def preset(name: str) -> dict:
    p = presets()
    if name not in p:
        raise KeyError(f"no preset named {name!r}; known: {', '.join(sorted(p))}")
    return dict(p[name])
