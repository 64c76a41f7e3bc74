"""Named configurations: config.json files kept under presets/ (two tiny Gemma 2
configurations and the 2B, 9B and 27B shapes)."""
from __future__ import annotations

import json
import os

_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "presets")


def preset_names():
    return sorted(f[:-5] for f in os.listdir(_DIR) if f.endswith(".json"))


def preset(name: str) -> dict:
    """The parsed config.json of a preset, e.g. 'gemma2-2b' (a bare '2b' is read as 'gemma2-2b')."""
    for cand in (name, "gemma2-" + name):
        path = os.path.join(_DIR, cand + ".json")
        if os.path.exists(path):
            with open(path) as f:
                return json.load(f)
    raise KeyError(f"unknown preset '{name}'; known: {preset_names()}")
