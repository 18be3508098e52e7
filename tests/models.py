"""Tiny test models: config.json dictionaries plus how their random weights are drawn. They differ
in every size and option: head counts and groups, sizes that are no power of two, layers,
vocabulary, eps, theta, tied or untied head, window."""

from __future__ import annotations

from pathlib import Path

from miniserve_amd.config.presets import preset
from miniserve_amd.weights.random_init import Init, write_model_folder

TINY = {
    # name: (config, seed, init)
    "tinyA": (preset("tinyA"), 0, Init(0.02, None)),
    "tinyB": (preset("tinyB"), 1, Init(0.05, (0.5, 1.5))),
    "tinyC": (preset("tinyC"), 2, Init(0.04, (0.7, 1.3))),
    "tinyD": (preset("tinyD"), 3, Init(0.03, (0.8, 1.2))),
    "tinyE": (preset("tinyE"), 4, Init(0.04, (0.5, 1.5))),
}


def make_folder(tmp: Path, name: str) -> Path:
    cfg, seed, init = TINY[name]
    return write_model_folder(Path(tmp) / name, cfg, seed, init)
