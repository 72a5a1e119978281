"""Imports the in-tree built HIP extensions (arks_amd/ops/_build/<name>/<name>.so).

Raises ImportError if the extension has not been built — callers on a GPU box
must fail loudly rather than fall back to eager PyTorch.
"""

from __future__ import annotations

import importlib.util

import torch  # noqa: F401  (the extension links against libtorch)

from .build import built_so_path



_loaded: dict = {}


def __getattr__(attr: str):
    if attr == "C":  # the main extension, loaded on first use
        return load("arks_amd_C")
    raise AttributeError(attr)


def load(name: str):
    if name in _loaded:
        return _loaded[name]
    so = built_so_path(name)
    if so is None:
        raise ImportError(
            f"{name}.so not found in arks_amd/ops/_build/{name} — run "
            f"`python -m arks_amd.ops.build {name}`"
        )
    spec = importlib.util.spec_from_file_location(name, so)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    _loaded[name] = mod
    return mod
