"""Architectures and parts that live outside this package.

A plugin is a Python file (or an importable module) that, when executed, calls
the registries: `register_architecture(name, ConfigClass)` for a whole
architecture, `MIXERS.register(kind, Class)` and its siblings for parts.  The
command line and the replay tool load the plugins they are given before they
read a model's config.json, so a model folder of an architecture the package has
never heard of runs through the same loader, cache, step function and scheduler.

The reference's counterpart is the word table that each program fills before it
runs its model (`insert_native_word`, v1/tensortype/dag.hpp:389-394;
v1/models/qwen2-7b/chat.cpp:214-215).
"""
from __future__ import annotations

import importlib
import importlib.util
import os
import sys
from typing import Iterable, List

ENV_VAR = "VT_TRANSFORMER_PLUGINS"      # file paths or module names, separated like PATH

_loaded: List[str] = []


def load_plugin(spec: str) -> None:
    """Run one plugin: a path to a .py file, or a module name."""
    spec = spec.strip()
    if not spec or spec in _loaded:
        return
    if spec.endswith(".py") or os.sep in spec:
        path = os.path.abspath(spec)
        if not os.path.isfile(path):
            raise FileNotFoundError(f"plugin file '{spec}' does not exist")
        name = "vt_plugin_" + os.path.splitext(os.path.basename(path))[0] + f"_{len(_loaded)}"
        mod_spec = importlib.util.spec_from_file_location(name, path)
        module = importlib.util.module_from_spec(mod_spec)
        sys.modules[name] = module
        mod_spec.loader.exec_module(module)
    else:
        importlib.import_module(spec)
    _loaded.append(spec)


def load_plugins(specs: Iterable[str] = ()) -> List[str]:
    """The given plugins, then those that the environment names; returns what has been loaded so far."""
    for s in specs:
        load_plugin(s)
    for s in os.environ.get(ENV_VAR, "").split(os.pathsep):
        load_plugin(s)
    return list(_loaded)
