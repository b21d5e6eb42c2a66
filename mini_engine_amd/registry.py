"""Architecture name (config.json `architectures[0]`) -> the function that builds its model.

The reference hard-wires its one model class (engine/model_runner.py:5,36). Here
`register_architecture` makes a builder known, and `register_config`
(config/model_config.py) its typed config; both can be called from outside the
package, so another architecture needs no change to these files.
"""
from __future__ import annotations

from typing import Callable

from .config.model_config import ConfigError, config_class_for, register_config  # noqa: F401

_BUILDERS: dict[str, Callable] = {}


def register_architecture(name: str):
    def deco(fn):
        _BUILDERS[name] = fn
        return fn

    return deco


def builder_for(name: str) -> Callable:
    _load_builtin()
    try:
        return _BUILDERS[name]
    except KeyError:
        raise ConfigError(f"no model registered for architecture {name!r}; "
                          f"registered: {', '.join(sorted(_BUILDERS)) or '<none>'}") from None


def architectures() -> list:
    _load_builtin()
    return sorted(_BUILDERS)


def build_model(model_config, checkpoint_names=None):
    """Build the (unloaded) model of a typed config. A builder that has a parameter `checkpoint_names`
    is told which tensors the checkpoint stores (None: there is no checkpoint, weights will be drawn),
    for architectures whose shape depends on it (a head that is stored or not)."""
    import inspect

    builder = builder_for(type(model_config).architecture_name)
    if "checkpoint_names" in inspect.signature(builder).parameters:
        return builder(model_config, checkpoint_names=checkpoint_names)
    return builder(model_config)


def _load_builtin() -> None:
    from .models import qwen3  # noqa: F401  (registers itself)
