"""Model registry: which class serves a model folder, chosen by its config.json.

A model class registers under the names its configuration files carry ("architecture", "architectures"[0] or "model_type") and offers
    from_config(cfg: dict, dtype, device) -> model        (no weights yet)
    load_weights(checkpoint) -> model                     (checkpoint: name -> CPU tensor mapping, e.g. checkpoint.load_dir)
`load_model(folder)` is the one entry point that the command line, the trace replayer and the tests use.
"""
import json
import os

from ._lib import ZLError

_MODELS = {}


def register_model(*names):
    def deco(cls):
        for n in names:
            _MODELS[n.lower()] = cls
        return cls
    return deco


def _ensure_builtin():
    from . import tupitar  # noqa: F401  (registers itself)
    from . import retotar  # noqa: F401
    from . import gutivik  # noqa: F401
    from . import gaparax  # noqa: F401
    from . import llama    # noqa: F401


def config_names(cfg):
    names = []
    if isinstance(cfg.get("architecture"), str):
        names.append(cfg["architecture"])
    names += [a for a in cfg.get("architectures", []) if isinstance(a, str)]
    if isinstance(cfg.get("model_type"), str):
        names.append(cfg["model_type"])
    return names


def model_class(cfg):
    _ensure_builtin()
    for n in config_names(cfg):
        if n.lower() in _MODELS:
            return _MODELS[n.lower()]
    raise ZLError(f"no registered model for {config_names(cfg) or 'a config without architecture / model_type'}; known: {sorted(_MODELS)}")


def registered():
    _ensure_builtin()
    return sorted(_MODELS)


def read_config(folder):
    with open(os.path.join(folder, "config.json")) as fh:
        return json.load(fh)


def load_model(folder, dtype="bfloat16", device="cuda:0"):
    from . import checkpoint
    cfg = read_config(folder)
    model = model_class(cfg).from_config(cfg, dtype=dtype, device=device)
    return model.load_weights(checkpoint.load_dir(folder))
