"""Model registry: config.json's `architecture` (or `architectures[0]`) -> the class that builds the served model.

A served model class provides
    from_config(config: dict, weights: dict[name -> tensor], ops, device) -> model
and the model
    vocab, width          sizes
    cache_rows            list of cache row widths (elements per token; (n, w): n pools of one allocation), one per paged pool
    state_specs           (optional) list of qserve_amd.serving.cache.StateSpec: fixed-size state per sequence
    forward(batch, pools[, states=]) -> the float residual stream after the last layer (whatever `logits` reads)
    logits(x, rows)       -> float [len(rows), vocab]
Families that run through another engine of this package register with `engine=` naming it (see qserve_amd.models).
"""
import importlib
import json
import os

_MODELS = {}
_BUILTIN = ("qserve_amd.models.vekalorn", "qserve_amd.models.mumelix", "qserve_amd.models.vepolix", "qserve_amd.models.pemolorn",
            "qserve_amd.models.llama_w4a8")


def register_model(architecture, engine="paged"):
    def deco(cls):
        _MODELS[architecture] = (cls, engine)
        return cls
    return deco


def _load_builtin():
    for m in _BUILTIN:
        importlib.import_module(m)


def architectures():
    _load_builtin()
    return {k: e for k, (_, e) in sorted(_MODELS.items())}


def read_config(model_dir):
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def architecture_of(config):
    a = config.get("architecture")
    if a is None and config.get("architectures"):
        a = config["architectures"][0]
    if a is None:
        raise ValueError("config.json names no architecture")
    return a


def resolve_model(config):
    """-> (class, engine kind) for a parsed config.json."""
    _load_builtin()
    a = architecture_of(config)
    if a not in _MODELS:
        raise ValueError(f"no served model registered for architecture {a!r} (known: {', '.join(sorted(_MODELS))})")
    return _MODELS[a]
