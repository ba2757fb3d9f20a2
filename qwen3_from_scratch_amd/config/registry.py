"""One registry from an architecture's name to its configuration class and model
builder, and one from a part's (kind, name) to its class.

The reference keeps a single component registry keyed by slot and name
(src/qwen3_from_scratch/factory/factory.py:12-54) and hard-codes the model
class; here the model class is looked up by config.json's `architectures[0]`.
"""

import importlib
import json
import os

from .model_config import ConfigError

# Modules named here (comma-separated, importable) are imported the first time an
# architecture or a part is looked up and not found: they register architectures and
# parts that live outside this package, for the programs that take only a model folder.
PLUGINS_VARIABLE = "QWEN3_FROM_SCRATCH_AMD_PLUGINS"
_plugins_imported = False

_ARCHITECTURES = {}
_PARTS = {}

PART_KINDS = ("embedding", "position", "norm", "mixer", "feed_forward", "block", "head")


def register_architecture(name, config_class, build_spec):
    """`config_class.from_dict(json)` gives the typed configuration and
    `build_spec(config)` the model's description (a ModelSpec)."""
    _ARCHITECTURES[name] = (config_class, build_spec)


def architectures():
    return sorted(_ARCHITECTURES)


def import_plugins():
    """Import the modules that $QWEN3_FROM_SCRATCH_AMD_PLUGINS names, once."""
    global _plugins_imported
    if _plugins_imported:
        return
    _plugins_imported = True
    for module in os.environ.get(PLUGINS_VARIABLE, "").split(","):
        module = module.strip()
        if module:
            try:
                importlib.import_module(module)
            except ImportError as exc:
                raise ConfigError("$%s names %r, which cannot be imported: %s" % (PLUGINS_VARIABLE, module, exc)) from exc


def lookup_architecture(name):
    if name not in _ARCHITECTURES:
        import_plugins()
    if name not in _ARCHITECTURES:
        raise ConfigError(
            "architecture %r is not registered; known: %s" % (name, ", ".join(architectures()))
        )
    return _ARCHITECTURES[name]


def load_model_config(model_dir):
    """Read `model_dir`/config.json into the typed configuration of its architecture."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError("no config.json in %s" % model_dir)
    with open(path) as fh:
        data = json.load(fh)
    names = data.get("architectures")
    if not names or not isinstance(names, list):
        raise ConfigError(
            "config.json: 'architectures' must name the model class; known: %s"
            % ", ".join(architectures())
        )
    config_class, _ = lookup_architecture(names[0])
    return config_class.from_dict(data)


def register_part(kind, name):
    """Class decorator: make a part available as PartSpec(kind, name, ...)."""
    if kind not in PART_KINDS:
        raise ValueError("unknown part kind %r; kinds: %s" % (kind, ", ".join(PART_KINDS)))

    def decorate(cls):
        _PARTS.setdefault(kind, {})[name] = cls
        return cls

    return decorate


def lookup_part(kind, name):
    if name not in _PARTS.get(kind, {}):
        import_plugins()
    try:
        return _PARTS[kind][name]
    except KeyError:
        raise ConfigError(
            "no %s part named %r; registered: %s"
            % (kind, name, ", ".join(sorted(_PARTS.get(kind, {}))))
        ) from None


def part_names(kind):
    return sorted(_PARTS.get(kind, {}))
