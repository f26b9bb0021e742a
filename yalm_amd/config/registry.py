"""One registry from an architecture's name (config.json `architectures[0]`) to
its typed configuration, and through `to_spec()` to its model.  A configuration
class offers `from_dict(config_json) -> cfg`, `cfg.to_dict()`, `cfg.to_spec()
-> ModelSpec` and optionally `cfg.with_window(n)`."""
import json
import os

from .llama import ConfigError, LlamaConfig

_ARCHITECTURES = {}


def register_architecture(name, config_class, replace=False):
    if name in _ARCHITECTURES and not replace and _ARCHITECTURES[name] is not config_class:
        raise ValueError("architecture %r is already registered" % name)
    _ARCHITECTURES[name] = config_class


def unregister_architecture(name):
    _ARCHITECTURES.pop(name, None)


def registered_architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(d):
    """The typed configuration of a config.json dictionary, chosen by its architecture."""
    archs = d.get("architectures") or []
    name = archs[0] if archs else None
    if name not in _ARCHITECTURES:
        # convert.py:24-27: an unknown architecture is an error that lists the known ones
        raise ConfigError("architecture %r is not supported; registered: %s" % (name, registered_architectures()))
    return _ARCHITECTURES[name].from_dict(d)


def config_from_folder(path):
    f = os.path.join(path, "config.json")
    if not os.path.exists(f):
        raise ConfigError("no config.json in %s" % path)                # convert.py:223-224
    with open(f) as fh:
        return config_from_dict(json.load(fh))


for _name in LlamaConfig.ARCHITECTURES:
    register_architecture(_name, LlamaConfig)
