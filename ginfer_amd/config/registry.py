"""One registry from an architecture's name to its typed configuration (and through it, its model).

config.json's `architectures[0]` is the key; `model_type` is accepted as a second name, which is
what the reference dispatches on (ginfer/model/model_factory.h:16-27).
"""
import json
import os

_ARCHITECTURES = {}


class ConfigError(ValueError):
    pass


def register_architecture(*names):
    """Class decorator: `cls.from_dict(dict) -> config` and `config.model_spec() -> ModelSpec`."""
    def deco(cls):
        for n in names:
            _ARCHITECTURES[n] = cls
        return cls
    return deco


def registered_architectures():
    return sorted(_ARCHITECTURES)


def config_class(name):
    if name not in _ARCHITECTURES:
        raise ConfigError("unknown architecture %r; registered: %s"
                          % (name, ", ".join(registered_architectures())))
    return _ARCHITECTURES[name]


def config_from_dict(d):
    archs = d.get("architectures") or []
    names = list(archs[:1]) + ([d["model_type"]] if "model_type" in d else [])
    if not names:
        raise ConfigError("config.json has neither 'architectures' nor 'model_type'; registered: %s"
                          % ", ".join(registered_architectures()))
    for n in names:
        if n in _ARCHITECTURES:
            return _ARCHITECTURES[n].from_dict(d)
    raise ConfigError("unknown architecture %s (from config.json 'architectures'/'model_type'); "
                      "registered: %s" % (" / ".join(map(repr, names)),
                                          ", ".join(registered_architectures())))


def config_from_folder(folder):
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError("no config.json in %s" % folder)
    with open(path) as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError("%s is not valid JSON: %s" % (path, e))
    return config_from_dict(d)
