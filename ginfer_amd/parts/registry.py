"""Registries of part kinds.  A part is built from a `PartSpec` (kind + parameters); nothing else
reaches it, so no part knows which model it is in.  New kinds register themselves with the
decorators below; the model builder looks kinds up here and nowhere else."""

_REGISTRIES = {"mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "embedding": {}, "head": {},
               "arrangement": {}}


def _register(role, kind):
    def deco(cls):
        _REGISTRIES[role][kind] = cls
        return cls
    return deco


def register_mixer(kind):
    return _register("mixer", kind)


def register_feed_forward(kind):
    return _register("feed_forward", kind)


def register_norm(kind):
    return _register("norm", kind)


def register_position(kind):
    return _register("position", kind)


def register_embedding(kind):
    return _register("embedding", kind)


def register_head(kind):
    return _register("head", kind)


def register_arrangement(kind):
    return _register("arrangement", kind)


def lookup(role, kind):
    reg = _REGISTRIES[role]
    if kind not in reg:
        raise KeyError("no %s part of kind %r is registered (known: %s)" % (role, kind, ", ".join(sorted(reg)) or "none"))
    return reg[kind]


def registered(role):
    return sorted(_REGISTRIES[role])
