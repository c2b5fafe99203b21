"""Binding weights to a model by tensor name.

The model says which tensors it expects (`model.weight_specs()`: full name -> `WeightSpec`); the
file says which it holds.  Every disagreement (missing, unexpected, wrong shape, wrong kind of
dtype) is collected and raised as ONE error; tensors that the model does not read are, by themselves,
a warning (an error with `strict`).  Floating tensors are kept in the compute dtype
(bfloat16 or float32); integer tables become int32; a tensor whose spec says `keep_32bit` stays in
32-bit when the file stores it so.  The reference binds the same names without checking shapes
(ginfer/model/qwen2.cc:34-46, ginfer/model/loader/safetensor_loader.cc:44-81).
"""
from dataclasses import dataclass
from typing import Tuple

import torch

from .safetensors_file import open_model_files


@dataclass
class WeightSpec:
    shape: Tuple[int, ...]
    kind: str = "float"          # "float" or "int"
    init: str = "normal"         # "normal" N(0, std), "one_plus_normal" 1 + N(0, std), "zeros", "ones"
    std: float = 0.02
    keep_32bit: bool = False     # a tensor stored in 32-bit stays in 32-bit


class WeightError(ValueError):
    pass


def check_against(specs, available, where, unread=(), strict=False):
    """specs: name -> WeightSpec; available: name -> (dtype, shape); unread: names the file may hold
    although the model reads none of them.  Raises one WeightError that lists everything that is wrong
    (missing tensors, unexpected ones, wrong shapes or kinds), or returns the list of unexpected tensors.
    Tensors that the model does not read are no fault by themselves: the reference looks tensors up by name and
    never sees the others (ginfer/model/loader/safetensor_loader.cc:44-81), and checkpoints carry such tensors
    (a rotary table, say).  Where they are all that is wrong they are named in a warning; with `strict` they are
    an error."""
    missing = [n for n in specs if n not in available]
    unexpected = [n for n in available if n not in specs and n not in unread]
    wrong = []
    for n, s in specs.items():
        if n not in available:
            continue
        dtype, shape = available[n]
        if tuple(shape) != tuple(s.shape):
            wrong.append("%s: expected shape %s, found %s" % (n, list(s.shape), list(shape)))
        elif s.kind == "float" and not dtype.is_floating_point:
            wrong.append("%s: expected a floating tensor, found %s" % (n, dtype))
        elif s.kind == "int" and (dtype.is_floating_point or dtype == torch.bool):
            wrong.append("%s: expected an integer tensor, found %s" % (n, dtype))
    if not (missing or wrong) and not (strict and unexpected):
        if unexpected:
            import sys
            sys.stderr.write("[ginfer_amd] warning: %s holds %d tensor(s) that the model does not read: %s\n"
                             % (where, len(unexpected), ", ".join(sorted(unexpected))))
        return sorted(unexpected)
    lines = ["weights in %s do not match the model:" % where]
    if missing:
        lines.append("  missing tensors (%d): %s" % (len(missing), ", ".join(sorted(missing))))
    if unexpected:
        lines.append("  unexpected tensors (%d): %s" % (len(unexpected), ", ".join(sorted(unexpected))))
    if wrong:
        lines.append("  wrong tensors (%d):" % len(wrong))
        lines.extend("    " + w for w in wrong)
    err = WeightError("\n".join(lines))
    err.missing, err.unexpected, err.wrong = sorted(missing), sorted(unexpected), wrong
    raise err


def target_dtype(spec, stored_dtype, compute_dtype):
    if spec.kind == "int":
        return torch.int32
    if spec.keep_32bit and stored_dtype == torch.float32:
        return torch.float32
    return compute_dtype


class TensorsOnDemand:
    """A mapping name -> tensor that makes a tensor when it is asked for and keeps nothing: a model that binds
    part by part then never holds a second copy of more than one part's tensors (a part may stack or
    re-lay-out what it is given)."""

    def __init__(self, names, make):
        self._names, self._make = set(names), make

    def __getitem__(self, name):
        if name not in self._names:
            raise KeyError(name)
        return self._make(name)

    def __contains__(self, name):
        return name in self._names

    def keys(self):
        return sorted(self._names)


def load_weights(model, folder, device, strict=False):
    """Reads every tensor the model expects from `folder`, converts, uploads, and hands the
    dictionary to `model.bind_weights`.  strict: a tensor in the folder that the model does not read is an error
    instead of a warning."""
    specs = model.weight_specs()
    files = open_model_files(folder)
    available = {n: f.info(n) for n, f in files.items()}
    check_against(specs, available, folder, unread=set(getattr(model, "unread_weights", list)()), strict=strict)
    def fetch(name):
        cpu = files[name].tensor(name)
        dt = target_dtype(specs[name], cpu.dtype, model.dtype)
        # upload in the stored dtype, convert on the device: no host copy of a large checkpoint
        return cpu.to(device=device).to(dt).contiguous()
    model.bind_weights(TensorsOnDemand(specs, fetch))
    return model
