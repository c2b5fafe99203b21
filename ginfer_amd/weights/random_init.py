"""Random-weights mode: a model folder (config.json, model.safetensors) from a configuration and
a seed.  The reference has no such mode (it loads checkpoints only, ginfer/model/qwen2.cc:28-49).

Matrices, embeddings and biases are drawn from N(0, std); norm gains from 1 + N(0, std), as each
part's `WeightSpec.init` says.  The generator is counter-based: an element is a function of (seed, the
tensor's name, its index) alone, so a tensor's values do not depend on which other tensors the model has,
and the same function runs on the host (here) and on the device (`bind_random_weights`), bit for bit.
"""
import hashlib
import json
import os

import torch

from .safetensors_file import write_safetensors

_STORAGE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def _tensor_seed(seed, name):
    h = hashlib.sha256(("%d:%s" % (seed, name)).encode()).digest()
    return int.from_bytes(h[:8], "little") & ((1 << 63) - 1)


def draw(spec, seed, name, dtype, std_scale=1.0):
    """One tensor on the host: element i is mean + std * normal(key of (seed, name), i) from the counter-based
    generator that the device kernel shares (csrc/random_normal.h), rounded once to `dtype`."""
    if spec.kind == "int":
        return torch.zeros(spec.shape, dtype=torch.int32)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype)
    if spec.init == "ones":
        return torch.ones(spec.shape, dtype=dtype)
    if spec.init not in ("normal", "one_plus_normal"):
        raise ValueError("unknown init %r for %s" % (spec.init, name))
    import ctypes
    from ..kernels import build
    lib = build.load_host("random_fill_host")
    t = torch.empty(spec.shape, dtype=torch.float32)
    rc = lib.ga_random_normal_fill_host(ctypes.c_void_p(t.data_ptr()), ctypes.c_int64(t.numel()),
                                        ctypes.c_uint64(_tensor_seed(seed, name)),
                                        ctypes.c_float(1.0 if spec.init == "one_plus_normal" else 0.0),
                                        ctypes.c_float(spec.std * std_scale), ctypes.c_int(min(16, os.cpu_count() or 1)))
    if rc != 0:
        raise RuntimeError("the host's random fill failed for %s (code %d)" % (name, rc))
    return t.to(dtype)


def bind_random_weights(model, seed, device, std_scale=1.0):
    """Draws every tensor the model expects on the device and binds it: for shapes too large to pass
    through a file in reasonable time (a 72B shape is 145 GB).  Same generator and the same key (seed, tensor name)
    as `draw`: the model made here holds, bit for bit, what `write_random_model` writes for the same seed in the
    model's dtype."""
    from ..kernels import ops
    from .loader import TensorsOnDemand, target_dtype
    specs = model.weight_specs()

    def make(name):
        spec = specs[name]
        if spec.kind == "int":
            return torch.zeros(spec.shape, dtype=torch.int32, device=device)
        dt = target_dtype(spec, model.dtype, model.dtype)       # as a checkpoint stored in the compute dtype would load
        if spec.init in ("zeros", "ones"):
            return torch.full(spec.shape, 0.0 if spec.init == "zeros" else 1.0, dtype=dt, device=device)
        if spec.init not in ("normal", "one_plus_normal"):
            raise ValueError("unknown init %r for %s" % (spec.init, name))
        out = torch.empty(spec.shape, dtype=dt, device=device)
        ops.random_normal_fill(out, _tensor_seed(seed, name), 1.0 if spec.init == "one_plus_normal" else 0.0,
                               spec.std * std_scale)
        return out
    tensors = TensorsOnDemand(specs, make)
    model.bind_weights(tensors)
    return model


def write_random_model(folder, config, seed, dtype="bfloat16", std_scale=1.0):
    """Writes `folder/config.json` and `folder/model.safetensors`; returns the folder.  std_scale widens every
    normal draw: with the usual 0.02 a tiny model's blocks add so little to the embedding that greedy generation
    repeats one token."""
    from ..parts.model import build_model
    if dtype not in _STORAGE:
        raise ValueError("dtype must be one of %s" % sorted(_STORAGE))
    os.makedirs(folder, exist_ok=True)
    d = config.to_dict()
    d["torch_dtype"] = dtype
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(d, f, indent=1, sort_keys=True)
    model = build_model(config.model_spec(), _STORAGE[dtype], device=None)
    tensors = {}
    for name, spec in model.weight_specs().items():
        tensors[name] = draw(spec, seed, name, _STORAGE[dtype], std_scale)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": seed})
    return folder
