"""Random weights from a configuration and a seed.

Every element is a function of (seed, tensor name, element index) alone: a
64-bit mixing function over the index, keyed by a hash of seed and name, so a
tensor's values depend neither on the order in which tensors are made nor on
the device that makes them (up to the last bit of log/cos for the normal ones).
Distributions: embeddings N(0,1); linear weights U(-1/sqrt(in), 1/sqrt(in));
norm weights 1 + U(-0.1, 0.1).  `write_random_model` writes a model folder
(config.json + model.safetensors) that loads like any other."""
import hashlib
import json
import math
import os

import torch

from .safetensors_io import write_file

_CHUNK = 1 << 24
_MASK64 = (1 << 64) - 1


def _i64(v):
    v &= _MASK64
    return v - (1 << 64) if v >= (1 << 63) else v


_C1 = _i64(0xBF58476D1CE4E5B9)
_C2 = _i64(0x94D049BB133111EB)
_GOLD = _i64(0x9E3779B97F4A7C15)


def _lsr(x, n):
    """Logical shift right of int64 tensors (torch's >> keeps the sign)."""
    return (x >> n) & ((1 << (64 - n)) - 1)


def _mix(x):
    x = (x ^ _lsr(x, 30)) * _C1
    x = (x ^ _lsr(x, 27)) * _C2
    return x ^ _lsr(x, 31)


def tensor_key(seed, name):
    h = hashlib.blake2b(("%d/%s" % (seed, name)).encode(), digest_size=8).digest()
    return _i64(int.from_bytes(h, "little"))


def _uniform01(key, start, count, stream, device):
    """count numbers in [0, 1) with 24 random bits, for the indices start.. ."""
    idx = torch.arange(start, start + count, dtype=torch.int64, device=device)
    bits = _mix(_mix(idx * _GOLD + key) + stream)
    return _lsr(bits, 40).to(torch.float32) * (1.0 / (1 << 24))


def random_values(name, shape, init, fan_in, seed, device="cpu"):
    """A float32 tensor of the given shape drawn as `init` says."""
    numel = 1
    for s in shape:
        numel *= s
    key = tensor_key(seed, name)
    out = torch.empty(numel, dtype=torch.float32, device=device)
    for start in range(0, numel, _CHUNK):
        n = min(_CHUNK, numel - start)
        u = _uniform01(key, start, n, 0, device)
        if init == "linear":
            a = 1.0 / math.sqrt(fan_in)
            v = (u * 2.0 - 1.0) * a
        elif init == "norm":
            v = 1.0 + (u * 2.0 - 1.0) * 0.1
        elif init == "embedding":
            u2 = _uniform01(key, start, n, 1, device)
            v = torch.sqrt(-2.0 * torch.log(u + (1.0 / (1 << 24)))) * torch.cos((2.0 * math.pi) * u2)
        elif init == "zeros":
            v = torch.zeros(n, dtype=torch.float32, device=device)
        else:
            raise ValueError("unknown init %r for %s" % (init, name))
        out[start:start + n] = v
    return out.reshape(shape)


def write_random_model(folder, config, seed, dtype=torch.float32, device="cpu"):
    """Writes config.json and model.safetensors for `config` (a config.json
    dictionary or a typed configuration) with weights drawn from `seed`, stored
    in `dtype`.  device: where the values are drawn (a GPU makes billions of them
    in seconds).  Returns the folder."""
    from ..config import config_from_dict
    from ..engine.model import param_specs_of
    cfg = config_from_dict(config) if isinstance(config, dict) else config
    os.makedirs(folder, exist_ok=True)
    tensors = {}
    for spec in param_specs_of(cfg.to_spec()):
        if spec.optional:
            continue
        tensors[spec.name] = random_values(spec.name, spec.shape, spec.init, spec.fan_in, seed,
                                           device=device).to(dtype).cpu()
    write_file(os.path.join(folder, "model.safetensors"), tensors, {"format": "pt", "seed": seed})
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg.to_dict(), f, indent=1)
    return folder
