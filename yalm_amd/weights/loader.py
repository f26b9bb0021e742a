"""Weights by tensor name.  Parts declare the tensors they need (ParamSpec); the
loader opens every *.safetensors of a model folder (convert.py:229-230), checks
the declared set against the files in one pass, and fails with ONE error that
lists missing tensors, unexpected tensors and wrong shapes (the reference's
get_tensor / check_tensor, src/model.cpp:98-126, stop at the first).  Tensors
that no part declared are not an error by themselves: the reference's converter
picks what it needs by name and passes over the rest (convert.py:127-207), and
real folders carry such extras (`...rotary_emb.inv_freq` buffers, an
`lm_head.weight` stored next to a tied embedding); they are named in a warning,
and in the error if there is one, where a misspelt name shows as a missing and
an unexpected tensor side by side.

Precision on the device: with compute dtype float32 every floating tensor
becomes float32; with bfloat16, matrices become bfloat16 while a vector that is
stored in 32-bit stays so (norm weights, model.cpp:156-161); integer tables
become int32."""
import os
import sys
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile


class WeightsError(ValueError):
    pass


@dataclass(frozen=True)
class ParamSpec:
    """A tensor a part needs: full name in the folder, shape, and how random
    weights are drawn for it ('linear': U(-1/sqrt(fan_in), 1/sqrt(fan_in));
    'norm': 1 + U(-0.1, 0.1); 'embedding': N(0, 1); 'zeros')."""
    name: str
    shape: Tuple[int, ...]
    init: str = "linear"
    fan_in: Optional[int] = None
    optional: bool = False


class TensorSource:
    """Every tensor of a model folder, by name, as CPU views of the mapped files."""

    def __init__(self, folder):
        self.folder = folder
        names = sorted(n for n in os.listdir(folder) if n.endswith(".safetensors"))
        if not names:
            raise WeightsError("no .safetensors files found in %s" % folder)             # convert.py:231-232
        self.files = []
        self.where = {}
        for n in names:
            try:
                f = SafetensorsFile(os.path.join(folder, n))
            except SafetensorsError as e:
                raise WeightsError(str(e)) from None
            self.files.append(f)
            for key in f.entries:
                if key in self.where:                                                   # convert.py:139
                    raise WeightsError("tensor %r occurs in both %s and %s" % (key, self.where[key].path, f.path))
                self.where[key] = f

    def names(self):
        return set(self.where)

    def shape(self, name):
        return self.where[name].entries[name].shape

    def dtype(self, name):
        return self.where[name].entries[name].torch_dtype

    def has(self, name):
        return name in self.where

    def get(self, name):
        return self.where[name].tensor(name)

    def check(self, specs, strict=False):
        """Compares the declared tensors with the files; one error for everything.  Tensors that
        nobody declared are an error only with strict=True; else they are passed over with a
        warning.  Returns their names."""
        want = {}
        for s in specs:
            want[s.name] = s
        missing = [n for n, s in want.items() if n not in self.where and not s.optional]
        unexpected = sorted(self.names() - set(want))
        wrong = []
        for n, s in want.items():
            if n in self.where:
                if tuple(self.shape(n)) != tuple(s.shape):
                    wrong.append("%s: expected %s, found %s" % (n, list(s.shape), list(self.shape(n))))
                elif not self.dtype(n).is_floating_point and s.init != "table":
                    wrong.append("%s: expected a floating-point tensor, found %s" % (n, self.dtype(n)))
        if missing or wrong or (unexpected and strict):
            lines = ["the tensors in %s do not match the model:" % self.folder]
            if missing:
                lines.append("  missing (%d): %s" % (len(missing), ", ".join(sorted(missing))))
            if unexpected:
                lines.append("  unexpected (%d): %s" % (len(unexpected), ", ".join(unexpected)))
            if wrong:
                lines.append("  wrong shape or dtype (%d): %s" % (len(wrong), "; ".join(sorted(wrong))))
            raise WeightsError("\n".join(lines))
        if unexpected:
            shown = ", ".join(unexpected[:8]) + (", ..." if len(unexpected) > 8 else "")
            sys.stderr.write("[yalm_amd] %d tensors in %s are not used by the model and are passed over: %s\n"
                             % (len(unexpected), self.folder, shown))
        return unexpected


def device_dtype(stored_dtype, ndim, compute_dtype):
    """The dtype a tensor takes on the device (see the module text)."""
    if not stored_dtype.is_floating_point:
        return torch.int32
    if compute_dtype == torch.float32:
        return torch.float32
    if ndim <= 1 and stored_dtype in (torch.float32, torch.float64):
        return torch.float32
    return compute_dtype


def place(t, compute_dtype, device):
    """Copies a CPU tensor to the device in the dtype `device_dtype` gives it."""
    return t.to(device=device, dtype=device_dtype(t.dtype, t.dim(), compute_dtype)).contiguous()
