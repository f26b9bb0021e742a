"""Rotary position encoding.  The angles pos * f_p are computed once on the host
in float64 and kept as a float32 table of (cos, sin); the kernels rotate
adjacent pairs (x[2p], x[2p+1]) (src/infer.cpp:202-215).  Frequencies:
f_p = theta^(-2p / rotary_dim), optionally rescaled the llama3 way (not in the
reference): with wavelength lam = 2 pi / f and L the original context length,
lam < L/high -> f; lam > L/low -> f/factor; between, the linear blend
(1-s) f/factor + s f with s = (L/lam - low) / (high - low).

A model folder keeps q/k projection rows in the half-split order (pair p with
p + rotary_dim/2); `interleave_rows` re-orders them for adjacent pairs, as
convert.py:145-158 does offline."""
import math

import torch

from .base import Part, part


def inverse_frequencies(head_dim, rotary_dim, theta, scaling=None):
    """float64 [rotary_dim // 2]."""
    p = torch.arange(rotary_dim // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * p / max(rotary_dim, 1))
    if scaling:
        kind = scaling.get("rope_type", scaling.get("type"))
        if kind != "llama3":
            raise ValueError("rope scaling %r is not supported" % (kind,))
        factor = float(scaling["factor"])
        low, high = float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
        L = float(scaling["original_max_position_embeddings"])
        lam = 2.0 * math.pi / f
        s = (L / lam - low) / (high - low)
        blend = (1.0 - s) * f / factor + s * f
        f = torch.where(lam < L / high, f, torch.where(lam > L / low, f / factor, blend))
    return f


def interleave_rows(w, n_heads, head_dim, rotary_dim):
    """Rows of a [n_heads * head_dim, in] projection from half-split to adjacent-pair order."""
    if rotary_dim == 0:
        return w
    w = w.reshape(n_heads, head_dim, -1)
    rot = w[:, :rotary_dim].reshape(n_heads, 2, rotary_dim // 2, -1).transpose(1, 2).reshape(n_heads, rotary_dim, -1)
    return torch.cat([rot, w[:, rotary_dim:]], dim=1).reshape(n_heads * head_dim, -1)


@part("position", "rope")
class RotaryEncoding(Part):
    share_by_spec = True              # no tensors of its own: mixers that name the same spec share one table

    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.head_dim = int(p["head_dim"])
        self.rotary_dim = int(p.get("rotary_dim", self.head_dim))
        self.theta = float(p["theta"])
        self.scaling = p.get("scaling")
        self.weight_rows = p.get("weight_rows", "interleaved")
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ValueError("rotary_dim %d does not fit head_dim %d" % (self.rotary_dim, self.head_dim))
        self.table = None

    def prepare(self, n_positions, device):
        """The (cos, sin) table for positions < n_positions: float32 [n, rotary_dim/2, 2]."""
        if self.rotary_dim == 0:
            self.table = None
            return
        f = inverse_frequencies(self.head_dim, self.rotary_dim, self.theta, self.scaling)
        ang = torch.arange(n_positions, dtype=torch.float64)[:, None] * f[None, :]
        self.table = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).to(torch.float32).contiguous().to(device)

    @property
    def n_positions(self):
        return 0 if self.table is None else self.table.shape[0]

    def arrange_projection_rows(self, w, n_heads):
        """Brings q/k projection rows into the order the rotation kernel pairs."""
        if self.weight_rows == "half_split":
            return interleave_rows(w, n_heads, self.head_dim, self.rotary_dim)
        return w


@part("position", "none")
class NoPositionEncoding(Part):
    """No rotation at all (a mixer that needs no positions, or test parts)."""
    share_by_spec = True
    rotary_dim = 0
    table = None
    n_positions = 0

    def prepare(self, n_positions, device):
        pass

    def arrange_projection_rows(self, w, n_heads):
        return w
