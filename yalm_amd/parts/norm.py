"""RMSNorm: out = x * rsqrt(mean(x^2) + eps) * weight, sums in float32
(src/infer.cpp:136-146, src/infer.cu:525-539)."""
import torch

from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, part


@part("norm", "rmsnorm")
class RMSNorm(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        self.eps = float(spec.params["eps"])
        self.weight = None

    def param_specs(self):
        return [ParamSpec(self.prefix + "weight", (self.dim,), init="norm")]

    def load(self, get, compute_dtype, device):
        self.weight = place(get(self.prefix + "weight"), compute_dtype, device)
        self.weight_f32 = self.weight if self.weight.dtype == torch.float32 else self.weight.float()

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()

    def fused(self):
        """(float32 weight, eps) for a consumer that folds this norm into its first product."""
        return self.weight_f32, self.eps

    def forward(self, x, out, ctx, row_index=None):
        return kernels.rmsnorm(x, self.weight, out, self.eps, row_index)
