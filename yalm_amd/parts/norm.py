"""RMSNorm: out = x * rsqrt(mean(x^2) + eps) * weight, sums in float32
(src/infer.cpp:136-146, src/infer.cu:525-539).  The parameter `tensor` names the weight behind the
part's prefix (default "weight"); with `offset` c the stored tensor is the weight's distance from c (weight = c +
stored, formed in float32 and kept so, whatever the compute dtype: the sum has no bfloat16 of its own).  `add_normed` is the norm of a layer that norms a sublayer's OUTPUT:
x += norm(y)."""
import torch

from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, part


@part("norm", "rmsnorm")
class RMSNorm(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        self.eps = float(spec.params["eps"])
        self.tensor = self.prefix + str(spec.params.get("tensor", "weight"))
        self.offset = float(spec.params.get("offset", 0.0) or 0.0)
        self.weight = None

    def param_specs(self):
        return [ParamSpec(self.tensor, (self.dim,), init="norm_offset" if self.offset else "norm")]

    def load(self, get, compute_dtype, device):
        if self.offset:
            self.weight = (get(self.tensor).to(torch.float32) + self.offset).to(device).contiguous()
        else:
            self.weight = place(get(self.tensor), compute_dtype, device)
        self.weight_f32 = self.weight if self.weight.dtype == torch.float32 else self.weight.float()

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()

    def fused(self):
        """(float32 weight, eps) for a consumer that folds this norm into its first product."""
        return self.weight_f32, self.eps

    def forward(self, x, out, ctx, row_index=None):
        return kernels.rmsnorm(x, self.weight, out, self.eps, row_index)

    def add_normed(self, y, x, ctx, h_out=None, next_norm=None):
        """x += norm(y) (both float32 [T, dim]); h_out, if given, receives the new x in the compute dtype, or with
        next_norm (a norm that offers fused()) that norm's output for the new x."""
        return kernels.norm_add(y, self.weight, self.eps, x, h_out, None if next_norm is None else next_norm.fused())
