"""Feed-forward of two matrices without a gate: x += down(act(up h)), act the gelu with the error function
(`activation` "gelu_erf": z/2 (1 + erf(z / sqrt 2))), its tanh form ("gelu_tanh") or silu.  The first product's sums
stay float32 until the activation has been applied; its result is rounded to the compute dtype once, for the second
product, whose epilogue adds to the float32 residual stream."""
import torch

from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, part


@part("feed_forward", "dense_mlp")
class DenseMLP(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        self.hidden = int(spec.params["hidden"])
        self.activation = str(spec.params.get("activation", "gelu_erf"))
        if self.activation not in kernels.ACTIVATIONS:
            raise ValueError("feed-forward activation %r is not offered (%s)" % (self.activation, ", ".join(kernels.ACTIVATIONS)))
        self.names = {"up": "up_proj.weight", "down": "down_proj.weight"}
        self.names.update(spec.params.get("tensors") or {})
        self.w_up = self.w_down = None

    def param_specs(self):
        D, F = self.dim, self.hidden
        return [ParamSpec(self.prefix + self.names["up"], (F, D), fan_in=D),
                ParamSpec(self.prefix + self.names["down"], (D, F), fan_in=F)]

    def load(self, get, compute_dtype, device):
        self.w_up = place(get(self.prefix + self.names["up"]), compute_dtype, device)
        self.w_down = place(get(self.prefix + self.names["down"]), compute_dtype, device)

    def weight_bytes(self):
        return 2 * self.hidden * self.dim * self.w_down.element_size()

    def row_elements(self):
        return self.hidden

    def describe(self, compute_dtype):
        return "feed-forward of two matrices, %s between them, hidden %d" % (self.activation, self.hidden), False

    def _hidden(self, h, ctx):
        T = h.shape[0]
        z = ctx.ws.get("mlp.z", (T, self.hidden), torch.float32)
        self._gemm(ctx, h, self.w_up, z, kernels.EPI_STORE_F32)
        return kernels.activate(z, ctx.ws.get("mlp.mid", (T, self.hidden), h.dtype), self.activation)

    def forward(self, h, x, ctx):
        """Adds the result to x."""
        self._gemm(ctx, self._hidden(h, ctx), self.w_down, x, kernels.EPI_ADD_F32)

    def forward_to(self, h, y, ctx):
        """Writes the result to y (float32 [T, dim])."""
        self._gemm(ctx, self._hidden(h, ctx), self.w_down, y, kernels.EPI_STORE_F32)
