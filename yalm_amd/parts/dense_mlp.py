"""Feed-forward of two matrices without a gate: x += down(act(up h)), act the gelu with the error function
(`activation` "gelu_erf": z/2 (1 + erf(z / sqrt 2))), its tanh form ("gelu_tanh") or silu.  The first product's sums
stay float32 until the activation has been applied; its result is rounded to the compute dtype once, for the second
product, whose epilogue adds to the float32 residual stream.  With `gated` there is a third matrix and the middle is
act(gate h) * (up h) (gate and up are one product); with `biases` every product has a bias (tensors "<name>.b" unless
named otherwise): those of the first products are added before the activation, the last one's goes to the stream
with the kernel of the middle."""
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
        self.gated = bool(spec.params.get("gated", False))
        self.biases = bool(spec.params.get("biases", False))
        self.names = {"up": "up_proj.weight", "down": "down_proj.weight", "gate": "gate_proj.weight"}
        self.names.update(spec.params.get("tensors") or {})
        for k in ("up", "down", "gate"):
            self.names.setdefault(k + "_bias", self.names[k] + ".b")
        self.w_up = self.w_down = self.b_up = self.b_down = None

    def _first(self):
        return ("gate", "up") if self.gated else ("up",)

    def param_specs(self):
        D, F = self.dim, self.hidden
        out = [ParamSpec(self.prefix + self.names[k], (F, D), fan_in=D) for k in self._first()]
        out.append(ParamSpec(self.prefix + self.names["down"], (D, F), fan_in=F))
        if self.biases:
            out += [ParamSpec(self.prefix + self.names[k + "_bias"], (F,), init="bias") for k in self._first()]
            out.append(ParamSpec(self.prefix + self.names["down_bias"], (D,), init="bias"))
        return out

    def load(self, get, compute_dtype, device):
        self.w_up = place(torch.cat([get(self.prefix + self.names[k]) for k in self._first()], dim=0), compute_dtype, device)
        self.w_down = place(get(self.prefix + self.names["down"]), compute_dtype, device)
        if self.biases:
            self.b_up = torch.cat([get(self.prefix + self.names[k + "_bias"]).to(torch.float32).reshape(-1)
                                   for k in self._first()]).to(device).contiguous()
            self.b_down = get(self.prefix + self.names["down_bias"]).to(torch.float32).reshape(-1).to(device).contiguous()

    def weight_bytes(self):
        return (3 if self.gated else 2) * self.hidden * self.dim * self.w_down.element_size()

    def row_elements(self):
        return self.hidden

    def describe(self, compute_dtype):
        return "feed-forward of two matrices, %s between them, hidden %d" % (self.activation, self.hidden), False

    def _hidden(self, h, ctx, x=None):
        """The middle of the layer in the compute dtype; with x, the last product's bias is added to x on the way."""
        T = h.shape[0]
        z = ctx.ws.get("mlp.z", (T, self.w_up.shape[0]), torch.float32)
        self._gemm(ctx, h, self.w_up, z, kernels.EPI_STORE_F32)
        mid = ctx.ws.get("mlp.mid", (T, self.hidden), h.dtype)
        if not self.gated and not self.biases:
            return kernels.activate(z, mid, self.activation)
        if not self.gated:
            raise ValueError("biases on an ungated feed-forward are not offered")
        return kernels.gated_bias_act(z, self.b_up, mid, self.activation, x, self.b_down if x is not None else None)

    def forward(self, h, x, ctx):
        """Adds the result to x."""
        self._gemm(ctx, self._hidden(h, ctx, x if self.biases else None), self.w_down, x, kernels.EPI_ADD_F32)

    def forward_to(self, h, y, ctx):
        """Writes the result to y (float32 [T, dim])."""
        if self.biases:
            raise ValueError("a feed-forward with biases adds to the stream only")
        self._gemm(ctx, self._hidden(h, ctx), self.w_down, y, kernels.EPI_STORE_F32)
