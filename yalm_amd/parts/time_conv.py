"""A short causal convolution over time on every channel of a sublayer's input, added to that input:
out[t] = h[t] + sum_j w[:, j] * h[t - (taps - 1) + j], zeros before a sequence's start (`residual` false: the
convolution alone).  The last taps - 1 inputs of a sequence are per-sequence state, kept in the cache's fixed-size state
under the line the layer hands it; the sums are float32."""
import torch

from ..cache.manager import StateRequest
from ..ops import kernels
from ..weights.loader import ParamSpec
from .base import Part, part


@part("input_filter", "time_conv")
class TimeConv(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        self.taps = int(spec.params["taps"])
        if not 0 < self.taps <= kernels.TIME_CONV_MAX_TAPS:
            raise ValueError("a convolution of %d taps is not offered (1 to %d)" % (self.taps, kernels.TIME_CONV_MAX_TAPS))
        self.residual = bool(spec.params.get("residual", True))
        self.tensor = self.prefix + str(spec.params.get("tensor", "conv"))
        self.w = None

    def param_specs(self):
        return [ParamSpec(self.tensor, (self.dim, self.taps), init="taps")]

    def load(self, get, compute_dtype, device):
        self.w = get(self.tensor).to(torch.float32).t().contiguous().to(device)      # tap by tap: [taps, dim]

    def weight_bytes(self):
        return self.dim * self.taps * 4

    def cache_request(self):
        return StateRequest((self.taps - 1, self.dim), torch.float32) if self.taps > 1 else None

    def forward(self, h, out, ctx, line):
        """out = h (+) conv(h) over the step's tokens, from the inputs that the line's state holds, which it leaves advanced."""
        carried = ctx.cache.group_of(line).line_state(line) if self.taps > 1 else None
        return kernels.time_conv(h, self.w, carried, out, ctx.tok_seq, ctx.cu_seqlens, ctx.seq_slot, self.residual,
                                 one_token_each=ctx.mode == "decode")
