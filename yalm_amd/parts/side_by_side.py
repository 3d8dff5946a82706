"""Two mixers side by side as one mixer: both read the same input, each result is normed over the model's width
(RMS, a plain weight of its own), and `weight` times their sum goes to the stream (`weight` 1/2: their mean).

The two are any registered mixers that offer forward_to (which writes a result instead of adding it); each keeps what
it keeps (keys and values in pages, a fixed-size state) under a cache line of its own: this mixer's cache request is
the pair {"left": ..., "right": ...}, and the cache manager gives line (l, "left") and (l, "right") to the members
of line l."""
import torch

from ..ops import kernels
from ..weights.loader import ParamSpec
from .base import Part, build_part, part


@part("mixer", "side_by_side")
class SideBySide(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.left = build_part("mixer", p["left"], dim, prefix)
        self.right = build_part("mixer", p["right"], dim, prefix)
        for m in (self.left, self.right):
            if not hasattr(m, "forward_to"):
                raise ValueError("a %s cannot stand beside another mixer: it has no forward_to" % type(m).__name__)
        self.eps = float(p.get("eps", 1e-6))
        self.weight = float(p.get("weight", 0.5))
        names = p.get("tensors") or {}
        self.left_norm = self.prefix + str(names.get("left_norm", "left.out"))
        self.right_norm = self.prefix + str(names.get("right_norm", "right.out"))
        self.w_left = self.w_right = None

    def children(self):
        return [self.left, self.right]

    @property
    def prompt_tables(self):
        return tuple(getattr(self.left, "prompt_tables", ())) + tuple(getattr(self.right, "prompt_tables", ()))

    def param_specs(self):
        return [ParamSpec(self.left_norm, (self.dim,), init="norm"), ParamSpec(self.right_norm, (self.dim,), init="norm")]

    def load(self, get, compute_dtype, device):
        # the share of each side rides on its norm's weight (exact for a power of two)
        self.w_left = (get(self.left_norm).to(torch.float32) * self.weight).to(device).contiguous()
        self.w_right = (get(self.right_norm).to(torch.float32) * self.weight).to(device).contiguous()

    def weight_bytes(self):
        return 2 * self.dim * 4

    def cache_request(self):
        return {"left": self.left.cache_request(), "right": self.right.cache_request()}

    def describe(self, compute_dtype):
        return "two mixers side by side, each normed over the width", False

    def forward(self, h, x, ctx, line, writes_cache=True):
        T = h.shape[0]
        y = ctx.ws.get("side.y", (T, self.dim), torch.float32)
        self.left.forward_to(h, y, ctx, (line, "left"), writes_cache)
        kernels.norm_add(y, self.w_left, self.eps, x)
        self.right.forward_to(h, y, ctx, (line, "right"), writes_cache)
        kernels.norm_add(y, self.w_right, self.eps, x)
