"""HGRN2 as a mixer: a gated linear recurrence whose forget gate also decides what is written.  Per head a state S
[key_dim, value_dim] in float32, zero for a new sequence and kept from one step to the next in the cache's fixed-size
per-sequence state.

Per token: q = silu(W_q h) and f = l + (1 - l) sigmoid(W_f h + b) (`n_heads` heads of `key_dim`; l, the gate's lower
bound per head and channel, is a tensor), v = W_v h (`n_heads` heads of `value_dim`); per head
    S <- diag(f) S + (1 - f) v^T;   o = S^T q
(there is no key of its own: what the gate forgets of a row is what the row takes in of the new values).  Each head's
o is divided by its root mean square, multiplied by a weight shared by the heads, and W_o carries the heads to the
stream.  q | f | v are one product with float32 results; everything behind it is float32 (ops.kernels.hgrn2)."""
import torch

from ..cache.manager import StateRequest
from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, part

NAMES = {"q": "q", "f": "f", "f_bias": "f.b", "lower": "lower", "v": "v", "norm": "norm", "out": "o"}


@part("mixer", "hgrn2")
class HGRN2(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.n_heads = int(p["n_heads"])
        self.key_dim = int(p["key_dim"])
        self.value_dim = int(p.get("value_dim") or self.key_dim)
        self.eps = float(p.get("eps", 1e-6))
        if self.n_heads <= 0 or not 0 < self.key_dim <= kernels.HGRN2_MAX_KEY_DIM or self.value_dim <= 0:
            raise ValueError("HGRN2: %d heads with keys of %d (at most %d) and values of %d are not offered"
                             % (self.n_heads, self.key_dim, kernels.HGRN2_MAX_KEY_DIM, self.value_dim))
        self.names = dict(NAMES)
        self.names.update(p.get("tensors") or {})
        self.qk = self.n_heads * self.key_dim
        self.vv = self.n_heads * self.value_dim
        self.w_in = self.wo = self.f_bias = self.lower = self.w_norm = None

    def _n(self, key):
        return self.prefix + self.names[key]

    def param_specs(self):
        D = self.dim
        return [ParamSpec(self._n("q"), (self.qk, D), fan_in=D), ParamSpec(self._n("f"), (self.qk, D), fan_in=D),
                ParamSpec(self._n("f_bias"), (self.qk,), init="bias"), ParamSpec(self._n("lower"), (self.qk,), init="fraction"),
                ParamSpec(self._n("v"), (self.vv, D), fan_in=D), ParamSpec(self._n("norm"), (self.value_dim,), init="norm"),
                ParamSpec(self._n("out"), (D, self.vv), fan_in=self.vv)]

    def load(self, get, compute_dtype, device):
        def f32(key):
            return get(self._n(key)).to(torch.float32).reshape(-1).to(device).contiguous()
        self.w_in = place(torch.cat([get(self._n(k)) for k in ("q", "f", "v")], dim=0), compute_dtype, device)
        self.wo = place(get(self._n("out")), compute_dtype, device)
        self.f_bias, self.lower, self.w_norm = f32("f_bias"), f32("lower"), f32("norm")

    def weight_bytes(self):
        return (self.w_in.numel() + self.wo.numel()) * self.w_in.element_size()

    def cache_request(self):
        return StateRequest((kernels.hgrn2_state_elements(self.n_heads, self.key_dim, self.value_dim),), torch.float32)

    def row_elements(self):
        return 2 * self.qk + self.vv

    def describe(self, compute_dtype):
        return "HGRN2, %d heads of %d x %d: a state column in the registers of eight lanes, float32" % (
            self.n_heads, self.key_dim, self.value_dim), False

    def forward(self, h, x, ctx, line, writes_cache=True):
        """Adds the mixer's result to the stream x."""
        return self._run(h, x, ctx, line, kernels.EPI_ADD_F32)

    def forward_to(self, h, y, ctx, line, writes_cache=True):
        """Writes the mixer's result to y (float32 [T, dim])."""
        return self._run(h, y, ctx, line, kernels.EPI_STORE_F32)

    def _run(self, h, x, ctx, line, epilogue):
        T = h.shape[0]
        ws = ctx.ws
        proj = ws.get("hgrn2.proj", (T, 2 * self.qk + self.vv), torch.float32)
        self._gemm(ctx, h, self.w_in, proj, kernels.EPI_STORE_F32)
        raw = ws.get("hgrn2.raw", (T, self.vv), torch.float32)
        o = ws.get("hgrn2.o", (T, self.vv), h.dtype)
        state = ctx.cache.group_of(line).line_state(line)
        kernels.hgrn2(proj, self.f_bias, self.lower, self.w_norm, state, raw, ctx.cu_seqlens, ctx.seq_slot, o, self.n_heads,
                      self.key_dim, self.value_dim, self.eps)
        self._gemm(ctx, o, self.wo, x, epilogue)
