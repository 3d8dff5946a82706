"""The gated delta rule with a decay per key channel as a mixer: per head a state S [d, dv] in float32, zero for a new
sequence and kept from one step to the next in the cache's fixed-size per-sequence state, together with the last
inputs of the short convolutions.

Per token: q = W_q h and k = W_k h (`n_qk_heads` heads of `key_dim`), v = W_v h (`n_heads` heads of `value_dim`; head h
uses query/key head h / (n_heads / n_qk_heads)); each passes a causal convolution over time per channel (`conv_taps`
taps, the last one the current token's, zeros before the sequence's start) and silu; q and k become unit vectors a head,
x / sqrt(sum x^2 + unit_floor), q also times q_scale; beta = sigmoid(W_b h) per head; a decay per head and key channel,
g = exp(-exp(decay_log_h) softplus(W_a2 (W_a1 h) + decay_bias)); then per head
    S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
(the read-out sees the token's own write).  Each head's o is divided by its root mean square, multiplied by a weight
shared by the heads and by sigmoid(W_g2 (W_g1 h)), and W_o adds the result to the residual stream.

Products: q | k | v | b are one matrix with float32 results; the two low-rank pairs are two more products, the first
(a1 | g1, their inner sizes padded to multiples of 32 with zero rows) left in the compute dtype for the second (a2 and
g2 side by side on the diagonal of one matrix), whose float32 results the recurrence's kernels take.  Everything behind
the products is float32: see ops.kernels.gated_delta."""
import torch

from ..cache.manager import StateRequest
from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, part

NAMES = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "beta": "beta",
         "decay_log": "decay_log", "decay_bias": "decay_bias", "decay_in": "decay_in", "decay_out": "decay_out",
         "gate_in": "gate_in", "gate_out": "gate_out", "norm": "norm", "out": "o"}
RANK_PAD = 32


def _pad(n):
    return (n + RANK_PAD - 1) // RANK_PAD * RANK_PAD


@part("mixer", "gated_delta")
class GatedDelta(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.n_heads = int(p["n_heads"])
        self.n_qk_heads = int(p.get("n_qk_heads") or self.n_heads)
        self.key_dim = int(p["key_dim"])
        self.value_dim = int(p.get("value_dim") or self.key_dim)
        self.taps = int(p["conv_taps"])
        self.decay_rank = int(p["decay_rank"])
        self.gate_rank = int(p["gate_rank"])
        self.q_scale = float(p.get("q_scale") or self.key_dim ** -0.5)
        self.unit_floor = float(p.get("unit_floor", 1e-6))
        self.eps = float(p.get("eps", 1e-6))
        if self.n_heads % self.n_qk_heads:
            raise ValueError("n_heads %d is no multiple of n_qk_heads %d" % (self.n_heads, self.n_qk_heads))
        if not 0 < self.key_dim <= kernels.GATED_DELTA_MAX_KEY_DIM or not 0 < self.taps <= kernels.GATED_DELTA_MAX_TAPS:
            raise ValueError("gated delta rule: key heads of %d (at most %d) with %d taps (at most %d) are not offered"
                             % (self.key_dim, kernels.GATED_DELTA_MAX_KEY_DIM, self.taps, kernels.GATED_DELTA_MAX_TAPS))
        self.names = dict(NAMES)
        self.names.update(p.get("tensors") or {})
        self.qk = self.n_qk_heads * self.key_dim
        self.vv = self.n_heads * self.value_dim
        self.gk = self.n_heads * self.key_dim                 # the decays: a number per head and key channel
        self.channels = 2 * self.qk + self.vv
        self.w_in = self.w_low = self.w_low2 = self.wo = None
        self.conv_w = self.decay_log = self.decay_bias = self.w_norm = None

    def _n(self, key):
        return self.prefix + self.names[key]

    def param_specs(self):
        D, H, t = self.dim, self.n_heads, self.taps
        return [ParamSpec(self._n("q"), (self.qk, D), fan_in=D), ParamSpec(self._n("k"), (self.qk, D), fan_in=D),
                ParamSpec(self._n("v"), (self.vv, D), fan_in=D),
                ParamSpec(self._n("q_conv"), (self.qk, t), init="taps"), ParamSpec(self._n("k_conv"), (self.qk, t), init="taps"),
                ParamSpec(self._n("v_conv"), (self.vv, t), init="taps"),
                ParamSpec(self._n("beta"), (H, D), fan_in=D), ParamSpec(self._n("decay_log"), (H,), init="decay_log"),
                ParamSpec(self._n("decay_bias"), (self.gk,), init="bias"),
                ParamSpec(self._n("decay_in"), (self.decay_rank, D), fan_in=D),
                ParamSpec(self._n("decay_out"), (self.gk, self.decay_rank), fan_in=self.decay_rank),
                ParamSpec(self._n("gate_in"), (self.gate_rank, D), fan_in=D),
                ParamSpec(self._n("gate_out"), (self.vv, self.gate_rank), fan_in=self.gate_rank),
                ParamSpec(self._n("norm"), (self.value_dim,), init="norm"), ParamSpec(self._n("out"), (D, self.vv), fan_in=self.vv)]

    def load(self, get, compute_dtype, device):
        def f32(key):
            return get(self._n(key)).to(torch.float32).to(device).contiguous()
        self.w_in = place(torch.cat([get(self._n(k)) for k in ("q", "k", "v", "beta")], dim=0), compute_dtype, device)
        ra, rg = _pad(self.decay_rank), _pad(self.gate_rank)
        a1, g1, a2, g2 = (get(self._n(k)) for k in ("decay_in", "gate_in", "decay_out", "gate_out"))
        low = torch.zeros((ra + rg, self.dim), dtype=a1.dtype)
        low[:self.decay_rank] = a1
        low[ra:ra + self.gate_rank] = g1
        low2 = torch.zeros((self.gk + self.vv, ra + rg), dtype=a2.dtype)
        low2[:self.gk, :self.decay_rank] = a2
        low2[self.gk:, ra:ra + self.gate_rank] = g2
        self.w_low, self.w_low2 = place(low, compute_dtype, device), place(low2, compute_dtype, device)
        self.wo = place(get(self._n("out")), compute_dtype, device)
        self.conv_w = torch.cat([f32("q_conv"), f32("k_conv"), f32("v_conv")], dim=0).contiguous()
        self.decay_log, self.decay_bias, self.w_norm = f32("decay_log").reshape(-1), f32("decay_bias").reshape(-1), f32("norm").reshape(-1)

    def weight_bytes(self):
        return (self.w_in.numel() + self.w_low.numel() + self.w_low2.numel() + self.wo.numel()) * self.w_in.element_size()

    def state_elements(self):
        return kernels.gated_delta_state_elements(self.n_heads, self.n_qk_heads, self.key_dim, self.value_dim, self.taps)

    def cache_request(self):
        return StateRequest((self.state_elements(),), torch.float32)

    def row_elements(self):
        return self.channels + self.n_heads + self.gk

    def describe(self, compute_dtype):
        return "gated delta rule, %d heads of %d x %d on %d query heads, %d taps: a state column in the registers of four lanes, float32" % (
            self.n_heads, self.key_dim, self.value_dim, self.n_qk_heads, self.taps), False

    def forward(self, h, x, ctx, line, writes_cache=True):
        T = h.shape[0]
        ws, H = ctx.ws, self.n_heads
        proj = ws.get("gdelta.proj", (T, self.channels + H), torch.float32)
        self._gemm(ctx, h, self.w_in, proj, kernels.EPI_STORE_F32)
        mid = ws.get("gdelta.mid", (T, self.w_low.shape[0]), h.dtype)
        self._gemm(ctx, h, self.w_low, mid, kernels.EPI_STORE)
        low = ws.get("gdelta.low", (T, self.gk + self.vv), torch.float32)
        self._gemm(ctx, mid, self.w_low2, low, kernels.EPI_STORE_F32)
        prep = ws.get("gdelta.prep", (T, self.row_elements()), torch.float32)
        raw = ws.get("gdelta.raw", (T, self.vv), torch.float32)
        o = ws.get("gdelta.o", (T, self.vv), h.dtype)
        state = ctx.cache.group_of(line).line_state(line)
        kernels.gated_delta(proj, low, self.conv_w, self.decay_log, self.decay_bias, self.w_norm, state, prep, raw, ctx.tok_seq,
                            ctx.cu_seqlens, ctx.seq_slot, o, H, self.n_qk_heads, self.key_dim, self.value_dim, self.taps,
                            self.q_scale, self.unit_floor, self.eps)
        self._gemm(ctx, o, self.wo, x, kernels.EPI_ADD_F32)
