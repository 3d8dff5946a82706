"""Mixture of experts: `n_experts` small gated feed-forwards, of which a token uses the `top` whose router
scores are largest.

Router: s = softmax(W_router h (+ a bias, the tensor `router_bias`)) over all experts, in float32; the chosen experts'
weights are their scores (`renormalize`: divided by their sum; "chosen": the experts with the largest logits, weighted
by the softmax over the chosen logits alone).  Expert: g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit),
out = W_down (g sigmoid(alpha g) (u + up_shift)) (limit 0: no clamping; up_shift defaults to 1; alpha 1 and up_shift 0
make silu(gate) * up).  The part's result is the weighted sum over
a token's chosen experts, in the order of their scores.  With `shared` = {hidden, prefix, gate} one more expert of the
same form (its tensors behind `prefix`, its own hidden size) runs for every token and is added, times sigmoid(w . h), one
number a token (w: the tensor `gate` behind the prefix, [1, width]; no `gate`: added as it is).

The experts' matrices are stacked at load ([E, F, D], [E, F, D], [E, D, F]); routing happens on the device
(nothing of it reaches the host, so a decode step stays a captured graph), and every (token, choice) pair is
served from its expert's weights.  A step of GROUPED_MIN_ROWS rows or more (bfloat16; whole prompts, and decode
batches of 16 and more) groups the pairs by expert instead and multiplies every expert's rows as tiles on the
matrix cores, all experts in one launch a product: the grouped products read every chosen expert once while the
pairs would read it once a pair (measured at width 4,096, 32 experts of 2,048,
4 a token, four layers: batch 8 1.01 against 1.03 ms a step, batch 16 1.46 against 1.15, batch 64 3.32 against 1.44,
batch 128 5.54 against 1.60).  Both ways are decided on the device, so a decode step stays a captured graph."""
import torch

from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, part
from .swiglu import interleave_gate_up


GROUPED_MIN_ROWS = 9             # steps of this many rows and more group the pairs by expert


@part("feed_forward", "moe")
class MixtureOfExperts(Part):
    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.hidden = int(p["hidden"])
        self.n_experts = int(p["n_experts"])
        self.top = int(p["top"])
        self.limit = float(p.get("limit", 0.0) or 0.0)
        self.alpha = float(p.get("alpha", 1.0))
        self.up_shift = float(p.get("up_shift", 1.0))
        self.renormalize = p.get("renormalize", False)
        self.renormalize = "chosen" if self.renormalize == "chosen" else bool(self.renormalize)
        self.expert_prefix = str(p.get("expert_prefix", "experts.%d."))
        self.names = {"router": "router", "gate": "gate", "up": "up", "down": "down"}
        self.names.update(p.get("tensors") or {})
        self.router_bias = self.names.get("router_bias")           # a tensor's name, or no bias
        if not 0 < self.top <= self.n_experts or self.n_experts > kernels.MOE_MAX_EXPERTS:
            raise ValueError("mixture of experts: %d of %d experts is not offered (at most %d experts)"
                             % (self.top, self.n_experts, kernels.MOE_MAX_EXPERTS))
        self.w_router = self.w_gate = self.w_up = self.w_down = self.b_router = None
        self.shared = None
        if p.get("shared"):
            s = p["shared"]
            if self.limit or self.alpha != 1.0 or self.up_shift:
                raise ValueError("a shared expert is silu(gate) * up: it goes with limit 0, alpha 1 and up_shift 0")
            self.shared = {"hidden": int(s["hidden"]), "prefix": str(s.get("prefix", "shared.")), "gate": s.get("gate")}
        self.ws_gate_up = self.ws_down = self.ws_gate = None

    def _expert(self, e, key):
        return self.prefix + (self.expert_prefix % e) + self.names[key]

    def param_specs(self):
        D, F = self.dim, self.hidden
        out = [ParamSpec(self.prefix + self.names["router"], (self.n_experts, D), fan_in=D)]
        if self.router_bias:
            out.append(ParamSpec(self.prefix + self.router_bias, (self.n_experts,), init="bias"))
        for e in range(self.n_experts):
            out += [ParamSpec(self._expert(e, "gate"), (F, D), fan_in=D), ParamSpec(self._expert(e, "up"), (F, D), fan_in=D),
                    ParamSpec(self._expert(e, "down"), (D, F), fan_in=F)]
        if self.shared:
            Fs = self.shared["hidden"]
            out += [ParamSpec(self._shared("gate"), (Fs, D), fan_in=D), ParamSpec(self._shared("up"), (Fs, D), fan_in=D),
                    ParamSpec(self._shared("down"), (D, Fs), fan_in=Fs)]
            if self.shared["gate"]:
                out.append(ParamSpec(self.prefix + self.shared["prefix"] + self.shared["gate"], (1, D), fan_in=D))
        return out

    def _shared(self, key):
        return self.prefix + self.shared["prefix"] + self.names[key]

    def load(self, get, compute_dtype, device):
        E = self.n_experts
        self.w_router = place(get(self.prefix + self.names["router"]), compute_dtype, device)
        if self.router_bias:
            self.b_router = get(self.prefix + self.router_bias).to(torch.float32).to(device).contiguous()
        self.w_gate = place(torch.stack([get(self._expert(e, "gate")) for e in range(E)]), compute_dtype, device)
        self.w_up = place(torch.stack([get(self._expert(e, "up")) for e in range(E)]), compute_dtype, device)
        self.w_down = place(torch.stack([get(self._expert(e, "down")) for e in range(E)]), compute_dtype, device)
        if self.shared:
            self.ws_gate_up = place(interleave_gate_up(get(self._shared("gate")), get(self._shared("up"))), compute_dtype, device)
            self.ws_down = place(get(self._shared("down")), compute_dtype, device)
            if self.shared["gate"]:
                w = get(self.prefix + self.shared["prefix"] + self.shared["gate"]).reshape(-1)
                self.ws_gate = w.to(device=device, dtype=compute_dtype).contiguous()     # the activations' dtype

    def weight_bytes(self):
        """What a token's step reads: the router, `top` experts and the shared expert."""
        item = self.w_down.element_size()
        shared = (3 * self.shared["hidden"] + 1) * self.dim if self.shared else 0
        return (self.n_experts * self.dim + self.top * 3 * self.hidden * self.dim + shared) * item

    def row_elements(self):
        return max(self.top * self.hidden, self.shared["hidden"] if self.shared else 0)

    def _run(self, h, out, ctx, accumulate):
        self._routed(h, out, ctx, accumulate)
        if self.shared:                                   # after the routed experts: `out` holds their sum by now
            T, Fs = h.shape[0], self.shared["hidden"]
            mid = ctx.ws.get("moe.shared.hidden", (T, Fs), h.dtype)
            self._gemm(ctx, h, self.ws_gate_up, mid, kernels.EPI_GATED, hidden=Fs)
            if self.ws_gate is None:
                self._gemm(ctx, mid, self.ws_down, out, kernels.EPI_ADD_F32)
            else:
                y = ctx.ws.get("moe.shared.y", (T, self.dim), torch.float32)
                self._gemm(ctx, mid, self.ws_down, y, kernels.EPI_STORE_F32)
                kernels.gated_add(y, h, self.ws_gate, out, True)
        return out

    def _routed(self, h, out, ctx, accumulate):
        T = h.shape[0]
        ws = ctx.ws
        ids = ws.get("moe.ids", (T, self.top), torch.int32)
        wts = ws.get("moe.weights", (T, self.top), torch.float32)
        logits = ws.get("moe.logits", (T, self.n_experts), torch.float32)        # products exact, sums in float32
        self._gemm(ctx, h, self.w_router, logits, kernels.EPI_STORE_F32)
        kernels.moe_select(logits, ids, wts, self.renormalize, bias=self.b_router)
        if T >= GROUPED_MIN_ROWS and kernels.can_moe_grouped(self.dim, self.hidden, h.dtype, T * self.top, self.n_experts):
            return kernels.moe_grouped(h, self.w_gate, self.w_up, self.w_down, ids, wts, self.limit, self.alpha, ws.get,
                                       out, accumulate, up_shift=self.up_shift)
        mid = ws.get("moe.hidden", (T * self.top, self.hidden), h.dtype)
        kernels.moe_pair_gate_up(h, self.w_gate, self.w_up, ids, self.limit, self.alpha, mid, up_shift=self.up_shift)
        kernels.moe_pair_down(mid, self.w_down, ids, wts, out, accumulate)
        return out

    def forward(self, h, x, ctx):
        """Adds the result to x."""
        return self._run(h, x, ctx, True)

    def forward_to(self, h, y, ctx):
        """Writes the result to y (float32 [T, dim])."""
        return self._run(h, y, ctx, False)
