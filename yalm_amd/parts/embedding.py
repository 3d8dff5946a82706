"""Token embedding (optionally scaled, optionally with a sinusoidal position vector) and the LM head.  The head is the embedding table itself
when tied (src/model.cpp:389-398); one copy on the device either way."""
from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .base import Part, build_part, part


@part("embedding", "token_embedding")
class TokenEmbedding(Part):
    """x[t] = float(table[token[t]]) (src/infer.cpp:454-475), times `scale` (default 1), plus, with `sinusoid_base` b,
    a position vector whose entry 2i is sin(p b^(-2i / width)) and whose entry 2i + 1 is the cosine of the same angle
    (the frequencies are made in float64 and the angle is exact at every position), or, with `position_tensor` (a
    tensor's name) and `n_positions`, plus the row of that learned table [n_positions, width] at the token's position.
    With `norm` (a norm's PartSpec) the result passes that norm at once, in float32; with `keep_output` a copy of what the
    part leaves stays in the step's buffer "embed.kept" for layers that read it again (the way into looped layers)."""

    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        self.vocab_size = int(spec.params["vocab_size"])
        self.tensor = self.prefix + str(spec.params.get("tensor", "weight"))      # the table's name in a folder
        self.scale = float(spec.params.get("scale", 1.0))
        self.sinusoid_base = spec.params.get("sinusoid_base")
        self.position_tensor = spec.params.get("position_tensor")
        self.n_positions = int(spec.params.get("n_positions", 0) or 0)
        if self.position_tensor and (self.sinusoid_base or self.n_positions <= 0):
            raise ValueError("a learned position table needs n_positions, and goes without the sinusoid")
        self.table = None
        self.freq = None
        self.positions = None
        self.norm = build_part("norm", spec.params["norm"], dim, prefix) if spec.params.get("norm") else None
        self.keep_output = bool(spec.params.get("keep_output", False))

    def children(self):
        return [self.norm] if self.norm is not None else []

    def param_specs(self):
        out = [ParamSpec(self.tensor, (self.vocab_size, self.dim), init="embedding")]
        if self.position_tensor:
            out.append(ParamSpec(self.prefix + str(self.position_tensor), (self.n_positions, self.dim), init="embedding"))
        return out

    def load(self, get, compute_dtype, device):
        self.table = place(get(self.tensor), compute_dtype, device)
        if self.position_tensor:
            self.positions = place(get(self.prefix + str(self.position_tensor)), compute_dtype, device)
        if self.sinusoid_base:
            import torch
            i = torch.arange((self.dim + 1) // 2, dtype=torch.float64)
            base = torch.tensor(float(self.sinusoid_base), dtype=torch.float64)
            self.freq = torch.pow(base, -2.0 * i / self.dim).to(device)

    def weight_bytes(self):
        return (2 if self.positions is not None else 1) * self.dim * self.table.element_size()     # one row per token

    def forward(self, tokens, x, ctx):
        import torch
        kept = ctx.ws.get("embed.kept", tuple(x.shape), torch.float32) if self.keep_output else None
        if self.norm is None:
            self._rows(tokens, x, ctx)
            if kept is not None:
                self._rows(tokens, kept, ctx)
            return x
        raw = ctx.ws.get("embed.raw", tuple(x.shape), torch.float32)
        self._rows(tokens, raw, ctx)
        self.norm.forward(raw, x, ctx)
        if kept is not None:
            self.norm.forward(raw, kept, ctx)
        return x

    def _rows(self, tokens, x, ctx):
        if self.positions is not None:
            if ctx.max_position >= self.n_positions:
                raise ValueError("position %d is beyond the %d rows of the position table" % (ctx.max_position, self.n_positions))
            return kernels.embed_learned(self.table, self.positions, tokens, ctx.tok_pos, self.scale, x)
        if self.freq is None and self.scale == 1.0:
            return kernels.embed(self.table, tokens, x)
        return kernels.embed_sinusoid(self.table, tokens, ctx.tok_pos, self.freq, self.scale, x)


@part("head", "lm_head")
class LMHead(Part):
    """logits = W h in float32; W is the embedding table when tied (src/infer.cpp:508-521)."""

    def __init__(self, spec, dim, prefix, embedding=None):
        super().__init__(spec, dim, prefix)
        self.vocab_size = int(spec.params["vocab_size"])
        self.tied = bool(spec.params.get("tied", False))
        self.tensor = self.prefix + str(spec.params.get("tensor", "weight"))
        self.embedding = embedding
        self.weight = None
        if self.tied and embedding is None:
            raise ValueError("a tied head needs the embedding part")

    def param_specs(self):
        if self.tied:
            return []
        return [ParamSpec(self.tensor, (self.vocab_size, self.dim), init="linear", fan_in=self.dim)]

    def load(self, get, compute_dtype, device):
        self.weight = self.embedding.table if self.tied else place(get(self.tensor), compute_dtype, device)

    def weight_bytes(self):
        return self.weight.numel() * self.weight.element_size()

    def fuses_norm(self, norm, x, ctx):
        if not hasattr(norm, "fused") or ctx.mode != "decode":
            return False
        if id(norm) in ctx.normed:
            return True                                   # whoever prepared it checked the shape
        return kernels.can_fuse_norm(x.shape[0], self.dim, self.weight.dtype)

    def forward_prenorm(self, x, norm, logits, ctx):
        """logits for every row of x (no row selection)."""
        src = ctx.normed.pop(id(norm), None)
        if src is not None and src[1] is None:            # the norm's output is ready
            return self._gemm(ctx, src[0], self.weight, logits, kernels.EPI_STORE_F32)
        if src is not None:
            xn, ss, eps = src
            if kernels.can_chain(xn.shape[0], self.dim, self.weight.dtype):
                return kernels.gemm_chain(xn, self.weight, logits, kernels.EPI_STORE_F32, scale_from=(ss, eps))
            return self._gemm(ctx, xn, self.weight, logits, kernels.EPI_STORE_F32, scale_from=(ss, eps))
        nw, eps = norm.fused()
        return kernels.gemm_norm(x, nw, eps, self.weight, logits, kernels.EPI_STORE_F32)

    def forward(self, h, logits, ctx):
        return self._gemm(ctx, h, self.weight, logits, kernels.EPI_STORE_F32)
