"""The arrangement of a layer's parts.  `prenorm_residual` is the reference's
(src/infer.cpp:256-386): x += mixer(norm(x)); x += feed_forward(norm(x)), the
residual stream in float32 and no scaling of the residual adds.  next_norm is the
norm that reads the residual stream after this layer (the next layer's, or the final
one): a part that can prepares that norm's activations on the way."""
from .base import Part, build_part, part


@part("block", "prenorm_residual")
class PreNormResidualBlock(Part):
    def __init__(self, layer_spec, dim, prefix=""):
        super().__init__(None, dim, layer_spec.prefix)
        p = layer_spec.prefix
        self.mixer_norm = build_part("norm", layer_spec.mixer_norm, dim, p)
        self.mixer = build_part("mixer", layer_spec.mixer, dim, p)
        self.feed_forward = self.feed_forward_norm = None             # a layer may have no feed-forward
        if layer_spec.part("feed_forward") is not None:
            self.feed_forward_norm = build_part("norm", layer_spec.feed_forward_norm, dim, p)
            self.feed_forward = build_part("feed_forward", layer_spec.feed_forward, dim, p)
        # optional member mixer_input: a filter between the first norm and the mixer (a short convolution over time)
        self.mixer_input = None
        if layer_spec.part("mixer_input") is not None:
            self.mixer_input = build_part("input_filter", layer_spec.mixer_input, dim, p)

    def children(self):
        return [c for c in (self.mixer_norm, self.mixer_input, self.mixer, self.feed_forward_norm, self.feed_forward)
                if c is not None]

    def cache_request(self):
        """What the layer keeps for a sequence: the mixer's, and beside it what the filter in front of the mixer keeps."""
        if self.mixer_input is None:
            return self.mixer.cache_request()
        return {"mixer": self.mixer.cache_request(), "input": self.mixer_input.cache_request()}

    def first_norm(self):
        """The norm that reads the residual stream first when this layer runs (the layer before
        may prepare its activations), or None."""
        return self.mixer_norm

    def forward(self, x, ctx, line, writes_cache=True, next_norm=None):
        plain_end = False                 # whether the layer's last sublayer ran behind a norm kernel of its own
        if self.mixer_input is not None:
            left = ctx.normed.pop(id(self.mixer_norm), None)
            if left is not None and left[1] is None:      # the layer before has left this norm's output
                h = left[0]
            else:
                h = ctx.ws.get("block.h", (x.shape[0], self.dim), ctx.act_dtype)
                self.mixer_norm.forward(x, h, ctx)
            filtered = ctx.ws.get("block.filtered", (x.shape[0], self.dim), ctx.act_dtype)
            self.mixer_input.forward(h, filtered, ctx, (line, "input"))
            self.mixer.forward(filtered, x, ctx, (line, "mixer"), writes_cache)
            plain_end = self.feed_forward is None
        elif self.mixer.fuses_norm(self.mixer_norm, x, ctx):
            self.mixer.forward_prenorm(x, self.mixer_norm, ctx, line, writes_cache,
                                       emit_for=self.feed_forward_norm if self.feed_forward is not None else next_norm)
        else:
            left = ctx.normed.pop(id(self.mixer_norm), None)
            if left is not None and left[1] is None:      # the layer before has left this norm's output
                h = left[0]
            else:
                h = ctx.ws.get("block.h", (x.shape[0], self.dim), ctx.act_dtype)
                self.mixer_norm.forward(x, h, ctx)
            self.mixer.forward(h, x, ctx, line, writes_cache)
            plain_end = self.feed_forward is None
        if self.feed_forward is not None:
            if self.feed_forward.fuses_norm(self.feed_forward_norm, x, ctx):
                self.feed_forward.forward_prenorm(x, self.feed_forward_norm, ctx, emit_for=next_norm)
            else:
                h = ctx.ws.get("block.h", (x.shape[0], self.dim), ctx.act_dtype)
                self.feed_forward_norm.forward(x, h, ctx)
                self.feed_forward.forward(h, x, ctx)
                plain_end = True
        # sublayers that fold no norm into their products leave nothing for whoever reads the stream next: in a decode
        # step the layer then ends with that norm as a kernel of its own, so that the head's product (or the next
        # layer's first) takes its output as it is instead of norming the rows again for every tile of its weights
        if plain_end and ctx.mode == "decode" and next_norm is not None and hasattr(next_norm, "fused") \
                and id(next_norm) not in ctx.normed:
            ahead = ctx.ws.get("block.ahead", (x.shape[0], self.dim), ctx.act_dtype)
            next_norm.forward(x, ahead, ctx)
            ctx.normed[id(next_norm)] = (ahead, None, None)


@part("block", "parallel_residual")
class ParallelResidualBlock(Part):
    """x += mixer(h) + feed_forward(h) with h = norm(x): one norm, and both sublayers read its output.  Members: norm,
    mixer, and optionally feed_forward.  Each sublayer adds its result to the float32 stream in the epilogue of its
    last product, the mixer first.  In a decode step the layer ends with the norm that reads the stream next (the next
    layer's, or the final one, whose output the head's product then takes as it is)."""

    def __init__(self, layer_spec, dim, prefix=""):
        super().__init__(None, dim, layer_spec.prefix)
        p = layer_spec.prefix
        self.norm = build_part("norm", layer_spec.norm, dim, p)
        self.mixer = build_part("mixer", layer_spec.mixer, dim, p)
        self.feed_forward = None
        if layer_spec.part("feed_forward") is not None:
            self.feed_forward = build_part("feed_forward", layer_spec.feed_forward, dim, p)

    def children(self):
        return [c for c in (self.norm, self.mixer, self.feed_forward) if c is not None]

    def first_norm(self):
        return self.norm

    def forward(self, x, ctx, line, writes_cache=True, next_norm=None):
        left = ctx.normed.pop(id(self.norm), None)
        if left is not None and left[1] is None:          # the layer before has left this norm's output
            h = left[0]
        else:
            h = ctx.ws.get("block.h", (x.shape[0], self.dim), ctx.act_dtype)
            self.norm.forward(x, h, ctx)
        self.mixer.forward(h, x, ctx, line, writes_cache)
        if self.feed_forward is not None:
            self.feed_forward.forward(h, x, ctx)
        if ctx.mode == "decode" and next_norm is not None and hasattr(next_norm, "fused"):
            other = "block.h" if h.data_ptr() != ctx.ws.get("block.h", (x.shape[0], self.dim), ctx.act_dtype).data_ptr() else "block.h2"
            ahead = ctx.ws.get(other, (x.shape[0], self.dim), ctx.act_dtype)      # not the buffer this layer has just read
            next_norm.forward(x, ahead, ctx)
            ctx.normed[id(next_norm)] = (ahead, None, None)


class StreamInput:
    """What `first_norm()` of a block that reads the residual stream itself hands to the layer before it: the
    place under which that layer may leave the stream in the compute dtype (ctx.normed[id(...)] = (h, None,
    None)), so that no kernel runs only to convert it."""


@part("block", "postnorm_residual")
class PostNormResidualBlock(Part):
    """x += norm(mixer(x)); x += norm(feed_forward(x)): the sublayers read the residual stream itself and
    the norms act on their OUTPUTS.  Members: mixer, mixer_norm, and optionally feed_forward with
    feed_forward_norm (a layer may have no feed-forward).  The sublayers offer forward_to(h, y, ...),
    which writes their result to y instead of adding it to the stream; the norm's add_normed(y, x, h_out)
    adds it normed and hands the new stream on in the compute dtype.  With float32 as the compute dtype the
    sublayers read the stream's own memory."""

    def __init__(self, layer_spec, dim, prefix=""):
        super().__init__(None, dim, layer_spec.prefix)
        p = layer_spec.prefix
        self.mixer = build_part("mixer", layer_spec.mixer, dim, p)
        self.mixer_norm = build_part("norm", layer_spec.mixer_norm, dim, p)
        self.feed_forward = self.feed_forward_norm = None
        if layer_spec.part("feed_forward") is not None:
            self.feed_forward = build_part("feed_forward", layer_spec.feed_forward, dim, p)
            self.feed_forward_norm = build_part("norm", layer_spec.feed_forward_norm, dim, p)
        self.entry = StreamInput()

    def children(self):
        return [c for c in (self.mixer, self.mixer_norm, self.feed_forward, self.feed_forward_norm) if c is not None]

    def first_norm(self):
        return self.entry

    def forward(self, x, ctx, line, writes_cache=True, next_norm=None):
        import torch
        from ..ops import kernels
        T = x.shape[0]
        same = ctx.act_dtype == torch.float32          # the sublayers read x itself
        left = ctx.normed.pop(id(self.entry), None)
        if same:
            h = x
        elif left is not None:
            h = left[0]
        else:
            h = kernels.cast(x, ctx.ws.get("block.h", (T, self.dim), ctx.act_dtype))
        hand_on = None if same or not isinstance(next_norm, StreamInput) else ctx.ws.get("block.h", (T, self.dim), ctx.act_dtype)
        # the last layer of a decode step leaves the final norm's output for the head
        final = next_norm if ctx.mode == "decode" and hasattr(next_norm, "fused") else None
        if final is not None:
            hand_on = ctx.ws.get("block.normed", (T, self.dim), ctx.act_dtype)
        y = ctx.ws.get("block.y", (T, self.dim), torch.float32)
        self.mixer.forward_to(h, y, ctx, line, writes_cache)
        if self.feed_forward is None:
            self.mixer_norm.add_normed(y, x, ctx, h_out=hand_on, next_norm=final)
        else:
            h = x if same else ctx.ws.get("block.h", (T, self.dim), ctx.act_dtype)
            self.mixer_norm.add_normed(y, x, ctx, h_out=None if same else h)
            self.feed_forward.forward_to(h, y, ctx)
            self.feed_forward_norm.add_normed(y, x, ctx, h_out=hand_on, next_norm=final)
        if hand_on is not None:
            ctx.normed[id(next_norm)] = (hand_on, None, None)


@part("block", "loop_entry")
class LoopEntryBlock(Part):
    """The way into a walk of looped layers: x <- W [x; x0] + start, x0 being what the embedding left (it keeps a copy
    when its `keep_output` is set) and `start` row `walk` of a table [walks, dim].  No mixer and no cache line; the
    product reads both streams rounded to the compute dtype and adds to the float32 stream, which the packing kernel
    has set to `start`.  Parameters: `walk`, `walks`, `matrix` and `starts` (tensor names)."""

    def __init__(self, layer_spec, dim, prefix=""):
        super().__init__(None, dim, layer_spec.prefix)
        p = layer_spec.entry.params
        self.walk, self.walks = int(p["walk"]), int(p["walks"])
        if not 0 <= self.walk < self.walks:
            raise ValueError("walk %d of %d" % (self.walk, self.walks))
        self.matrix = self.prefix + str(p.get("matrix", "in"))
        self.starts = self.prefix + str(p.get("starts", "step"))
        self.w = self.start = None

    def param_specs(self):
        from ..weights.loader import ParamSpec
        return [ParamSpec(self.matrix, (self.dim, 2 * self.dim), fan_in=2 * self.dim),
                ParamSpec(self.starts, (self.walks, self.dim), init="bias")]

    def load(self, get, compute_dtype, device):
        import torch
        from ..weights.loader import place
        self.w = place(get(self.matrix), compute_dtype, device)
        self.start = get(self.starts).to(torch.float32)[self.walk].to(device).contiguous()

    def weight_bytes(self):
        return self.w.numel() * self.w.element_size()

    def first_norm(self):
        return None

    def forward(self, x, ctx, line, writes_cache=True, next_norm=None):
        import torch
        from ..ops import kernels
        T = x.shape[0]
        x0 = ctx.ws.get("embed.kept", (T, self.dim), torch.float32)
        both = ctx.ws.get("loop.both", (T, 2 * self.dim), ctx.act_dtype)
        kernels.loop_pack(x, x0, self.start, both)
        self._gemm(ctx, both, self.w, x, kernels.EPI_ADD_F32)
