"""Grouped-query attention whose scores are shaped: every piece is a parameter and may be left out.

Per token: q, k, v = W h (+ biases); RMS norms over the WHOLE query and key projections (all heads at once, plain
weights; `projection_norm`); the query times 1 + coef ln(floor((p + 1) / every) + 1) at position p (`q_temp`);
score = (q . k) * scale, capped as cap tanh(score / cap) (`softcap`), plus the position part's term by the
distance (a slope a head); a window, and/or `block`: a query sees the keys of its own block of that many positions
only, blocks counted from position 0 of the sequence (the cache then keeps a ring of a block's pages, as for a window
of that width); a softmax whose denominator also holds exp(sink_h), a learned logit a head
without key or value (`sink_logit`); the values of a layer with `value_blend` "later" are (1 - lam) v + lam v_first,
v_first being the values that the layer with "first" made for the same token (lam a tensor), and the blended
values are what the cache keeps.  Key and value heads may differ in size.

Further pieces: `head_norm`, RMS norms over each query and key head instead (weights of key_dim elements shared by the
heads); `values` "keys": no value projection, a head's values are its keys as projected, before their norm; a `position`
that is a rotation (kind "rope": behind the norms, the first rotary_dim elements of every query and key head are
turned; the projections' rows and the norms' weights are brought into the kernel's order of pairs at load);
`log_distance`: two numbers a head (tensors), a and b, take a ln(1 + b (i - j)) off the score of query i and key j,
behind the cap; `gate`: the heads' results are multiplied by sigmoid(W_g h) before the output projection.
forward_to writes the mixer's result instead of adding it to the stream.

The cache and the attention kernels are the library's grouped-query ones: a head is stored `pad` elements wide
(the larger of key and value size, rounded up to 16, zeros behind), the output projection's columns are spread
to that width at load, and scale * sqrt(pad) rides on the query, since the kernels divide by sqrt(pad)."""
import math

import torch

from ..cache.manager import KVRequest
from ..ops import kernels
from ..weights.loader import ParamSpec, place
from .attention import decode_splits, kv_tiles
from .base import Part, build_part, part

# A prompt step of at least this many tokens leaves its values row by row and transposes them a tile of 64 tokens at a
# time (whole lines into the staging tiles and pages instead of two bytes a token and element)
V_TILES_MIN_TOKENS = 64

NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "out": "o_proj.weight",
         "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "q_norm": "q_norm.weight",
         "k_norm": "k_norm.weight", "sink": "sink", "blend": "value_blend", "gate": "g_proj.weight", "log_a": "log_a",
         "log_b": "log_b"}


@part("mixer", "shaped_attention")
class ShapedAttention(Part):
    prompt_tables = (kv_tiles,)

    def __init__(self, spec, dim, prefix):
        super().__init__(spec, dim, prefix)
        p = spec.params
        self.n_heads = int(p["n_heads"])
        self.n_kv_heads = int(p.get("n_kv_heads") or self.n_heads)
        self.key_dim = int(p["key_dim"])
        self.value_dim = int(p.get("value_dim") or self.key_dim)
        self.scale = float(p.get("scale") or self.key_dim ** -0.5)
        self.softcap = float(p.get("softcap") or 0.0)
        self.window = int(p.get("window", 0) or 0)
        self.block = int(p.get("block", 0) or 0)
        if self.window < 0 or self.block < 0:
            raise ValueError("a window and a block of positions are positive (0: none)")
        self.q_temp = tuple(p["q_temp"]) if p.get("q_temp") else None
        self.projection_norm = bool(p.get("projection_norm", False))
        self.head_norm = bool(p.get("head_norm", False))
        self.values_from_keys = p.get("values", "own") == "keys"
        if p.get("values", "own") not in ("own", "keys"):
            raise ValueError("values %r are neither 'own' nor 'keys'" % (p.get("values"),))
        self.has_gate = bool(p.get("gate", False))
        self.has_log_distance = bool(p.get("log_distance", False))
        self.eps = float(p.get("eps", 1e-6))
        self.biases = bool(p.get("biases", False))
        self.has_sink = bool(p.get("sink_logit", False))
        self.value_blend = p.get("value_blend")
        self.blend_name = str(p.get("blend_name", "blend"))
        if self.value_blend not in (None, "first", "later"):
            raise ValueError("value_blend %r is not None, 'first' or 'later'" % (self.value_blend,))
        if self.n_heads % self.n_kv_heads:
            raise ValueError("n_heads %d is no multiple of n_kv_heads %d" % (self.n_heads, self.n_kv_heads))
        if self.projection_norm and self.head_norm:
            raise ValueError("norms over the whole projections and norms a head do not go together")
        if self.values_from_keys and (self.value_dim != self.key_dim or self.value_blend is not None):
            raise ValueError("values that are the keys are as wide as the keys (%d, not %d) and are not blended"
                             % (self.key_dim, self.value_dim))
        self.pad = (max(self.key_dim, self.value_dim) + 15) // 16 * 16
        if self.pad > kernels.MAX_HEAD_DIM:
            raise ValueError("heads of %d are not supported (at most %d)" % (self.pad, kernels.MAX_HEAD_DIM))
        self.q_dim, self.k_dim, self.v_dim = self.n_heads * self.key_dim, self.n_kv_heads * self.key_dim, self.n_kv_heads * self.value_dim
        self.n_proj = self.q_dim + self.k_dim + (0 if self.values_from_keys else self.v_dim)      # a token's row of the first product
        if (self.q_dim + self.k_dim + self.v_dim) * 4 > 64 * 1024:
            raise ValueError("a token's queries, keys and values (%d numbers) are more than the packing kernel holds"
                             % (self.q_dim + self.k_dim + self.v_dim))
        self.names = dict(NAMES)
        self.names.update(p.get("tensors") or {})
        self.position = build_part("position", p["position"], dim, prefix) if p.get("position") else None
        self.rot_dims = int(getattr(self.position, "rotary_dim", 0) or 0)
        if self.rot_dims > self.key_dim:
            raise ValueError("%d turned elements do not fit key heads of %d" % (self.rot_dims, self.key_dim))
        self.wqkv = self.wo = self.bias = self.w_qn = self.w_kn = self.sink = self.lam = self.wg = self.log_ab = None

    def children(self):
        return [self.position] if self.position is not None else []

    def _n(self, key):
        return self.prefix + self.names[key]

    def param_specs(self):
        D = self.dim
        out = [ParamSpec(self._n("q"), (self.q_dim, D), fan_in=D), ParamSpec(self._n("k"), (self.k_dim, D), fan_in=D),
               ParamSpec(self._n("out"), (D, self.n_heads * self.value_dim), fan_in=self.n_heads * self.value_dim)]
        if not self.values_from_keys:
            out.append(ParamSpec(self._n("v"), (self.v_dim, D), fan_in=D))
        if self.has_gate:
            out.append(ParamSpec(self._n("gate"), (self.n_heads * self.value_dim, D), fan_in=D))
        if self.head_norm:
            out += [ParamSpec(self._n("q_norm"), (self.key_dim,), init="norm"), ParamSpec(self._n("k_norm"), (self.key_dim,), init="norm")]
        if self.has_log_distance:
            out += [ParamSpec(self._n("log_a"), (self.n_heads,), init="fraction"), ParamSpec(self._n("log_b"), (self.n_heads,), init="fraction")]
        if self.biases:
            out += [ParamSpec(self._n("q_bias"), (self.q_dim,), init="bias"), ParamSpec(self._n("k_bias"), (self.k_dim,), init="bias"),
                    ParamSpec(self._n("v_bias"), (self.v_dim,), init="bias")]
        if self.projection_norm:
            out += [ParamSpec(self._n("q_norm"), (self.q_dim,), init="norm"), ParamSpec(self._n("k_norm"), (self.k_dim,), init="norm")]
        if self.has_sink:
            out.append(ParamSpec(self._n("sink"), (self.n_heads,), init="embedding"))
        if self.value_blend is not None:
            # the first blending layer's number is in the folder and is not used
            out.append(ParamSpec(self._n("blend"), (), init="fraction"))
        return out

    def load(self, get, compute_dtype, device):
        def f32(key):
            return get(self._n(key)).to(torch.float32).reshape(-1).to(device).contiguous()
        def paired(t, n_heads):            # rows (or a norm's weights) in the order in which the rotation kernel pairs them
            if not self.rot_dims:
                return t
            flat = t.dim() == 1
            out = self.position.arrange_projection_rows(t.reshape(n_heads * self.key_dim, -1), n_heads)
            return out.reshape(-1) if flat else out
        rows = [paired(get(self._n("q")), self.n_heads), paired(get(self._n("k")), self.n_kv_heads)]
        if not self.values_from_keys:
            rows.append(get(self._n("v")))
        self.wqkv = place(torch.cat(rows, dim=0), compute_dtype, device)
        self.wg = place(get(self._n("gate")), compute_dtype, device) if self.has_gate else None
        wo = get(self._n("out"))
        if self.pad != self.value_dim:                    # the attention's result is `pad` wide a head, zeros behind
            spread = torch.zeros((self.dim, self.n_heads, self.pad), dtype=wo.dtype)
            spread[:, :, :self.value_dim] = wo.reshape(self.dim, self.n_heads, self.value_dim)
            wo = spread.reshape(self.dim, self.n_heads * self.pad)
        self.wo = place(wo, compute_dtype, device)
        self.bias = None
        if self.biases:
            b = [paired(get(self._n("q_bias")).reshape(-1), self.n_heads), paired(get(self._n("k_bias")).reshape(-1), self.n_kv_heads)]
            if not self.values_from_keys:
                b.append(get(self._n("v_bias")).reshape(-1))
            self.bias = torch.cat([t.to(torch.float32) for t in b]).to(device).contiguous()
        self.w_qn = self.w_kn = None
        if self.projection_norm:
            self.w_qn = paired(get(self._n("q_norm")).to(torch.float32).reshape(-1), self.n_heads).to(device).contiguous()
            self.w_kn = paired(get(self._n("k_norm")).to(torch.float32).reshape(-1), self.n_kv_heads).to(device).contiguous()
        elif self.head_norm:
            self.w_qn = paired(get(self._n("q_norm")).to(torch.float32).reshape(-1), 1).to(device).contiguous()
            self.w_kn = paired(get(self._n("k_norm")).to(torch.float32).reshape(-1), 1).to(device).contiguous()
        self.log_ab = (f32("log_a"), f32("log_b")) if self.has_log_distance else None
        self.sink = f32("sink") if self.has_sink else None
        self.lam = f32("blend") if self.value_blend == "later" else None

    def weight_bytes(self):
        return (self.wqkv.numel() + self.wo.numel() + (self.wg.numel() if self.wg is not None else 0)) * self.wqkv.element_size()

    def cache_request(self):
        # a query inside a block sees fewer than `block` keys back: the ring of a window of that width holds them
        reach = min(self.window, self.block) if self.window and self.block else (self.window or self.block)
        return KVRequest(self.n_kv_heads, self.pad, reach, 0)

    def row_elements(self):
        return max(self.q_dim + self.k_dim + self.v_dim, self.n_heads * self.pad)

    def describe(self, compute_dtype):
        what = "shaped attention, %d heads in %d groups, keys of %d and values of %d in heads of %d%s" % (
            self.n_heads, self.n_kv_heads, self.key_dim, self.value_dim, self.pad,
            (", window %d" % self.window if self.window else "") + (", blocks of %d" % self.block if self.block else ""))
        if compute_dtype != torch.bfloat16:
            return what + ": float32-arithmetic kernels", False
        if self.pad in kernels.MFMA_HEAD_DIMS:
            return what + ": matrix-core kernels", False
        return what + ": float32-arithmetic kernels on bfloat16 storage (the matrix-core kernels take head sizes " \
                      "of 16 to 128 in steps of 16, not %d): correct, several times slower" % self.pad, True

    @property
    def score_bias(self):
        return getattr(self.position, "score_bias", None)

    @property
    def slopes(self):
        return getattr(self.position, "slopes", None)

    def forward(self, h, x, ctx, line, writes_cache=True):
        """Adds the mixer's result to the stream x."""
        return self._run(h, x, ctx, line, writes_cache, kernels.EPI_ADD_F32)

    def forward_to(self, h, y, ctx, line, writes_cache=True):
        """Writes the mixer's result to y (float32 [T, dim])."""
        return self._run(h, y, ctx, line, writes_cache, kernels.EPI_STORE_F32)

    def _run(self, h, x, ctx, line, writes_cache, epilogue):
        T = h.shape[0]
        act, ws = h.dtype, ctx.ws
        H, G, P = self.n_heads, self.n_kv_heads, self.pad
        if self.position is not None and ctx.max_position >= self.position.n_positions:
            raise ValueError("position %d is beyond the %d distances the score table holds"
                             % (ctx.max_position, self.position.n_positions))
        prefill = ctx.mode == "prefill"
        qkv = ws.get("attn.qkv", (T, self.n_proj), torch.float32)
        self._gemm(ctx, h, self.wqkv, qkv, kernels.EPI_STORE_F32)
        q = ws.get("attn.q", (T, H * P), act)
        group = ctx.cache.group_of(line)
        k_pages, v_pages = group.line_pages(line)
        kst = vst = seq_tile0 = None
        if prefill:
            tiles = ctx.tables["kv_tiles"]
            seq_tile0, n_tiles = tiles["seq_tile0"], tiles["n_tiles"]
            kst = ws.get("attn.stage.k", (n_tiles, G, kernels.PAGE, P), act)
            vst = ws.get("attn.stage.v", (n_tiles, G, P, kernels.PAGE), act)
        v_first, blend = None, 0
        if self.value_blend is not None:
            # the first blending layer of a step leaves its values here for the later ones of the same step
            v_first = ws.get("attn.blend." + self.blend_name, (T, self.v_dim), torch.float32)
            blend = 1 if self.value_blend == "first" else 2
        v_rows = None
        if prefill and T >= V_TILES_MIN_TOKENS and kernels.can_v_tiles(P, act):
            v_rows = ws.get("attn.vrows", (T, G * P), act)
        kernels.qkv_pack(qkv, self.bias, self.w_qn, self.w_kn, self.eps, self.q_temp, self.scale * math.sqrt(P), v_first,
                         blend, self.lam, q, kst, vst, seq_tile0, k_pages if writes_cache else None,
                         v_pages if writes_cache else None, group.table, group.ring_pages, ctx.tok_seq, ctx.tok_pos,
                         ctx.seq_slot, ctx.seq_len, H, G, self.key_dim, self.value_dim, P, v_rows=v_rows,
                         head_norm=self.head_norm, v_from_k=self.values_from_keys,
                         cos_sin=self.position.table if self.rot_dims else None, rot_dims=self.rot_dims)
        if v_rows is not None:
            kernels.v_tiles(v_rows, vst, v_pages if writes_cache else None, ctx.cu_seqlens, seq_tile0, group.table,
                            group.ring_pages, ctx.seq_slot, ctx.seq_len, G, P)
        o = ws.get("attn.o", (T, H * P), act)
        if prefill:
            kernels.attn_prefill(q, kst, vst, o, ctx.cu_seqlens, seq_tile0, ctx.tok_seq, ctx.tok_pos, H, G, P, self.window,
                                 tiles.get("tile_order"), score_bias=self.score_bias, softcap=self.softcap,
                                 sink_logit=self.sink, slopes=self.slopes, block=self.block, log_distance=self.log_ab)
        else:
            n_splits = decode_splits(H, G, P, T, min(group.ring_pages, ctx.pages_bucket), ctx.ragged)
            partial = ws.get("attn.partial", (kernels.attn_decode_workspace_floats(T, H, P, n_splits),), torch.float32)
            kernels.attn_decode(q, k_pages, v_pages, group.table, group.ring_pages, ctx.seq_slot, ctx.seq_len, o, partial,
                                H, G, P, self.window, n_splits, step_max_len=ctx.step_max_len, seq_order=ctx.seq_order,
                                score_bias=self.score_bias, softcap=self.softcap, sink_logit=self.sink, slopes=self.slopes,
                                block=self.block, log_distance=self.log_ab)
        if self.has_gate:
            gates = ws.get("attn.gate", (T, H * self.value_dim), torch.float32)
            self._gemm(ctx, h, self.wg, gates, kernels.EPI_STORE_F32)
            kernels.sigmoid_gate(o, gates, H, self.value_dim, P)
        self._gemm(ctx, o, self.wo, x, epilogue)
