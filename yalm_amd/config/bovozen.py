"""Typed configuration of the Bovozen design: a decoder whose layers are listed one by one in config.json, each
pre-norm (x += mixer(norm1(x)); x += ff(norm2(x))), with an attention without rotation or a gated delta rule as
mixer, and a two-matrix feed-forward or a mixture of experts beside a shared expert (or no feed-forward).  The token
embedding gets a learned position vector; the head is the embedding table.

config.json: `architecture` "Bovozen", `vocab`, `width`, `max_positions`, `norm.eps`, and `layers`, a list of
  {"type": "attention",
   "mixer": {heads, kv_heads, dim, vdim, scale, mask?: {size}, v_mix?: bool},
   "mlp": null | {"kind": "dense", "ff": n}
               | {"kind": "moe", "expert": {ff}, "router": {experts, top}, "shared"?: {ff}}}
  {"type": "channel_delta", "mixer": {heads, kv_heads, dim, vdim, conv, decay_rank?, gate_rank?}, "mlp": ...}.
Tensors: `embed`, `pos`, `final.norm`, and for layer i `l<i>.norm1`, `l<i>.norm2`;
  attention: `l<i>.mix.{q,k,v,o}`, `l<i>.mix.{q,k}.norm`, `l<i>.mix.vmix`;
  channel_delta: `l<i>.mix.{q,k,v}` each with `.conv`, `l<i>.mix.{b,A_log,dt_bias,a1,a2,g1,g2,norm,o}`;
  feed-forward: `l<i>.mlp.{up,down}` or `l<i>.mlp.{router,router.b,e<k>.{gate,up,down},shared.{gate,up,down,sg}}`.
The inner sizes of the two low-rank products of a channel_delta mixer (`a1`/`a2` for the decay, `g1`/`g2` for the output
gate) are the tensors' own: a folder's configuration takes them from the shapes of `a1` and `g1` (`with_tensor_shapes`);
`decay_rank` and `gate_rank` name them where there is no folder yet (random models, and `to_dict` writes them).

What the design fixes and this file therefore states: head h of H has the slope 2^(-8 (h + 1) / H) on the distance of
query and key; a query sees the keys of its own block of `mask.size` positions, blocks counted from position 0; the
norms' stored weights are distances from one; the unit vectors' floor 1e-6 and the delta rule's query scale dim^(-1/2);
the dense feed-forward's activation is the erf gelu; the experts are silu(gate) * up, a token's weights the softmax over
its chosen logits, and the shared expert is gated by a sigmoid of one number a token; among the layers with `v_mix` the
earliest keeps its own values and hands them to the others, which blend theirs with them."""
import copy
from dataclasses import dataclass, field, replace
from typing import Any, Dict, List, Optional

from .llama import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec

MIXERS = ("attention", "channel_delta")
SLOPE_EXPONENT = 8.0             # slope of head h of H: 2^(-SLOPE_EXPONENT (h + 1) / H)
UNIT_FLOOR = 1e-6                # under the root of a unit vector's sum of squares
NORM_OFFSET = 1.0                # a norm's weight is this plus what is stored


def _need(d, key, where):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError("config.json lacks the key %r in %s" % (key, where))
    return d[key]


@dataclass(frozen=True)
class BovozenConfig:
    vocab: int
    width: int
    eps: float
    max_positions: int
    layers: List[Dict[str, Any]] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    eos_token_ids: List[int] = field(default_factory=list)

    ARCHITECTURES = ("Bovozen",)
    architecture = "Bovozen"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d):
        arch = d.get("architecture") or (d.get("architectures") or [None])[0]
        if arch not in cls.ARCHITECTURES:
            raise ConfigError("architecture %r is not one of %s" % (arch, list(cls.ARCHITECTURES)))
        layers = _need(d, "layers", "config.json")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("`layers` must be a list with at least one layer")
        eos = d.get("eos_token_id")
        eos_ids = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, (list, tuple)) else [int(eos)])
        cfg = cls(vocab=int(_need(d, "vocab", "config.json")), width=int(_need(d, "width", "config.json")),
                  eps=float(_need(_need(d, "norm", "config.json"), "eps", "norm")),
                  max_positions=int(_need(d, "max_positions", "config.json")),
                  layers=[cls._layer(i, l) for i, l in enumerate(layers)],
                  bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]), eos_token_ids=eos_ids)
        cfg.validate()
        return cfg

    @staticmethod
    def _layer(i, l):
        where = "layer %d" % i
        kind = _need(l, "type", where)
        if kind not in MIXERS:
            raise ConfigError("%s: mixer type %r is not one of %s" % (where, kind, list(MIXERS)))
        m = _need(l, "mixer", where)
        heads = int(_need(m, "heads", where))
        mixer = {"heads": heads, "kv_heads": int(m.get("kv_heads") or heads), "dim": int(_need(m, "dim", where)),
                 "vdim": int(m.get("vdim") or m["dim"])}
        if kind == "channel_delta":
            mixer["conv"] = int(_need(m, "conv", where))
            for k in ("decay_rank", "gate_rank"):
                if m.get(k) is not None:
                    mixer[k] = int(m[k])
        else:
            mixer["scale"] = float(_need(m, "scale", where))
            if m.get("mask"):
                mixer["mask"] = {"size": int(_need(m["mask"], "size", where + ".mask"))}
            if m.get("v_mix"):
                mixer["v_mix"] = True
        mlp = l.get("mlp")
        if mlp is not None:
            k = _need(mlp, "kind", where + ".mlp")
            if k == "dense":
                mlp = {"kind": "dense", "ff": int(_need(mlp, "ff", where + ".mlp"))}
            elif k == "moe":
                ex, ro = _need(mlp, "expert", where + ".mlp"), _need(mlp, "router", where + ".mlp")
                out = {"kind": "moe", "expert": {"ff": int(_need(ex, "ff", where + ".expert"))},
                       "router": {"experts": int(_need(ro, "experts", where + ".router")),
                                  "top": int(_need(ro, "top", where + ".router"))}}
                if mlp.get("shared"):
                    out["shared"] = {"ff": int(_need(mlp["shared"], "ff", where + ".shared"))}
                mlp = out
            else:
                raise ConfigError("%s: feed-forward kind %r is not 'dense' or 'moe'" % (where, k))
        return {"type": kind, "mixer": mixer, "mlp": mlp}

    def validate(self):
        if self.vocab <= 0 or self.width <= 0 or self.max_positions <= 0 or not self.eps > 0:
            raise ConfigError("vocab, width, max_positions and norm.eps must be positive")
        first_blend = None
        for i, l in enumerate(self.layers):
            m, where = l["mixer"], "layer %d" % i
            for k in ("heads", "kv_heads", "dim", "vdim"):
                if m[k] <= 0:
                    raise ConfigError("%s: %s must be positive" % (where, k))
            if m["heads"] % m["kv_heads"]:
                raise ConfigError("%s: heads %d is no multiple of kv_heads %d" % (where, m["heads"], m["kv_heads"]))
            if l["type"] == "attention":
                if m.get("mask") and m["mask"]["size"] <= 0:
                    raise ConfigError("%s: mask.size must be positive" % where)
                if m.get("v_mix"):
                    mine = (m["kv_heads"], m["vdim"])
                    if first_blend is None:
                        first_blend = mine
                    elif mine != first_blend:
                        raise ConfigError("%s: v_mix blends with the first such layer's values, which are %d heads of "
                                          "%d, not %d of %d" % ((where,) + first_blend + mine))
            else:
                if m["conv"] <= 0:
                    raise ConfigError("%s: conv (the number of taps) must be positive" % where)
                if m.get("decay_rank", 1) <= 0 or m.get("gate_rank", 1) <= 0:
                    raise ConfigError("%s: decay_rank and gate_rank must be positive" % where)
            mlp = l["mlp"]
            if mlp and mlp["kind"] == "dense" and mlp["ff"] <= 0:
                raise ConfigError("%s: ff must be positive" % where)
            if mlp and mlp["kind"] == "moe":
                if mlp["expert"]["ff"] <= 0 or not 0 < mlp["router"]["top"] <= mlp["router"]["experts"]:
                    raise ConfigError("%s: the experts need a positive ff and 0 < top <= experts" % where)
                if mlp.get("shared") and mlp["shared"]["ff"] <= 0:
                    raise ConfigError("%s: the shared expert's ff must be positive" % where)

    def with_tensor_shapes(self, shape_of):
        """The configuration with the sizes that only a folder's tensors give: `shape_of(name)` is a tensor's shape
        or None.  A channel_delta mixer's decay_rank and gate_rank are the rows of its `a1` and `g1`."""
        layers = copy.deepcopy(self.layers)
        for i, l in enumerate(layers):
            if l["type"] != "channel_delta":
                continue
            for key, tensor in (("decay_rank", "a1"), ("gate_rank", "g1")):
                shape = shape_of("l%d.mix.%s" % (i, tensor))
                if shape is not None and len(shape) == 2:
                    l["mixer"][key] = int(shape[0])
        cfg = replace(self, layers=layers)
        cfg.validate()
        return cfg

    # ------------------------------------------------------------------ writing
    def to_dict(self):
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
             "max_positions": self.max_positions, "norm": {"eps": self.eps}, "layers": copy.deepcopy(self.layers)}
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    # ------------------------------------------------------------------ the model as data
    def to_spec(self):
        norm = {"eps": self.eps, "offset": NORM_OFFSET}
        layers = []
        blend_seen = False
        for i, l in enumerate(self.layers):
            m = l["mixer"]
            if l["type"] == "channel_delta":
                for k in ("decay_rank", "gate_rank"):
                    if k not in m:
                        raise ConfigError("layer %d: %s is neither in the configuration nor taken from a folder's tensors"
                                          % (i, k))
                mixer = PartSpec("gated_delta", {
                    "n_heads": m["heads"], "n_qk_heads": m["kv_heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                    "conv_taps": m["conv"], "decay_rank": m["decay_rank"], "gate_rank": m["gate_rank"],
                    "q_scale": m["dim"] ** -0.5, "unit_floor": UNIT_FLOOR, "eps": self.eps,
                    "tensors": {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv",
                                "beta": "b", "decay_log": "A_log", "decay_bias": "dt_bias", "decay_in": "a1",
                                "decay_out": "a2", "gate_in": "g1", "gate_out": "g2", "norm": "norm", "out": "o"}},
                    prefix="mix.")
            else:
                blend = None
                if m.get("v_mix"):
                    blend = "later" if blend_seen else "first"
                    blend_seen = True
                position = PartSpec("distance_slopes", {"n_heads": m["heads"], "exponent": SLOPE_EXPONENT})
                mixer = PartSpec("shaped_attention", {
                    "n_heads": m["heads"], "n_kv_heads": m["kv_heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
                    "scale": m["scale"], "block": m["mask"]["size"] if m.get("mask") else 0, "projection_norm": True,
                    "eps": self.eps, "biases": False, "sink_logit": False, "value_blend": blend, "blend_name": "vmix",
                    "position": position,
                    "tensors": {"q": "q", "k": "k", "v": "v", "out": "o", "q_norm": "q.norm", "k_norm": "k.norm",
                                "blend": "vmix"}}, prefix="mix.")
            members = {"mixer": mixer, "mixer_norm": PartSpec("rmsnorm", dict(norm, tensor="norm1"))}
            mlp = l["mlp"]
            if mlp is not None:
                members["feed_forward_norm"] = PartSpec("rmsnorm", dict(norm, tensor="norm2"))
            if mlp is not None and mlp["kind"] == "dense":
                members["feed_forward"] = PartSpec("dense_mlp", {
                    "hidden": mlp["ff"], "activation": "gelu_erf", "tensors": {"up": "up", "down": "down"}}, prefix="mlp.")
            elif mlp is not None:
                params = {"hidden": mlp["expert"]["ff"], "limit": 0.0, "alpha": 1.0, "up_shift": 0.0,
                          "n_experts": mlp["router"]["experts"], "top": mlp["router"]["top"], "renormalize": "chosen",
                          "expert_prefix": "e%d.", "tensors": {"router_bias": "router.b"}}
                if mlp.get("shared"):
                    params["shared"] = {"hidden": mlp["shared"]["ff"], "prefix": "shared.", "gate": "sg"}
                members["feed_forward"] = PartSpec("moe", params, prefix="mlp.")
            layers.append(LayerSpec("prenorm_residual", parts=members, prefix="l%d." % i))
        return ModelSpec(
            architecture=self.architecture, dim=self.width, vocab_size=self.vocab, max_positions=self.max_positions,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "tensor": "embed", "position_tensor": "pos",
                                                   "n_positions": self.max_positions}),
            layers=layers, final_norm=PartSpec("rmsnorm", dict(norm, tensor="final.norm")),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "tied": True}),
            bos_token_id=self.bos_token_id, eos_token_ids=list(self.eos_token_ids))
