"""Typed configuration of the Rekirax design: a decoder whose token embedding is normed at once and whose layers are
listed one by one in config.json, each pre-norm (x += mixer(c(norm1(x))); x += ff(norm2(x))), c being a short causal
convolution over time that is added to its own input.  A run of layers may be walked several times with the same
weights; every walk has memories of its own and is entered through x <- W_in [x; x0] + step[walk], x0 the embedding's
output.  The head is the embedding table.

config.json: `architecture` "Rekirax", `vocab`, `width`, `norm.eps`, `canon.taps` (absent: no convolution),
`loop` {start, stop, times} (absent: every layer once), and `layers`, a list of
  {"type": "attention", "mixer": {heads, kv_heads, dim, vdim, scale, softcap?, mask?: {size}}, "mlp": null | {"kind": "dense", "ff": n}}
  {"type": "parallel", "mixer": {"left": {heads, kv_heads, dim, vdim, scale, mask?: {size}, rot?: {dims, base}},
                                 "right": {heads, dim, vdim}}, "mlp": ...}.
Tensors: `embed`, `embed.norm`, `final.norm`, `loop.in` [width, 2 width], `loop.step` [times, width], and for layer i
`l<i>.norm1`, `l<i>.norm2`, `l<i>.canon1` [width, taps];
  attention: `l<i>.mix.{q,k,o}`, `l<i>.mix.{q,k}.norm` [dim], `l<i>.mix.{r1,r2}` [heads];
  parallel: `l<i>.mix.left.{q,k,v,g,o}`, `l<i>.mix.left.{q,k}.norm` (whole projections), `l<i>.mix.right.{q,f,f.b,lower,v,norm,o}`,
  `l<i>.mix.{left,right}.out` [width];
  feed-forward: `l<i>.mlp.{gate,up,down}` and their biases `.b`.

What the design fixes and this file therefore states: the `attention` mixer has no value projection (its values are the
keys before their norm), norms a head, a cap on the scores and r1 ln(1 + r2 distance) taken off them, and sees a sliding
window of mask.size positions; the left half of `parallel` norms whole projections, turns the first rot.dims elements
of each head (element i with element i + dims/2), sees only its own chunk of mask.size positions and gates its heads
with a sigmoid; the right half is HGRN2; the two halves are normed over the width and averaged; the norms' stored
weights are distances from one, the halves' and the heads' norms plain; the feed-forward is gated with the tanh gelu
and every product of it has a bias."""
import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .llama import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

MIXERS = ("attention", "parallel")
NORM_OFFSET = 1.0                # a layer norm's weight is this plus what is stored
HALVES_WEIGHT = 0.5              # of the sum of the two sides of a parallel mixer
POSITIONS = 1 << 18              # the design names no longest sequence: the cache bounds it (and this, where nothing else does)


def _need(d, key, where):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError("config.json lacks the key %r in %s" % (key, where))
    return d[key]


def _heads(m, where, kv=True):
    heads = int(_need(m, "heads", where))
    out = {"heads": heads}
    if kv:
        out["kv_heads"] = int(m.get("kv_heads") or heads)
    out["dim"] = int(_need(m, "dim", where))
    out["vdim"] = int(m.get("vdim") or out["dim"])
    return out


@dataclass(frozen=True)
class RekiraxConfig:
    vocab: int
    width: int
    eps: float
    taps: int = 0                                    # of the convolution in front of every mixer (0: none)
    loop: Optional[Dict[str, int]] = None            # {start, stop, times}
    layers: List[Dict[str, Any]] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    eos_token_ids: List[int] = field(default_factory=list)

    ARCHITECTURES = ("Rekirax",)
    architecture = "Rekirax"

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
        loop = None
        if d.get("loop"):
            lp = d["loop"]
            loop = {k: int(_need(lp, k, "loop")) for k in ("start", "stop", "times")}
        cfg = cls(vocab=int(_need(d, "vocab", "config.json")), width=int(_need(d, "width", "config.json")),
                  eps=float(_need(_need(d, "norm", "config.json"), "eps", "norm")),
                  taps=int(_need(d["canon"], "taps", "canon")) if d.get("canon") else 0, loop=loop,
                  layers=[cls._layer(i, l) for i, l in enumerate(layers)],
                  bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]), eos_token_ids=eos_ids)
        cfg.validate()
        return cfg

    @staticmethod
    def _attention(m, where, rotary):
        out = _heads(m, where)
        out["scale"] = float(_need(m, "scale", where))
        if m.get("softcap"):
            out["softcap"] = float(m["softcap"])
        if m.get("mask"):
            out["mask"] = {"size": int(_need(m["mask"], "size", where + ".mask"))}
        if rotary and m.get("rot"):
            out["rot"] = {"dims": int(_need(m["rot"], "dims", where + ".rot")), "base": float(_need(m["rot"], "base", where + ".rot"))}
        return out

    @classmethod
    def _layer(cls, i, l):
        where = "layer %d" % i
        kind = _need(l, "type", where)
        if kind not in MIXERS:
            raise ConfigError("%s: mixer type %r is not one of %s" % (where, kind, list(MIXERS)))
        m = _need(l, "mixer", where)
        if kind == "attention":
            mixer = cls._attention(m, where, rotary=False)
        else:
            mixer = {"left": cls._attention(_need(m, "left", where), where + ".left", rotary=True),
                     "right": _heads(_need(m, "right", where), where + ".right", kv=False)}
        mlp = l.get("mlp")
        if mlp is not None:
            k = _need(mlp, "kind", where + ".mlp")
            if k != "dense":
                raise ConfigError("%s: feed-forward kind %r is not 'dense'" % (where, k))
            mlp = {"kind": "dense", "ff": int(_need(mlp, "ff", where + ".mlp"))}
        return {"type": kind, "mixer": mixer, "mlp": mlp}

    def validate(self):
        if self.vocab <= 0 or self.width <= 0 or not self.eps > 0 or self.taps < 0:
            raise ConfigError("vocab, width and norm.eps must be positive, canon.taps not negative")
        if self.loop is not None:
            lp = self.loop
            if not (0 <= lp["start"] < lp["stop"] <= len(self.layers)) or lp["times"] < 1:
                raise ConfigError("loop: layers %d..%d of %d, %d times, is no run of layers"
                                  % (lp["start"], lp["stop"] - 1, len(self.layers), lp["times"]))
        for i, l in enumerate(self.layers):
            where = "layer %d" % i
            sides = [(where, l["mixer"])] if l["type"] == "attention" else \
                [(where + ".left", l["mixer"]["left"]), (where + ".right", l["mixer"]["right"])]
            for w, m in sides:
                for k in ("heads", "kv_heads", "dim", "vdim"):
                    if k in m and m[k] <= 0:
                        raise ConfigError("%s: %s must be positive" % (w, k))
                if "kv_heads" in m and m["heads"] % m["kv_heads"]:
                    raise ConfigError("%s: heads %d is no multiple of kv_heads %d" % (w, m["heads"], m["kv_heads"]))
                if m.get("mask") and m["mask"]["size"] <= 0:
                    raise ConfigError("%s: mask.size must be positive" % w)
                if m.get("rot") and (m["rot"]["dims"] < 0 or m["rot"]["dims"] % 2 or m["rot"]["dims"] > m["dim"] or not m["rot"]["base"] > 0):
                    raise ConfigError("%s: rot.dims must be even and at most dim, rot.base positive" % w)
                if m.get("softcap", 1.0) <= 0:
                    raise ConfigError("%s: softcap must be positive" % w)
            if l["type"] == "attention" and l["mixer"]["vdim"] != l["mixer"]["dim"]:
                raise ConfigError("%s: the values of this mixer are its keys, so vdim is dim (%d, not %d)"
                                  % (where, l["mixer"]["dim"], l["mixer"]["vdim"]))
            if l["mlp"] and l["mlp"]["ff"] <= 0:
                raise ConfigError("%s: ff must be positive" % where)

    # ------------------------------------------------------------------ writing
    def to_dict(self):
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "layers": copy.deepcopy(self.layers)}
        if self.taps:
            d["canon"] = {"taps": self.taps}
        if self.loop is not None:
            d["loop"] = dict(self.loop)
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    # ------------------------------------------------------------------ the model as data
    def run_order(self):
        """[(layer, walk)] in the order in which the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, 0) for i in range(n)]
        lp = self.loop
        order = [(i, 0) for i in range(lp["start"])]
        for t in range(lp["times"]):
            order += [(i, t) for i in range(lp["start"], lp["stop"])]
        return order + [(i, 0) for i in range(lp["stop"], n)]

    def _window_attention(self, m):
        return PartSpec("shaped_attention", {
            "n_heads": m["heads"], "n_kv_heads": m["kv_heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
            "scale": m["scale"], "softcap": m.get("softcap", 0.0), "window": m["mask"]["size"] if m.get("mask") else 0,
            "head_norm": True, "values": "keys", "log_distance": True, "eps": self.eps,
            "tensors": {"q": "q", "k": "k", "out": "o", "q_norm": "q.norm", "k_norm": "k.norm", "log_a": "r1", "log_b": "r2"}},
            prefix="mix.")

    def _side_by_side(self, m):
        left, right = m["left"], m["right"]
        position = None
        if left.get("rot") and left["rot"]["dims"]:
            position = PartSpec("rope", {"head_dim": left["dim"], "rotary_dim": left["rot"]["dims"], "theta": left["rot"]["base"],
                                         "weight_rows": "half_split"})
        attention = PartSpec("shaped_attention", {
            "n_heads": left["heads"], "n_kv_heads": left["kv_heads"], "key_dim": left["dim"], "value_dim": left["vdim"],
            "scale": left["scale"], "softcap": left.get("softcap", 0.0), "block": left["mask"]["size"] if left.get("mask") else 0,
            "projection_norm": True, "gate": True, "eps": self.eps, "position": position,
            "tensors": {"q": "q", "k": "k", "v": "v", "out": "o", "q_norm": "q.norm", "k_norm": "k.norm", "gate": "g"}},
            prefix="left.")
        recurrence = PartSpec("hgrn2", {"n_heads": right["heads"], "key_dim": right["dim"], "value_dim": right["vdim"], "eps": self.eps},
                              prefix="right.")
        return PartSpec("side_by_side", {"left": attention, "right": recurrence, "eps": self.eps, "weight": HALVES_WEIGHT,
                                         "tensors": {"left_norm": "left.out", "right_norm": "right.out"}}, prefix="mix.")

    def to_spec(self):
        norm = {"eps": self.eps, "offset": NORM_OFFSET}
        layers = []
        for i, l in enumerate(self.layers):
            mixer = self._window_attention(l["mixer"]) if l["type"] == "attention" else self._side_by_side(l["mixer"])
            members = {"mixer": mixer, "mixer_norm": PartSpec("rmsnorm", dict(norm, tensor="norm1"))}
            if self.taps:
                members["mixer_input"] = PartSpec("time_conv", {"taps": self.taps, "residual": True, "tensor": "canon1"})
            if l["mlp"] is not None:
                members["feed_forward_norm"] = PartSpec("rmsnorm", dict(norm, tensor="norm2"))
                members["feed_forward"] = PartSpec("dense_mlp", {
                    "hidden": l["mlp"]["ff"], "activation": "gelu_tanh", "gated": True, "biases": True,
                    "tensors": {"gate": "gate", "up": "up", "down": "down"}}, prefix="mlp.")
            layers.append(LayerSpec("prenorm_residual", parts=members, prefix="l%d." % i))
        n = len(layers)
        schedule = []
        if self.loop is not None:        # the ways into the walks: layers of their own, without mixer and cache line
            for t in range(self.loop["times"]):
                layers.append(LayerSpec("loop_entry", prefix="loop.", entry=PartSpec("loop_entry", {
                    "walk": t, "walks": self.loop["times"], "matrix": "in", "starts": "step"})))
        for i, t in self.run_order():
            if self.loop is not None and i == self.loop["start"]:
                schedule.append(ScheduleEntry(layer=n + t, cache=len(schedule)))
            schedule.append(ScheduleEntry(layer=i, cache=len(schedule)))
        return ModelSpec(
            architecture=self.architecture, dim=self.width, vocab_size=self.vocab, max_positions=POSITIONS,
            embedding=PartSpec("token_embedding", {"vocab_size": self.vocab, "tensor": "embed",
                                                   "norm": PartSpec("rmsnorm", dict(norm, tensor="embed.norm")),
                                                   "keep_output": self.loop is not None}),
            layers=layers, final_norm=PartSpec("rmsnorm", dict(norm, tensor="final.norm")),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "tied": True}), schedule=schedule,
            bos_token_id=self.bos_token_id, eos_token_ids=list(self.eos_token_ids))
