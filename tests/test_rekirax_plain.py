"""The Rekirax design without a GPU: its configuration reader, the order in which its layers run, the tensors it
declares, the cache lines its layers ask for, and the plain implementation against itself (whole prompt against pieces
and token by token through its memory, the recurrence against its unrolled sum, the convolution's carried inputs, the
edges of a window and of a chunk, the rotation's pairs, the distance term)."""
import copy
import math

import pytest
import torch

import rekirax_configs as KC
from plain import rekirax_plain as P

F64 = torch.float64


def random_weights(cfg, seed=0):
    from yalm_amd.config import config_from_dict
    from yalm_amd.engine.model import param_specs_of
    from yalm_amd.weights import random_init
    specs = param_specs_of(config_from_dict(cfg).to_spec())
    return {s.name: random_init.random_values(s.name, s.shape, s.init, s.fan_in, seed).to(F64) for s in specs}


def test_configuration_round_trip():
    from yalm_amd.config import RekiraxConfig, config_from_dict
    cfg = config_from_dict(KC.MIXED)
    assert isinstance(cfg, RekiraxConfig)
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    spec = cfg.to_spec()
    assert [l.block for l in spec.layers] == ["prenorm_residual"] * 5 + ["loop_entry"] * 3
    assert [l.mixer.kind for l in spec.layers[:5]] == ["side_by_side", "shaped_attention", "side_by_side", "shaped_attention", "side_by_side"]
    left, right = spec.layers[0].mixer.params["left"], spec.layers[0].mixer.params["right"]
    assert left.kind == "shaped_attention" and left.params["block"] == 20 and left.params["window"] if "window" in left.params else True
    assert left.params["projection_norm"] and left.params["gate"] and left.params["position"].params["rotary_dim"] == 4
    assert left.params["position"].params["weight_rows"] == "half_split" and left.params["scale"] == 0.3
    assert right.kind == "hgrn2" and (right.params["n_heads"], right.params["key_dim"], right.params["value_dim"]) == (3, 8, 20)
    assert spec.layers[4].mixer.params["left"].params["position"] is None
    w = spec.layers[1].mixer.params
    assert w["window"] == 33 and w["softcap"] == 5.0 and w["head_norm"] and w["values"] == "keys" and w["log_distance"]
    assert spec.layers[1].part("feed_forward") is None and spec.layers[0].feed_forward.params["gated"]
    assert spec.layers[0].feed_forward.params["biases"] and spec.layers[0].feed_forward.params["activation"] == "gelu_tanh"
    assert spec.layers[0].mixer_input.params["taps"] == 3 and spec.layers[0].mixer_norm.params["offset"] == 1.0
    assert spec.embedding.params["norm"].params["tensor"] == "embed.norm" and spec.embedding.params["keep_output"]
    assert spec.head.params["tied"] and spec.final_norm.params["offset"] == 1.0
    assert [l.entry.params["walk"] for l in spec.layers[5:]] == [0, 1, 2]


def test_the_order_of_layers():
    """Layers before the loop once, the looped run `times` times with a way in before each walk, then the rest; every
    run has a cache line of its own."""
    from yalm_amd.config import config_from_dict
    spec = config_from_dict(KC.MIXED).to_spec()
    assert [e.layer for e in spec.schedule] == [0, 5, 1, 2, 3, 6, 1, 2, 3, 7, 1, 2, 3, 4]
    assert [e.cache for e in spec.schedule] == list(range(14)) and all(e.writes_cache for e in spec.schedule)
    assert P.run_order(5, KC.MIXED["loop"]) == [(0, 0), (1, 0), (2, 0), (3, 0), (1, 1), (2, 1), (3, 1), (1, 2), (2, 2), (3, 2), (4, 0)]
    assert [e.layer for e in config_from_dict(KC.WINDOWS).to_spec().schedule] == list(range(6))
    assert [e.layer for e in config_from_dict(KC.ODD).to_spec().schedule] == [0, 1, 3, 2, 4, 2]
    assert [e.layer for e in config_from_dict(KC.CHUNKS).to_spec().schedule] == [5, 0, 1, 2, 3, 4]
    assert not config_from_dict(KC.WINDOWS).to_spec().embedding.params["keep_output"]


def test_declared_tensors():
    from yalm_amd.config import config_from_dict
    from yalm_amd.engine.model import param_specs_of
    shapes = {s.name: tuple(s.shape) for s in param_specs_of(config_from_dict(KC.MIXED).to_spec())}
    assert shapes["embed"] == (173, 72) and shapes["embed.norm"] == (72,) and shapes["final.norm"] == (72,) and "head" not in shapes
    assert shapes["loop.in"] == (72, 144) and shapes["loop.step"] == (3, 72)
    assert shapes["l0.canon1"] == (72, 3) and shapes["l1.canon1"] == (72, 3)
    assert shapes["l0.mix.left.q"] == (48, 72) and shapes["l0.mix.left.k"] == (16, 72) and shapes["l0.mix.left.v"] == (24, 72)
    assert shapes["l0.mix.left.q.norm"] == (48,) and shapes["l0.mix.left.k.norm"] == (16,) and shapes["l0.mix.left.g"] == (72, 72)
    assert shapes["l0.mix.left.o"] == (72, 72) and shapes["l0.mix.left.out"] == (72,) and shapes["l0.mix.right.out"] == (72,)
    assert shapes["l0.mix.right.q"] == (24, 72) and shapes["l0.mix.right.f"] == (24, 72) and shapes["l0.mix.right.f.b"] == (24,)
    assert shapes["l0.mix.right.lower"] == (24,) and shapes["l0.mix.right.v"] == (60, 72) and shapes["l0.mix.right.norm"] == (20,)
    assert shapes["l0.mix.right.o"] == (72, 60)
    assert shapes["l1.mix.q"] == (96, 72) and shapes["l1.mix.k"] == (48, 72) and "l1.mix.v" not in shapes
    assert shapes["l1.mix.q.norm"] == (24,) and shapes["l1.mix.k.norm"] == (24,) and shapes["l1.mix.r1"] == (4,) and shapes["l1.mix.r2"] == (4,)
    assert shapes["l1.mix.o"] == (72, 96) and "l1.mix.g" not in shapes
    assert not any(k.startswith("l1.mlp") or k == "l1.norm2" for k in shapes)
    assert shapes["l0.mlp.gate"] == (88, 72) and shapes["l0.mlp.up.b"] == (88,) and shapes["l0.mlp.down.b"] == (72,)
    plain = {s.name for s in param_specs_of(config_from_dict(KC.PLAIN).to_spec())}
    assert not any("canon" in n or n.startswith("loop.") for n in plain)


def test_cache_lines_of_a_layer_s_members():
    """A layer keeps its convolution's inputs beside what its mixer keeps, and a side-by-side mixer keys and values for
    its left and a state for its right: the cache manager gives each a line of its own."""
    from yalm_amd.cache.manager import CacheManager, KVRequest, StateRequest
    from yalm_amd.config import config_from_dict
    from yalm_amd.engine.model import Model
    model = Model(config_from_dict(KC.MIXED).to_spec())
    req = model.cache_requests()
    assert req[1] is None and req[5] is None                     # the ways into the walks keep nothing
    assert req[0]["input"] == StateRequest((2, 72), torch.float32)
    assert req[0]["mixer"]["left"] == KVRequest(2, 16, 20, 0) and req[0]["mixer"]["right"] == StateRequest((3 * 8 * 20,), torch.float32)
    assert req[2]["mixer"] == KVRequest(2, 32, 33, 0)
    cache = CacheManager(req, 512, 512, torch.float32, "cpu", n_slots=3)
    assert cache.group_of((0, "input")).line_state((0, "input")).shape == (3, 2, 72)
    assert cache.group_of(((0, "mixer"), "right")).line_state(((0, "mixer"), "right")).shape == (3, 480)
    assert cache.group_of(((0, "mixer"), "left")).request.window == 20 and cache.group_of((2, "mixer")).request.window == 33
    # the three walks of layer 1 have three lines
    assert len({cache.group_of((c, "mixer")).line_pages((c, "mixer"))[0].data_ptr() for c in (2, 6, 10)}) == 3
    a = cache.acquire(1)
    cache.group_of((0, "input")).line_state((0, "input"))[a[0]].fill_(3.0)
    cache.release(a)
    assert float(cache.group_of((0, "input")).line_state((0, "input"))[cache.acquire(1)[0]].abs().sum()) == 0.0


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=4), "multiple"),
    (lambda c: c["layers"][1]["mixer"].update(vdim=8), "values"),
    (lambda c: c["layers"][0].update(type="latent_attention"), "not one of"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), "mask"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=3), "rot"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=10), "rot"),
    (lambda c: c["layers"][0]["mixer"].pop("right"), "right"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "kind"),
    (lambda c: c["loop"].update(stop=6), "loop"),
    (lambda c: c["loop"].update(times=0), "loop"),
    (lambda c: c["loop"].update(start=4), "loop"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
])
def test_refused_configurations(change, message):
    from yalm_amd.config import ConfigError, config_from_dict
    cfg = copy.deepcopy(KC.MIXED)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(cfg)


def test_optional_keys_may_be_absent():
    from yalm_amd.config import config_from_dict
    cfg = copy.deepcopy(KC.PLAIN)
    del cfg["layers"][0]["mixer"]["kv_heads"], cfg["layers"][0]["mixer"]["vdim"], cfg["layers"][0]["mixer"]["mask"]
    del cfg["layers"][0]["mixer"]["softcap"], cfg["layers"][1]["mixer"]["left"]["rot"], cfg["layers"][1]["mixer"]["left"]["mask"]
    spec = config_from_dict(cfg).to_spec()
    m = spec.layers[0].mixer.params
    assert m["n_kv_heads"] == 2 and m["value_dim"] == 16 and m["window"] == 0 and not m["softcap"]
    left = spec.layers[1].mixer.params["left"].params
    assert left["position"] is None and left["block"] == 0
    assert spec.layers[0].part("mixer_input") is None and len(spec.layers) == 2


# ------------------------------------------------------------------------------------------ the plain implementation against itself
@pytest.mark.parametrize("name", ["mixed", "odd", "chunks", "windows"])
def test_pieces_and_single_tokens_agree_with_the_whole_prompt(name):
    cfg = KC.ALL[name]
    w = random_weights(cfg, seed=3)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, cfg["vocab"], (45,), generator=g).tolist()
    whole = P.forward(cfg, w, toks)
    for cuts in ([45], [1, 44], [7, 2, 30, 6], [1] * 45):
        mem, rows, at = {}, [], 0
        for n in cuts:
            rows.append(P.forward(cfg, w, toks[at:at + n], memory=mem, start=at))
            at += n
        assert torch.allclose(torch.cat(rows), whole, rtol=1e-9, atol=1e-9), cuts


def test_the_recurrence_is_its_unrolled_sum():
    """S_t = sum_s (prod_{s < u <= t} f_u) (1 - f_s) v_s^T, row by row, and o_t = S_t^T q_t."""
    g = torch.Generator().manual_seed(2)
    T, H, d, dv = 9, 2, 3, 4
    q, v = torch.randn(T, H, d, generator=g, dtype=F64), torch.randn(T, H, dv, generator=g, dtype=F64)
    f = torch.rand(T, H, d, generator=g, dtype=F64)
    o, S = P.hgrn2_recurrence(q, f, v, torch.zeros(H, d, dv, dtype=F64))
    for t in (0, 4, 8):
        want = torch.zeros(H, d, dv, dtype=F64)
        for s in range(t + 1):
            keep = torch.ones(H, d, dtype=F64)
            for u in range(s + 1, t + 1):
                keep = keep * f[u]
            want += (keep * (1 - f[s]))[:, :, None] * v[s][:, None, :]
        assert torch.allclose(torch.einsum("hdv,hd->hv", want, q[t]), o[t], rtol=1e-12, atol=1e-12)
    assert torch.allclose(S, want)
    # a gate at its lower bound 1 forgets nothing and takes nothing in
    w = {"m.lower": torch.ones(6, dtype=F64), "m.f": torch.randn(6, 5, generator=g, dtype=F64), "m.f.b": torch.zeros(6, dtype=F64)}
    assert torch.equal(P.forget_gates(torch.randn(4, 5, generator=g, dtype=F64), w, "m."), torch.ones(4, 6, dtype=F64))


def test_the_convolution_carries_its_inputs():
    g = torch.Generator().manual_seed(3)
    h, taps = torch.randn(12, 5, generator=g, dtype=F64), torch.randn(5, 4, generator=g, dtype=F64)
    whole = P.input_conv(h, taps, {})
    want = h.clone()
    for t in range(12):
        for j in range(4):
            if t - 3 + j >= 0:
                want[t] += taps[:, j] * h[t - 3 + j]
    assert torch.allclose(whole, want, rtol=1e-12, atol=1e-12)
    mem = {}
    pieces = torch.cat([P.input_conv(h[a:b], taps, mem) for a, b in ((0, 1), (1, 3), (3, 4), (4, 12))])
    assert torch.allclose(pieces, whole, rtol=1e-12, atol=1e-12) and torch.equal(mem["conv"], h[9:])


def test_edges_of_windows_and_chunks():
    assert [j for j in range(12) if P.sees_window(10, j, 4)] == [7, 8, 9, 10]
    assert [j for j in range(12) if P.sees_window(2, j, 4)] == [0, 1, 2]
    assert [j for j in range(12) if P.sees_window(5, j, 1)] == [5]
    assert [j for j in range(12) if P.sees_chunk(10, j, 4)] == [8, 9, 10]
    assert [j for j in range(12) if P.sees_chunk(8, j, 4)] == [8]
    assert [j for j in range(12) if P.sees_chunk(7, j, 4)] == [4, 5, 6, 7]


def test_the_rotation_pairs_an_element_with_the_one_half_the_turned_part_on():
    x = torch.arange(1.0, 9.0, dtype=F64).reshape(1, 1, 8)
    y = P.rotate_half(x, [3], 4, 100.0)[0, 0]
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5
    assert math.isclose(y[0], 1 * math.cos(a0) - 3 * math.sin(a0)) and math.isclose(y[2], 3 * math.cos(a0) + 1 * math.sin(a0))
    assert math.isclose(y[1], 2 * math.cos(a1) - 4 * math.sin(a1)) and math.isclose(y[3], 4 * math.cos(a1) + 2 * math.sin(a1))
    assert torch.equal(y[4:], x[0, 0, 4:]) and torch.equal(P.rotate_half(x, [3], 0, 100.0), x)
    # scores of turned queries and keys depend on the distance alone
    g = torch.Generator().manual_seed(4)
    q, k = torch.randn(1, 1, 8, generator=g, dtype=F64), torch.randn(1, 1, 8, generator=g, dtype=F64)
    s = lambda i, j: float((P.rotate_half(q, [i], 6, 50.0) * P.rotate_half(k, [j], 6, 50.0)).sum())
    assert math.isclose(s(9, 4), s(105, 100), rel_tol=1e-9)


def test_the_distance_term_and_the_cap():
    """One head, two keys with equal products: the nearer one weighs (1 + r2 distance)^r1 times the farther one."""
    w = {"a.q": torch.eye(2, dtype=F64), "a.k": torch.zeros(2, 2, dtype=F64), "a.q.norm": torch.ones(2, dtype=F64),
         "a.k.norm": torch.ones(2, dtype=F64), "a.r1": torch.tensor([1.5], dtype=F64), "a.r2": torch.tensor([0.5], dtype=F64),
         "a.o": torch.eye(2, dtype=F64)}
    mixer = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 1.0, "softcap": 3.0, "mask": {"size": 3}}
    mem = {"k": torch.zeros(3, 1, 2, dtype=F64), "v": torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]], [[5.0, 5.0]]], dtype=F64)}
    out = P.window_attention(torch.ones(1, 2, dtype=F64), [3], mixer, w, "a.", 1e-6, mem)[0]
    # position 3 sees 1, 2, 3 (not 0); its own key and value are zeros
    w1, w2, w3 = (1 + 0.5 * 2) ** -1.5, (1 + 0.5 * 1) ** -1.5, 1.0
    assert torch.allclose(out, torch.tensor([0.0 * w1 + 5 * w2, 1 * w1 + 5 * w2], dtype=F64) / (w1 + w2 + w3), rtol=1e-12)
    cap = lambda s: 3.0 * math.tanh(s / 3.0)
    assert cap(100.0) < 3.0 + 1e-12 and math.isclose(cap(0.01), 0.01, rel_tol=1e-4)
