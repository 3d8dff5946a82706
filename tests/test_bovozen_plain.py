"""The Bovozen design without a GPU: its configuration reader, the tensors it declares, and the plain
implementation against itself (whole prompt against pieces and token by token through its memory, the delta rule
against its closed form for orthogonal keys, the convolution's carried inputs, a block's edge, the router)."""
import copy
import json
import math
import os

import pytest
import torch

import bovozen_configs as BC
from plain import bovozen_plain as P

F64 = torch.float64


def random_weights(cfg, seed=0):
    from yalm_amd.config import config_from_dict
    from yalm_amd.engine.model import param_specs_of
    from yalm_amd.weights import random_init
    specs = param_specs_of(config_from_dict(cfg).to_spec())
    return {s.name: random_init.random_values(s.name, s.shape, s.init, s.fan_in, seed).to(F64) for s in specs}


def test_configuration_round_trip():
    from yalm_amd.config import BovozenConfig, config_from_dict
    cfg = config_from_dict(BC.MIXED)
    assert isinstance(cfg, BovozenConfig)
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    spec = cfg.to_spec()
    assert [l.block for l in spec.layers] == ["prenorm_residual"] * 7
    assert [l.mixer.kind for l in spec.layers] == ["gated_delta", "shaped_attention", "shaped_attention", "shaped_attention",
                                                  "gated_delta", "shaped_attention", "shaped_attention"]
    assert [l.mixer.params.get("value_blend") for l in spec.layers] == [None, "first", None, "later", None, None, "later"]
    assert spec.layers[2].part("feed_forward") is None and spec.layers[2].mixer.params["block"] == 0
    assert spec.layers[1].mixer.params["block"] == 20 and spec.layers[1].mixer.params["scale"] == 0.3
    assert spec.layers[0].mixer.params["conv_taps"] == 4 and spec.layers[4].mixer.params["decay_rank"] == 1
    assert spec.layers[0].mixer.params["q_scale"] == 8 ** -0.5 and spec.layers[0].mixer.params["n_qk_heads"] == 2
    assert spec.layers[1].feed_forward.params["renormalize"] == "chosen"
    assert spec.layers[1].feed_forward.params["shared"]["hidden"] == 40 and "shared" not in spec.layers[3].feed_forward.params
    assert spec.layers[0].mixer_norm.params["offset"] == 1.0 and spec.final_norm.params["offset"] == 1.0
    assert spec.head.params["tied"] and spec.embedding.params["n_positions"] == 700


def test_declared_tensors():
    from yalm_amd.config import config_from_dict
    from yalm_amd.engine.model import param_specs_of
    shapes = {s.name: tuple(s.shape) for s in param_specs_of(config_from_dict(BC.MIXED).to_spec())}
    assert shapes["embed"] == (173, 72) and shapes["pos"] == (700, 72) and shapes["final.norm"] == (72,) and "head" not in shapes
    assert shapes["l0.mix.q"] == (16, 72) and shapes["l0.mix.k"] == (16, 72) and shapes["l0.mix.v"] == (48, 72)
    assert shapes["l0.mix.q.conv"] == (16, 4) and shapes["l0.mix.v.conv"] == (48, 4) and shapes["l0.mix.b"] == (4, 72)
    assert shapes["l0.mix.A_log"] == (4,) and shapes["l0.mix.dt_bias"] == (32,) and shapes["l0.mix.norm"] == (12,)
    assert shapes["l0.mix.a1"] == (4, 72) and shapes["l0.mix.a2"] == (32, 4) and shapes["l0.mix.g1"] == (6, 72)
    assert shapes["l0.mix.g2"] == (48, 6) and shapes["l0.mix.o"] == (72, 48)
    assert shapes["l0.mlp.up"] == (88, 72) and shapes["l0.mlp.down"] == (72, 88) and "l0.mlp.gate" not in shapes
    assert shapes["l1.mix.q"] == (48, 72) and shapes["l1.mix.k"] == (16, 72) and shapes["l1.mix.v"] == (40, 72)
    assert shapes["l1.mix.q.norm"] == (48,) and shapes["l1.mix.k.norm"] == (16,) and shapes["l1.mix.vmix"] == ()
    assert shapes["l1.mix.o"] == (72, 120) and "l1.mix.q.b" not in shapes and "l1.mix.sink" not in shapes
    assert "l2.mix.vmix" not in shapes and "l2.norm1" in shapes and not any(k.startswith("l2.mlp") or k == "l2.norm2" for k in shapes)
    assert shapes["l1.mlp.router"] == (5, 72) and shapes["l1.mlp.router.b"] == (5,) and shapes["l1.mlp.e4.up"] == (24, 72)
    assert shapes["l1.mlp.shared.gate"] == (40, 72) and shapes["l1.mlp.shared.down"] == (72, 40) and shapes["l1.mlp.shared.sg"] == (1, 72)
    assert "l3.mlp.shared.sg" not in shapes and shapes["l4.mlp.shared.up"] == (8, 72)


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "multiple"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=24), "v_mix"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "top"),
    (lambda c: c["layers"][0].update(type="latent_attention"), "not one of"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), "mask"),
    (lambda c: c["layers"][0]["mixer"].update(conv=0), "conv"),
    (lambda c: c["layers"][0]["mixer"].pop("conv"), "conv"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "kind"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.pop("max_positions"), "max_positions"),
    (lambda c: c["norm"].pop("eps"), "eps"),
])
def test_configurations_that_are_refused(change, message):
    import re
    from yalm_amd.config import ConfigError, config_from_dict
    cfg = copy.deepcopy(BC.MIXED)
    change(cfg)
    with pytest.raises(ConfigError) as e:
        config_from_dict(cfg)
    assert re.search(message, str(e.value))


def test_low_rank_sizes_come_from_a_folders_tensors(tmp_path):
    """A folder's config.json need not name the inner sizes of the decay's and the gate's pairs of matrices: the shapes
    of the first matrices give them."""
    from yalm_amd.config import ConfigError, config_from_dict
    from yalm_amd.config.registry import config_from_folder
    from yalm_amd.weights import write_random_model
    folder = write_random_model(str(tmp_path / "m"), BC.ONLY_MOE, seed=1)
    bare = copy.deepcopy(BC.ONLY_MOE)
    for k in ("decay_rank", "gate_rank"):
        del bare["layers"][0]["mixer"][k]
    with pytest.raises(ConfigError):
        config_from_dict(bare).to_spec()
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(bare, f)
    cfg = config_from_folder(folder)
    assert cfg.layers[0]["mixer"]["decay_rank"] == 4 and cfg.layers[0]["mixer"]["gate_rank"] == 6
    assert cfg.to_spec().layers[0].mixer.params["gate_rank"] == 6


@pytest.mark.parametrize("name", ["mixed", "blocks", "only_blend", "odd"])
def test_plain_whole_prompt_equals_pieces_and_single_tokens(name):
    cfg = BC.ALL[name]
    w = random_weights(cfg, 3)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, cfg["vocab"], (90,), generator=g).tolist()
    whole = P.forward(cfg, w, toks)
    for cuts in ([40, 90], [1, 2, 66, 67, 90], list(range(1, 91))):
        mem, start, rows = {}, 0, []
        for end in cuts:
            rows.append(P.forward(cfg, w, toks[start:end], memory=mem, start=start))
            start = end
        assert torch.allclose(torch.cat(rows), whole, rtol=0, atol=1e-9), (name, cuts[:3])


def test_delta_rule_with_orthogonal_keys_stores_and_replaces():
    """Keys along the axes, no decay, step size 1: writing k_a with v_1 and then k_a with v_2 leaves v_2 alone under
    k_a (the rule takes the old value off), k_b's value is untouched, and the read-out sees the token's own write."""
    d, dv = 4, 3
    e = torch.eye(d, dtype=F64)
    k = torch.stack([e[0], e[1], e[0], e[2]]).reshape(4, 1, d)
    v = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0], [-1.0, 0.5, 9.0], [7.0, 7.0, 7.0]], dtype=F64).reshape(4, 1, dv)
    q = torch.stack([e[0], e[0] + e[1], e[0] + e[1], e[1] + e[2]]).reshape(4, 1, d)
    ones = torch.ones(4, 1, dtype=F64)
    o, S = P.delta_recurrence(q, k, v, ones, torch.ones(4, 1, d, dtype=F64), torch.zeros(1, d, dv, dtype=F64))
    assert torch.allclose(o[0, 0], v[0, 0]) and torch.allclose(o[1, 0], v[0, 0] + v[1, 0])
    assert torch.allclose(o[2, 0], v[2, 0] + v[1, 0]) and torch.allclose(o[3, 0], v[1, 0] + v[3, 0])
    assert torch.allclose(S[0, 0], v[2, 0]) and torch.allclose(S[0, 3], torch.zeros(dv, dtype=F64))
    # step size 1/2 moves the stored value half way; a decay on channel 0 alone shrinks that row alone
    half = torch.full((1, 1), 0.5, dtype=F64)
    decay = torch.ones(1, 1, d, dtype=F64)
    decay[0, 0, 0] = 0.25
    o2, S2 = P.delta_recurrence(q[:1], k[:1], v[3:4], half, decay, S.clone())
    assert torch.allclose(S2[0, 0], 0.25 * v[2, 0] + 0.5 * (v[3, 0] - 0.25 * v[2, 0])) and torch.allclose(S2[0, 1], S[0, 1])


def test_short_convolution_carries_its_last_inputs():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(9, 5, generator=g, dtype=F64)
    taps = torch.randn(5, 4, generator=g, dtype=F64)
    whole, last = P.short_conv(x, taps, torch.zeros(3, 5, dtype=F64))
    assert torch.allclose(whole[0], taps[:, 3] * x[0]) and torch.allclose(whole[1], taps[:, 3] * x[1] + taps[:, 2] * x[0])
    assert torch.allclose(whole[5], sum(taps[:, 3 - b] * x[5 - b] for b in range(4)))
    assert torch.equal(last, x[6:])
    before, rows = torch.zeros(3, 5, dtype=F64), []
    for cut in ([0, 1], [1, 3], [3, 9]):
        y, before = P.short_conv(x[cut[0]:cut[1]], taps, before)
        rows.append(y)
    assert torch.allclose(torch.cat(rows), whole, rtol=0, atol=1e-12)
    one, nothing = P.short_conv(x, taps[:, :1], torch.zeros(0, 5, dtype=F64))      # one tap keeps nothing
    assert torch.allclose(one, taps[:, 0] * x) and nothing.shape[0] == 0


def test_a_block_hides_what_lies_before_it_and_slopes_take_the_distance_off():
    assert P.visible(13, 7, 7) and not P.visible(14, 13, 7) and P.visible(14, 14, 7) and not P.visible(6, 7, 7)
    assert P.visible(300, 0, 0) and not P.visible(0, 1, 0)
    assert P.head_slopes(4) == [0.25, 0.0625, 0.015625, 0.00390625]
    cfg = BC.ONLY_ATTN
    w = random_weights(cfg, 1)
    m = cfg["layers"][0]["mixer"]
    h = torch.randn(9, 32, generator=torch.Generator().manual_seed(2), dtype=F64)
    out, v = P.attention(h, list(range(9)), m, w, "l0.mix.", 1e-5, {})
    # position 7 opens a block of its own: it sees itself alone, so its result is its value through W_o
    want = torch.cat([v[7, 0], v[7, 0]]) @ w["l0.mix.o"].T
    assert torch.allclose(out[7], want, rtol=0, atol=1e-12)
    # position 8 sees 7 and 8: two keys, the farther one a slope lower
    q = P.rms_div(h @ w["l0.mix.q"].T, 1e-5) * w["l0.mix.q.norm"]
    k = P.rms_div(h @ w["l0.mix.k"].T, 1e-5) * w["l0.mix.k.norm"]
    rows = []
    for hd in range(2):
        s = torch.stack([(q[8, hd * 8:hd * 8 + 8] @ k[7]) * m["scale"] - P.head_slopes(2)[hd], (q[8, hd * 8:hd * 8 + 8] @ k[8]) * m["scale"]])
        p = torch.softmax(s, 0)
        rows.append(p[0] * v[7, 0] + p[1] * v[8, 0])
    assert torch.allclose(out[8], torch.cat(rows) @ w["l0.mix.o"].T, rtol=0, atol=1e-12)


def test_router_weights_are_the_softmax_over_the_chosen_and_the_shared_expert_has_its_gate():
    w = {"r.router": torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0], [-1.0, 0.5]], dtype=F64),
         "r.router.b": torch.tensor([0.0, 0.5, -3.0, 0.25], dtype=F64)}
    h = torch.tensor([[2.0, 1.0]], dtype=F64)
    ids, wts = P.route(h, w, "r.", 2)
    z = torch.tensor([2.0, 1.5, 0.0, -1.25], dtype=F64)
    assert ids.tolist() == [[0, 1]]
    assert torch.allclose(wts[0], torch.softmax(z[:2], 0))
    assert abs(float(P.route_margin(h, w, "r.", 2)[0]) - 1.5) < 1e-12
    g = torch.Generator().manual_seed(0)
    for e in range(4):
        for k, s in (("gate", (3, 2)), ("up", (3, 2)), ("down", (2, 3))):
            w["r.e%d.%s" % (e, k)] = torch.randn(s, generator=g, dtype=F64)
    for k, s in (("gate", (5, 2)), ("up", (5, 2)), ("down", (2, 5)), ("sg", (1, 2))):
        w["r.shared." + k] = torch.randn(s, generator=g, dtype=F64)
    mlp = {"kind": "moe", "router": {"experts": 4, "top": 2}, "shared": {"ff": 5}}
    got = P.moe_ff(h, mlp, w, "r.")
    want = wts[0, 0] * P.gated_ff(h, w, "r.e0.") + wts[0, 1] * P.gated_ff(h, w, "r.e1.") \
        + P.gated_ff(h, w, "r.shared.") / (1.0 + math.exp(-float(h[0] @ w["r.shared.sg"][0])))
    assert torch.allclose(got, want, rtol=0, atol=1e-12)
    assert torch.allclose(P.moe_ff(h, dict(mlp, shared=None), w, "r."),
                          wts[0, 0] * P.gated_ff(h, w, "r.e0.") + wts[0, 1] * P.gated_ff(h, w, "r.e1."), rtol=0, atol=1e-12)
